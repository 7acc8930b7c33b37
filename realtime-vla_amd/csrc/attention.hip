// Softmax attention on MFMA, flash style (online softmax, logits never leave registers).
//
//  * mqa_kernel    - attention of G query heads that share one K/V head of width HD, query rows = token*G + head,
//                    i.e. a [rows x HD] x [keys x HD]^T problem against one shared K and V, optionally batched
//                    over independent K/V heads (blockIdx.y).  G = 8, HD = 256: Gemma multi-query attention, the
//                    prefix pass (/root/reference/pi0_infer.py:819-824, pi05_infer.py:335-360) and the
//                    action-expert suffix pass with its masks (pi0_infer.py:1041-1120, pi05_infer.py:382-478).
//                    G = 2, HD = 128, 8 K/V heads: DM0's grouped-query attention, causal in the prefix
//                    (/root/reference/dm0_infer.py:913-918) and unmasked in the action expert (:822-826).
//                    (DM0's ViT attention, long on both sides, is csrc/flash.hip.)
//  * vision_kernel - SigLIP attention, 16 heads x 72 per view, 256 keys (pi0_infer.py:588-596).
//
// Both compute the transposed logits S^T = K Q^T so that each lane holds 16 keys of ONE query row:
// the softmax statistics are per-lane scalars and the probabilities are already in the register
// layout of the MFMA B operand for O^T = V^T P^T, provided V is read with the matching key
// permutation.  V is therefore kept transposed in memory ([d][key]) by the producing GEMM.
//
// The suffix pass has only ~26 row tiles but ~840 keys, and one CU can pull only ~100 GB/s through its
// L2 port, so a workgroup that walks all keys is bound by that port.  Its keys are therefore split over
// several workgroups, each writing an un-normalised partial (O, row max, row sum); a second small
// kernel (attn_merge_kernel) combines the partials.  Merging inside the first kernel (last workgroup to
// finish does it) was measured slower, twice: with the partials crossing XCDs, whose L2s are not coherent with each
// other, device-scope fences or write-through accesses cost more than one extra launch; and with all key splits of a
// row block dealt to ONE XCD (no fence at all: write-through stores, an arrival counter in that XCD's L2, the last
// workgroup reading the others' records from the cache they were written to) the single launch took 8.3 us against 7.7 us
// for the pair - store acknowledge, atomic round trip and the dependent loads of the tail add up to a launch boundary,
// and every XCD then fetches all of K / V^T.
#include "kernels.h"

namespace {

constexpr float NEG_BIG = -1.0e30f;

RTVLA_DEVICE bf16x8 cat44(bf16x4 lo, bf16x4 hi) {
    bf16x8 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[j] = lo[j]; v[4 + j] = hi[j]; }
    return v;
}

// where element (row, d) of the output goes: row-major [token][ld_tok] with the G heads of a token side by side (and the
// batch index split into an outer and an inner part with a stride each), or the fragment-tiled [tokens][32 out_cols32]
// matrix the action-expert O projection reads
struct AttnOutRow { bf16_t* base; int tok, col; };
RTVLA_DEVICE AttnOutRow attn_out_row(const AttnP& p, int batch, int row, int hd) {
    const int tok = row / p.group, sub = row - tok * p.group;
    if (p.out_tiled) return {p.out, tok, batch * p.out_bcol + sub * hd};
    const int bo = batch / p.batch_inner, bi = batch - bo * p.batch_inner;
    return {p.out + (size_t)bo * p.out_ostride + (size_t)bi * p.out_istride + (size_t)tok * p.ld_tok + sub * hd, tok, 0};
}
RTVLA_DEVICE bf16_t* attn_out_at(const AttnP& p, const AttnOutRow& o, int d) {
    return p.out_tiled ? o.base + ft_index(o.tok, o.col + d, p.out_cols32) : o.base + d;
}
RTVLA_DEVICE bf16_t* attn_out_ptr(const AttnP& p, int batch, int row, int d, int hd) { return attn_out_at(p, attn_out_row(p, batch, row, hd), d); }

template <int WAVES, int MQ, int NTK, int HD, bool CAUSAL>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(1, HD == 256 ? 1 : 2)))
void mqa_kernel(AttnP p) {
    constexpr int KD = HD / 32;                                       // 32-wide steps of the Q K^T contraction
    constexpr int DT = HD / 16;                                       // 16-wide tiles of the output
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    f32x4* obuf = (f32x4*)smem_raw;                                   // [WAVES][DT][64]
    float* ms = (float*)(smem_raw + (size_t)WAVES * DT * 64 * 16);    // [WAVES][MQ][16]
    float* ls = ms + WAVES * MQ * 16;                                 // [WAVES][MQ][16]
    const int batch = blockIdx.y;
    const bf16_t* const qbase = p.q + (size_t)batch * p.q_bstride;
    const bf16_t* const kbase = p.k + (size_t)batch * p.k_bstride;
    const bf16_t* const vbase = p.vt + (size_t)batch * p.vt_bstride;

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = lane >> 4, r = lane & 15;
    // Workgroup ids are dealt round-robin over the 8 XCDs.  With a key split the id is decoded so that all row
    // blocks of one split land on the same XCD: its slice of K / V^T is then fetched into one L2 instead of eight.
    const int nsplit = p.nsplit_eff;
    int rowblk, split;
    if (nsplit == 1) { rowblk = blockIdx.x; split = 0; }
    else {
        const int spx = (nsplit + 7) >> 3;                           // splits per XCD
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        split = xcd + 8 * (idx % spx); rowblk = idx / spx;
        if (split >= nsplit) return;                                 // (whole workgroup, before any barrier)
    }
    const int m0 = rowblk * (16 * MQ);

    int vl = p.prefix_alloc;
    if (p.valid_len) vl = max(0, min(*p.valid_len, p.prefix_alloc));
    const int vis_lim = min(vl, p.keys);                             // keys below this are visible to every row (causal aside)
    const float sc2 = p.scale * 1.4426950408889634f;

    bf16x8 qf[MQ][KD];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
        // fragment-tiled Q: one contiguous 1 KB read per fragment (row tiles past the end are padding)
        const bf16_t* qp = qbase + ((size_t)(rowblk * MQ + mq) * KD * 64 + lane) * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) qf[mq][kd] = *(const bf16x8*)(qp + kd * 512);
    }
    f32x4 o[MQ][DT];
    float mrun[MQ], lrun[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
        mrun[mq] = NEG_BIG; lrun[mq] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[mq][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    constexpr int KBS = NTK * 16;                    // keys per block
    int nkb = (p.keys + KBS - 1) / KBS;
    // causal: the last row of this block sees keys up to its own token
    if constexpr (CAUSAL) nkb = min(nkb, (min(m0 + 16 * MQ, p.rows) - 1) / p.group / KBS + 1);
    const int kb_begin = split * p.kb_per_split, kb_end = min(nkb, kb_begin + p.kb_per_split);
    const int keys32 = p.ldvt >> 5;
    bf16x8 kf[NTK][KD];       // K fragments of one key block (A operand of S^T = K Q^T)
    bf16x8 vf[DT][NTK / 2];      // V^T fragments of the block, in the key order the P registers have
    auto load_k = [&](int kb) {
#pragma unroll
        for (int nt = 0; nt < NTK; ++nt) {
            const bf16_t* kp = kbase + ((size_t)(kb * NTK + nt) * KD * 64 + lane) * 8;
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) kf[nt][kd] = *(const bf16x8*)(kp + kd * 512);
        }
    };
    auto load_v = [&](int kb) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16_t* vp = vbase + ((size_t)(dt * keys32 + kb * (NTK / 2)) * 64 + lane) * 8;
#pragma unroll
            for (int kk = 0; kk < NTK / 2; ++kk) vf[dt][kk] = *(const bf16x8*)(vp + kk * 512);
        }
    };
    if (kb_begin + w < kb_end) { load_k(kb_begin + w); load_v(kb_begin + w); }
    __builtin_amdgcn_sched_barrier(0);

    for (int kb = kb_begin + w; kb < kb_end; kb += WAVES) {
        const int key0 = kb * KBS;
        const int kb_next = kb + WAVES;
        f32x4 st[MQ][NTK];
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
            for (int nt = 0; nt < NTK; ++nt) st[mq][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nt = 0; nt < NTK; ++nt)
#pragma unroll
            for (int kd = 0; kd < KD; ++kd)
#pragma unroll
                for (int mq = 0; mq < MQ; ++mq) st[mq][nt] = mfma16(kf[nt][kd], qf[mq][kd], st[mq][nt]);
        __builtin_amdgcn_sched_barrier(0);
        if (kb + WAVES < kb_end) load_k(kb_next);            // next block's K flies during softmax and P V (the suffix pass has one block per wave: nothing to fetch)
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 pb[MQ][NTK / 2];
        bool full = key0 + KBS <= vis_lim;
        if constexpr (CAUSAL) full = full && key0 + KBS - 1 <= m0 / p.group;
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) {
            const int row = m0 + mq * 16 + r;
            int own = 0;                                      // causal: the row's own token, the last key it sees
            if constexpr (CAUSAL) own = row / p.group;
            // logits in the base-2 domain (scale * log2 e folded into one multiply); a block every row sees whole (all but the
            // last of a prefix pass) takes the path without mask arithmetic
            float mx = NEG_BIG;
            bool vis[NTK][4];
            if (full) {
#pragma unroll
                for (int nt = 0; nt < NTK; ++nt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) { st[mq][nt][v] *= sc2; mx = fmaxf(mx, st[mq][nt][v]); vis[nt][v] = true; }
            } else {
#pragma unroll
                for (int nt = 0; nt < NTK; ++nt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = key0 + nt * 16 + 4 * g + v;
                        bool ok = key < p.keys;
                        if (key < p.prefix_alloc) ok = ok && key < vl;
                        else ok = ok && (row >= p.state_rows || key == p.prefix_alloc);
                        if constexpr (CAUSAL) ok = ok && key <= own;
                        vis[nt][v] = ok;
                        const float s = ok ? st[mq][nt][v] * sc2 : NEG_BIG;
                        st[mq][nt][v] = s;
                        mx = fmaxf(mx, s);
                    }
            }
            mx = rows_max(mx);
            if (__any(mx > mrun[mq])) {                       // the accumulator is rescaled only when some row's maximum grew
                const float mnew = fmaxf(mrun[mq], mx);
                const float alpha = __builtin_amdgcn_exp2f(mrun[mq] - mnew);
                lrun[mq] *= alpha;
                mrun[mq] = mnew;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[mq][dt] *= alpha;
            }
            float sum = 0.f;
#pragma unroll
            for (int nt = 0; nt < NTK; ++nt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float e = vis[nt][v] ? __builtin_amdgcn_exp2f(st[mq][nt][v] - mrun[mq]) : 0.f;
                    st[mq][nt][v] = e;
                    sum += e;
                }
            sum = rows_sum(sum);
            lrun[mq] += sum;
#pragma unroll
            for (int kk = 0; kk < NTK / 2; ++kk) pb[mq][kk] = cat44(pack4(st[mq][2 * kk]), pack4(st[mq][2 * kk + 1]));
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < NTK / 2; ++kk) {
#pragma unroll
                for (int mq = 0; mq < MQ; ++mq) o[mq][dt] = mfma16(vf[dt][kk], pb[mq][kk], o[mq][dt]);
            }
        __builtin_amdgcn_sched_barrier(0);
        if (kb + WAVES < kb_end) load_v(kb_next);
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- merge the key splits of the WAVES waves ----
    if (g == 0) {
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) ms[(w * MQ + mq) * 16 + r] = mrun[mq];
    }
    __syncthreads();
    float mgl[MQ];
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
        float mg = NEG_BIG;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) mg = fmaxf(mg, ms[(ww * MQ + mq) * 16 + r]);
        const float sc = __builtin_amdgcn_exp2f(mrun[mq] - mg);
        lrun[mq] *= sc;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[mq][dt] *= sc;
        if (g == 0) ls[(w * MQ + mq) * 16 + r] = lrun[mq];
        mgl[mq] = mg;
    }
    // partial record of one (row block, split): MQ x { O [DT][64] f32x4 | max [16] | sum [16] }
    constexpr int REC = DT * 64 * 4 + 32;
    float* const mine = p.partial + (((size_t)batch * p.row_blocks + rowblk) * nsplit + split) * (MQ * REC);
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
        __syncthreads();                       // ls written / previous obuf round consumed
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) obuf[((size_t)w * DT + dt) * 64 + lane] = o[mq][dt];
        __syncthreads();
        float lt = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) lt += ls[(ww * MQ + mq) * 16 + r];
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        const int row = m0 + mq * 16 + r;
        const AttnOutRow orow = attn_out_row(p, batch, min(row, p.rows - 1), HD);
        if (nsplit > 1 && w == 0 && g == 0) { mine[mq * REC + DT * 256 + r] = mgl[mq]; mine[mq * REC + DT * 256 + 16 + r] = lt; }
        for (int dt = w; dt < DT; dt += WAVES) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) t += obuf[((size_t)ww * DT + dt) * 64 + lane];
            if (nsplit > 1) {
                *(f32x4*)(mine + mq * REC + (dt * 64 + lane) * 4) = t;
            } else if (row < p.rows) {
                store4(attn_out_at(p, orow, dt * 16 + 4 * g), pack4(t * inv));
            }
        }
    }
}

// Suffix pass with at most one 32-key block per wave (key splits of 128 keys): the four waves of a workgroup share the
// PROBABILITIES instead of merging their outputs.  Wave w computes the logits of key block w (it alone reads that block
// of K), the row maxima and then the probabilities are exchanged through LDS (16 floats and one 1 KB fragment per wave),
// and every wave multiplies all four probability fragments with ITS quarter of the head width of V^T (16 / 4 d tiles x 4
// key blocks: the same 16 fragments it would read of one key block), so each wave ends up with finished columns of the
// partial and stores them straight to memory: no output exchange (64 KB each way), one barrier less.  Q is loaded once
// per workgroup (each wave fetches a quarter) and shared through LDS.
template <int HD>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2)))
void suffix_attn_kernel(AttnP p) {
    constexpr int KD = HD / 32, DT = HD / 16, DTW = DT / 4, QW = KD / 4;
    static_assert(KD % 4 == 0, "Q fragments are dealt over four waves");
    __shared__ bf16x8 qsh[KD][64];
    __shared__ bf16x8 psh[4][64];
    __shared__ float msh[4][16], lsh[4][16];
    const int batch = blockIdx.y;
    const bf16_t* const qbase = p.q + (size_t)batch * p.q_bstride;
    const bf16_t* const kbase = p.k + (size_t)batch * p.k_bstride;
    const bf16_t* const vbase = p.vt + (size_t)batch * p.vt_bstride;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int riders = p.riders;                                         // a multiple of 8, so that the decode below still sees the XCD in the low bits
    if ((int)blockIdx.x < riders) {                                      // riding workgroups: weight tiles of a later launch
        if (blockIdx.y == 0) prefetch_tile<256>(p.pf_attn, blockIdx.x, tid);
        return;
    }
    const int nsplit = p.nsplit_eff;
    // all row blocks of one split on one XCD (see mqa_kernel); the launcher uses this kernel for split passes only
    const int spx = (nsplit + 7) >> 3;
    const int bx = blockIdx.x - riders;
    const int xcd = bx & 7, idx = bx >> 3;
    const int split = xcd + 8 * (idx % spx), rowblk = idx / spx;
    if (split >= nsplit) return;                                         // (whole workgroup, before any barrier)
    const int m0 = rowblk * 16;
    int vl = p.prefix_alloc;
    if (p.valid_len) vl = max(0, min(*p.valid_len, p.prefix_alloc));
    const int vis_lim = min(vl, p.keys);
    const float sc2 = p.scale * 1.4426950408889634f;
    const int nkb = (p.keys + 31) >> 5, keys32 = p.ldvt >> 5;
    const int kb_begin = split * p.kb_per_split, kb_end = min(nkb, kb_begin + p.kb_per_split);
    const int kb = kb_begin + w;
    const bool have = kb < kb_end;                                       // (wave-uniform)

    // everything this wave needs from memory, requested up front: its quarter of Q, its key block of K, its d tiles of V^T
    bf16x8 qmine[QW];
#pragma unroll
    for (int i = 0; i < QW; ++i) qmine[i] = *(const bf16x8*)(qbase + ((size_t)(rowblk * KD + w * QW + i) * 64 + lane) * 8);
    bf16x8 kf[2][KD];
    if (have) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int kd = 0; kd < KD; ++kd) kf[nt][kd] = *(const bf16x8*)(kbase + ((size_t)((kb * 2 + nt) * KD + kd) * 64 + lane) * 8);
    }
    bf16x8 vf[DTW][4];
#pragma unroll
    for (int i = 0; i < DTW; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)                                      // blocks past the end are clamped: their probabilities are zero
            vf[i][j] = *(const bf16x8*)(vbase + ((size_t)((w * DTW + i) * keys32 + min(kb_begin + j, keys32 - 1)) * 64 + lane) * 8);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < QW; ++i) qsh[w * QW + i][lane] = qmine[i];
    __syncthreads();

    // ---- logits of this wave's key block, base-2 domain ----
    f32x4 st[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    bool vis[2][4];
    float mx = NEG_BIG;
    const int row = m0 + r;
    if (have) {
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const bf16x8 qf = qsh[kd][lane];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) st[nt] = mfma16(kf[nt][kd], qf, st[nt]);
        }
        const int key0 = kb * 32;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int key = key0 + nt * 16 + 4 * g + v;
                bool ok = key < p.keys;
                if (key0 + 32 > vis_lim) {                               // (uniform) a block every row sees whole needs no mask arithmetic
                    if (key < p.prefix_alloc) ok = ok && key < vl;
                    else ok = ok && (row >= p.state_rows || key == p.prefix_alloc);
                }
                vis[nt][v] = ok;
                const float sv = ok ? st[nt][v] * sc2 : NEG_BIG;
                st[nt][v] = sv;
                mx = fmaxf(mx, sv);
            }
        mx = rows_max(mx);
    } else {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) vis[nt][v] = false;
    }
    if (g == 0) msh[w][r] = mx;
    __syncthreads();
    const float mg = fmaxf(fmaxf(msh[0][r], msh[1][r]), fmaxf(msh[2][r], msh[3][r]));
    float sum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float e = vis[nt][v] ? __builtin_amdgcn_exp2f(st[nt][v] - mg) : 0.f;
            st[nt][v] = e;
            sum += e;
        }
    sum = rows_sum(sum);
    psh[w][lane] = cat44(pack4(st[0]), pack4(st[1]));
    if (g == 0) lsh[w][r] = sum;
    __syncthreads();

    // ---- this wave's d tiles of O^T = V^T P^T over all four key blocks ----
    bf16x8 pb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) pb[j] = psh[j][lane];
    const float lt = lsh[0][r] + lsh[1][r] + lsh[2][r] + lsh[3][r];
    f32x4 o[DTW];
#pragma unroll
    for (int i = 0; i < DTW; ++i) {
        o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) o[i] = mfma16(vf[i][j], pb[j], o[i]);
    }
    // partial record of one (row block, split): { O [DT][64] f32x4 | max [16] | sum [16] }, combined by attn_merge_kernel
    constexpr int REC = DT * 64 * 4 + 32;
    float* const mine = p.partial + (((size_t)batch * p.row_blocks + rowblk) * nsplit + split) * REC;
#pragma unroll
    for (int i = 0; i < DTW; ++i) *(f32x4*)(mine + ((w * DTW + i) * 64 + lane) * 4) = o[i];
    if (w == 0 && g == 0) { mine[DT * 256 + r] = mg; mine[DT * 256 + 16 + r] = lt; }
}

// Combine the key-split partials of mqa_kernel: one wave per (row block, 16-wide d tile), 4 waves per workgroup, K/V heads
// along blockIdx.y.  All loads of a wave are independent, so the kernel is one memory round trip long.
template <int MQ, int NS, int HD>
__global__ __launch_bounds__(256)
void attn_merge_kernel(AttnP p, int nsplit) {
    constexpr int DT = HD / 16;
    constexpr int REC = DT * 64 * 4 + 32;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int batch = blockIdx.y;
    const int rb = blockIdx.x / (DT / 4), dt = (blockIdx.x % (DT / 4)) * 4 + w;
    const float* const all = p.partial + ((size_t)batch * p.row_blocks + rb) * nsplit * (MQ * REC);
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) {
        float ms[NS], ls[NS];
        f32x4 os[NS];
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) {
            const float* rec = all + (size_t)min(sp, nsplit - 1) * (MQ * REC) + mq * REC;
            ms[sp] = rec[DT * 256 + r]; ls[sp] = rec[DT * 256 + 16 + r];
            os[sp] = *(const f32x4*)(rec + (dt * 64 + lane) * 4);
        }
        float mg = NEG_BIG;
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) if (sp < nsplit) mg = fmaxf(mg, ms[sp]);
        float lt = 0.f;
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) {
            const float wgt = sp < nsplit ? __builtin_amdgcn_exp2f(ms[sp] - mg) : 0.f;      // the maxima are base-2 logits
            lt += wgt * ls[sp];
            t += os[sp] * wgt;
        }
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        const int row = (rb * MQ + mq) * 16 + r;
        if (row < p.rows) {
            const int d = dt * 16 + 4 * g;
            store4(attn_out_ptr(p, batch, row, d, HD), pack4(t * inv));
        }
    }
}

// SigLIP: per (view, head) Q and K are fragment-tiled [256 tokens][96] (head dim 72 zero padded),
// V^T is [80][256] in the permuted-key tile layout; out is row-major [views*256][1152].
// One wave per 16 query rows over all 256 keys; 4 waves per workgroup.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void vision_attn_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ vt,
                        bf16_t* __restrict__ out) {
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int blk = blockIdx.x;                  // (view*16 + head)*4 + quarter
    const int quarter = blk & 3, vh = blk >> 2, head = vh & 15, view = vh >> 4;
    const int mtile = quarter * 4 + w;                             // 16-row tile of this wave inside the view
    const int row = view * 256 + mtile * 16 + r;                   // query token (global row)
    const float scale = 0.11785113019775792f * 1.4426950408889634f; // 1 / sqrt(72), in the base-2 domain

    const bf16_t* qb = q + (size_t)vh * (256 * 96) + lane * 8;
    const bf16_t* kb_ = k + (size_t)vh * (256 * 96) + lane * 8;
    const bf16_t* vb = vt + (size_t)vh * (80 * 256) + lane * 8;
    bf16x8 qf[3];
#pragma unroll
    for (int kd = 0; kd < 3; ++kd) qf[kd] = *(const bf16x8*)(qb + (size_t)(mtile * 3 + kd) * 512);
    // all K and V^T fragments of the 256 keys are requested up front (88 x 1 KB loads per wave)
    bf16x8 kf[16][3];
    bf16x8 vf[5][8];
#pragma unroll
    for (int nt = 0; nt < 16; ++nt)
#pragma unroll
        for (int kd = 0; kd < 3; ++kd) kf[nt][kd] = *(const bf16x8*)(kb_ + (size_t)(nt * 3 + kd) * 512);
#pragma unroll
    for (int dt = 0; dt < 5; ++dt)
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) vf[dt][kk] = *(const bf16x8*)(vb + (size_t)(dt * 8 + kk) * 512);
    __builtin_amdgcn_sched_barrier(0);

    f32x4 o[5];
#pragma unroll
    for (int dt = 0; dt < 5; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrun = NEG_BIG, lrun = 0.f;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
        f32x4 st[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            st[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kd = 0; kd < 3; ++kd) st[nt] = mfma16(kf[kb * 4 + nt][kd], qf[kd], st[nt]);
        }
        float mx = NEG_BIG;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) { st[nt][v] *= scale; mx = fmaxf(mx, st[nt][v]); }
        mx = rows_max(mx);
        if (__any(mx > mrun)) {
            const float mnew = fmaxf(mrun, mx);
            const float alpha = __builtin_amdgcn_exp2f(mrun - mnew);
            lrun *= alpha;
            mrun = mnew;
#pragma unroll
            for (int dt = 0; dt < 5; ++dt) o[dt] *= alpha;
        }
        float sum = 0.f;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) { st[nt][v] = __builtin_amdgcn_exp2f(st[nt][v] - mrun); sum += st[nt][v]; }
        sum = rows_sum(sum);
        lrun += sum;
        bf16x8 pb[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) pb[kk] = cat44(pack4(st[2 * kk]), pack4(st[2 * kk + 1]));
#pragma unroll
        for (int dt = 0; dt < 5; ++dt) {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) o[dt] = mfma16(vf[dt][kb * 2 + kk], pb[kk], o[dt]);
        }
    }
    const float inv = 1.0f / lrun;
#pragma unroll
    for (int dt = 0; dt < 5; ++dt) {
        const int d = dt * 16 + 4 * g;
        if (d < 72) store4(out + (size_t)row * 1152 + head * 72 + d, pack4(o[dt] * inv));
    }
}

template <int WAVES, int MQ, int NTK, int HD, bool CAUSAL = false>
int launch_mqa_inst(AttnP p, hipStream_t s, int* nk) {
    const size_t smem = (size_t)WAVES * (HD / 16) * 64 * 16 + (size_t)2 * WAVES * MQ * 16 * 4;
    auto kern = mqa_kernel<WAVES, MQ, NTK, HD, CAUSAL>;
    if (CAUSAL != (p.causal != 0)) return 1;
    if (smem > 65536) {
        static std::atomic<uint64_t> done{0};
        if (int rc = ensure_dynamic_lds((const void*)kern, smem, done)) return rc;
    }
    const int blocks = (p.rows + 16 * MQ - 1) / (16 * MQ);
    const int nkb = (p.keys + NTK * 16 - 1) / (NTK * 16);
    const int want = p.nsplit > 1 ? p.nsplit : 1;
    p.kb_per_split = (nkb + want - 1) / want;
    const int nsplit = (nkb + p.kb_per_split - 1) / p.kb_per_split;
    if (nsplit > 1) {
        if (!p.partial || nsplit > 16 || HD < 64 || p.causal) return 1;           // the key split over workgroups exists for the suffix passes
        if ((size_t)p.batch * blocks * nsplit * MQ * ((HD / 16) * 64 * 4 + 32) > p.partial_floats) return 3;
    }
    p.nsplit_eff = nsplit;
    p.row_blocks = blocks;
    if (MQ == 1 && NTK == 2 && WAVES == 4 && !CAUSAL && nsplit > 1 && p.kb_per_split <= 4) {    // one key block per wave: the probability-sharing kernel
        p.riders = prefetch_wgs(p.pf_attn);
        if (p.riders & 7) return 1;
        hipLaunchKernelGGL((suffix_attn_kernel<HD>), dim3(8 * ((nsplit + 7) / 8) * blocks + p.riders, p.batch), dim3(256), 0, s, p);
    } else
    hipLaunchKernelGGL(kern, dim3(nsplit == 1 ? blocks : 8 * ((nsplit + 7) / 8) * blocks, p.batch), dim3(WAVES * 64), smem, s, p);
    if (nsplit > 8) hipLaunchKernelGGL((attn_merge_kernel<MQ, 16, HD>), dim3(blocks * (HD / 64), p.batch), dim3(256), 0, s, p, nsplit);
    else if (nsplit > 1) hipLaunchKernelGGL((attn_merge_kernel<MQ, 8, HD>), dim3(blocks * (HD / 64), p.batch), dim3(256), 0, s, p, nsplit);
    if (nk) *nk = nsplit > 1 ? 2 : 1;
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

// unit-level entry point only: caller tensors -> operand layouts
__global__ void attn_tile_operands_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v, bf16_t* __restrict__ qt,
                                          bf16_t* __restrict__ kt, bf16_t* __restrict__ vtt, int tokens, int keys, int kv_heads, int group, int hd, int hd_pad,
                                          size_t q_bstride, size_t k_bstride, size_t vt_bstride, int keys_pad, int seq) {
    const size_t nq = (size_t)tokens * kv_heads * group * hd, nk = (size_t)keys * kv_heads * hd;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nq) {
        const int d = (int)(i % hd); size_t t = i / hd;
        const int h = (int)(t % group); t /= group;
        const int b = (int)(t % kv_heads); int tok = (int)(t / kv_heads);
        int bb = b;
        if (seq > 0) { bb = (tok / seq) * kv_heads + b; tok %= seq; }
        qt[(size_t)bb * q_bstride + ft_index(tok * group + h, d, hd_pad >> 5)] = q[i];
        return;
    }
    i -= nq;
    if (i >= 2 * nk) return;
    const bool is_v = i >= nk;
    if (is_v) i -= nk;
    const int d = (int)(i % hd); size_t t = i / hd;
    const int b = (int)(t % kv_heads); int key = (int)(t / kv_heads);
    int bb = b;
    if (seq > 0) { bb = (key / seq) * kv_heads + b; key %= seq; }
    if (is_v) vtt[(size_t)bb * vt_bstride + vt_index(d, key, keys_pad >> 5)] = v[i];
    else kt[(size_t)bb * k_bstride + ft_index(key, d, hd_pad >> 5)] = k[i];
}

}  // namespace

void launch_attn_tile_operands(const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* qt, bf16_t* kt, bf16_t* vtt, int tokens, int keys,
                               int kv_heads, int group, int hd, int hd_pad, size_t q_bstride, size_t k_bstride, size_t vt_bstride, int keys_pad,
                               int seq, hipStream_t s) {
    const size_t n = (size_t)tokens * kv_heads * group * hd + 2 * (size_t)keys * kv_heads * hd;
    hipLaunchKernelGGL(attn_tile_operands_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, q, k, v, qt, kt, vtt, tokens, keys, kv_heads, group, hd,
                       hd_pad, q_bstride, k_bstride, vt_bstride, keys_pad, seq);
}

int launch_mqa_attention(const AttnP& p0, int variant, hipStream_t s, int* nk) {
    AttnP p = p0;
    if (p.rows <= 0 || p.keys <= 0 || (p.ldvt & 31) || p.ldvt < ((p.keys + 31) / 32) * 32) return 1;
    if (p.batch < 1) p.batch = 1;
    if (p.batch_inner < 1) p.batch_inner = 1;
    if (p.group < 1) return 1;
    switch (variant) {                                          // template: waves, row tiles per workgroup, 16-key tiles per wave round, head width
        case ATTN_PREFIX: return launch_mqa_inst<4, 2, 2, 256>(p, s, nk);
        case ATTN_SUFFIX: return launch_mqa_inst<4, 1, 2, 256>(p, s, nk);
        case ATTN_GQA128_PREFIX: return launch_mqa_inst<4, 2, 2, 128, true>(p, s, nk);
        case ATTN_GQA128_SUFFIX: return launch_mqa_inst<4, 1, 2, 128>(p, s, nk);
    }
    return 2;
}

void launch_vision_attention(const bf16_t* q, const bf16_t* k, const bf16_t* vt, bf16_t* out, int views, hipStream_t s) {
    hipLaunchKernelGGL(vision_attn_kernel, dim3(views * 16 * 4), dim3(256), 0, s, q, k, vt, out);
}
