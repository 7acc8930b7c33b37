// Softmax attention for long query AND key sequences on v_mfma_f32_32x32x16_bf16, flash style: DM0's ViT attention,
// 2705 tokens per (image, head), head width 64 (/root/reference/dm0_infer.py:589-598), 3 x 16 independent heads.
//
// One workgroup = 4 waves = 128 consecutive query rows of one K/V head; each wave owns 32 query rows and walks ALL keys,
// so there is no merge at the end.  K and V^T tiles of 64 keys go from global memory straight into LDS (global_load_lds,
// three stages, one barrier per tile) and are shared by the four waves: the L2 port of a CU carries each tile once per
// 128 query rows instead of once per wave.  The tiles keep the byte layout they have in memory (MFMA fragments of 1 KB:
// Q and K fragment-tiled [rows][HD], V^T in the permuted-key layout), so staging is a plain copy of 1 KB pieces and every
// operand read is a conflict-free ds_read_b128.
//
// Per 32-key block the wave computes S^T = K Q^T (32 keys x 32 queries): lane (h = lane / 32, n = lane % 32) holds the 16
// logits of query n for keys 8 j + 4 h + v.  The softmax statistics are therefore per-lane scalars shared with ONE other
// lane, the running sum is kept per lane and combined once at the end, and the accumulator is only rescaled when some
// row's maximum grew by more than 2^8 (a wave-uniform branch, taken a few times per row).  The probabilities of
// accumulator groups j = q and j = q + 2 are, packed to bf16, exactly the B operand of O^T += V^T P^T for the q-th 16-key
// step in the key order of the stored V^T: no shuffles between the two products.  The loop is software-pipelined over the
// 32-key blocks (see flash_kernel).
//
// Measured on MI355X (48 heads x 2705 tokens): 146 us where the version without the pipeline, with register staging and a
// rescale in most tiles took 161 us on the same machine; 71 us for 48 x 2048 tokens, which fit one round of 768
// workgroups (0.72 PFLOP/s).  LDS reads (ds_read_b128: 256 B/clk per CU measured) are 18 % busy, the MFMA pipe 37 %, the
// VALU 59 %; the second, a third full round of 2705-token heads (1 056 workgroups on 768 places) costs about 45 us.
#include "kernels.h"
#include <type_traits>

namespace {

constexpr float NEG_BIG = -1.0e30f;

RTVLA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

RTVLA_DEVICE bf16x8 pack8(const f32x16& s, int a, int b) {
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = (bf16_t)s[4 * a + i]; v[4 + i] = (bf16_t)s[4 * b + i]; }
    return v;
}

RTVLA_DEVICE bf16_t* flash_out_ptr(const AttnP& p, int batch, int row, int d, int hd) {
    const int tok = row / p.group, sub = row - tok * p.group;
    if (p.out_tiled) return p.out + ft_index(tok, batch * p.out_bcol + sub * hd + d, p.out_cols32);
    const int bo = batch / p.batch_inner, bi = batch - bo * p.batch_inner;
    return p.out + (size_t)bo * p.out_ostride + (size_t)bi * p.out_istride + (size_t)tok * p.ld_tok + sub * hd + d;
}

// Threshold (in bits of the exponent) below which a grown row maximum does not trigger a rescale: the probabilities of later
// keys are then at most 2^8 instead of 1 until the next rescale, which fp32 sums and the bf16 rounding (relative) do not
// mind, and the accumulator is touched a few times per row instead of in most blocks.
constexpr float RESCALE_BITS = 8.0f;
constexpr int FLASH_STAGES = 3;

// The key loop is software-pipelined over 32-key blocks so that every MFMA has independent VALU work to run under: while
// the softmax of block g is computed (VALU), the matrix pipe takes S^T of block g+1 and O^T += V^T P^T of block g-1.
// A block needs 8 MFMAs (256 cycles) and ~65 VALU instructions of one wave; issued back to back by one wave, or by
// several waves in turn, the two streams mostly add up on a SIMD, interleaved one MFMA to a handful of VALU
// instructions they overlap.  Three LDS stages: tile T+2 is requested when tile T-1 has been read by every wave.
template <int HD>
__global__ __launch_bounds__(256, 3)
void flash_kernel(AttnP p, int items_per_batch, int batches_per_xcd) {
    static_assert(HD == 64, "fragment bookkeeping below is written out for a head width of 64");
    constexpr int KD = HD / 32;                         // 32-wide chunks of the head dimension in the fragment layouts
    constexpr int DS = HD / 16;                         // 16-wide steps of the Q K^T contraction
    constexpr int DT2 = HD / 32;                        // 32-wide tiles of the output's head dimension
    constexpr int KBYTES = 64 * HD * 2;                 // one K tile (64 keys); a V^T tile is as large
    constexpr int NPT = KBYTES / 16 / 256;              // 16-byte pieces per thread and operand
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // FLASH_STAGES x { K tile | V^T tile }

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int h = lane >> 5, n = lane & 31;
    // Workgroup ids are dealt round-robin over the 8 XCDs: decode the id so that all row blocks of one K/V head run on
    // one XCD and its K / V^T are fetched into one L2.
    int batch, item;
    if (batches_per_xcd > 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        batch = xcd * batches_per_xcd + idx / items_per_batch; item = idx % items_per_batch;
    } else { batch = blockIdx.x / items_per_batch; item = blockIdx.x % items_per_batch; }
    const bf16_t* const qbase = p.q + (size_t)batch * p.q_bstride;
    const uint4* const kbase = (const uint4*)(p.k + (size_t)batch * p.k_bstride);
    const uint4* const vbase = (const uint4*)(p.vt + (size_t)batch * p.vt_bstride);
    const int row0 = (item * 4 + w) * 32;
    const bool active = row0 < p.rows;                  // a wave past the last row still stages tiles and meets the barriers

    bf16x8 qf[DS];
#pragma unroll
    for (int s4 = 0; s4 < DS; ++s4) {
        const size_t piece = ((size_t)((row0 >> 4) + (n >> 4)) * KD + (s4 >> 1)) * 64 + (2 * (s4 & 1) + h) * 16 + (n & 15);
        qf[s4] = active ? *(const bf16x8*)(qbase + piece * 8) : bf16x8{};
    }
    f32x16 o[DT2];
#pragma unroll
    for (int t = 0; t < DT2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    float m = NEG_BIG, l = 0.f;
    const float c = p.scale * 1.4426950408889634f;
    const float slack = RESCALE_BITS / c;               // the same threshold in units of the raw logits

    const int keys32 = (p.keys + 31) >> 5, ldvt32 = p.ldvt >> 5;
    int ntiles = (p.keys + 63) >> 6;
    if (p.causal) ntiles = min(ntiles, ((min(item * 128 + 128, p.rows) - 1) / p.group >> 6) + 1);

    // Staging: each wave copies whole 1 KB pieces (64 lanes x 16 bytes, contiguous on both sides) from global memory straight
    // into LDS; no staging registers and no LDS write instructions.  Tiles are requested in order, each into the stage after
    // the previous one's.  Only the last tile can reach past the allocated rows (an odd number of 32-key blocks): its second
    // block is then replaced by the first (finite data; those keys are masked below).  A request past the last tile repeats
    // the last tile (into a stage nobody reads any more), so the loops below need no branch around it.
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    const int wu = __builtin_amdgcn_readfirstlane(w);                           // wave-uniform copy: LDS addresses stay scalar
    const unsigned char* ksrc0 = (const unsigned char*)kbase;                   // byte addresses of the next tile (wave-uniform)
    const unsigned char* vsrc0 = (const unsigned char*)vbase;
    unsigned koff[NPT], voff[NPT];                                              // this lane's byte offsets inside a tile
#pragma unroll
    for (int cc = 0; cc < NPT; ++cc) {
        const int i0 = wu * 64 + 256 * cc;                                      // first piece of this wave's 1 KB
        koff[cc] = (unsigned)(i0 + lane) * 16u;
        voff[cc] = (unsigned)(((i0 >> 7) * ldvt32 + ((i0 & 127) >> 6)) * 64 + lane) * 16u;
    }
    const int half_tile = (keys32 & 1) ? (keys32 >> 1) : -1;                    // the tile that holds a single 32-key block
    int next_tile = 0;
    unsigned wr_off = 0;                                                         // LDS byte offset of the stage the next request fills
    auto stage_next = [&]() {
        unsigned char* const dst = smem + wr_off;
        if (next_tile + 1 < ntiles) {                                           // the common case: a whole tile, pointers move on
#pragma unroll
            for (int cc = 0; cc < NPT; ++cc) {
                const int i0 = wu * 64 + 256 * cc;
                __builtin_amdgcn_global_load_lds((gptr_t)(ksrc0 + koff[cc]), (lptr_t)(dst + (size_t)i0 * 16), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(vsrc0 + voff[cc]), (lptr_t)(dst + KBYTES + (size_t)i0 * 16), 16, 0, 0);
            }
            ksrc0 += KBYTES;
            vsrc0 += 128 * 16;
        } else {
            const bool half = ntiles - 1 == half_tile;
#pragma unroll
            for (int cc = 0; cc < NPT; ++cc) {
                const int i0 = wu * 64 + 256 * cc;
                const bool second = ((i0 / (KD * 128)) & 1) != 0;               // K: pieces of keys 32..63 of the tile
                __builtin_amdgcn_global_load_lds((gptr_t)(ksrc0 + koff[cc] - ((half && second) ? KD * 128 * 16 : 0)),
                                                 (lptr_t)(dst + (size_t)i0 * 16), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(vsrc0 + voff[cc] - ((half && ((i0 & 127) >> 6)) ? 64 * 16 : 0)),
                                                 (lptr_t)(dst + KBYTES + (size_t)i0 * 16), 16, 0, 0);
            }
        }
        ++next_tile;
        wr_off = wr_off == (FLASH_STAGES - 1) * 2 * KBYTES ? 0 : wr_off + 2 * KBYTES;
    };

    // fragment reads of a 32-key block: the lane-dependent part of the address is shared by all of them, the stage is a
    // scalar byte offset that rotates once per tile
    const int lane_piece = ((n >> 4) * KD * 64 + h * 16 + (n & 15)) * 16;
    const int lane_piece_v = ((n >> 4) * 2 * 64 + h * 16 + (n & 15)) * 16 + KBYTES;
    auto read_k = [&](unsigned stage_off, int b, bf16x8 (&kf)[DS]) __attribute__((always_inline)) {
        const unsigned char* kt = smem + stage_off + lane_piece;
#pragma unroll
        for (int s4 = 0; s4 < DS; ++s4) kf[s4] = *(const bf16x8*)(kt + ((2 * b * KD + (s4 >> 1)) * 64 + 2 * (s4 & 1) * 16) * 16);
    };
    auto read_v = [&](unsigned stage_off, int b, bf16x8 (&vf)[2][DT2]) __attribute__((always_inline)) {
        const unsigned char* vt = smem + stage_off + lane_piece_v;
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int t = 0; t < DT2; ++t) vf[q][t] = *(const bf16x8*)(vt + ((2 * t * 2 + b) * 64 + 2 * q * 16) * 16);
    };
    const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
    // One pipeline step for block g = 2 T + b.  On entry: s_cur = S^T(g), kf = K fragments of block g+1, vf = V^T fragments and
    // p_prev = probabilities of block g-1.  On exit: s_next = S^T(g+1), kf = K fragments of g+2, vf / p_cur those of block g.
    // `off_v` is the stage of tile T, `off_k` that of the tile block g+2 lies in (T+1).
    auto step = [&](auto edge_tag, int g, int b, unsigned off_v, unsigned off_k, f32x16& s_cur, f32x16& s_next, bf16x8 (&kf)[DS],
                    bf16x8 (&vf)[2][DT2], bf16x8 (&p_prev)[2], bf16x8 (&p_cur)[2]) __attribute__((always_inline)) {
        constexpr bool EDGE = decltype(edge_tag)::value;
        if (EDGE) {      // masks: keys past the end, and (causal) keys after the row's own token
            const int key0 = g * 32;
            const int last = p.causal ? min(p.keys - 1, (row0 + n) / p.group) : p.keys - 1;
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (key0 + 8 * (e >> 2) + 4 * h + (e & 3) > last) s_cur[e] = NEG_BIG;
        }
        float mx0 = s_cur[0], mx1 = s_cur[8];
#pragma unroll
        for (int e = 1; e < 8; ++e) { mx0 = fmaxf(mx0, s_cur[e]); mx1 = fmaxf(mx1, s_cur[8 + e]); }
        const float mx = halves_max(fmaxf(mx0, mx1));
        if (__any(mx > m + slack)) {
            // rare: the accumulator and the pending probabilities of block g-1 (still in the old scale) move to the new one
            const float mnew = fmaxf(m, mx);
            const float alpha = __builtin_amdgcn_exp2f((m - mnew) * c);
            l *= alpha;
#pragma unroll
            for (int t = 0; t < DT2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int j = 0; j < 8; ++j) p_prev[q][j] = (bf16_t)((float)p_prev[q][j] * alpha);
            m = mnew;
        }
        // ---- the straight-line part: 8 MFMAs, the softmax of block g, 8 fragment reads ----
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int t = 0; t < DT2; ++t) o[t] = mfma32(vf[q][t], p_prev[q], o[t]);
        read_v(off_v, b, vf);
#pragma unroll
        for (int e = 0; e < 16; ++e) s_next[e] = 0.f;
#pragma unroll
        for (int s4 = 0; s4 < DS; ++s4) s_next = mfma32(kf[s4], qf[s4], s_next);
        read_k(off_k, b, kf);
        const float mc = m * c;
#pragma unroll
        for (int e = 0; e < 16; ++e) s_cur[e] = __builtin_amdgcn_exp2f(s_cur[e] * c - mc);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            p_cur[q] = pack8(s_cur, q, q + 2);
            // the row sum takes the rounded probabilities, two per instruction (v_dot2_f32_bf16)
#pragma unroll
            for (int j = 0; j < 8; j += 2) l = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{p_cur[q][j], p_cur[q][j + 1]}, ones, l, false);
        }
        // issue order: one MFMA to every six VALU instructions of the softmax; the fragment reads of the next step go into
        // the registers the MFMAs before them have consumed
#pragma unroll
        for (int i = 0; i < 2 * DT2; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x402, 6, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * DT2, 0);
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x402, 6, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, DS, 0);
        __builtin_amdgcn_sched_barrier(0);
    };

    for (int i = 0; i < FLASH_STAGES; ++i) stage_next();
    __builtin_amdgcn_s_waitcnt(0x0f70);                 // vmcnt(0): this wave's pieces are in LDS
    __syncthreads();

    f32x16 sA, sB;
    bf16x8 kf[DS], vf[2][DT2], pP[2], pC[2];
    read_k(0, 0, kf);
#pragma unroll
    for (int e = 0; e < 16; ++e) sA[e] = 0.f;
#pragma unroll
    for (int s4 = 0; s4 < DS; ++s4) sA = mfma32(kf[s4], qf[s4], sA);
    read_k(0, 1, kf);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        pP[q] = bf16x8{};                               // "block -1": zero probabilities, any finite V^T
#pragma unroll
        for (int t = 0; t < DT2; ++t) vf[q][t] = bf16x8{};
    }
    unsigned off_v = 0, off_k = 2 * KBYTES;             // stages of tile T and of tile T+1
    auto tile = [&](auto edge_tag, int T) __attribute__((always_inline)) {
        step(edge_tag, 2 * T, 0, off_v, off_k, sA, sB, kf, vf, pP, pC);
        step(edge_tag, 2 * T + 1, 1, off_v, off_k, sB, sA, kf, vf, pC, pP);   // (K reads past the last tile: stale LDS, never used)
        __builtin_amdgcn_s_waitcnt(0x0f70);             // vmcnt(0): this wave's pieces of tile T+2 have landed
        __syncthreads();                                // ... everybody's have, and everybody is done reading tile T
        stage_next();                                   // tile T+3 into the stage of tile T
        off_v = off_k;
        off_k = off_k == (FLASH_STAGES - 1) * 2 * KBYTES ? 0 : off_k + 2 * KBYTES;
    };
    // only the last tile of a non-causal pass has keys to mask
    const int plain_tiles = p.causal ? 0 : ntiles - 1;
    for (int T = 0; T < plain_tiles; ++T) tile(std::false_type{}, T);
    for (int T = plain_tiles; T < ntiles; ++T) tile(std::true_type{}, T);
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int t = 0; t < DT2; ++t) o[t] = mfma32(vf[q][t], pP[q], o[t]);

    l = halves_sum(l);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const int row = row0 + n;
    if (row < p.rows) {
#pragma unroll
        for (int t = 0; t < DT2; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                store4(flash_out_ptr(p, batch, row, 32 * t + 8 * j + 4 * h, HD),
                       pack4(o[t][4 * j] * inv, o[t][4 * j + 1] * inv, o[t][4 * j + 2] * inv, o[t][4 * j + 3] * inv));
    }
}

}  // namespace

// p as for launch_mqa_attention, without the prefix / state masks and without a key split.  Q must be allocated in whole
// 32-row blocks up to the last valid row, K up to keys rounded up to 32 rows, V^T with p.ldvt >= that many key columns.
int launch_flash_attention(const AttnP& p0, int hd, hipStream_t s) {
    AttnP p = p0;
    if (p.rows <= 0 || p.keys <= 0 || (p.ldvt & 31) || p.ldvt < ((p.keys + 31) / 32) * 32 || p.group < 1) return 1;
    if (p.valid_len || p.state_rows || p.prefix_alloc < p.keys || p.nsplit > 1) return 1;
    if (p.batch < 1) p.batch = 1;
    if (p.batch_inner < 1) p.batch_inner = 1;
    const int items = (p.rows + 127) / 128;
    const int bpx = (p.batch % 8 == 0) ? p.batch / 8 : 0;
    if (hd != 64) return 2;
    hipLaunchKernelGGL((flash_kernel<64>), dim3(items * p.batch), dim3(256), FLASH_STAGES * 2 * 64 * 64 * 2, s, p, items, bpx);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}
