// Softmax attention for long query AND key sequences on v_mfma_f32_32x32x16_bf16, flash style: DM0's ViT attention,
// 2705 tokens per (image, head), head width 64 (/root/reference/dm0_infer.py:589-598), 3 x 16 independent heads.
//
// One workgroup = 4 waves = 128 consecutive query rows of one K/V head; each wave owns 32 query rows and walks ALL keys,
// so there is no merge at the end.  K and V^T tiles of 64 keys are staged through LDS (double buffered, one barrier per
// tile) and shared by the four waves: the L2 port of a CU (64 B/clk) carries each tile once per 128 query rows instead
// of once per wave.  The tiles keep the byte layout they have in memory (MFMA fragments of 1 KB: Q and K fragment-tiled
// [rows][HD], V^T in the permuted-key layout), so staging is a plain 16-byte copy per thread and every operand read is a
// conflict-free ds_read_b128.
//
// Per 32-key block the wave computes S^T = K Q^T (32 keys x 32 queries): lane (h = lane / 32, n = lane % 32) holds the 16
// logits of query n for keys 8 j + 4 h + v.  The softmax statistics are therefore per-lane scalars shared with ONE other
// lane, the running sum is kept per lane and combined once at the end, and the accumulator is only rescaled when some
// row's maximum actually grew (a wave-uniform branch; after the first few tiles it is rarely taken).  The probabilities
// of accumulator groups j = q and j = q + 2 are, packed to bf16, exactly the B operand of O^T += V^T P^T for the q-th
// 16-key step in the key order of the stored V^T: no shuffles between the two products.
#include "kernels.h"

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

template <int HD>
__global__ __launch_bounds__(256)
void flash_kernel(AttnP p, int items_per_batch, int batches_per_xcd) {
    constexpr int KD = HD / 32;                         // 32-wide chunks of the head dimension in the fragment layouts
    constexpr int DS = HD / 16;                         // 16-wide steps of the Q K^T contraction
    constexpr int DT2 = HD / 32;                        // 32-wide tiles of the output's head dimension
    constexpr int KBYTES = 64 * HD * 2;                 // one K tile (64 keys); a V^T tile is as large
    constexpr int NPT = KBYTES / 16 / 256;              // 16-byte pieces per thread and operand
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // 2 stages x { K tile | V^T tile }

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

    const int keys32 = (p.keys + 31) >> 5, ldvt32 = p.ldvt >> 5;
    int ntiles = (p.keys + 63) >> 6;
    if (p.causal) ntiles = min(ntiles, ((min(item * 128 + 128, p.rows) - 1) / p.group >> 6) + 1);

    uint4 stg[2 * NPT];
    auto gload = [&](int T) {
#pragma unroll
        for (int cc = 0; cc < NPT; ++cc) {
            const int i = tid + 256 * cc;
            const int tile16 = T * 4 + i / (KD * 64);
            stg[cc] = tile16 * 16 < keys32 * 32 ? kbase[(size_t)T * (KBYTES / 16) + i] : uint4{0, 0, 0, 0};
            const int dt = i >> 7, within = i & 127, blk = 2 * T + (within >> 6);
            stg[NPT + cc] = blk < keys32 ? vbase[((size_t)dt * ldvt32 + 2 * T) * 64 + within] : uint4{0, 0, 0, 0};
        }
    };
    auto lstore = [&](int stage) {
        uint4* dst = (uint4*)(smem + (size_t)stage * 2 * KBYTES);
#pragma unroll
        for (int cc = 0; cc < NPT; ++cc) { dst[tid + 256 * cc] = stg[cc]; dst[KBYTES / 16 + tid + 256 * cc] = stg[NPT + cc]; }
    };

    gload(0);
    lstore(0);
    __syncthreads();
    for (int T = 0; T < ntiles; ++T) {
        const bool more = T + 1 < ntiles;
        if (more) gload(T + 1);
        const bf16x8* const kt = (const bf16x8*)(smem + (size_t)(T & 1) * 2 * KBYTES);
        const bf16x8* const vt = kt + KBYTES / 16;
        f32x16 s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int e = 0; e < 16; ++e) s[b][e] = 0.f;
#pragma unroll
            for (int s4 = 0; s4 < DS; ++s4)
                s[b] = mfma32(kt[((2 * b + (n >> 4)) * KD + (s4 >> 1)) * 64 + (2 * (s4 & 1) + h) * 16 + (n & 15)], qf[s4], s[b]);
        }
        // masks: keys past the end, and (causal) keys after the row's own token
        const int key0 = T * 64;
        const int row = row0 + n;
        const bool edge = key0 + 64 > p.keys || (p.causal && key0 + 63 > row0 / p.group);
        if (edge) {
            const int last = p.causal ? min(p.keys - 1, row / p.group) : p.keys - 1;
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (key0 + b * 32 + 8 * (e >> 2) + 4 * h + (e & 3) > last) s[b][e] = NEG_BIG;
        }
        float mx = s[0][0];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[b][e]);
        mx = halves_max(mx);
        if (__any(mx > m)) {
            const float mnew = fmaxf(m, mx);
            const float alpha = __builtin_amdgcn_exp2f((m - mnew) * c);
            l *= alpha;
#pragma unroll
            for (int t = 0; t < DT2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
            m = mnew;
        }
        const float mc = m * c;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) { s[b][e] = __builtin_amdgcn_exp2f(s[b][e] * c - mc); l += s[b][e]; }
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const bf16x8 pb = pack8(s[b], q, q + 2);
#pragma unroll
                for (int t = 0; t < DT2; ++t)
                    o[t] = mfma32(vt[((2 * t + (n >> 4)) * 2 + b) * 64 + (2 * q + h) * 16 + (n & 15)], pb, o[t]);
            }
        if (more) lstore((T + 1) & 1);
        __syncthreads();
    }

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
    hipLaunchKernelGGL((flash_kernel<64>), dim3(items * p.batch), dim3(256), 4 * 64 * 64 * 2, s, p, items, bpx);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}
