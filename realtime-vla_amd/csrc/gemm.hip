// Large-M bf16 GEMM on MFMA for the SigLIP and Gemma-prefix layers
// (replaces the Triton GEMM family of /root/reference/pi0_infer.py:5-346, :664-691, :777-810).
//
// out[M][N] = epilogue(A[M][K] * W[K][N]).  The activations A are staged through LDS in MFMA
// operand-fragment order (each wave reads whole 1 KB fragments with ds_read_b128, conflict
// free) and are shared by all waves of the workgroup; the weights are read straight from
// their pre-tiled layout in HBM into registers (one coalesced 1 KB load per fragment, no LDS
// round trip), each wave owning its own column tiles.  The product is computed transposed
// (weights as the MFMA A operand) so that every lane ends up with 4 consecutive output columns
// of one row: 8-byte packed stores, and RoPE pairs / GeGLU partners sit in the same lane.
#include "kernels.h"

namespace {

template <int EPI> struct EpiTraits { static constexpr bool dual = (EPI == EPI_GEGLU); };

// tiles of at most 128 rows are compiled to fit two workgroups per CU (<= 256 registers per lane) so
// that one workgroup's MFMAs run under the other's memory latency
template <int WN, int MT, int NT, int EPI>
__global__ __launch_bounds__(WN * 64, (MT <= 8 ? 2 : 1))
void gemm_mfma_kernel(GemmP p, int m_blocks, int n_blocks, int stages_total, int stages_per_split) {
    constexpr int NTH = WN * 64;
    constexpr int BM = MT * 16;
    constexpr int A_CHUNKS = BM * 8;                       // 16-byte chunks per 64-wide K stage
    constexpr int AIT = (A_CHUNKS + NTH - 1) / NTH;
    constexpr int STAGE_ELEMS = BM * 64;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    bf16_t* lds = (bf16_t*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wn = tid >> 6;
    const int g = lane >> 4, r = lane & 15;

    const int total = m_blocks * n_blocks * p.nsplit;
    const int lid = xcd_remap(blockIdx.x, total);
    const int split = lid / (m_blocks * n_blocks);
    const int rem = lid - split * (m_blocks * n_blocks);
    const int n_blk = rem / m_blocks;
    const int m_blk = rem - n_blk * m_blocks;
    const int m0 = m_blk * BM;
    const int s_begin = split * stages_per_split;
    const int s_end = min(s_begin + stages_per_split, stages_total);

    // column tiles of this wave
    constexpr int HALF = EpiTraits<EPI>::dual ? NT / 2 : NT;
    int tile_of[NT];
    const bf16_t* bptr[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int t = (n_blk * WN + wn) * HALF + (j % HALF);
        tile_of[j] = t;
        const bf16_t* base = (EpiTraits<EPI>::dual && j >= HALF) ? p.B1 : p.B0;
        const int G = p.bgroup;
        const int tc = min(t, ((p.N16 + G - 1) / G) * G - 1);
        bptr[j] = base + ((size_t)(tc / G) * p.K32p * G + (tc % G)) * 512 + lane * 8;
    }

    const size_t bstep = (size_t)p.bgroup * 512;          // distance between consecutive k32 blocks of one column tile
    f32x4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    bf16x8 areg[AIT];
    bf16x8 breg0[NT][2], breg1[NT][2];

    // LDS stage layout: fragment (row tile i, k half kk) is 1 KB, lane (g, r) at slot (r ^ 8 kk) + 16 g.
    // The xor spreads the 64 lanes of a staging write (8 rows x 8 chunks) over all banks; a
    // fragment read still touches every bank exactly once.
    auto load_a = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            // a ragged last round re-reads the final chunk instead of branching
            const int c = min(it * NTH + tid, A_CHUNKS - 1);
            const int row = c >> 3, kc = c & 7;
            const int gr = min(m0 + row, p.a_rows - 1);
            areg[it] = *(const bf16x8*)(p.A + (size_t)gr * p.lda + s * 64 + kc * 8);
        }
    };
    auto store_a = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            const int c = min(it * NTH + tid, A_CHUNKS - 1);      // duplicates write identical data
            const int row = c >> 3, kc = c & 7, kk = kc >> 2;
            const int off = ((((row >> 4) * 2 + kk) * 64) + ((row & 15) ^ (kk << 3)) + 16 * (kc & 3)) * 8;
            *(bf16x8*)(lds + buf * STAGE_ELEMS + off) = areg[it];
        }
    };
    auto load_b = [&](int s, bf16x8 (&br)[NT][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
                br[j][kk] = *(const bf16x8*)(bptr[j] + (size_t)(s * 2 + kk) * bstep);
    };
    const int lane_off[2] = {(r + 16 * g) * 8, ((r ^ 8) + 16 * g) * 8};
    auto compute = [&](int buf, bf16x8 (&br)[NT][2]) __attribute__((always_inline)) {
        const bf16_t* base = lds + buf * STAGE_ELEMS;
        // all A fragments of the stage are requested from LDS before the first MFMA waits on one
        bf16x8 af[2][MT];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int i = 0; i < MT; ++i) af[kk][i] = *(const bf16x8*)(base + (i * 2 + kk) * 512 + lane_off[kk]);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) acc[i][j] = mfma16(br[j][kk], af[kk][i], acc[i][j]);
        // instruction order for the scheduler: PRE fragment reads ahead, then per further read NT MFMAs
        // and one of the next stage's global loads, so that load issue runs under the MFMAs
        constexpr int PRE = 4;
        constexpr int NLOADS = AIT + 2 * NT;
        __builtin_amdgcn_sched_group_barrier(0x100, PRE, 0);
#pragma unroll
        for (int t = 0; t < 2 * MT - PRE; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (t < NLOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
#pragma unroll
        for (int t = 0; t < PRE; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);
            if (t + 2 * MT - PRE < NLOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
    };

    // K loop: the loads of stage s+1 fly under the MFMAs of stage s (register-staged A, weights in
    // a second register set); two stages per trip so the sets alternate without a runtime index and
    // the body has a single exit.  Past the end the prefetch re-reads the last stage instead of
    // branching around the loads.
    const int n_st = s_end - s_begin;
    if (n_st > 0) {
        const int last = s_end - 1;
        load_a(s_begin);
        load_b(s_begin, breg0);
        store_a(0);
        __syncthreads();
        for (int s = s_begin; s < s_end; s += 2) {          // the host guarantees an even stage count per split
            load_a(s + 1); load_b(s + 1, breg1);
            compute(0, breg0);
            __builtin_amdgcn_sched_barrier(0);
            store_a(1);
            __syncthreads();
            load_a(min(s + 2, last)); load_b(min(s + 2, last), breg0);
            compute(1, breg1);
            __builtin_amdgcn_sched_barrier(0);
            store_a(0);
            __syncthreads();
        }
    }

    // ---- epilogue: lane (g, r) holds rows m = m0 + 16 i + r, columns n = 16 tile + 4 g + v ----
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = m0 + i * 16 + r;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < HALF; ++j) {
            const int t = tile_of[j];
            if (t >= p.N16) continue;
            const int n0 = t * 16 + 4 * g;
            f32x4 v = acc[i][j];
            if constexpr (EPI == EPI_PARTIAL) {
                *(f32x4*)(p.partial + (size_t)split * p.pstride + (size_t)m * p.ldp + n0) = v;
            } else if constexpr (EPI == EPI_GEGLU) {
                const f32x4 u = acc[i][j + HALF];
                store4(p.out + (size_t)m * p.ldo + n0,
                       pack4(gelu_tanh(v[0]) * u[0], gelu_tanh(v[1]) * u[1], gelu_tanh(v[2]) * u[2], gelu_tanh(v[3]) * u[3]));
            } else if constexpr (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU || EPI == EPI_PATCH) {
                const bf16x4 b = load4(p.bias + n0);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += bf2f(b[e]);
                if constexpr (EPI == EPI_PATCH) {
                    const bf16x4 rs = load4(p.res + (size_t)(m % p.res_mod) * p.ldr + n0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += bf2f(rs[e]);
                }
                if constexpr (EPI == EPI_BIAS_GELU) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
                }
                store4(p.out + (size_t)m * p.ldo + n0, pack4(v));
            } else if constexpr (EPI == EPI_QKV_ROPE) {
                // the reference rounds the accumulator to bf16 before the rotation (pi0_infer.py:793)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = round_bf16(v[e]);
                if (n0 < 2304) {
                    const bf16x4 cs = load4(p.rope + (size_t)m * 256 + (n0 & 255));
                    const float c0 = bf2f(cs[0]), s0 = bf2f(cs[1]), c1 = bf2f(cs[2]), s1 = bf2f(cs[3]);
                    const f32x4 w = v;
                    v[0] = w[0] * c0 - w[1] * s0; v[1] = w[1] * c0 + w[0] * s0;
                    v[2] = w[2] * c1 - w[3] * s1; v[3] = w[3] * c1 + w[2] * s1;
                    // Q rows are token*8 + head; Q and K are kept fragment-tiled for the attention kernel
                    if (n0 < 2048) store4(p.q + ft_index(m * 8 + (n0 >> 8), n0 & 255, 8), pack4(v));
                    else store4(p.k + ft_index(m, n0 - 2048, 8), pack4(v));
                } else {
                    const int d = n0 - 2304;
#pragma unroll
                    for (int e = 0; e < 4; ++e) p.vt[vt_index(d + e, m, p.ldvt >> 5)] = f2bf(v[e]);
                }
            } else if constexpr (EPI == EPI_VIS_QKV) {
                const bf16x4 b = load4(p.bias + n0);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += bf2f(b[e]);
                // per (view, head): Q and K as fragment-tiled [256 tokens][96] (72 padded), V^T as [80][256]
                const int which = n0 / 1152, c = n0 - which * 1152, head = c / 72, d = c - head * 72;
                const int view = m >> 8, tok = m & 255;
                const size_t vh = (size_t)(view * 16 + head);
                if (which == 0) store4(p.q + vh * (256 * 96) + ft_index(tok, d, 3), pack4(v));
                else if (which == 1) store4(p.k + vh * (256 * 96) + ft_index(tok, d, 3), pack4(v));
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) p.vt[vh * (80 * 256) + vt_index(d + e, tok, 8)] = f2bf(v[e]);
                }
            }
        }
    }
}

template <int WN, int MT, int NT, int EPI>
int launch_cfg(const GemmP& p, hipStream_t s) {
    constexpr int BM = MT * 16;
    constexpr int HALF = EpiTraits<EPI>::dual ? NT / 2 : NT;
    const int m_blocks = (p.M + BM - 1) / BM;
    const int n_blocks = (p.N16 + WN * HALF - 1) / (WN * HALF);
    const int stages_total = p.K32p / 2;
    const int nsplit = p.nsplit < 1 ? 1 : p.nsplit;
    const int sps = (stages_total + nsplit - 1) / nsplit;
    if ((nsplit - 1) * sps >= stages_total) return 3;      // an empty split would leave its partial unwritten
    if ((sps & 1) || (stages_total & 1)) return 3;          // the kernel consumes K stages in pairs
    GemmP q = p; q.nsplit = nsplit;
    const size_t smem = (size_t)2 * BM * 64 * sizeof(bf16_t);
    auto kern = gemm_mfma_kernel<WN, MT, NT, EPI>;
    if (smem > 65536) {
        static bool done = false;
        if (!done) { if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return 4; done = true; }
    }
    hipLaunchKernelGGL(kern, dim3(m_blocks * n_blocks * nsplit), dim3(WN * 64), smem, s, q, m_blocks, n_blocks, stages_total, sps);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

template <int EPI>
int launch_epi(const GemmP& p, int tile, hipStream_t s) {
    switch (tile) {
        case TILE_256x256: return launch_cfg<4, 16, 4, EPI>(p, s);
        case TILE_208x256: return launch_cfg<4, 13, 4, EPI>(p, s);
        case TILE_128x256: return launch_cfg<4, 8, 4, EPI>(p, s);
        case TILE_128x128: return launch_cfg<4, 8, 2, EPI>(p, s);
        case TILE_64x256:  return launch_cfg<4, 4, 4, EPI>(p, s);
    }
    return 2;
}

}  // namespace

int gemm_tile_bm(int tile) { static const int v[TILE_COUNT] = {256, 208, 128, 128, 64}; return v[tile]; }
int gemm_tile_bn(int tile) { static const int v[TILE_COUNT] = {256, 256, 256, 128, 256}; return v[tile]; }

int launch_gemm(const GemmP& p, int epi, int tile, hipStream_t s) {
    if (p.M <= 0 || p.N16 <= 0 || p.K32p <= 0 || (p.K32p & 1) || p.a_rows <= 0 || p.bgroup < 1) return 1;
    if (epi != EPI_PARTIAL && p.nsplit > 1) return 1;
    switch (epi) {
        case EPI_BIAS:      return launch_epi<EPI_BIAS>(p, tile, s);
        case EPI_BIAS_GELU: return launch_epi<EPI_BIAS_GELU>(p, tile, s);
        case EPI_PATCH:     return launch_epi<EPI_PATCH>(p, tile, s);
        case EPI_GEGLU:     return launch_epi<EPI_GEGLU>(p, tile, s);
        case EPI_PARTIAL:   return launch_epi<EPI_PARTIAL>(p, tile, s);
        case EPI_QKV_ROPE:  return launch_epi<EPI_QKV_ROPE>(p, tile, s);
        case EPI_VIS_QKV:   return launch_epi<EPI_VIS_QKV>(p, tile, s);
    }
    return 2;
}
