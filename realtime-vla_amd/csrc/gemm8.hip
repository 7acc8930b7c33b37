// Eight-wave variant of the large-M bf16 GEMM (csrc/gemm.hip): the same workgroup tile (MT 32-row tiles x 256 columns),
// the same operand layouts and v_mfma_f32_32x32x16_bf16 product, but the tile is shared by 2 x 4 waves instead of 1 x 4:
// wave (wm, wn) owns the upper or lower half of the row tiles and 64 columns, i.e. at most 128 accumulator registers, so
// TWO waves sit on every SIMD and one wave's waits (LDS reads, weight loads, the barrier) are covered by the other wave's
// MFMAs instead of by a hand-ordered instruction schedule.  The activations go through LDS once per workgroup as before;
// the two waves that share a column slice both read its weight fragments (the second read is served by the CU's vector
// cache, the workgroup runs in step).  Row-major epilogues only (bias, GELU, patch, GeGLU, SwiGLU, split-K partial).
#include "kernels.h"
#include <algorithm>

namespace {

template <int EPI> struct Epi8 { static constexpr bool dual = (EPI == EPI_GEGLU || EPI == EPI_SWIGLU); };

RTVLA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

template <int MT, int EPI>
RTVLA_DEVICE void gemm8_block(const GemmP& p, unsigned char* smem_raw, int m0, int n_blk, int split, int stages_total, int stages_per_split) {
    constexpr int WN = 4, NT = 2, NTH = 512;
    constexpr int BM = MT * 32;
    constexpr int MTW = (MT + 1) / 2;                      // row tiles of the upper wave; the lower one has MT / 2
    constexpr int A_CHUNKS = BM * 8;                       // 16-byte chunks per 64-wide K stage
    constexpr int AIT = (A_CHUNKS + NTH - 1) / NTH;
    constexpr int STAGE_ELEMS = BM * 64;
    constexpr int HALF = Epi8<EPI>::dual ? 1 : 2;
    bf16_t* lds = (bf16_t*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 3, wm = wave >> 2;               // waves w and w + 4 share a SIMD: the two halves of one column slice
    const int h = lane >> 5, r = lane & 31;
    const int i0 = wm ? MTW : 0, mtw = wm ? MT / 2 : MTW;
    const int s_begin = split * stages_per_split;
    const int s_end = min(s_begin + stages_per_split, stages_total);

    int tile_of[NT];
    const bf16_t* bptr[NT];
    const int n32 = (p.N16 + 1) >> 1;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int t = (n_blk * WN + wn) * HALF + (j % HALF);
        tile_of[j] = t;
        const bf16_t* base = (Epi8<EPI>::dual && j >= HALF) ? p.B1 : p.B0;
        const int G = p.bgroup;
        const int tc = min(t, ((n32 + G - 1) / G) * G - 1);
        bptr[j] = base + ((size_t)(tc / G) * (p.K32p * 2) * G + (tc % G)) * 512 + lane * 8;
    }
    const size_t bstep = (size_t)p.bgroup * 512;

    f32x16 acc[MTW][NT];
#pragma unroll
    for (int i = 0; i < MTW; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    bf16x8 areg[AIT];
    bf16x8 breg[NT][4];
    auto load_a = [&](int s) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            const int c = min(it * NTH + tid, A_CHUNKS - 1);
            const int row = c >> 3, kc = c & 7;
            const int gr = min(m0 + row, p.a_rows - 1);
            areg[it] = *(const bf16x8*)(p.A + (size_t)gr * p.lda + s * 64 + kc * 8);
        }
    };
    // same conflict-free slot permutation as the four-wave kernel: chunk (row rr of a 32-row tile, k16 step ks, k half hh)
    // sits at slot 8 ((rr >> 3) + 4 hh) + ((rr + 2 ks + hh) & 7) of fragment (row tile, ks)
    auto store_a = [&](bf16_t* buf) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            const int c = min(it * NTH + tid, A_CHUNKS - 1);
            const int row = c >> 3, kc = c & 7, ks = kc >> 1, hh = kc & 1;
            const int rr = row & 31;
            const int off = ((((row >> 5) * 4 + ks) * 64) + 8 * ((rr >> 3) + 4 * hh) + ((rr + 2 * ks + hh) & 7)) * 8;
            *(bf16x8*)(buf + off) = areg[it];
        }
    };
    auto load_b_half = [&](int s, int kk) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int q = 0; q < 2; ++q) breg[j][2 * kk + q] = *(const bf16x8*)(bptr[j] + (size_t)(s * 4 + 2 * kk + q) * bstep);
    };
    int lane_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) lane_off[ks] = (8 * ((r >> 3) + 4 * h) + ((r + 2 * ks + h) & 7)) * 8;

    const int n_st = s_end - s_begin;
    if (n_st > 0) {
        const int last = s_end - 1;
        load_a(s_begin);
        load_b_half(s_begin, 0); load_b_half(s_begin, 1);
        store_a(lds);
        __syncthreads();
        for (int s = s_begin; s < s_end; ++s) {
            const bf16_t* rd = lds + ((s - s_begin) & 1) * STAGE_ELEMS;
            bf16_t* wr = lds + ((s - s_begin + 1) & 1) * STAGE_ELEMS;
            const int sn = min(s + 1, last);                 // past the end the prefetch re-reads the last stage
            load_a(sn);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int ks = 2 * kk + q;
#pragma unroll
                    for (int i = 0; i < MTW; ++i) {
                        if (i < mtw) {
                            const bf16x8 af = *(const bf16x8*)(rd + ((i0 + i) * 4 + ks) * 512 + lane_off[ks]);
#pragma unroll
                            for (int j = 0; j < NT; ++j) acc[i][j] = mfma32(breg[j][ks], af, acc[i][j]);
                        }
                    }
                }
                load_b_half(sn, kk);                         // this half's weight registers are free again
            }
            store_a(wr);
            __syncthreads();
        }
    }

    if constexpr (EPI == EPI_VIT_QKV_ROPE) {
        // DM0 ViT (dm0_infer.py:589-598), as in the four-wave kernel: + fp32 bias, rounded to bf16, 2-D rotary embedding on Q and
        // K, per (image, head) Q and K as fragment-tiled [seq_pad][64] (16-byte pieces after a half swap between lane pairs),
        // V^T transposed through a wave-private 2.3 KB of LDS into whole pieces of the permuted-key fragments
#pragma unroll
        for (int k = 0; k < MTW; ++k) {
            const int m = m0 + (i0 + k) * 32 + r;
            if (k >= mtw || m0 + (i0 + k) * 32 >= p.M) continue;
            const int img = m / p.seq_pad, tok = m - img * p.seq_pad;
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int nt0 = tile_of[j] * 32;
                if (nt0 >= p.N16 * 16) continue;
                const int which = nt0 >> 10, head = (nt0 & 1023) >> 6, d0 = nt0 & 63;
                const size_t vh = (size_t)(img * 16 + head);
                uint2 qk[4];
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int n0 = nt0 + 8 * grp + 4 * h;
                    f32x4 v = {acc[k][j][4 * grp], acc[k][j][4 * grp + 1], acc[k][j][4 * grp + 2], acc[k][j][4 * grp + 3]};
                    v += *(const f32x4*)(p.bias_f32 + n0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = round_bf16(v[e]);
                    if (which < 2) {
                        const bf16x4 cs = load4(p.rope + (size_t)min(tok, p.seq - 1) * 64 + d0 + 8 * grp + 4 * h);
                        const float c0 = bf2f(cs[0]), s0 = bf2f(cs[1]), c1 = bf2f(cs[2]), s1 = bf2f(cs[3]);
                        const f32x4 w = v;
                        v[0] = w[0] * c0 - w[1] * s0; v[1] = w[1] * c0 + w[0] * s0;
                        v[2] = w[2] * c1 - w[3] * s1; v[3] = w[3] * c1 + w[2] * s1;
                        const bf16x4 pk = pack4(v);
                        qk[grp] = *(const uint2*)&pk;
                    } else {
                        volatile bf16_t* tb = (volatile bf16_t*)(smem_raw + wave * 2304);
#pragma unroll
                        for (int e = 0; e < 4; ++e) tb[(8 * grp + 4 * h + e) * 36 + r] = f2bf(v[e]);
                    }
                }
                if (which < 2) {
                    bf16_t* const dst = (which == 0 ? p.q : p.k) + vh * ((size_t)p.seq_pad * 64);
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        const uint2 keep = h ? qk[2 * pr + 1] : qk[2 * pr], send = h ? qk[2 * pr] : qk[2 * pr + 1];
                        const uint2 recv = {(unsigned)__shfl_xor((int)send.x, 32, 64), (unsigned)__shfl_xor((int)send.y, 32, 64)};
                        *(uint4*)(dst + ft_index(tok, d0 + 8 * (2 * pr + h), 2)) = h ? uint4{recv.x, recv.y, keep.x, keep.y} : uint4{keep.x, keep.y, recv.x, recv.y};
                    }
                } else {
                    const int tok0 = tok - r;
                    const int gq = lane >> 4, rq = lane & 15;
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt) {
                        const volatile uint2* src = (const volatile uint2*)(smem_raw + wave * 2304 + (16 * dt + rq) * 72 + gq * 8);
                        const uint2 lo = {src[0].x, src[0].y}, hi = {src[4].x, src[4].y};
                        const size_t frag = (size_t)(((d0 >> 4) + dt) * (p.seq_pad >> 5) + (tok0 >> 5)) * 64 + lane;
                        *(uint4*)(p.vt + vh * ((size_t)64 * p.seq_pad) + frag * 8) = uint4{lo.x, lo.y, hi.x, hi.y};
                    }
                }
            }
        }
        return;
    }
    // ---- epilogue: lane (h, r) holds rows m0 + 32 (i0 + i) + r, columns 32 tile + 8 grp + 4 h + e.  The k-th row tiles of
    // the two wave halves are converted into two LDS tiles and copied out together as 16-byte chunks of row segments.
    constexpr int ESZ = (EPI == EPI_PARTIAL) ? 4 : 2;
    constexpr int OUTW = WN * HALF * 32;
    constexpr int ROWB = OUTW * ESZ + 16;
    constexpr int CPR = OUTW * ESZ / 16;
    constexpr int TILE_B = 32 * ROWB;
    constexpr int CIT = 2 * 32 * CPR / NTH;
    static_assert((2 * 32 * CPR) % NTH == 0, "copy-out mapping");
    unsigned char* obuf = smem_raw;
    const int nbase = n_blk * OUTW;
    const int ncols = p.N16 * 16;
#pragma unroll
    for (int k = 0; k < MTW; ++k) {
        const int i = i0 + k;
        if (k < mtw && m0 + i * 32 < p.M) {
            const int m = m0 + i * 32 + r;
            unsigned char* const tbuf = obuf + wm * TILE_B;
#pragma unroll
            for (int j = 0; j < HALF; ++j) {
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int cl = (wn * HALF + j) * 32 + 8 * grp + 4 * h;
                    const int n0 = min(nbase + cl, ncols - 4);
                    f32x4 v = {acc[k][j][4 * grp], acc[k][j][4 * grp + 1], acc[k][j][4 * grp + 2], acc[k][j][4 * grp + 3]};
                    unsigned char* dst = tbuf + r * ROWB + cl * ESZ;
                    if constexpr (EPI == EPI_PARTIAL) {
                        *(f32x4*)dst = v;
                    } else if constexpr (EPI == EPI_GEGLU) {
                        const f32x4 u = {acc[k][j + HALF][4 * grp], acc[k][j + HALF][4 * grp + 1], acc[k][j + HALF][4 * grp + 2], acc[k][j + HALF][4 * grp + 3]};
                        *(bf16x4*)dst = pack4(gelu_tanh(v[0]) * u[0], gelu_tanh(v[1]) * u[1], gelu_tanh(v[2]) * u[2], gelu_tanh(v[3]) * u[3]);
                    } else if constexpr (EPI == EPI_SWIGLU) {
                        const float f = p.rowscale[min(m, p.M - 1)];
                        f32x4 u = {acc[k][j + HALF][4 * grp], acc[k][j + HALF][4 * grp + 1], acc[k][j + HALF][4 * grp + 2], acc[k][j + HALF][4 * grp + 3]};
                        v *= f; u *= f;
                        *(bf16x4*)dst = pack4(siluf(v[0]) * u[0], siluf(v[1]) * u[1], siluf(v[2]) * u[2], siluf(v[3]) * u[3]);
                    } else {
                        if (p.bias_f32) v += *(const f32x4*)(p.bias_f32 + n0);
                        else {
                            const bf16x4 b = load4(p.bias + n0);
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] += bf2f(b[e]);
                        }
                        if constexpr (EPI == EPI_PATCH) {
                            const bf16x4 rs = load4(p.res + (size_t)(min(m, p.M - 1) % p.res_mod) * p.ldr + n0);
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] += bf2f(rs[e]);
                        }
                        if constexpr (EPI == EPI_BIAS_GELU) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
                        }
                        *(bf16x4*)dst = pack4(v);
                    }
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < CIT; ++it) {
            const int idx = it * NTH + tid;
            const int half = idx / (32 * CPR), rem = idx - half * (32 * CPR);
            const int row = rem / CPR, ch = rem - row * CPR;
            const int ii = (half ? MTW : 0) + k;
            const int mm = m0 + ii * 32 + row;
            const int n = nbase + ch * (16 / ESZ);
            if (k < (half ? MT / 2 : MTW) && mm < p.M && n < ncols) {
                const uint4 val = *(const uint4*)(obuf + half * TILE_B + row * ROWB + ch * 16);
                if constexpr (EPI == EPI_PARTIAL) *(uint4*)(p.partial + (size_t)split * p.pstride + (size_t)mm * p.ldp + n) = val;
                else *(uint4*)(p.out + (size_t)mm * p.ldo + n) = val;
            }
        }
        if (k + 1 < MTW) __syncthreads();
    }
}

template <int MT, int EPI, bool MIXED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(MT <= 4 ? 4 : 2, MT <= 4 ? 4 : 2)))
void gemm8_kernel(GemmP p, int m_blocks, int n_blocks, int stages_total, int stages_per_split, int n_big) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int total = m_blocks * n_blocks * p.nsplit;
    const int lid = xcd_remap(blockIdx.x, total);
    const int split = lid / (m_blocks * n_blocks);
    const int rem = lid - split * (m_blocks * n_blocks);
    const int n_blk = rem / m_blocks;
    const int m_blk = rem - n_blk * m_blocks;
    if constexpr (MIXED) {
        if (m_blk < n_big) gemm8_block<MT, EPI>(p, smem_raw, m_blk * (MT * 32), n_blk, split, stages_total, stages_per_split);
        else gemm8_block<MT - 1, EPI>(p, smem_raw, n_big * (MT * 32) + (m_blk - n_big) * ((MT - 1) * 32), n_blk, split, stages_total, stages_per_split);
    } else {
        gemm8_block<MT, EPI>(p, smem_raw, m_blk * (MT * 32), n_blk, split, stages_total, stages_per_split);
    }
}

template <int MT, int EPI>
int launch8_cfg(const GemmP& p, hipStream_t s) {
    constexpr int HALF = Epi8<EPI>::dual ? 1 : 2;
    constexpr int ESZ = (EPI == EPI_PARTIAL) ? 4 : 2;
    const int tiles = (p.M + 31) / 32;
    const int m_blocks = (tiles + MT - 1) / MT;
    int n_big = tiles - m_blocks * (MT - 1);
    if (n_big < 0) n_big = 0;
    const int n_blocks = ((p.N16 + 1) / 2 + 4 * HALF - 1) / (4 * HALF);
    const int stages_total = p.K32p / 2;
    const int nsplit = p.nsplit < 1 ? 1 : p.nsplit;
    const int sps = (stages_total + nsplit - 1) / nsplit;
    if ((nsplit - 1) * sps >= stages_total) return 3;
    GemmP q = p; q.nsplit = nsplit;
    const size_t smem = std::max((size_t)2 * MT * 32 * 64 * 2, (size_t)2 * 32 * (4 * HALF * 32 * ESZ + 16));
    auto kern = gemm8_kernel<MT, EPI, true>;
    if (smem > 65536) {
        static std::atomic<uint64_t> done{0};
        if (int rc = ensure_dynamic_lds((const void*)kern, smem, done)) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(m_blocks * n_blocks * nsplit), dim3(512), smem, s, q, m_blocks, n_blocks, stages_total, sps, n_big);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

template <int EPI>
int launch8_epi(const GemmP& p, int tile, hipStream_t s) {
    switch (tile) {
        case TILE8_256x256: return launch8_cfg<8, EPI>(p, s);
        case TILE8_224x256: return launch8_cfg<7, EPI>(p, s);
        case TILE8_192x256: return launch8_cfg<6, EPI>(p, s);
        case TILE8_128x256: return launch8_cfg<4, EPI>(p, s);
    }
    return 2;
}

}  // namespace

int launch_gemm8(const GemmP& p, int epi, int tile, hipStream_t s) {
    if (p.M <= 0 || p.N16 <= 0 || p.K32p <= 0 || (p.K32p & 1) || p.a_rows <= 0 || p.bgroup < 1) return 1;
    if (epi != EPI_PARTIAL && p.nsplit > 1) return 1;
    switch (epi) {
        case EPI_BIAS:      return launch8_epi<EPI_BIAS>(p, tile, s);
        case EPI_BIAS_GELU: return launch8_epi<EPI_BIAS_GELU>(p, tile, s);
        case EPI_GEGLU:     return launch8_epi<EPI_GEGLU>(p, tile, s);
        case EPI_PARTIAL:   return launch8_epi<EPI_PARTIAL>(p, tile, s);
        case EPI_SWIGLU:    return launch8_epi<EPI_SWIGLU>(p, tile, s);
        case EPI_VIT_QKV_ROPE: return launch8_epi<EPI_VIT_QKV_ROPE>(p, tile, s);
    }
    return 2;
}
