// Large-M bf16 GEMM on MFMA for the SigLIP and Gemma-prefix layers
// (replaces the Triton GEMM family of /root/reference/pi0_infer.py:5-346, :664-691, :777-810).
//
// out[M][N] = epilogue(A[M][K] * W[K][N]) with v_mfma_f32_32x32x16_bf16: measured on MI355X this
// instruction sustains ~2.1 PFLOP/s with a single wave per SIMD, while streams of independent
// 16x16x32 MFMAs issue at half that rate.  The activations A are staged through LDS in MFMA
// operand-fragment order (each wave reads whole 1 KB fragments with ds_read_b128, conflict free) and
// are shared by all waves of the workgroup; the weights are read straight from their pre-tiled layout
// in HBM into registers (one coalesced 1 KB load per fragment, no LDS round trip), each wave owning
// its own column tiles.  The product is computed transposed (weights as the MFMA A operand) so that
// every lane ends up with 4 groups of 4 consecutive output columns of one row: 8-byte packed stores,
// and RoPE pairs / GeGLU partners sit in the same lane.
#include "kernels.h"
#include <algorithm>

namespace {

template <int EPI> struct EpiTraits { static constexpr bool dual = (EPI == EPI_GEGLU || EPI == EPI_SWIGLU); };

RTVLA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

// MT, NT: 32-row tiles per workgroup and 32-column tiles per wave.  Small tiles are compiled to fit two
// workgroups per CU so that one workgroup's MFMAs run under the other's memory latency.
// One block tile of MT 32-row tiles starting at row m0: K loop and epilogue.
template <int WN, int MT, int NT, int EPI>
RTVLA_DEVICE void gemm_block(const GemmP& p, unsigned char* smem_raw, int m0, int n_blk, int split, int stages_total, int stages_per_split) {
    constexpr int NTH = WN * 64;
    constexpr int BM = MT * 32;
    constexpr int A_CHUNKS = BM * 8;                       // 16-byte chunks per 64-wide K stage
    constexpr int AIT = (A_CHUNKS + NTH - 1) / NTH;
    constexpr int STAGE_ELEMS = BM * 64;
    bf16_t* lds = (bf16_t*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wn = tid >> 6;
    const int h = lane >> 5, r = lane & 31;
    const int s_begin = split * stages_per_split;
    const int s_end = min(s_begin + stages_per_split, stages_total);

    // 32-column tiles of this wave
    constexpr int HALF = EpiTraits<EPI>::dual ? NT / 2 : NT;
    int tile_of[NT];
    const bf16_t* bptr[NT];
    const int n32 = (p.N16 + 1) >> 1;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int t = (n_blk * WN + wn) * HALF + (j % HALF);
        tile_of[j] = t;
        const bf16_t* base = (EpiTraits<EPI>::dual && j >= HALF) ? p.B1 : p.B0;
        const int G = p.bgroup;
        const int tc = min(t, ((n32 + G - 1) / G) * G - 1);
        bptr[j] = base + ((size_t)(tc / G) * (p.K32p * 2) * G + (tc % G)) * 512 + lane * 8;
    }

    const size_t bstep = (size_t)p.bgroup * 512;          // distance between consecutive k16 blocks of one column tile
    f32x16 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    bf16x8 areg0[AIT], areg1[AIT];
    bf16x8 breg0[NT][4], breg1[NT][4];

    // LDS stage layout: fragment (row tile i, k16 step ks) is 1 KB = 64 slots of 16 bytes; the chunk of row r
    // (0..31) and k half hh sits at slot 8 ((r >> 3) + 4 hh) + ((r + 2 ks + hh) & 7).  The low three bits pick
    // the 128-byte bank group: any 8 consecutive lanes of a fragment read (8 rows, one hh) and any 8
    // consecutive lanes of a staging write (one row, 8 chunks = 4 ks x 2 hh) land in 8 different bank
    // groups, so neither side conflicts.
    auto load_a = [&](int s, bf16x8 (&ar)[AIT]) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            // a ragged last round re-reads the final chunk instead of branching
            const int c = min(it * NTH + tid, A_CHUNKS - 1);
            const int row = c >> 3, kc = c & 7;
            const int gr = min(m0 + row, p.a_rows - 1);
            ar[it] = *(const bf16x8*)(p.A + (size_t)gr * p.lda + s * 64 + kc * 8);
        }
    };
    auto store_a = [&](bf16_t* buf, bf16x8 (&ar)[AIT]) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < AIT; ++it) {
            const int c = min(it * NTH + tid, A_CHUNKS - 1);      // duplicates write identical data
            const int row = c >> 3, kc = c & 7, ks = kc >> 1, hh = kc & 1;
            const int rr = row & 31;
            const int off = ((((row >> 5) * 4 + ks) * 64) + 8 * ((rr >> 3) + 4 * hh) + ((rr + 2 * ks + hh) & 7)) * 8;
            *(bf16x8*)(buf + off) = ar[it];
        }
    };
    auto load_b_half = [&](int s, bf16x8 (&br)[NT][4], int kk) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int q = 0; q < 2; ++q) br[j][2 * kk + q] = *(const bf16x8*)(bptr[j] + (size_t)(s * 4 + 2 * kk + q) * bstep);
    };
    int lane_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) lane_off[ks] = (8 * ((r >> 3) + 4 * h) + ((r + 2 * ks + h) & 7)) * 8;
    // One K stage, software-pipelined so that nothing but MFMAs sits on the critical path:
    //  * LDS holds THREE stage buffers.  Stage t reads buffer `rd`; in its first half it also writes the
    //    activations of stage t+1 into `wr`, and the single barrier of the stage sits in the MIDDLE, between
    //    the two k halves, with MFMAs queued on both sides.  A wave that runs ahead into stage t+1 writes the
    //    third buffer, which everybody finished reading before that barrier, so one barrier per stage is
    //    enough, and the first fragments of stage t+1 are read before stage t ends (carried in `afn`).
    //  * global loads run two stages ahead: the activations of stage t+2 go to the register set that was
    //    stored to LDS during stage t-1, and each half of the weight registers is re-loaded with stage t+2 as
    //    soon as the MFMAs of stage t have consumed it, so no third register set is needed.
    //  * the scheduler is given the instruction order explicitly: fragment reads run PRE ahead of the MFMAs
    //    that use them and loads / LDS writes are spread one per MFMA group.
    constexpr int PRE = MT >= 3 ? 3 : MT;
    constexpr int HR = 2 * MT;                                          // fragment reads per k half
    static_assert(HR >= 2 * NT && AIT <= HR, "not enough MFMA groups to spread the loads over");
    bf16x8 afn[PRE];                                                    // first fragments of the coming stage
    auto frag = [&](const bf16_t* base, int f) __attribute__((always_inline)) {     // f = ks * MT + i
        const int ks = f / MT, i = f - ks * MT;
        return *(const bf16x8*)(base + (i * 4 + ks) * 512 + lane_off[ks]);
    };
    auto stage = [&](const bf16_t* rd, bf16_t* wr, int s_next, bf16x8 (&br)[NT][4], bf16x8 (&ar_next)[AIT], bf16x8 (&ar_store)[AIT]) __attribute__((always_inline)) {
        // ---- first k half ----
        load_a(s_next, ar_next);
        bf16x8 af[4 * MT];
#pragma unroll
        for (int f = 0; f < PRE; ++f) af[f] = afn[f];
#pragma unroll
        for (int f = PRE; f < HR + PRE; ++f) af[f] = frag(rd, f);      // includes the first PRE fragments of the second half
#pragma unroll
        for (int f = 0; f < HR; ++f)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[f % MT][j] = mfma32(br[j][f / MT], af[f], acc[f % MT][j]);
        store_a(wr, ar_store);
#pragma unroll
        for (int t = 0; t < HR; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (t < AIT) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                        // activation loads of stage t+2
            if (t >= HR - AIT) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                  // LDS writes of stage t+1
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        // ---- second k half ----
        load_b_half(s_next, br, 0);
#pragma unroll
        for (int f = HR + PRE; f < 2 * HR; ++f) af[f] = frag(rd, f);
#pragma unroll
        for (int f = 0; f < PRE; ++f) afn[f] = frag(wr, f);            // written before the barrier above
#pragma unroll
        for (int f = HR; f < 2 * HR; ++f)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[f % MT][j] = mfma32(br[j][f / MT], af[f], acc[f % MT][j]);
        load_b_half(s_next, br, 1);
#pragma unroll
        for (int t = 0; t < HR; ++t) {
            __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (t < 2 * NT) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                     // weight loads, k half 0 of stage t+2
        }
        __builtin_amdgcn_sched_group_barrier(0x020, 2 * NT, 0);                                    // weight loads, k half 1
        __builtin_amdgcn_sched_barrier(0);
    };

    // K loop, two stages per trip so the register sets alternate without a runtime index and the body has a
    // single exit; for the tiles of at most 128 rows an odd stage count ends in one peeled stage (the larger ones
    // need an even count).  The LDS buffers rotate through three
    // pointers.  Past the end the prefetch re-reads the last stage instead of branching.
    const int n_st = s_end - s_begin;
    if (n_st > 0) {
        const int last = s_end - 1;
        bf16_t* b0 = lds; bf16_t* b1 = lds + STAGE_ELEMS; bf16_t* b2 = lds + 2 * STAGE_ELEMS;
        load_a(s_begin, areg0);
        load_b_half(s_begin, breg0, 0); load_b_half(s_begin, breg0, 1);
        load_a(min(s_begin + 1, last), areg1);
        load_b_half(min(s_begin + 1, last), breg1, 0); load_b_half(min(s_begin + 1, last), breg1, 1);
        store_a(b0, areg0);
        __syncthreads();
#pragma unroll
        for (int f = 0; f < PRE; ++f) afn[f] = frag(b0, f);
        int s = s_begin;
        for (; s + 1 < s_end; s += 2) {
            stage(b0, b1, min(s + 2, last), breg0, areg0, areg1);
            stage(b1, b2, min(s + 3, last), breg1, areg1, areg0);
            bf16_t* t0 = b0; b0 = b2; b2 = b1; b1 = t0;     // (b0, b1, b2) <- (b2, b0, b1)
        }
        if constexpr (MT <= 4) {                            // (the large tiles have no registers to spare for a third copy of the stage)
            if (s < s_end) stage(b0, b1, last, breg0, areg0, areg1);
        }
    }
    __syncthreads();                                        // the epilogue reuses the stage buffers

    // ---- epilogue: lane (h, r) holds rows m = m0 + 32 i + r, columns n = 32 tile + 8 grp + 4 h + e ----
    // Row-major outputs go through LDS one 32-row tile at a time so that the global stores are whole
    // 16-byte chunks of contiguous row segments (256 B - 1 KB per row) instead of 8-byte pieces of 32 rows.
    constexpr bool ROWMAJOR = (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU || EPI == EPI_PATCH || EPI == EPI_GEGLU || EPI == EPI_SWIGLU || EPI == EPI_PARTIAL);
    if constexpr (ROWMAJOR) {
        constexpr int ESZ = (EPI == EPI_PARTIAL) ? 4 : 2;
        constexpr int OUTW = WN * HALF * 32;                       // output columns of the workgroup
        constexpr int ROWB = OUTW * ESZ + 16;                      // padded LDS row pitch in bytes
        constexpr int CPR = OUTW * ESZ / 16;                       // 16-byte chunks per row
        constexpr int RPP = NTH / CPR;                             // rows per copy pass
        static_assert(NTH % CPR == 0 && 32 % RPP == 0, "copy-out mapping");
        unsigned char* obuf = smem_raw;
        const int nbase = n_blk * OUTW;
        const int ncols = p.N16 * 16;
        // As many 32-row tiles as fit into the stage buffers are converted and staged back to back, then copied out
        // back to back: one barrier pair per group instead of one per tile, and the stores of a group stream.
        constexpr int TILE_B = 32 * ROWB;
        constexpr int GROUP = (3 * BM * 128) / TILE_B >= MT ? MT : ((3 * BM * 128) / TILE_B < 1 ? 1 : (3 * BM * 128) / TILE_B);
#pragma unroll
        for (int g0 = 0; g0 < MT; g0 += GROUP) {
#pragma unroll
          for (int i = g0; i < (g0 + GROUP < MT ? g0 + GROUP : MT); ++i) {
            if (m0 + i * 32 >= p.M) continue;                                     // a row tile past the end (uniform)
            const int m = m0 + i * 32 + r;
            unsigned char* const tbuf = obuf + (i - g0) * TILE_B;
#pragma unroll
            for (int j = 0; j < HALF; ++j) {
#pragma unroll
                for (int grp = 0; grp < 4; ++grp) {
                    const int cl = (wn * HALF + j) * 32 + 8 * grp + 4 * h;        // column inside the workgroup tile
                    const int n0 = min(nbase + cl, ncols - 4);                    // clamped: out-of-range columns are never copied out
                    f32x4 v = {acc[i][j][4 * grp], acc[i][j][4 * grp + 1], acc[i][j][4 * grp + 2], acc[i][j][4 * grp + 3]};
                    unsigned char* dst = tbuf + r * ROWB + cl * ESZ;
                    if constexpr (EPI == EPI_PARTIAL) {
                        *(f32x4*)dst = v;
                    } else if constexpr (EPI == EPI_GEGLU) {
                        const f32x4 u = {acc[i][j + HALF][4 * grp], acc[i][j + HALF][4 * grp + 1], acc[i][j + HALF][4 * grp + 2], acc[i][j + HALF][4 * grp + 3]};
                        *(bf16x4*)dst = pack4(gelu_tanh(v[0]) * u[0], gelu_tanh(v[1]) * u[1], gelu_tanh(v[2]) * u[2], gelu_tanh(v[3]) * u[3]);
                    } else if constexpr (EPI == EPI_SWIGLU) {
                        const float f = p.rowscale[min(m, p.M - 1)];
                        f32x4 u = {acc[i][j + HALF][4 * grp], acc[i][j + HALF][4 * grp + 1], acc[i][j + HALF][4 * grp + 2], acc[i][j + HALF][4 * grp + 3]};
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
          for (int i = g0; i < (g0 + GROUP < MT ? g0 + GROUP : MT); ++i) {
            const unsigned char* const tbuf = obuf + (i - g0) * TILE_B;
#pragma unroll
            for (int ps = 0; ps < 32 / RPP; ++ps) {
                const int row = ps * RPP + tid / CPR, ch = tid % CPR;
                const int mm = m0 + i * 32 + row;
                const int n = nbase + ch * (16 / ESZ);
                if (mm < p.M && n < ncols) {
                    const uint4 val = *(const uint4*)(tbuf + row * ROWB + ch * 16);
                    // (streaming hint: the output is read once by the next launch and should not displace the operand tiles in L2)
                    if constexpr (EPI == EPI_PARTIAL) __builtin_nontemporal_store(*(const f32x4*)&val, (f32x4*)(p.partial + (size_t)split * p.pstride + (size_t)mm * p.ldp + n));
                    else __builtin_nontemporal_store(*(const f32x4*)&val, (f32x4*)(p.out + (size_t)mm * p.ldo + n));
                }
            }
          }
          if (g0 + GROUP < MT) __syncthreads();
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = m0 + i * 32 + r;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < HALF; ++j) {
          uint2 qk[4];                                                  // (EPI_VIT_QKV_ROPE: the rotated values of the four groups)
#pragma unroll
          for (int grp = 0; grp < 4; ++grp) {
            const int n0 = tile_of[j] * 32 + 8 * grp + 4 * h;
            if (n0 >= p.N16 * 16) continue;
            f32x4 v = {acc[i][j][4 * grp], acc[i][j][4 * grp + 1], acc[i][j][4 * grp + 2], acc[i][j][4 * grp + 3]};
            if constexpr (EPI == EPI_PARTIAL) {
                *(f32x4*)(p.partial + (size_t)split * p.pstride + (size_t)m * p.ldp + n0) = v;
            } else if constexpr (EPI == EPI_GEGLU) {
                const f32x4 u = {acc[i][j + HALF][4 * grp], acc[i][j + HALF][4 * grp + 1], acc[i][j + HALF][4 * grp + 2], acc[i][j + HALF][4 * grp + 3]};
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
            } else if constexpr (EPI == EPI_VIT_QKV_ROPE) {
                // DM0 ViT (dm0_infer.py:589-598): + fp32 bias, rounded to bf16 as the reference's QKV buffer is, then the 2-D rotary
                // embedding on Q and K; per (image, head) Q and K as fragment-tiled [seq_pad][64], V^T as [64][seq_pad].  The rows
                // are laid out as seq_pad (a multiple of 32) per image, so a 32-row tile is one 32-key block of one image.
                v += *(const f32x4*)(p.bias_f32 + n0);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = round_bf16(v[e]);
                const int which = n0 >> 10, cc = n0 & 1023, head = cc >> 6, d = cc & 63;
                const int img = m / p.seq_pad, tok = m - img * p.seq_pad;
                const size_t vh = (size_t)(img * 16 + head);
                if (which < 2) {
                    const bf16x4 cs = load4(p.rope + (size_t)min(tok, p.seq - 1) * 64 + d);
                    const float c0 = bf2f(cs[0]), s0 = bf2f(cs[1]), c1 = bf2f(cs[2]), s1 = bf2f(cs[3]);
                    const f32x4 w = v;
                    v[0] = w[0] * c0 - w[1] * s0; v[1] = w[1] * c0 + w[0] * s0;
                    v[2] = w[2] * c1 - w[3] * s1; v[3] = w[3] * c1 + w[2] * s1;
                    // lanes h = 0 / 1 of a row hold the two halves of every 8-wide chunk: swap halves so that each lane owns two
                    // whole 16-byte pieces of the fragment-tiled Q / K
                    const bf16x4 pk = pack4(v);
                    qk[grp] = *(const uint2*)&pk;
                    if (grp == 3) {
                        bf16_t* const dst = (which == 0 ? p.q : p.k) + vh * ((size_t)p.seq_pad * 64);
                        const int d0 = (tile_of[j] * 32) & 63;
#pragma unroll
                        for (int pr = 0; pr < 2; ++pr) {
                            const uint2 keep = h ? qk[2 * pr + 1] : qk[2 * pr], send = h ? qk[2 * pr] : qk[2 * pr + 1];
                            const uint2 recv = {(unsigned)__shfl_xor((int)send.x, 32, 64), (unsigned)__shfl_xor((int)send.y, 32, 64)};
                            *(uint4*)(dst + ft_index(tok, d0 + 8 * (2 * pr + h), 2)) = h ? uint4{recv.x, recv.y, keep.x, keep.y} : uint4{keep.x, keep.y, recv.x, recv.y};
                        }
                    }
                } else {
                    // V^T: the wave's 32 keys x 32 d tile is transposed through a private 2.3 KB of LDS ([d][key], 72-byte pitch)
                    // so that it leaves as whole 16-byte pieces of the permuted-key fragments instead of 2-byte stores
                    volatile bf16_t* tb = (volatile bf16_t*)(smem_raw + wn * 2304);
#pragma unroll
                    for (int e = 0; e < 4; ++e) tb[(8 * grp + 4 * h + e) * 36 + r] = f2bf(v[e]);
                    if (grp == 3) {
                        const int tok0 = tok - r;                                   // first key of the tile: a multiple of 32
                        const int d0 = (tile_of[j] * 32) & 63;                      // head-local d of the tile's first column
                        const int gq = lane >> 4, rq = lane & 15;
#pragma unroll
                        for (int dt = 0; dt < 2; ++dt) {
                            const volatile uint2* src = (const volatile uint2*)(smem_raw + wn * 2304 + (16 * dt + rq) * 72 + gq * 8);
                            const uint2 lo = {src[0].x, src[0].y}, hi = {src[4].x, src[4].y};       // keys 4 gq .. +3 and 16 + 4 gq .. +3
                            const size_t frag = (size_t)(((d0 >> 4) + dt) * (p.seq_pad >> 5) + (tok0 >> 5)) * 64 + lane;
                            *(uint4*)(p.vt + vh * ((size_t)64 * p.seq_pad) + frag * 8) = uint4{lo.x, lo.y, hi.x, hi.y};
                        }
                    }
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
}

// Workgroup -> block tile.  Row blocks come in two sizes when MIXED: the first n_big blocks have MT 32-row tiles, the
// others MT - 1, so that M rows are covered with ceil(M / 32) tiles instead of a multiple of MT (788 rows: 7 + 6 + 6 + 6 =
// 25 tiles where four 7-tile blocks would compute 28).
template <int WN, int MT, int NT, int EPI, bool MIXED>
__global__ __launch_bounds__(WN * 64, (MT <= 2 && WN == 4 ? 2 : 1))
void gemm_mfma_kernel(GemmP p, int m_blocks, int n_blocks, int stages_total, int stages_per_split, int n_big) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int total = m_blocks * n_blocks * p.nsplit;
    const int lid = xcd_remap(blockIdx.x, total);
    const int split = lid / (m_blocks * n_blocks);
    const int rem = lid - split * (m_blocks * n_blocks);
    const int n_blk = rem / m_blocks;
    const int m_blk = rem - n_blk * m_blocks;
    if constexpr (MIXED) {
        if (m_blk < n_big) gemm_block<WN, MT, NT, EPI>(p, smem_raw, m_blk * (MT * 32), n_blk, split, stages_total, stages_per_split);
        else gemm_block<WN, MT - 1, NT, EPI>(p, smem_raw, n_big * (MT * 32) + (m_blk - n_big) * ((MT - 1) * 32), n_blk, split, stages_total, stages_per_split);
    } else {
        gemm_block<WN, MT, NT, EPI>(p, smem_raw, m_blk * (MT * 32), n_blk, split, stages_total, stages_per_split);
    }
}

template <int WN, int MT, int NT, int EPI, bool MIXED>
int launch_cfg(const GemmP& p, hipStream_t s) {
    constexpr int BM = MT * 32;
    constexpr int HALF = EpiTraits<EPI>::dual ? NT / 2 : NT;
    const int tiles = (p.M + 31) / 32;
    int m_blocks = (tiles + MT - 1) / MT, n_big = m_blocks;
    if (MIXED) {
        n_big = tiles - m_blocks * (MT - 1);               // blocks that need the MT-th tile
        if (n_big < 0) n_big = 0;
    }
    const int n_blocks = ((p.N16 + 1) / 2 + WN * HALF - 1) / (WN * HALF);
    const int stages_total = p.K32p / 2;
    const int nsplit = p.nsplit < 1 ? 1 : p.nsplit;
    const int sps = (stages_total + nsplit - 1) / nsplit;
    if ((nsplit - 1) * sps >= stages_total) return 3;      // an empty split would leave its partial unwritten
    if (MT > 4 && ((sps & 1) || (stages_total & 1))) return 3;              // the large tiles consume K stages in pairs
    GemmP q = p; q.nsplit = nsplit;
    // three K-stage buffers; the row-major epilogues stage 32-row output tiles in the same memory
    const size_t epi_bytes = (size_t)32 * (WN * HALF * 32 * (EPI == EPI_PARTIAL ? 4 : 2) + 16);
    const size_t smem = std::max((size_t)3 * BM * 64 * sizeof(bf16_t), epi_bytes);
    auto kern = gemm_mfma_kernel<WN, MT, NT, EPI, MIXED>;
    if (smem > 65536) {
        static std::atomic<uint64_t> done{0};
        if (int rc = ensure_dynamic_lds((const void*)kern, smem, done)) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(m_blocks * n_blocks * nsplit), dim3(WN * 64), smem, s, q, m_blocks, n_blocks, stages_total, sps, n_big);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

template <int EPI>
int launch_epi(const GemmP& p, int tile, hipStream_t s) {
    switch (tile) {
        case TILE_224x256: return launch_cfg<4, 7, 2, EPI, true>(p, s);
        case TILE_192x256: return launch_cfg<4, 6, 2, EPI, true>(p, s);
        case TILE_160x256: return launch_cfg<4, 5, 2, EPI, true>(p, s);
        case TILE_128x256: return launch_cfg<4, 4, 2, EPI, true>(p, s);
        case TILE_64x256:  return launch_cfg<4, 2, 2, EPI, false>(p, s);
        case TILE_64x128:  if constexpr (!EpiTraits<EPI>::dual) return launch_cfg<4, 2, 1, EPI, false>(p, s); else return 2;
        case TILE_128x128: if constexpr (!EpiTraits<EPI>::dual) return launch_cfg<4, 4, 1, EPI, false>(p, s); else return 2;
        case TILE_96x128:  if constexpr (!EpiTraits<EPI>::dual) return launch_cfg<4, 3, 1, EPI, false>(p, s); else return 2;
    }
    return 2;
}

}  // namespace

int gemm_tile_bm(int tile) { static const int v[TILE_COUNT] = {224, 192, 160, 128, 64, 64, 128, 256, 224, 192, 128, 96}; return v[tile]; }
int gemm_tile_bn(int tile) { return (tile == TILE_64x128 || tile == TILE_128x128 || tile == TILE_96x128) ? 128 : 256; }

int launch_gemm(const GemmP& p, int epi, int tile, hipStream_t s) {
    if (p.M <= 0 || p.N16 <= 0 || p.K32p <= 0 || (p.K32p & 1) || p.a_rows <= 0 || p.bgroup < 1) return 1;
    if (epi != EPI_PARTIAL && p.nsplit > 1) return 1;
    if (gemm_tile_eight_waves(tile)) return launch_gemm8(p, epi, tile, s);
    switch (epi) {
        case EPI_BIAS:      return launch_epi<EPI_BIAS>(p, tile, s);
        case EPI_BIAS_GELU: return launch_epi<EPI_BIAS_GELU>(p, tile, s);
        case EPI_PATCH:     return launch_epi<EPI_PATCH>(p, tile, s);
        case EPI_GEGLU:     return launch_epi<EPI_GEGLU>(p, tile, s);
        case EPI_PARTIAL:   return launch_epi<EPI_PARTIAL>(p, tile, s);
        case EPI_QKV_ROPE:  return launch_epi<EPI_QKV_ROPE>(p, tile, s);
        case EPI_VIS_QKV:   return launch_epi<EPI_VIS_QKV>(p, tile, s);
        case EPI_SWIGLU:    return launch_epi<EPI_SWIGLU>(p, tile, s);
        case EPI_VIT_QKV_ROPE: return launch_epi<EPI_VIT_QKV_ROPE>(p, tile, s);
    }
    return 2;
}
