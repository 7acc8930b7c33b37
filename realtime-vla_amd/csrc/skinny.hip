// Weight-streaming GEMM for the action expert (M <= 128 rows, in row blocks of 64 or 16), replacing the decoder-side Triton
// kernels of /root/reference/pi0_infer.py:82-124, :693-725, :939-1039, :1122-1163 and
// /root/reference/pi05_infer.py:22-64, :78-113, :127-195.
//
// One workgroup owns one 16-column tile of the output, MTS 16-row tiles and all of K; its 8 waves split K.
// (A workgroup has to pull its rows of the activations through its own CU's L2 port, which moves only
// ~100 GB/s: the few-column projections (O, down: 64 column tiles) therefore run one row tile per
// workgroup so that 256 CUs share that traffic, the wide ones keep all rows and read the weights once.)  Each wave
// issues all of its weight-fragment loads up front (coalesced 1 KB reads of the pre-tiled layout,
// straight into registers), reads its slice of the activations in MFMA operand order from L2,
// multiplies, and the waves reduce through LDS.  Because the workgroup sees every activation row
// over all of K, the RMS / adaRMS normalisation that precedes the GEMM in the reference is computed
// here from the same registers (wavefront reduction, no separate launch), and the epilogue applies
// RoPE + KV-cache append, GeGLU, residual (+gate) or the Euler update in place.
#include "kernels.h"

namespace {

constexpr int SK_WAVES = 8;
constexpr int SK_CH = 4;       // k32 blocks per A-prefetch chunk

template <int NCH, int NORM, int EPI, int SK_MTS>
__global__ __launch_bounds__(SK_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void skinny_kernel(SkinnyP p) {
    constexpr int KBW = NCH * SK_CH;
    constexpr bool DUAL = (EPI == SK_GEGLU || EPI == SK_SWIGLU);
    constexpr int NB = DUAL ? 2 : 1;
    static_assert(NORM == SN_NONE || NCH == 1, "the fused norm needs the whole K slice in registers");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    f32x4* red = (f32x4*)smem_raw;                                        // [WAVES][NB*MTS][64]
    float* ssq = (float*)(smem_raw + (size_t)SK_WAVES * NB * SK_MTS * 64 * 16);   // [WAVES][64]

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int tile = blockIdx.x;
    const int m_base = blockIdx.y * (SK_MTS * 16);
    const int kb0 = w * KBW;

    // ---- weight fragments: the HBM stream, all in flight at once ----
    bf16x8 b[NB][KBW];
    {
        const bf16_t* bp0 = p.B0 + ((size_t)tile * p.K32p + kb0) * 512 + lane * 8;
#pragma unroll
        for (int i = 0; i < KBW; ++i) b[0][i] = *(const bf16x8*)(bp0 + (size_t)i * 512);
        if constexpr (DUAL) {
            const bf16_t* bp1 = p.B1 + ((size_t)tile * p.K32p + kb0) * 512 + lane * 8;
#pragma unroll
            for (int i = 0; i < KBW; ++i) b[1][i] = *(const bf16x8*)(bp1 + (size_t)i * 512);
        }
    }
    // activation fragments: with the fragment-tiled layout (and no row offset) each is one
    // contiguous 1 KB read; astep is the distance between consecutive k32 blocks of a row
    const bf16_t* arow[SK_MTS];
    const int astep = p.a_tiled ? 512 : 32;
#pragma unroll
    for (int mt = 0; mt < SK_MTS; ++mt) {
        const int row = min(m_base + mt * 16 + r, p.M - 1) + p.a_row0;
        arow[mt] = p.a_tiled ? p.A + ft_index(row, kb0 * 32 + 8 * g, p.lda >> 5) : p.A + (size_t)row * p.lda + kb0 * 32 + 8 * g;
    }
    f32x4 acc[NB][SK_MTS];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mt = 0; mt < SK_MTS; ++mt) acc[nb][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    bf16x8 a[2][SK_MTS][SK_CH];
    auto load_a = [&](int c, bf16x8 (&dst)[SK_MTS][SK_CH]) {
#pragma unroll
        for (int mt = 0; mt < SK_MTS; ++mt)
#pragma unroll
            for (int i = 0; i < SK_CH; ++i) dst[mt][i] = *(const bf16x8*)(arow[mt] + (c * SK_CH + i) * astep);
    };
    load_a(0, a[0]);
    // what the epilogue will need from memory (old residual, RoPE pair, bias, gate) is requested now as well, by the
    // waves that will finish a row tile, so that no memory round trip is left after the reduction
    bf16x4 pre_old = {}, pre_cs = {}, pre_bias = {}, pre_gate = {};
    f32x4 pre_cb0 = {0.f, 0.f, 0.f, 0.f}, pre_cb1 = {0.f, 0.f, 0.f, 0.f};
    if (w < SK_MTS) {
        const int me = min(m_base + w * 16 + r, p.M - 1);
        const int ne = tile * 16 + 4 * g;
        if constexpr (EPI == SK_RES) {
            pre_old = load4(p.out_tiled ? p.out + ft_index(me + p.out_row0, ne, p.ldo >> 5) : p.out + (size_t)me * p.ldo + ne);
            if (p.gate) pre_gate = load4(p.gate + ne);
            if (p.bias) pre_bias = load4(p.bias + ne);
        } else if constexpr (EPI == SK_BIAS || EPI == SK_BIAS_SILU) {
            pre_bias = load4(p.bias + ne);
        } else if constexpr (EPI == SK_QKV_ROPE) {
            if (ne < 2304) pre_cs = load4(p.rope + (size_t)me * 256 + (ne & 255));
        }
        if constexpr (NORM == SN_RMS && (EPI == SK_QKV_ROPE || EPI == SK_GEGLU)) {
            if (p.col_bias0) pre_cb0 = *(const f32x4*)(p.col_bias0 + ne);
            if (p.col_bias1) pre_cb1 = *(const f32x4*)(p.col_bias1 + ne);
        }
    }
    // keep every load above in flight before anything waits on one of them
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        if (c + 1 < NCH) { load_a(c + 1, a[(c + 1) & 1]); __builtin_amdgcn_sched_barrier(0); }
        if constexpr (NORM != SN_NONE) {
            // row sums of squares over this wave's K slice
            float ss[SK_MTS];
#pragma unroll
            for (int mt = 0; mt < SK_MTS; ++mt) {
                float s = 0.f;
#pragma unroll
                for (int i = 0; i < SK_CH; ++i)
#pragma unroll
                    for (int j = 0; j < 8; j += 2) {                       // v_dot2_f32_bf16: two squares per instruction, no conversions
                        const bf16x2 x2 = {a[0][mt][i][j], a[0][mt][i][j + 1]};
                        s = __builtin_amdgcn_fdot2_f32_bf16(x2, x2, s, false);
                    }
                s = rows_sum(s);
                ss[mt] = s;
            }
            if (g == 0) {
#pragma unroll
                for (int mt = 0; mt < SK_MTS; ++mt) ssq[w * 64 + mt * 16 + r] = ss[mt];
            }
        }
        if constexpr (NORM == SN_ADARMS) {
            // adaptive RMS: x^ (1 + scale) + shift is not a row scaling, so the rows are normalised before the product
            __syncthreads();
            float f[SK_MTS];
#pragma unroll
            for (int mt = 0; mt < SK_MTS; ++mt) {
                float t = 0.f;
#pragma unroll
                for (int ww = 0; ww < SK_WAVES; ++ww) t += ssq[ww * 64 + mt * 16 + r];
                f[mt] = rsqrtf(t / (float)p.K + p.eps);
            }
#pragma unroll
            for (int i = 0; i < SK_CH; ++i) {
                const bf16x8 sc = *(const bf16x8*)(p.style + (kb0 + i) * 32 + 8 * g);
                const bf16x8 sh = *(const bf16x8*)(p.style + p.K + (kb0 + i) * 32 + 8 * g);
#pragma unroll
                for (int mt = 0; mt < SK_MTS; ++mt)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        a[0][mt][i][j] = f2bf(bf2f(a[0][mt][i][j]) * f[mt] * (1.0f + bf2f(sc[j])) + bf2f(sh[j]));
            }
        }
        // plain RMS (no learned scale left: it is folded into the weights) is a per-row factor and is applied to
        // the accumulator after the product, as the reference does for QKV (pi0_infer.py:1005-1015): the MFMAs
        // start as soon as the operands arrive and the statistics ride along with the K-split reduction
#pragma unroll
        for (int i = 0; i < SK_CH; ++i)
#pragma unroll
            for (int mt = 0; mt < SK_MTS; ++mt)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[nb][mt] = mfma16(b[nb][c * SK_CH + i], a[c & 1][mt][i], acc[nb][mt]);
    }

    // ---- reduce the 8 K-slices through LDS; wave mt finishes row tile mt ----
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mt = 0; mt < SK_MTS; ++mt) red[((size_t)w * NB * SK_MTS + nb * SK_MTS + mt) * 64 + lane] = acc[nb][mt];
    __syncthreads();
    if (w >= SK_MTS) return;
    const int mt = w;
    const int m = m_base + mt * 16 + r;
    f32x4 v[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ww = 0; ww < SK_WAVES; ++ww) t += red[((size_t)ww * NB * SK_MTS + nb * SK_MTS + mt) * 64 + lane];
        v[nb] = t;
    }
    if constexpr (NORM == SN_RMS) {
        float t = 0.f;
#pragma unroll
        for (int ww = 0; ww < SK_WAVES; ++ww) t += ssq[ww * 64 + mt * 16 + r];
        float f = rsqrtf(t / (float)p.K + p.eps);
        if (!p.factor_f32) f = round_bf16(f);                            // the Pi0 reference keeps the factor in bf16, DM0 in fp32
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) v[nb] *= f;
        if constexpr (EPI == SK_QKV_ROPE || EPI == SK_GEGLU) {
            v[0] += pre_cb0;
            if constexpr (NB == 2) v[1] += pre_cb1;
        }
    }
    if (m >= p.M) return;
    const int n0 = tile * 16 + 4 * g;
    bf16_t* const optr = p.out_tiled ? p.out + ft_index(m + p.out_row0, n0, p.ldo >> 5) : p.out + (size_t)m * p.ldo + n0;
    if constexpr (EPI == SK_BIAS || EPI == SK_BIAS_SILU) {
        f32x4 o = v[0];
        const bf16x4 bb = pre_bias;
#pragma unroll
        for (int e = 0; e < 4; ++e) { o[e] += bf2f(bb[e]); if (EPI == SK_BIAS_SILU) o[e] = siluf(o[e]); }
        store4(optr, pack4(o));
    } else if constexpr (EPI == SK_RES) {
        f32x4 o = v[0];
        if (p.gate) { for (int e = 0; e < 4; ++e) o[e] *= bf2f(pre_gate[e]); }
        if (p.bias) { for (int e = 0; e < 4; ++e) o[e] += bf2f(pre_bias[e]); }
        const bf16x4 old = pre_old;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] += bf2f(old[e]);
        store4(optr, pack4(o));
    } else if constexpr (EPI == SK_GEGLU) {
        store4(optr,
               pack4(gelu_tanh(v[0][0]) * v[1][0], gelu_tanh(v[0][1]) * v[1][1], gelu_tanh(v[0][2]) * v[1][2], gelu_tanh(v[0][3]) * v[1][3]));
    } else if constexpr (EPI == SK_SWIGLU) {
        store4(optr, pack4(siluf(v[0][0]) * v[1][0], siluf(v[0][1]) * v[1][1], siluf(v[0][2]) * v[1][2], siluf(v[0][3]) * v[1][3]));
    } else if constexpr (EPI == SK_QKV_ROPE) {
        f32x4 o = v[0];
        if (n0 < 2304) {
            const bf16x4 cs = pre_cs;
            const float c0 = bf2f(cs[0]), s0 = bf2f(cs[1]), c1 = bf2f(cs[2]), s1 = bf2f(cs[3]);
            const f32x4 x = o;
            o[0] = x[0] * c0 - x[1] * s0; o[1] = x[1] * c0 + x[0] * s0;
            o[2] = x[2] * c1 - x[3] * s1; o[3] = x[3] * c1 + x[2] * s1;
            if (n0 < 2048) store4(p.q + ft_index(m * 8 + (n0 >> 8), n0 & 255, 8), pack4(o));
            else store4(p.k + ft_index(p.kv_row0 + m, n0 - 2048, 8), pack4(o));
        } else {
            const int d = n0 - 2304;
#pragma unroll
            for (int e = 0; e < 4; ++e) p.vt[vt_index(d + e, p.kv_row0 + m, p.ldvt >> 5)] = f2bf(o[e]);
        }
    }
}

template <int NCH, int NORM, int EPI, int SK_MTS>
int launch_inst(const SkinnyP& p, hipStream_t s) {
    constexpr int NB = (EPI == SK_GEGLU || EPI == SK_SWIGLU) ? 2 : 1;
    const size_t smem = (size_t)SK_WAVES * NB * SK_MTS * 64 * 16 + (size_t)SK_WAVES * 64 * 4;
    auto kern = skinny_kernel<NCH, NORM, EPI, SK_MTS>;
    if (smem > 65536) {
        static std::atomic<uint64_t> done{0};
        if (int rc = ensure_dynamic_lds((const void*)kern, smem, done)) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(p.N16, (p.M + SK_MTS * 16 - 1) / (SK_MTS * 16)), dim3(SK_WAVES * 64), smem, s, p);
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

}  // namespace

int launch_skinny(const SkinnyP& p, int epi, hipStream_t s) {
    if (p.M <= 0 || p.M > 128 || p.N16 <= 0) return 1;      // (the row blocks of blockIdx.y; the callers' buffers hold at most 128 rows)
    if (p.K != 1024 && p.K != 2048 && p.K != 4096) return 1;
    if (p.K32p < p.K / 32 || p.lda < p.K || (p.lda & 31)) return 1;
    if (p.out_tiled && (p.ldo & 31)) return 1;
    const int nch = p.K / (32 * SK_WAVES * SK_CH);
    if (p.norm != SN_NONE && nch != 1) return 1;
    if (p.norm == SN_ADARMS && !p.style) return 1;
#define SK_CASE(NCH_, NORM_, EPI_, MTS_) if (nch == NCH_ && p.norm == NORM_ && epi == EPI_) return launch_inst<NCH_, NORM_, EPI_, MTS_>(p, s)
    SK_CASE(1, SN_RMS, SK_QKV_ROPE, 4);
    SK_CASE(1, SN_RMS, SK_GEGLU, 4);
    SK_CASE(1, SN_RMS, SK_SWIGLU, 4);
    SK_CASE(1, SN_NONE, SK_BIAS, 4);
    SK_CASE(1, SN_NONE, SK_BIAS_SILU, 4);
    SK_CASE(1, SN_RMS, SK_RES, 4);
    SK_CASE(1, SN_ADARMS, SK_RES, 4);
    SK_CASE(2, SN_NONE, SK_RES, 1);
    SK_CASE(4, SN_NONE, SK_RES, 1);
#undef SK_CASE
    return 2;
}
