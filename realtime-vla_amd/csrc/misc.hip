// Bandwidth-trivial kernels around the GEMMs: weight pre-tiling, split-K reduce fused with
// bias / residual / LayerNorm / RMSNorm, patch im2col, tiny-K linear layers, RoPE tables.
#include "kernels.h"

namespace {

// ---------------------------------------------------------------------------------------------
// W[K][N] -> MFMA fragment tiles [nb][kb][lane][8] (see kernels.h)
__global__ void pretile_kernel(const bf16_t* __restrict__ W, int K, int N, bf16_t* __restrict__ out, int KBp, int G, int wide, size_t chunks,
                               const bf16_t* __restrict__ rowscale) {
    const size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= chunks) return;
    const int lane = (int)(c & 63);
    const size_t tile = c >> 6;                             // order [nb / G][kb][nb % G]
    const size_t per_group = (size_t)KBp * G;              // KBp: padded K in blocks of 32 (or of 16 for wide tiles)
    const int group = (int)(tile / per_group), rem = (int)(tile % per_group);
    const int kb = rem / G, nb = group * G + rem % G;
    const int n = wide ? nb * 32 + (lane & 31) : nb * 16 + (lane & 15);
    const int k0 = wide ? kb * 16 + 8 * (lane >> 5) : kb * 32 + 8 * (lane >> 4);
    bf16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int k = k0 + j;
        v[j] = (n < N && k < K) ? W[(size_t)k * N + n] : (bf16_t)0.0f;
        if (rowscale && k < K) v[j] = f2bf(bf2f(v[j]) * (1.0f + bf2f(rowscale[k])));
    }
    *(bf16x8*)(out + c * 8) = v;
}

// ---------------------------------------------------------------------------------------------
// One workgroup per row: x = bf16(res + bias + sum_s partial[s]); optional normalised copy.
// Replaces merge_split_k_bias_res + layer_norm_small_kernel / rms_norm_kernel
// (/root/reference/pi0_infer.py:325-346, :366-382, :648-663).
template <int NORM, int NSPLIT>
__global__ __launch_bounds__(256)
void reduce_kernel(ReduceP p) {
    __shared__ float red[8];
    const int m = blockIdx.x;
    const int tid = threadIdx.x;
    const int nq = p.N >> 2;                   // float4 groups per row (N <= 2048 -> at most 2 per thread)
    f32x4 v[2];
    float s = 0.f;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int c = tid + it * 256;
        v[it] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (c < nq) {
            const int n0 = c * 4;
            // the split count is a template argument so that every partial is requested before the first add
            f32x4 part[NSPLIT > 0 ? NSPLIT : 1];
#pragma unroll
            for (int sp = 0; sp < NSPLIT; ++sp) part[sp] = *(const f32x4*)(p.partial + (size_t)sp * p.pstride + (size_t)m * p.ldp + n0);
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int sp = 0; sp < NSPLIT; ++sp) a += part[sp];
            if (p.bias) { const bf16x4 b = load4(p.bias + n0); for (int e = 0; e < 4; ++e) a[e] += bf2f(b[e]); }
            if (p.res) { const bf16x4 rr = load4(p.res + (size_t)m * p.ldr + n0); for (int e = 0; e < 4; ++e) a[e] += bf2f(rr[e]); }
            const bf16x4 xb = pack4(a);
            if (p.x) store4(p.x + (size_t)m * p.ldx + n0, xb);
            for (int e = 0; e < 4; ++e) a[e] = bf2f(xb[e]);       // the norm reads the bf16 stream
            v[it] = a;
            if (NORM == NORM_RMS) s += a[0] * a[0] + a[1] * a[1] + a[2] * a[2] + a[3] * a[3];
            else s += a[0] + a[1] + a[2] + a[3];
        }
    }
    if (NORM == NORM_NONE) return;
    auto block_sum = [&](float x) {
        x = wave_sum(x);
        __syncthreads();
        if ((tid & 63) == 0) red[tid >> 6] = x;
        __syncthreads();
        return red[0] + red[1] + red[2] + red[3];
    };
    const float tot = block_sum(s);
    const float inv_n = 1.0f / (float)p.N;
    if (NORM == NORM_RMS) {
        const float f = rsqrtf(tot * inv_n + p.eps);
        if (p.factor && tid == 0) p.factor[m] = f;
        if (p.xn) {
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const int c = tid + it * 256;
                if (c < nq) store4(p.xn + (size_t)m * p.ldxn + c * 4, pack4(v[it] * f));
            }
        }
    } else {
        const float mean = tot * inv_n;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int c = tid + it * 256;
            if (c < nq) for (int e = 0; e < 4; ++e) { const float d = v[it][e] - mean; q += d * d; }
        }
        const float var = block_sum(q) * inv_n;
        const float inv_std = 1.0f / sqrtf(var + p.eps);
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int c = tid + it * 256;
            if (c < nq) {
                const int n0 = c * 4;
                const bf16x4 w = load4(p.nw + n0), b = load4(p.nb + n0);
                f32x4 o;
                for (int e = 0; e < 4; ++e) o[e] = (v[it][e] - mean) * inv_std * bf2f(w[e]) + bf2f(b[e]);
                store4(p.xn + (size_t)m * p.ldxn + n0, pack4(o));
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// NHWC images [v][224][224][3] -> patch rows [v*256][ldp], feature order (dy, dx, c), zero padded
// to ldp (/root/reference/pi0_infer.py:348-350).
__global__ void im2col_kernel(const bf16_t* __restrict__ img, bf16_t* __restrict__ out, int ldp, int rows) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int per_row = ldp;
    if (idx >= rows * per_row) return;
    const int row = idx / per_row, k = idx - row * per_row;
    bf16_t val = (bf16_t)0.0f;
    if (k < 588) {
        const int view = row >> 8, py = (row >> 4) & 15, px = row & 15;
        const int dy = k / 42, rem = k - dy * 42;       // rem = dx * 3 + c, contiguous in memory
        val = img[(((size_t)view * 224 + py * 14 + dy) * 224 + px * 14) * 3 + rem];
    }
    out[idx] = val;
}

// tiny-K linear: one thread per output element, W[K][N] row-major (coalesced over n)
RTVLA_DEVICE void small_linear_one(const SmallLinearJob& j, int idx) {
    const int m = idx / j.N, n = idx - m * j.N;
    float acc = j.bias ? bf2f(j.bias[n]) : 0.f;
    if (j.K == 32) {
        // every operand is requested before the first use: a dependent load per k would cost 32 memory round trips
        bf16x8 xr[4];
        bf16_t wc[32];
#pragma unroll
        for (int q = 0; q < 4; ++q) xr[q] = *(const bf16x8*)(j.x + (size_t)m * j.ldx + q * 8);
#pragma unroll
        for (int k = 0; k < 32; ++k) wc[k] = j.W[(size_t)k * j.N + n];
#pragma unroll
        for (int k = 0; k < 32; ++k) acc += bf2f(xr[k >> 3][k & 7]) * bf2f(wc[k]);
    } else {
        for (int k = 0; k < j.K; ++k) acc += bf2f(j.x[(size_t)m * j.ldx + k]) * bf2f(j.W[(size_t)k * j.N + n]);
    }
    if (j.act_silu) acc = siluf(acc);
    if (j.out_tiled) j.out[ft_index(m + j.out_row0, n, j.ldo >> 5)] = f2bf(acc);
    else j.out[(size_t)m * j.ldo + n] = f2bf(acc);
}
// one launch for up to two independent tiny linears (the state-token and the action input projections of a flow step)
__global__ void small_linear_kernel(SmallLinearJob a, SmallLinearJob b) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int na = a.M * a.N;
    if (idx < na) small_linear_one(a, idx);
    else if (idx - na < b.M * b.N) small_linear_one(b, idx - na);
}

__global__ void copy_rows_kernel(const bf16_t* __restrict__ src, int lds, bf16_t* __restrict__ dst, int ldd, int rows, int cols8) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * cols8) return;
    const int r = idx / cols8, c = idx - r * cols8;
    *(uint4*)(dst + (size_t)r * ldd + c * 8) = *(const uint4*)(src + (size_t)r * lds + c * 8);
}

// Pi05 prompt staging on the device (replaces the host-side embedding lookup, scaling and RoPE slicing of
// /root/reference/pi05_infer.py:769-785, :811-822): row i < prompt_rows of the prompt gets
// bf16(embedding[ids[i]] * scale) when S_v + i < *valid_len (rows past the prompt keep their contents, they are
// masked), and the decoder's RoPE rows are rope_full[*valid_len - 1 + r].  One workgroup per row.
__global__ void prompt_stage_kernel(const bf16_t* __restrict__ emb, int vocab, const int* __restrict__ ids, const int* __restrict__ valid_len,
                                    bf16_t* __restrict__ x_rows, int prompt_rows, int s_v, float scale,
                                    const bf16_t* __restrict__ rope_full, int rope_rows, bf16_t* __restrict__ dec_rope, int dec_rows) {
    const int b = blockIdx.x, tid = threadIdx.x;                    // 256 threads x 8 elements = one 2048-wide row
    const int vl = *valid_len;
    if (b < prompt_rows) {
        if (s_v + b >= vl) return;
        const int id = min(max(ids[b], 0), vocab - 1);
        const bf16x8 v = *(const bf16x8*)(emb + (size_t)id * 2048 + tid * 8);
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f2bf(bf2f(v[j]) * scale);
        *(bf16x8*)(x_rows + (size_t)b * 2048 + tid * 8) = o;
    } else {
        const int r = b - prompt_rows;
        if (r >= dec_rows || tid >= 32) return;
        const int src = min(max(vl - 1 + r, 0), rope_rows - 1);
        *(bf16x8*)(dec_rope + (size_t)r * 256 + tid * 8) = *(const bf16x8*)(rope_full + (size_t)src * 256 + tid * 8);
    }
}

__global__ void fill_zero_kernel(uint4* p, size_t n16) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) p[i] = uint4{0, 0, 0, 0};
}

__global__ void copy_bytes_kernel(const uint4* src, uint4* dst, size_t n16) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

__global__ void scale_kernel(bf16_t* p, size_t n, float f) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = f2bf(bf2f(p[i]) * f);
}

}  // namespace

void launch_pretile(const bf16_t* W, int K, int N, bf16_t* out, int G, int wide, hipStream_t s, const bf16_t* rowscale) {
    const int KBp = wide ? k32_padded(K) * 2 : k32_padded(K);
    const size_t chunks = (wide ? tiled_elems_wide(K, N, G) : tiled_elems(K, N, G)) / 8;
    hipLaunchKernelGGL(pretile_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, W, K, N, out, KBp, G, wide, chunks, rowscale);
}

__global__ void vec_mat_kernel(const bf16_t* __restrict__ v, const bf16_t* __restrict__ W, int K, int N, float* __restrict__ out) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    float acc = 0.f;
    for (int k = 0; k < K; ++k) acc += bf2f(v[k]) * bf2f(W[(size_t)k * N + n]);
    out[n] = acc;
}
void launch_vec_mat(const bf16_t* v, const bf16_t* W, int K, int N, float* out, hipStream_t s) {
    hipLaunchKernelGGL(vec_mat_kernel, dim3((N + 127) / 128), dim3(128), 0, s, v, W, K, N, out);
}

// W has K rows; the tiles are laid out as for K_pad rows (a multiple of 128), the rows past K zero: for a kernel that only takes
// the padded K
void launch_pretile_padded(const bf16_t* W, int K, int K_pad, int N, bf16_t* out, hipStream_t s) {
    const size_t chunks = tiled_elems(K_pad, N, 1) / 8;
    hipLaunchKernelGGL(pretile_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, W, K, N, out, k32_padded(K_pad), 1, 0, chunks, (const bf16_t*)nullptr);
}

template <int NORM>
static int launch_reduce_norm(const ReduceP& p, hipStream_t s) {
    const dim3 grid(p.M), block(256);
    switch (p.nsplit) {
        case 0: hipLaunchKernelGGL((reduce_kernel<NORM, 0>), grid, block, 0, s, p); break;
        case 1: hipLaunchKernelGGL((reduce_kernel<NORM, 1>), grid, block, 0, s, p); break;
        case 2: hipLaunchKernelGGL((reduce_kernel<NORM, 2>), grid, block, 0, s, p); break;
        case 3: hipLaunchKernelGGL((reduce_kernel<NORM, 3>), grid, block, 0, s, p); break;
        case 4: hipLaunchKernelGGL((reduce_kernel<NORM, 4>), grid, block, 0, s, p); break;
        case 6: hipLaunchKernelGGL((reduce_kernel<NORM, 6>), grid, block, 0, s, p); break;
        case 8: hipLaunchKernelGGL((reduce_kernel<NORM, 8>), grid, block, 0, s, p); break;
        default: return 2;
    }
    return hipGetLastError() == hipSuccess ? 0 : 5;
}

int launch_reduce(const ReduceP& p, hipStream_t s) {
    if (p.M <= 0 || p.N <= 0 || (p.N & 3) || p.N > 2048) return 1;
    if (p.norm == NORM_LAYER && !p.xn) return 1;
    if (p.norm == NORM_RMS && !p.xn && !p.factor) return 1;
    if (p.norm == NORM_LAYER && (!p.nw || !p.nb)) return 1;
    switch (p.norm) {
        case NORM_NONE:  return launch_reduce_norm<NORM_NONE>(p, s);
        case NORM_RMS:   return launch_reduce_norm<NORM_RMS>(p, s);
        case NORM_LAYER: return launch_reduce_norm<NORM_LAYER>(p, s);
    }
    return 2;
}

void launch_im2col(const bf16_t* images, bf16_t* patches, int ldp, int views, hipStream_t s) {
    const int rows = views * 256;
    const int total = rows * ldp;
    hipLaunchKernelGGL(im2col_kernel, dim3((total + 255) / 256), dim3(256), 0, s, images, patches, ldp, rows);
}

void launch_small_linear(const bf16_t* x, int ldx, const bf16_t* W, const bf16_t* bias, bf16_t* out, int ldo,
                         int M, int K, int N, int act_silu, int out_tiled, int out_row0, hipStream_t s) {
    SmallLinearJob j{x, ldx, W, bias, out, ldo, M, K, N, act_silu, out_tiled, out_row0};
    launch_small_linear2(j, SmallLinearJob{}, s);
}

void launch_small_linear2(const SmallLinearJob& a, const SmallLinearJob& b, hipStream_t s) {
    const int total = a.M * a.N + b.M * b.N;
    if (total <= 0) return;
    hipLaunchKernelGGL(small_linear_kernel, dim3((total + 255) / 256), dim3(256), 0, s, a, b);
}

void launch_copy_rows(const bf16_t* src, int lds, bf16_t* dst, int ldd, int rows, int cols, hipStream_t s) {
    if (rows <= 0 || cols <= 0) return;
    const int cols8 = cols / 8;
    const int total = rows * cols8;
    hipLaunchKernelGGL(copy_rows_kernel, dim3((total + 255) / 256), dim3(256), 0, s, src, lds, dst, ldd, rows, cols8);
}

void launch_prompt_stage(const bf16_t* emb, int vocab, const int* ids, const int* valid_len, bf16_t* x_rows, int prompt_rows, int s_v,
                         float scale, const bf16_t* rope_full, int rope_rows, bf16_t* dec_rope, int dec_rows, hipStream_t s) {
    hipLaunchKernelGGL(prompt_stage_kernel, dim3(prompt_rows + dec_rows), dim3(256), 0, s, emb, vocab, ids, valid_len, x_rows, prompt_rows, s_v,
                       scale, rope_full, rope_rows, dec_rope, dec_rows);
}

void launch_fill_zero(void* p, size_t bytes, hipStream_t s) {
    const size_t n16 = bytes / 16;
    if (!n16) return;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, (uint4*)p, n16);
}

void launch_copy_bytes(const void* src, void* dst, size_t bytes, hipStream_t s) {
    const size_t n16 = bytes / 16;
    if (!n16) return;
    hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, (const uint4*)src, (uint4*)dst, n16);
}

void launch_scale_inplace(bf16_t* p, size_t n, float f, hipStream_t s) {
    if (!n) return;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n, f);
}
