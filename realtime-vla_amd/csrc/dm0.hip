// DM0-specific small kernels around the shared GEMM / attention / weight-streaming kernels
// (/root/reference/dm0_infer.py): patch gather from NCHW images, class token + position embedding + ln_pre,
// NHWC im2col of the stride-2 3x3 down-sampling convolutions, token-embedding gather, and the
// scale + QK-norm + RoPE + cache-scatter step that follows every QKV GEMM.
#include "kernels.h"

namespace {

constexpr int DM0_GRID = 52;               // 728 / 14 patches per side
constexpr int DM0_SEQ = 52 * 52 + 1;       // + class token

// images NCHW [n][3][728][728] -> patch rows [n*2704][ldp], feature order (c, dy, dx), zero padded to ldp
// (dm0_infer.py:695-696)
__global__ void dm0_im2col_nchw_kernel(const bf16_t* __restrict__ img, bf16_t* __restrict__ out, int ldp, int rows) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * ldp) return;
    const int row = idx / ldp, k = idx - row * ldp;
    bf16_t val = (bf16_t)0.0f;
    if (k < 588) {
        const int n = row / (DM0_GRID * DM0_GRID), pr = row - n * (DM0_GRID * DM0_GRID);
        const int py = pr / DM0_GRID, px = pr - py * DM0_GRID;
        const int c = k / 196, rem = k - c * 196, dy = rem / 14, dx = rem - dy * 14;
        val = img[(((size_t)n * 3 + c) * 728 + py * 14 + dy) * 728 + px * 14 + dx];
    }
    out[idx] = val;
}

// One workgroup per token row of the ViT: x = bf16(patch embedding or class embedding + position embedding), then
// ln_pre in place: (x - mean) * rsqrt(E[x^2] - mean^2 + 1e-5) * w + b  (dm0_infer.py:699-712, :442-454, :561-579).
__global__ __launch_bounds__(256)
void dm0_embed_ln_kernel(const bf16_t* __restrict__ conv, const bf16_t* __restrict__ cls, const bf16_t* __restrict__ pos,
                         const bf16_t* __restrict__ w, const bf16_t* __restrict__ b, bf16_t* __restrict__ x, int x_img_rows) {
    __shared__ float red[2][4];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int n = row / DM0_SEQ, tok = row - n * DM0_SEQ;
    const bf16_t* src = tok == 0 ? cls : conv + ((size_t)n * (DM0_SEQ - 1) + tok - 1) * 1024;
    const bf16x4 a = load4(src + tid * 4), pe = load4(pos + (size_t)tok * 1024 + tid * 4);
    float v[4], s = 0.f, q = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = round_bf16(bf2f(a[e]) + bf2f(pe[e])); s += v[e]; q += v[e] * v[e]; }
    s = wave_sum(s); q = wave_sum(q);
    if ((tid & 63) == 0) { red[0][tid >> 6] = s; red[1][tid >> 6] = q; }
    __syncthreads();
    const float mean = (red[0][0] + red[0][1] + red[0][2] + red[0][3]) * (1.0f / 1024.0f);
    const float var = (red[1][0] + red[1][1] + red[1][2] + red[1][3]) * (1.0f / 1024.0f) - mean * mean;
    const float rstd = rsqrtf(var + 1e-5f);
    const bf16x4 ww = load4(w + tid * 4), bb = load4(b + tid * 4);
    store4(x + ((size_t)n * x_img_rows + tok) * 1024 + tid * 4, pack4((v[0] - mean) * rstd * bf2f(ww[0]) + bf2f(bb[0]), (v[1] - mean) * rstd * bf2f(ww[1]) + bf2f(bb[1]),
                                                   (v[2] - mean) * rstd * bf2f(ww[2]) + bf2f(bb[2]), (v[3] - mean) * rstd * bf2f(ww[3]) + bf2f(bb[3])));
}

// NHWC im2col of a 3x3 stride-2 pad-1 convolution (dm0_infer.py:532-559), 8 channels per thread.  The input image b is
// in_h x in_w pixels of C channels whose pixel (y, x) is row  b * img_rows + row0 + y * in_w + x  of `in` (row0 skips the
// class token of the ViT output).  col [b*oh*ow][9*C], column order (ky, kx, c).
__global__ void dm0_im2col3x3_kernel(const bf16_t* __restrict__ in, int img_rows, int row0, int in_h, int in_w, int C,
                                     bf16_t* __restrict__ col, int oh, int ow, size_t chunks) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= chunks) return;
    const int c8 = C >> 3;
    const int cc = (int)(idx % c8);
    size_t rem = idx / c8;
    const int tap = (int)(rem % 9); rem /= 9;
    const int ox = (int)(rem % ow); rem /= ow;
    const int oy = (int)(rem % oh);
    const int b = (int)(rem / oh);
    const int iy = oy * 2 - 1 + tap / 3, ix = ox * 2 - 1 + tap % 3;
    uint4 v = uint4{0, 0, 0, 0};
    if (iy >= 0 && iy < in_h && ix >= 0 && ix < in_w) v = *(const uint4*)(in + ((size_t)b * img_rows + row0 + iy * in_w + ix) * C + cc * 8);
    *(uint4*)(col + idx * 8) = v;
}

// dst row i = table[ids[i]] (dm0_infer.py:753-755), 256 threads x 8 elements per 2048-wide row
__global__ void dm0_gather_rows_kernel(const bf16_t* __restrict__ table, int table_rows, const int* __restrict__ ids, bf16_t* __restrict__ dst) {
    const int id = min(max(ids[blockIdx.x], 0), table_rows - 1);
    *(uint4*)(dst + (size_t)blockIdx.x * 2048 + threadIdx.x * 8) = *(const uint4*)(table + (size_t)id * 2048 + threadIdx.x * 8);
}

// dm0_infer.py:236-306.  One wave per (row, head) of the bf16 QKV rows [rows][32 heads x 128]: value * RMS factor of the row;
// Q and K heads are RMS-normalised over their 128 features (eps 1e-6), scaled by the norm weight and rotated on adjacent
// pairs by the row's (cos, sin) table; V heads are only scaled.  Lane l holds features 2l, 2l+1 (one rotation pair).
// Q head h goes to the fragment-tiled [rows*2][128] matrix of K/V head h/2 at row token*2 + h%2, K to cache row
// key_row0 + token, V transposed to cache column key_row0 + token.  The factor is read from `factor` or, when that is
// null, computed from the row of the fragment-tiled activation matrix x [64][1024].
__global__ __launch_bounds__(256)
void dm0_qknorm_rope_kernel(const bf16_t* __restrict__ qkv, int ld, const float* __restrict__ factor, const bf16_t* __restrict__ x_tiled,
                            const bf16_t* __restrict__ qw, const bf16_t* __restrict__ kw, const bf16_t* __restrict__ rope,
                            bf16_t* __restrict__ q, size_t q_bstride, bf16_t* __restrict__ k, size_t k_bstride,
                            bf16_t* __restrict__ vt, size_t vt_bstride, int keys32, int key_row0, int rows) {
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (wave >= rows * 32) return;
    const int row = wave >> 5, head = wave & 31;
    float f;
    if (factor) f = factor[row];
    else {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const bf16x8 v = *(const bf16x8*)(x_tiled + ft_index(row, (lane * 2 + i) * 8, 32));
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += bf2f(v[j]) * bf2f(v[j]);
        }
        f = rsqrtf(wave_sum(ss) * (1.0f / 1024.0f) + 1e-6f);
    }
    const bf16_t* src = qkv + (size_t)row * ld + head * 128 + lane * 2;
    float v0 = bf2f(src[0]) * f, v1 = bf2f(src[1]) * f;
    if (head < 24) {
        const float inv = rsqrtf(wave_sum(v0 * v0 + v1 * v1) * (1.0f / 128.0f) + 1e-6f);
        const bf16_t* nw = head < 16 ? qw : kw;
        v0 = v0 * inv * bf2f(nw[lane * 2]); v1 = v1 * inv * bf2f(nw[lane * 2 + 1]);
        const float c = bf2f(rope[(size_t)row * 128 + lane * 2]), s = bf2f(rope[(size_t)row * 128 + lane * 2 + 1]);
        const float r0 = v0 * c - v1 * s, r1 = v1 * c + v0 * s;
        v0 = r0; v1 = r1;
    }
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 o; o[0] = f2bf(v0); o[1] = f2bf(v1);
    if (head < 16) *(bf16x2*)(q + (size_t)(head >> 1) * q_bstride + ft_index(row * 2 + (head & 1), lane * 2, 4)) = o;
    else if (head < 24) *(bf16x2*)(k + (size_t)(head - 16) * k_bstride + ft_index(key_row0 + row, lane * 2, 4)) = o;
    else {
        bf16_t* dst = vt + (size_t)(head - 24) * vt_bstride;
        dst[vt_index(lane * 2, key_row0 + row, keys32)] = o[0];
        dst[vt_index(lane * 2 + 1, key_row0 + row, keys32)] = o[1];
    }
}

__global__ void fill_bf16_kernel(bf16_t* p, size_t n, float v) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = f2bf(v);
}

}  // namespace

void launch_dm0_im2col_nchw(const bf16_t* images, bf16_t* patches, int ldp, int n_images, hipStream_t s) {
    const int rows = n_images * DM0_GRID * DM0_GRID;
    const int total = rows * ldp;
    hipLaunchKernelGGL(dm0_im2col_nchw_kernel, dim3((total + 255) / 256), dim3(256), 0, s, images, patches, ldp, rows);
}

void launch_dm0_embed_ln(const bf16_t* conv, const bf16_t* cls, const bf16_t* pos, const bf16_t* w, const bf16_t* b, bf16_t* x, int x_img_rows, int n_images, hipStream_t s) {
    hipLaunchKernelGGL(dm0_embed_ln_kernel, dim3(n_images * DM0_SEQ), dim3(256), 0, s, conv, cls, pos, w, b, x, x_img_rows);
}

void launch_dm0_im2col3x3(const bf16_t* in, int img_rows, int row0, int in_h, int in_w, int C, bf16_t* col, int n_images, hipStream_t s) {
    const int oh = (in_h + 2 - 3) / 2 + 1, ow = (in_w + 2 - 3) / 2 + 1;
    const size_t chunks = (size_t)n_images * oh * ow * 9 * (C >> 3);
    hipLaunchKernelGGL(dm0_im2col3x3_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, in, img_rows, row0, in_h, in_w, C, col, oh, ow, chunks);
}

void launch_dm0_gather_rows(const bf16_t* table, int table_rows, const int* ids, bf16_t* dst, int rows, hipStream_t s) {
    if (rows > 0) hipLaunchKernelGGL(dm0_gather_rows_kernel, dim3(rows), dim3(256), 0, s, table, table_rows, ids, dst);
}

void launch_dm0_qknorm_rope(const bf16_t* qkv, int ld, const float* factor, const bf16_t* x_tiled, const bf16_t* qw, const bf16_t* kw, const bf16_t* rope,
                            bf16_t* q, size_t q_bstride, bf16_t* k, size_t k_bstride, bf16_t* vt, size_t vt_bstride, int keys32, int key_row0, int rows,
                            hipStream_t s) {
    hipLaunchKernelGGL(dm0_qknorm_rope_kernel, dim3((rows * 32 + 3) / 4), dim3(256), 0, s, qkv, ld, factor, x_tiled, qw, kw, rope, q, q_bstride, k, k_bstride,
                       vt, vt_bstride, keys32, key_row0, rows);
}

__global__ void fill_f32_kernel(float* p, size_t n, float v) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
void launch_fill_f32(float* p, size_t n, float v, hipStream_t s) {
    if (n) hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n, v);
}
void launch_fill_bf16(bf16_t* p, size_t n, float v, hipStream_t s) {
    if (n) hipLaunchKernelGGL(fill_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n, v);
}
