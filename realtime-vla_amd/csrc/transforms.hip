// Observation pre-/post-processing either side of the forward pass, on the device:
// /root/reference/test.py:88-201 (`_resize_with_pad`, `_normalize_image`, `_normalize_state`, `_digitize_state`,
// `_unnormalize_actions`, and the delta-to-absolute step of `infer`), which the reference runs in numpy / Pillow on
// the host per observation.
//
// The resize reproduces Pillow's `Image.resize(..., BILINEAR)` bit for bit: triangle filter with the support stretched
// by the shrink factor, double-precision weights normalised per output pixel, 22-bit fixed point, a horizontal pass to
// an 8-bit intermediate and a vertical pass, each rounded to nearest and clipped.  Every thread derives the weights of
// its own output pixel (a dozen double operations per tap), so there are no coefficient tables to upload and the
// kernels can be captured in a graph.  This file is compiled with floating-point contraction off: a fused
// multiply-add would round the weights differently from the C code being matched.
#include "../../include/rtvla.h"
#include "common.h"
#include <math.h>
#include <mutex>

// 8-bit intermediate of the horizontal pass for rtvla_preprocess_image_static: part of the code object, so every
// GPU the library runs on holds its own copy at its own address from load until the process ends.  Host code
// never passes this name to a kernel; it uses the per-device address resolved in static_scratch_ptr().
static __device__ __align__(256) unsigned char scratch[RTVLA_STATIC_SCRATCH_BYTES];

namespace {

constexpr int PRECISION_BITS = 32 - 8 - 2;
constexpr int MAX_TAPS = 64;            // ceil(scale) * 2 + 1 taps: shrink factors up to 31

struct Window { int first, count; double center, ss, ww; };

// the source window and weight sum of output index xx (Resample.c: precompute_coeffs)
RTVLA_DEVICE Window window_of(int xx, int in_size, int out_size) {
    const double scale = (double)in_size / (double)out_size;
    const double filterscale = scale < 1.0 ? 1.0 : scale;
    const double support = 1.0 * filterscale;
    Window w;
    w.center = 0.0 + (xx + 0.5) * scale;
    w.ss = 1.0 / filterscale;
    int xmin = (int)(w.center - support + 0.5);
    if (xmin < 0) xmin = 0;
    int xmax = (int)(w.center + support + 0.5);
    if (xmax > in_size) xmax = in_size;
    w.first = xmin; w.count = xmax - xmin;
    double ww = 0.0;
    for (int x = 0; x < w.count; ++x) {
        double a = (x + xmin - w.center + 0.5) * w.ss;
        if (a < 0.0) a = -a;
        ww += a < 1.0 ? 1.0 - a : 0.0;
    }
    w.ww = ww;
    return w;
}

RTVLA_DEVICE int tap_weight(const Window& w, int x) {
    double a = (x + w.first - w.center + 0.5) * w.ss;
    if (a < 0.0) a = -a;
    double k = a < 1.0 ? 1.0 - a : 0.0;
    if (w.ww != 0.0) k /= w.ww;
    return k < 0 ? (int)(-0.5 + k * (double)(1 << PRECISION_BITS)) : (int)(0.5 + k * (double)(1 << PRECISION_BITS));
}

RTVLA_DEVICE int clip8(int v) { v >>= PRECISION_BITS; return v < 0 ? 0 : (v > 255 ? 255 : v); }

// horizontal pass: src [h][w][3] -> tmp [h][rw][3]
__global__ void resample_h_kernel(const uint8_t* __restrict__ src, int h, int w, int rw, uint8_t* __restrict__ tmp) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= h * rw) return;
    const int y = idx / rw, xx = idx - y * rw;
    const Window win = window_of(xx, w, rw);
    int acc[3] = {1 << (PRECISION_BITS - 1), 1 << (PRECISION_BITS - 1), 1 << (PRECISION_BITS - 1)};
    const uint8_t* row = src + ((size_t)y * w + win.first) * 3;
    for (int x = 0; x < win.count; ++x) {
        const int k = tap_weight(win, x);
        acc[0] += row[x * 3 + 0] * k; acc[1] += row[x * 3 + 1] * k; acc[2] += row[x * 3 + 2] * k;
    }
    uint8_t* o = tmp + (size_t)idx * 3;
    o[0] = (uint8_t)clip8(acc[0]); o[1] = (uint8_t)clip8(acc[1]); o[2] = (uint8_t)clip8(acc[2]);
}

// vertical pass + paste on the black 224 x 224 canvas + x / 255 * 2 - 1 -> bf16 NHWC
__global__ void resample_v_pad_norm_kernel(const uint8_t* __restrict__ tmp, int h, int rw, int rh, int pad_top, int pad_left,
                                           bf16_t* __restrict__ dst) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= 224 * 224) return;
    const int yy = idx / 224, xx = idx - yy * 224;
    int v[3] = {0, 0, 0};
    const int ry = yy - pad_top, rx = xx - pad_left;
    if (ry >= 0 && ry < rh && rx >= 0 && rx < rw) {
        const Window win = window_of(ry, h, rh);
        int acc[3] = {1 << (PRECISION_BITS - 1), 1 << (PRECISION_BITS - 1), 1 << (PRECISION_BITS - 1)};
        for (int y = 0; y < win.count; ++y) {
            const int k = tap_weight(win, y);
            const uint8_t* p = tmp + ((size_t)(win.first + y) * rw + rx) * 3;
            acc[0] += p[0] * k; acc[1] += p[1] * k; acc[2] += p[2] * k;
        }
        v[0] = clip8(acc[0]); v[1] = clip8(acc[1]); v[2] = clip8(acc[2]);
    }
#pragma unroll
    for (int c = 0; c < 3; ++c) dst[(size_t)idx * 3 + c] = f2bf((float)v[c] / 255.0f * 2.0f - 1.0f);
}

// state: mode 0 (Pi0) (x - a) / (b + 1e-6), a = mean, b = std; mode 1 (Pi05) (x - a) / (b - a + 1e-6) * 2 - 1, a = q01, b = q99
// (statistics and state zero-padded to 32 like _pad_to_dim); then float32 -> bf16 for the model and the 256-bin index
__global__ void state_kernel(const double* __restrict__ state, int n, const double* __restrict__ a, const double* __restrict__ b, int n_stats,
                             int mode, bf16_t* __restrict__ out_bf16, double* __restrict__ out_f64, int32_t* __restrict__ bins) {
    const int i = threadIdx.x;
    if (i >= 32) return;
    const double x = i < n ? state[i] : 0.0, av = i < n_stats ? a[i] : 0.0, bv = i < n_stats ? b[i] : 0.0;
    const double z = mode == 0 ? (x - av) / (bv + 1e-6) : (x - av) / (bv - av + 1e-6) * 2.0 - 1.0;
    if (out_f64) out_f64[i] = z;
    if (out_bf16) out_bf16[i] = f2bf((float)z);
    if (bins) {
        // np.digitize(z, linspace(-1, 1, 257)[:-1]) - 1: number of edges <= z, minus one; edge j is what
        // numpy's linspace yields: -1 + j * (2 / 256) (the step is exact in binary)
        int cnt = 0;
        for (int j = 0; j < 256; ++j) cnt += (-1.0 + j * (2.0 / 256.0)) <= z;
        bins[i] = cnt - 1;
    }
}

// actions: bf16 [chunk][32] -> float32 -> un-normalise in double -> first action_dim columns + state, gripper columns
// (every 7th) get the state taken off again, exactly in the reference's order of operations
__global__ void actions_kernel(const bf16_t* __restrict__ actions, int chunk, const double* __restrict__ a, const double* __restrict__ b,
                               int n_stats, int mode, const double* __restrict__ ori_state, int action_dim, double* __restrict__ out) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= chunk * action_dim) return;
    const int r = idx / action_dim, d = idx - r * action_dim;
    const float x = bf2f(actions[r * 32 + d]);
    const double av = d < n_stats ? a[d] : 0.0, bv = d < n_stats ? b[d] : 0.0;
    double v;
    if (mode == 0) v = (double)x * (bv + 1e-6) + av;                               // a = mean, b = std
    else v = (double)((x + 1.0f) / 2.0f) * (bv - av + 1e-6) + av;                  // a = q01, b = q99; (x + 1) / 2 stays float32
    v = v + ori_state[d];
    if (d % 7 == 6 && d < (action_dim / 7) * 7) v = v - ori_state[d];
    out[idx] = v;
}

// geometry, limits and the two launches shared by rtvla_preprocess_image and rtvla_preprocess_image_static;
// `get_scratch` is asked for the intermediate buffer only after every size check has passed
template <typename GetScratch>
int preprocess_image_impl(const void* src_u8, int height, int width, void* dst_bf16, size_t scratch_bytes, int too_small_code,
                          GetScratch get_scratch, void* stream) {
    if (!src_u8 || !dst_bf16 || height <= 0 || width <= 0) return RTVLA_ERR_ARG;
    // geometry of test.py:105-116 (Python float arithmetic = C double arithmetic)
    int rh = 224, rw = 224, pad_top = 0, pad_left = 0;
    if (!(width == 224 && height == 224)) {
        const double rwf = (double)width / 224, rhf = (double)height / 224;
        const double ratio = rwf > rhf ? rwf : rhf;
        rh = (int)((double)height / ratio); rw = (int)((double)width / ratio);
        pad_top = (int)((double)(224 - rh) / 2); if (pad_top < 0) pad_top = 0;
        pad_left = (int)((double)(224 - rw) / 2); if (pad_left < 0) pad_left = 0;
    }
    if (rh < 1 || rw < 1 || rh > 224 || rw > 224) return RTVLA_ERR_ARG;
    const double sx = (double)width / rw, sy = (double)height / rh;
    if ((int)ceil(sx > 1.0 ? sx : 1.0) * 2 + 1 > MAX_TAPS || (int)ceil(sy > 1.0 ? sy : 1.0) * 2 + 1 > MAX_TAPS) return RTVLA_ERR_LIMIT;
    if (scratch_bytes < (size_t)height * rw * 3) return too_small_code;
    uint8_t* tmp = nullptr;
    hipStream_t s = (hipStream_t)stream;
    if (int rc = get_scratch(&tmp, s)) return rc;
    const int n1 = height * rw;
    hipLaunchKernelGGL(resample_h_kernel, dim3((n1 + 255) / 256), dim3(256), 0, s, (const uint8_t*)src_u8, height, width, rw, tmp);
    hipLaunchKernelGGL(resample_v_pad_norm_kernel, dim3((224 * 224 + 255) / 256), dim3(256), 0, s, (const uint8_t*)tmp, height, rw, rh,
                       pad_top, pad_left, (bf16_t*)dst_bf16);
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

// Device address of `scratch` on the current device, resolved once per device with that device current.
constexpr int MAX_DEVICES = 64;
std::mutex static_scratch_mutex;
void* static_scratch_addr[MAX_DEVICES] = {};

// The lookup loads the code object and is not stream work: it must not happen while `s` is being captured into a graph,
// so a first call on a device that comes under capture is refused (RTVLA_ERR_STATE) and any earlier eager call resolves it.
int static_scratch_ptr(uint8_t** out, hipStream_t s) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return RTVLA_ERR_DEVICE;
    std::lock_guard<std::mutex> lock(static_scratch_mutex);
    if (!static_scratch_addr[dev]) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cap) != hipSuccess) return RTVLA_ERR_DEVICE;
        if (cap != hipStreamCaptureStatusNone) return RTVLA_ERR_STATE;
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return RTVLA_ERR_DEVICE;
        static_scratch_addr[dev] = ptr;
    }
    *out = (uint8_t*)static_scratch_addr[dev];
    return RTVLA_OK;
}

}  // namespace

extern "C" {

size_t rtvla_preprocess_image_scratch(int height, int width) {
    if (height <= 0 || width <= 0) return 0;
    return ((size_t)height * 224 * 3 + 255) & ~(size_t)255;       // the horizontal pass never produces more than 224 columns
}

int rtvla_preprocess_image(const void* src_u8, int height, int width, void* dst_bf16, void* scratch_arg, size_t scratch_bytes, void* stream) {
    if (!scratch_arg) return RTVLA_ERR_ARG;
    return preprocess_image_impl(src_u8, height, width, dst_bf16, scratch_bytes, RTVLA_ERR_SIZE,
                                 [&](uint8_t** out, hipStream_t) { *out = (uint8_t*)scratch_arg; return (int)RTVLA_OK; }, stream);
}

int rtvla_preprocess_image_static(const void* src_u8, int height, int width, void* dst_bf16, void* stream) {
    return preprocess_image_impl(src_u8, height, width, dst_bf16, (size_t)RTVLA_STATIC_SCRATCH_BYTES, RTVLA_ERR_LIMIT, static_scratch_ptr, stream);
}

int rtvla_preprocess_state(const double* state, int n, const double* stat_a, const double* stat_b, int n_stats, int mode,
                           void* out_bf16, double* out_f64, int32_t* out_bins, void* stream) {
    if (!state || !stat_a || !stat_b || n < 0 || n > 32 || n_stats < 0 || n_stats > 32 || (mode != 0 && mode != 1)) return RTVLA_ERR_ARG;
    hipLaunchKernelGGL(state_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, state, n, stat_a, stat_b, n_stats, mode, (bf16_t*)out_bf16, out_f64, out_bins);
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

int rtvla_postprocess_actions(const void* actions_bf16, int chunk, const double* stat_a, const double* stat_b, int n_stats, int mode,
                              const double* ori_state, int action_dim, double* out, void* stream) {
    if (!actions_bf16 || !stat_a || !stat_b || !ori_state || !out || chunk <= 0 || action_dim <= 0 || action_dim > 32 || n_stats < 0 || n_stats > 32 ||
        (mode != 0 && mode != 1)) return RTVLA_ERR_ARG;
    const int n = chunk * action_dim;
    hipLaunchKernelGGL(actions_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)actions_bf16, chunk, stat_a, stat_b, n_stats,
                       mode, ori_state, action_dim, out);
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

}  // extern "C"
