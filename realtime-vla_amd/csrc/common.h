// Shared device helpers for the gfx950 kernels: bf16 vector types, MFMA wrapper,
// packing, activation functions and the XCD-aware block remap.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define RTVLA_DEVICE __device__ __forceinline__

// D[16x16] += A[16x32] * B[32x16] on one wavefront.
// Operand layout (lane l, g = l / 16, r = l % 16):
//   a[j] = A[r][8 g + j], b[j] = B[8 g + j][r], d[v] = D[4 g + v][r].
RTVLA_DEVICE f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

RTVLA_DEVICE float bf2f(bf16_t x) { return (float)x; }
RTVLA_DEVICE bf16_t f2bf(float x) { return (bf16_t)x; }
RTVLA_DEVICE float round_bf16(float x) { return (float)(bf16_t)x; }

RTVLA_DEVICE bf16x4 pack4(float a, float b, float c, float d) {
    bf16x4 r;
    r[0] = (bf16_t)a; r[1] = (bf16_t)b; r[2] = (bf16_t)c; r[3] = (bf16_t)d;
    return r;
}
RTVLA_DEVICE bf16x4 pack4(f32x4 v) { return pack4(v[0], v[1], v[2], v[3]); }

RTVLA_DEVICE bf16x4 load4(const bf16_t* p) { return *(const bf16x4*)p; }
RTVLA_DEVICE void store4(bf16_t* p, bf16x4 v) { *(bf16x4*)p = v; }

// hardware reciprocal and base-2 exponential (1 ulp each) instead of an IEEE division and expf: two transcendental
// instructions and no range fix-ups; the result is rounded to bf16 anyway.  exp2 saturates to 0 / inf, so the
// sigmoid is exactly 1 / 0 at the far ends and never NaN for finite input.
RTVLA_DEVICE float sigmoidf_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x)); }
// tanh-approximated GELU written as a * sigmoid(2 sqrt(2/pi) (a + 0.044715 a^3)), the constants pre-multiplied by -log2(e)
RTVLA_DEVICE float gelu_tanh(float a) {
    const float w = a * (-2.3022081981462776f + -0.10294323958057285f * (a * a));
    return a * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(w));
}
RTVLA_DEVICE float siluf(float a) { return a * sigmoidf_fast(a); }

// The hardware dispatcher deals consecutive workgroup ids round-robin over the 8 XCDs
// (each with a private L2).  Map the hardware id to a logical id so that consecutive
// logical ids share an XCD; callers make tiles that share an operand consecutive.
RTVLA_DEVICE int xcd_remap(int bid, int total) {
    const int q = total >> 3, r = total & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    return xcd * q + (xcd < r ? xcd : r) + idx;
}

// Fragment-tiled activation layout: a [rows][cols] matrix (cols a multiple of 32) stored as MFMA
// operand fragments, tile (row/16, col/32) = 64 lanes x 8 bf16 with lane = row%16 + 16*((col%32)/8).
// A wave reads one fragment as one contiguous 1 KB load (lane l takes bytes 16 l .. 16 l + 15).
RTVLA_DEVICE size_t ft_index(int row, int col, int cols32) {
    return ((size_t)((row >> 4) * cols32 + (col >> 5)) * 64 + (row & 15) + 16 * ((col & 31) >> 3)) * 8 + (col & 7);
}
// Transposed-V layout for attention: element (d, key) of V^T, tile (d/16, key/32); inside a tile the
// 32 keys are permuted so that lane 16 g + r, register j holds key 4 g + (j & 3) + 16 (j >> 2): the
// order in which the probabilities come out of the S^T = K Q^T accumulators.
RTVLA_DEVICE size_t vt_index(int d, int key, int keys32) {
    const int mm = key & 31;
    return ((size_t)((d >> 4) * keys32 + (key >> 5)) * 64 + (d & 15) + 16 * ((mm & 15) >> 2)) * 8 + 4 * (mm >> 4) + (mm & 3);
}

// Reductions across the four 16-lane rows of a wavefront (lanes that differ in bits 4 and 5) with gfx950's register-file
// swaps instead of LDS permutes: v_permlane16_swap exchanges the odd rows of one register with the even rows of another,
// v_permlane32_swap the upper half of one with the lower half of the other, so after swapping a value with its own copy
// every lane holds its own and its partner's value in the two registers (a dependent ds_bpermute costs an LDS round trip).
typedef unsigned rtvla_u2 __attribute__((ext_vector_type(2)));
RTVLA_DEVICE float rows_max(float v) {
    rtvla_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
RTVLA_DEVICE float rows_sum(float v) {
    rtvla_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
RTVLA_DEVICE float halves_max(float v) {
    const rtvla_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
RTVLA_DEVICE float halves_sum(float v) {
    const rtvla_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

RTVLA_DEVICE float wave_sum(float v) {
    v = rows_sum(v);
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
