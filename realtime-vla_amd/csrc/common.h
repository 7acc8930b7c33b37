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

// Pulling weight tiles that a LATER launch of the same graph will stream towards the caches: every thread reads one word of
// each 128-byte line of its share of a tile and throws it away (the empty asm keeps the loads alive and makes the wave wait for
// them before it ends).  What the later launch gains is the memory-side cache: its own L2 fills for those tiles stay the same
// (FETCH_SIZE of the consumer does not drop: an XCD's L2 does not carry lines across a launch boundary), they only come
// back sooner.  Workgroup e is still given the tile that the consumer processes on the same XCD (tile index = workgroup index
// modulo 8 when both grids are dealt round-robin over the XCDs), which costs nothing.  A launch cannot end before its riders'
// loads have come back, and such touches draw only ~3.5 TB/s from HBM: measured on the action expert, riders that fetch the
// 4 MB of the output projection during the suffix attention pay (0.7 us per layer), riders that fetch the 16.8 MB of the gate /
// up weights during the attention or the merge launch lengthen that launch by 4-6 us and save 2.3 us in the consumer.
struct PrefetchP {
    const char* base[4];        // up to four weight blocks
    int tile_bytes[4];          // contiguous bytes per tile (at most 4 x 128 x the workgroup's thread count)
    int n_tiles[4];             // tiles (= riding workgroups) per block, multiples of 8; 0 ends the list
};
static inline int prefetch_wgs(const PrefetchP& p) { int n = 0; for (int k = 0; k < 4 && p.n_tiles[k] > 0; ++k) n += p.n_tiles[k]; return n; }
template <int NTHREADS>
RTVLA_DEVICE void prefetch_tile(const PrefetchP& p, int e, int tid) {
    // every field is read before the first branch: one round of scalar loads instead of a dependent chain
    const int n0 = p.n_tiles[0], n1 = p.n_tiles[1], n2 = p.n_tiles[2], n3 = p.n_tiles[3];
    const int b0 = p.tile_bytes[0], b1 = p.tile_bytes[1], b2 = p.tile_bytes[2], b3 = p.tile_bytes[3];
    const char* const a0 = p.base[0]; const char* const a1 = p.base[1]; const char* const a2 = p.base[2]; const char* const a3 = p.base[3];
    const int e1 = e - n0, e2 = e1 - n1, e3 = e2 - n2;
    const char* a = a0; int bytes = b0, idx = e;
    if (e1 >= 0) { a = a1; bytes = b1; idx = e1; }
    if (e2 >= 0) { a = a2; bytes = b2; idx = e2; }
    if (e3 >= 0) { a = a3; bytes = b3; idx = e3; }
    if (e3 >= n3) return;
    const char* t = a + (size_t)idx * bytes;
    unsigned v[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int off = min((i * NTHREADS + tid) * 128, bytes - 128);       // (tiles shorter than the unrolled reach re-read their last line)
        v[i] = *(const unsigned*)(t + off);
    }
    asm volatile("" ::"v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]));
}
