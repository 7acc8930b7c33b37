// Host-side launch interface of the kernel files.  Every launcher enqueues on the given
// stream, allocates nothing and never synchronises, so all of them can be recorded
// into a HIP graph.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include "common.h"

// Kernels that need more than 64 KB of dynamic LDS have the limit raised once per device: the attribute belongs to the
// device's copy of the kernel, so a process that drives several GPUs sets it on each.  `done` is one bit mask per kernel
// instantiation (a function-local static of its launcher).  Returns 0 or the launcher error code 4.
#include <atomic>
inline int ensure_dynamic_lds(const void* kernel, size_t bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 4;
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && (done.load(std::memory_order_acquire) >> dev & 1)) return 0;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return 4;
    if (tracked) done.fetch_or((uint64_t)1 << dev, std::memory_order_release);
    return 0;
}

// ----- pre-tiled weights ------------------------------------------------------------
// A weight W[K][N] (row-major, "in x out") is re-laid out once as MFMA operand fragments:
// tile (nb, kb) holds the 16 columns nb*16.. and 32 rows kb*32.. as 64 lanes x 8 bf16,
// lane l = 16 g + r carrying W[kb*32 + 8 g + j][nb*16 + r], j = 0..7.  Tiles are stored
// [nb][kb] so that one column block streams contiguously along K.  K is padded to a
// multiple of 128 (the GEMM consumes 64-wide K stages in pairs) and N to a multiple of 16 with zeros.
static inline int k32_padded(int K) { return ((K + 127) / 128) * 4; }
static inline int n16_tiles(int N) { return (N + 15) / 16; }
// Tiles may further be grouped: with group size G the order is [nb / G][kb][nb % G], so that the G
// column tiles one GEMM workgroup consumes per K step are contiguous in memory (N padded to 16 G).
static inline size_t tiled_elems(int K, int N, int G = 1) { return (size_t)((n16_tiles(N) + G - 1) / G) * G * k32_padded(K) * 512; }
// The large-M GEMM uses 32x32x16 MFMAs and therefore "wide" tiles: 32 columns x 16 rows, lane l carrying
// W[kb*16 + 8 (l >> 5) + j][nb*32 + (l & 31)], stored [nb / G][kb][nb % G] with the same K padding.
static inline size_t tiled_elems_wide(int K, int N, int G) { return (size_t)(((N + 31) / 32 + G - 1) / G) * G * k32_padded(K) * 2 * 512; }

// rowscale (optional, K values): row k of W is multiplied by 1 + rowscale[k] before the rounding to bf16
void launch_pretile(const bf16_t* W, int K, int N, bf16_t* out, int G, int wide, hipStream_t s, const bf16_t* rowscale = nullptr);
// out[n] = sum_k v[k] W[k][n] in fp32 (one-time work at prepare)
void launch_vec_mat(const bf16_t* v, const bf16_t* W, int K, int N, float* out, hipStream_t s);
void launch_pretile_padded(const bf16_t* W, int K, int K_pad, int N, bf16_t* out, hipStream_t s);

// ----- large-M MFMA GEMM --------------------------------------------------------------
enum GemmEpilogue {
    EPI_BIAS = 0,      // out = acc + bias
    EPI_BIAS_GELU,     // out = gelu_tanh(acc + bias)
    EPI_PATCH,         // out = acc + bias + res[row % res_mod]
    EPI_GEGLU,         // out = gelu_tanh(acc(B0)) * acc(B1)
    EPI_PARTIAL,       // fp32 split-K partial
    EPI_QKV_ROPE,      // Gemma prefix: bf16 -> interleaved RoPE on Q,K -> Q / K cache / transposed V cache
    EPI_VIS_QKV,       // SigLIP: +bias, Q|K row-major, V transposed per (view, head)
    EPI_SWIGLU,        // out = silu(acc(B0) * rowscale[row]) * (acc(B1) * rowscale[row])   (DM0 prefix MLP)
    EPI_VIT_QKV_ROPE,  // DM0 ViT: +bias, bf16, 2-D rotary on Q and K (16 heads x 64), Q / K / V^T per (image, head)
};

struct GemmP {
    const bf16_t* A; int lda; int a_rows;      // activations, rows clamped to a_rows - 1
    const bf16_t* B0; const bf16_t* B1;        // pre-tiled weights
    int bgroup;                                // their (wide) tile group size G
    int M, N16, K32p;                          // valid rows, column tiles, padded k32 count
    int nsplit;                                // split-K factor (EPI_PARTIAL only when > 1)
    bf16_t* out; int ldo;
    const bf16_t* bias;
    const float* bias_f32;                     // fp32 bias instead of `bias` (DM0's folded LayerNorm biases)
    const float* rowscale;                     // per-row factor applied to the accumulators (EPI_SWIGLU)
    int seq, seq_pad;                          // EPI_VIT_QKV_ROPE: tokens per image and their padded count in the Q / K / V^T tiles
    const bf16_t* res; int ldr; int res_mod;
    float* partial; int ldp; size_t pstride;   // [split][row][ldp]
    const bf16_t* rope;                        // [row][256] = cos0 sin0 cos1 sin1 ...
    bf16_t* q; bf16_t* k; bf16_t* vt; int ldvt;
};
// workgroup tile (rows x columns), 4 waves each owning 64 columns (two 32-column MFMA tiles).  The tiles of 128 rows and
// more by 256 columns are upper bounds: their launches mix row blocks of that many and of 32 fewer rows so that the
// blocks cover ceil(M / 32) 32-row tiles exactly.
enum GemmTile { TILE_224x256 = 0, TILE_192x256, TILE_160x256, TILE_128x256, TILE_64x256, TILE_64x128, TILE_128x128,
                // the same 256-column tiles computed by eight waves (csrc/gemm8.hip), row-major epilogues only
                TILE8_256x256, TILE8_224x256, TILE8_192x256, TILE8_128x256,
                TILE_96x128, TILE_COUNT };
inline bool gemm_tile_eight_waves(int tile) { return tile >= TILE8_256x256 && tile <= TILE8_128x256; }
int gemm_tile_bm(int tile);
int gemm_tile_bn(int tile);
int launch_gemm(const GemmP& p, int epi, int tile, hipStream_t s);
int launch_gemm8(const GemmP& p, int epi, int tile, hipStream_t s);

// ----- split-K reduce + bias + residual (+ gate) + normalisation -----------------------
enum NormMode { NORM_NONE = 0, NORM_RMS, NORM_LAYER };
struct ReduceP {
    const float* partial; size_t pstride; int ldp; int nsplit;   // nsplit may be 0
    const bf16_t* bias; const bf16_t* res; int ldr;
    bf16_t* x; int ldx;                         // new residual stream (may be null)
    bf16_t* xn; int ldxn;                       // normalised copy (may be null)
    int M, N;
    int norm; const bf16_t* nw; const bf16_t* nb; float eps;
    float* factor;                              // NORM_RMS: the row's rsqrt(mean x^2 + eps) as fp32 (may be null; xn may then be null too)
};
int launch_reduce(const ReduceP& p, hipStream_t s);

// ----- skinny (M <= 64) weight-streaming GEMM ---------------------------------------------
enum SkinnyEpilogue {
    SK_BIAS = 0,       // out = acc + bias
    SK_BIAS_SILU,      // out = silu(acc + bias)
    SK_RES,            // out += acc (* gate[col])
    SK_QKV_ROPE,       // RoPE + scatter to Q / K cache rows / transposed V cache columns
    SK_GEGLU,          // out = gelu_tanh(acc(B0)) * acc(B1)
    SK_SWIGLU,         // out = silu(acc(B0)) * acc(B1)
};
enum SkinnyNorm { SN_NONE = 0, SN_RMS, SN_ADARMS };
struct SkinnyP {
    const bf16_t* A; int lda; int M;           // valid rows (<= 64)
    int a_tiled; int a_row0;                   // A in the fragment-tiled layout; first row inside it
    int out_tiled; int out_row0;               // same for `out`
    const bf16_t* B0; const bf16_t* B1; int K; int N16; int K32p;
    int norm; const bf16_t* style;             // SN_ADARMS: [scale | shift | gate] each K wide
    float eps;
    int factor_f32;                            // SN_RMS: keep the row factor in fp32 (DM0) instead of rounding it to bf16 (Pi0)
    bf16_t* out; int ldo;
    const bf16_t* bias; const bf16_t* gate;    // per-column
    const float* col_bias0; const float* col_bias1;   // SN_RMS with SK_QKV_ROPE / SK_GEGLU: fp32 per-column terms added after the row factor
                                               // (Pi05: the shift of the adaptive RMS norm times the weights, see Sched::prepare)
    const bf16_t* rope;                        // [row][256]
    bf16_t* q; bf16_t* k; bf16_t* vt; int ldvt; int kv_row0;
};
int launch_skinny(const SkinnyP& p, int epi, hipStream_t s);

// out[m][n] = act(bias[n] + sum_k x[m][k] W[k][n]) for tiny K (<= 64), W in its original layout
// (`out` fragment-tiled with first row out_row0 when out_tiled)
void launch_small_linear(const bf16_t* x, int ldx, const bf16_t* W, const bf16_t* bias, bf16_t* out, int ldo,
                         int M, int K, int N, int act_silu, int out_tiled, int out_row0, hipStream_t s);
struct SmallLinearJob { const bf16_t* x; int ldx; const bf16_t* W; const bf16_t* bias; bf16_t* out; int ldo; int M, K, N, act_silu, out_tiled, out_row0; };
void launch_small_linear2(const SmallLinearJob& a, const SmallLinearJob& b, hipStream_t s);      // two independent jobs in one launch (b.M = 0: one)

// ----- attention --------------------------------------------------------------------------
struct AttnP {
    // query rows are token * group + head for the `group` query heads that share the K/V head; HD = head width
    const bf16_t* q;                 // fragment-tiled [rows padded to the workgroup tile][HD]
    const bf16_t* k;                 // fragment-tiled [keys padded to 32][HD]
    const bf16_t* vt; int ldvt;      // permuted-key tiled V^T [HD][ldvt], ldvt = keys padded to 32
    int batch; size_t q_bstride, k_bstride, vt_bstride;        // independent K/V heads (blockIdx.y) and their strides, in elements
    int group;
    // output element (row, d): row-major  out[bo * out_ostride + bi * out_istride + token * ld_tok + head * HD + d]  with the batch
    // index split as bo * batch_inner + bi, or (out_tiled) the fragment-tiled [tokens][32 out_cols32] matrix at column
    // batch * out_bcol + head * HD + d
    bf16_t* out; int ld_tok; int batch_inner; size_t out_ostride, out_istride;
    int out_tiled, out_bcol, out_cols32;
    int rows, keys;
    float scale;
    int causal;                      // key j visible to row r only if j <= r / group (keys and tokens count from the same origin)
    // masking: key j is visible to row r iff
    //   j < prefix_alloc ? j < *valid_len (or prefix_alloc if valid_len == null)
    //                    : (r >= state_rows || j == prefix_alloc)
    int prefix_alloc; const int* valid_len; int state_rows;
    // key split over workgroups (nsplit > 1, at most 16): fp32 partial records, combined by a second launch
    int nsplit; float* partial; size_t partial_floats;
    int kb_per_split, nsplit_eff, row_blocks;    // filled by the launcher
    // key-split suffix passes only: weight tiles of a later launch that extra ("riding") workgroups of the attention launch pull
    // towards the caches (the launch streams no weights itself and its grid leaves CUs idle)
    PrefetchP pf_attn;
    int riders;                                  // filled by the launcher: riding workgroups, first in the grid (a multiple of 8)
};
// Gemma (HD 256): many rows, two row tiles per workgroup / few rows, one row tile and a key split; DM0 grouped-query (HD 128)
// prefix and suffix (the ViT attention, HD 64, is launch_flash_attention)
enum AttnVariant { ATTN_PREFIX = 0, ATTN_SUFFIX = 1, ATTN_GQA128_PREFIX, ATTN_GQA128_SUFFIX };
int launch_mqa_attention(const AttnP& p, int variant, hipStream_t s, int* kernels_launched = nullptr);
// long sequences on both sides (csrc/flash.hip): 128 query rows per workgroup, K / V^T tiles shared through LDS; hd = 64
int launch_flash_attention(const AttnP& p, int hd, hipStream_t s);
// SigLIP attention: q, k fragment-tiled [views*16][256][96], vt tiled [views*16][80][256], out row-major
void launch_vision_attention(const bf16_t* q, const bf16_t* k, const bf16_t* vt, bf16_t* out, int views, hipStream_t s);

// Row-major q [tokens][kv_heads][group][hd], k / v [keys][kv_heads][hd] -> the kernels' layouts per K/V head b: Q fragment-tiled
// [row = local token * group + head][hd_pad] at qt + b' * q_bstride, K fragment-tiled [key][hd_pad], V^T tiled [hd][keys_pad];
// with seq > 0 the tokens / keys form independent sequences of `seq` (SigLIP views) and b' = sequence * kv_heads + b.  The
// destination must be zero beforehand (padding).
void launch_attn_tile_operands(const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* qt, bf16_t* kt, bf16_t* vtt, int tokens, int keys,
                               int kv_heads, int group, int hd, int hd_pad, size_t q_bstride, size_t k_bstride, size_t vt_bstride, int keys_pad,
                               int seq, hipStream_t s);

// ----- small helpers ------------------------------------------------------------------------
void launch_prompt_stage(const bf16_t* emb, int vocab, const int* ids, const int* valid_len, bf16_t* x_rows, int prompt_rows, int s_v,
                         float scale, const bf16_t* rope_full, int rope_rows, bf16_t* dec_rope, int dec_rows, hipStream_t s);
void launch_im2col(const bf16_t* images, bf16_t* patches, int ldp, int views, hipStream_t s);
void launch_copy_rows(const bf16_t* src, int lds, bf16_t* dst, int ldd, int rows, int cols, hipStream_t s);
void launch_fill_zero(void* p, size_t bytes, hipStream_t s);
void launch_fill_bf16(bf16_t* p, size_t n, float v, hipStream_t s);
void launch_fill_f32(float* p, size_t n, float v, hipStream_t s);

// ----- DM0 (csrc/dm0.hip) ---------------------------------------------------------------------
void launch_dm0_im2col_nchw(const bf16_t* images, bf16_t* patches, int ldp, int n_images, hipStream_t s);
void launch_dm0_embed_ln(const bf16_t* conv, const bf16_t* cls, const bf16_t* pos, const bf16_t* w, const bf16_t* b, bf16_t* x, int x_img_rows, int n_images, hipStream_t s);
void launch_dm0_im2col3x3(const bf16_t* in, int img_rows, int row0, int in_h, int in_w, int C, bf16_t* col, int n_images, hipStream_t s);
void launch_dm0_gather_rows(const bf16_t* table, int table_rows, const int* ids, bf16_t* dst, int rows, hipStream_t s);
void launch_dm0_qknorm_rope(const bf16_t* qkv, int ld, const float* factor, const bf16_t* x_tiled, const bf16_t* qw, const bf16_t* kw, const bf16_t* rope,
                            bf16_t* q, size_t q_bstride, bf16_t* k, size_t k_bstride, bf16_t* vt, size_t vt_bstride, int keys32, int key_row0, int rows,
                            hipStream_t s);
void launch_scale_inplace(bf16_t* p, size_t n, float f, hipStream_t s);
void launch_copy_bytes(const void* src, void* dst, size_t bytes, hipStream_t s);
