/* rtvla - C ABI of the MI355X (gfx950) Pi0 / Pi05 / DM0 single-observation forward pass.
 *
 * The reference (Dexmal/realtime-vla) has no native layer: its device code is Triton JIT and its
 * "operator interface" is the Python object Pi0Inference / Pi05Inference / DM0Inference.  This ABI is what a
 * Python (ctypes) front end with that object's signature binds instead of the Triton kernels.
 * Every entry point takes plain pointers and sizes, returns an int status (0 = ok, see
 * rtvla_status) and never throws; device memory is always owned by the caller.
 *
 * Life cycle:   rtvla_create -> rtvla_bind (every weight / io buffer) -> rtvla_bind_workspace
 *            -> rtvla_prepare -> [rtvla_graph_capture] -> rtvla_forward / rtvla_graph_launch ...
 *            -> rtvla_destroy.
 * One context = one static shape set (views, prompt length, chunk); single host thread per
 * context; calls that enqueue work on the same context must not overlap.
 */
#ifndef RTVLA_H
#define RTVLA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rtvla_ctx rtvla_ctx;

enum rtvla_status {
    RTVLA_OK = 0,
    RTVLA_ERR_ARG = 1,        /* null pointer, bad size, unsupported dimension            */
    RTVLA_ERR_NAME = 2,       /* unknown tensor name                                       */
    RTVLA_ERR_SIZE = 3,       /* byte size does not match the tensor's shape               */
    RTVLA_ERR_STATE = 4,      /* call out of order (e.g. forward before prepare)           */
    RTVLA_ERR_UNBOUND = 5,    /* a required tensor was never bound                         */
    RTVLA_ERR_DEVICE = 6,     /* HIP runtime error; text in rtvla_last_error               */
    RTVLA_ERR_LIMIT = 7       /* shape outside the supported range                         */
};

enum rtvla_model { RTVLA_PI0 = 0, RTVLA_PI05 = 1, RTVLA_DM0 = 2 };

/* Static shape set of one inference object.
 * Replaces the constructor arguments and literals of Pi0Inference.__init__
 * (/root/reference/pi0_infer.py:1239-1243, :1289-1290), Pi05Inference.__init__
 * (/root/reference/pi05_infer.py:531-561, :615-616) and DM0Inference.__init__
 * (/root/reference/dm0_infer.py:965-983).
 *
 * RTVLA_DM0 (the reference's third model, dm0_infer.py): num_views images of 728x728 (bf16 NCHW, already normalised),
 * prompt_len = max_lang_len token ids (int32 "input_ids", looked up in "vision_embed_tokens_w"), a ViT of
 * vision_layers (23) layers of width 1024 over 2705 tokens per image, two stride-2 convolutions and a projector to
 * 169 tokens of width 2048 per image, llm_layers (28) causal grouped-query prefix layers and as many action-expert
 * layers.  Its tensor table is dm0_infer.py:986-1026 by name; the 4-byte tensors among the weights (the folded
 * LayerNorm biases and column sums, :1013-1018) are fp32, every other weight is bf16.  The caller also binds the three
 * rotary tables: "vision_rope" bf16 [2705][64] = (cos, sin) per rotation pair of the 2-D embedding (:671-688),
 * "prefix_rope_weights" [169 views + prompt_len][128] and "decoder_rope_weights" [chunk][128] (:1080-1094). */
typedef struct rtvla_dims {
    int32_t model;           /* rtvla_model                                                          */
    int32_t num_views;       /* 1..4 camera views of 224x224x3 (DM0: images of 728x728)               */
    int32_t prompt_len;      /* Pi0: rows of language_embeds; Pi05: max_prompt_len (allocated rows);
                                DM0: max_lang_len (token ids)                                          */
    int32_t chunk_size;      /* action chunk; Pi0 suffix = chunk+1 rows, Pi05 / DM0 = chunk rows (Pi0 / Pi05: <= 128 rows, DM0: <= 64) */
    int32_t num_steps;       /* Euler flow steps.  Pi0 / DM0: exactly 10, because the converted checkpoint has dt = -1/10 folded
                                into the output projection and 10 fused time biases (RTVLA_ERR_LIMIT otherwise); Pi05: 1..10 */
    int32_t vision_layers;   /* SigLIP layers (27); DM0: ViT layers (23)                               */
    int32_t llm_layers;      /* prefix layers == action-expert layers (18; DM0: 28)                    */
} rtvla_dims;

/* Stages of the forward schedule, for per-stage execution (layer taps, profiling).
 * A whole forward is: VISION_EMBED, VISION_LAYER x vision_layers, PROJECT,
 * PREFIX_LAYER x llm_layers, SUFFIX_INIT, then per step SUFFIX_STEP_BEGIN,
 * SUFFIX_LAYER x llm_layers, SUFFIX_STEP_END. */
enum rtvla_stage {
    /* (DM0: dm0_infer.py:695-712 patch embedding + class token + ln_pre; :717-733 one ViT layer; :734-761 the two
     *  down-sampling convolutions, projector and token embedding; :874-951 one prefix layer; :763-872 the action expert) */
    RTVLA_STAGE_VISION_EMBED = 0,   /* pi0_infer.py:348-364 conv2d_embed_n256_1152_res               */
    RTVLA_STAGE_VISION_LAYER = 1,   /* pi0_infer.py:607-646 one SigLIP layer                         */
    RTVLA_STAGE_PROJECT = 2,        /* pi0_infer.py:753-775 + :1344 final LN, projector, prompt rows */
    RTVLA_STAGE_PREFIX_LAYER = 3,   /* pi0_infer.py:851-884 one Gemma prefix layer (KV cache fill)   */
    RTVLA_STAGE_SUFFIX_INIT = 4,    /* pi0_infer.py:1166-1171 state token (Pi0 only)                 */
    RTVLA_STAGE_SUFFIX_STEP_BEGIN = 5, /* pi0_infer.py:1173-1185 / pi05_infer.py:420-425             */
    RTVLA_STAGE_SUFFIX_LAYER = 6,   /* pi0_infer.py:1186-1223 / pi05_infer.py:427-509                */
    RTVLA_STAGE_SUFFIX_STEP_END = 7 /* pi0_infer.py:1224-1230 / pi05_infer.py:511-523 Euler update   */
};

/* Library version (no reference counterpart): raised whenever a kernel or the schedule changes, so that a
 * measurement recorded for one version is not mistaken for the current kernels. */
#define RTVLA_VERSION 9
int rtvla_version(void);

/* Create a context for one shape set.  Replaces the tensor allocation block of
 * Pi0Inference.__init__ (pi0_infer.py:1245-1317) / Pi05Inference.__init__ (pi05_infer.py:563-653):
 * validates the dimensions and lays out the workspace; allocates no device memory. */
int rtvla_create(const rtvla_dims* dims, rtvla_ctx** out);

/* Release host state (device memory belongs to the caller). */
int rtvla_destroy(rtvla_ctx* ctx);

/* Text of the last error on this context (never null). */
const char* rtvla_last_error(const rtvla_ctx* ctx);

/* Number of tensors the context knows by name, and their description: name, element size,
 * rank and shape (up to 4 dims), whether it is a weight (1) or an io buffer (0), and whether
 * it must be bound before rtvla_prepare.  Names and shapes are exactly the keys of
 * `self.weights` / `self.buffers` in the reference (pi0_infer.py:1245-1317,
 * pi05_infer.py:563-653) for the tensors that cross the boundary. */
int rtvla_tensor_count(const rtvla_ctx* ctx);
int rtvla_tensor_info(const rtvla_ctx* ctx, int index, const char** name, int32_t* elem_bytes,
                      int32_t* rank, int64_t shape[4], int32_t* is_weight, int32_t* required);

/* Bind a caller-owned device tensor by its reference name; `bytes` must equal the tensor's size.
 * Replaces `self.weights[k].copy_(v)` (pi0_infer.py:1337-1338): the library reads the caller's
 * tensor in place.  Unknown name -> RTVLA_ERR_NAME (the reference raises KeyError).
 *
 * Pi05 only, optional (required = 0): binding all three of
 *   "embedding_weight"  bf16 [rows][2048]  - the embedding table (pi05_infer.py:727-746); any row count,
 *                                            taken from `bytes`
 *   "prompt_token_ids"  int32 [prompt_len] - the caller writes the tokenised prompt here
 *   "rope_table"        bf16 [256 views + prompt_len + chunk][256] - the RoPE table of pi05_infer.py:655-667
 * before rtvla_prepare moves the per-call prompt staging of pi05_infer.py:769-785, :811-822 into the
 * forward: rows [256 views, valid_encoder_len) of encoder_x become embedding[ids] * sqrt(2048) and
 * decoder_rope_weights becomes rope_table[valid_encoder_len - 1 ...], so a call only writes the ids,
 * valid_encoder_len, the images and the noise. */
int rtvla_bind(rtvla_ctx* ctx, const char* name, void* device_ptr, size_t bytes);

/* Bytes of scratch the context needs (re-tiled weights, activations, KV cache), and binding of a
 * caller-owned, 256-byte aligned device allocation of at least that size. */
size_t rtvla_workspace_bytes(const rtvla_ctx* ctx);
int rtvla_bind_workspace(rtvla_ctx* ctx, void* device_ptr, size_t bytes);

/* Location of a named internal activation inside the workspace, for taps and for the
 * `buffers` views of the Python object: byte offset, rows, cols, leading dimension (elements),
 * element size.  Names follow the reference's buffer keys where one exists (vision_x, encoder_x,
 * encoder_K, decoder_x, ...); encoder_Vt is the transposed V cache. */
int rtvla_buffer_count(const rtvla_ctx* ctx);
int rtvla_buffer_info(const rtvla_ctx* ctx, int index, const char** name, size_t* offset,
                      int64_t* rows, int64_t* cols, int64_t* ld, int32_t* elem_bytes);

/* One-time device work after all weights are bound: re-tile weights into MFMA fragment order,
 * clear the workspace, Pi05: scale the output projection by -1/num_steps, compute the
 * time-conditioning style vectors (pi05_infer.py:669-722) and fold each (flow step, layer)'s adaptive RMS norm
 * (pi05_infer.py:127-195) into a row-scaled copy of the weights that consume it plus an fp32 per-column term
 * (num_steps x layers copies of the action expert's QKV / gate / up weights: 3.96 GB at full size).  Enqueued on `hip_stream` (a
 * hipStream_t passed as void*); the caller synchronises. */
int rtvla_prepare(rtvla_ctx* ctx, void* hip_stream);

/* Saving the re-tiled weights across processes (no reference counterpart; the reference re-reads its checkpoint and
 * has no derived layout).  After rtvla_prepare the first rtvla_tiled_bytes bytes of the workspace hold every re-tiled
 * weight and nothing else; they depend only on the weights, the model kind, the layer counts and the tile layout
 * (rtvla_tile_layout_version, raised whenever that layout changes).  A caller may save that region and, in a later
 * process with the same weights bound, copy it back to the start of the workspace and call rtvla_prepare_with_tiles
 * instead of rtvla_prepare: it does everything rtvla_prepare does except the re-tiling. */
#define RTVLA_TILE_LAYOUT_VERSION 2
size_t rtvla_tiled_bytes(const rtvla_ctx* ctx);
int rtvla_tile_layout_version(void);
int rtvla_prepare_with_tiles(rtvla_ctx* ctx, void* hip_stream);

/* Enqueue one whole forward (pi0_model pi0_infer.py:1232-1236 / pi05_model pi05_infer.py:525-528)
 * on the stream: no allocation, no synchronisation, no host read - capturable.  Inputs are read
 * from the bound io buffers; the result is left in `diffusion_noise`. */
int rtvla_forward(rtvla_ctx* ctx, void* hip_stream);

/* Enqueue a single stage (see rtvla_stage); `layer` and `step` are ignored where meaningless. */
int rtvla_forward_stage(rtvla_ctx* ctx, int stage, int layer, int step, void* hip_stream);

/* Capture rtvla_forward into a HIP graph held by the context / replay it on a stream.
 * Replaces record_infer_graph and infer_graph.replay() (pi0_infer.py:1347-1354, :1360). */
int rtvla_graph_capture(rtvla_ctx* ctx, void* hip_stream);
/* A graph records the addresses bound at capture time: rtvla_bind and rtvla_bind_workspace drop it, and
 * rtvla_graph_launch then returns RTVLA_ERR_STATE until rtvla_prepare and rtvla_graph_capture have run again. */
int rtvla_graph_launch(rtvla_ctx* ctx, void* hip_stream);

/* Number of kernels the last forward (or stage) enqueued: the kernel nodes of the captured graph. */
int rtvla_launch_count(const rtvla_ctx* ctx);

/* Measurement helper (no reference counterpart): record `stage` `iters` times back to back into a temporary HIP
 * graph, replay it on the stream between two HIP events recorded on that same stream and return the mean
 * milliseconds per run (a graph, because the forward runs as one and eager launches of microsecond kernels would
 * measure the host's launch rate).  With layer = -1 every layer of the stage runs in turn (weights cold, as inside a forward) and the
 * mean is per layer.  Synchronises the stream. */
int rtvla_time_stage(rtvla_ctx* ctx, int stage, int layer, int step, int iters, void* hip_stream, float* mean_ms);

/* Measurement helper (no reference counterpart): as rtvla_time_stage, but enqueue only the
 * `launch_index`-th kernel launch of the stage (0-based, in schedule order), so that one kernel's
 * mean duration is measured live with HIP events on the stream it is launched on.  The launch's
 * name is copied to name_out.  Returns RTVLA_ERR_ARG when the stage has fewer launches.  With layer = -1 the
 * launch is enqueued once per layer in turn (per iteration), so every launch streams weights that nothing has
 * touched since the previous pass - the condition it meets inside a forward; a fixed layer measures it cache-warm. */
int rtvla_time_launch(rtvla_ctx* ctx, int stage, int layer, int step, int launch_index, int iters, void* hip_stream,
                      float* mean_ms, char* name_out, size_t name_cap);

/* Measurement helper: time `iters` graph replays (or eager forwards when no graph is captured)
 * individually with HIP events on the stream; writes per-iteration milliseconds to ms_out[iters]. */
int rtvla_time_forward(rtvla_ctx* ctx, int iters, void* hip_stream, float* ms_out);

/* Unit-level entry points used by the per-kernel parity tests: one kernel family on caller tensors.  (No reference
 * counterpart as an ABI; they stand where the reference's per-shape wrappers stand, e.g. matmul_small_bias
 * pi0_infer.py:126-158, matmul_split_k + merge_split_k_bias_res :292-346, matmul_k_1024_1024_bias :927-937.)
 *
 * rtvla_pretile: W[K][N] bf16 row-major -> the 16-column x 32-row MFMA fragment order the action-expert kernels
 * stream (rtvla_pretile_elems elements).
 *
 * rtvla_linear: out[M][N] = x[M][K] w[K][N] + bias[N] (bias may be null), all bf16 row-major, fp32 accumulation,
 * K a multiple of 8, N a multiple of 16.  `tile` selects the kernel: 0 .. count-1 one block tile of the large-M MFMA
 * GEMM (rtvla_linear_tile_shape tells its rows x columns and fails past the last one), -1 the tile the forward's
 * cost model picks for this shape, RTVLA_TILE_SKINNY the weight-streaming kernel of the action expert (M <= 128,
 * K = 1024, 2048 or 4096).  `nsplit`: 1 = one pass with the bias epilogue; 2..8 = split-K into fp32 partials that the
 * reduce kernel sums (N <= 2048); 0 = the split the cost model picks, through the partial + reduce route the
 * residual GEMMs of the forward take.  RTVLA_ERR_LIMIT when the tile cannot take the shape (the tiles of more than
 * 128 rows consume K in steps of 128 per split).  `workspace`: rtvla_linear_workspace_bytes, 256-byte aligned. */
#define RTVLA_TILE_SKINNY (-2)
size_t rtvla_pretile_elems(int K, int N);
int rtvla_pretile(const void* w, int K, int N, void* w_tiled, void* hip_stream);
size_t rtvla_linear_workspace_bytes(int M, int K, int N, int tile, int nsplit);
int rtvla_linear(const void* x, int M, int K, const void* w, int N, const void* bias, void* out, void* workspace,
                 size_t workspace_bytes, int tile, int nsplit, void* hip_stream);
int rtvla_linear_tile_shape(int tile, int* rows, int* cols);
/* Measurement helper: as rtvla_linear without bias, then the compute launches alone (GEMM, and reduce when split)
 * `iters` times in a temporary graph on `hip_stream` (not the null stream), mean milliseconds of one. */
int rtvla_time_linear(const void* x, int M, int K, const void* w, int N, void* out, void* workspace, size_t workspace_bytes,
                      int tile, int nsplit, int iters, void* hip_stream, float* mean_ms);

/* rtvla_linear_act: the fused epilogues of the large-M GEMM that write a plain row-major output (pi0_infer.py:534-561 bias + GELU,
 * :664-691 / :727-733 GeGLU; dm0_infer.py:281-307 SwiGLU): out[M][N] =
 *     act = RTVLA_ACT_BIAS_GELU : gelu_tanh(x w + bias)            (w_up null)
 *     act = RTVLA_ACT_GEGLU     : gelu_tanh(x w) * (x w_up)
 *     act = RTVLA_ACT_SWIGLU    : silu(x w) * (x w_up)
 * Operands as for rtvla_linear; `tile` -1 (the forward's choice) or a block tile, which for the two gated forms must be 256 columns wide
 * (RTVLA_ERR_LIMIT otherwise).
 *
 * rtvla_reduce_norm: the pass that follows a split-K residual GEMM (pi0_infer.py:292-346 merge_split_k_bias_res, :366-382
 * LayerNorm, :648-663 RMSNorm): x_out[M][N] = sum of the nsplit fp32 partials [split][M][N] (nsplit 0..4, 6, 8) + bias + residual, all optional
 * but one; xn_out = its LayerNorm with norm_w / norm_b (norm = RTVLA_NORM_LAYER) or x_out * rsqrt(mean x^2 + eps) (RTVLA_NORM_RMS),
 * computed from the bf16-rounded x_out as the forward does; N a multiple of 4, at most 2048; x_out or xn_out may be null. */
enum rtvla_act { RTVLA_ACT_BIAS_GELU = 1, RTVLA_ACT_GEGLU = 2, RTVLA_ACT_SWIGLU = 3 };
enum rtvla_norm { RTVLA_NORM_NONE = 0, RTVLA_NORM_RMS = 1, RTVLA_NORM_LAYER = 2 };
size_t rtvla_linear_act_workspace_bytes(int M, int K, int N, int act, int tile);
int rtvla_linear_act(const void* x, int M, int K, const void* w, const void* w_up, int N, const void* bias, int act, void* out,
                     void* workspace, size_t workspace_bytes, int tile, void* hip_stream);
int rtvla_reduce_norm(const float* partials, int nsplit, int M, int N, const void* bias, const void* residual, int norm,
                      const void* norm_w, const void* norm_b, float eps, void* x_out, void* xn_out, void* hip_stream);

/* rtvla_attention: one attention kernel family on caller tensors, all bf16 row-major (stands where the reference calls
 * torch SDPA, pi0_infer.py:588-596, :819-824, or its own logits / softmax / P V kernels, pi0_infer.py:1041-1120,
 * pi05_infer.py:282-309, :382-416, dm0_infer.py:822-826, :913-918):
 *     q   [tokens][kv_heads][group][head_dim]      k, v   [keys][kv_heads][head_dim]      out   as q
 * out = softmax(mask(scale q k^T)) v per K/V head, each shared by `group` query heads.  `kind` fixes the kernel and with it
 * head_dim and group:
 *     RTVLA_ATTN_GEMMA_PREFIX  (256, 8)  the Gemma-2B prefix pass            RTVLA_ATTN_GEMMA_SUFFIX  (256, 8)  the action-expert pass
 *     RTVLA_ATTN_GQA128_PREFIX (128, 2)  DM0 prefix, causal                  RTVLA_ATTN_GQA128_SUFFIX (128, 2)  DM0 action expert
 *     RTVLA_ATTN_VIT64         (64, 1)   DM0 ViT (keys == tokens)            RTVLA_ATTN_SIGLIP        (72, 1)   SigLIP: tokens == keys == 256 x
 *                                                                                                                 views, kv_heads == 16, every view apart
 * Mask (the reference's predicate, pi0_infer.py:1089-1096, pi05_infer.py:294-299): key j is visible to query token t iff
 *     j < prefix_alloc ? j < valid_len : (t >= state_tokens || j == prefix_alloc)
 * and, for the causal kind, j <= t.  valid_len is read from device memory (`valid_len_dev`, int32) or is prefix_alloc when
 * that pointer is null; prefix_alloc = keys means no suffix part.  The two suffix kinds split the keys over workgroups and
 * combine fp32 partials in a second launch, as in the forward.  `workspace`: rtvla_attention_workspace_bytes, 256-byte
 * aligned (operands re-laid out in the kernels' fragment order, partial records).  RTVLA_ERR_LIMIT for shapes outside a
 * kind's range (suffix kinds: at most 128 tokens; the vision kinds take no mask; the SigLIP kernel has scale = 72^-1/2 built in
 * and refuses another). */
enum rtvla_attention_kind {
    RTVLA_ATTN_GEMMA_PREFIX = 0, RTVLA_ATTN_GEMMA_SUFFIX = 1, RTVLA_ATTN_GQA128_PREFIX = 2, RTVLA_ATTN_GQA128_SUFFIX = 3,
    RTVLA_ATTN_VIT64 = 4, RTVLA_ATTN_SIGLIP = 5
};
size_t rtvla_attention_workspace_bytes(int kind, int tokens, int keys, int kv_heads);
int rtvla_attention(int kind, const void* q, const void* k, const void* v, void* out, int tokens, int keys, int kv_heads,
                    float scale, int prefix_alloc, const int32_t* valid_len_dev, int state_tokens, void* workspace,
                    size_t workspace_bytes, void* hip_stream);

/* ---- observation pre-/post-processing either side of the forward (context-free, capturable) ----------------
 * The reference does these on the host per observation (test.py:88-201).  All pointers are device pointers. */

/* Replaces _resize_with_pad + _normalize_image (test.py:104-119) for one uint8 HWC RGB image: aspect-preserving
 * bilinear resize that matches Pillow's Image.resize(BILINEAR) bit for bit, pasted centred on a black 224x224
 * canvas, then x / 255 * 2 - 1, written as bf16 [224][224][3] - i.e. straight into one view of
 * observation_images_normalized.  `scratch` holds the 8-bit intermediate of the horizontal pass
 * (rtvla_preprocess_image_scratch bytes).  RTVLA_ERR_LIMIT for shrink factors above 31. */
size_t rtvla_preprocess_image_scratch(int height, int width);
int rtvla_preprocess_image(const void* src_u8, int height, int width, void* dst_bf16, void* scratch, size_t scratch_bytes,
                           void* hip_stream);

/* The same computation for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The 8-bit
 * intermediate lives in a device array that is part of the library's code object (RTVLA_STATIC_SCRATCH_BYTES, held by
 * every GPU the library is loaded on until the process ends); the call allocates nothing.  Frames whose intermediate
 * (height x resized width x 3 bytes, resized width <= 224) exceeds that size - more than 2160 rows at full width - are
 * rejected with RTVLA_ERR_LIMIT before anything is enqueued.  All calls on one GPU share the one array: calls that
 * overlap on the same GPU (different streams or threads) race; calls on one stream are ordered.  Nothing in the array
 * has to start at zero: the horizontal pass writes every byte the vertical pass reads.  The array's device address is
 * looked up on the first call on each GPU; that lookup is not stream work, so the first call on a GPU must not come while
 * `hip_stream` is being captured (RTVLA_ERR_STATE then: make one eager call first, later calls may be captured). */
#define RTVLA_STATIC_SCRATCH_BYTES (2160 * 224 * 3)
int rtvla_preprocess_image_static(const void* src_u8, int height, int width, void* dst_bf16, void* hip_stream);

/* Replaces _normalize_state (+ _digitize_state) (test.py:121-137): state[n] and the statistics [n_stats] are
 * zero-padded to 32 like _pad_to_dim; mode 0 (Pi0): (x - a) / (b + 1e-6) with a = mean, b = std; mode 1 (Pi05):
 * (x - a) / (b - a + 1e-6) * 2 - 1 with a = q01, b = q99, all in double as numpy computes it.  Outputs (each may
 * be null): the value as float32 -> bf16 [32] (= observation_state_normalized), as double [32], and its 256-bin
 * index np.digitize(z, linspace(-1, 1, 257)[:-1]) - 1 as int32 [32]. */
int rtvla_preprocess_state(const double* state, int n, const double* stat_a, const double* stat_b, int n_stats, int mode,
                           void* out_bf16, double* out_f64, int32_t* out_bins, void* hip_stream);

/* Replaces _unnormalize_actions and the delta-to-absolute step of infer (test.py:139-151, :196-201): bf16 actions
 * [chunk][32] -> float32 -> (mode 0) x * (b + 1e-6) + a or (mode 1) (x + 1) / 2 * (b - a + 1e-6) + a in double, first
 * action_dim columns, + ori_state, with the state taken off again on every 7th column.  out: double [chunk][action_dim]. */
int rtvla_postprocess_actions(const void* actions_bf16, int chunk, const double* stat_a, const double* stat_b, int n_stats,
                              int mode, const double* ori_state, int action_dim, double* out, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* RTVLA_H */
