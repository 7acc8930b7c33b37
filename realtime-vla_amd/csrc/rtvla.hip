// Context, workspace layout, static launch schedule and C ABI (include/rtvla.h) of the
// Pi0 / Pi05 forward pass.  The schedule restates pi0_model (/root/reference/pi0_infer.py:1232-1236)
// and pi05_model (/root/reference/pi05_infer.py:525-528) as a fixed list of kernel launches that
// touch only caller-owned memory, so the whole forward can be captured into one HIP graph.
#include "../../include/rtvla.h"
#include "kernels.h"
#include "tuning.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace {

struct Tensor {
    std::string name;
    int elem = 2;
    int rank = 0;
    int64_t shape[4] = {0, 0, 0, 0};
    bool weight = true;
    bool required = true;
    void* ptr = nullptr;
    bool bound = false;
    size_t bytes() const { size_t n = elem; for (int i = 0; i < rank; ++i) n *= (size_t)shape[i]; return n; }
};

struct WsBuf {
    std::string name;
    size_t offset = 0;
    int64_t rows = 0, cols = 0, ld = 0;
    int elem = 2;
    size_t bytes() const { return (size_t)rows * ld * elem; }
};

struct TileChoice { int tile; int nsplit; };

}  // namespace

struct rtvla_ctx {
    rtvla_dims d;
    int S_v = 0, S_e = 0, S_d = 0, keys = 0, keys_pad = 0;
    std::vector<Tensor> tensors;
    std::map<std::string, int> tindex;
    std::vector<WsBuf> bufs;
    std::map<std::string, int> bindex;
    size_t ws_bytes = 0;
    size_t act_begin = 0;          // activations start here (cleared at prepare)
    char* ws = nullptr;
    bool prepared = false;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipStream_t timing_stream = nullptr;     // the measurement helpers capture graphs, which the null stream cannot
    hipStream_t fork_stream = nullptr;       // second branch of the captured graph (default priority), see Sched::prefix_with_first_step
    std::vector<hipEvent_t> fork_events;     // one per prefix layer + fork + join
    std::string err;
    int launches = 0;              // scheduler launches enqueued so far (index space of rtvla_time_launch)
    int kernels = 0;               // kernels behind them (the key-split attention is two)
    int status = 0;

    // ---- helpers ----
    int fail(int code, const std::string& msg) { err = msg; return code; }
    Tensor& T(const char* n) { return tensors[tindex.at(n)]; }
    bf16_t* W(const char* n) { return (bf16_t*)tensors[tindex.at(n)].ptr; }
    bf16_t* W(const char* n, size_t layer_elems, int layer) { return (bf16_t*)tensors[tindex.at(n)].ptr + layer_elems * layer; }
    template <typename X = bf16_t> X* B(const char* n) { return (X*)(ws + bufs[bindex.at(n)].offset); }
    const WsBuf& BI(const char* n) const { return bufs[bindex.at(n)]; }

    void add_tensor(const char* name, bool weight, int elem, std::initializer_list<int64_t> shape) {
        Tensor t; t.name = name; t.weight = weight; t.elem = elem; t.rank = (int)shape.size();
        int i = 0; for (auto s : shape) t.shape[i++] = s;
        tindex[name] = (int)tensors.size();
        tensors.push_back(t);
    }
    void add_buf(const char* name, int64_t rows, int64_t cols, int64_t ld, int elem = 2) {
        WsBuf b; b.name = name; b.rows = rows; b.cols = cols; b.ld = ld; b.elem = elem;
        b.offset = ws_bytes;
        ws_bytes += (b.bytes() + 255) & ~(size_t)255;
        bindex[name] = (int)bufs.size();
        bufs.push_back(b);
    }
    std::map<std::string, int> tgroup;          // tile group size of each re-tiled weight
    std::map<std::string, int> twide;           // 1: wide (32-column) tiles for the large-M GEMM
    void add_tiled(const char* name, int K, int N, int layers, int G = 1, int wide = 0) {
        const int64_t e = (int64_t)(wide ? tiled_elems_wide(K, N, G) : tiled_elems(K, N, G));
        add_buf(name, layers, e, e);
        tgroup[name] = G; twide[name] = wide;
    }
    bf16_t* TW(const char* n, int layer = 0) { const WsBuf& b = BI(n); return (bf16_t*)(ws + b.offset) + (size_t)b.ld * layer; }

    int only = -1;                 // >= 0: enqueue only the launch with this index (per-kernel timing)
    std::string last_name;
    bool want(const char* what) {
        const bool yes = only < 0 || only == launches;
        if (yes) last_name = what;
        if (!yes) ++launches;
        return yes;
    }
    void note(int rc, const char* what, int nkernels = 1) {
        ++launches; kernels += nkernels;
        if (rc != 0 && status == 0) { status = RTVLA_ERR_DEVICE; err = std::string("launch failed: ") + what + " (code " + std::to_string(rc) + ")"; }
    }
};

namespace {

constexpr int PATCH_LD = 640;      // 588 patch features padded to a multiple of 64
constexpr int VHID_LD = 4352;      // 4304 padded to a multiple of 64
constexpr int XN_LD = 2048 + 64;   // row strides that are a large power of two put every row of a K stage on the same L2 channel
constexpr int EHID_LD = 16384 + 64;
constexpr int64_t ATTN_PARTIAL_FLOATS = 64 * 16 * (16 * 64 * 4 + 32);   // 64 row blocks (128 suffix rows x 8 heads) x 16 key splits of the suffix attention

// Pick block tile and split-K factor from a cost model fitted to measurements on MI355X.  One K stage of a
// workgroup takes the larger of its MFMA time (32 cycles per 32x32x16 MFMA at the ~2.05 GHz the chip sustains,
// 75 % issue efficiency) and a latency-bound load time (0.1 us + 6.7 us per MB of operands pulled by the
// workgroup); tiles of 64 rows run two workgroups per CU, which then share the MFMA pipe but overlap
// their load latency; all workgroups together cannot pull more than ~20 TB/s out of L2; every launch pays a
// fixed ramp and an epilogue that grows with the tile; split-K adds the reduce pass over the fp32 partials.
TileChoice choose_tile(int M, int ncols16, int stages, bool dual, bool splittable, const char* what, int eight = 0) {
    static const int tiles[] = {TILE_224x256, TILE_192x256, TILE_160x256, TILE_128x256, TILE_64x256, TILE_128x128, TILE_64x128};
    static const int splits[] = {1, 2, 3, 4, 6, 8};
    { TileChoice forced; if (tuning_forced_tile(what, splittable, &forced.tile, &forced.nsplit)) return forced; }
    // measured (M = 8115, K = 1024, N = 4096, bias + GELU): the eight-wave 256 x 256 tile takes 84-89 us where the best four-wave
    // tile takes 98-101 us; with 788 rows, with the gated epilogues and with fp32 split-K partials the four-wave tiles win
    // (eight: 1 = bias (+ GELU) epilogue, 2 = the ViT QKV epilogue, measured 75 us with the eight-wave 128 x 256 tile against 93 us)
    if (eight && M >= 4096 && stages <= 32 && ncols16 >= 128) return TileChoice{eight == 1 ? TILE8_256x256 : TILE8_128x256, 1};
    // shapes where timing the launch inside a layer (weights streamed from HBM) disagrees with the model below: the K = 4304
    // SigLIP down-projection gains from four K splits (more workgroups pulling the 9.9 MB of weights at once, 22.1 -> 19.3 us
    // with the reduce pass at 768 rows, 20.4 -> 14.4 us at 256 rows), the 788-row prefix QKV from 96-row tiles (22.0 -> 20.5 us), and so does
    // the SigLIP QKV GEMM at three views (768 rows as 8 x 27 = 216 workgroups, one per CU, instead of 324 on 256 CUs: 14.8 -> 12.4 us)
    struct Measured { int ncols16, stages, splittable, m_lo, m_hi, tile, nsplit; };
    static const Measured measured[] = {
        {72, 68, 1, 1, 512, TILE_64x128, 4},
        {72, 68, 1, 513, 768, TILE_128x128, 4},
        {160, 32, 0, 769, 1024, TILE_96x128, 1},
        {216, 18, 0, 673, 768, TILE_96x128, 1},
    };
    if (!dual)
        for (const Measured& e : measured)
            if (e.ncols16 == ncols16 && e.stages == stages && e.splittable == (splittable ? 1 : 0) && M >= e.m_lo && M <= e.m_hi) return TileChoice{e.tile, e.nsplit};
    double best = 1e30; TileChoice bc{TILE_128x256, 1};
    for (int tile : tiles) {
        const int bm = gemm_tile_bm(tile);
        const int bn = gemm_tile_bn(tile);
        if (dual && bn < 256) continue;
        const int bn16 = bn / 16 / (dual ? 2 : 1);
        const int mb = (M + bm - 1) / bm, nb = (ncols16 + bn16 - 1) / bn16;
        const int nt = bn / 128;
        // the 256-column tiles of 128 rows and more mix row blocks of bm and bm - 32 rows: average 32-row tiles per block
        const double mt = (bm >= 128 && bn == 256) ? (double)((M + 31) / 32) / mb : bm / 32;
        if (!dual && tile == TILE_64x256) continue;        // measured: 64x128 is never slower than 64x256 for the single-weight GEMMs
        const int occ = bm <= 64 ? 2 : 1;
        for (int sp : splits) {
            if (sp > 1 && !splittable) break;
            const int sps = (stages + sp - 1) / sp;
            if ((sp - 1) * sps >= stages) continue;
            const int tail = stages - (sp - 1) * sps;                   // stages of the last split
            if (bm > 128 && ((sps & 1) || (tail & 1))) continue;          // the large tiles consume K stages in pairs
            const int blocks = mb * nb * sp;
            const int per_cu = (blocks + 255) / 256;
            const int together = std::min(occ, per_cu);
            const int rounds = (per_cu + occ - 1) / occ;
            const double mfma_us = mt * nt * 4 * 32 / 2050.0 / 0.75;
            const double stage_bytes = (double)(bm + bn) * 64 * 2;
            const double stage_us = std::max(together * mfma_us, 0.1 + stage_bytes / 1.5e5);
            double t = std::max(rounds * sps * stage_us, blocks * (double)sps * stage_bytes / 20.0e6);
            t += 3.5 + 2.0 + 1.2 * mt * (splittable ? 1.5 : 1.0);
            if (splittable) t += 3.5 + (double)sp * M * ncols16 * 16 * 4.0 / 4.0e6;    // the reduce pass reads the partials at ~4 TB/s
            if (t < best) { best = t; bc = TileChoice{tile, sp}; }
        }
    }
    tuning_report_tile(what, M, ncols16 * 16, stages, gemm_tile_bm(bc.tile), gemm_tile_bn(bc.tile), bc.nsplit, best);
    return bc;
}

int build_tables(rtvla_ctx* c) {
    const rtvla_dims& d = c->d;
    const int64_t V = d.vision_layers, L = d.llm_layers, v = d.num_views, ch = d.chunk_size;
    const bool pi05 = d.model == RTVLA_PI05;
    // ---- tensors that cross the boundary (reference names and shapes) ----
    c->add_tensor("vision_patch_embedding_w", true, 2, {14, 14, 3, 1152});
    c->add_tensor("vision_patch_embedding_b", true, 2, {1152});
    c->add_tensor("vision_position_embedding", true, 2, {256, 1152});
    c->add_tensor("vision_attn_qkv_w", true, 2, {V, 1152, 3456});
    c->add_tensor("vision_attn_qkv_b", true, 2, {V, 3456});
    c->add_tensor("vision_attn_o_w", true, 2, {V, 1152, 1152});
    c->add_tensor("vision_attn_o_b", true, 2, {V, 1152});
    c->add_tensor("vision_ffn_up_w", true, 2, {V, 1152, 4304});
    c->add_tensor("vision_ffn_up_b", true, 2, {V, 4304});
    c->add_tensor("vision_ffn_down_w", true, 2, {V, 4304, 1152});
    c->add_tensor("vision_ffn_down_b", true, 2, {V, 1152});
    c->add_tensor("vision_pre_attn_norm_w", true, 2, {V, 1152});
    c->add_tensor("vision_pre_attn_norm_b", true, 2, {V, 1152});
    c->add_tensor("vision_pre_ffn_norm_w", true, 2, {V, 1152});
    c->add_tensor("vision_pre_ffn_norm_b", true, 2, {V, 1152});
    c->add_tensor("vision_final_norm_w", true, 2, {1152});
    c->add_tensor("vision_final_norm_b", true, 2, {1152});
    c->add_tensor("encoder_multi_modal_projector_w", true, 2, {1152, 2048});
    c->add_tensor("encoder_multi_modal_projector_b", true, 2, {2048});
    c->add_tensor("encoder_attn_qkv_w", true, 2, {L, 2048, 2560});
    c->add_tensor("encoder_attn_o_w", true, 2, {L, 2048, 2048});
    c->add_tensor("encoder_ffn_gate_w", true, 2, {L, 2048, 16384});
    c->add_tensor("encoder_ffn_up_w", true, 2, {L, 2048, 16384});
    c->add_tensor("encoder_ffn_down_w", true, 2, {L, 16384, 2048});
    if (!pi05) {
        c->add_tensor("decoder_state_in_proj_w", true, 2, {32, 1024});
        c->add_tensor("decoder_state_in_proj_b", true, 2, {1024});
        c->add_tensor("decoder_action_fused_in_proj_w", true, 2, {32, 1024});
        c->add_tensor("decoder_action_fused_time_biases", true, 2, {10, 1024});
        c->add_tensor("decoder_action_mlp_w", true, 2, {1024, 1024});
        c->add_tensor("decoder_action_mlp_b", true, 2, {1024});
    } else {
        c->add_tensor("decoder_time_embeds", true, 2, {10, 1024});
        c->add_tensor("decoder_time_mlp_in_w", true, 2, {1024, 1024});
        c->add_tensor("decoder_time_mlp_in_b", true, 2, {1024});
        c->add_tensor("decoder_time_mlp_out_w", true, 2, {1024, 1024});
        c->add_tensor("decoder_time_mlp_out_b", true, 2, {1024});
        c->add_tensor("decoder_action_in_proj_w", true, 2, {32, 1024});
        c->add_tensor("decoder_action_in_proj_b", true, 2, {1024});
        c->add_tensor("decoder_pre_attn_norm_mod_w", true, 2, {L, 1024, 3072});
        c->add_tensor("decoder_pre_attn_norm_mod_b", true, 2, {L, 3072});
        c->add_tensor("decoder_pre_ffn_norm_mod_w", true, 2, {L, 1024, 3072});
        c->add_tensor("decoder_pre_ffn_norm_mod_b", true, 2, {L, 3072});
    }
    c->add_tensor("decoder_attn_qkv_w", true, 2, {L, 1024, 2560});
    c->add_tensor("decoder_attn_o_w", true, 2, {L, 2048, 1024});
    c->add_tensor("decoder_ffn_gate_w", true, 2, {L, 1024, 4096});
    c->add_tensor("decoder_ffn_up_w", true, 2, {L, 1024, 4096});
    c->add_tensor("decoder_ffn_down_w", true, 2, {L, 4096, 1024});
    if (!pi05) {
        c->add_tensor("decoder_action_fused_out_proj_w", true, 2, {1024, 32});
        c->add_tensor("decoder_action_fused_out_proj_b", true, 2, {32});
        c->add_tensor("language_embeds", true, 2, {d.prompt_len, 2048});
    } else {
        c->add_tensor("decoder_action_out_proj_w", true, 2, {1024, 32});
        c->add_tensor("decoder_action_out_proj_b", true, 2, {32});
        c->add_tensor("decoder_final_norm_mod_w", true, 2, {1024, 3072});
        c->add_tensor("decoder_final_norm_mod_b", true, 2, {3072});
    }
    c->add_tensor("observation_images_normalized", false, 2, {v, 224, 224, 3});
    if (!pi05) c->add_tensor("observation_state_normalized", false, 2, {32});
    c->add_tensor("diffusion_noise", false, 2, {ch, 32});
    c->add_tensor("encoder_rope_weights", false, 2, {c->S_e, 256});
    c->add_tensor("decoder_rope_weights", false, 2, {c->S_d, 256});
    if (pi05) {
        c->add_tensor("valid_encoder_len", false, 4, {1});
        // optional device-side prompt staging: token ids -> embedding rows and decoder RoPE rows inside the graph.
        // embedding_weight may have any number of rows (its row count is taken from the bound size).
        c->add_tensor("embedding_weight", true, 2, {257152, 2048}); c->tensors.back().required = false;
        c->add_tensor("prompt_token_ids", false, 4, {d.prompt_len}); c->tensors.back().required = false;
        c->add_tensor("rope_table", false, 2, {c->S_e + ch, 256}); c->tensors.back().required = false;
    }

    // ---- workspace: re-tiled weights first, then activations ----
    c->add_tiled("t_vision_patch_embedding_w", 588, 1152, 1, 8, 1);
    c->add_tiled("t_vision_attn_qkv_w", 1152, 3456, V, 8, 1);
    c->add_tiled("t_vision_attn_o_w", 1152, 1152, V, 8, 1);
    c->add_tiled("t_vision_ffn_up_w", 1152, 4304, V, 8, 1);
    c->add_tiled("t_vision_ffn_down_w", 4304, 1152, V, 8, 1);
    c->add_tiled("t_encoder_multi_modal_projector_w", 1152, 2048, 1, 8, 1);
    c->add_tiled("t_encoder_attn_qkv_w", 2048, 2560, L, 8, 1);
    c->add_tiled("t_encoder_attn_o_w", 2048, 2048, L, 8, 1);
    c->add_tiled("t_encoder_ffn_gate_w", 2048, 16384, L, 4, 1);
    c->add_tiled("t_encoder_ffn_up_w", 2048, 16384, L, 4, 1);
    c->add_tiled("t_encoder_ffn_down_w", 16384, 2048, L, 8, 1);
    c->add_tiled("t_decoder_attn_qkv_w", 1024, 2560, L);
    c->add_tiled("t_decoder_attn_o_w", 2048, 1024, L);
    c->add_tiled("t_decoder_ffn_gate_w", 1024, 4096, L);
    c->add_tiled("t_decoder_ffn_up_w", 1024, 4096, L);
    c->add_tiled("t_decoder_ffn_down_w", 4096, 1024, L);
    c->add_tiled("t_decoder_out_proj_w", 1024, 32, 1);
    if (!pi05) {
        c->add_tiled("t_decoder_action_mlp_w", 1024, 1024, 1);
    } else {
        c->add_tiled("t_decoder_time_mlp_in_w", 1024, 1024, 1);
        c->add_tiled("t_decoder_time_mlp_out_w", 1024, 1024, 1);
        c->add_tiled("t_decoder_pre_attn_norm_mod_w", 1024, 3072, L);
        c->add_tiled("t_decoder_pre_ffn_norm_mod_w", 1024, 3072, L);
        c->add_tiled("t_decoder_final_norm_mod_w", 1024, 3072, 1);
        // The adaptive RMS norm folded into its consumers: with y = x f (1 + scale) + shift (f the row's RMS factor),
        // y W = f (x diag(1 + scale) W) + shift W.  Per (flow step, layer) the row-scaled weights are tiled once at prepare and
        // shift W becomes an fp32 per-column term, so that the action-expert kernels run the same post-scaled product as Pi0's.
        c->add_tiled("t_decoder_attn_qkv_ada", 1024, 2560, d.num_steps * L);
        c->add_tiled("t_decoder_ffn_gate_ada", 1024, 4096, d.num_steps * L);
        c->add_tiled("t_decoder_ffn_up_ada", 1024, 4096, d.num_steps * L);
        c->add_buf("decoder_out_proj_w_scaled", 1024, 32, 32);
        c->add_buf("decoder_out_proj_b_scaled", 1, 32, 32);
    }
    c->act_begin = c->ws_bytes;
    const int64_t S_v = c->S_v, S_e = c->S_e, S_d = c->S_d;
    c->add_buf("vision_patches", S_v, PATCH_LD, PATCH_LD);
    c->add_buf("vision_x", S_v, 1152, 1152);
    c->add_buf("vision_x_norm", S_v, 1152, 1152);
    c->add_buf("vision_Q", v * 16, 256 * 96, 256 * 96);          // fragment-tiled [256][96] per (view, head)
    c->add_buf("vision_K", v * 16, 256 * 96, 256 * 96);
    c->add_buf("vision_Vt", v * 16, 80 * 256, 80 * 256);         // tiled V^T [80][256] per (view, head)
    c->add_buf("vision_attn", S_v, 1152, 1152);
    c->add_buf("vision_hidden", S_v, 4304, VHID_LD);
    c->add_buf("encoder_x", S_e, 2048, 2048);
    c->add_buf("encoder_x_norm", S_e, 2048, XN_LD);
    c->add_buf("encoder_Q", ((8 * S_e + 31) / 32) * 32, 256, 256);   // fragment-tiled, rows = token*8 + head
    c->add_buf("encoder_attn", S_e, 2048, 2048);
    c->add_buf("encoder_hidden", S_e, 16384, EHID_LD);
    c->add_buf("encoder_K", L * c->keys_pad, 256, 256);           // fragment-tiled [keys_pad][256] per layer
    c->add_buf("encoder_Vt", L * 256, c->keys_pad, c->keys_pad);  // tiled V^T [256][keys_pad] per layer
    const int64_t Rd = ((S_d + 63) / 64) * 64;                    // suffix rows padded to the 64-row blocks of the action-expert kernels
    c->add_buf("decoder_x", Rd, 1024, 1024);                      // the decoder_* activations are fragment-tiled
    c->add_buf("decoder_x_buf", Rd, 1024, 1024);
    c->add_buf("decoder_q_buf", 8 * Rd, 256, 256);
    c->add_buf("decoder_attn", Rd, 2048, 2048);
    c->add_buf("decoder_hidden", Rd, 4096, 4096);
    if (pi05) {
        c->add_buf("decoder_time_emb", 64, 1024, 1024);           // fragment-tiled, one row per step
        c->add_buf("decoder_style_attn", d.num_steps, L * 3072, L * 3072);
        c->add_buf("decoder_style_ffn", d.num_steps, L * 3072, L * 3072);
        c->add_buf("decoder_style_final", d.num_steps, 3072, 3072);
        c->add_buf("decoder_ada_bias_qkv", d.num_steps * L, 2560, 2560, 4);      // fp32: shift W per (step, layer)
        c->add_buf("decoder_ada_bias_gate", d.num_steps * L, 4096, 4096, 4);
        c->add_buf("decoder_ada_bias_up", d.num_steps * L, 4096, 4096, 4);
    }
    const int64_t pmax = std::max(S_v * 1152, S_e * 2048) * 8;
    c->add_buf("splitk_partial", 1, pmax, pmax, 4);
    c->add_buf("attn_partial", 1, ATTN_PARTIAL_FLOATS, ATTN_PARTIAL_FLOATS, 4);
    return 0;
}

// DM0 (/root/reference/dm0_infer.py:965-1076): tensors under the reference's names, then the workspace.
constexpr int DM0_SEQ = 2705;          // 52 x 52 patches + class token per image
constexpr int DM0_SEQ_PAD = 2720;      // rows per image in every ViT buffer: whole 32-row GEMM tiles and 32-key attention blocks
constexpr int DM0_TOK = 169;           // tokens per image after the two stride-2 convolutions

int build_tables_dm0(rtvla_ctx* c) {
    const rtvla_dims& d = c->d;
    const int64_t V = d.vision_layers, L = d.llm_layers, n = d.num_views, P = c->S_e, ch = d.chunk_size;
    c->add_tensor("decoder_attn_qkv_w", true, 2, {L, 1024, 4096});
    c->add_tensor("decoder_q_norm_w", true, 2, {L, 128});
    c->add_tensor("decoder_k_norm_w", true, 2, {L, 128});
    c->add_tensor("decoder_attn_o_w", true, 2, {L, 2048, 1024});
    c->add_tensor("decoder_ffn_gate_w", true, 2, {L, 1024, 1536});
    c->add_tensor("decoder_ffn_up_w", true, 2, {L, 1024, 1536});
    c->add_tensor("decoder_ffn_down_w", true, 2, {L, 1536, 1024});
    c->add_tensor("decoder_action_fused_in_proj_w", true, 2, {32, 1024});
    c->add_tensor("decoder_action_fused_time_biases", true, 2, {10, 1024});
    c->add_tensor("decoder_action_mlp_w", true, 2, {1024, 1024});
    c->add_tensor("decoder_action_mlp_b", true, 2, {1024});
    c->add_tensor("decoder_action_fused_out_proj_w", true, 2, {1024, 32});
    c->add_tensor("decoder_action_fused_out_proj_b", true, 2, {32});
    c->add_tensor("llm_attn_qkv_w", true, 2, {L, 2048, 4096});
    c->add_tensor("llm_q_norm_w", true, 2, {L, 128});
    c->add_tensor("llm_k_norm_w", true, 2, {L, 128});
    c->add_tensor("llm_attn_o_w", true, 2, {L, 2048, 2048});
    c->add_tensor("llm_ffn_gate_w", true, 2, {L, 2048, 6144});
    c->add_tensor("llm_ffn_up_w", true, 2, {L, 2048, 6144});
    c->add_tensor("llm_ffn_down_w", true, 2, {L, 6144, 2048});
    c->add_tensor("vision_conv1_w_t", true, 2, {588, 1024});
    c->add_tensor("vision_class_embedding", true, 2, {1024});
    c->add_tensor("vision_pos_emb", true, 2, {DM0_SEQ, 1024});
    c->add_tensor("vision_ln_pre_w", true, 2, {1024});
    c->add_tensor("vision_ln_pre_b", true, 2, {1024});
    c->add_tensor("vision_fused_qkv_w", true, 2, {V, 1024, 3072});
    c->add_tensor("vision_fused_qkv_b", true, 4, {V, 3072});          // fp32 (weights of 4-byte elements are fp32)
    c->add_tensor("vision_qkv_col_sum", true, 4, {V, 3072});          // bound for the reference's key set; the LayerNorm is applied to the rows instead
    c->add_tensor("vision_out_proj_w", true, 2, {V, 1024, 1024});
    c->add_tensor("vision_out_proj_b", true, 2, {V, 1024});
    c->add_tensor("vision_fused_fc_w", true, 2, {V, 1024, 4096});
    c->add_tensor("vision_fused_fc_b", true, 4, {V, 4096});
    c->add_tensor("vision_fc_col_sum", true, 4, {V, 4096});
    c->add_tensor("vision_proj_w", true, 2, {V, 4096, 1024});
    c->add_tensor("vision_proj_b", true, 2, {V, 1024});
    c->add_tensor("vision_ds1_w", true, 2, {3, 3, 1024, 2048});
    c->add_tensor("vision_ds1_b", true, 2, {2048});
    c->add_tensor("vision_ds2_w", true, 2, {3, 3, 2048, 4096});
    c->add_tensor("vision_ds2_b", true, 2, {4096});
    c->add_tensor("vision_projector_w_t", true, 2, {4096, 2048});
    c->add_tensor("vision_embed_tokens_w", true, 2, {152701, 2048});   // any row count, taken from the bound size
    c->add_tensor("images", false, 2, {n, 3, 728, 728});
    c->add_tensor("input_ids", false, 4, {d.prompt_len});              // int32
    c->add_tensor("diffusion_noise", false, 2, {ch, 32});
    c->add_tensor("prefix_rope_weights", false, 2, {P, 128});
    c->add_tensor("decoder_rope_weights", false, 2, {ch, 128});
    c->add_tensor("vision_rope", false, 2, {DM0_SEQ, 64});             // (cos, sin) per rotation pair of the 2-D rotary embedding

    // ---- workspace: re-tiled weights first, then activations ----
    c->add_tiled("t_vision_conv1_w_t", 588, 1024, 1, 8, 1);
    c->add_tiled("t_vision_fused_qkv_w", 1024, 3072, V, 8, 1);
    c->add_tiled("t_vision_out_proj_w", 1024, 1024, V, 8, 1);
    c->add_tiled("t_vision_fused_fc_w", 1024, 4096, V, 8, 1);
    c->add_tiled("t_vision_proj_w", 4096, 1024, V, 8, 1);
    c->add_tiled("t_vision_ds1_w", 9216, 2048, 1, 8, 1);
    c->add_tiled("t_vision_ds2_w", 18432, 4096, 1, 8, 1);
    c->add_tiled("t_vision_projector_w_t", 4096, 2048, 1, 8, 1);
    c->add_tiled("t_llm_attn_qkv_w", 2048, 4096, L, 8, 1);
    c->add_tiled("t_llm_attn_o_w", 2048, 2048, L, 8, 1);
    c->add_tiled("t_llm_ffn_gate_w", 2048, 6144, L, 4, 1);
    c->add_tiled("t_llm_ffn_up_w", 2048, 6144, L, 4, 1);
    c->add_tiled("t_llm_ffn_down_w", 6144, 2048, L, 8, 1);
    c->add_tiled("t_decoder_attn_qkv_w", 1024, 4096, L);
    c->add_tiled("t_decoder_attn_o_w", 2048, 1024, L);
    c->add_tiled("t_decoder_ffn_gate_w", 1024, 1536, L);
    c->add_tiled("t_decoder_ffn_up_w", 1024, 1536, L);
    c->add_tiled("t_decoder_ffn_down_w", 2048, 1024, L);              // K = 1536 zero-padded to the 2048 the streaming kernel takes
    c->add_tiled("t_decoder_action_mlp_w", 1024, 1024, 1);
    c->add_tiled("t_decoder_out_proj_w", 1024, 32, 1);
    c->act_begin = c->ws_bytes;
    const int64_t M = n * DM0_SEQ_PAD;                                       // every image owns 2720 rows of the row-major ViT buffers
    c->add_buf("const_ones", 1, 1024, 1024);
    c->add_buf("const_zeros", 1, 6144, 6144);
    c->add_buf("vision_patches", n * 2704, PATCH_LD, PATCH_LD);
    c->add_buf("vision_conv1_buf", n * 2704, 1024, 1024);
    c->add_buf("vision_x_2d", M, 1024, 1024);
    c->add_buf("vision_x_norm", M, 1024, 1024);
    c->add_buf("vision_Q", n * 16, DM0_SEQ_PAD * 64, DM0_SEQ_PAD * 64);    // fragment-tiled [2720][64] per (image, head)
    c->add_buf("vision_K", n * 16, DM0_SEQ_PAD * 64, DM0_SEQ_PAD * 64);
    c->add_buf("vision_Vt", n * 16, 64 * DM0_SEQ_PAD, 64 * DM0_SEQ_PAD);   // tiled V^T [64][2720]
    c->add_buf("vision_attn", M, 1024, 1024);
    c->add_buf("vision_fc", M, 4096, 4096);
    c->add_buf("vision_col1", n * 676, 9216, 9216);
    c->add_buf("vision_mm1", n * 676, 2048, 2048);
    c->add_buf("vision_col2", n * DM0_TOK, 18432, 18432);
    c->add_buf("vision_mm2", n * DM0_TOK, 4096, 4096);
    c->add_buf("prefix_x", P, 2048, 2048);
    c->add_buf("prefix_qkv", P, 4096, 4096);
    c->add_buf("prefix_Q", 8, ((2 * P + 31) / 32) * 32 * 128, ((2 * P + 31) / 32) * 32 * 128);     // per K/V head: fragment-tiled [token*2 + head][128]
    c->add_buf("prefix_attn", P, 2048, 2048);
    c->add_buf("prefix_hidden", P, 6144, 6144);
    c->add_buf("prefix_norm_factor", 1, P, P, 4);
    c->add_buf("kv_K", L * 8, c->keys_pad * 128, c->keys_pad * 128);       // per (layer, K/V head): fragment-tiled [keys_pad][128]
    c->add_buf("kv_Vt", L * 8, 128 * c->keys_pad, 128 * c->keys_pad);      // tiled V^T [128][keys_pad]
    c->add_buf("decoder_x", 64, 1024, 1024);                               // the decoder_* activations are fragment-tiled
    c->add_buf("decoder_x_buf", 64, 1024, 1024);
    c->add_buf("decoder_qkv", 64, 4096, 4096);                             // row-major
    c->add_buf("decoder_Q", 8, 128 * 128, 128 * 128);
    c->add_buf("decoder_attn", 64, 2048, 2048);
    c->add_buf("decoder_hidden", 64, 2048, 2048);                          // 1536 columns used, the rest stays zero
    const int64_t pmax = std::max(M * 1024, P * 2048) * 8;
    c->add_buf("splitk_partial", 1, pmax, pmax, 4);
    c->add_buf("attn_partial", 1, ATTN_PARTIAL_FLOATS, ATTN_PARTIAL_FLOATS, 4);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// schedule
// ------------------------------------------------------------------------------------------------
struct Sched {
    rtvla_ctx* c;
    hipStream_t s;
    const rtvla_dims& d;
    bool pi05;
    Sched(rtvla_ctx* c_, hipStream_t s_) : c(c_), s(s_), d(c_->d), pi05(c_->d.model == RTVLA_PI05) {}

    void gemm(const bf16_t* A, int lda, int a_rows, int M, const bf16_t* B0, const bf16_t* B1, int K, int N, int epi, GemmP extra, const char* what) {
        const int bgroup = (epi == EPI_GEGLU || epi == EPI_SWIGLU) ? 4 : 8;
        GemmP p = extra;
        p.A = A; p.lda = lda; p.a_rows = a_rows; p.M = M; p.B0 = B0; p.B1 = B1;
        p.N16 = n16_tiles(N); p.K32p = k32_padded(K); p.bgroup = bgroup;
        const TileChoice tc = choose_tile(M, p.N16, p.K32p / 2, epi == EPI_GEGLU || epi == EPI_SWIGLU, epi == EPI_PARTIAL, what, (epi == EPI_BIAS || epi == EPI_BIAS_GELU) ? 1 : epi == EPI_VIT_QKV_ROPE ? 2 : 0);
        p.nsplit = tc.nsplit;
        if (epi == EPI_PARTIAL) {
            p.partial = c->B<float>("splitk_partial"); p.ldp = N; p.pstride = (size_t)M * N;
        }
        last_split = tc.nsplit;
        if (c->want(what)) {
            // the name a measurement reports carries the kernel variant: block tile and split-K factor
            c->last_name = std::string(what) + " [" + std::to_string(gemm_tile_bm(tc.tile)) + "x" + std::to_string(gemm_tile_bn(tc.tile)) +
                           (gemm_tile_eight_waves(tc.tile) ? " 8 waves" : "") + " split " + std::to_string(tc.nsplit) + "]";
            c->note(launch_gemm(p, epi, tc.tile, s), what);
        }
    }
    int last_split = 1;

    void reduce(int M, int N, const bf16_t* bias, const bf16_t* res, int ldr, bf16_t* x, int ldx, bf16_t* xn, int ldxn,
                int norm, const bf16_t* nw, const bf16_t* nb, float eps, int nsplit, const char* what, float* factor = nullptr) {
        ReduceP p{};
        p.factor = factor;
        p.partial = c->B<float>("splitk_partial"); p.pstride = (size_t)M * N; p.ldp = N; p.nsplit = nsplit;
        p.bias = bias; p.res = res; p.ldr = ldr; p.x = x; p.ldx = ldx; p.xn = xn; p.ldxn = ldxn;
        p.M = M; p.N = N; p.norm = norm; p.nw = nw; p.nb = nb; p.eps = eps;
        if (c->want(what)) c->note(launch_reduce(p, s), what);
    }

    void vision_embed() {
        const int S_v = c->S_v;
        if (c->want("im2col")) { launch_im2col(c->W("observation_images_normalized"), c->B("vision_patches"), PATCH_LD, d.num_views, s); c->note(0, "im2col"); }
        GemmP e{}; e.out = c->B("vision_x"); e.ldo = 1152; e.bias = c->W("vision_patch_embedding_b");
        e.res = c->W("vision_position_embedding"); e.ldr = 1152; e.res_mod = 256;
        gemm(c->B("vision_patches"), PATCH_LD, S_v, S_v, c->TW("t_vision_patch_embedding_w"), nullptr, 588, 1152, EPI_PATCH, e, "patch embed");
        reduce(S_v, 1152, nullptr, c->B("vision_x"), 1152, nullptr, 0, c->B("vision_x_norm"), 1152, NORM_LAYER,
               c->W("vision_pre_attn_norm_w"), c->W("vision_pre_attn_norm_b"), 1e-5f, 0, "vision LN0");
    }

    void vision_layer(int i) {
        const int S_v = c->S_v, V = d.vision_layers;
        GemmP e{}; e.bias = c->W("vision_attn_qkv_b", 3456, i); e.q = c->B("vision_Q"); e.k = c->B("vision_K"); e.vt = c->B("vision_Vt");
        gemm(c->B("vision_x_norm"), 1152, S_v, S_v, c->TW("t_vision_attn_qkv_w", i), nullptr, 1152, 3456, EPI_VIS_QKV, e, "vision qkv");
        if (c->want("vision attn")) { launch_vision_attention(c->B("vision_Q"), c->B("vision_K"), c->B("vision_Vt"), c->B("vision_attn"), d.num_views, s); c->note(0, "vision attn"); }
        gemm(c->B("vision_attn"), 1152, S_v, S_v, c->TW("t_vision_attn_o_w", i), nullptr, 1152, 1152, EPI_PARTIAL, GemmP{}, "vision o");
        reduce(S_v, 1152, c->W("vision_attn_o_b", 1152, i), c->B("vision_x"), 1152, c->B("vision_x"), 1152, c->B("vision_x_norm"), 1152,
               NORM_LAYER, c->W("vision_pre_ffn_norm_w", 1152, i), c->W("vision_pre_ffn_norm_b", 1152, i), 1e-5f, last_split, "vision o reduce");
        GemmP u{}; u.out = c->B("vision_hidden"); u.ldo = VHID_LD; u.bias = c->W("vision_ffn_up_b", 4304, i);
        gemm(c->B("vision_x_norm"), 1152, S_v, S_v, c->TW("t_vision_ffn_up_w", i), nullptr, 1152, 4304, EPI_BIAS_GELU, u, "vision up");
        gemm(c->B("vision_hidden"), VHID_LD, S_v, S_v, c->TW("t_vision_ffn_down_w", i), nullptr, 4304, 1152, EPI_PARTIAL, GemmP{}, "vision down");
        const bool last = i == V - 1;
        const bf16_t* nw = last ? c->W("vision_final_norm_w") : c->W("vision_pre_attn_norm_w", 1152, i + 1);
        const bf16_t* nb = last ? c->W("vision_final_norm_b") : c->W("vision_pre_attn_norm_b", 1152, i + 1);
        reduce(S_v, 1152, c->W("vision_ffn_down_b", 1152, i), c->B("vision_x"), 1152, c->B("vision_x"), 1152, c->B("vision_x_norm"), 1152,
               NORM_LAYER, nw, nb, 1e-5f, last_split, "vision down reduce");
    }

    void project() {
        const int S_v = c->S_v, S_e = c->S_e;
        GemmP e{}; e.out = c->B("encoder_x"); e.ldo = 2048; e.bias = c->W("encoder_multi_modal_projector_b");
        gemm(c->B("vision_x_norm"), 1152, S_v, S_v, c->TW("t_encoder_multi_modal_projector_w"), nullptr, 1152, 2048, EPI_BIAS, e, "projector");
        if (pi05 && d.prompt_len > 0 && c->T("embedding_weight").bound && c->T("prompt_token_ids").bound && c->T("rope_table").bound) {
            if (c->want("prompt stage")) {
                launch_prompt_stage(c->W("embedding_weight"), (int)c->T("embedding_weight").shape[0], (const int*)c->T("prompt_token_ids").ptr, valid_len(),
                                    c->B("encoder_x") + (size_t)S_v * 2048, d.prompt_len, S_v, 45.254833995939045f /* sqrt(2048) */,
                                    c->W("rope_table"), S_e + d.chunk_size, c->W("decoder_rope_weights"), d.chunk_size, s);
                c->note(0, "prompt stage");
            }
        }
        if (!pi05 && d.prompt_len > 0) {
            if (c->want("prompt rows")) { launch_copy_rows(c->W("language_embeds"), 2048, c->B("encoder_x") + (size_t)S_v * 2048, 2048, d.prompt_len, 2048, s); c->note(0, "prompt rows"); }
        }
        reduce(S_e, 2048, nullptr, c->B("encoder_x"), 2048, nullptr, 0, c->B("encoder_x_norm"), XN_LD, NORM_RMS, nullptr, nullptr, 1e-6f, 0, "prefix rms0");
    }

    bf16_t* Kc(int i) { return c->B("encoder_K") + (size_t)i * c->keys_pad * 256; }
    bf16_t* Vt(int i) { return c->B("encoder_Vt") + (size_t)i * 256 * c->keys_pad; }
    const int* valid_len() { return pi05 ? (const int*)c->tensors[c->tindex.at("valid_encoder_len")].ptr : nullptr; }

    void prefix_layer(int i) { prefix_layer_kv(i); prefix_layer_rest(i); }

    // the part of a prefix layer that fills its K / V cache rows: all that the action expert's layer i needs of the prefix
    void prefix_layer_kv(int i) {
        const int S_e = c->S_e;
        GemmP e{}; e.rope = c->W("encoder_rope_weights"); e.q = c->B("encoder_Q"); e.k = Kc(i); e.vt = Vt(i); e.ldvt = c->keys_pad;
        gemm(c->B("encoder_x_norm"), XN_LD, S_e, S_e, c->TW("t_encoder_attn_qkv_w", i), nullptr, 2048, 2560, EPI_QKV_ROPE, e, "prefix qkv");
    }

    void prefix_layer_rest(int i) {
        const int S_e = c->S_e, L = d.llm_layers;
        if (i == L - 1) return;                      // the last layer only fills the KV cache
        AttnP a{};
        a.q = c->B("encoder_Q"); a.k = Kc(i); a.vt = Vt(i); a.ldvt = c->keys_pad;
        a.out = c->B("encoder_attn"); a.group = 8; a.ld_tok = 2048; a.out_tiled = 0; a.rows = 8 * S_e; a.keys = S_e; a.scale = 0.0625f;
        a.prefix_alloc = S_e; a.valid_len = valid_len(); a.state_rows = 0;
        if (c->want("prefix attn")) c->note(launch_mqa_attention(a, ATTN_PREFIX, s), "prefix attn");
        gemm(c->B("encoder_attn"), 2048, S_e, S_e, c->TW("t_encoder_attn_o_w", i), nullptr, 2048, 2048, EPI_PARTIAL, GemmP{}, "prefix o");
        reduce(S_e, 2048, nullptr, c->B("encoder_x"), 2048, c->B("encoder_x"), 2048, c->B("encoder_x_norm"), XN_LD, NORM_RMS, nullptr, nullptr, 1e-6f, last_split, "prefix o reduce");
        GemmP g{}; g.out = c->B("encoder_hidden"); g.ldo = EHID_LD;
        gemm(c->B("encoder_x_norm"), XN_LD, S_e, S_e, c->TW("t_encoder_ffn_gate_w", i), c->TW("t_encoder_ffn_up_w", i), 2048, 16384, EPI_GEGLU, g, "prefix geglu");
        gemm(c->B("encoder_hidden"), EHID_LD, S_e, S_e, c->TW("t_encoder_ffn_down_w", i), nullptr, 16384, 2048, EPI_PARTIAL, GemmP{}, "prefix down");
        reduce(S_e, 2048, nullptr, c->B("encoder_x"), 2048, c->B("encoder_x"), 2048, c->B("encoder_x_norm"), XN_LD, NORM_RMS, nullptr, nullptr, 1e-6f, last_split, "prefix down reduce");
    }

    // action-expert activations live in the fragment-tiled layout (64 rows x cols)
    void skinny(const bf16_t* A, int lda, int M, const bf16_t* B0, const bf16_t* B1, int K, int N, int norm, const bf16_t* style,
                int epi, SkinnyP extra, const char* what) {
        SkinnyP p = extra;
        p.A = A; p.lda = lda; p.M = M; p.B0 = B0; p.B1 = B1; p.K = K; p.N16 = n16_tiles(N); p.K32p = k32_padded(K);
        p.norm = norm; p.style = style; p.eps = 1e-6f;
        if (c->want(what)) c->note(launch_skinny(p, epi, s), what);
    }
    static SkinnyP tiled_io(int a_row0 = 0, int out_row0 = 0) {
        SkinnyP p{}; p.a_tiled = 1; p.a_row0 = a_row0; p.out_tiled = 1; p.out_row0 = out_row0; return p;
    }

    void suffix_init() {}

    void suffix_step_begin(int t) {
        const int ch = d.chunk_size;
        if (!pi05) {
            // state token -> row 0 of the residual stream (re-projected every step: the stream is updated in place) and the fused
            // action/time input projection + SiLU -> decoder_x_buf, as ONE launch: the two are independent
            if (c->want("state + action in")) {
                SmallLinearJob st{c->W("observation_state_normalized"), 32, c->W("decoder_state_in_proj_w"), c->W("decoder_state_in_proj_b"),
                                  c->B("decoder_x"), 1024, 1, 32, 1024, 0, 1, 0};
                SmallLinearJob ai{c->W("diffusion_noise"), 32, c->W("decoder_action_fused_in_proj_w"), c->W("decoder_action_fused_time_biases", 1024, t % 10),
                                  c->B("decoder_x_buf"), 1024, ch, 32, 1024, 1, 1, 0};
                launch_small_linear2(st, ai, s);
                c->note(0, "state + action in");
            }
            SkinnyP e = tiled_io(0, 1); e.out = c->B("decoder_x"); e.ldo = 1024; e.bias = c->W("decoder_action_mlp_b");
            skinny(c->B("decoder_x_buf"), 1024, ch, c->TW("t_decoder_action_mlp_w"), nullptr, 1024, 1024, SN_NONE, nullptr, SK_BIAS, e, "action mlp");
        } else {
            if (c->want("action in")) {
                launch_small_linear(c->W("diffusion_noise"), 32, c->W("decoder_action_in_proj_w"), c->W("decoder_action_in_proj_b"),
                                    c->B("decoder_x"), 1024, ch, 32, 1024, 0, 1, 0, s);
                c->note(0, "action in");
            }
        }
    }

    void suffix_layer(int t, int i) {
        const int S_d = c->S_d, S_e = c->S_e, L = d.llm_layers;
        const int norm = pi05 ? SN_ADARMS : SN_RMS;
        const bf16_t* st_attn = pi05 ? c->B("decoder_style_attn") + ((size_t)t * L + i) * 3072 : nullptr;
        const bf16_t* st_ffn = pi05 ? c->B("decoder_style_ffn") + ((size_t)t * L + i) * 3072 : nullptr;
        SkinnyP q = tiled_io(); q.rope = c->W("decoder_rope_weights"); q.q = c->B("decoder_q_buf"); q.k = Kc(i); q.vt = Vt(i); q.ldvt = c->keys_pad; q.kv_row0 = S_e;
        if (pi05) {                                                  // adaptive RMS folded into the weights of this (step, layer)
            const size_t tl = (size_t)t * L + i;
            q.factor_f32 = 1; q.col_bias0 = c->B<float>("decoder_ada_bias_qkv") + tl * 2560;
            skinny(c->B("decoder_x"), 1024, S_d, c->TW("t_decoder_attn_qkv_ada", (int)tl), nullptr, 1024, 2560, SN_RMS, nullptr, SK_QKV_ROPE, q, "suffix qkv");
        } else
        skinny(c->B("decoder_x"), 1024, S_d, c->TW("t_decoder_attn_qkv_w", i), nullptr, 1024, 2560, norm, st_attn, SK_QKV_ROPE, q, "suffix qkv");
        AttnP a{};
        a.q = c->B("decoder_q_buf"); a.k = Kc(i); a.vt = Vt(i); a.ldvt = c->keys_pad;
        a.out = c->B("decoder_attn"); a.group = 8; a.out_tiled = 1; a.out_cols32 = 64; a.rows = 8 * S_d; a.keys = S_e + S_d; a.scale = 0.0625f;
        a.prefix_alloc = S_e; a.valid_len = valid_len(); a.state_rows = pi05 ? 0 : 8;
        a.nsplit = std::min(16, (a.keys + 127) / 128); a.partial = c->B<float>("attn_partial"); a.partial_floats = ATTN_PARTIAL_FLOATS;
        // the attention launch streams no weights and leaves a quarter of the CUs idle: 64 workgroups riding along it pull the 64 tiles
        // (64 KB each) of the output projection that follows towards the caches (measured: 0.7 us per layer)
        a.pf_attn = PrefetchP{{(const char*)c->TW("t_decoder_attn_o_w", i)}, {65536}, {64}};
        if (c->want("suffix attn")) { int nk = 1; const int rc = launch_mqa_attention(a, ATTN_SUFFIX, s, &nk); c->note(rc, "suffix attn", nk); }
        SkinnyP o = tiled_io(); o.out = c->B("decoder_x"); o.ldo = 1024; o.gate = pi05 ? st_attn + 2048 : nullptr;
        skinny(c->B("decoder_attn"), 2048, S_d, c->TW("t_decoder_attn_o_w", i), nullptr, 2048, 1024, SN_NONE, nullptr, SK_RES, o, "suffix o");
        SkinnyP g = tiled_io(); g.out = c->B("decoder_hidden"); g.ldo = 4096;
        if (pi05) {
            const size_t tl = (size_t)t * L + i;
            g.factor_f32 = 1; g.col_bias0 = c->B<float>("decoder_ada_bias_gate") + tl * 4096; g.col_bias1 = c->B<float>("decoder_ada_bias_up") + tl * 4096;
            skinny(c->B("decoder_x"), 1024, S_d, c->TW("t_decoder_ffn_gate_ada", (int)tl), c->TW("t_decoder_ffn_up_ada", (int)tl), 1024, 4096, SN_RMS, nullptr, SK_GEGLU, g, "suffix geglu");
        } else
        skinny(c->B("decoder_x"), 1024, S_d, c->TW("t_decoder_ffn_gate_w", i), c->TW("t_decoder_ffn_up_w", i), 1024, 4096, norm, st_ffn, SK_GEGLU, g, "suffix geglu");
        SkinnyP dn = tiled_io(); dn.out = c->B("decoder_x"); dn.ldo = 1024; dn.gate = pi05 ? st_ffn + 2048 : nullptr;
        skinny(c->B("decoder_hidden"), 4096, S_d, c->TW("t_decoder_ffn_down_w", i), nullptr, 4096, 1024, SN_NONE, nullptr, SK_RES, dn, "suffix down");
    }

    void suffix_step_end(int t) {
        const int ch = d.chunk_size;
        SkinnyP e{}; e.a_tiled = 1; e.out = c->W("diffusion_noise"); e.ldo = 32;       // noise stays row-major [chunk][32]
        if (!pi05) {
            e.a_row0 = 1;                                                               // action rows follow the state token
            e.bias = c->W("decoder_action_fused_out_proj_b");
            skinny(c->B("decoder_x"), 1024, ch, c->TW("t_decoder_out_proj_w"), nullptr, 1024, 32, SN_RMS, nullptr, SK_RES, e, "euler");
        } else {
            e.bias = c->B("decoder_out_proj_b_scaled");
            skinny(c->B("decoder_x"), 1024, ch, c->TW("t_decoder_out_proj_w"), nullptr, 1024, 32, SN_ADARMS,
                   c->B("decoder_style_final") + (size_t)t * 3072, SK_RES, e, "euler");
        }
    }

    // ---- DM0 (/root/reference/dm0_infer.py) ----
    bf16_t* dK(int i) { return c->B("kv_K") + (size_t)i * 8 * c->keys_pad * 128; }
    bf16_t* dVt(int i) { return c->B("kv_Vt") + (size_t)i * 8 * 128 * c->keys_pad; }
    const float* WF(const char* n, size_t layer_elems, int layer) { return (const float*)c->tensors[c->tindex.at(n)].ptr + layer_elems * layer; }

    // dm0_infer.py:695-712: patch embedding, class token, position embedding, ln_pre; then the first layer's LayerNorm
    void dm0_vision_embed() {
        const int n = d.num_views, M = n * DM0_SEQ_PAD;
        if (c->want("im2col")) { launch_dm0_im2col_nchw(c->W("images"), c->B("vision_patches"), PATCH_LD, n, s); c->note(0, "im2col"); }
        GemmP e{}; e.out = c->B("vision_conv1_buf"); e.ldo = 1024; e.bias = c->B("const_zeros");
        gemm(c->B("vision_patches"), PATCH_LD, n * 2704, n * 2704, c->TW("t_vision_conv1_w_t"), nullptr, 588, 1024, EPI_BIAS, e, "patch embed");
        if (c->want("class + pos + ln_pre")) {
            launch_dm0_embed_ln(c->B("vision_conv1_buf"), c->W("vision_class_embedding"), c->W("vision_pos_emb"), c->W("vision_ln_pre_w"), c->W("vision_ln_pre_b"),
                                c->B("vision_x_2d"), DM0_SEQ_PAD, n, s);
            c->note(0, "class + pos + ln_pre");
        }
        reduce(M, 1024, nullptr, c->B("vision_x_2d"), 1024, nullptr, 0, c->B("vision_x_norm"), 1024, NORM_LAYER, c->B("const_ones"), c->B("const_zeros"), 1e-5f, 0, "vit LN0");
    }

    // dm0_infer.py:718-736.  The LayerNorm scale and shift are folded into the weights; the rows are normalised by the reduce
    // kernel (x_norm), which equals the reference's  rstd (x W' - mean colsum(W')) + b'  up to the rounding of x_norm.
    void dm0_vision_layer(int i) {
        const int n = d.num_views, M = n * DM0_SEQ_PAD;
        GemmP e{}; e.bias_f32 = WF("vision_fused_qkv_b", 3072, i); e.rope = c->W("vision_rope"); e.seq = DM0_SEQ; e.seq_pad = DM0_SEQ_PAD;
        e.q = c->B("vision_Q"); e.k = c->B("vision_K"); e.vt = c->B("vision_Vt");
        gemm(c->B("vision_x_norm"), 1024, M, M, c->TW("t_vision_fused_qkv_w", i), nullptr, 1024, 3072, EPI_VIT_QKV_ROPE, e, "vit qkv");
        AttnP a{};
        a.q = c->B("vision_Q"); a.k = c->B("vision_K"); a.vt = c->B("vision_Vt"); a.ldvt = DM0_SEQ_PAD;
        a.batch = n * 16; a.q_bstride = a.k_bstride = (size_t)DM0_SEQ_PAD * 64; a.vt_bstride = (size_t)64 * DM0_SEQ_PAD;
        a.group = 1; a.rows = DM0_SEQ; a.keys = DM0_SEQ; a.scale = 0.125f; a.prefix_alloc = DM0_SEQ;
        a.out = c->B("vision_attn"); a.ld_tok = 1024; a.batch_inner = 16; a.out_ostride = (size_t)DM0_SEQ_PAD * 1024; a.out_istride = 64;
        if (c->want("vit attn")) c->note(launch_flash_attention(a, 64, s), "vit attn");
        gemm(c->B("vision_attn"), 1024, M, M, c->TW("t_vision_out_proj_w", i), nullptr, 1024, 1024, EPI_PARTIAL, GemmP{}, "vit o");
        reduce(M, 1024, c->W("vision_out_proj_b", 1024, i), c->B("vision_x_2d"), 1024, c->B("vision_x_2d"), 1024, c->B("vision_x_norm"), 1024,
               NORM_LAYER, c->B("const_ones"), c->B("const_zeros"), 1e-5f, last_split, "vit o reduce");
        GemmP u{}; u.out = c->B("vision_fc"); u.ldo = 4096; u.bias_f32 = WF("vision_fused_fc_b", 4096, i);
        gemm(c->B("vision_x_norm"), 1024, M, M, c->TW("t_vision_fused_fc_w", i), nullptr, 1024, 4096, EPI_BIAS_GELU, u, "vit fc");
        gemm(c->B("vision_fc"), 4096, M, M, c->TW("t_vision_proj_w", i), nullptr, 4096, 1024, EPI_PARTIAL, GemmP{}, "vit proj");
        // (nothing reads the normalised copy after the last layer: the down-sampling convolutions take the stream itself)
        const bool last = i == d.vision_layers - 1;
        reduce(M, 1024, c->W("vision_proj_b", 1024, i), c->B("vision_x_2d"), 1024, c->B("vision_x_2d"), 1024, last ? nullptr : c->B("vision_x_norm"), 1024,
               last ? NORM_NONE : NORM_LAYER, c->B("const_ones"), c->B("const_zeros"), 1e-5f, last_split, "vit proj reduce");
    }

    // dm0_infer.py:738-756: drop the class token, two stride-2 3x3 convolutions, projector, token embeddings; then the RMS
    // factor of the first prefix layer
    void dm0_project() {
        const int n = d.num_views, P = c->S_e, T = n * DM0_TOK;
        if (c->want("im2col ds1")) { launch_dm0_im2col3x3(c->B("vision_x_2d"), DM0_SEQ_PAD, 1, 52, 52, 1024, c->B("vision_col1"), n, s); c->note(0, "im2col ds1"); }
        GemmP e{}; e.out = c->B("vision_mm1"); e.ldo = 2048; e.bias = c->W("vision_ds1_b");
        gemm(c->B("vision_col1"), 9216, n * 676, n * 676, c->TW("t_vision_ds1_w"), nullptr, 9216, 2048, EPI_BIAS, e, "ds1");
        if (c->want("im2col ds2")) { launch_dm0_im2col3x3(c->B("vision_mm1"), 676, 0, 26, 26, 2048, c->B("vision_col2"), n, s); c->note(0, "im2col ds2"); }
        GemmP f{}; f.out = c->B("vision_mm2"); f.ldo = 4096; f.bias = c->W("vision_ds2_b");
        gemm(c->B("vision_col2"), 18432, T, T, c->TW("t_vision_ds2_w"), nullptr, 18432, 4096, EPI_BIAS, f, "ds2");
        GemmP g{}; g.out = c->B("prefix_x"); g.ldo = 2048; g.bias = c->B("const_zeros");
        gemm(c->B("vision_mm2"), 4096, T, T, c->TW("t_vision_projector_w_t"), nullptr, 4096, 2048, EPI_BIAS, g, "projector");
        if (d.prompt_len > 0 && c->want("token embeddings")) {
            launch_dm0_gather_rows(c->W("vision_embed_tokens_w"), (int)c->T("vision_embed_tokens_w").shape[0], (const int*)c->T("input_ids").ptr,
                                   c->B("prefix_x") + (size_t)T * 2048, d.prompt_len, s);
            c->note(0, "token embeddings");
        }
        reduce(P, 2048, nullptr, c->B("prefix_x"), 2048, nullptr, 0, nullptr, 0, NORM_RMS, nullptr, nullptr, 1e-6f, 0, "prefix factor0", c->B<float>("prefix_norm_factor"));
    }

    // dm0_infer.py:874-951
    void dm0_prefix_layer(int i) { dm0_prefix_layer_kv(i); dm0_prefix_layer_rest(i); }

    void dm0_prefix_layer_kv(int i) {
        const int P = c->S_e, kp = c->keys_pad;
        const size_t qstride = (size_t)((2 * P + 31) / 32) * 32 * 128;
        GemmP e{}; e.out = c->B("prefix_qkv"); e.ldo = 4096; e.bias = c->B("const_zeros");
        gemm(c->B("prefix_x"), 2048, P, P, c->TW("t_llm_attn_qkv_w", i), nullptr, 2048, 4096, EPI_BIAS, e, "prefix qkv");
        if (c->want("prefix qk-norm rope")) {
            launch_dm0_qknorm_rope(c->B("prefix_qkv"), 4096, c->B<float>("prefix_norm_factor"), nullptr, c->W("llm_q_norm_w", 128, i), c->W("llm_k_norm_w", 128, i),
                                   c->W("prefix_rope_weights"), c->B("prefix_Q"), qstride, dK(i), (size_t)kp * 128, dVt(i), (size_t)128 * kp, kp >> 5, 0, P, s);
            c->note(0, "prefix qk-norm rope");
        }
    }

    void dm0_prefix_layer_rest(int i) {
        const int P = c->S_e, kp = c->keys_pad;
        const size_t qstride = (size_t)((2 * P + 31) / 32) * 32 * 128;
        if (i == d.llm_layers - 1) return;           // the action expert reads only the K / V cache of the last prefix layer
        AttnP a{};
        a.q = c->B("prefix_Q"); a.k = dK(i); a.vt = dVt(i); a.ldvt = kp;
        a.batch = 8; a.q_bstride = qstride; a.k_bstride = (size_t)kp * 128; a.vt_bstride = (size_t)128 * kp;
        a.group = 2; a.rows = 2 * P; a.keys = P; a.scale = 0.08838834764831845f; a.prefix_alloc = P; a.causal = 1;
        a.out = c->B("prefix_attn"); a.ld_tok = 2048; a.batch_inner = 8; a.out_istride = 256;
        if (c->want("prefix attn")) c->note(launch_mqa_attention(a, ATTN_GQA128_PREFIX, s), "prefix attn");
        gemm(c->B("prefix_attn"), 2048, P, P, c->TW("t_llm_attn_o_w", i), nullptr, 2048, 2048, EPI_PARTIAL, GemmP{}, "prefix o");
        reduce(P, 2048, nullptr, c->B("prefix_x"), 2048, c->B("prefix_x"), 2048, nullptr, 0, NORM_RMS, nullptr, nullptr, 1e-6f, last_split, "prefix o reduce",
               c->B<float>("prefix_norm_factor"));
        GemmP g{}; g.out = c->B("prefix_hidden"); g.ldo = 6144; g.rowscale = c->B<float>("prefix_norm_factor");
        gemm(c->B("prefix_x"), 2048, P, P, c->TW("t_llm_ffn_gate_w", i), c->TW("t_llm_ffn_up_w", i), 2048, 6144, EPI_SWIGLU, g, "prefix swiglu");
        gemm(c->B("prefix_hidden"), 6144, P, P, c->TW("t_llm_ffn_down_w", i), nullptr, 6144, 2048, EPI_PARTIAL, GemmP{}, "prefix down");
        reduce(P, 2048, nullptr, c->B("prefix_x"), 2048, c->B("prefix_x"), 2048, nullptr, 0, NORM_RMS, nullptr, nullptr, 1e-6f, last_split, "prefix down reduce",
               c->B<float>("prefix_norm_factor"));
    }

    // dm0_infer.py:763-780
    void dm0_step_begin(int t) {
        const int ch = d.chunk_size;
        if (c->want("action in")) {
            launch_small_linear(c->W("diffusion_noise"), 32, c->W("decoder_action_fused_in_proj_w"), c->W("decoder_action_fused_time_biases", 1024, t % 10),
                                c->B("decoder_x_buf"), 1024, ch, 32, 1024, 1, 1, 0, s);
            c->note(0, "action in");
        }
        SkinnyP e = tiled_io(); e.out = c->B("decoder_x"); e.ldo = 1024; e.bias = c->W("decoder_action_mlp_b");
        skinny(c->B("decoder_x_buf"), 1024, ch, c->TW("t_decoder_action_mlp_w"), nullptr, 1024, 1024, SN_NONE, nullptr, SK_BIAS, e, "action mlp");
    }

    // dm0_infer.py:782-851
    void dm0_suffix_layer(int t, int i) {
        const int ch = d.chunk_size, P = c->S_e, kp = c->keys_pad;
        SkinnyP q{}; q.a_tiled = 1; q.out = c->B("decoder_qkv"); q.ldo = 4096; q.bias = c->B("const_zeros");
        skinny(c->B("decoder_x"), 1024, ch, c->TW("t_decoder_attn_qkv_w", i), nullptr, 1024, 4096, SN_NONE, nullptr, SK_BIAS, q, "suffix qkv");
        if (c->want("suffix qk-norm rope")) {
            launch_dm0_qknorm_rope(c->B("decoder_qkv"), 4096, nullptr, c->B("decoder_x"), c->W("decoder_q_norm_w", 128, i), c->W("decoder_k_norm_w", 128, i),
                                   c->W("decoder_rope_weights"), c->B("decoder_Q"), (size_t)128 * 128, dK(i), (size_t)kp * 128, dVt(i), (size_t)128 * kp, kp >> 5, P, ch, s);
            c->note(0, "suffix qk-norm rope");
        }
        AttnP a{};
        a.q = c->B("decoder_Q"); a.k = dK(i); a.vt = dVt(i); a.ldvt = kp;
        a.batch = 8; a.q_bstride = (size_t)128 * 128; a.k_bstride = (size_t)kp * 128; a.vt_bstride = (size_t)128 * kp;
        a.group = 2; a.rows = 2 * ch; a.keys = P + ch; a.scale = 0.08838834764831845f; a.prefix_alloc = P + ch;
        a.pf_attn = PrefetchP{{(const char*)c->TW("t_decoder_attn_o_w", i)}, {65536}, {64}};      // as in suffix_layer
        a.out = c->B("decoder_attn"); a.out_tiled = 1; a.out_bcol = 256; a.out_cols32 = 64;
        a.nsplit = std::min(16, (a.keys + 127) / 128); a.partial = c->B<float>("attn_partial"); a.partial_floats = ATTN_PARTIAL_FLOATS;
        if (c->want("suffix attn")) { int nk = 1; const int rc = launch_mqa_attention(a, ATTN_GQA128_SUFFIX, s, &nk); c->note(rc, "suffix attn", nk); }
        SkinnyP o = tiled_io(); o.out = c->B("decoder_x"); o.ldo = 1024;
        skinny(c->B("decoder_attn"), 2048, ch, c->TW("t_decoder_attn_o_w", i), nullptr, 2048, 1024, SN_NONE, nullptr, SK_RES, o, "suffix o");
        SkinnyP g = tiled_io(); g.out = c->B("decoder_hidden"); g.ldo = 2048; g.factor_f32 = 1;
        skinny(c->B("decoder_x"), 1024, ch, c->TW("t_decoder_ffn_gate_w", i), c->TW("t_decoder_ffn_up_w", i), 1024, 1536, SN_RMS, nullptr, SK_SWIGLU, g, "suffix swiglu");
        SkinnyP dn = tiled_io(); dn.out = c->B("decoder_x"); dn.ldo = 1024;
        skinny(c->B("decoder_hidden"), 2048, ch, c->TW("t_decoder_ffn_down_w", i), nullptr, 2048, 1024, SN_NONE, nullptr, SK_RES, dn, "suffix down");
    }

    // dm0_infer.py:863-872, :99-120
    void dm0_step_end(int t) {
        SkinnyP e{}; e.a_tiled = 1; e.out = c->W("diffusion_noise"); e.ldo = 32; e.bias = c->W("decoder_action_fused_out_proj_b"); e.factor_f32 = 1;
        skinny(c->B("decoder_x"), 1024, d.chunk_size, c->TW("t_decoder_out_proj_w"), nullptr, 1024, 32, SN_RMS, nullptr, SK_RES, e, "euler");
    }

    void dm0_prepare(bool tiles_loaded) {
        const int V = d.vision_layers, L = d.llm_layers;
        launch_fill_zero(c->ws + c->act_begin, c->ws_bytes - c->act_begin, s);
        launch_fill_bf16(c->B("const_ones"), 1024, 1.0f, s);
        if (tiles_loaded) return;
        auto tile = [&](const char* src, const char* dst, int K, int N, int layers) {
            for (int i = 0; i < layers; ++i) launch_pretile(c->W(src, (size_t)K * N, i), K, N, c->TW(dst, i), c->tgroup.at(dst), c->twide.at(dst), s);
        };
        tile("vision_conv1_w_t", "t_vision_conv1_w_t", 588, 1024, 1);
        tile("vision_fused_qkv_w", "t_vision_fused_qkv_w", 1024, 3072, V);
        tile("vision_out_proj_w", "t_vision_out_proj_w", 1024, 1024, V);
        tile("vision_fused_fc_w", "t_vision_fused_fc_w", 1024, 4096, V);
        tile("vision_proj_w", "t_vision_proj_w", 4096, 1024, V);
        tile("vision_ds1_w", "t_vision_ds1_w", 9216, 2048, 1);
        tile("vision_ds2_w", "t_vision_ds2_w", 18432, 4096, 1);
        tile("vision_projector_w_t", "t_vision_projector_w_t", 4096, 2048, 1);
        tile("llm_attn_qkv_w", "t_llm_attn_qkv_w", 2048, 4096, L);
        tile("llm_attn_o_w", "t_llm_attn_o_w", 2048, 2048, L);
        tile("llm_ffn_gate_w", "t_llm_ffn_gate_w", 2048, 6144, L);
        tile("llm_ffn_up_w", "t_llm_ffn_up_w", 2048, 6144, L);
        tile("llm_ffn_down_w", "t_llm_ffn_down_w", 6144, 2048, L);
        tile("decoder_attn_qkv_w", "t_decoder_attn_qkv_w", 1024, 4096, L);
        tile("decoder_attn_o_w", "t_decoder_attn_o_w", 2048, 1024, L);
        tile("decoder_ffn_gate_w", "t_decoder_ffn_gate_w", 1024, 1536, L);
        tile("decoder_ffn_up_w", "t_decoder_ffn_up_w", 1024, 1536, L);
        for (int i = 0; i < L; ++i)       // K = 1536 rows of the checkpoint, laid out for K = 2048 with zero rows behind
            launch_pretile_padded(c->W("decoder_ffn_down_w", (size_t)1536 * 1024, i), 1536, 2048, 1024, c->TW("t_decoder_ffn_down_w", i), s);
        tile("decoder_action_mlp_w", "t_decoder_action_mlp_w", 1024, 1024, 1);
        tile("decoder_action_fused_out_proj_w", "t_decoder_out_proj_w", 1024, 32, 1);
    }

    int dm0_stage(int st, int layer, int step) {
        switch (st) {
            case RTVLA_STAGE_VISION_EMBED: dm0_vision_embed(); break;
            case RTVLA_STAGE_VISION_LAYER: if (layer < 0 || layer >= d.vision_layers) return RTVLA_ERR_ARG; dm0_vision_layer(layer); break;
            case RTVLA_STAGE_PROJECT: dm0_project(); break;
            case RTVLA_STAGE_PREFIX_LAYER: if (layer < 0 || layer >= d.llm_layers) return RTVLA_ERR_ARG; dm0_prefix_layer(layer); break;
            case RTVLA_STAGE_SUFFIX_INIT: break;
            case RTVLA_STAGE_SUFFIX_STEP_BEGIN: if (step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG; dm0_step_begin(step); break;
            case RTVLA_STAGE_SUFFIX_LAYER:
                if (layer < 0 || layer >= d.llm_layers || step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG;
                dm0_suffix_layer(step, layer); break;
            case RTVLA_STAGE_SUFFIX_STEP_END: if (step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG; dm0_step_end(step); break;
            default: return RTVLA_ERR_ARG;
        }
        return 0;
    }

    void dm0_forward(hipStream_t fork = nullptr, hipEvent_t* ev = nullptr) {
        dm0_vision_embed();
        for (int i = 0; i < d.vision_layers; ++i) dm0_vision_layer(i);
        dm0_project();
        prefix_with_first_step(fork, ev, [&](int i) { dm0_prefix_layer_kv(i); }, [&](int i) { dm0_prefix_layer_rest(i); },
                               [&]() { dm0_step_begin(0); }, [&](int i) { dm0_suffix_layer(0, i); });
        dm0_step_end(0);
        for (int t = 1; t < d.num_steps; ++t) {
            dm0_step_begin(t);
            for (int i = 0; i < d.llm_layers; ++i) dm0_suffix_layer(t, i);
            dm0_step_end(t);
        }
    }

    int stage(int st, int layer, int step) {
        if (d.model == RTVLA_DM0) return dm0_stage(st, layer, step);
        switch (st) {
            case RTVLA_STAGE_VISION_EMBED: vision_embed(); break;
            case RTVLA_STAGE_VISION_LAYER: if (layer < 0 || layer >= d.vision_layers) return RTVLA_ERR_ARG; vision_layer(layer); break;
            case RTVLA_STAGE_PROJECT: project(); break;
            case RTVLA_STAGE_PREFIX_LAYER: if (layer < 0 || layer >= d.llm_layers) return RTVLA_ERR_ARG; prefix_layer(layer); break;
            case RTVLA_STAGE_SUFFIX_INIT: suffix_init(); break;
            case RTVLA_STAGE_SUFFIX_STEP_BEGIN: if (step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG; suffix_step_begin(step); break;
            case RTVLA_STAGE_SUFFIX_LAYER:
                if (layer < 0 || layer >= d.llm_layers || step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG;
                suffix_layer(step, layer); break;
            case RTVLA_STAGE_SUFFIX_STEP_END: if (step < 0 || step >= d.num_steps) return RTVLA_ERR_ARG; suffix_step_end(step); break;
            default: return RTVLA_ERR_ARG;
        }
        return 0;
    }

    // Layer i of the action expert's FIRST flow step needs of the prefix pass only the K / V rows of prefix layer i, which exist as
    // soon as that layer's QKV launch is done.  With a side stream (`fork`, only while both streams are being captured into one graph)
    // the first flow step therefore runs as a second branch of the graph next to prefix layers i+1 ..: its small latency-bound
    // launches fill the gaps of the large GEMMs instead of following them.  Same launches, same operands, same results as the
    // one-stream order.  Returns a HIP error from the event calls, if any.
    hipError_t fork_step0 = hipSuccess;
    template <typename KV, typename Rest, typename Begin, typename Layer>
    void prefix_with_first_step(hipStream_t fork, hipEvent_t* ev, KV kv, Rest rest, Begin begin, Layer layer) {
        const int L = d.llm_layers;
        if (!fork) {
            for (int i = 0; i < L; ++i) { kv(i); rest(i); }
            begin();
            for (int i = 0; i < L; ++i) layer(i);
            return;
        }
        hipStream_t main = s;
        auto ok = [&](hipError_t e) { if (e != hipSuccess && fork_step0 == hipSuccess) fork_step0 = e; };
        // An edge between the branches costs the main chain ~10 us (measured), so the first flow step follows in groups: after the
        // K / V launch of prefix layers L-2, L-2-G, L-2-2G, ... the side branch runs all action-expert layers whose prefix rows exist
        // by then; the group that ends at L-2 hides under prefix layer L-2, the last layer follows the join.  (Measured, Pi0 headline
        // shape: one edge per layer 11.87 ms, G = 3: 11.79, 6: 11.81, 9: 11.82, a single group: 11.94 = no gain; DM0 23.28 -> 23.01 ms.
        // The large GEMMs own every register of a CU, so the side branch's workgroups take turns with them rather than run beside
        // them: what is saved is the launch latency of the small kernels, not their CU time.)
        const int G = tuning_fork_group(4);
        int next = 0;
        for (int i = 0; i < L; ++i) {
            kv(i);
            if (i <= L - 2 && (L - 2 - i) % G == 0) {
                ok(hipEventRecord(ev[i], main)); ok(hipStreamWaitEvent(fork, ev[i], 0));      // (the side stream joins the capture at the first of these)
                s = fork;
                if (next == 0) begin();
                for (; next <= i; ++next) layer(next);
                s = main;
            }
            rest(i);
        }
        if (next > 0) { ok(hipEventRecord(ev[L], fork)); ok(hipStreamWaitEvent(main, ev[L], 0)); }
        else begin();
        for (; next < L; ++next) layer(next);
    }

    void forward(hipStream_t fork = nullptr, hipEvent_t* ev = nullptr) {
        if (d.model == RTVLA_DM0) { dm0_forward(fork, ev); return; }
        vision_embed();
        for (int i = 0; i < d.vision_layers; ++i) vision_layer(i);
        project();
        suffix_init();
        prefix_with_first_step(fork, ev, [&](int i) { prefix_layer_kv(i); }, [&](int i) { prefix_layer_rest(i); },
                               [&]() { suffix_step_begin(0); }, [&](int i) { suffix_layer(0, i); });
        suffix_step_end(0);
        for (int t = 1; t < d.num_steps; ++t) {
            suffix_step_begin(t);
            for (int i = 0; i < d.llm_layers; ++i) suffix_layer(t, i);
            suffix_step_end(t);
        }
    }

    // one-time device work.  With `tiles_loaded` the re-tiled weights (the first rtvla_tiled_bytes of the workspace) were
    // filled in by the caller from a copy saved after an earlier prepare, and only the rest is done.
    void prepare(bool tiles_loaded) {
        if (d.model == RTVLA_DM0) { dm0_prepare(tiles_loaded); return; }
        const int V = d.vision_layers, L = d.llm_layers;
        launch_fill_zero(c->ws + c->act_begin, c->ws_bytes - c->act_begin, s);
        auto tile = [&](const char* src, const char* dst, int K, int N, int layers) {
            if (tiles_loaded) return;
            for (int i = 0; i < layers; ++i) launch_pretile(c->W(src, (size_t)K * N, i), K, N, c->TW(dst, i), c->tgroup.at(dst), c->twide.at(dst), s);
        };
        tile("vision_patch_embedding_w", "t_vision_patch_embedding_w", 588, 1152, 1);
        tile("vision_attn_qkv_w", "t_vision_attn_qkv_w", 1152, 3456, V);
        tile("vision_attn_o_w", "t_vision_attn_o_w", 1152, 1152, V);
        tile("vision_ffn_up_w", "t_vision_ffn_up_w", 1152, 4304, V);
        tile("vision_ffn_down_w", "t_vision_ffn_down_w", 4304, 1152, V);
        tile("encoder_multi_modal_projector_w", "t_encoder_multi_modal_projector_w", 1152, 2048, 1);
        tile("encoder_attn_qkv_w", "t_encoder_attn_qkv_w", 2048, 2560, L);
        tile("encoder_attn_o_w", "t_encoder_attn_o_w", 2048, 2048, L);
        tile("encoder_ffn_gate_w", "t_encoder_ffn_gate_w", 2048, 16384, L);
        tile("encoder_ffn_up_w", "t_encoder_ffn_up_w", 2048, 16384, L);
        tile("encoder_ffn_down_w", "t_encoder_ffn_down_w", 16384, 2048, L);
        tile("decoder_attn_qkv_w", "t_decoder_attn_qkv_w", 1024, 2560, L);
        tile("decoder_attn_o_w", "t_decoder_attn_o_w", 2048, 1024, L);
        tile("decoder_ffn_gate_w", "t_decoder_ffn_gate_w", 1024, 4096, L);
        tile("decoder_ffn_up_w", "t_decoder_ffn_up_w", 1024, 4096, L);
        tile("decoder_ffn_down_w", "t_decoder_ffn_down_w", 4096, 1024, L);
        if (!pi05) {
            tile("decoder_action_mlp_w", "t_decoder_action_mlp_w", 1024, 1024, 1);
            tile("decoder_action_fused_out_proj_w", "t_decoder_out_proj_w", 1024, 32, 1);
            return;
        }
        // Pi05: out-proj scaled by -1/num_steps (pi05_infer.py:669-671), then the time conditioning (:673-722)
        const float dt = -1.0f / (float)d.num_steps;
        if (!tiles_loaded) {                               // (the scaled copies sit in the saved region as well)
            launch_copy_bytes(c->W("decoder_action_out_proj_w"), c->B("decoder_out_proj_w_scaled"), 1024 * 32 * 2, s);
            launch_scale_inplace(c->B("decoder_out_proj_w_scaled"), 1024 * 32, dt, s);
            launch_copy_bytes(c->W("decoder_action_out_proj_b"), c->B("decoder_out_proj_b_scaled"), 64, s);
            launch_scale_inplace(c->B("decoder_out_proj_b_scaled"), 32, dt, s);
            launch_pretile(c->B("decoder_out_proj_w_scaled"), 1024, 32, c->TW("t_decoder_out_proj_w"), 1, 0, s);
        }
        tile("decoder_time_mlp_in_w", "t_decoder_time_mlp_in_w", 1024, 1024, 1);
        tile("decoder_time_mlp_out_w", "t_decoder_time_mlp_out_w", 1024, 1024, 1);
        tile("decoder_pre_attn_norm_mod_w", "t_decoder_pre_attn_norm_mod_w", 1024, 3072, L);
        tile("decoder_pre_ffn_norm_mod_w", "t_decoder_pre_ffn_norm_mod_w", 1024, 3072, L);
        tile("decoder_final_norm_mod_w", "t_decoder_final_norm_mod_w", 1024, 3072, 1);
        const int T = d.num_steps;
        SkinnyP e{}; e.out_tiled = 1; e.out = c->B("decoder_x_buf"); e.ldo = 1024; e.bias = c->W("decoder_time_mlp_in_b");
        skinny(c->W("decoder_time_embeds"), 1024, T, c->TW("t_decoder_time_mlp_in_w"), nullptr, 1024, 1024, SN_NONE, nullptr, SK_BIAS_SILU, e, "time mlp in");
        e.a_tiled = 1; e.out = c->B("decoder_time_emb"); e.bias = c->W("decoder_time_mlp_out_b");
        skinny(c->B("decoder_x_buf"), 1024, T, c->TW("t_decoder_time_mlp_out_w"), nullptr, 1024, 1024, SN_NONE, nullptr, SK_BIAS_SILU, e, "time mlp out");
        for (int i = 0; i < L; ++i) {
            SkinnyP m{}; m.a_tiled = 1; m.ldo = L * 3072;
            m.out = c->B("decoder_style_attn") + (size_t)i * 3072; m.bias = c->W("decoder_pre_attn_norm_mod_b", 3072, i);
            skinny(c->B("decoder_time_emb"), 1024, T, c->TW("t_decoder_pre_attn_norm_mod_w", i), nullptr, 1024, 3072, SN_NONE, nullptr, SK_BIAS, m, "style attn");
            m.out = c->B("decoder_style_ffn") + (size_t)i * 3072; m.bias = c->W("decoder_pre_ffn_norm_mod_b", 3072, i);
            skinny(c->B("decoder_time_emb"), 1024, T, c->TW("t_decoder_pre_ffn_norm_mod_w", i), nullptr, 1024, 3072, SN_NONE, nullptr, SK_BIAS, m, "style ffn");
        }
        SkinnyP f{}; f.a_tiled = 1; f.ldo = 3072; f.out = c->B("decoder_style_final"); f.bias = c->W("decoder_final_norm_mod_b");
        skinny(c->B("decoder_time_emb"), 1024, T, c->TW("t_decoder_final_norm_mod_w"), nullptr, 1024, 3072, SN_NONE, nullptr, SK_BIAS, f, "style final");
        // the adaptive RMS norm of every (step, layer) folded into its consumers' weights: style = [scale | shift | gate]
        for (int t = 0; t < T; ++t)
            for (int i = 0; i < L; ++i) {
                const size_t tl = (size_t)t * L + i;
                const bf16_t* sa = c->B("decoder_style_attn") + tl * 3072;
                const bf16_t* sf = c->B("decoder_style_ffn") + tl * 3072;
                const bf16_t* wq = c->W("decoder_attn_qkv_w", (size_t)1024 * 2560, i);
                const bf16_t* wg = c->W("decoder_ffn_gate_w", (size_t)1024 * 4096, i);
                const bf16_t* wu = c->W("decoder_ffn_up_w", (size_t)1024 * 4096, i);
                if (!tiles_loaded) {
                    launch_pretile(wq, 1024, 2560, c->TW("t_decoder_attn_qkv_ada", (int)tl), 1, 0, s, sa);
                    launch_pretile(wg, 1024, 4096, c->TW("t_decoder_ffn_gate_ada", (int)tl), 1, 0, s, sf);
                    launch_pretile(wu, 1024, 4096, c->TW("t_decoder_ffn_up_ada", (int)tl), 1, 0, s, sf);
                }
                launch_vec_mat(sa + 1024, wq, 1024, 2560, c->B<float>("decoder_ada_bias_qkv") + tl * 2560, s);
                launch_vec_mat(sf + 1024, wg, 1024, 4096, c->B<float>("decoder_ada_bias_gate") + tl * 4096, s);
                launch_vec_mat(sf + 1024, wu, 1024, 4096, c->B<float>("decoder_ada_bias_up") + tl * 4096, s);
            }
    }
};

int check_ready(rtvla_ctx* c, bool need_prepared) {
    if (!c) return RTVLA_ERR_ARG;
    if (!c->ws) return c->fail(RTVLA_ERR_STATE, "workspace not bound");
    for (auto& t : c->tensors)
        if (t.required && !t.bound) return c->fail(RTVLA_ERR_UNBOUND, "tensor not bound: " + t.name);
    if (need_prepared && !c->prepared) return c->fail(RTVLA_ERR_STATE, "rtvla_prepare has not run");
    return 0;
}

int hip_fail(rtvla_ctx* c, hipError_t e, const char* what) {
    return c->fail(RTVLA_ERR_DEVICE, std::string(what) + ": " + hipGetErrorString(e));
}

// A captured graph holds the addresses that were bound when it was recorded: any later binding makes it stale.
void drop_graph(rtvla_ctx* c) {
    if (c->exec) { hipGraphExecDestroy(c->exec); c->exec = nullptr; }
    if (c->graph) { hipGraphDestroy(c->graph); c->graph = nullptr; }
}

}  // namespace

extern "C" {

int rtvla_version(void) { return RTVLA_VERSION; }

int rtvla_create(const rtvla_dims* dims, rtvla_ctx** out) {
    if (!dims || !out) return RTVLA_ERR_ARG;
    *out = nullptr;
    const rtvla_dims& d = *dims;
    if (d.model != RTVLA_PI0 && d.model != RTVLA_PI05 && d.model != RTVLA_DM0) return RTVLA_ERR_ARG;
    if (d.num_views < 1 || d.num_views > 4 || d.prompt_len < 0 || d.chunk_size < 1 || d.num_steps < 1) return RTVLA_ERR_ARG;
    if (d.vision_layers < 1 || d.llm_layers < 1) return RTVLA_ERR_ARG;
    const int S_d = d.chunk_size + (d.model == RTVLA_PI0 ? 1 : 0);
    if (S_d > (d.model == RTVLA_DM0 ? 64 : 128)) return RTVLA_ERR_LIMIT;        // two 64-row blocks of the action-expert kernels (DM0's buffers hold one)
    // Pi0 / DM0: the converted checkpoint is tied to 10 steps (dt = -1/10 folded into the output projection, 10 fused time
    // biases: convert_from_jax.py:176-194); Pi05 scales by -1/num_steps itself but its time table has 10 rows
    if (d.model == RTVLA_PI05 ? d.num_steps > 10 : d.num_steps != 10) return RTVLA_ERR_LIMIT;
    if (d.prompt_len > 4096) return RTVLA_ERR_LIMIT;
    rtvla_ctx* c = new (std::nothrow) rtvla_ctx();
    if (!c) return RTVLA_ERR_ARG;
    c->d = d;
    c->S_v = (d.model == RTVLA_DM0 ? DM0_TOK : 256) * d.num_views;
    c->S_e = c->S_v + d.prompt_len;
    c->S_d = S_d;
    c->keys = c->S_e + c->S_d;
    c->keys_pad = ((c->keys + 63) / 64) * 64;
    if (d.model == RTVLA_DM0) build_tables_dm0(c); else build_tables(c);
    *out = c;
    return RTVLA_OK;
}

int rtvla_destroy(rtvla_ctx* c) {
    if (!c) return RTVLA_ERR_ARG;
    drop_graph(c);
    if (c->timing_stream) hipStreamDestroy(c->timing_stream);
    if (c->fork_stream) hipStreamDestroy(c->fork_stream);
    for (hipEvent_t e : c->fork_events) hipEventDestroy(e);
    delete c;
    return RTVLA_OK;
}

const char* rtvla_last_error(const rtvla_ctx* c) { return c ? c->err.c_str() : "null context"; }

int rtvla_tensor_count(const rtvla_ctx* c) { return c ? (int)c->tensors.size() : 0; }

int rtvla_tensor_info(const rtvla_ctx* c, int index, const char** name, int32_t* elem_bytes, int32_t* rank,
                      int64_t shape[4], int32_t* is_weight, int32_t* required) {
    if (!c || index < 0 || index >= (int)c->tensors.size()) return RTVLA_ERR_ARG;
    const Tensor& t = c->tensors[index];
    if (name) *name = t.name.c_str();
    if (elem_bytes) *elem_bytes = t.elem;
    if (rank) *rank = t.rank;
    if (shape) for (int i = 0; i < 4; ++i) shape[i] = t.shape[i];
    if (is_weight) *is_weight = t.weight;
    if (required) *required = t.required;
    return RTVLA_OK;
}

int rtvla_bind(rtvla_ctx* c, const char* name, void* ptr, size_t bytes) {
    if (!c || !name) return RTVLA_ERR_ARG;
    auto it = c->tindex.find(name);
    if (it == c->tindex.end()) return c->fail(RTVLA_ERR_NAME, std::string("unknown tensor: ") + name);
    Tensor& t = c->tensors[it->second];
    if ((t.name == "embedding_weight" || t.name == "vision_embed_tokens_w") && bytes > 0 && bytes % 4096 == 0) t.shape[0] = (int64_t)(bytes / 4096);
    if (bytes != t.bytes()) return c->fail(RTVLA_ERR_SIZE, std::string("size mismatch for ") + name + ": got " + std::to_string(bytes) + ", want " + std::to_string(t.bytes()));
    if (!ptr && bytes) return c->fail(RTVLA_ERR_ARG, std::string("null pointer for ") + name);
    if (((uintptr_t)ptr & 15) != 0) return c->fail(RTVLA_ERR_ARG, std::string("pointer not 16-byte aligned: ") + name);
    t.ptr = ptr; t.bound = true;
    c->prepared = false;
    drop_graph(c);
    return RTVLA_OK;
}

size_t rtvla_workspace_bytes(const rtvla_ctx* c) { return c ? c->ws_bytes : 0; }

int rtvla_bind_workspace(rtvla_ctx* c, void* ptr, size_t bytes) {
    if (!c || !ptr) return RTVLA_ERR_ARG;
    if (bytes < c->ws_bytes) return c->fail(RTVLA_ERR_SIZE, "workspace too small");
    if (((uintptr_t)ptr & 255) != 0) return c->fail(RTVLA_ERR_ARG, "workspace not 256-byte aligned");
    c->ws = (char*)ptr; c->prepared = false;
    drop_graph(c);
    return RTVLA_OK;
}

int rtvla_buffer_count(const rtvla_ctx* c) { return c ? (int)c->bufs.size() : 0; }

int rtvla_buffer_info(const rtvla_ctx* c, int index, const char** name, size_t* offset, int64_t* rows, int64_t* cols,
                      int64_t* ld, int32_t* elem_bytes) {
    if (!c || index < 0 || index >= (int)c->bufs.size()) return RTVLA_ERR_ARG;
    const WsBuf& b = c->bufs[index];
    if (name) *name = b.name.c_str();
    if (offset) *offset = b.offset;
    if (rows) *rows = b.rows;
    if (cols) *cols = b.cols;
    if (ld) *ld = b.ld;
    if (elem_bytes) *elem_bytes = b.elem;
    return RTVLA_OK;
}

static int prepare_impl(rtvla_ctx* c, void* stream, bool tiles_loaded) {
    if (int rc = check_ready(c, false)) return rc;
    c->status = 0; c->launches = 0; c->kernels = 0;
    Sched(c, (hipStream_t)stream).prepare(tiles_loaded);
    if (c->status) return c->status;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(c, e, "prepare");
    c->prepared = true;
    return RTVLA_OK;
}

int rtvla_prepare(rtvla_ctx* c, void* stream) { return prepare_impl(c, stream, false); }
int rtvla_prepare_with_tiles(rtvla_ctx* c, void* stream) { return prepare_impl(c, stream, true); }
size_t rtvla_tiled_bytes(const rtvla_ctx* c) { return c ? c->act_begin : 0; }
int rtvla_tile_layout_version(void) { return RTVLA_TILE_LAYOUT_VERSION; }

int rtvla_forward(rtvla_ctx* c, void* stream) {
    if (int rc = check_ready(c, true)) return rc;
    c->status = 0; c->launches = 0; c->kernels = 0;
    Sched(c, (hipStream_t)stream).forward();
    return c->status;
}

int rtvla_forward_stage(rtvla_ctx* c, int stage, int layer, int step, void* stream) {
    if (int rc = check_ready(c, true)) return rc;
    c->status = 0; c->launches = 0; c->kernels = 0;
    int rc = Sched(c, (hipStream_t)stream).stage(stage, layer, step);
    if (rc) return c->fail(rc, "bad stage / layer / step");
    return c->status;
}

int rtvla_graph_capture(rtvla_ctx* c, void* stream) {
    if (int rc = check_ready(c, true)) return rc;
    hipStream_t s = (hipStream_t)stream;
    // one eager run first: sets per-kernel attributes outside the capture and surfaces launch errors
    if (int rc = rtvla_forward(c, stream)) return rc;
    hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(c, e, "eager forward before capture");
    drop_graph(c);
    // the side stream and the events that fork / join the second branch (created once, outside the capture)
    if (!c->fork_stream && hipStreamCreateWithFlags(&c->fork_stream, hipStreamNonBlocking) != hipSuccess) return c->fail(RTVLA_ERR_DEVICE, "side stream");
    while ((int)c->fork_events.size() < c->d.llm_layers + 2) {
        hipEvent_t ev = nullptr;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) return c->fail(RTVLA_ERR_DEVICE, "hipEventCreate");
        c->fork_events.push_back(ev);
    }
    e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return hip_fail(c, e, "hipStreamBeginCapture");
    c->status = 0; c->launches = 0; c->kernels = 0;
    Sched sc(c, s);
    sc.forward(c->fork_stream, c->fork_events.data());
    e = hipStreamEndCapture(s, &c->graph);
    if (e != hipSuccess) return hip_fail(c, e, "hipStreamEndCapture");
    if (sc.fork_step0 != hipSuccess) return hip_fail(c, sc.fork_step0, "forking the first flow step");
    if (c->status) return c->status;
    e = hipGraphInstantiate(&c->exec, c->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) return hip_fail(c, e, "hipGraphInstantiate");
    return RTVLA_OK;
}

int rtvla_graph_launch(rtvla_ctx* c, void* stream) {
    if (!c) return RTVLA_ERR_ARG;
    if (!c->exec || !c->prepared) return c->fail(RTVLA_ERR_STATE, "no graph captured since the last rtvla_bind / rtvla_prepare");
    hipError_t e = hipGraphLaunch(c->exec, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(c, e, "hipGraphLaunch");
    return RTVLA_OK;
}

int rtvla_launch_count(const rtvla_ctx* c) { return c ? c->kernels : 0; }

// Both measurement helpers record their launches into a temporary HIP graph and time one replay of it with events on
// the stream: back-to-back eager launches of kernels that last a few microseconds would measure the host's launch
// rate, not the kernels, and the forward itself runs as a graph.
static int time_replay(rtvla_ctx* c, hipStream_t s, int stage, int layer, int step, int launch_index, int iters, float* mean_ms, int* enqueued_out) {
    if (!s) {
        // the null stream cannot be captured: finish what it holds, then launch and time on a stream of the context's own
        hipError_t e0 = hipStreamSynchronize(nullptr);
        if (e0 == hipSuccess && !c->timing_stream) e0 = hipStreamCreateWithFlags(&c->timing_stream, hipStreamNonBlocking);
        if (e0 != hipSuccess) return hip_fail(c, e0, "timing stream");
        s = c->timing_stream;
    }
    Sched sc(c, s);
    const bool cycle = layer == -1;
    const int n_layers = !cycle ? 1 : (stage == RTVLA_STAGE_VISION_LAYER ? c->d.vision_layers :
                                       (stage == RTVLA_STAGE_PREFIX_LAYER || stage == RTVLA_STAGE_SUFFIX_LAYER) ? c->d.llm_layers : 1);
    const int first = cycle ? 0 : layer;
    c->status = 0; c->only = launch_index; c->last_name.clear();
    c->launches = 0; c->kernels = 0;
    int rc = sc.stage(stage, first, step);      // eager warm-up: sets kernel attributes outside the capture, tells whether the index exists
    if (!rc && launch_index >= 0 && c->launches <= launch_index) rc = c->fail(RTVLA_ERR_ARG, "launch index past the end of the stage");
    if (rc) { c->only = -1; return rc; }
    hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) { c->only = -1; return hip_fail(c, e, "warm-up launch"); }
    hipGraph_t g = nullptr; hipGraphExec_t ge = nullptr;
    e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) { c->only = -1; return hip_fail(c, e, "hipStreamBeginCapture"); }
    int enqueued = 0;
    for (int i = 0; i < iters && !rc; ++i)
        for (int l = first; l < first + n_layers && !rc; ++l) {
            c->launches = 0; c->kernels = 0;
            rc = sc.stage(stage, l, step);
            enqueued += launch_index < 0 ? 1 : (c->launches > launch_index);          // (the last prefix layer has fewer launches)
        }
    e = hipStreamEndCapture(s, &g);
    c->only = -1;
    if (e != hipSuccess) return hip_fail(c, e, "hipStreamEndCapture");
    if (!rc && c->status) rc = c->status;
    if (!rc) { e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0); if (e != hipSuccess) rc = hip_fail(c, e, "hipGraphInstantiate"); }
    hipEvent_t a = nullptr, b = nullptr;
    if (!rc && (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess)) rc = c->fail(RTVLA_ERR_DEVICE, "hipEventCreate");
    if (!rc) {
        hipGraphLaunch(ge, s);                  // one untimed replay
        hipEventRecord(a, s);
        hipGraphLaunch(ge, s);
        hipEventRecord(b, s);
        e = hipEventSynchronize(b);
        if (e != hipSuccess) rc = hip_fail(c, e, "timed replay");
        else { float ms = 0.f; hipEventElapsedTime(&ms, a, b); *mean_ms = ms / (enqueued > 0 ? enqueued : 1); }
    }
    if (a) hipEventDestroy(a);
    if (b) hipEventDestroy(b);
    if (ge) hipGraphExecDestroy(ge);
    if (g) hipGraphDestroy(g);
    if (enqueued_out) *enqueued_out = enqueued;
    return rc;
}

int rtvla_time_stage(rtvla_ctx* c, int stage, int layer, int step, int iters, void* stream, float* mean_ms) {
    if (int rc = check_ready(c, true)) return rc;
    if (iters < 1 || !mean_ms) return RTVLA_ERR_ARG;
    // layer -1: every layer of the stage in turn (weights cold, as inside a forward), mean per layer
    return time_replay(c, (hipStream_t)stream, stage, layer, step, -1, iters, mean_ms, nullptr);
}

int rtvla_time_launch(rtvla_ctx* c, int stage, int layer, int step, int launch_index, int iters, void* stream,
                      float* mean_ms, char* name_out, size_t name_cap) {
    if (int rc = check_ready(c, true)) return rc;
    if (iters < 1 || !mean_ms || launch_index < 0) return RTVLA_ERR_ARG;
    // layer -1: one launch per layer in turn, so that every launch streams weights nobody has touched since the
    // previous pass (what the kernel sees inside a forward); otherwise the same layer over and over (cache-warm)
    const int rc = time_replay(c, (hipStream_t)stream, stage, layer, step, launch_index, iters, mean_ms, nullptr);
    if (name_out && name_cap) { strncpy(name_out, c->last_name.c_str(), name_cap - 1); name_out[name_cap - 1] = 0; }
    return rc;
}

int rtvla_time_forward(rtvla_ctx* c, int iters, void* stream, float* ms_out) {
    if (int rc = check_ready(c, true)) return rc;
    if (iters < 1 || !ms_out) return RTVLA_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    hipEvent_t a, b;
    if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return c->fail(RTVLA_ERR_DEVICE, "hipEventCreate");
    int rc = 0;
    for (int i = 0; i < iters && !rc; ++i) {
        hipEventRecord(a, s);
        rc = c->exec ? rtvla_graph_launch(c, stream) : rtvla_forward(c, stream);      // (a re-bind drops the graph)
        hipEventRecord(b, s);
        hipError_t e = hipEventSynchronize(b);
        if (e != hipSuccess) rc = hip_fail(c, e, "time_forward");
        else hipEventElapsedTime(&ms_out[i], a, b);
    }
    hipEventDestroy(a); hipEventDestroy(b);
    return rc;
}

// ---- unit-level linear layer on caller tensors (per-kernel parity tests) ----
namespace {
struct LinearPlan { size_t a_off, w_off, bias_off, part_off, total; int K128, tile, nsplit; bool skinny, partial; };

int plan_linear(int M, int K, int N, int tile, int nsplit, LinearPlan* pl) {
    if (M <= 0 || K <= 0 || N <= 0 || (K & 7) || (N & 15) || nsplit < 0 || nsplit > 8) return RTVLA_ERR_ARG;
    LinearPlan p{};
    p.skinny = tile == RTVLA_TILE_SKINNY;
    p.K128 = k32_padded(K) * 32;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    if (p.skinny) {
        if (M > 128 || (K != 1024 && K != 2048 && K != 4096) || nsplit > 1) return RTVLA_ERR_LIMIT;
        p.tile = tile; p.nsplit = 1;
        p.w_off = 0; p.bias_off = up(tiled_elems(K, N) * 2); p.total = p.bias_off + up((size_t)N * 2);
        *pl = p; return RTVLA_OK;
    }
    if (tile >= (int)TILE_COUNT || tile < -1) return RTVLA_ERR_ARG;
    TileChoice tc{tile, nsplit < 1 ? 1 : nsplit};
    if (tile < 0) {
        tc = choose_tile(M, n16_tiles(N), k32_padded(K) / 2, false, nsplit == 0, "linear");
        if (nsplit >= 1) tc.nsplit = nsplit;
    }
    p.tile = tc.tile; p.nsplit = tc.nsplit;
    p.partial = nsplit == 0 || tc.nsplit > 1;              // the residual-GEMM route: fp32 partials + reduce
    if (p.partial && N > 2048) return RTVLA_ERR_LIMIT;     // the reduce kernel handles rows of at most 2048 columns
    p.a_off = 0;
    p.w_off = up((size_t)M * p.K128 * 2);
    p.bias_off = p.w_off + up(tiled_elems_wide(K, N, 8) * 2);
    p.part_off = p.bias_off + up((size_t)N * 2);
    p.total = p.part_off + (p.partial ? up((size_t)p.nsplit * M * N * 4) : 0);
    *pl = p; return RTVLA_OK;
}
}  // namespace

size_t rtvla_linear_workspace_bytes(int M, int K, int N, int tile, int nsplit) {
    LinearPlan pl;
    return plan_linear(M, K, N, tile, nsplit, &pl) == RTVLA_OK ? pl.total : 0;
}

static int linear_impl(const void* x, int M, int K, const void* w, int N, const void* bias, void* out, void* workspace, size_t workspace_bytes,
                       int tile, int nsplit, hipStream_t s, int timed_iters, float* mean_ms) {
    if (!x || !w || !out || !workspace || ((uintptr_t)workspace & 255)) return RTVLA_ERR_ARG;
    LinearPlan pl;
    if (int rc = plan_linear(M, K, N, tile, nsplit, &pl)) return rc;
    if (workspace_bytes < pl.total) return RTVLA_ERR_SIZE;
    char* ws = (char*)workspace;
    bf16_t* zbias = (bf16_t*)(ws + pl.bias_off);
    launch_fill_zero(zbias, ((size_t)N * 2 + 255) & ~(size_t)255, s);
    const bf16_t* b = bias ? (const bf16_t*)bias : zbias;
    bf16_t* a = (bf16_t*)(ws + pl.a_off);
    bf16_t* wt = (bf16_t*)(ws + pl.w_off);
    // operands into the layouts the kernels read
    if (pl.skinny) launch_pretile((const bf16_t*)w, K, N, wt, 1, 0, s);
    else {
        launch_fill_zero(a, ((size_t)M * pl.K128 * 2 + 255) & ~(size_t)255, s);       // K is zero-padded to the 128-wide stage pair
        launch_copy_rows((const bf16_t*)x, K, a, pl.K128, M, K, s);
        launch_pretile((const bf16_t*)w, K, N, wt, 8, 1, s);
    }
    auto compute = [&]() -> int {
        if (pl.skinny) {
            SkinnyP p{};
            p.A = (const bf16_t*)x; p.lda = K; p.M = M; p.B0 = wt; p.K = K; p.N16 = n16_tiles(N); p.K32p = k32_padded(K);
            p.norm = SN_NONE; p.eps = 1e-6f; p.out = (bf16_t*)out; p.ldo = N; p.bias = b;
            if (K == 1024) return launch_skinny(p, SK_BIAS, s);
            // the K = 2048 / 4096 variants exist with the residual epilogue only (O and down projections): out = 0 + acc + bias
            launch_fill_zero(out, (size_t)M * N * 2, s);
            return launch_skinny(p, SK_RES, s);
        }
        GemmP p{};
        p.A = a; p.lda = pl.K128; p.a_rows = M; p.M = M; p.B0 = wt; p.bgroup = 8;
        p.N16 = n16_tiles(N); p.K32p = k32_padded(K); p.nsplit = pl.nsplit;
        if (!pl.partial) {
            p.out = (bf16_t*)out; p.ldo = N; p.bias = b;
            return launch_gemm(p, EPI_BIAS, pl.tile, s);
        }
        float* part = (float*)(ws + pl.part_off);
        p.partial = part; p.ldp = N; p.pstride = (size_t)M * N;
        if (int rc = launch_gemm(p, EPI_PARTIAL, pl.tile, s)) return rc;
        ReduceP r{};
        r.partial = part; r.pstride = p.pstride; r.ldp = N; r.nsplit = pl.nsplit; r.bias = b;
        r.x = (bf16_t*)out; r.ldx = N; r.M = M; r.N = N; r.norm = NORM_NONE;
        return launch_reduce(r, s);
    };
    int rc = compute();
    if (rc) return rc == 3 ? RTVLA_ERR_LIMIT : RTVLA_ERR_DEVICE;      // 3: this tile cannot take this K / split
    if (hipGetLastError() != hipSuccess) return RTVLA_ERR_DEVICE;
    if (timed_iters <= 0) return RTVLA_OK;
    // measurement: the compute launches alone, `timed_iters` times in a temporary graph, one untimed and one timed replay
    if (hipStreamSynchronize(s) != hipSuccess) return RTVLA_ERR_DEVICE;
    hipGraph_t g = nullptr; hipGraphExec_t ge = nullptr; hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal) != hipSuccess) return RTVLA_ERR_DEVICE;
    for (int i = 0; i < timed_iters && !rc; ++i) rc = compute();
    if (hipStreamEndCapture(s, &g) != hipSuccess || rc) rc = RTVLA_ERR_DEVICE;
    if (!rc && hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) != hipSuccess) rc = RTVLA_ERR_DEVICE;
    if (!rc && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = RTVLA_ERR_DEVICE;
    if (!rc) {
        hipGraphLaunch(ge, s);
        hipEventRecord(e0, s); hipGraphLaunch(ge, s); hipEventRecord(e1, s);
        if (hipEventSynchronize(e1) != hipSuccess) rc = RTVLA_ERR_DEVICE;
        else { float ms = 0.f; hipEventElapsedTime(&ms, e0, e1); *mean_ms = ms / timed_iters; }
    }
    if (e0) hipEventDestroy(e0);
    if (e1) hipEventDestroy(e1);
    if (ge) hipGraphExecDestroy(ge);
    if (g) hipGraphDestroy(g);
    return rc;
}

int rtvla_linear(const void* x, int M, int K, const void* w, int N, const void* bias, void* out, void* workspace, size_t workspace_bytes,
                 int tile, int nsplit, void* stream) {
    return linear_impl(x, M, K, w, N, bias, out, workspace, workspace_bytes, tile, nsplit, (hipStream_t)stream, 0, nullptr);
}

int rtvla_time_linear(const void* x, int M, int K, const void* w, int N, void* out, void* workspace, size_t workspace_bytes,
                      int tile, int nsplit, int iters, void* stream, float* mean_ms) {
    if (iters < 1 || !mean_ms || !stream) return RTVLA_ERR_ARG;      // (a graph cannot be captured on the null stream)
    return linear_impl(x, M, K, w, N, nullptr, out, workspace, workspace_bytes, tile, nsplit, (hipStream_t)stream, iters, mean_ms);
}

int rtvla_linear_tile_shape(int tile, int* rows, int* cols) {
    if (tile < 0 || tile >= (int)TILE_COUNT || !rows || !cols) return RTVLA_ERR_ARG;
    *rows = gemm_tile_bm(tile); *cols = gemm_tile_bn(tile);
    return RTVLA_OK;
}

// ---- unit-level fused GEMM epilogues and the reduce / normalise pass (per-kernel parity tests) ----
namespace {
struct ActPlan { size_t a_off, w0_off, w1_off, bias_off, scale_off, total; int K128, tile; bool dual; };

int plan_linear_act(int M, int K, int N, int act, int tile, ActPlan* out) {
    if (M <= 0 || K <= 0 || N <= 0 || (K & 7) || (N & 15)) return RTVLA_ERR_ARG;
    if (act != RTVLA_ACT_BIAS_GELU && act != RTVLA_ACT_GEGLU && act != RTVLA_ACT_SWIGLU) return RTVLA_ERR_ARG;
    if (tile < -1 || tile >= (int)TILE_COUNT) return RTVLA_ERR_ARG;
    ActPlan p{};
    p.dual = act != RTVLA_ACT_BIAS_GELU;
    p.K128 = k32_padded(K) * 32;
    p.tile = tile >= 0 ? tile : choose_tile(M, n16_tiles(N), k32_padded(K) / 2, p.dual, false, "linear act", p.dual ? 0 : 1).tile;
    if (p.dual && (gemm_tile_bn(p.tile) != 256 || gemm_tile_eight_waves(p.tile))) return RTVLA_ERR_LIMIT;      // gate and up share a 256-column workgroup tile
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const int G = p.dual ? 4 : 8;
    p.a_off = 0;
    p.w0_off = up((size_t)M * p.K128 * 2);
    p.w1_off = p.w0_off + up(tiled_elems_wide(K, N, G) * 2);
    p.bias_off = p.w1_off + (p.dual ? up(tiled_elems_wide(K, N, G) * 2) : 0);
    p.scale_off = p.bias_off + up((size_t)N * 2);
    p.total = p.scale_off + up((size_t)M * 4);
    *out = p;
    return RTVLA_OK;
}
}  // namespace

size_t rtvla_linear_act_workspace_bytes(int M, int K, int N, int act, int tile) {
    ActPlan pl;
    return plan_linear_act(M, K, N, act, tile, &pl) == RTVLA_OK ? pl.total : 0;
}

int rtvla_linear_act(const void* x, int M, int K, const void* w, const void* w_up, int N, const void* bias, int act, void* out, void* workspace,
                     size_t workspace_bytes, int tile, void* stream) {
    if (!x || !w || !out || !workspace || ((uintptr_t)workspace & 255)) return RTVLA_ERR_ARG;
    ActPlan pl;
    if (int rc = plan_linear_act(M, K, N, act, tile, &pl)) return rc;
    if (pl.dual != (w_up != nullptr)) return RTVLA_ERR_ARG;
    if (workspace_bytes < pl.total) return RTVLA_ERR_SIZE;
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    bf16_t* a = (bf16_t*)(ws + pl.a_off);
    launch_fill_zero(a, ((size_t)M * pl.K128 * 2 + 255) & ~(size_t)255, s);
    launch_copy_rows((const bf16_t*)x, K, a, pl.K128, M, K, s);
    const int G = pl.dual ? 4 : 8;
    launch_pretile((const bf16_t*)w, K, N, (bf16_t*)(ws + pl.w0_off), G, 1, s);
    if (pl.dual) launch_pretile((const bf16_t*)w_up, K, N, (bf16_t*)(ws + pl.w1_off), G, 1, s);
    bf16_t* zbias = (bf16_t*)(ws + pl.bias_off);
    launch_fill_zero(zbias, ((size_t)N * 2 + 255) & ~(size_t)255, s);
    GemmP p{};
    p.A = a; p.lda = pl.K128; p.a_rows = M; p.M = M; p.B0 = (bf16_t*)(ws + pl.w0_off); p.B1 = pl.dual ? (bf16_t*)(ws + pl.w1_off) : nullptr;
    p.bgroup = G; p.N16 = n16_tiles(N); p.K32p = k32_padded(K); p.nsplit = 1;
    p.out = (bf16_t*)out; p.ldo = N; p.bias = bias ? (const bf16_t*)bias : zbias;
    int epi = EPI_BIAS_GELU;
    if (act == RTVLA_ACT_GEGLU) epi = EPI_GEGLU;
    if (act == RTVLA_ACT_SWIGLU) {
        epi = EPI_SWIGLU;
        float* ones = (float*)(ws + pl.scale_off);                       // the SwiGLU epilogue multiplies by a per-row factor (DM0's RMS norm): 1 here
        launch_fill_f32(ones, M, 1.0f, s);
        p.rowscale = ones;
    }
    const int rc = launch_gemm(p, epi, pl.tile, s);
    if (rc) return (rc == 2 || rc == 3) ? RTVLA_ERR_LIMIT : RTVLA_ERR_DEVICE;
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

int rtvla_reduce_norm(const float* partials, int nsplit, int M, int N, const void* bias, const void* residual, int norm, const void* norm_w,
                      const void* norm_b, float eps, void* x_out, void* xn_out, void* stream) {
    if (M <= 0 || N <= 0 || (N & 3) || N > 2048) return RTVLA_ERR_ARG;
    if (nsplit < 0 || nsplit > 8 || nsplit == 5 || nsplit == 7) return RTVLA_ERR_ARG;
    if ((nsplit > 0 && !partials) || (nsplit == 0 && !residual) || (!x_out && !xn_out)) return RTVLA_ERR_ARG;
    if (norm != RTVLA_NORM_NONE && norm != RTVLA_NORM_RMS && norm != RTVLA_NORM_LAYER) return RTVLA_ERR_ARG;
    if (norm != RTVLA_NORM_NONE && !xn_out) return RTVLA_ERR_ARG;
    if (norm == RTVLA_NORM_LAYER && (!norm_w || !norm_b)) return RTVLA_ERR_ARG;
    ReduceP r{};
    r.partial = partials; r.pstride = (size_t)M * N; r.ldp = N; r.nsplit = nsplit;
    r.bias = (const bf16_t*)bias; r.res = (const bf16_t*)residual; r.ldr = N;
    r.x = (bf16_t*)x_out; r.ldx = N; r.xn = (bf16_t*)xn_out; r.ldxn = N;
    r.M = M; r.N = N; r.norm = norm == RTVLA_NORM_RMS ? NORM_RMS : norm == RTVLA_NORM_LAYER ? NORM_LAYER : NORM_NONE;
    r.nw = (const bf16_t*)norm_w; r.nb = (const bf16_t*)norm_b; r.eps = eps;
    if (launch_reduce(r, (hipStream_t)stream)) return RTVLA_ERR_DEVICE;
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

// ---- unit-level attention on caller tensors (per-kernel parity tests) ----
namespace {
struct AttnPlan { int hd, hd_pad, vd_pad, group, rows_pad, keys_pad, batch, nsplit; size_t q_off, k_off, vt_off, part_off, part_floats, total; };

int plan_attention(int kind, int tokens, int keys, int kv_heads, AttnPlan* out) {
    if (tokens <= 0 || keys <= 0 || kv_heads <= 0) return RTVLA_ERR_ARG;
    AttnPlan p{};
    p.batch = kv_heads; p.nsplit = 1;
    int seq_rows = tokens, seq_keys = keys;
    switch (kind) {
        case RTVLA_ATTN_GEMMA_PREFIX: case RTVLA_ATTN_GEMMA_SUFFIX: p.hd = p.hd_pad = p.vd_pad = 256; p.group = 8; if (kv_heads != 1) return RTVLA_ERR_LIMIT; break;
        case RTVLA_ATTN_GQA128_PREFIX: case RTVLA_ATTN_GQA128_SUFFIX: p.hd = p.hd_pad = p.vd_pad = 128; p.group = 2; break;
        case RTVLA_ATTN_VIT64: p.hd = p.hd_pad = p.vd_pad = 64; p.group = 1; if (keys != tokens) return RTVLA_ERR_LIMIT; break;
        case RTVLA_ATTN_SIGLIP:
            p.hd = 72; p.hd_pad = 96; p.vd_pad = 80; p.group = 1;
            if (kv_heads != 16 || keys != tokens || tokens % 256 || tokens > 4 * 256) return RTVLA_ERR_LIMIT;
            p.batch = 16 * (tokens / 256); seq_rows = seq_keys = 256;
            break;
        default: return RTVLA_ERR_ARG;
    }
    if (tokens > 16384 || keys > 16384 || kv_heads > 64) return RTVLA_ERR_LIMIT;
    const bool suffix = kind == RTVLA_ATTN_GEMMA_SUFFIX || kind == RTVLA_ATTN_GQA128_SUFFIX;
    if (suffix && tokens > 128) return RTVLA_ERR_LIMIT;                       // the action-expert passes hold at most 128 rows per head
    p.rows_pad = ((seq_rows * p.group + 127) / 128) * 128;
    p.keys_pad = ((seq_keys + 63) / 64) * 64;
    if (suffix) p.nsplit = std::min(16, (keys + 127) / 128);                 // as Sched::suffix_layer
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    p.q_off = 0;
    p.k_off = up((size_t)p.batch * p.rows_pad * p.hd_pad * 2);
    p.vt_off = p.k_off + up((size_t)p.batch * p.keys_pad * p.hd_pad * 2);
    p.part_off = p.vt_off + up((size_t)p.batch * p.vd_pad * p.keys_pad * 2);
    p.part_floats = p.nsplit > 1 ? (size_t)p.batch * ((seq_rows * p.group + 15) / 16) * p.nsplit * ((p.hd / 16) * 256 + 32) : 0;
    p.total = p.part_off + up(p.part_floats * 4);
    *out = p;
    return RTVLA_OK;
}
}  // namespace

size_t rtvla_attention_workspace_bytes(int kind, int tokens, int keys, int kv_heads) {
    AttnPlan pl;
    return plan_attention(kind, tokens, keys, kv_heads, &pl) == RTVLA_OK ? pl.total : 0;
}

int rtvla_attention(int kind, const void* q, const void* k, const void* v, void* out, int tokens, int keys, int kv_heads, float scale, int prefix_alloc,
                    const int32_t* valid_len_dev, int state_tokens, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !out || !workspace || ((uintptr_t)workspace & 255)) return RTVLA_ERR_ARG;
    AttnPlan pl;
    if (int rc = plan_attention(kind, tokens, keys, kv_heads, &pl)) return rc;
    if (workspace_bytes < pl.total) return RTVLA_ERR_SIZE;
    if (prefix_alloc < 0 || prefix_alloc > keys || state_tokens < 0 || state_tokens > tokens) return RTVLA_ERR_ARG;
    const bool masked = prefix_alloc < keys || valid_len_dev || state_tokens;
    if (masked && (kind == RTVLA_ATTN_VIT64 || kind == RTVLA_ATTN_SIGLIP)) return RTVLA_ERR_LIMIT;      // the vision kernels take no masks
    if (kind == RTVLA_ATTN_SIGLIP && fabsf(scale - 0.11785113019775792f) > 1e-6f) return RTVLA_ERR_LIMIT;   // 72^-1/2 is built into that kernel
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    bf16_t* qt = (bf16_t*)(ws + pl.q_off); bf16_t* kt = (bf16_t*)(ws + pl.k_off); bf16_t* vtt = (bf16_t*)(ws + pl.vt_off);
    launch_fill_zero(ws, pl.part_off, s);
    const size_t qb = (size_t)pl.rows_pad * pl.hd_pad, kb = (size_t)pl.keys_pad * pl.hd_pad, vb = (size_t)pl.vd_pad * pl.keys_pad;
    launch_attn_tile_operands((const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, qt, kt, vtt, tokens, keys, kv_heads, pl.group, pl.hd, pl.hd_pad, qb, kb, vb,
                              pl.keys_pad, kind == RTVLA_ATTN_SIGLIP ? 256 : 0, s);
    int rc = 0;
    if (kind == RTVLA_ATTN_SIGLIP) {
        launch_vision_attention(qt, kt, vtt, (bf16_t*)out, tokens / 256, s);
    } else {
        AttnP a{};
        a.q = qt; a.k = kt; a.vt = vtt; a.ldvt = pl.keys_pad;
        a.batch = kv_heads; a.q_bstride = qb; a.k_bstride = kb; a.vt_bstride = vb;
        a.group = pl.group; a.rows = pl.group * tokens; a.keys = keys; a.scale = scale;
        a.out = (bf16_t*)out; a.ld_tok = kv_heads * pl.group * pl.hd; a.batch_inner = kv_heads; a.out_istride = (size_t)pl.group * pl.hd;
        a.prefix_alloc = prefix_alloc; a.valid_len = valid_len_dev; a.state_rows = state_tokens * pl.group;
        a.causal = kind == RTVLA_ATTN_GQA128_PREFIX;
        a.nsplit = pl.nsplit; a.partial = (float*)(ws + pl.part_off); a.partial_floats = pl.part_floats;
        switch (kind) {
            case RTVLA_ATTN_GEMMA_PREFIX:  rc = launch_mqa_attention(a, ATTN_PREFIX, s); break;
            case RTVLA_ATTN_GEMMA_SUFFIX:  rc = launch_mqa_attention(a, ATTN_SUFFIX, s); break;
            case RTVLA_ATTN_GQA128_PREFIX: rc = launch_mqa_attention(a, ATTN_GQA128_PREFIX, s); break;
            case RTVLA_ATTN_GQA128_SUFFIX: rc = launch_mqa_attention(a, ATTN_GQA128_SUFFIX, s); break;
            case RTVLA_ATTN_VIT64:         rc = launch_flash_attention(a, 64, s); break;
        }
    }
    if (rc) return rc == 3 ? RTVLA_ERR_LIMIT : RTVLA_ERR_DEVICE;
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

size_t rtvla_pretile_elems(int K, int N) { return (K > 0 && N > 0) ? tiled_elems(K, N) : 0; }

int rtvla_pretile(const void* w, int K, int N, void* w_tiled, void* stream) {
    if (!w || !w_tiled || K <= 0 || N <= 0) return RTVLA_ERR_ARG;
    launch_pretile((const bf16_t*)w, K, N, (bf16_t*)w_tiled, 1, 0, (hipStream_t)stream);
    return hipGetLastError() == hipSuccess ? RTVLA_OK : RTVLA_ERR_DEVICE;
}

}  // extern "C"
