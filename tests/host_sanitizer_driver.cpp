// Host-side exercise of the C ABI (include/rtvla.h) for a build whose host code carries AddressSanitizer and
// UndefinedBehaviorSanitizer: context tables, binding, workspace layout, size planning and every error path that
// returns before a device is touched.  No kernel is launched and no GPU is needed; pointers handed to rtvla_bind are
// never dereferenced by the library.  Built and run by tests/test_host_sanitizer.py.
#include "../include/rtvla.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { fprintf(stderr, "CHECK failed at line %d: %s\n", __LINE__, #cond); ++failures; } } while (0)

static rtvla_ctx* make(int model, int views, int prompt, int chunk, int steps = 10, int vl = 27, int ll = 18, int* rc_out = nullptr) {
    rtvla_dims d{model, views, prompt, chunk, steps, vl, ll};
    rtvla_ctx* c = nullptr;
    const int rc = rtvla_create(&d, &c);
    if (rc_out) *rc_out = rc;
    return c;
}

static void walk_tables(rtvla_ctx* c) {
    // every tensor and buffer record, with and without output pointers
    const int nt = rtvla_tensor_count(c);
    CHECK(nt > 0);
    for (int i = -1; i <= nt; ++i) {
        const char* name = nullptr; int32_t elem = 0, rank = 0, w = 0, req = 0; int64_t shape[4];
        const int rc = rtvla_tensor_info(c, i, &name, &elem, &rank, shape, &w, &req);
        CHECK((rc == RTVLA_OK) == (i >= 0 && i < nt));
        if (rc == RTVLA_OK) { CHECK(name && strlen(name) > 0 && rank >= 1 && rank <= 4 && (elem == 2 || elem == 4)); }
        rtvla_tensor_info(c, i, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
    }
    const int nb = rtvla_buffer_count(c);
    CHECK(nb > 0);
    size_t end_max = 0;
    for (int i = -1; i <= nb; ++i) {
        const char* name = nullptr; size_t off = 0; int64_t rows = 0, cols = 0, ld = 0; int32_t elem = 0;
        const int rc = rtvla_buffer_info(c, i, &name, &off, &rows, &cols, &ld, &elem);
        CHECK((rc == RTVLA_OK) == (i >= 0 && i < nb));
        if (rc == RTVLA_OK) { CHECK(off % 256 == 0 && cols <= ld); end_max = std::max(end_max, off + (size_t)rows * ld * elem); }
        rtvla_buffer_info(c, i, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
    }
    CHECK(end_max <= rtvla_workspace_bytes(c));
    CHECK(rtvla_tiled_bytes(c) > 0 && rtvla_tiled_bytes(c) < rtvla_workspace_bytes(c));
}

static void bind_everything_with_fake_pointers(rtvla_ctx* c) {
    // the library stores the pointers; nothing here makes it read through them
    const int nt = rtvla_tensor_count(c);
    for (int i = 0; i < nt; ++i) {
        const char* name = nullptr; int32_t elem = 0, rank = 0, w = 0, req = 0; int64_t shape[4];
        CHECK(rtvla_tensor_info(c, i, &name, &elem, &rank, shape, &w, &req) == RTVLA_OK);
        size_t bytes = elem; for (int k = 0; k < rank; ++k) bytes *= (size_t)shape[k];
        const std::string n(name);
        CHECK(rtvla_bind(c, n.c_str(), bytes ? (void*)(uintptr_t)(4096 + 256 * i) : nullptr, bytes) == RTVLA_OK);
        if (bytes) {
            CHECK(rtvla_bind(c, n.c_str(), (void*)(uintptr_t)4096, bytes + 2) == RTVLA_ERR_SIZE || n == "embedding_weight" || n == "vision_embed_tokens_w");
            CHECK(strstr(rtvla_last_error(c), n.c_str()) != nullptr || n == "embedding_weight" || n == "vision_embed_tokens_w");
            CHECK(rtvla_bind(c, n.c_str(), (void*)(uintptr_t)4097, bytes) == RTVLA_ERR_ARG);
            CHECK(rtvla_bind(c, n.c_str(), nullptr, bytes) == RTVLA_ERR_ARG);
        }
    }
}

int main() {
    CHECK(rtvla_version() >= 1 && rtvla_tile_layout_version() >= 1);
    // ---- create: argument and limit checks ----
    int rc = 0;
    CHECK(rtvla_create(nullptr, nullptr) == RTVLA_ERR_ARG);
    { rtvla_dims d{0, 1, 0, 50, 10, 27, 18}; CHECK(rtvla_create(&d, nullptr) == RTVLA_ERR_ARG); }
    const int bad[][4] = {{0, 0, 0, 50}, {0, 5, 0, 50}, {0, 1, -1, 50}, {0, 1, 0, 0}, {3, 1, 0, 50}, {-1, 1, 0, 50}, {2, 0, 10, 50}};
    for (auto& b : bad) { rtvla_ctx* c = make(b[0], b[1], b[2], b[3], 10, 27, 18, &rc); CHECK(!c && rc == RTVLA_ERR_ARG); }
    { rtvla_ctx* c = make(RTVLA_PI0, 1, 0, 128, 10, 27, 18, &rc); CHECK(!c && rc == RTVLA_ERR_LIMIT); }
    { rtvla_ctx* c = make(RTVLA_DM0, 1, 10, 65, 10, 23, 28, &rc); CHECK(!c && rc == RTVLA_ERR_LIMIT); }
    { rtvla_ctx* c = make(RTVLA_PI0, 1, 0, 50, 7, 27, 18, &rc); CHECK(!c && rc == RTVLA_ERR_LIMIT); }
    { rtvla_ctx* c = make(RTVLA_PI05, 1, 8, 50, 11, 27, 18, &rc); CHECK(!c && rc == RTVLA_ERR_LIMIT); }
    { rtvla_ctx* c = make(RTVLA_PI0, 1, 4097, 50, 10, 27, 18, &rc); CHECK(!c && rc == RTVLA_ERR_LIMIT); }
    { rtvla_ctx* c = make(RTVLA_PI0, 1, 0, 50, 10, 0, 18, &rc); CHECK(!c && rc == RTVLA_ERR_ARG); }

    // ---- tables of every model kind, smallest and largest shapes ----
    const int shapes[][7] = {{RTVLA_PI0, 1, 0, 1, 10, 1, 1},   {RTVLA_PI0, 3, 20, 50, 10, 27, 18},  {RTVLA_PI0, 4, 4096, 127, 10, 27, 18},
                             {RTVLA_PI05, 1, 1, 1, 1, 1, 1},   {RTVLA_PI05, 3, 52, 50, 10, 27, 18}, {RTVLA_PI05, 4, 4096, 128, 10, 27, 18},
                             {RTVLA_DM0, 1, 0, 1, 10, 1, 1},   {RTVLA_DM0, 3, 100, 50, 10, 23, 28}, {RTVLA_DM0, 4, 4096, 64, 10, 23, 28}};
    for (auto& sh : shapes) {
        rtvla_ctx* c = make(sh[0], sh[1], sh[2], sh[3], sh[4], sh[5], sh[6], &rc);
        CHECK(c && rc == RTVLA_OK);
        if (!c) continue;
        walk_tables(c);
        // out-of-order calls: nothing bound yet
        CHECK(rtvla_prepare(c, nullptr) == RTVLA_ERR_STATE);
        CHECK(rtvla_forward(c, nullptr) == RTVLA_ERR_STATE);
        CHECK(rtvla_graph_launch(c, nullptr) == RTVLA_ERR_STATE);
        CHECK(rtvla_bind_workspace(c, (void*)(uintptr_t)4096, 1024) == RTVLA_ERR_SIZE);
        CHECK(rtvla_bind_workspace(c, (void*)(uintptr_t)4100, rtvla_workspace_bytes(c)) == RTVLA_ERR_ARG);
        CHECK(rtvla_bind_workspace(c, nullptr, rtvla_workspace_bytes(c)) == RTVLA_ERR_ARG);
        CHECK(rtvla_bind_workspace(c, (void*)(uintptr_t)(1 << 20), rtvla_workspace_bytes(c)) == RTVLA_OK);
        CHECK(rtvla_forward(c, nullptr) == RTVLA_ERR_UNBOUND && strlen(rtvla_last_error(c)) > 0);
        CHECK(rtvla_bind(c, "no_such_tensor", (void*)(uintptr_t)4096, 16) == RTVLA_ERR_NAME);
        CHECK(strstr(rtvla_last_error(c), "no_such_tensor") != nullptr);
        CHECK(rtvla_bind(c, nullptr, (void*)(uintptr_t)4096, 16) == RTVLA_ERR_ARG);
        CHECK(rtvla_bind(c, std::string(5000, 'x').c_str(), (void*)(uintptr_t)4096, 16) == RTVLA_ERR_NAME);
        bind_everything_with_fake_pointers(c);
        CHECK(rtvla_forward(c, nullptr) == RTVLA_ERR_STATE);            // bound but not prepared
        CHECK(rtvla_forward_stage(c, 99, 0, 0, nullptr) == RTVLA_ERR_STATE);
        float ms = 0.f; char name[8];
        CHECK(rtvla_time_stage(c, RTVLA_STAGE_PREFIX_LAYER, 0, 0, 1, nullptr, &ms) == RTVLA_ERR_STATE);
        CHECK(rtvla_time_launch(c, RTVLA_STAGE_PREFIX_LAYER, 0, 0, 0, 1, nullptr, &ms, name, sizeof name) == RTVLA_ERR_STATE);
        CHECK(rtvla_time_forward(c, 1, nullptr, &ms) == RTVLA_ERR_STATE);
        CHECK(rtvla_launch_count(c) == 0);
        CHECK(rtvla_destroy(c) == RTVLA_OK);
    }
    CHECK(rtvla_destroy(nullptr) == RTVLA_ERR_ARG && rtvla_forward(nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_tensor_count(nullptr) == 0 && rtvla_buffer_count(nullptr) == 0 && rtvla_workspace_bytes(nullptr) == 0);
    CHECK(strlen(rtvla_last_error(nullptr)) > 0);

    // ---- size planning of the unit-level entry points ----
    for (int M : {1, 16, 51, 128, 129, 768, 788, 8115})
        for (int K : {8, 12, 588, 1024, 1152, 2048, 4096, 4304, 16384})
            for (int N : {16, 24, 32, 1024, 1152, 2048, 4304 - 4304 % 16, 16384})
                for (int tile = -2; tile <= 13; ++tile)
                    for (int ns : {-1, 0, 1, 2, 4, 8, 9}) {
                        const size_t b = rtvla_linear_workspace_bytes(M, K, N, tile, ns);
                        if ((K & 7) || (N & 15) || ns < 0 || ns > 8 || tile > 11) CHECK(b == 0);
                        if (b) CHECK(b >= (size_t)N * 2 && b < ((size_t)64 << 30));
                    }
    CHECK(rtvla_linear_workspace_bytes(129, 1024, 64, -2, 1) == 0);
    void* p = (void*)(uintptr_t)4096;
    CHECK(rtvla_linear(p, 16, 128, p, 16, nullptr, p, p, 16, -1, 1, nullptr) == RTVLA_ERR_SIZE);
    CHECK(rtvla_linear(nullptr, 16, 128, p, 16, nullptr, p, p, (size_t)1 << 20, -1, 1, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_linear(p, 16, 128, p, 16, nullptr, p, (void*)(uintptr_t)4100, (size_t)1 << 20, -1, 1, nullptr) == RTVLA_ERR_ARG);
    for (int tile = -3; tile < 16; ++tile) { int r = 0, cc = 0; const int st = rtvla_linear_tile_shape(tile, &r, &cc); if (st == RTVLA_OK) CHECK(r >= 64 && cc >= 128); }
    CHECK(rtvla_linear_tile_shape(0, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_pretile_elems(588, 1152) == (size_t)72 * 20 * 512 && rtvla_pretile_elems(0, 16) == 0 && rtvla_pretile_elems(16, -1) == 0);
    CHECK(rtvla_pretile(nullptr, 16, 16, p, nullptr) == RTVLA_ERR_ARG);
    // ---- fused epilogues and the reduce pass: planning and argument checks ----
    for (int act = 0; act <= 4; ++act)
        for (int tile = -2; tile <= 13; ++tile)
            for (int N : {16, 24, 272, 4304 - 4304 % 16, 16384}) {
                const size_t b = rtvla_linear_act_workspace_bytes(788, 2048, N, act, tile);
                if (act < 1 || act > 3 || tile < -1 || tile > 11 || (N & 15)) CHECK(b == 0);
                if (b) CHECK(b >= (size_t)788 * 2048 * 2);
            }
    CHECK(rtvla_linear_act(p, 788, 2048, p, nullptr, 16384, nullptr, RTVLA_ACT_GEGLU, p, p, (size_t)1 << 32, -1, nullptr) == RTVLA_ERR_ARG);     // gated without w_up
    CHECK(rtvla_linear_act(p, 788, 2048, p, p, 16384, nullptr, RTVLA_ACT_GEGLU, p, p, 16, -1, nullptr) == RTVLA_ERR_SIZE);
    CHECK(rtvla_reduce_norm(nullptr, 2, 16, 64, nullptr, nullptr, 0, nullptr, nullptr, 1e-6f, p, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_reduce_norm((const float*)p, 5, 16, 64, nullptr, nullptr, 0, nullptr, nullptr, 1e-6f, p, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_reduce_norm((const float*)p, 2, 16, 4096, nullptr, nullptr, 0, nullptr, nullptr, 1e-6f, p, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_reduce_norm((const float*)p, 2, 16, 64, nullptr, nullptr, RTVLA_NORM_LAYER, nullptr, nullptr, 1e-5f, p, p, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_reduce_norm((const float*)p, 2, 16, 64, nullptr, nullptr, RTVLA_NORM_RMS, nullptr, nullptr, 1e-6f, p, nullptr, nullptr) == RTVLA_ERR_ARG);
    // ---- unit-level attention: planning and argument checks ----
    for (int kind = -1; kind <= 6; ++kind)
        for (int tokens : {0, 1, 51, 128, 129, 256, 768, 2705, 20000})
            for (int keys : {0, 1, 33, 256, 768, 839, 2277, 2705})
                for (int heads : {0, 1, 8, 16, 65}) {
                    const size_t b = rtvla_attention_workspace_bytes(kind, tokens, keys, heads);
                    if (kind < 0 || kind > 5 || tokens <= 0 || keys <= 0 || heads <= 0 || heads > 64 || tokens > 16384) CHECK(b == 0);
                    if (b) CHECK(b >= (size_t)keys * heads * 64 * 2 && b < ((size_t)8 << 30));
                }
    CHECK(rtvla_attention_workspace_bytes(RTVLA_ATTN_GEMMA_SUFFIX, 129, 900, 1) == 0);
    CHECK(rtvla_attention_workspace_bytes(RTVLA_ATTN_GEMMA_PREFIX, 788, 788, 2) == 0);
    CHECK(rtvla_attention_workspace_bytes(RTVLA_ATTN_SIGLIP, 768, 768, 16) > 0 && rtvla_attention_workspace_bytes(RTVLA_ATTN_SIGLIP, 700, 700, 16) == 0);
    CHECK(rtvla_attention(RTVLA_ATTN_GEMMA_PREFIX, p, p, p, p, 788, 788, 1, 0.0625f, 788, nullptr, 0, p, 16, nullptr) == RTVLA_ERR_SIZE);
    CHECK(rtvla_attention(RTVLA_ATTN_GEMMA_PREFIX, nullptr, p, p, p, 788, 788, 1, 0.0625f, 788, nullptr, 0, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_attention(RTVLA_ATTN_GEMMA_SUFFIX, p, p, p, p, 51, 839, 1, 0.0625f, 900, nullptr, 1, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_attention(RTVLA_ATTN_VIT64, p, p, p, p, 100, 100, 4, 0.125f, 50, nullptr, 0, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_LIMIT);
    CHECK(rtvla_attention(RTVLA_ATTN_SIGLIP, p, p, p, p, 256, 256, 16, 0.5f, 256, nullptr, 0, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_LIMIT);
    // ---- pre-/post-processing: argument and size checks come before any launch ----
    CHECK(rtvla_preprocess_image_scratch(0, 10) == 0 && rtvla_preprocess_image_scratch(480, 640) >= (size_t)480 * 224 * 3);
    CHECK(rtvla_preprocess_image(nullptr, 480, 640, p, p, 1 << 20, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_preprocess_image(p, 480, 640, p, nullptr, 1 << 20, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_preprocess_image(p, 480, 640, p, p, 16, nullptr) == RTVLA_ERR_SIZE);
    CHECK(rtvla_preprocess_image(p, 100000, 8, p, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_LIMIT || rtvla_preprocess_image(p, 100000, 8, p, p, (size_t)1 << 30, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_preprocess_image_static(p, 2400, 2400, p, nullptr) == RTVLA_ERR_LIMIT);
    CHECK(rtvla_preprocess_image_static(p, -1, 2400, p, nullptr) == RTVLA_ERR_ARG);
    double st[40] = {0};
    CHECK(rtvla_preprocess_state(st, 33, st, st, 7, 0, p, nullptr, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_preprocess_state(st, 7, st, st, 7, 2, p, nullptr, nullptr, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_postprocess_actions(p, 50, st, st, 7, 0, st, 33, st, nullptr) == RTVLA_ERR_ARG);
    CHECK(rtvla_postprocess_actions(p, 0, st, st, 7, 0, st, 7, st, nullptr) == RTVLA_ERR_ARG);
    if (failures) { fprintf(stderr, "%d check(s) failed\n", failures); return 1; }
    printf("host sanitizer driver: all checks passed\n");
    return 0;
}
