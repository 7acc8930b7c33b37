"""Per-kernel GPU parity through the C ABI: the large-M MFMA GEMM (every block tile, with and without split-K) and the
action-expert weight-streaming kernel on the shapes the models produce and on ragged ones, against torch.matmul in
fp32 on the same bf16 operands.  Tolerance: the result is one bf16 rounding of an fp32 sum whose order differs from
the checker's, so single-ulp flips are expected and nothing more: relative L2 <= 3e-3, and every element within
one bf16 spacing (2^-7 relative) plus 1e-3 of the output's RMS for the elements that cancel to nearly zero."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
_P = ctypes.c_void_p
REL_TOL = 3e-3


def _run(lib, capi, M, K, N, tile, nsplit, bias=True, seed=0):
    g = torch.Generator(device="cuda:0").manual_seed(seed * 7919 + M + K + N)
    x = torch.randn(M, K, device="cuda:0", generator=g).to(torch.bfloat16)
    w = (torch.randn(K, N, device="cuda:0", generator=g) * 0.05).to(torch.bfloat16)
    b = torch.randn(N, device="cuda:0", generator=g).to(torch.bfloat16) if bias else None
    need = lib.rtvla_linear_workspace_bytes(M, K, N, tile, nsplit)
    if need == 0:
        return None
    ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
    out = torch.full((M, N), 77.0, dtype=torch.bfloat16, device="cuda:0")
    rc = lib.rtvla_linear(_P(x.data_ptr()), M, K, _P(w.data_ptr()), N, _P(b.data_ptr()) if bias else None, _P(out.data_ptr()),
                          _P(ws.data_ptr()), need, tile, nsplit, _P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    if rc == capi.ERR_LIMIT:
        return None
    assert rc == 0, rc
    ref = x.float() @ w.float()
    if bias:
        ref = ref + b.float()
    got = out.float()
    rel = ((got - ref).norm() / ref.norm()).item()
    excess = (got - ref).abs() / (ref.abs() * 2.0 ** -7 + 1e-3 * ref.pow(2).mean().sqrt())
    return rel, excess.max().item()


def _tiles(lib):
    out, r, c = [], ctypes.c_int(), ctypes.c_int()
    t = 0
    while lib.rtvla_linear_tile_shape(t, ctypes.byref(r), ctypes.byref(c)) == 0:
        out.append((t, r.value, c.value)); t += 1
    return out


@pytest.mark.parametrize("M,K,N", [
    (768, 1152, 3456),      # SigLIP QKV
    (768, 1152, 1152),      # SigLIP O
    (768, 1152, 4304),      # SigLIP up (N = 16 * 269)
    (768, 4304, 1152),      # SigLIP down (K padded to 4352)
    (788, 2048, 2560),      # Gemma prefix QKV at the headline shape
    (788, 2048, 2048),      # prefix O
    (968, 2048, 2048),      # 968-token prefix
    (256, 1152, 2048),      # projector, one view
    (37, 136, 48),          # ragged everything: one partial row tile, K below one stage pair, three column tiles
    (225, 264, 272),        # one row past the largest tile, ragged K and N
])
def test_mfma_gemm_every_tile_and_split_against_fp32_matmul(M, K, N):
    import rtvla_capi as capi
    lib = capi.load()
    tiles = _tiles(lib)
    assert len(tiles) >= 4
    ran = 0
    for tile, rows, cols in tiles:
        for nsplit in (1, 2, 3, 4, 8):
            if nsplit > 1 and N > 2048:
                continue
            res = _run(lib, capi, M, K, N, tile, nsplit)
            if res is None:
                continue                                   # this tile cannot take this K / split (reported as RTVLA_ERR_LIMIT)
            ran += 1
            assert res[0] <= REL_TOL and res[1] <= 1.01, ("tile %dx%d split %d" % (rows, cols, nsplit), res)
    assert ran >= 4
    # the forward's own choice for this shape, one pass and through the partial + reduce route
    for nsplit in (1, 0):
        if nsplit == 0 and N > 2048:
            continue
        res = _run(lib, capi, M, K, N, capi.TILE_AUTO, nsplit, bias=(nsplit == 1))
        assert res is not None and res[0] <= REL_TOL and res[1] <= 1.01, (nsplit, res)


@pytest.mark.parametrize("M,K,N", [(51, 1024, 2560), (51, 2048, 1024), (51, 4096, 1024), (64, 1024, 4096), (1, 1024, 1024), (17, 2048, 48),
                                   (101, 1024, 2560), (128, 4096, 1024), (65, 2048, 1024)])      # (the last three: two 64-row blocks / up to eight 16-row blocks)
def test_weight_streaming_kernel_against_fp32_matmul(M, K, N):
    import rtvla_capi as capi
    lib = capi.load()
    res = _run(lib, capi, M, K, N, capi.TILE_SKINNY, 1)
    assert res is not None and res[0] <= REL_TOL and res[1] <= 1.01, res


def test_unit_entry_rejects_what_it_cannot_run():
    import rtvla_capi as capi
    lib = capi.load()
    assert lib.rtvla_linear_workspace_bytes(16, 12, 16, -1, 1) == 0          # K not a multiple of 8
    assert lib.rtvla_linear_workspace_bytes(16, 16, 24, -1, 1) == 0          # N not a multiple of 16
    assert lib.rtvla_linear_workspace_bytes(129, 1024, 64, capi.TILE_SKINNY, 1) == 0
    assert lib.rtvla_linear_workspace_bytes(16, 512, 64, capi.TILE_SKINNY, 1) == 0
    assert lib.rtvla_linear_workspace_bytes(64, 128, 4096, 0, 2) == 0        # split-K rows wider than the reduce kernel takes
    x = torch.zeros(16, 128, dtype=torch.bfloat16, device="cuda:0")
    ws = torch.empty(256, dtype=torch.uint8, device="cuda:0")
    rc = lib.rtvla_linear(_P(x.data_ptr()), 16, 128, _P(x.data_ptr()), 16, None, _P(x.data_ptr()), _P(ws.data_ptr()), 256, -1, 1, None)
    assert rc == capi.ERR_SIZE


def test_a_graph_captured_before_a_rebind_is_refused():
    """rtvla_bind after rtvla_graph_capture drops the graph: replaying it would read the old addresses."""
    import synthetic as syn
    import rtvla_capi as capi
    from pi0_infer import Pi0Inference
    ck = syn.pi0_checkpoint(5, 2, "cuda:0", 1, 1)
    img, state, noise = syn.observation(5, 1, 8, "cuda:0")
    m = Pi0Inference(ck, 1, 8)
    a = m.forward(img, state, noise).clone()
    ctx, stream = m._engine.ctx, torch.cuda.current_stream().cuda_stream
    other = torch.zeros_like(m.buffers["diffusion_noise"])
    ctx.bind("diffusion_noise", other.data_ptr(), other.numel() * 2)
    with pytest.raises(capi.RtvlaError) as e:
        ctx.graph_launch(stream)
    assert e.value.code == capi.ERR_STATE
    with pytest.raises(capi.RtvlaError):
        ctx.forward(stream)                                  # not prepared either
    m.buffers["diffusion_noise"] = other
    m._engine.prepare()
    m.record_infer_graph()
    b = m.forward(img, state, noise)
    assert b.data_ptr() == other.data_ptr() and torch.equal(a, b)


# ---------------------------------------------------------------------------------------------------------
# fused GEMM epilogues with a row-major output, and the reduce / normalise pass, each on its own
def _gelu_tanh(a):
    return a * torch.sigmoid(1.5957691216057308 * a * (1.0 + 0.044715 * a * a))


def _run_act(lib, capi, M, K, N, act, tile, seed=0):
    g = torch.Generator(device="cuda:0").manual_seed(seed * 104729 + M + K + N + act)
    x = torch.randn(M, K, device="cuda:0", generator=g).to(torch.bfloat16)
    w = (torch.randn(K, N, device="cuda:0", generator=g) * 0.05).to(torch.bfloat16)
    dual = act != capi.ACT_BIAS_GELU
    w2 = (torch.randn(K, N, device="cuda:0", generator=g) * 0.05).to(torch.bfloat16) if dual else None
    b = None if dual else torch.randn(N, device="cuda:0", generator=g).to(torch.bfloat16)
    need = lib.rtvla_linear_act_workspace_bytes(M, K, N, act, tile)
    if need == 0:
        return None
    ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
    out = torch.full((M, N), 77.0, dtype=torch.bfloat16, device="cuda:0")
    rc = lib.rtvla_linear_act(_P(x.data_ptr()), M, K, _P(w.data_ptr()), _P(w2.data_ptr()) if dual else None, N, _P(b.data_ptr()) if b is not None else None,
                              act, _P(out.data_ptr()), _P(ws.data_ptr()), need, tile, _P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    if rc == capi.ERR_LIMIT:
        return None
    assert rc == 0, rc
    a = x.float() @ w.float()
    if act == capi.ACT_BIAS_GELU:
        ref = _gelu_tanh(a + b.float())
    elif act == capi.ACT_GEGLU:
        ref = _gelu_tanh(a) * (x.float() @ w2.float())
    else:
        ref = a * torch.sigmoid(a) * (x.float() @ w2.float())
    got = out.float()
    rel = ((got - ref).norm() / ref.norm()).item()
    excess = (got - ref).abs() / (ref.abs() * 2.0 ** -7 + 2e-3 * ref.pow(2).mean().sqrt())      # (the activations use the hardware exp2 / rcp)
    return rel, excess.max().item()


@pytest.mark.parametrize("M,K,N,act", [
    (768, 1152, 4304, 1),       # SigLIP up-projection: bias + GELU
    (788, 2048, 16384, 2),      # Gemma prefix gate / up: GeGLU, 25 row tiles in mixed blocks
    (607, 2048, 6144, 3),       # DM0 prefix gate / up: SwiGLU
    (8115, 1024, 4096, 1),      # DM0 ViT fc: bias + GELU on the eight-wave tile
    (37, 136, 48, 1), (37, 136, 48, 2), (225, 264, 272, 3),      # ragged rows, K and columns
])
def test_fused_activation_epilogues_against_fp32(M, K, N, act):
    import rtvla_capi as capi
    lib = capi.load()
    ran = 0
    for tile, rows, cols in [(capi.TILE_AUTO, 0, 0)] + _tiles(lib):
        if M > 1000 and tile != capi.TILE_AUTO and rows < 128:
            continue                                        # (keeps the 8115-row case short)
        res = _run_act(lib, capi, M, K, N, act, tile)
        if res is None:
            continue                                        # a gated epilogue needs a 256-column tile; the large tiles need an even stage count
        ran += 1
        assert res[0] <= REL_TOL and res[1] <= 1.01, ("tile %dx%d" % (rows, cols), res)
    assert ran >= 3


@pytest.mark.parametrize("M,N,nsplit,norm,has_bias,has_res", [
    (768, 1152, 2, 2, True, True),        # SigLIP O projection: split 2 + bias + residual + LayerNorm
    (768, 1152, 4, 2, True, True),        # SigLIP down projection
    (768, 1152, 0, 2, False, True),       # LayerNorm of a stream alone (first layer)
    (788, 2048, 1, 1, False, True),       # prefix O projection: one partial + residual + RMS norm
    (788, 2048, 4, 1, False, True),       # prefix down projection
    (968, 2048, 8, 1, False, True), (33, 2048, 6, 1, True, False), (5, 1024, 3, 0, True, True), (2705, 1024, 1, 2, True, True),
])
def test_reduce_bias_residual_norm_against_fp32(M, N, nsplit, norm, has_bias, has_res):
    import rtvla_capi as capi
    lib = capi.load()
    g = torch.Generator(device="cuda:0").manual_seed(M * 31 + N + nsplit)
    parts = torch.randn(max(nsplit, 1), M, N, device="cuda:0", generator=g)
    bias = torch.randn(N, device="cuda:0", generator=g).bfloat16() if has_bias else None
    res = (torch.randn(M, N, device="cuda:0", generator=g) * 2 + 0.5).bfloat16() if has_res else None
    nw = (1 + 0.1 * torch.randn(N, device="cuda:0", generator=g)).bfloat16()
    nb = (0.1 * torch.randn(N, device="cuda:0", generator=g)).bfloat16()
    x = torch.full((M, N), 9.0, dtype=torch.bfloat16, device="cuda:0")
    xn = torch.full((M, N), 9.0, dtype=torch.bfloat16, device="cuda:0")
    eps = 1e-5 if norm == 2 else 1e-6
    rc = lib.rtvla_reduce_norm(_P(parts.data_ptr()) if nsplit else None, nsplit, M, N, _P(bias.data_ptr()) if has_bias else None,
                               _P(res.data_ptr()) if has_res else None, norm, _P(nw.data_ptr()), _P(nb.data_ptr()), ctypes.c_float(eps),
                               _P(x.data_ptr()), _P(xn.data_ptr()) if norm else None, _P(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, rc
    torch.cuda.synchronize()
    want = (parts[:nsplit].sum(0) if nsplit else torch.zeros(M, N, device="cuda:0"))
    if has_bias:
        want = want + bias.float()
    if has_res:
        want = want + res.float()
    assert ((x.float() - want).norm() / want.norm()).item() <= REL_TOL
    assert ((x.float() - want).abs() <= want.abs() * 2.0 ** -7 + 1e-3).all()
    if norm:
        xb = x.float()                                      # the norm reads the rounded stream, as the forward's next GEMM input does
        if norm == 2:
            ref = torch.nn.functional.layer_norm(xb, (N,), nw.float(), nb.float(), eps)
        else:
            ref = xb * torch.rsqrt(xb.pow(2).mean(-1, keepdim=True) + eps)
        assert ((xn.float() - ref).norm() / ref.norm()).item() <= REL_TOL
        assert ((xn.float() - ref).abs() <= ref.abs() * 2.0 ** -7 + 2e-3).all()
