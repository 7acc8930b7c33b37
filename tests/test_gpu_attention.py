"""Every attention kernel on its own, through the C ABI (rtvla_attention), against fp32 scaled-dot-product attention with the
mask written out explicitly (the reference's predicate: /root/reference/pi0_infer.py:1089-1096, pi05_infer.py:294-299;
causal grouped-query: dm0_infer.py:913-918).  Shapes sit on the kernels' edges: one key block, keys = 1 mod 32, the state-row
mask, a valid prefix shorter than the allocated one, causal grouped-query heads, more than four key blocks per key split."""
import ctypes

import pytest
import torch

import rtvla_capi as capi

pytestmark = pytest.mark.gpu
_P = ctypes.c_void_p
KINDS = {  # kind: (head_dim, group)
    capi.ATTN_GEMMA_PREFIX: (256, 8), capi.ATTN_GEMMA_SUFFIX: (256, 8), capi.ATTN_GQA128_PREFIX: (128, 2), capi.ATTN_GQA128_SUFFIX: (128, 2),
    capi.ATTN_VIT64: (64, 1), capi.ATTN_SIGLIP: (72, 1)}
REL_TOL = 1e-2      # relative L2 of the bf16 output against the fp32 result (probabilities and outputs are rounded to bf16 once each)
ABS_TOL = 3e-2      # largest element error, outputs are O(1)


def reference(kind, q, k, v, scale, prefix_alloc, valid_len, state_tokens):
    """fp32, mask as a dense boolean [tokens][keys]; q [T][B][G][D], k / v [K][B][D]."""
    T, B, G, D = q.shape
    K = k.shape[0]
    t = torch.arange(T, device=q.device)[:, None]
    j = torch.arange(K, device=q.device)[None, :]
    vis = torch.where(j < prefix_alloc, j < valid_len, (t >= state_tokens) | (j == prefix_alloc))
    if kind == capi.ATTN_GQA128_PREFIX:
        vis = vis & (j <= t)
    if kind == capi.ATTN_SIGLIP:
        vis = (t // 256) == (j // 256)
    logits = torch.einsum("tbgd,kbd->bgtk", q.float(), k.float()) * scale
    logits = logits.masked_fill(~vis[None, None], float("-inf"))
    return torch.einsum("bgtk,kbd->tbgd", torch.softmax(logits, -1), v.float())


def run(kind, tokens, keys, kv_heads, prefix_alloc=None, valid_len=None, state_tokens=0, seed=0, sharp=1.0, ramp=0.0):
    lib = capi.load()
    D, G = KINDS[kind]
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    q = (torch.randn(tokens, kv_heads, G, D, device="cuda:0", generator=g) * sharp).bfloat16()
    k = torch.randn(keys, kv_heads, D, device="cuda:0", generator=g).bfloat16()
    v = torch.randn(keys, kv_heads, D, device="cuda:0", generator=g).bfloat16()
    if ramp:            # logits that climb with the key index: the running maximum grows all the way through the key loop
        q = q.float(); q[..., 0] += 4.0; q = q.bfloat16()
        k = k.float(); k[..., 0] += ramp * torch.arange(keys, device="cuda:0")[:, None] / keys; k = k.bfloat16()
    out = torch.full_like(q, 9.0)
    scale = D ** -0.5
    prefix_alloc = keys if prefix_alloc is None else prefix_alloc
    vl = None if valid_len is None else torch.tensor([valid_len], dtype=torch.int32, device="cuda:0")
    need = lib.rtvla_attention_workspace_bytes(kind, tokens, keys, kv_heads)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
    rc = lib.rtvla_attention(kind, _P(q.data_ptr()), _P(k.data_ptr()), _P(v.data_ptr()), _P(out.data_ptr()), tokens, keys, kv_heads,
                             ctypes.c_float(scale), prefix_alloc, _P(vl.data_ptr()) if vl is not None else None, state_tokens,
                             _P(ws.data_ptr()), need, _P(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, rc
    torch.cuda.synchronize()
    ref = reference(kind, q, k, v, scale, prefix_alloc, prefix_alloc if valid_len is None else valid_len, state_tokens)
    err = (out.float() - ref)
    rel = (err.norm() / ref.norm()).item()
    assert torch.isfinite(out.float()).all()
    assert rel <= REL_TOL and err.abs().max().item() <= ABS_TOL, (rel, err.abs().max().item())
    return rel


@pytest.mark.parametrize("tokens", [1, 17, 32, 33, 257, 788, 968])
def test_gemma_prefix_pass(tokens):
    run(capi.ATTN_GEMMA_PREFIX, tokens, tokens, 1, seed=tokens)


@pytest.mark.parametrize("tokens,valid", [(820, 789), (820, 1), (300, 288), (64, 64)])
def test_gemma_prefix_pass_with_a_valid_length_below_the_allocated_prefix(tokens, valid):
    """Pi05: prompt rows past valid_encoder_len are allocated but masked as keys (their own outputs are never read)."""
    lib = capi.load()
    D, G = 256, 8
    g = torch.Generator(device="cuda:0").manual_seed(valid)
    q = torch.randn(tokens, 1, G, D, device="cuda:0", generator=g).bfloat16()
    k = torch.randn(tokens, 1, D, device="cuda:0", generator=g).bfloat16()
    v = torch.randn(tokens, 1, D, device="cuda:0", generator=g).bfloat16()
    out = torch.zeros_like(q)
    vl = torch.tensor([valid], dtype=torch.int32, device="cuda:0")
    need = lib.rtvla_attention_workspace_bytes(capi.ATTN_GEMMA_PREFIX, tokens, tokens, 1)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
    assert lib.rtvla_attention(capi.ATTN_GEMMA_PREFIX, _P(q.data_ptr()), _P(k.data_ptr()), _P(v.data_ptr()), _P(out.data_ptr()), tokens, tokens, 1,
                               ctypes.c_float(D ** -0.5), tokens, _P(vl.data_ptr()), 0, _P(ws.data_ptr()), need, _P(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    ref = reference(capi.ATTN_GEMMA_PREFIX, q, k, v, D ** -0.5, tokens, valid, 0)
    err = out.float()[:valid] - ref[:valid]
    assert (err.norm() / ref[:valid].norm()).item() <= REL_TOL


@pytest.mark.parametrize("tokens,prefix,valid,state", [
    (51, 788, None, 1),      # the headline shape: 839 keys, 7 key splits, state-token row sees itself only
    (51, 270, None, 1),      # 321 keys = 1 mod 32: the last key block holds one key
    (51, 13, None, 1),       # 64 keys: a single key split of two blocks
    (1, 5, None, 0),         # one query token, six keys: one key block
    (50, 820, 789, 0),       # Pi05: no state token, valid prefix shorter than the allocated one
    (50, 820, 1, 0),         # ... down to one visible prefix key
    (64, 768, None, 1),      # chunk 63
    (101, 259, None, 1),     # two 64-row blocks of suffix rows
    (128, 261, 200, 0),      # the 128-row limit
    (21, 2256, None, 1),     # 2277 keys: more than four key blocks per split, the general kernel with a key split
])
def test_gemma_suffix_pass_masks_and_key_splits(tokens, prefix, valid, state):
    run(capi.ATTN_GEMMA_SUFFIX, tokens, prefix + tokens, 1, prefix_alloc=prefix, valid_len=valid, state_tokens=state, seed=prefix)


@pytest.mark.parametrize("tokens,heads", [(1, 8), (31, 8), (32, 8), (33, 1), (170, 8), (607, 8)])
def test_causal_grouped_query_prefix_pass(tokens, heads):
    run(capi.ATTN_GQA128_PREFIX, tokens, tokens, heads, seed=tokens)


@pytest.mark.parametrize("tokens,prefix,heads", [(50, 607, 8), (50, 33, 8), (64, 200, 2), (7, 1, 8)])
def test_grouped_query_suffix_pass(tokens, prefix, heads):
    run(capi.ATTN_GQA128_SUFFIX, tokens, prefix + tokens, heads, seed=prefix)


@pytest.mark.parametrize("tokens,heads", [(1, 16), (63, 3), (64, 8), (96, 2), (128, 4), (129, 16), (192, 3), (200, 2), (257, 5), (2705, 16)])
def test_vit_flash_attention(tokens, heads):
    """One to 43 key tiles of 64: a single tile, an odd number of 32-key blocks (the half-filled last tile), three and more
    tiles (the three LDS stages wrap), the DM0 shape."""
    run(capi.ATTN_VIT64, tokens, tokens, heads, seed=tokens)


@pytest.mark.parametrize("tokens", [96, 700, 2705])
def test_vit_flash_attention_with_a_maximum_that_keeps_growing(tokens):
    """The ViT kernel rescales its accumulator only when a row maximum grew by 2^8 and moves the probabilities of the block in
    flight to the new scale: logits that climb by ~90 bits over the keys take that path about a dozen times per row."""
    run(capi.ATTN_VIT64, tokens, tokens, 3, seed=tokens + 1, ramp=128.0)


@pytest.mark.parametrize("views", [1, 3])
def test_siglip_attention_keeps_views_apart(views):
    run(capi.ATTN_SIGLIP, 256 * views, 256 * views, 16, seed=views)


def test_peaked_softmax_rows_survive_the_running_maximum():
    """Large logits (|q| scaled up): one key dominates each row, the running-maximum rescale path is exercised in every kernel."""
    run(capi.ATTN_GEMMA_PREFIX, 300, 300, 1, seed=5, sharp=6.0)
    run(capi.ATTN_GEMMA_SUFFIX, 51, 839, 1, prefix_alloc=788, state_tokens=1, seed=6, sharp=6.0)
    run(capi.ATTN_VIT64, 500, 500, 4, seed=7, sharp=6.0)
    run(capi.ATTN_GQA128_PREFIX, 300, 300, 8, seed=8, sharp=6.0)
