"""Pins of the DM0 oracle (oracle/dm0.py) against independent statements of the same mathematics: the LayerNorm folded
into a GEMM against F.layer_norm + matmul, both im2col paths against conv2d, the two rotary embeddings against complex
rotations and closed-form angles, grouped-query attention against scaled_dot_product_attention with repeated KV heads,
one whole layer against per-token loops, and a complete reduced-depth forward against a second implementation."""
import math

import pytest
import torch
import torch.nn.functional as F

import synthetic as syn
from oracle import dm0, ops

ID = ops.identity
torch.manual_seed(0)


@pytest.fixture(scope="module")
def ck():
    return syn.dm0_checkpoint(51, vision_layers=2, llm_layers=2, vocab=64)


def W(ck, name, i=None):
    t = ck[name] if i is None else ck[name][i]
    return t.float()


def test_folded_layernorm_gemm_equals_layernorm_then_gemm():
    """dm0_infer.py:456-495: with W' = diag(gamma) W, colsum = column sums of W', b' = beta W + b."""
    x = torch.randn(7, 96) * 2 + 0.7
    gamma, beta = 1 + 0.2 * torch.randn(96), 0.3 * torch.randn(96)
    w, b = torch.randn(96, 40) * 0.1, torch.randn(40)
    want = F.layer_norm(x, (96,), gamma, beta, eps=1e-5) @ w + b
    wf = gamma[:, None] * w
    got = dm0.ln_folded_gemm(x, wf, wf.sum(0), beta @ w + b)
    assert torch.allclose(got, want, atol=2e-4)
    mean, rstd = dm0.ln_stats(x)
    assert torch.allclose(mean[:, 0], x.mean(-1), atol=1e-6) and torch.allclose(rstd[:, 0], 1 / torch.sqrt(x.var(-1, unbiased=False) + 1e-5), atol=1e-5)


def test_patch_embedding_equals_stride14_convolution(ck):
    """dm0_infer.py:695-698: NCHW input, feature order (c, dy, dx)."""
    img = torch.randn(1, 3, 728, 728)
    got = dm0.vision_patches(img) @ W(ck, "vision_conv1_w_t")
    weight = W(ck, "vision_conv1_w_t").t().reshape(1024, 3, 14, 14)
    want = F.conv2d(img, weight, stride=14).flatten(2).transpose(1, 2).reshape(2704, 1024)
    assert torch.allclose(got, want, atol=2e-3, rtol=1e-3)


def test_vision_rope_table_closed_form():
    cos, sin = dm0.vision_rope_table()
    assert cos.shape == (2705, 64) and torch.all(cos[0] == 1) and torch.all(sin[0] == 0)          # the class token is not rotated
    for (y, x) in ((0, 0), (3, 17), (51, 51)):
        tok = 1 + y * 52 + x
        for i in (0, 5, 15):
            f = 10000.0 ** (-(2 * i) / 32)
            for half, idx in ((0, x + 1), (1, y + 1)):                                                  # first 32 angles follow the column, last 32 the row
                ang = torch.tensor(idx * f).bfloat16().float()
                for rep in (0, 1):
                    c = cos[tok, half * 32 + 2 * i + rep].item()
                    assert abs(c - math.cos(ang.item())) < 4e-3
                    assert abs(sin[tok, half * 32 + 2 * i + rep].item() - math.sin(ang.item())) < 4e-3


def test_vision_rope_is_a_rotation_of_adjacent_pairs():
    cos, sin = dm0.vision_rope_table()
    t = torch.randn(2, 5, 64)
    c, s = cos[7:12], sin[7:12]
    got = dm0.vision_rope(t, c, s)
    z = torch.view_as_complex(t.reshape(2, 5, 32, 2).contiguous()) * torch.complex(c[:, 0::2], s[:, 0::2])
    assert torch.allclose(got, torch.view_as_real(z).reshape(2, 5, 64), atol=1e-6)
    assert torch.equal(dm0.vision_rope(t[:, :1], cos[:1], sin[:1]), t[:, :1])


def test_vision_attention_against_sdpa():
    n = 1
    qkv = torch.randn(n * dm0.SEQ, 3072)
    cos, sin = dm0.vision_rope_table()
    got = dm0.vision_attention(qkv, n, cos, sin, ID)
    q, k, v = qkv.split(1024, dim=-1)
    sp = lambda t: t.reshape(n, dm0.SEQ, 16, 64).transpose(1, 2)
    rot = torch.complex(cos[:, 0::2], sin[:, 0::2])
    rope = lambda t: torch.view_as_real(torch.view_as_complex(t.reshape(n, 16, dm0.SEQ, 32, 2).contiguous()) * rot).reshape(n, 16, dm0.SEQ, 64)
    want = F.scaled_dot_product_attention(rope(sp(q)), rope(sp(k)), sp(v), scale=0.125).transpose(1, 2).reshape(n * dm0.SEQ, 1024)
    assert torch.allclose(got, want, atol=2e-4)


def test_conv_downsample_equals_conv2d():
    """dm0_infer.py:631-658: weight HWIO, stride 2, padding 1, NHWC activations."""
    x = torch.randn(2, 10, 10, 24)
    w, b = torch.randn(3, 3, 24, 16) * 0.1, torch.randn(16)
    got = dm0.conv_downsample(x, w, b, ID)
    want = F.conv2d(x.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1), b, stride=2, padding=1).permute(0, 2, 3, 1)
    assert got.shape == (2, 5, 5, 16) and torch.allclose(got, want, atol=1e-4)
    odd = dm0.conv_downsample(torch.randn(1, 13, 13, 8), torch.randn(3, 3, 8, 4), torch.zeros(4), ID)
    assert odd.shape == (1, 7, 7, 4)
    # the two reference stages: 52 -> 26 -> 13
    col, oh, ow = dm0.im2col_nhwc(torch.zeros(1, 52, 52, 4), 3, 2, 1)
    assert (oh, ow, col.shape) == (26, 26, (676, 36))


def test_llm_rope_table_and_qknorm_split_against_loops(ck):
    tab = dm0.rope_table(5, 3)
    for r, pos in enumerate((5, 6, 7)):
        for j in (0, 9, 63):
            ang = pos * 1000000.0 ** (-2 * j / 128)
            assert abs(tab[r, 2 * j].item() - math.cos(ang)) < 4e-3 and abs(tab[r, 2 * j + 1].item() - math.sin(ang)) < 4e-3
    rows = 3
    qkv = torch.randn(rows, 4096)
    factor = torch.rand(rows, 1) + 0.5
    qn, kn = W(ck, "llm_q_norm_w", 1), W(ck, "llm_k_norm_w", 1)
    q, k, v = dm0.qknorm_rope_split(qkv, factor, qn, kn, tab, ID)
    assert q.shape == (rows, 16, 128) and k.shape == (rows, 8, 128) and v.shape == (rows, 8, 128)
    for r in range(rows):
        for head in (0, 7, 15, 16, 23, 24, 31):
            val = qkv[r, head * 128:(head + 1) * 128] * factor[r, 0]
            if head < 24:
                nw = qn if head < 16 else kn
                val = val / torch.sqrt((val * val).mean() + 1e-6) * nw
                out = val.clone()
                for j in range(64):
                    c, s = tab[r, 2 * j], tab[r, 2 * j + 1]
                    out[2 * j] = val[2 * j] * c - val[2 * j + 1] * s
                    out[2 * j + 1] = val[2 * j + 1] * c + val[2 * j] * s
                got = q[r, head] if head < 16 else k[r, head - 16]
            else:
                out, got = val, v[r, head - 24]
            assert torch.allclose(got, out, atol=1e-5)


def test_grouped_query_attention_against_sdpa():
    rows = 9
    q, k, v = torch.randn(rows, 16, 128), torch.randn(rows, 8, 128), torch.randn(rows, 8, 128)
    got = dm0.gqa_attention(q, k, v, ID, causal=True).reshape(rows, 16, 128)
    rep = lambda t: t.repeat_interleave(2, dim=1).transpose(0, 1)                      # query head h reads KV head h // 2
    want = F.scaled_dot_product_attention(q.transpose(0, 1), rep(k), rep(v), is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)
    # decoder form: more keys than rows, no mask
    kk, vv = torch.randn(20, 8, 128), torch.randn(20, 8, 128)
    got = dm0.gqa_attention(q, kk, vv, ID, causal=False).reshape(rows, 16, 128)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), rep(kk), rep(vv)).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)
    # row 0 of the causal form sees key 0 only
    assert torch.allclose(dm0.gqa_attention(q, k, v, ID, causal=True).reshape(rows, 16, 128)[0, 5], v[0, 2], atol=1e-6)


def _layer_by_loops(ck, pre, i, x, pos0, kp=None, vp=None):
    rows = x.shape[0]
    wqkv = W(ck, pre + "_attn_qkv_w", i)
    qn, kn = W(ck, pre + "_q_norm_w", i), W(ck, pre + "_k_norm_w", i)

    def rot(vec, pos):
        out = vec.clone()
        for j in range(64):
            ang = torch.tensor(float(pos)) * (1.0 / (1000000.0 ** (torch.tensor(2.0 * j) / 128)))
            c, s = torch.cos(ang).bfloat16().float(), torch.sin(ang).bfloat16().float()
            out[2 * j] = vec[2 * j] * c - vec[2 * j + 1] * s
            out[2 * j + 1] = vec[2 * j + 1] * c + vec[2 * j] * s
        return out
    qs, ks, vs = [], [], []
    for t in range(rows):
        f = 1.0 / torch.sqrt((x[t] * x[t]).mean() + 1e-6)
        full = (x[t] @ wqkv) * f
        heads = full.reshape(32, 128)
        nrm = lambda h, nw: h / torch.sqrt((h * h).mean() + 1e-6) * nw
        qs.append(torch.stack([rot(nrm(heads[h], qn), pos0 + t) for h in range(16)]))
        ks.append(torch.stack([rot(nrm(heads[16 + h], kn), pos0 + t) for h in range(8)]))
        vs.append(heads[24:])
    q, k, v = torch.stack(qs), torch.stack(ks), torch.stack(vs)
    keys = k if kp is None else torch.cat([kp, k])
    vals = v if vp is None else torch.cat([vp, v])
    attn = torch.zeros(rows, 2048)
    for t in range(rows):
        for h in range(16):
            logits = (keys[:, h // 2] @ q[t, h]) / math.sqrt(128.0)
            if kp is None:
                logits[t + 1:] = float("-inf")                                        # causal among the prefix rows
            attn[t, h * 128:(h + 1) * 128] = torch.softmax(logits, 0) @ vals[:, h // 2]
    x1 = x + attn @ W(ck, pre + "_attn_o_w", i)
    n1 = torch.stack([r / torch.sqrt((r * r).mean() + 1e-6) for r in x1])
    hdn = F.silu(n1 @ W(ck, pre + "_ffn_gate_w", i)) * (n1 @ W(ck, pre + "_ffn_up_w", i))
    return x1 + hdn @ W(ck, pre + "_ffn_down_w", i), k, v


def test_prefix_layer_against_per_token_loops(ck):
    """dm0_infer.py:874-951 for layer 1."""
    x = torch.randn(5, 2048)
    got, k, v = dm0.llm_layer(ck, "llm", 1, x, dm0.rope_table(0, 5), ID)
    want, wk, wv = _layer_by_loops(ck, "llm", 1, x, 0)
    assert torch.allclose(got, want, atol=3e-4, rtol=1e-4) and torch.allclose(k, wk, atol=1e-5) and torch.allclose(v, wv, atol=1e-5)
    # causal: changing a later row leaves the earlier rows alone
    x2 = x.clone(); x2[4] = torch.randn(2048)
    again, _, _ = dm0.llm_layer(ck, "llm", 1, x2, dm0.rope_table(0, 5), ID)
    assert torch.equal(again[:4], got[:4]) and not torch.allclose(again[4], got[4])


def test_action_expert_layer_against_per_token_loops(ck):
    """dm0_infer.py:782-851: the new K / V rows sit behind the prefix rows, every key is visible, positions start at the
    prefix length."""
    prefix = 6
    x = torch.randn(4, 1024)
    kp, vp = torch.randn(prefix, 8, 128), torch.randn(prefix, 8, 128)
    got, _, _ = dm0.llm_layer(ck, "decoder", 0, x, dm0.rope_table(prefix, 4), ID, kp, vp)
    want, _, _ = _layer_by_loops(ck, "decoder", 0, x, prefix, kp, vp)
    assert torch.allclose(got, want, atol=3e-4, rtol=1e-4)
    x2 = x.clone(); x2[3] = torch.randn(1024)                                          # no mask among the action rows
    again, _, _ = dm0.llm_layer(ck, "decoder", 0, x2, dm0.rope_table(prefix, 4), ID, kp, vp)
    assert not torch.allclose(again[0], got[0], atol=1e-6)


# ---- the whole forward a second time, in a different style ----
def alt_forward(ck, images, ids, noise):
    n = images.shape[0]
    wconv = W(ck, "vision_conv1_w_t").t().reshape(1024, 3, 14, 14)
    x = F.conv2d(images.float(), wconv, stride=14).flatten(2).transpose(1, 2)                           # [n, 2704, 1024]
    x = torch.cat([W(ck, "vision_class_embedding").expand(n, 1, 1024), x], dim=1) + W(ck, "vision_pos_emb")[None]
    x = F.layer_norm(x, (1024,), W(ck, "vision_ln_pre_w"), W(ck, "vision_ln_pre_b"), 1e-5)
    cos, sin = dm0.vision_rope_table()
    rotor = torch.complex(cos[:, 0::2], sin[:, 0::2])
    rope = lambda t: torch.view_as_real(torch.view_as_complex(t.reshape(*t.shape[:-1], -1, 2).contiguous()) * rotor[:t.shape[-2]]).reshape(t.shape)
    for i in range(ck["vision_fused_qkv_w"].shape[0]):
        # un-fold the LayerNorm: the synthetic column sums are the sums of the folded weight, so LN without affine, then GEMM
        xh = F.layer_norm(x, (1024,), eps=1e-5)
        q, k, v = (xh @ W(ck, "vision_fused_qkv_w", i) + W(ck, "vision_fused_qkv_b", i)).split(1024, dim=-1)
        sp = lambda t: t.reshape(n, 2705, 16, 64).transpose(1, 2)
        a = F.scaled_dot_product_attention(rope(sp(q)), rope(sp(k)), sp(v), scale=0.125).transpose(1, 2).reshape(n, 2705, 1024)
        x = x + a @ W(ck, "vision_out_proj_w", i) + W(ck, "vision_out_proj_b", i)
        xh = F.layer_norm(x, (1024,), eps=1e-5)
        x = x + F.gelu(xh @ W(ck, "vision_fused_fc_w", i) + W(ck, "vision_fused_fc_b", i), approximate="tanh") @ W(ck, "vision_proj_w", i) + W(ck, "vision_proj_b", i)
    x = x[:, 1:].reshape(n, 52, 52, 1024).permute(0, 3, 1, 2)
    x = F.conv2d(x, W(ck, "vision_ds1_w").permute(3, 2, 0, 1), W(ck, "vision_ds1_b"), stride=2, padding=1)
    x = F.conv2d(x, W(ck, "vision_ds2_w").permute(3, 2, 0, 1), W(ck, "vision_ds2_b"), stride=2, padding=1)
    x = x.permute(0, 2, 3, 1).reshape(-1, 4096) @ W(ck, "vision_projector_w_t")
    x = torch.cat([x, F.embedding(ids.long(), W(ck, "vision_embed_tokens_w"))])
    plen = x.shape[0]

    def rms(t):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6)

    def rope_llm(t, pos):                                                                               # t [rows, heads, 128]
        inv = 1.0 / (1000000.0 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
        ph = pos.float()[:, None] * inv[None, :]
        rt = torch.complex(torch.cos(ph).bfloat16().float(), torch.sin(ph).bfloat16().float())
        return torch.view_as_real(torch.view_as_complex(t.reshape(t.shape[0], t.shape[1], 64, 2).contiguous()) * rt[:, None, :]).reshape(t.shape)

    def layer(pre, i, x, pos, cache=None):
        rows = x.shape[0]
        heads = (rms(x) @ W(ck, pre + "_attn_qkv_w", i)).reshape(rows, 32, 128)
        q = rope_llm(rms(heads[:, :16]) * W(ck, pre + "_q_norm_w", i), pos)
        k = rope_llm(rms(heads[:, 16:24]) * W(ck, pre + "_k_norm_w", i), pos)
        v = heads[:, 24:]
        kk, vv = (k, v) if cache is None else (torch.cat([cache[0], k]), torch.cat([cache[1], v]))
        rep = lambda t: t.repeat_interleave(2, dim=1).transpose(0, 1)
        a = F.scaled_dot_product_attention(q.transpose(0, 1), rep(kk), rep(vv), is_causal=cache is None).transpose(0, 1).reshape(rows, 2048)
        x = x + a @ W(ck, pre + "_attn_o_w", i)
        n1 = rms(x)
        return x + (F.silu(n1 @ W(ck, pre + "_ffn_gate_w", i)) * (n1 @ W(ck, pre + "_ffn_up_w", i))) @ W(ck, pre + "_ffn_down_w", i), (k, v)
    caches = []
    for i in range(ck["llm_attn_qkv_w"].shape[0]):
        x, kv = layer("llm", i, x, torch.arange(plen))
        caches.append(kv)
    noise = noise.float()
    for t in range(10):
        y = F.silu(noise @ W(ck, "decoder_action_fused_in_proj_w") + W(ck, "decoder_action_fused_time_biases", t)) @ W(ck, "decoder_action_mlp_w") \
            + W(ck, "decoder_action_mlp_b")
        for i in range(ck["decoder_attn_qkv_w"].shape[0]):
            y, _ = layer("decoder", i, y, plen + torch.arange(50), caches[i])
        noise = noise + rms(y) @ W(ck, "decoder_action_fused_out_proj_w") + W(ck, "decoder_action_fused_out_proj_b")
    return noise


def test_whole_dm0_forward_against_a_second_implementation(ck):
    img, ids, noise = syn.dm0_observation(51, 1, max_lang_len=5, vocab=64)
    got = dm0.forward(ck, img, ids, noise, bf16_boundaries=False)
    want = alt_forward(ck, img, ids, noise)
    assert got.shape == (50, 32)
    assert torch.allclose(got, want, atol=3e-4), (got - want).abs().max()
    assert (got - noise.float()).abs().mean() > 1e-2                                                    # the flow really moves the noise
    bf = dm0.forward(ck, img, ids, noise)
    assert (bf - got).abs().mean() < 1e-2


def test_dm0_language_tokens_follow_the_image_tokens(ck):
    img, ids, noise = syn.dm0_observation(52, 1, max_lang_len=4, vocab=64)
    x = dm0.vision_forward(ck, img, ids, ID)
    assert x.shape == (169 + 4, 2048) and torch.equal(x[169:], ck["vision_embed_tokens_w"][ids].float())


def test_host_side_rope_pair_table_matches_the_oracle_tables():
    """The product's table (realtime-vla_amd/dm0_infer.py) holds one (cos, sin) per rotation pair; the reference's 64 angles
    repeat each frequency for both elements of a pair."""
    from dm0_infer import vision_rope_pairs
    tab = vision_rope_pairs("cpu").float()
    cos, sin = dm0.vision_rope_table()
    assert tab.shape == (2705, 64)
    assert torch.equal(tab[:, 0::2], cos[:, 0::2]) and torch.equal(tab[:, 0::2], cos[:, 1::2])
    assert torch.equal(tab[:, 1::2], sin[:, 0::2]) and torch.equal(tab[:, 1::2], sin[:, 1::2])
