"""Independent restatements of the oracle's layer bodies and of the whole schedule.

Each layer function of oracle/pi0.py and oracle/pi05.py is compared (all-fp32 mode) with a second statement of
the same mathematics written token by token and head by head from the reference's kernels, with every tensor
sliced by hand: a dropped residual, a swapped norm, a wrong cache row, mask row or RoPE position fails here.
The last two tests restate the whole Pi0 / Pi05 forward in a different style (conv2d patch embedding, F.layer_norm,
scaled_dot_product_attention, complex-number RoPE, boolean masks built by loops) and compare complete
reduced-depth forwards.  LayerNorm weights and biases are random and distinct per layer throughout.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import synthetic as syn
from oracle import ops, pi0, pi05

ID = ops.identity


@pytest.fixture(scope="module")
def ck0():
    return syn.pi0_checkpoint(31, 3, vision_layers=2, llm_layers=2, norms="random")


@pytest.fixture(scope="module")
def ck5():
    return syn.pi05_checkpoint(32, 3, vision_layers=2, llm_layers=2, state_tokens=2, norms="random")


def W(ck, name, i=None):
    t = ck[name] if i is None else ck[name][i]
    return t.float()


def rot(vec, pos):
    """Interleaved-pair rotation of one 256-wide head by the angles of position `pos`
    (/root/reference/pi0_infer.py:794-800, table :1319-1335: cos and sin rounded to bf16)."""
    out = vec.clone()
    for j in range(128):
        ang = torch.tensor(float(pos), dtype=torch.float32) * (1.0 / (10000 ** (torch.tensor(2.0 * j) / 256)))
        c = torch.cos(ang).bfloat16().float()
        s = torch.sin(ang).bfloat16().float()
        out[2 * j] = vec[2 * j] * c - vec[2 * j + 1] * s
        out[2 * j + 1] = vec[2 * j + 1] * c + vec[2 * j] * s
    return out


def rms_rows(x):
    return torch.stack([row / torch.sqrt((row * row).sum() / row.numel() + 1e-6) for row in x])


# ---------------------------------------------------------------------------------------------------------
def test_norm_parameters_are_distinct_per_layer(ck0):
    a, b = ck0["vision_pre_attn_norm_w"].float(), ck0["vision_pre_ffn_norm_b"].float()
    assert (a[0] - a[1]).abs().mean() > 0.05 and (a - 1).abs().mean() > 0.05 and b.abs().mean() > 0.05
    assert not torch.equal(ck0["vision_pre_attn_norm_w"], ck0["vision_pre_ffn_norm_w"])
    assert (ck0["vision_final_norm_b"].float().abs().mean() > 0.05)
    ones = syn.pi0_checkpoint(31, 3, vision_layers=1, llm_layers=1)
    assert torch.all(ones["vision_pre_attn_norm_w"] == 1) and torch.all(ones["vision_final_norm_b"] == 0)


def test_siglip_layer_against_per_token_loops(ck0):
    """/root/reference/pi0_infer.py:607-646 with the attention of :588-596, for layer 1 (so that a layer-0
    parameter picked by mistake shows)."""
    i = 1
    torch.manual_seed(2)
    x = torch.randn(256, 1152) * 2 + 0.3
    got = pi0.vision_layer(ck0, i, x, ID)

    n = F.layer_norm(x, (1152,), W(ck0, "vision_pre_attn_norm_w", i), W(ck0, "vision_pre_attn_norm_b", i), eps=1e-5)
    wqkv, bqkv = W(ck0, "vision_attn_qkv_w", i), W(ck0, "vision_attn_qkv_b", i)
    qkv = torch.stack([n[t] @ wqkv + bqkv for t in range(256)])              # [Q | K | V], each 16 heads x 72
    attn = torch.zeros(256, 1152)
    for h in range(16):
        q = qkv[:, 72 * h: 72 * h + 72]
        k = qkv[:, 1152 + 72 * h: 1152 + 72 * h + 72]
        v = qkv[:, 2304 + 72 * h: 2304 + 72 * h + 72]
        for t in range(0, 256, 17):                                           # a sample of query rows per head
            p = torch.softmax((k @ q[t]) / math.sqrt(72.0), 0)
            attn[t, 72 * h: 72 * h + 72] = p @ v
    rows = list(range(0, 256, 17))
    x1 = x[rows] + attn[rows] @ W(ck0, "vision_attn_o_w", i) + W(ck0, "vision_attn_o_b", i)
    n1 = F.layer_norm(x1, (1152,), W(ck0, "vision_pre_ffn_norm_w", i), W(ck0, "vision_pre_ffn_norm_b", i), eps=1e-5)
    hdn = F.gelu(n1 @ W(ck0, "vision_ffn_up_w", i) + W(ck0, "vision_ffn_up_b", i), approximate="tanh")
    want = x1 + hdn @ W(ck0, "vision_ffn_down_w", i) + W(ck0, "vision_ffn_down_b", i)
    assert torch.allclose(got[rows], want, atol=2e-4, rtol=1e-4)
    # the residual really is carried: without it the result is far off
    assert (got[rows] - (want - x1)).abs().mean() > 0.5


def test_vision_encoder_views_do_not_mix(ck0):
    """Attention is per view (/root/reference/pi0_infer.py:590): changing view 1 leaves view 0's tokens alone, and
    every view gets the same position embedding rows."""
    img = syn.observation(31, 2, 4)[0].float()
    a = pi0.vision_encoder(ck0, img, ID)
    img2 = img.clone(); img2[1] = -img2[1]
    b = pi0.vision_encoder(ck0, img2, ID)
    assert torch.equal(a[:256], b[:256]) and not torch.allclose(a[256:], b[256:])
    same = torch.stack([img[0], img[0]])
    c = pi0.vision_encoder(ck0, same, ID)
    assert torch.allclose(c[:256], c[256:], atol=1e-5)


def test_project_and_concat_against_per_token_statement(ck0):
    """/root/reference/pi0_infer.py:753-775 and :1343-1345: final LayerNorm, projector with bias, image tokens NOT
    scaled by sqrt(2048), prompt rows appended unchanged."""
    torch.manual_seed(3)
    vx = torch.randn(256, 1152) * 1.7 - 0.2
    prompt = torch.randn(3, 2048)
    got = pi0.project_and_concat(ck0, vx, prompt, ID)
    assert got.shape == (259, 2048)
    n = F.layer_norm(vx, (1152,), W(ck0, "vision_final_norm_w"), W(ck0, "vision_final_norm_b"), eps=1e-5)
    for t in (0, 100, 255):
        want = n[t] @ W(ck0, "encoder_multi_modal_projector_w") + W(ck0, "encoder_multi_modal_projector_b")
        assert torch.allclose(got[t], want, atol=1e-4)
    assert torch.equal(got[256:], prompt)
    # the final norm's own parameters, not a layer's
    wrong = F.layer_norm(vx, (1152,), W(ck0, "vision_pre_attn_norm_w", 0), W(ck0, "vision_pre_attn_norm_b", 0), eps=1e-5)
    assert (got[0] - (wrong[0] @ W(ck0, "encoder_multi_modal_projector_w") + W(ck0, "encoder_multi_modal_projector_b"))).abs().mean() > 1e-2


def _suffix_reference_pi0(ck, i, x, kp, vp, s_e):
    """One Pi0 action-expert layer token by token (/root/reference/pi0_infer.py:1186-1223; factor :939-951, QKV
    :966-1031, logits :1041-1066, mask :1085, P V :1108-1120, O :1122-1135, GeGLU :693-725, down :1150-1163)."""
    s_d = x.shape[0]
    wqkv = W(ck, "decoder_attn_qkv_w", i)
    full = []
    for t in range(s_d):
        f = 1.0 / torch.sqrt((x[t] * x[t]).mean() + 1e-6)
        full.append((x[t] @ wqkv) * f)
    full = torch.stack(full)
    k_new = torch.stack([rot(full[t, 2048:2304], s_e + t) for t in range(s_d)])
    v_new = full[:, 2304:]
    keys = torch.cat([kp, k_new])             # cache rows [0, s_e) prefix, [s_e, s_e + s_d) suffix
    vals = torch.cat([vp, v_new])
    attn = torch.zeros(s_d, 2048)
    for t in range(s_d):
        for h in range(8):
            r = t * 8 + h
            q = rot(full[t, 256 * h: 256 * h + 256], s_e + t)
            logits = (keys @ q) / 16.0
            for j in range(keys.shape[0]):
                if not (r >= 8 or j <= s_e):
                    logits[j] = float("-inf")
            p = torch.softmax(logits, 0)
            attn[t, 256 * h: 256 * h + 256] = p @ vals
    x1 = x + attn @ W(ck, "decoder_attn_o_w", i)
    n1 = rms_rows(x1)
    g = F.gelu(n1 @ W(ck, "decoder_ffn_gate_w", i), approximate="tanh") * (n1 @ W(ck, "decoder_ffn_up_w", i))
    return x1 + g @ W(ck, "decoder_ffn_down_w", i), k_new, v_new


def test_pi0_suffix_layer_against_per_token_loops(ck0):
    i, s_e, s_d = 1, 5, 4
    torch.manual_seed(4)
    x = torch.randn(s_d, 1024)
    kp, vp = torch.randn(s_e, 256), torch.randn(s_e, 256)
    table = ops.rope_table(s_e, s_d)
    mask = ops.pi0_suffix_mask(s_d, s_e)
    got = pi0.suffix_layer(ck0, i, x, kp, vp, table, mask, ID)
    want, _, _ = _suffix_reference_pi0(ck0, i, x, kp, vp, s_e)
    assert torch.allclose(got, want, atol=3e-4, rtol=1e-4)


def test_pi0_state_token_sees_only_the_prefix_and_itself(ck0):
    """Mask in situ: the state row's output must not move when the action rows change, while an action row's
    output does depend on the state row (/root/reference/pi0_infer.py:1085)."""
    i, s_e, s_d = 0, 5, 4
    torch.manual_seed(5)
    x = torch.randn(s_d, 1024)
    kp, vp = torch.randn(s_e, 256), torch.randn(s_e, 256)
    table, mask = ops.rope_table(s_e, s_d), ops.pi0_suffix_mask(s_d, s_e)
    a = pi0.suffix_layer(ck0, i, x, kp, vp, table, mask, ID)
    x2 = x.clone(); x2[1:] = torch.randn(s_d - 1, 1024)
    b = pi0.suffix_layer(ck0, i, x2, kp, vp, table, mask, ID)
    assert torch.equal(a[0], b[0]) and not torch.allclose(a[1], b[1])
    x3 = x.clone(); x3[0] = torch.randn(1024)
    c = pi0.suffix_layer(ck0, i, x3, kp, vp, table, mask, ID)
    assert not torch.allclose(a[2], c[2], atol=1e-6)
    # and every suffix row depends on the prefix cache
    d = pi0.suffix_layer(ck0, i, x, kp + 1.0, vp, table, mask, ID)
    assert not torch.allclose(a[0], d[0], atol=1e-6) and not torch.allclose(a[3], d[3], atol=1e-6)


def test_pi0_euler_step_against_direct_formula(ck0):
    torch.manual_seed(6)
    x, noise = torch.randn(4, 1024), torch.randn(3, 32)
    got = pi0.euler_step(ck0, x, noise, ID)
    want = noise + rms_rows(x[1:]) @ W(ck0, "decoder_action_fused_out_proj_w") + W(ck0, "decoder_action_fused_out_proj_b")
    assert torch.allclose(got, want, atol=1e-5)


def test_pi05_suffix_layer_against_per_token_loops(ck5):
    """/root/reference/pi05_infer.py:427-509 (adaRMS :78-113, gated residual :22-64, mask :382-416); the prefix is
    allocated for more rows than are valid, the suffix keys sit behind the ALLOCATED rows and RoPE positions
    start at valid_len - 1 (:787-790)."""
    i, s_alloc, valid, s_d = 1, 7, 5, 3
    torch.manual_seed(7)
    x = torch.randn(s_d, 1024)
    kp, vp = torch.randn(s_alloc, 256), torch.randn(s_alloc, 256)
    st_a, st_f = torch.randn(3072) * 0.3, torch.randn(3072) * 0.3
    table = ops.rope_table(valid - 1, s_d)
    mask = ops.pi05_suffix_mask(s_d, s_alloc, valid)
    got = pi05.suffix_layer(ck5, i, x, kp, vp, st_a, st_f, table, mask, ID)

    def ada(row, style):
        xh = row / torch.sqrt((row * row).mean() + 1e-6)
        return xh * (1.0 + style[:1024]) + style[1024:2048]
    wqkv = W(ck5, "decoder_attn_qkv_w", i)
    full = torch.stack([ada(x[t], st_a) @ wqkv for t in range(s_d)])
    k_new = torch.stack([rot(full[t, 2048:2304], valid - 1 + t) for t in range(s_d)])
    keys, vals = torch.cat([kp, k_new]), torch.cat([vp, full[:, 2304:]])
    attn = torch.zeros(s_d, 2048)
    for t in range(s_d):
        for h in range(8):
            q = rot(full[t, 256 * h: 256 * h + 256], valid - 1 + t)
            logits = (keys @ q) / 16.0
            for j in range(s_alloc):
                if j >= valid:
                    logits[j] = float("-inf")
            p = torch.softmax(logits, 0)
            attn[t, 256 * h: 256 * h + 256] = p @ vals
    x1 = x + (attn @ W(ck5, "decoder_attn_o_w", i)) * st_a[2048:]
    n1 = torch.stack([ada(x1[t], st_f) for t in range(s_d)])
    g = F.gelu(n1 @ W(ck5, "decoder_ffn_gate_w", i), approximate="tanh") * (n1 @ W(ck5, "decoder_ffn_up_w", i))
    want = x1 + (g @ W(ck5, "decoder_ffn_down_w", i)) * st_f[2048:]
    assert torch.allclose(got, want, atol=3e-4, rtol=1e-4)
    # masked prefix rows are inert
    kp2, vp2 = kp.clone(), vp.clone(); kp2[valid:] = 50.0; vp2[valid:] = -50.0
    assert torch.allclose(got, pi05.suffix_layer(ck5, i, x, kp2, vp2, st_a, st_f, table, mask, ID), atol=1e-5)


# ---------------------------------------------------------------------------------------------------------
# the whole schedule, written a second time in a different style
def _alt_rope(x, pos):
    """x [rows, heads, 256] rotated as 128 complex numbers per head by exp(i theta), theta = pos * 10000^(-2j/256)."""
    inv = 1.0 / (10000 ** (torch.arange(0, 256, 2, dtype=torch.float32) / 256))
    ph = pos.to(torch.float32)[:, None] * inv[None, :]
    rotor = torch.complex(torch.cos(ph).bfloat16().float(), torch.sin(ph).bfloat16().float())      # the table is bf16
    z = torch.view_as_complex(x.reshape(x.shape[0], x.shape[1], 128, 2).contiguous())
    return torch.view_as_real(z * rotor[:, None, :]).reshape(x.shape)


def _alt_rms(x):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)


def _alt_vision(ck, img):
    v = img.shape[0]
    w = ck["vision_patch_embedding_w"].float().permute(3, 2, 0, 1)                  # [1152, 3, 14, 14]
    x = F.conv2d(img.float().permute(0, 3, 1, 2), w, ck["vision_patch_embedding_b"].float(), stride=14)
    x = x.flatten(2).transpose(1, 2) + ck["vision_position_embedding"].float()[None]      # [v, 256, 1152]
    for i in range(ck["vision_attn_qkv_w"].shape[0]):
        n = F.layer_norm(x, (1152,), W(ck, "vision_pre_attn_norm_w", i), W(ck, "vision_pre_attn_norm_b", i), 1e-5)
        q, k, val = (n @ W(ck, "vision_attn_qkv_w", i) + W(ck, "vision_attn_qkv_b", i)).split(1152, dim=-1)
        sp = lambda t: t.reshape(v, 256, 16, 72).transpose(1, 2)
        a = F.scaled_dot_product_attention(sp(q), sp(k), sp(val)).transpose(1, 2).reshape(v, 256, 1152)
        x = x + a @ W(ck, "vision_attn_o_w", i) + W(ck, "vision_attn_o_b", i)
        n = F.layer_norm(x, (1152,), W(ck, "vision_pre_ffn_norm_w", i), W(ck, "vision_pre_ffn_norm_b", i), 1e-5)
        x = x + F.gelu(n @ W(ck, "vision_ffn_up_w", i) + W(ck, "vision_ffn_up_b", i), approximate="tanh") @ W(ck, "vision_ffn_down_w", i) \
            + W(ck, "vision_ffn_down_b", i)
    n = F.layer_norm(x, (1152,), W(ck, "vision_final_norm_w"), W(ck, "vision_final_norm_b"), 1e-5)
    return (n @ W(ck, "encoder_multi_modal_projector_w") + W(ck, "encoder_multi_modal_projector_b")).reshape(v * 256, 2048)


def _alt_mqa(q, k, v, visible):
    """q [rows, 8, 256], one shared k, v [keys, 256]; visible [rows, keys] bool (same for every head)."""
    qh = q.transpose(0, 1)                                                           # [8, rows, 256]
    out = F.scaled_dot_product_attention(qh, k[None].expand(8, -1, -1), v[None].expand(8, -1, -1),
                                         attn_mask=visible[None].expand(8, -1, -1), scale=1.0 / 16.0)
    return out.transpose(0, 1).reshape(q.shape[0], 2048)


def _alt_prefix(ck, x, valid):
    s = x.shape[0]
    pos = torch.arange(s)
    visible = torch.zeros(s, s, dtype=torch.bool)
    for j in range(s):
        visible[:, j] = j < valid
    L = ck["encoder_attn_qkv_w"].shape[0]
    cache = []
    for i in range(L):
        qkv = _alt_rms(x) @ W(ck, "encoder_attn_qkv_w", i)
        q = _alt_rope(qkv[:, :2048].reshape(s, 8, 256), pos)
        k = _alt_rope(qkv[:, 2048:2304].reshape(s, 1, 256), pos)[:, 0]
        v = qkv[:, 2304:]
        cache.append((k, v))
        if i == L - 1:
            break                                                                   # the last layer only fills the cache
        x = x + _alt_mqa(q, k, v, visible) @ W(ck, "encoder_attn_o_w", i)
        n = _alt_rms(x)
        x = x + (F.gelu(n @ W(ck, "encoder_ffn_gate_w", i), approximate="tanh") * (n @ W(ck, "encoder_ffn_up_w", i))) @ W(ck, "encoder_ffn_down_w", i)
    return cache


def alt_pi0_forward(ck, img, state, noise):
    e = torch.cat([_alt_vision(ck, img), ck["language_embeds"].float()])
    s_e = e.shape[0]
    cache = _alt_prefix(ck, e, s_e)
    chunk = noise.shape[0]
    s_d = chunk + 1
    pos = s_e + torch.arange(s_d)
    visible = torch.ones(s_d, s_e + s_d, dtype=torch.bool)
    visible[0, s_e + 1:] = False                                                     # the state token: prefix and itself
    noise = noise.float()
    st = state.float()[None] @ W(ck, "decoder_state_in_proj_w") + W(ck, "decoder_state_in_proj_b")
    for t in range(10):
        u = F.silu(noise @ W(ck, "decoder_action_fused_in_proj_w") + W(ck, "decoder_action_fused_time_biases", t))
        x = torch.cat([st, u @ W(ck, "decoder_action_mlp_w") + W(ck, "decoder_action_mlp_b")])
        for i, (kp, vp) in enumerate(cache):
            qkv = _alt_rms(x) @ W(ck, "decoder_attn_qkv_w", i)
            q = _alt_rope(qkv[:, :2048].reshape(s_d, 8, 256), pos)
            k = _alt_rope(qkv[:, 2048:2304].reshape(s_d, 1, 256), pos)[:, 0]
            x = x + _alt_mqa(q, torch.cat([kp, k]), torch.cat([vp, qkv[:, 2304:]]), visible) @ W(ck, "decoder_attn_o_w", i)
            n = _alt_rms(x)
            x = x + (F.gelu(n @ W(ck, "decoder_ffn_gate_w", i), approximate="tanh") * (n @ W(ck, "decoder_ffn_up_w", i))) @ W(ck, "decoder_ffn_down_w", i)
        noise = noise + _alt_rms(x[1:]) @ W(ck, "decoder_action_fused_out_proj_w") + W(ck, "decoder_action_fused_out_proj_b")
    return noise


def alt_pi05_forward(ck, img, noise, alloc_prompt):
    prompt = ck["language_embeds"].float()
    s_v = img.shape[0] * 256
    valid = s_v + prompt.shape[0]
    junk = torch.full((alloc_prompt - prompt.shape[0], 2048), 3.0)                   # rows past the prompt: arbitrary, masked
    e = torch.cat([_alt_vision(ck, img), prompt, junk])
    s_alloc = e.shape[0]
    cache = _alt_prefix(ck, e, valid)
    s_d = noise.shape[0]
    pos = valid - 1 + torch.arange(s_d)
    visible = torch.ones(s_d, s_alloc + s_d, dtype=torch.bool)
    visible[:, valid:s_alloc] = False
    noise = noise.float()
    w_out, b_out = W(ck, "decoder_action_out_proj_w") * -0.1, W(ck, "decoder_action_out_proj_b") * -0.1

    def ada(x, style):
        sc, sh, gt = style.split(1024)
        return _alt_rms(x) * (1 + sc) + sh, gt
    for t in range(10):
        h = F.silu(W(ck, "decoder_time_embeds", t) @ W(ck, "decoder_time_mlp_in_w") + W(ck, "decoder_time_mlp_in_b"))
        temb = F.silu(h @ W(ck, "decoder_time_mlp_out_w") + W(ck, "decoder_time_mlp_out_b"))
        x = noise @ W(ck, "decoder_action_in_proj_w") + W(ck, "decoder_action_in_proj_b")
        for i, (kp, vp) in enumerate(cache):
            n, gt = ada(x, temb @ W(ck, "decoder_pre_attn_norm_mod_w", i) + W(ck, "decoder_pre_attn_norm_mod_b", i))
            qkv = n @ W(ck, "decoder_attn_qkv_w", i)
            q = _alt_rope(qkv[:, :2048].reshape(s_d, 8, 256), pos)
            k = _alt_rope(qkv[:, 2048:2304].reshape(s_d, 1, 256), pos)[:, 0]
            x = x + (_alt_mqa(q, torch.cat([kp, k]), torch.cat([vp, qkv[:, 2304:]]), visible) @ W(ck, "decoder_attn_o_w", i)) * gt
            n, gt = ada(x, temb @ W(ck, "decoder_pre_ffn_norm_mod_w", i) + W(ck, "decoder_pre_ffn_norm_mod_b", i))
            x = x + ((F.gelu(n @ W(ck, "decoder_ffn_gate_w", i), approximate="tanh") * (n @ W(ck, "decoder_ffn_up_w", i))) @ W(ck, "decoder_ffn_down_w", i)) * gt
        n, _ = ada(x, temb @ W(ck, "decoder_final_norm_mod_w") + W(ck, "decoder_final_norm_mod_b"))
        noise = noise + n @ w_out + b_out
    return noise


def test_whole_pi0_forward_against_a_second_implementation(ck0):
    img, state, noise = syn.observation(31, 2, 5)
    got = pi0.forward(ck0, img, state, noise, bf16_boundaries=False)
    want = alt_pi0_forward(ck0, img, state, noise)
    assert got.shape == (5, 32)
    assert torch.allclose(got, want, atol=2e-4), (got - want).abs().max()
    # the flow really moves the noise, so agreement is not vacuous
    assert (got - noise.float()).abs().mean() > 1e-2


def test_whole_pi05_forward_against_a_second_implementation(ck5):
    img, _, noise = syn.observation(32, 1, 6)
    got = pi05.forward(ck5, img, noise, max_prompt_len=9, bf16_boundaries=False)
    want = alt_pi05_forward(ck5, img, noise, alloc_prompt=9)
    assert torch.allclose(got, want, atol=2e-4), (got - want).abs().max()
    assert (got - noise.float()).abs().mean() > 1e-2
