"""Pins every op of the CPU oracle against an independent statement of the same mathematics
(torch.nn.functional routines, brute-force loops, closed forms, invariants).  The reference ships
no golden vectors for this path, so these are the checks a dropped term, a wrong sign or index or
a transposed operand in the oracle would fail."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ops

torch.manual_seed(0)


def test_gemm_against_float64():
    x = torch.randn(7, 33).bfloat16().float()
    w = torch.randn(33, 19).bfloat16()
    ref = (x.double().numpy() @ w.double().numpy())
    assert np.allclose(ops.gemm(x, w).numpy(), ref, rtol=1e-5, atol=1e-5)
    # "in x out": a one-hot row picks a weight ROW
    e = torch.zeros(1, 33); e[0, 5] = 1.0
    assert torch.equal(ops.gemm(e, w)[0], w[5].float())


def test_activations_against_torch():
    a = torch.linspace(-6, 6, 1001)
    assert torch.allclose(ops.gelu_tanh(a), F.gelu(a, approximate="tanh"), atol=2e-6)
    assert torch.allclose(ops.silu(a), F.silu(a), atol=1e-6)


def test_layer_norm_against_torch():
    x = torch.randn(5, 1152) * 3 + 1.5
    w, b = torch.randn(1152).bfloat16(), torch.randn(1152).bfloat16()
    ref = F.layer_norm(x, (1152,), w.float(), b.float(), eps=1e-5)
    assert torch.allclose(ops.layer_norm(x, w, b), ref, atol=2e-5)
    # eps is 1e-5, not 1e-6: a row whose variance is comparable to eps exposes it
    c = torch.randn(1, 64) * 0.003
    got = ops.layer_norm(c, torch.ones(64), torch.zeros(64))
    assert torch.allclose(got, F.layer_norm(c, (64,), eps=1e-5), atol=1e-4)
    assert (got - F.layer_norm(c, (64,), eps=1e-6)).abs().max().item() > 1e-2


def test_rms_factor_closed_form():
    x = torch.full((2, 1024), 3.0)
    assert torch.allclose(ops.rms_factor(x), torch.full((2, 1), 1.0 / math.sqrt(9.0 + 1e-6)))
    y = torch.randn(4, 2048)
    n = y * ops.rms_factor(y)
    assert torch.allclose((n * n).mean(-1), torch.ones(4), atol=1e-4)


def test_rope_table_layout_and_values():
    t = ops.rope_table(3, 5)
    assert t.shape == (5, 256)
    for row, pos in enumerate(range(3, 8)):
        for i in (0, 1, 64, 127):
            ang = pos * 10000 ** (-2 * i / 256)
            assert abs(t[row, 2 * i].item() - math.cos(ang)) < 4e-3      # bf16 rounded
            assert abs(t[row, 2 * i + 1].item() - math.sin(ang)) < 4e-3
    assert torch.equal(ops.rope_table(0, 1)[0, 0::2], torch.ones(128)) and torch.all(ops.rope_table(0, 1)[0, 1::2] == 0)


def _exact_table(start, count):
    pos = torch.arange(start, start + count, dtype=torch.float64)
    inv = 10000 ** (-torch.arange(0, 256, 2, dtype=torch.float64) / 256)
    ph = pos[:, None] * inv[None, :]
    return torch.stack([torch.cos(ph), torch.sin(ph)], 2).reshape(count, 256).float()


def test_rope_interleaved_against_loops_and_invariants():
    x = torch.randn(3, 2 * 256)
    tab = _exact_table(5, 3)
    got = ops.rope_interleaved(x, tab)
    for r in range(3):
        for h in range(2):
            for j in (0, 7, 127):
                c, s = tab[r, 2 * j].item(), tab[r, 2 * j + 1].item()
                x0, x1 = x[r, h * 256 + 2 * j].item(), x[r, h * 256 + 2 * j + 1].item()
                assert abs(got[r, h * 256 + 2 * j].item() - (x0 * c - x1 * s)) < 1e-5
                assert abs(got[r, h * 256 + 2 * j + 1].item() - (x1 * c + x0 * s)) < 1e-5
    # a rotation: norm preserving, identity at position 0, and <rope(q,m), rope(k,n)> depends on m - n only
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)
    assert torch.allclose(ops.rope_interleaved(x[:1], _exact_table(0, 1)), x[:1], atol=1e-6)
    q, k = torch.randn(1, 256), torch.randn(1, 256)
    d1 = (ops.rope_interleaved(q, _exact_table(9, 1)) * ops.rope_interleaved(k, _exact_table(4, 1))).sum()
    d2 = (ops.rope_interleaved(q, _exact_table(25, 1)) * ops.rope_interleaved(k, _exact_table(20, 1))).sum()
    assert abs(d1.item() - d2.item()) < 1e-3


def test_patches_equal_stride14_convolution():
    img = torch.randn(2, 224, 224, 3)
    w = torch.randn(14, 14, 3, 8)
    got = ops.patches(img) @ w.reshape(588, 8)
    ref = F.conv2d(img.permute(0, 3, 1, 2), w.permute(3, 2, 0, 1), stride=14)      # [v, 8, 16, 16]
    ref = ref.permute(0, 2, 3, 1).reshape(2 * 256, 8)
    assert torch.allclose(got, ref, atol=2e-3, rtol=1e-4)


def test_vision_attention_against_sdpa():
    qkv = torch.randn(2 * 256, 3456)
    got = ops.vision_attention(qkv, ops.identity)
    t = qkv.view(2, 256, 3, 16, 72).permute(0, 2, 3, 1, 4)
    ref = F.scaled_dot_product_attention(t[:, 0], t[:, 1], t[:, 2]).transpose(1, 2).reshape(2 * 256, 1152)
    assert torch.allclose(got, ref, atol=1e-4)


def test_mqa_attention_against_per_head_loops():
    tokens, keys = 5, 11
    q = torch.randn(tokens * 8, 256)
    k, v = torch.randn(keys, 256), torch.randn(keys, 256)
    got = ops.mqa_attention(q, k, v, ops.identity).reshape(tokens, 8, 256)
    for t in range(tokens):
        for h in range(8):
            logits = torch.tensor([(q[t * 8 + h] * k[j]).sum().item() / 16.0 for j in range(keys)])
            p = torch.softmax(logits, 0)
            assert torch.allclose(got[t, h], (p[:, None] * v).sum(0), atol=1e-4)


def test_pi0_suffix_mask_rule():
    s_d, s_e = 4, 6
    m = ops.pi0_suffix_mask(s_d, s_e)
    assert m.shape == (8 * s_d, s_e + s_d)
    for r in range(8 * s_d):
        for j in range(s_e + s_d):
            token = r // 8
            want = True if token >= 1 else j <= s_e          # the state token sees the prefix and itself
            assert bool(m[r, j]) == want


def test_pi05_masks():
    m = ops.valid_len_mask(3, 10, 7)
    assert m[:, :7].all() and not m[:, 7:].any()
    d = ops.pi05_suffix_mask(2, 10, 7)
    assert d.shape == (16, 12) and d[:, :7].all() and not d[:, 7:10].any() and d[:, 10:].all()


def test_masked_attention_ignores_hidden_keys():
    q, k, v = torch.randn(8, 256), torch.randn(6, 256), torch.randn(6, 256)
    mask = ops.valid_len_mask(8, 6, 4)
    a = ops.mqa_attention(q, k, v, ops.identity, mask)
    k2, v2 = k.clone(), v.clone()
    k2[4:] = 100.0; v2[4:] = -100.0
    assert torch.allclose(a, ops.mqa_attention(q, k2, v2, ops.identity, mask), atol=1e-5)
    assert torch.allclose(a, ops.mqa_attention(q, k[:4], v[:4], ops.identity), atol=1e-5)


def test_round_bf16_is_round_to_nearest_even():
    # exact ties between neighbouring bf16 values go to the even mantissa
    x = torch.tensor([1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 1.0 + 2 ** -8 + 2 ** -20, -(1.0 + 2 ** -8)])
    assert ops.round_bf16(x).tolist() == [1.0, 1.0 + 2 ** -6, 1.0 + 2 ** -7, -1.0]
