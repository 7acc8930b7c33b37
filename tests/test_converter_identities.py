"""Algebraic identities behind the weight fusions the checkpoint converter bakes into the converted layout
(/root/reference/convert_from_jax.py), on random tensors: the forward on converted weights (as the oracle computes
it) must equal the un-fused model the converter started from.  CPU only, float64 where the identity is exact."""
import math

import torch

import synthetic as syn
from oracle import ops, pi0

torch.manual_seed(0)


def gemma_rms_norm(x, gamma):
    """Gemma RMSNorm with its learned scale: x / sqrt(mean x^2 + 1e-6) * (1 + gamma)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * (1.0 + gamma)


def test_rms_scale_folds_into_the_rows_of_the_next_weight():
    """convert_from_jax.py:52-54, :72-73 (and :95-97, :115-116 for the action expert): W *= (1 + gamma)[:, None]."""
    x = torch.randn(5, 64, dtype=torch.float64)
    gamma = torch.randn(64, dtype=torch.float64) * 0.3
    w = torch.randn(64, 48, dtype=torch.float64)
    unfused = gemma_rms_norm(x, gamma) @ w
    folded = w * (1.0 + gamma)[:, None]
    fused = (x * ops.rms_factor(x)) @ folded                      # what the forward does: no scale left in the norm
    assert torch.allclose(unfused, fused, atol=1e-12)
    # folding into columns instead (a transposed fold) is a different function
    assert not torch.allclose(unfused, (x * ops.rms_factor(x)) @ (w[:, :48] * (1.0 + gamma)[None, :48]), atol=1e-3)


def half_split_rope(v, pos):
    """RoPE as the un-converted model applies it to one 256-wide head laid out (2, 128): the first half is paired with
    the second half, angle pos * 10000^(-2j/256)."""
    j = torch.arange(128, dtype=torch.float64)
    ang = pos * 10000.0 ** (-2.0 * j / 256.0)
    a, b = v[:128], v[128:]
    return torch.cat([a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang)])


def exact_table(positions):
    j = torch.arange(128, dtype=torch.float64)
    ph = torch.tensor(positions, dtype=torch.float64)[:, None] * 10000.0 ** (-2.0 * j / 256.0)[None, :]
    return torch.stack([torch.cos(ph), torch.sin(ph)], 2).reshape(len(positions), 256)


def test_interleave_permutation_preserves_rotated_dot_products():
    """convert_from_jax.py:55-56 (:98-99): Q and K columns go from (2, 128) to (128, 2) per head, so that the forward's
    adjacent-pair rotation (pi0_infer.py:794-800) gives the same logits as the half-split rotation on the original."""
    K, heads = 32, 3
    wq = torch.randn(K, heads, 256, dtype=torch.float64)
    wk = torch.randn(K, 256, dtype=torch.float64)
    xq, xk = torch.randn(K, dtype=torch.float64), torch.randn(K, dtype=torch.float64)
    m, n = 7, 19
    # un-converted: project, rotate half-split
    q0 = torch.stack([half_split_rope(xq @ wq[:, h], m) for h in range(heads)])
    k0 = half_split_rope(xk @ wk, n)
    logits0 = q0 @ k0
    # converted: permute the weight columns, project, rotate adjacent pairs with the forward's routine
    wq_c = wq.reshape(K, heads, 2, 128).transpose(2, 3).reshape(K, heads * 256)
    wk_c = wk.reshape(K, 2, 128).transpose(1, 2).reshape(K, 256)
    q1 = ops.rope_interleaved((xq @ wq_c)[None, :], exact_table([m])).reshape(heads, 256)
    k1 = ops.rope_interleaved((xk @ wk_c)[None, :], exact_table([n]))[0]
    assert torch.allclose(q1 @ k1, logits0, atol=1e-9)
    # and the rotated vectors themselves are the same numbers in the permuted order
    assert torch.allclose(q1.reshape(heads, 128, 2).transpose(1, 2).reshape(heads, 256), q0, atol=1e-10)
    # V and O are untouched by the permutation (convert_from_jax.py:58-66): only the logits see Q and K
    assert not torch.allclose(ops.rope_interleaved((xq @ wq.reshape(K, -1))[None, :], exact_table([m])).reshape(heads, 256) @ k1, logits0, atol=1e-3)


def sincos_embedding(t, dim=1024, min_period=4e-3, max_period=4.0):
    """convert_from_jax.py:133-140 written out per element."""
    out = torch.zeros(dim, dtype=torch.float64)
    for i in range(dim // 2):
        frac = i / (dim // 2 - 1)
        period = min_period * (max_period / min_period) ** frac
        out[i] = math.sin(2.0 * math.pi / period * t)
        out[dim // 2 + i] = math.cos(2.0 * math.pi / period * t)
    return out


def test_time_embedding_of_the_synthetic_checkpoints_follows_the_converter_formula():
    for step in (0, 3, 9):
        t = 1.0 - step / 10
        want = sincos_embedding(t)
        got = syn._sincos_time(t)
        assert torch.allclose(got.double(), want, atol=2e-5)
    ck = syn.pi05_checkpoint(1, 0, vision_layers=1, llm_layers=1, state_tokens=0)
    assert torch.allclose(ck["decoder_time_embeds"][3].double(), sincos_embedding(0.7), atol=4e-3)      # bf16 rounded


def test_fused_action_time_input_projection():
    """convert_from_jax.py:176-187: with W_mlp = [W_a; W_t] acting on concat(action_in_proj(noise), time_emb),
       W_fused = W_in W_a   and   bias_t = W_a^T b_in + W_t^T sincos(t) + b_mlp
    give the same pre-activation as the two-step product."""
    chunk, d = 6, 40
    noise = torch.randn(chunk, 32, dtype=torch.float64)
    w_in, b_in = torch.randn(32, d, dtype=torch.float64), torch.randn(d, dtype=torch.float64)
    w_mlp, b_mlp = torch.randn(2 * d, d, dtype=torch.float64), torch.randn(d, dtype=torch.float64)
    temb = torch.randn(d, dtype=torch.float64)
    two_step = torch.cat([noise @ w_in + b_in, temb.expand(chunk, d)], dim=1) @ w_mlp + b_mlp
    w_a, w_t = w_mlp[:d], w_mlp[d:]
    fused_w = w_in @ w_a
    fused_b = w_a.T @ b_in + w_t.T @ temb + b_mlp
    assert torch.allclose(noise @ fused_w + fused_b, two_step, atol=1e-10)


def test_euler_step_with_dt_and_final_norm_folded_into_the_output_projection():
    """convert_from_jax.py:192-194: W_out' = W_out (1 + gamma_final)[:, None] dt, b_out' = b_out dt with dt = -0.1, so
    that the forward's `noise += rms(x) W_out' + b_out'` (pi0_infer.py:953-964) is one Euler step
    noise + dt * v,  v = gemma_rms_norm(x, gamma_final) W_out + b_out."""
    chunk = 5
    x = torch.randn(chunk + 1, 1024)
    noise = torch.randn(chunk, 32)
    gamma = torch.randn(1024) * 0.2
    w_out, b_out = torch.randn(1024, 32) * 0.05, torch.randn(32)
    v = gemma_rms_norm(x[1:], gamma) @ w_out + b_out
    want = noise + (-0.1) * v
    folded = {"decoder_action_fused_out_proj_w": w_out * (1.0 + gamma)[:, None] * -0.1, "decoder_action_fused_out_proj_b": b_out * -0.1}
    got = pi0.euler_step(folded, x, noise, ops.identity)
    assert torch.allclose(got, want, atol=1e-5)
    # ten such steps with a constant velocity field integrate to noise - v
    z = noise.clone()
    for _ in range(10):
        z = z + (-0.1) * v
    assert torch.allclose(z, noise - v, atol=1e-5)
    # the synthetic checkpoints carry the same fold: their output projection is the raw draw times -0.1
    ck = syn.pi0_checkpoint(2, 0, vision_layers=1, llm_layers=1)
    raw = syn.normal_bf16(2, "decoder_action_fused_out_proj_w", (1024, 32), 0.02)
    assert torch.equal(ck["decoder_action_fused_out_proj_w"], (raw.float() * -0.1).to(torch.bfloat16))


def test_qkv_concatenation_order_and_vision_head_layout():
    """convert_from_jax.py:58-61: [Q (8 x 256) | K (256) | V (256)]; :16-27 SigLIP [Q | K | V] each 16 heads x 72.
    The forward slices exactly these column ranges (pi0_infer.py:801-810, :590-593)."""
    x = torch.randn(4, 16, dtype=torch.float64)
    wq, wk, wv = torch.randn(16, 2048, dtype=torch.float64), torch.randn(16, 256, dtype=torch.float64), torch.randn(16, 256, dtype=torch.float64)
    qkv = x @ torch.cat([wq, wk, wv], dim=1)
    assert torch.allclose(qkv[:, :2048], x @ wq) and torch.allclose(qkv[:, 2048:2304], x @ wk) and torch.allclose(qkv[:, 2304:], x @ wv)
    # SigLIP: head h of Q is columns [72 h, 72 h + 72), of K 1152 + ..., of V 2304 + ...
    q = torch.randn(256, 16, 72); k = torch.randn(256, 16, 72); v = torch.randn(256, 16, 72)
    packed = torch.cat([q.flatten(1), k.flatten(1), v.flatten(1)], dim=1)
    got = ops.vision_attention(packed, ops.identity).reshape(256, 16, 72)
    h = 5
    p = torch.softmax(q[:, h] @ k[:, h].T / math.sqrt(72.0), dim=-1)
    assert torch.allclose(got[:, h], p @ v[:, h], atol=1e-5)
