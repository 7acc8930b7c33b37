"""Model-level pins of the CPU oracle: independent per-token / per-head restatements of one layer,
invariants of the schedule (Euler update, masks, padding, gating) and the committed golden vectors."""
import os

import pytest
import torch

import synthetic as syn
from oracle import ops, pi0, pi05

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "golden_small.pt")


@pytest.fixture(scope="module")
def small_pi0():
    ck = syn.pi0_checkpoint(7, 4, vision_layers=2, llm_layers=2, norms="random")
    img, st, nz = syn.observation(7, 1, 10)
    return ck, img, st, nz


@pytest.fixture(scope="module")
def small_pi05():
    ck = syn.pi05_checkpoint(9, 4, vision_layers=2, llm_layers=2, state_tokens=3, norms="random")
    img, _, nz = syn.observation(9, 1, 10)
    return ck, img, nz


def test_golden_small_vectors(small_pi0, small_pi05):
    g = torch.load(GOLDEN, weights_only=True)
    ck, img, st, nz = small_pi0
    taps = {}
    out = pi0.forward(ck, img, st, nz, taps=taps)
    # fp32 summation order inside the CPU BLAS depends on the host and thread count, so the pin is a
    # tight tolerance rather than bit equality
    close = lambda a, b, tol=3e-3: (a.float() - b.float()).abs().mean().item() <= tol
    assert close(out, g["pi0_small/actions"])
    assert torch.allclose(pi0.forward(ck, img, st, nz, bf16_boundaries=False), g["pi0_small/actions_fp32"], atol=1e-5)
    for name in ("vision_embed", "encoder_x0", "encoder_K/1", "decoder_x/9/1", "noise/9"):
        assert close(taps[name][:8], g["pi0_small/tap/" + name], 3e-3 * max(1.0, g["pi0_small/tap/" + name].float().abs().mean().item()))
    ck5, img5, nz5 = small_pi05
    out5 = pi05.forward(ck5, img5, nz5, max_prompt_len=12)
    assert close(out5, g["pi05_small/actions"])


def test_bf16_and_fp32_variants_agree_within_tolerance(small_pi0):
    ck, img, st, nz = small_pi0
    a = pi0.forward(ck, img, st, nz)
    b = pi0.forward(ck, img, st, nz, bf16_boundaries=False)
    assert (a - b).abs().mean().item() < 1e-2


def test_euler_update_with_zero_output_projection_returns_the_noise(small_pi0):
    ck, img, st, nz = small_pi0
    ck = dict(ck)
    ck["decoder_action_fused_out_proj_w"] = torch.zeros_like(ck["decoder_action_fused_out_proj_w"])
    ck["decoder_action_fused_out_proj_b"] = torch.zeros_like(ck["decoder_action_fused_out_proj_b"])
    assert torch.equal(pi0.forward(ck, img, st, nz), nz.float())


def test_euler_update_is_ten_bias_steps_when_weights_vanish(small_pi0):
    ck, img, st, nz = small_pi0
    ck = dict(ck)
    ck["decoder_action_fused_out_proj_w"] = torch.zeros_like(ck["decoder_action_fused_out_proj_w"])
    b = ck["decoder_action_fused_out_proj_b"].float()
    want = nz.float()
    for _ in range(10):
        want = ops.round_bf16(want + b)
    assert torch.equal(pi0.forward(ck, img, st, nz), want)


def test_prefix_layer_against_per_token_loops(small_pi0):
    """One Gemma prefix layer restated token by token and head by head (fp32, no rounding)."""
    ck = small_pi0[0]
    torch.manual_seed(1)
    s_e = 6
    x = torch.randn(s_e, 2048)
    tab = ops.rope_table(0, s_e)
    q, k, v = pi0.prefix_layer_qkv(ck, 0, x, tab, ops.identity)
    got = pi0.prefix_layer_rest(ck, 0, x, q, k, v, ops.identity)
    wq = ck["encoder_attn_qkv_w"][0].float()
    n = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    rows = []
    for t in range(s_e):
        full = n[t] @ wq                                   # [2560] = Q(8x256) | K | V
        rows.append(full)
    full = torch.stack(rows)

    def rot(vec, pos):                                     # interleaved pairs, angle pos * 10000^(-2j/256)
        out = vec.clone()
        for j in range(128):
            c, s = tab[pos, 2 * j], tab[pos, 2 * j + 1]
            out[2 * j] = vec[2 * j] * c - vec[2 * j + 1] * s
            out[2 * j + 1] = vec[2 * j + 1] * c + vec[2 * j] * s
        return out

    kk = torch.stack([rot(full[t, 2048:2304], t) for t in range(s_e)])
    vv = full[:, 2304:]
    attn = torch.zeros(s_e, 2048)
    for t in range(s_e):
        for h in range(8):
            qh = rot(full[t, h * 256:(h + 1) * 256], t)
            p = torch.softmax((kk @ qh) / 16.0, 0)
            attn[t, h * 256:(h + 1) * 256] = p @ vv
    x1 = x + attn @ ck["encoder_attn_o_w"][0].float()
    n1 = x1 / torch.sqrt((x1 * x1).mean(-1, keepdim=True) + 1e-6)
    g = torch.nn.functional.gelu(n1 @ ck["encoder_ffn_gate_w"][0].float(), approximate="tanh") * (n1 @ ck["encoder_ffn_up_w"][0].float())
    want = x1 + g @ ck["encoder_ffn_down_w"][0].float()
    assert torch.allclose(got, want, atol=2e-3, rtol=1e-3)


def test_pi05_is_independent_of_prefix_padding(small_pi05):
    """Rows past the valid prompt length are masked as keys and never read as queries, and the
    suffix RoPE offset follows the valid length: the allocation size must not change the result."""
    ck, img, nz = small_pi05
    a = pi05.forward(ck, img, nz, max_prompt_len=7, bf16_boundaries=False)
    b = pi05.forward(ck, img, nz, max_prompt_len=19, bf16_boundaries=False)
    assert torch.allclose(a, b, atol=1e-5)                 # (the CPU BLAS sums in a shape-dependent order, hence not bit-equal)
    a = pi05.forward(ck, img, nz, max_prompt_len=7)
    b = pi05.forward(ck, img, nz, max_prompt_len=19)
    assert (a - b).abs().mean().item() < 1e-4 and (a != b).float().mean().item() < 0.05      # a few single-ulp flips at most


def test_pi05_zero_gate_freezes_the_residual_stream(small_pi05):
    ck, img, nz = small_pi05
    ck = dict(ck)
    for k in ("decoder_pre_attn_norm_mod_w", "decoder_pre_ffn_norm_mod_w"):
        w = ck[k].clone(); w[:, :, 2048:] = 0; ck[k] = w
    for k in ("decoder_pre_attn_norm_mod_b", "decoder_pre_ffn_norm_mod_b"):
        b = ck[k].clone(); b[:, 2048:] = 0; ck[k] = b
    taps = {}
    pi05.forward(ck, img, nz, taps=taps)
    x0 = ops.round_bf16(ck["decoder_action_in_proj_b"].float() + nz.float() @ ck["decoder_action_in_proj_w"].float())
    assert torch.equal(taps["decoder_x/0/1"], x0)


def test_pi05_conditioning_against_direct_formula(small_pi05):
    ck = small_pi05[0]
    out_w, out_b, attn, ffn, final = pi05.conditioning(ck, ops.identity)
    t, i = 3, 1
    tau = ck["decoder_time_embeds"][t].float()
    h = torch.nn.functional.silu(tau @ ck["decoder_time_mlp_in_w"].float() + ck["decoder_time_mlp_in_b"].float())
    temb = torch.nn.functional.silu(h @ ck["decoder_time_mlp_out_w"].float() + ck["decoder_time_mlp_out_b"].float())
    want = temb @ ck["decoder_pre_ffn_norm_mod_w"][i].float() + ck["decoder_pre_ffn_norm_mod_b"][i].float()
    assert torch.allclose(ffn[t][i], want, atol=1e-4)
    assert torch.allclose(out_w, ck["decoder_action_out_proj_w"].float() * -0.1)
    assert len(attn) == 10 and len(attn[0]) == 2 and final[0].shape == (3072,)


def test_adarms_reduces_to_rms_norm_with_zero_style():
    x = torch.randn(4, 1024)
    n, gate = pi05.adarms(x, torch.zeros(3072), ops.identity)
    assert torch.allclose(n, x * ops.rms_factor(x)) and torch.all(gate == 0)


def test_pi0_runs_with_an_empty_prompt():
    ck = syn.pi0_checkpoint(8, 0, vision_layers=1, llm_layers=2, norms="random")
    img, st, nz = syn.observation(8, 1, 63)
    out = pi0.forward(ck, img, st, nz)
    g = torch.load(GOLDEN, weights_only=True)
    assert out.shape == (63, 32) and (out - g["pi0_small_noprompt_c63/actions"].float()).abs().mean().item() <= 3e-3
