"""Where the bf16-boundary oracle rounds.

The oracle has two modes: all-fp32 (pinned by tests/test_oracle_layers.py against second implementations) and the
"bf16-boundary" mode the HIP path is compared with, which rounds to bf16 where the reference writes a bf16 buffer.
Here every stage of the Pi0 and Pi05 forward is written a second time in another style (conv2d patch embedding,
F.layer_norm, complex-number RoPE, per-head attention loops) with every rounding point placed by hand from the
reference's buffer writes and NAMED:

  vision   pi0_infer.py:348-364 patch | :366-382 ln1, ln2, final_ln | :396-419 qkv | :588-596 attn | :498-532 o_res |
           :534-561 up | :563-586 down_res | :753-775 proj
  prefix   :648-663 rms1, rms2 | :777-817 qkv, rope_q, rope_k | :819-824 logits, probs, pv | :826-839 o_res |
           :664-691 geglu | :727-751 down_res
  suffix   Pi0 :886-937 state, u, xa | :939-1039 f1, rope_q, rope_k, v | :1041-1120 logits, probs, pv | :1122-1163 o_res |
           :693-725 f2, xs, geglu | :1224-1230 euler_f, euler_xs, noise
           Pi05 pi05_infer.py:669-722 out_w, out_b, time_h, temb, style | :22-64 x_in, o_res, down_res | :78-113 ada |
           :127-195 rope_q, rope_k, v | :282-309, :382-416 logits, probs, pv | :197-280 geglu | noise

A whole forward cannot tell a misplaced rounding from noise: two fp32 implementations that sum in a different order
already put a few values on the other side of a bf16 boundary, and ten flow steps amplify that to half a bf16 step of
the actions.  So each stage is run ALONE on the oracle's own input for it (its taps), and what is counted is the
fraction of output elements that differ from the oracle's output tap.  Two statements per stage: with all points in
place that fraction is tiny (summation order only), and leaving out any ONE point - or adding one where the reference
has none - raises it by an order of magnitude.  A rounding point that is missing or misplaced in the oracle cannot pass.
"""
import pytest
import torch
import torch.nn.functional as F

import synthetic as syn
from oracle import pi0, pi05


def W(ck, name, i=None):
    t = ck[name] if i is None else ck[name][i]
    return t.float()


class Rounder:
    """R(name, x): x rounded to bf16 unless `name` is skipped; `extra` names round where the reference does not."""
    def __init__(self, skip=(), extra=()):
        self.skip, self.extra, self.seen = set(skip), set(extra), set()

    def __call__(self, name, x):
        self.seen.add(name)
        return x if name in self.skip else x.bfloat16().float()

    def maybe(self, name, x):
        return x.bfloat16().float() if name in self.extra else x


def rope(x, pos):
    """x [rows, heads, 256] as 128 complex numbers per head times exp(i pos 10000^(-2j/256)), table entries bf16."""
    inv = 1.0 / (10000 ** (torch.arange(0, 256, 2, dtype=torch.float32) / 256))
    ph = pos.to(torch.float32)[:, None] * inv[None, :]
    rotor = torch.complex(torch.cos(ph).bfloat16().float(), torch.sin(ph).bfloat16().float())
    z = torch.view_as_complex(x.reshape(x.shape[0], x.shape[1], 128, 2).contiguous())
    return torch.view_as_real(z * rotor[:, None, :]).reshape(x.shape)


def factor(x):
    return torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)


def vision_embed(ck, img, R):
    w = ck["vision_patch_embedding_w"].float().permute(3, 2, 0, 1)
    x = F.conv2d(img.float().permute(0, 3, 1, 2), w, ck["vision_patch_embedding_b"].float(), stride=14)
    return R("v.patch", x.flatten(2).transpose(1, 2) + ck["vision_position_embedding"].float()[None]).reshape(-1, 1152)


def vision_attention_half(ck, i, x, R):
    v = x.shape[0] // 256
    x = x.reshape(v, 256, 1152)
    n = R("v.ln1", F.layer_norm(x, (1152,), W(ck, "vision_pre_attn_norm_w", i), W(ck, "vision_pre_attn_norm_b", i), 1e-5))
    qkv = R("v.qkv", n @ W(ck, "vision_attn_qkv_w", i) + W(ck, "vision_attn_qkv_b", i))
    q, k, val = (t.reshape(v, 256, 16, 72).transpose(1, 2) for t in qkv.split(1152, dim=-1))
    p = torch.softmax(R.maybe("v.logits", q @ k.transpose(-1, -2) * 72 ** -0.5), -1)
    a = R("v.attn", (p @ val).transpose(1, 2).reshape(v, 256, 1152))
    return R("v.o_res", x + a @ W(ck, "vision_attn_o_w", i) + W(ck, "vision_attn_o_b", i)).reshape(-1, 1152)


def vision_mlp_half(ck, i, x, R):
    n = R("v.ln2", F.layer_norm(x, (1152,), W(ck, "vision_pre_ffn_norm_w", i), W(ck, "vision_pre_ffn_norm_b", i), 1e-5))
    h = R("v.up", F.gelu(n @ W(ck, "vision_ffn_up_w", i) + W(ck, "vision_ffn_up_b", i), approximate="tanh"))
    return R("v.down_res", x + h @ W(ck, "vision_ffn_down_w", i) + W(ck, "vision_ffn_down_b", i))


def project(ck, x, R):
    n = R("v.final_ln", F.layer_norm(x, (1152,), W(ck, "vision_final_norm_w"), W(ck, "vision_final_norm_b"), 1e-5))
    return R("v.proj", n @ W(ck, "encoder_multi_modal_projector_w") + W(ck, "encoder_multi_modal_projector_b"))


def heads_attention(q, k, v, visible, R, tag):
    """q [rows, 8, 256] against one shared k, v [keys, 256], head by head; visible [rows, keys]."""
    out = []
    for h in range(8):
        lg = R(tag + ".logits", q[:, h] @ k.t() / 16.0).masked_fill(~visible, float("-inf"))
        out.append(R(tag + ".probs", torch.softmax(lg, -1)) @ v)
    return R(tag + ".pv", torch.stack(out, 1).reshape(q.shape[0], 2048))


def prefix_layer(ck, i, x, valid, R):
    """-> (next stream, K, V) of one Gemma prefix layer."""
    s = x.shape[0]
    pos = torch.arange(s)
    visible = (torch.arange(s)[None, :] < valid).expand(s, s)
    qkv = R("p.qkv", R("p.rms1", x * factor(x)) @ W(ck, "encoder_attn_qkv_w", i))
    q = R("p.rope_q", rope(qkv[:, :2048].reshape(s, 8, 256), pos))
    k = R("p.rope_k", rope(qkv[:, 2048:2304].reshape(s, 1, 256), pos))[:, 0]
    x = R("p.o_res", x + heads_attention(q, k, qkv[:, 2304:], visible, R, "p") @ W(ck, "encoder_attn_o_w", i))
    n = R("p.rms2", x * factor(x))
    g = R("p.geglu", F.gelu(R.maybe("p.gate", n @ W(ck, "encoder_ffn_gate_w", i)), approximate="tanh") * (n @ W(ck, "encoder_ffn_up_w", i)))
    return R("p.down_res", x + g @ W(ck, "encoder_ffn_down_w", i)), k, qkv[:, 2304:]


def pi0_step_begin(ck, state, noise, t, R):
    st = R("s.state", state.float()[None] @ W(ck, "decoder_state_in_proj_w") + W(ck, "decoder_state_in_proj_b"))
    u = R("s.u", F.silu(noise @ W(ck, "decoder_action_fused_in_proj_w") + W(ck, "decoder_action_fused_time_biases", t)))
    return torch.cat([st, R("s.xa", u @ W(ck, "decoder_action_mlp_w") + W(ck, "decoder_action_mlp_b"))])


def pi0_suffix_layer(ck, i, x, kp, vp, R):
    s_e, s_d = kp.shape[0], x.shape[0]
    pos = s_e + torch.arange(s_d)
    visible = torch.ones(s_d, s_e + s_d, dtype=torch.bool)
    visible[0, s_e + 1:] = False                                                                  # the state token: prefix and itself
    acc = R.maybe("s.acc", (x @ W(ck, "decoder_attn_qkv_w", i)) * R("s.f1", factor(x)))           # the factor multiplies the fp32 accumulator
    q = R("s.rope_q", rope(acc[:, :2048].reshape(s_d, 8, 256), pos))
    k = R("s.rope_k", rope(acc[:, 2048:2304].reshape(s_d, 1, 256), pos))[:, 0]
    v = R("s.v", acc[:, 2304:])
    x = R("s.o_res", x + heads_attention(q, torch.cat([kp, k]), torch.cat([vp, v]), visible, R, "s") @ W(ck, "decoder_attn_o_w", i))
    xs = R("s.xs", x * R("s.f2", factor(x)))                                                      # rounded rows before the dot
    g = R("s.geglu", F.gelu(xs @ W(ck, "decoder_ffn_gate_w", i), approximate="tanh") * (xs @ W(ck, "decoder_ffn_up_w", i)))
    return R("s.down_res", x + g @ W(ck, "decoder_ffn_down_w", i))


def pi0_euler(ck, x, noise, R):
    xs = R("s.euler_xs", x[1:] * R("s.euler_f", factor(x[1:])))
    return R("s.noise", noise + xs @ W(ck, "decoder_action_fused_out_proj_w") + W(ck, "decoder_action_fused_out_proj_b"))


def pi05_temb(ck, t, R):
    h = R("s.time_h", F.silu(W(ck, "decoder_time_embeds", t) @ W(ck, "decoder_time_mlp_in_w") + W(ck, "decoder_time_mlp_in_b")))
    return R("s.temb", F.silu(h @ W(ck, "decoder_time_mlp_out_w") + W(ck, "decoder_time_mlp_out_b")))


def pi05_ada(x, style, R):
    sc, sh, gt = style.split(1024)
    return R("s.ada", x * factor(x) * (1 + sc) + sh), gt


def pi05_suffix_layer(ck, i, t, x, kp, vp, valid, R):
    s_alloc, s_d = kp.shape[0], x.shape[0]
    pos = valid - 1 + torch.arange(s_d)
    visible = torch.ones(s_d, s_alloc + s_d, dtype=torch.bool)
    visible[:, valid:s_alloc] = False
    temb = pi05_temb(ck, t, R)
    n, gt = pi05_ada(x, R("s.style", temb @ W(ck, "decoder_pre_attn_norm_mod_w", i) + W(ck, "decoder_pre_attn_norm_mod_b", i)), R)
    acc = n @ W(ck, "decoder_attn_qkv_w", i)
    q = R("s.rope_q", rope(acc[:, :2048].reshape(s_d, 8, 256), pos))
    k = R("s.rope_k", rope(acc[:, 2048:2304].reshape(s_d, 1, 256), pos))[:, 0]
    v = R("s.v", acc[:, 2304:])
    a = heads_attention(q, torch.cat([kp, k]), torch.cat([vp, v]), visible, R, "s")
    x = R("s.o_res", x + (a @ W(ck, "decoder_attn_o_w", i)) * gt)
    n, gt = pi05_ada(x, R("s.style", temb @ W(ck, "decoder_pre_ffn_norm_mod_w", i) + W(ck, "decoder_pre_ffn_norm_mod_b", i)), R)
    g = R("s.geglu", F.gelu(n @ W(ck, "decoder_ffn_gate_w", i), approximate="tanh") * (n @ W(ck, "decoder_ffn_up_w", i)))
    return R("s.down_res", x + (g @ W(ck, "decoder_ffn_down_w", i)) * gt)


def pi05_step_end(ck, t, x, noise, R):
    w_out, b_out = R("s.out_w", W(ck, "decoder_action_out_proj_w") * -0.1), R("s.out_b", W(ck, "decoder_action_out_proj_b") * -0.1)
    n, _ = pi05_ada(x, R("s.style", pi05_temb(ck, t, R) @ W(ck, "decoder_final_norm_mod_w") + W(ck, "decoder_final_norm_mod_b")), R)
    return R("s.noise", noise + n @ w_out + b_out)


# ---------------------------------------------------------------------------------------------------------
BASE_MAX = 4e-2      # fraction of elements that may differ with every point in place (fp32 summation order, spread by the GEMMs of the stage)
LOUDER = 3.5         # one omission / addition must differ in at least this many times more elements, and in at least MIN_FRAC of them
MIN_FRAC = 3e-3


def mismatch(got, want):
    if not isinstance(got, (tuple, list)):
        got, want = [got], [want]
    bad = sum((g != w).sum().item() for g, w in zip(got, want))
    return bad / sum(w.numel() for w in want)


def check_stage(label, run, want, points, extra=()):
    full = Rounder()
    base = mismatch(run(full), want)
    assert set(points) <= full.seen, (label, set(points) - full.seen)
    assert base <= BASE_MAX, (label, base)
    floor = max(LOUDER * base, MIN_FRAC)
    report = {}
    for n in points:
        report["-" + n] = mismatch(run(Rounder(skip=[n])), want)
    for n in extra:
        report["+" + n] = mismatch(run(Rounder(extra=[n])), want)
    print("%-22s all points: %.1e of the elements differ; one point left out (-) or added (+): %s" %
          (label, base, ", ".join("%s %.1e" % kv for kv in report.items())))
    quiet = {k: v for k, v in report.items() if v < floor}
    assert not quiet, (label, base, quiet)


@pytest.fixture(scope="module")
def pi0_case():
    ck = syn.pi0_checkpoint(31, 3, vision_layers=2, llm_layers=3, norms="random")
    img, state, noise = syn.observation(31, 2, 5)
    taps = {}
    pi0.forward(ck, img, state, noise, bf16_boundaries=True, taps=taps)
    return ck, img, state, noise, taps


@pytest.fixture(scope="module")
def pi05_case():
    ck = syn.pi05_checkpoint(32, 3, vision_layers=1, llm_layers=2, state_tokens=2, norms="random")
    img, _, noise = syn.observation(32, 1, 6)
    taps = {}
    pi05.forward(ck, img, noise, max_prompt_len=9, bf16_boundaries=True, taps=taps)
    return ck, img, noise, taps


def test_pi0_vision_and_prefix_rounding_points(pi0_case):
    ck, img, state, noise, t = pi0_case
    print()
    check_stage("patch embedding", lambda R: vision_embed(ck, img, R), t["vision_embed"], ["v.patch"])
    check_stage("SigLIP layer 1, attention", lambda R: vision_attention_half(ck, 1, t["vision_x/0"], R), t["vision_mid/1"],
                ["v.ln1", "v.qkv", "v.attn", "v.o_res"], extra=["v.logits"])
    check_stage("SigLIP layer 1, MLP", lambda R: vision_mlp_half(ck, 1, t["vision_mid/1"], R), t["vision_x/1"], ["v.ln2", "v.up", "v.down_res"])
    s_v = 512
    check_stage("projector", lambda R: project(ck, t["vision_x/1"], R), t["encoder_x0"][:s_v], ["v.final_ln", "v.proj"])
    s_e = t["encoder_x0"].shape[0]
    check_stage("prefix layer 1", lambda R: prefix_layer(ck, 1, t["encoder_x/0"], s_e, R), (t["encoder_x/1"], t["encoder_K/1"], t["encoder_V/1"]),
                ["p.rms1", "p.qkv", "p.rope_q", "p.rope_k", "p.logits", "p.probs", "p.pv", "p.o_res", "p.rms2", "p.geglu", "p.down_res"], extra=["p.gate"])


def test_pi0_action_expert_rounding_points(pi0_case):
    ck, img, state, noise, t = pi0_case
    print()
    check_stage("step 3 inputs", lambda R: pi0_step_begin(ck, state, t["noise/2"], 3, R), t["decoder_in/3"], ["s.state", "s.u", "s.xa"])
    check_stage("action-expert layer 1", lambda R: pi0_suffix_layer(ck, 1, t["decoder_x/3/0"], t["encoder_K/1"], t["encoder_V/1"], R), t["decoder_x/3/1"],
                ["s.f1", "s.rope_q", "s.rope_k", "s.v", "s.logits", "s.probs", "s.pv", "s.o_res", "s.f2", "s.xs", "s.geglu", "s.down_res"], extra=["s.acc"])
    check_stage("Euler step 3", lambda R: pi0_euler(ck, t["decoder_x/3/2"], t["noise/2"], R), t["noise/3"], ["s.euler_f", "s.euler_xs", "s.noise"])


def test_pi05_action_expert_rounding_points(pi05_case):
    ck, img, noise, t = pi05_case
    valid = 256 + 3 + 2
    print()
    check_stage("Pi05 step 4 input", lambda R: R("s.x_in", t["noise/3"] @ W(ck, "decoder_action_in_proj_w") + W(ck, "decoder_action_in_proj_b")),
                t["decoder_in/4"], ["s.x_in"])
    check_stage("Pi05 action-expert layer 1", lambda R: pi05_suffix_layer(ck, 1, 4, t["decoder_x/4/0"], t["encoder_K/1"], t["encoder_V/1"], valid, R),
                t["decoder_x/4/1"], ["s.time_h", "s.temb", "s.style", "s.ada", "s.rope_q", "s.rope_k", "s.v", "s.logits", "s.probs", "s.pv",
                                     "s.o_res", "s.geglu", "s.down_res"])
    check_stage("Pi05 Euler step 4", lambda R: pi05_step_end(ck, 4, t["decoder_x/4/1"], t["noise/3"], R), t["noise/4"],
                ["s.out_w", "s.out_b", "s.time_h", "s.temb", "s.style", "s.ada", "s.noise"])
