"""Pi05 forward restated on the CPU (test infrastructure; see oracle/__init__.py).

Follows /root/reference/pi05_infer.py: constructor-time conditioning :669-722,
transformer_encoder :311-380, transformer_decoder :418-523, forward :804-826.
"""
import torch

from . import ops, pi0
from .ops import f32, gemm


def conditioning(w, rnd, num_steps=10):
    """pi05_infer.py:669-722: out-proj scaled by -1/num_steps; per step
    temb = silu(silu(tau W_in + b_in) W_out + b_out) and the [scale|shift|gate] style vectors
    of the 18 attention norms, 18 FFN norms and the final norm."""
    dt = -1.0 / num_steps
    out_w = rnd(f32(w["decoder_action_out_proj_w"]) * dt)
    out_b = rnd(f32(w["decoder_action_out_proj_b"]) * dt)
    layers = w["decoder_attn_qkv_w"].shape[0]
    attn, ffn, final = [], [], []
    for t in range(num_steps):
        tau = f32(w["decoder_time_embeds"][t])[None, :]
        h = rnd(ops.silu(f32(w["decoder_time_mlp_in_b"]) + gemm(tau, w["decoder_time_mlp_in_w"])))
        temb = rnd(ops.silu(f32(w["decoder_time_mlp_out_b"]) + gemm(h, w["decoder_time_mlp_out_w"])))
        attn.append([rnd(f32(w["decoder_pre_attn_norm_mod_b"][i]) + gemm(temb, w["decoder_pre_attn_norm_mod_w"][i]))[0] for i in range(layers)])
        ffn.append([rnd(f32(w["decoder_pre_ffn_norm_mod_b"][i]) + gemm(temb, w["decoder_pre_ffn_norm_mod_w"][i]))[0] for i in range(layers)])
        final.append(rnd(f32(w["decoder_final_norm_mod_b"]) + gemm(temb, w["decoder_final_norm_mod_w"]))[0])
    return out_w, out_b, attn, ffn, final


def adarms(x, style, rnd):
    """pi05_infer.py:78-113: fp32 RMS normalise, then x_hat * (1 + scale) + shift; returns (normed, gate)."""
    scale, shift, gate = style[:1024], style[1024:2048], style[2048:]
    return rnd(x * ops.rms_factor(x) * (1.0 + scale) + shift), gate


def suffix_layer(w, i, x, k_prefix, v_prefix, style_attn, style_ffn, table, mask, rnd):
    """pi05_infer.py:427-509, one action-expert layer: adaRMS(attention style) -> QKV -> RoPE -> K/V appended
    behind the allocated prefix rows -> prefix/suffix-masked attention -> gated O + residual ->
    adaRMS(FFN style) -> GeGLU -> gated down + residual."""
    s_d = x.shape[0]
    n, gate = adarms(x, style_attn, rnd)
    acc = gemm(n, w["decoder_attn_qkv_w"][i])
    q = rnd(ops.rope_interleaved(acc[:, :2048], table))
    k = rnd(ops.rope_interleaved(acc[:, 2048:2304], table))
    v = rnd(acc[:, 2304:])
    kk = torch.cat([k_prefix, k], dim=0)
    vv = torch.cat([v_prefix, v], dim=0)
    a = ops.mqa_attention(q.reshape(-1, 256), kk, vv, rnd, mask).reshape(s_d, 2048)
    x = rnd(x + gemm(a, w["decoder_attn_o_w"][i]) * gate)         # pi05_infer.py:58
    n, gate = adarms(x, style_ffn, rnd)
    g = rnd(ops.gelu_tanh(gemm(n, w["decoder_ffn_gate_w"][i])) * gemm(n, w["decoder_ffn_up_w"][i]))
    return rnd(x + gemm(g, w["decoder_ffn_down_w"][i]) * gate)


def transformer_decoder(w, ks, vs, noise, valid_len, rnd, taps=None, num_steps=10):
    """pi05_infer.py:418-523.  `ks`/`vs` hold the allocated prefix rows (valid or not); suffix
    RoPE positions start at valid_len - 1 (pi05_infer.py:787-790)."""
    s_e_alloc = ks[0].shape[0]
    s_d = noise.shape[0]
    out_w, out_b, st_attn, st_ffn, st_final = conditioning(w, rnd, num_steps)
    table = ops.rope_table(valid_len - 1, s_d)
    mask = ops.pi05_suffix_mask(s_d, s_e_alloc, valid_len)
    layers = w["decoder_attn_qkv_w"].shape[0]
    noise = f32(noise)
    for t in range(num_steps):
        x = rnd(f32(w["decoder_action_in_proj_b"]) + gemm(noise, w["decoder_action_in_proj_w"]))
        if taps is not None:
            taps["decoder_in/%d" % t] = x.clone()
        for i in range(layers):
            x = suffix_layer(w, i, x, ks[i], vs[i], st_attn[t][i], st_ffn[t][i], table, mask, rnd)
            if taps is not None:
                taps["decoder_x/%d/%d" % (t, i)] = x.clone()
        n, _ = adarms(x, st_final[t], rnd)
        noise = rnd(noise + out_b + n @ out_w)
        if taps is not None:
            taps["noise/%d" % t] = noise.clone()
    return noise


def forward(w, images, noise, prompt_embeds=None, max_prompt_len=None, bf16_boundaries=True, taps=None):
    """Pi05Inference.forward (pi05_infer.py:804-826) with the prompt given as embeddings
    (`language_embeds` route, :816-818).  The prefix is allocated for `max_prompt_len` tokens;
    rows past the valid length are zero here (uninitialised in the reference) and masked."""
    rnd = ops.round_bf16 if bf16_boundaries else ops.identity
    if prompt_embeds is None:
        prompt_embeds = w["language_embeds"]
    plen = prompt_embeds.shape[0]
    if max_prompt_len is None:
        max_prompt_len = plen
    with torch.no_grad():
        vx = pi0.vision_encoder(w, images, rnd, taps)
        pad = torch.zeros(max_prompt_len - plen, 2048)
        x = torch.cat([pi0.project_and_concat(w, vx, prompt_embeds, rnd), pad], dim=0)
        valid_len = vx.shape[0] + plen
        if taps is not None:
            taps["encoder_x0"] = x.clone()
        ks, vs = pi0.transformer_encoder(w, x, rnd, taps, valid_len=valid_len)
        return transformer_decoder(w, ks, vs, noise, valid_len, rnd, taps)
