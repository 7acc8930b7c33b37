"""Pi0 forward restated on the CPU (test infrastructure; see oracle/__init__.py).

Follows /root/reference/pi0_infer.py: vision_encoder :598-646, transformer_encoder
:841-884, transformer_decoder :1165-1230, Pi0Inference :1238-1361.
"""
import torch

from . import ops
from .ops import f32, gemm


def vision_layer(w, i, x, rnd, taps=None):
    """pi0_infer.py:607-646, one SigLIP layer: LN -> QKV(+bias) -> attention -> O(+bias) + residual ->
    LN -> up(+bias) -> GELU -> down(+bias) + residual.  (taps: the stream between the two halves as "vision_mid/i".)"""
    n = rnd(ops.layer_norm(x, w["vision_pre_attn_norm_w"][i], w["vision_pre_attn_norm_b"][i]))
    qkv = rnd(f32(w["vision_attn_qkv_b"][i]) + gemm(n, w["vision_attn_qkv_w"][i]))
    a = ops.vision_attention(qkv, rnd)
    x = rnd(x + f32(w["vision_attn_o_b"][i]) + gemm(a, w["vision_attn_o_w"][i]))
    if taps is not None:
        taps["vision_mid/%d" % i] = x.clone()
    n = rnd(ops.layer_norm(x, w["vision_pre_ffn_norm_w"][i], w["vision_pre_ffn_norm_b"][i]))
    h = rnd(ops.gelu_tanh(f32(w["vision_ffn_up_b"][i]) + gemm(n, w["vision_ffn_up_w"][i])))
    return rnd(x + f32(w["vision_ffn_down_b"][i]) + gemm(h, w["vision_ffn_down_w"][i]))


def vision_encoder(w, images, rnd, taps=None):
    """pi0_infer.py:598-646 -> vision_x [v*256, 1152]."""
    x = ops.patches(f32(images))
    pos = f32(w["vision_position_embedding"]).repeat(images.shape[0], 1)
    x = rnd(pos + f32(w["vision_patch_embedding_b"]) + gemm(x, w["vision_patch_embedding_w"].reshape(588, 1152)))
    if taps is not None:
        taps["vision_embed"] = x.clone()
    for i in range(w["vision_attn_qkv_w"].shape[0]):
        x = vision_layer(w, i, x, rnd, taps)
        if taps is not None:
            taps["vision_x/%d" % i] = x.clone()
    return x


def project_and_concat(w, vision_x, prompt_embeds, rnd):
    """pi0_infer.py:753-775 (final LN + projector, no sqrt(2048) scaling of image tokens)
    and :1343-1345 (language embeddings appended)."""
    n = rnd(ops.layer_norm(vision_x, w["vision_final_norm_w"], w["vision_final_norm_b"]))
    e = rnd(f32(w["encoder_multi_modal_projector_b"]) + gemm(n, w["encoder_multi_modal_projector_w"]))
    return torch.cat([e, f32(prompt_embeds)], dim=0)


def prefix_layer_qkv(w, i, x, table, rnd):
    """pi0_infer.py:812-817: RMS -> QKV GEMM -> bf16 -> interleaved RoPE on Q and K."""
    n = rnd(x * ops.rms_factor(x))
    qkv = rnd(gemm(n, w["encoder_attn_qkv_w"][i]))
    q = rnd(ops.rope_interleaved(qkv[:, :2048], table))
    k = rnd(ops.rope_interleaved(qkv[:, 2048:2304], table))
    v = qkv[:, 2304:]
    return q, k, v


def prefix_layer_rest(w, i, x, q, k, v, rnd, mask=None):
    """pi0_infer.py:862-884: MQA attention, O-proj + residual, RMS, GeGLU, down + residual."""
    a = ops.mqa_attention(q.reshape(-1, 256), k, v, rnd, mask).reshape(-1, 2048)
    x = rnd(x + gemm(a, w["encoder_attn_o_w"][i]))
    n = rnd(x * ops.rms_factor(x))
    g = rnd(ops.gelu_tanh(gemm(n, w["encoder_ffn_gate_w"][i])) * gemm(n, w["encoder_ffn_up_w"][i]))
    return rnd(x + gemm(g, w["encoder_ffn_down_w"][i]))


def transformer_encoder(w, x, rnd, taps=None, valid_len=None):
    """pi0_infer.py:841-884 -> per-layer prefix K and V ([S_e,256] each).  The last layer only
    fills the cache (:862).  `valid_len` (Pi05, pi05_infer.py:303) masks keys >= valid_len."""
    s_e = x.shape[0]
    table = ops.rope_table(0, s_e)
    layers = w["encoder_attn_qkv_w"].shape[0]
    mask = None if valid_len is None else ops.valid_len_mask(8 * s_e, s_e, valid_len)
    ks, vs = [], []
    for i in range(layers):
        q, k, v = prefix_layer_qkv(w, i, x, table, rnd)
        ks.append(k)
        vs.append(v)
        if i != layers - 1:
            x = prefix_layer_rest(w, i, x, q, k, v, rnd, mask)
            if taps is not None:
                taps["encoder_x/%d" % i] = x.clone()
    if taps is not None:
        for i in range(layers):
            taps["encoder_K/%d" % i] = ks[i].clone()
            taps["encoder_V/%d" % i] = vs[i].clone()
    return ks, vs


def suffix_layer(w, i, x, k_prefix, v_prefix, table, mask, rnd):
    """pi0_infer.py:1186-1223, one action-expert layer over the suffix rows x [S_d, 1024] (row 0 = state token):
    RMS factor -> QKV (factor applied to the fp32 accumulator, :1005) -> RoPE -> K/V appended behind the prefix
    rows of this layer's cache (:1191-1192) -> masked attention (:1085) -> O + residual -> RMS factor ->
    GeGLU on the pre-scaled rows (:718) -> down + residual."""
    s_d = x.shape[0]
    f = rnd(ops.rms_factor(x))
    acc = gemm(x, w["decoder_attn_qkv_w"][i]) * f
    q = rnd(ops.rope_interleaved(acc[:, :2048], table))
    k = rnd(ops.rope_interleaved(acc[:, 2048:2304], table))
    v = rnd(acc[:, 2304:])
    kk = torch.cat([k_prefix, k], dim=0)
    vv = torch.cat([v_prefix, v], dim=0)
    a = ops.mqa_attention(q.reshape(-1, 256), kk, vv, rnd, mask).reshape(s_d, 2048)
    x = rnd(x + gemm(a, w["decoder_attn_o_w"][i]))
    f = rnd(ops.rms_factor(x))
    xs = rnd(x * f)                                               # bf16 x * bf16 f -> bf16 before the dot (:718)
    g = rnd(ops.gelu_tanh(gemm(xs, w["decoder_ffn_gate_w"][i])) * gemm(xs, w["decoder_ffn_up_w"][i]))
    return rnd(x + gemm(g, w["decoder_ffn_down_w"][i]))


def euler_step(w, x, noise, rnd):
    """pi0_infer.py:953-964, :1224-1230: noise += (x[1:] * f) W_out + b_out (dt and the final norm scale are
    folded into W_out, b_out by the converter)."""
    xo = x[1:]
    f = rnd(ops.rms_factor(xo))
    xs = rnd(xo * f)                                              # :113
    return rnd(noise + f32(w["decoder_action_fused_out_proj_b"]) + gemm(xs, w["decoder_action_fused_out_proj_w"]))


def transformer_decoder(w, ks, vs, state, noise, rnd, taps=None, num_steps=10):
    """pi0_infer.py:1165-1230: state token + 10 Euler flow steps over the action expert."""
    s_e = ks[0].shape[0]
    chunk = noise.shape[0]
    s_d = chunk + 1
    table = ops.rope_table(s_e, s_d)
    mask = ops.pi0_suffix_mask(s_d, s_e)
    layers = w["decoder_attn_qkv_w"].shape[0]
    noise = f32(noise)
    s = rnd(f32(w["decoder_state_in_proj_b"]) + gemm(f32(state)[None, :], w["decoder_state_in_proj_w"]))
    for t in range(num_steps):
        u = rnd(ops.silu(f32(w["decoder_action_fused_time_biases"][t % 10]) + gemm(noise, w["decoder_action_fused_in_proj_w"])))
        xa = rnd(f32(w["decoder_action_mlp_b"]) + gemm(u, w["decoder_action_mlp_w"]))
        x = torch.cat([s, xa], dim=0)
        if taps is not None:
            taps["decoder_in/%d" % t] = x.clone()
        for i in range(layers):
            x = suffix_layer(w, i, x, ks[i], vs[i], table, mask, rnd)
            if taps is not None:
                taps["decoder_x/%d/%d" % (t, i)] = x.clone()
        noise = euler_step(w, x, noise, rnd)
        if taps is not None:
            taps["noise/%d" % t] = noise.clone()
    return noise


def forward(w, images, state, noise, bf16_boundaries=True, taps=None):
    """Pi0Inference.forward (pi0_infer.py:1356-1361) -> actions [chunk, 32] (fp32 container)."""
    rnd = ops.round_bf16 if bf16_boundaries else ops.identity
    with torch.no_grad():
        vx = vision_encoder(w, images, rnd, taps)
        x = project_and_concat(w, vx, w["language_embeds"], rnd)
        if taps is not None:
            taps["encoder_x0"] = x.clone()
        ks, vs = transformer_encoder(w, x, rnd, taps)
        return transformer_decoder(w, ks, vs, state, noise, rnd, taps)
