"""DM0 forward restated on the CPU (test infrastructure; see oracle/__init__.py).

Follows /root/reference/dm0_infer.py: run_vision_forward :690-761 (23-layer ViT on 728 x 728 images with a class
token, 2-D rotary embedding, LayerNorm folded into the following GEMM through column sums, two stride-2 3x3
convolutions and a projector), run_prefix_forward :874-955 (28 Qwen-style layers: RMS factor applied after the QKV
GEMM, per-head QK-norm, interleaved RoPE, causal grouped-query attention 16 q / 8 kv heads x 128, SiLU-gated MLP),
transformer_decoder :763-872 (10 Euler steps over a 28-layer action expert attending to the prefix cache),
DM0Inference :965-1116.  fp32 inside every dot product, reduction and transcendental; `rnd` rounds to bf16 where the
reference writes a bf16 buffer.

Parity status: the reference holds no vectors for this path; every function here is pinned by
tests/test_oracle_dm0.py against independent statements (F.layer_norm then matmul for the folded LayerNorm, conv2d
for both im2col paths, scaled_dot_product_attention with explicit masks and repeated KV heads for the grouped
attention, complex-number rotations for both rotary embeddings, per-token loops for a whole layer).  Unpinned at the
bit level: the order in which torch.compile fuses the bf16 arithmetic of the vision rotary embedding
(dm0_infer.py:581-598) and the in-place bf16 adds.
"""
import math

import torch

from . import ops
from .ops import f32, gemm

GRID = 52                      # 728 / 14 patches per side
SEQ = GRID * GRID + 1          # + class token
VIT_HEADS, VIT_HD = 16, 64
Q_HEADS, KV_HEADS, HD = 16, 8, 128


def silu(a):
    return a * torch.sigmoid(a)


def vision_patches(images):
    """dm0_infer.py:695-696: NCHW [n,3,728,728] -> [n*2704, 588], feature order (c, dy, dx)."""
    n = images.shape[0]
    return images.reshape(n, 3, GRID, 14, GRID, 14).permute(0, 2, 4, 1, 3, 5).reshape(n * GRID * GRID, 588)


def ln_stats(x):
    """dm0_infer.py:442-454: mean and rsqrt(E[x^2] - mean^2 + 1e-5) per row."""
    mean = x.mean(-1, keepdim=True)
    var = (x * x).mean(-1, keepdim=True) - mean * mean
    return mean, torch.rsqrt(var + 1e-5)


def ln_folded_gemm(x, w_fused, col_sum, bias_fused):
    """dm0_infer.py:456-495: rstd * (x W' - mean * colsum(W')) + b', the LayerNorm scale and shift folded into W', b'."""
    mean, rstd = ln_stats(x)
    return rstd * (gemm(x, w_fused) - mean * f32(col_sum)) + f32(bias_fused)


def vision_rope_table(grid_h=GRID, grid_w=GRID, head_dim=VIT_HD, theta=10000.0):
    """dm0_infer.py:671-688: per token (class token first, all zeros) 64 angles = [32 from the column index | 32 from the
    row index], each of the 16 frequencies repeated twice, indices starting at 1; angles rounded to bf16, then cos / sin
    rounded to bf16.  Returns (cos, sin) [1 + grid_h*grid_w, 64]."""
    dim_axis = head_dim // 2
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim_axis, 2)[: dim_axis // 2].float() / dim_axis))
    gh = torch.arange(grid_h, dtype=torch.float32) + 1
    gw = torch.arange(grid_w, dtype=torch.float32) + 1
    fh = (gh[:, None] * inv_freq[None, :]).repeat_interleave(2, dim=-1)[:, None, :].expand(grid_h, grid_w, -1)
    fw = (gw[:, None] * inv_freq[None, :]).repeat_interleave(2, dim=-1)[None, :, :].expand(grid_h, grid_w, -1)
    freqs = torch.cat([fw, fh], dim=-1).reshape(grid_h * grid_w, -1)
    freqs = torch.cat([torch.zeros(1, freqs.shape[-1]), freqs], dim=0)
    freqs = ops.round_bf16(freqs)
    return ops.round_bf16(freqs.cos()), ops.round_bf16(freqs.sin())


def vision_rope(t, cos, sin):
    """dm0_infer.py:581-587, :665-669: t * cos + rotate_half(t) * sin with rotate_half((a, b)) = (-b, a) on adjacent pairs.
    t [..., seq, 64]."""
    pairs = t.reshape(*t.shape[:-1], -1, 2)
    rot = torch.stack((-pairs[..., 1], pairs[..., 0]), dim=-1).reshape(t.shape)
    return t * cos + rot * sin


def vision_attention(qkv, n, cos, sin, rnd):
    """dm0_infer.py:589-598: [Q | K | V] each 16 heads x 64, rotary on Q and K, softmax(q k^T / 8) v per image and head."""
    q, k, v = qkv.reshape(n, SEQ, 3, VIT_HEADS, VIT_HD).permute(2, 0, 3, 1, 4)            # each [n, heads, seq, 64]
    q = rnd(vision_rope(q, cos, sin))
    k = rnd(vision_rope(k, cos, sin))
    p = torch.softmax((q @ k.transpose(-1, -2)) * (VIT_HD ** -0.5), dim=-1)
    return rnd((p @ v).transpose(1, 2).reshape(n * SEQ, VIT_HEADS * VIT_HD))


def vision_layer(w, i, x, n, cos, sin, rnd):
    """dm0_infer.py:718-736."""
    qkv = rnd(ln_folded_gemm(x, w["vision_fused_qkv_w"][i], w["vision_qkv_col_sum"][i], w["vision_fused_qkv_b"][i]))
    a = vision_attention(qkv, n, cos, sin, rnd)
    x = rnd(x + f32(w["vision_out_proj_b"][i]) + gemm(a, w["vision_out_proj_w"][i]))
    h = rnd(ops.gelu_tanh(ln_folded_gemm(x, w["vision_fused_fc_w"][i], w["vision_fc_col_sum"][i], w["vision_fused_fc_b"][i])))
    return rnd(x + f32(w["vision_proj_b"][i]) + gemm(h, w["vision_proj_w"][i]))


def im2col_nhwc(x, kernel, stride, padding):
    """dm0_infer.py:532-559: NHWC [b,h,w,c] -> [b*oh*ow, k*k*c], column order (ky, kx, c), zero padding."""
    b, h, w_, c = x.shape
    oh = (h + 2 * padding - kernel) // stride + 1
    ow = (w_ + 2 * padding - kernel) // stride + 1
    xp = torch.zeros(b, h + 2 * padding, w_ + 2 * padding, c, dtype=x.dtype)
    xp[:, padding:padding + h, padding:padding + w_] = x
    cols = []
    for ky in range(kernel):
        for kx in range(kernel):
            cols.append(xp[:, ky: ky + stride * oh: stride, kx: kx + stride * ow: stride, :])
    return torch.stack(cols, dim=3).reshape(b * oh * ow, kernel * kernel * c), oh, ow


def conv_downsample(x, weight, bias, rnd):
    """dm0_infer.py:631-658: 3x3 stride-2 pad-1 convolution as im2col + GEMM (rounded to bf16), then the bias added to the
    bf16 result in place (a second rounding)."""
    b = x.shape[0]
    col, oh, ow = im2col_nhwc(x, 3, 2, 1)
    out = rnd(gemm(col, weight.reshape(-1, weight.shape[-1])))
    return rnd(out + f32(bias)).reshape(b, oh, ow, -1)


def vision_forward(w, images, input_ids, rnd, taps=None):
    """dm0_infer.py:690-761 -> prefix_x [n*169 + len(input_ids), 2048]."""
    n = images.shape[0]
    x = rnd(gemm(vision_patches(f32(images)), w["vision_conv1_w_t"])).reshape(n, GRID * GRID, 1024)
    x = torch.cat([f32(w["vision_class_embedding"]).expand(n, 1, 1024), x], dim=1)
    x = rnd(x + f32(w["vision_pos_emb"])[None, :SEQ]).reshape(n * SEQ, 1024)
    mean, rstd = ln_stats(x)
    x = rnd((x - mean) * rstd * f32(w["vision_ln_pre_w"]) + f32(w["vision_ln_pre_b"]))
    if taps is not None:
        taps["vision_embed"] = x.clone()
    cos, sin = vision_rope_table()
    for i in range(w["vision_fused_qkv_w"].shape[0]):
        x = vision_layer(w, i, x, n, cos, sin, rnd)
        if taps is not None:
            taps["vision_x/%d" % i] = x.clone()
    x = x.reshape(n, SEQ, 1024)[:, 1:].reshape(n, GRID, GRID, 1024)
    x = conv_downsample(x, w["vision_ds1_w"], w["vision_ds1_b"], rnd)
    x = conv_downsample(x, w["vision_ds2_w"], w["vision_ds2_b"], rnd)
    tokens = rnd(gemm(x.reshape(-1, 4096), w["vision_projector_w_t"]))
    if taps is not None:
        taps["image_tokens"] = tokens.clone()
    if input_ids is not None and input_ids.numel():
        tokens = torch.cat([tokens, f32(w["vision_embed_tokens_w"][input_ids.long()])], dim=0)
    return tokens


def rope_table(start, count, theta=1000000.0):
    """dm0_infer.py:1087-1100: rows [cos_0, sin_0, cos_1, sin_1, ...] (bf16) for positions start .., 64 frequencies
    theta^(-2i/128)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, HD, 2, dtype=torch.float32) / HD))
    ang = torch.arange(start, start + count, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.stack([ops.round_bf16(torch.cos(ang)), ops.round_bf16(torch.sin(ang))], dim=2).reshape(count, HD)


def qknorm_rope_split(qkv, factor, q_norm_w, k_norm_w, table, rnd):
    """dm0_infer.py:236-306: the bf16 QKV rows times the row's RMS factor; every Q and K head RMS-normalised over its 128
    features (eps 1e-6) and scaled by the norm weight, then rotated on adjacent pairs; V only scaled.
    -> q [rows, 16, 128], k [rows, 8, 128], v [rows, 8, 128]."""
    rows = qkv.shape[0]
    val = (qkv * factor).reshape(rows, Q_HEADS + 2 * KV_HEADS, HD)
    q, k, v = val[:, :Q_HEADS], val[:, Q_HEADS:Q_HEADS + KV_HEADS], val[:, Q_HEADS + KV_HEADS:]

    def norm_rope(t, nw):
        return _rope_heads(t * torch.rsqrt((t * t).mean(-1, keepdim=True) + 1e-6) * f32(nw), table)
    return rnd(norm_rope(q, q_norm_w)), rnd(norm_rope(k, k_norm_w)), rnd(v)


def _rope_heads(t, table):
    """Rotate adjacent pairs of every head of t [rows, heads, 128] by the angles of table [rows, 128] = (cos, sin) pairs."""
    rows, heads, _ = t.shape
    th = t.reshape(rows, heads, HD // 2, 2)
    tb = table.reshape(rows, 1, HD // 2, 2)
    c, s = tb[..., 0], tb[..., 1]
    x0, x1 = th[..., 0], th[..., 1]
    return torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1).reshape(rows, heads, HD)


def gqa_attention(q, k, v, rnd, causal):
    """dm0_infer.py:913-918 (prefix, causal) and :822-826 (decoder, all keys): q [rows, 16, 128]; k, v [keys, 8, 128]; query
    head h reads KV head h // 2; scale 1/sqrt(128).  With `causal` query row r sees keys 0..r (rows == keys)."""
    rows, keys = q.shape[0], k.shape[0]
    group = Q_HEADS // KV_HEADS
    out = torch.empty(rows, Q_HEADS, HD)
    mask = torch.ones(rows, keys, dtype=torch.bool).tril() if causal else None
    for h in range(Q_HEADS):
        kv = h // group
        logits = (q[:, h] @ k[:, kv].t()) * (HD ** -0.5)
        if mask is not None:
            logits = logits.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(logits, dim=-1) @ v[:, kv]
    return rnd(out.reshape(rows, Q_HEADS * HD))


def llm_layer(w, pre, i, x, table, rnd, k_prefix=None, v_prefix=None):
    """One layer of the prefix (`pre` = "llm", dm0_infer.py:874-951, causal over its own rows) or of the action expert
    (`pre` = "decoder", :782-851, its K / V appended behind the prefix cache rows and no mask).  Returns (x, k, v) with
    k, v this layer's new cache rows [rows, 8, 128]."""
    factor = ops.rms_factor(x)
    qkv = rnd(gemm(x, w[pre + "_attn_qkv_w"][i]))                      # the GEMM sees the un-normalised rows
    q, k, v = qknorm_rope_split(qkv, factor, w[pre + "_q_norm_w"][i], w[pre + "_k_norm_w"][i], table, rnd)
    if k_prefix is None:
        a = gqa_attention(q, k, v, rnd, causal=True)
    else:
        a = gqa_attention(q, torch.cat([k_prefix, k]), torch.cat([v_prefix, v]), rnd, causal=False)
    x = rnd(x + gemm(a, w[pre + "_attn_o_w"][i]))
    factor = ops.rms_factor(x)
    g = gemm(x, w[pre + "_ffn_gate_w"][i]) * factor
    u = gemm(x, w[pre + "_ffn_up_w"][i]) * factor
    h = rnd(silu(g) * u)
    return rnd(x + gemm(h, w[pre + "_ffn_down_w"][i])), k, v


def prefix_forward(w, x, rnd, taps=None):
    """dm0_infer.py:953-955 -> per-layer K and V of the prefix rows."""
    table = rope_table(0, x.shape[0])
    ks, vs = [], []
    for i in range(w["llm_attn_qkv_w"].shape[0]):
        x, k, v = llm_layer(w, "llm", i, x, table, rnd)
        ks.append(k); vs.append(v)
        if taps is not None:
            taps["prefix_x/%d" % i] = x.clone()
            taps["prefix_K/%d" % i] = k.clone()
            taps["prefix_V/%d" % i] = v.clone()
    return ks, vs


def decoder_forward(w, ks, vs, noise, rnd, taps=None, num_steps=10):
    """dm0_infer.py:853-872: 10 Euler steps; every step embeds the noise (:763-780), runs the action expert and updates
    the noise with the fused output projection (:99-120)."""
    prefix_len = ks[0].shape[0]
    chunk = noise.shape[0]
    table = rope_table(prefix_len, chunk)
    noise = f32(noise)
    for t in range(num_steps):
        u = rnd(silu(f32(w["decoder_action_fused_time_biases"][t % 10]) + gemm(noise, w["decoder_action_fused_in_proj_w"])))
        x = rnd(f32(w["decoder_action_mlp_b"]) + gemm(u, w["decoder_action_mlp_w"]))
        if taps is not None:
            taps["decoder_in/%d" % t] = x.clone()
        for i in range(w["decoder_attn_qkv_w"].shape[0]):
            x, _, _ = llm_layer(w, "decoder", i, x, table, rnd, ks[i], vs[i])
            if taps is not None:
                taps["decoder_x/%d/%d" % (t, i)] = x.clone()
        factor = ops.rms_factor(x)
        noise = rnd(noise + f32(w["decoder_action_fused_out_proj_b"]) + gemm(x * factor, w["decoder_action_fused_out_proj_w"]))
        if taps is not None:
            taps["noise/%d" % t] = noise.clone()
    return noise


def forward(w, images, input_ids, noise, bf16_boundaries=True, taps=None):
    """DM0Inference.forward (dm0_infer.py:1111-1116) -> actions [50, 32] (fp32 container)."""
    rnd = ops.round_bf16 if bf16_boundaries else ops.identity
    with torch.no_grad():
        x = vision_forward(w, images, input_ids, rnd, taps)
        if taps is not None:
            taps["prefix_x0"] = x.clone()
        ks, vs = prefix_forward(w, x, rnd, taps)
        return decoder_forward(w, ks, vs, noise, rnd, taps)
