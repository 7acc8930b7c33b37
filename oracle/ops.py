"""Op-level restatements shared by the Pi0 and Pi05 oracles (test infrastructure).

Every function takes and returns fp32 tensors whose values are bf16-representable when
`rnd` is `round_bf16`; with `rnd = identity` the same code is the all-fp32 variant.
Citations are into /root/reference/.
"""
import math

import torch
import torch.nn.functional as F


def round_bf16(x):
    return x.to(torch.bfloat16).to(torch.float32)


def identity(x):
    return x


def f32(x):
    return x.to(torch.float32)


def gemm(x, w):
    """fp32-accumulated X[rows,K] @ W[K,N] (weights are 'in x out', pi0_infer.py:5-41)."""
    return x @ f32(w)


def gelu_tanh(a):
    """pi0_infer.py:285 / :689 - a * sigmoid(1.5957691216057308 * a * (1 + 0.044715 a^2))."""
    return a * torch.sigmoid(1.5957691216057308 * a * (1.0 + 0.044715 * a * a))


def silu(a):
    return a * torch.sigmoid(a)


def layer_norm(x, w, b, eps=1e-5):
    """pi0_infer.py:366-382: LayerNorm over the last dim (biased variance), affine.
    The reference evaluates this in bf16 arithmetic; here fp32 inside."""
    mean = x.mean(-1, keepdim=True)
    xc = x - mean
    var = (xc * xc).mean(-1, keepdim=True)
    return xc * (1.0 / torch.sqrt(var + eps)) * f32(w) + f32(b)


def rms_factor(x, eps=1e-6):
    """pi0_infer.py:648-663 / :939-951: rsqrt(mean(x^2) + eps) per row."""
    return torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)


def rope_table(start, count):
    """pi0_infer.py:1319-1335: rows [cos_0, sin_0, cos_1, sin_1, ...] (bf16-rounded) for
    positions start .. start+count-1, inverse frequencies 10000^(-2i/256), i = 0..127."""
    pos = torch.arange(start, start + count, dtype=torch.float32)
    inv_freq = 1.0 / (10000 ** (torch.arange(0, 256, 2, dtype=torch.float32) / 256))
    phase = inv_freq[None, :] * pos[:, None]
    cos = round_bf16(torch.cos(phase))
    sin = round_bf16(torch.sin(phase))
    return torch.stack([cos, sin], dim=2).reshape(count, 256)


def rope_interleaved(x, table):
    """pi0_infer.py:794-800: rotate adjacent pairs (x[2j], x[2j+1]) of every 256-wide head
    by the angle of table row = token.  x: [rows, heads*256], table: [rows, 256]."""
    rows = x.shape[0]
    xh = x.reshape(rows, -1, 128, 2)
    t = table.reshape(rows, 1, 128, 2)
    c, s = t[..., 0], t[..., 1]
    x0, x1 = xh[..., 0], xh[..., 1]
    return torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1).reshape(rows, -1)


def patches(images):
    """pi0_infer.py:348-350: NHWC [v,224,224,3] -> [v*256, 588], feature order (dy, dx, c)."""
    v = images.shape[0]
    return images.reshape(v, 16, 14, 16, 14, 3).permute(0, 1, 3, 2, 4, 5).reshape(v * 256, 588)


def vision_attention(qkv, rnd):
    """pi0_infer.py:588-596: per view, 16 heads x 72, softmax(q k^T / sqrt(72)) v."""
    v = qkv.shape[0] // 256
    t = qkv.reshape(v, 256, 3, 16, 72).permute(0, 2, 3, 1, 4)
    q, k, val = t[:, 0], t[:, 1], t[:, 2]
    p = torch.softmax((q @ k.transpose(-1, -2)) * (1.0 / math.sqrt(72.0)), dim=-1)
    o = p @ val
    return rnd(o.transpose(1, 2).reshape(v * 256, 1152))


def mqa_attention(q, k, v, rnd, mask=None):
    """pi0_infer.py:819-824 (prefix) and :1041-1120 (suffix): q [rows*8, 256] with
    row = token*8 + head, one shared K/V head [keys,256]; logits rounded to bf16 after the
    1/16 scale (pi0_infer.py:1063-1064), probabilities rounded to bf16 (:1091), P.V rounded.
    `mask` [rows*8, keys] bool, True = visible."""
    logits = rnd((q @ k.t()) * (1.0 / 16.0))
    if mask is not None:
        logits = logits.masked_fill(~mask, float("-inf"))
    p = rnd(torch.softmax(logits, dim=-1))
    return rnd(p @ v)


def pi0_suffix_mask(s_d, s_e):
    """pi0_infer.py:1085: softmax row r (= token*8 + head) sees key j iff r >= 8 or j <= s_e."""
    r = torch.arange(8 * s_d)[:, None]
    j = torch.arange(s_e + s_d)[None, :]
    return (r >= 8) | (j <= s_e)


def valid_len_mask(rows, keys, valid_len):
    """pi05_infer.py:303: key j visible iff j < valid_len."""
    return (torch.arange(keys)[None, :] < valid_len).expand(rows, keys)


def pi05_suffix_mask(s_d, s_e_alloc, valid_len):
    """pi05_infer.py:406-410: prefix keys visible iff j < valid_len; every suffix key visible."""
    j = torch.arange(s_e_alloc + s_d)[None, :]
    return ((j < valid_len) | (j >= s_e_alloc)).expand(8 * s_d, s_e_alloc + s_d)
