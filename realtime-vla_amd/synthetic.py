"""Seeded synthetic checkpoints and observations in the converted-checkpoint layout.

Everything here is integer-exact up to one IEEE multiply and one round-to-bf16, so the
same (seed, tensor name) gives bit-identical tensors on any CPU and on the GPU; the
generator runs on whatever torch device it is handed.  Used by the tests and by the
benchmark harness to stand in for a converted Pi0/Pi05 checkpoint (layout:
/root/reference/convert_from_jax.py:279-326, key list pi0_infer.py:1245-1287 and
pi05_infer.py:563-611).

Normal variates are an 8-term Irwin-Hall sum of 16-bit uniform fields of two
splitmix64 outputs (variance-matched to N(0,1), support +-4.9 sigma); uniforms use the
top 24 bits of one output.
"""
import math

import torch

_M64 = (1 << 64) - 1
_GOLD = 0x9E3779B97F4A7C15


def _to_i64(u):
    u &= _M64
    return u - (1 << 64) if u >= (1 << 63) else u


def _splitmix64_int(x):
    x = (x + _GOLD) & _M64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def _fnv1a64(name):
    h = 0xCBF29CE484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & _M64
    return h


def stream_key(seed, name):
    """64-bit key of the stream for (seed, tensor name)."""
    return _splitmix64_int((seed & _M64) ^ _fnv1a64(name))


def _lsr(x, s):
    # logical shift right on int64 tensors (torch's >> is arithmetic)
    return (x >> s) & ((1 << (64 - s)) - 1)


def _splitmix64(x):
    # x: int64 tensor; arithmetic wraps modulo 2^64
    z = x + _to_i64(_GOLD)
    z = (z ^ _lsr(z, 30)) * _to_i64(0xBF58476D1CE4E5B9)
    z = (z ^ _lsr(z, 27)) * _to_i64(0x94D049BB133111EB)
    return z ^ _lsr(z, 31)


_IH_SCALE = 1.0 / math.sqrt(8.0 * (65536.0 ** 2 - 1.0) / 12.0)
_CHUNK_CPU = 1 << 18
_CHUNK_GPU = 1 << 26


def _chunk(device):
    return _CHUNK_CPU if torch.device(device).type == "cpu" else _CHUNK_GPU


def _normal_chunk(key, start, n, scale, device):
    idx = torch.arange(start, start + n, dtype=torch.int64, device=device)
    s = None
    for half in range(2):
        h = _splitmix64(idx * 2 + (half + _to_i64(key)))
        # sum of the four 16-bit fields of h, two fields per 32-bit half at a time
        t = (h & 0x0000FFFF0000FFFF) + ((h >> 16) & 0x0000FFFF0000FFFF)
        t = (t & 0xFFFFFFFF) + ((t >> 32) & 0xFFFFFFFF)
        s = t if s is None else s + t
    c = torch.tensor(scale * _IH_SCALE, dtype=torch.float32, device=device)
    return (s - 4 * 65535).to(torch.float32) * c


def normal_bf16(seed, name, shape, std=1.0, device="cpu"):
    """bf16 tensor of approximately N(0, std^2) variates for stream (seed, name)."""
    n = int(math.prod(shape))
    key = stream_key(seed, name)
    out = torch.empty(n, dtype=torch.bfloat16, device=device)
    for start in range(0, n, _chunk(device)):
        m = min(_chunk(device), n - start)
        out[start:start + m] = _normal_chunk(key, start, m, std, device).to(torch.bfloat16)
    return out.view(*shape)


def uniform_pm1_bf16(seed, name, shape, device="cpu"):
    """bf16 tensor uniform in [-1, 1)."""
    n = int(math.prod(shape))
    key = stream_key(seed, name)
    out = torch.empty(n, dtype=torch.bfloat16, device=device)
    for start in range(0, n, _chunk(device)):
        m = min(_chunk(device), n - start)
        idx = torch.arange(start, start + m, dtype=torch.int64, device=device)
        u = _lsr(_splitmix64(idx + _to_i64(key)), 40).to(torch.float32)
        out[start:start + m] = ((u + 0.5) * (1.0 / 8388608.0) - 1.0).to(torch.bfloat16)
    return out.view(*shape)


def randint(seed, name, n, high, device="cpu"):
    """int64 tensor of n ids uniform in [0, high)."""
    key = stream_key(seed, name)
    idx = torch.arange(n, dtype=torch.int64, device=device)
    return _lsr(_splitmix64(idx + _to_i64(key)), 33) % high


def embedding_rows(seed, ids, device="cpu", std=0.02):
    """Rows `ids` of the virtual embedding table `embedding_weight` [257152, 2048]
    (N(0, std^2) bf16), without materialising the table."""
    key = stream_key(seed, "embedding_weight")
    rows = []
    for t in ids.tolist():
        rows.append(_normal_chunk(key, int(t) * 2048, 2048, std, device).to(torch.bfloat16))
    if not rows:
        return torch.empty(0, 2048, dtype=torch.bfloat16, device=device)
    return torch.stack(rows)


VOCAB = 257152
STATE_TOKEN_OFFSET = 256000   # documented constant: discrete state bin b -> vocabulary id 256000 + b


def language_embeds(seed, prompt_len, device="cpu", state_tokens=0):
    """Pre-scaled prompt embeddings [L, 2048]: `prompt_len` ids uniform in [0, VOCAB)
    followed by `state_tokens` ids uniform in [0,256) + STATE_TOKEN_OFFSET, each row
    embedding_weight[id] * sqrt(2048), rounded to bf16
    (/root/reference/convert_from_jax.py:241-263, pi05_infer.py:784)."""
    ids = randint(seed, "prompt_ids", prompt_len, VOCAB)
    if state_tokens:
        ids = torch.cat([ids, randint(seed, "state_ids", state_tokens, 256) + STATE_TOKEN_OFFSET])
    e = embedding_rows(seed, ids, device)
    return (e.float() * math.sqrt(2048.0)).to(torch.bfloat16)


def _sincos_time(t, dim=1024, min_period=4e-3, max_period=4.0):
    # closed-form flow-time embedding (/root/reference/convert_from_jax.py:133-140)
    frac = torch.linspace(0.0, 1.0, dim // 2, dtype=torch.float64)
    period = min_period * (max_period / min_period) ** frac
    ang = (2.0 * math.pi / period) * t
    return torch.cat([torch.sin(ang), torch.cos(ang)]).to(torch.float32)


def pi0_checkpoint(seed, prompt_len, device="cpu", vision_layers=27, llm_layers=18, std=0.02, norms="ones"):
    """Synthetic converted Pi0 checkpoint (keys/shapes of /root/reference/pi0_infer.py:1245-1287).
    Matrices N(0, std^2); LayerNorm parameters per `norms` (see _norm_params)."""
    V, L = vision_layers, llm_layers
    shapes = {
        "vision_patch_embedding_w": (14, 14, 3, 1152),
        "vision_patch_embedding_b": (1152,),
        "vision_position_embedding": (256, 1152),
        "vision_attn_qkv_w": (V, 1152, 3456),
        "vision_attn_qkv_b": (V, 3456),
        "vision_attn_o_w": (V, 1152, 1152),
        "vision_attn_o_b": (V, 1152),
        "vision_ffn_up_w": (V, 1152, 4304),
        "vision_ffn_up_b": (V, 4304),
        "vision_ffn_down_w": (V, 4304, 1152),
        "vision_ffn_down_b": (V, 1152),
        "encoder_multi_modal_projector_w": (1152, 2048),
        "encoder_multi_modal_projector_b": (2048,),
        "encoder_attn_qkv_w": (L, 2048, 2560),
        "encoder_attn_o_w": (L, 2048, 2048),
        "encoder_ffn_gate_w": (L, 2048, 16384),
        "encoder_ffn_up_w": (L, 2048, 16384),
        "encoder_ffn_down_w": (L, 16384, 2048),
        "decoder_state_in_proj_w": (32, 1024),
        "decoder_state_in_proj_b": (1024,),
        "decoder_action_fused_in_proj_w": (32, 1024),
        "decoder_action_fused_time_biases": (10, 1024),
        "decoder_action_mlp_w": (1024, 1024),
        "decoder_action_mlp_b": (1024,),
        "decoder_attn_qkv_w": (L, 1024, 2560),
        "decoder_attn_o_w": (L, 2048, 1024),
        "decoder_ffn_gate_w": (L, 1024, 4096),
        "decoder_ffn_up_w": (L, 1024, 4096),
        "decoder_ffn_down_w": (L, 4096, 1024),
        "decoder_action_fused_out_proj_w": (1024, 32),
        "decoder_action_fused_out_proj_b": (32,),
    }
    ck = {k: normal_bf16(seed, k, s, std, device) for k, s in shapes.items()}
    # the converter folds the Euler step dt = -0.1 into the fused output projection
    # (/root/reference/convert_from_jax.py:192-194); the synthetic checkpoint does the same
    for k in ("decoder_action_fused_out_proj_w", "decoder_action_fused_out_proj_b"):
        ck[k] = (ck[k].float() * -0.1).to(torch.bfloat16)
    _norm_params(ck, V, device, seed, norms)
    ck["language_embeds"] = language_embeds(seed, prompt_len, device)
    return ck


def _norm_params(ck, V, device, seed=0, norms="ones"):
    """SigLIP LayerNorm parameters.  "ones": weight 1, bias 0 (the benchmark configurations).  "random": every
    layer's weights 1 + N(0, 0.1^2) and biases N(0, 0.1^2), all distinct, so that the affine term and the choice
    of the layer's parameters show in the result."""
    shapes = {"vision_pre_attn_norm": (V, 1152), "vision_pre_ffn_norm": (V, 1152), "vision_final_norm": (1152,)}
    for name, shape in shapes.items():
        if norms == "ones":
            ck[name + "_w"] = torch.ones(*shape, dtype=torch.bfloat16, device=device)
            ck[name + "_b"] = torch.zeros(*shape, dtype=torch.bfloat16, device=device)
        elif norms == "random":
            ck[name + "_w"] = (1.0 + normal_bf16(seed, name + "_w", shape, 0.1, device).float()).to(torch.bfloat16)
            ck[name + "_b"] = normal_bf16(seed, name + "_b", shape, 0.1, device)
        else:
            raise ValueError("norms must be 'ones' or 'random'")


def pi05_checkpoint(seed, prompt_len, device="cpu", vision_layers=27, llm_layers=18, std=0.02,
                    state_tokens=32, norms="ones"):
    """Synthetic converted Pi05 checkpoint (keys/shapes of /root/reference/pi05_infer.py:563-611);
    `decoder_time_embeds` is the closed-form sin/cos embedding of t = 1.0, 0.9, ... 0.1
    (/root/reference/convert_from_jax_pi05.py:214-228)."""
    V, L = vision_layers, llm_layers
    shapes = {
        "vision_patch_embedding_w": (14, 14, 3, 1152),
        "vision_patch_embedding_b": (1152,),
        "vision_position_embedding": (256, 1152),
        "vision_attn_qkv_w": (V, 1152, 3456),
        "vision_attn_qkv_b": (V, 3456),
        "vision_attn_o_w": (V, 1152, 1152),
        "vision_attn_o_b": (V, 1152),
        "vision_ffn_up_w": (V, 1152, 4304),
        "vision_ffn_up_b": (V, 4304),
        "vision_ffn_down_w": (V, 4304, 1152),
        "vision_ffn_down_b": (V, 1152),
        "encoder_multi_modal_projector_w": (1152, 2048),
        "encoder_multi_modal_projector_b": (2048,),
        "encoder_attn_qkv_w": (L, 2048, 2560),
        "encoder_attn_o_w": (L, 2048, 2048),
        "encoder_ffn_gate_w": (L, 2048, 16384),
        "encoder_ffn_up_w": (L, 2048, 16384),
        "encoder_ffn_down_w": (L, 16384, 2048),
        "decoder_time_mlp_in_w": (1024, 1024),
        "decoder_time_mlp_in_b": (1024,),
        "decoder_time_mlp_out_w": (1024, 1024),
        "decoder_time_mlp_out_b": (1024,),
        "decoder_action_in_proj_w": (32, 1024),
        "decoder_action_in_proj_b": (1024,),
        "decoder_pre_attn_norm_mod_w": (L, 1024, 3072),
        "decoder_pre_attn_norm_mod_b": (L, 3072),
        "decoder_pre_ffn_norm_mod_w": (L, 1024, 3072),
        "decoder_pre_ffn_norm_mod_b": (L, 3072),
        "decoder_attn_qkv_w": (L, 1024, 2560),
        "decoder_attn_o_w": (L, 2048, 1024),
        "decoder_ffn_gate_w": (L, 1024, 4096),
        "decoder_ffn_up_w": (L, 1024, 4096),
        "decoder_ffn_down_w": (L, 4096, 1024),
        "decoder_action_out_proj_w": (1024, 32),
        "decoder_action_out_proj_b": (32,),
        "decoder_final_norm_mod_w": (1024, 3072),
        "decoder_final_norm_mod_b": (3072,),
    }
    ck = {k: normal_bf16(seed, k, s, std, device) for k, s in shapes.items()}
    _norm_params(ck, V, device, seed, norms)
    te = torch.stack([_sincos_time(1.0 - 0.1 * s) for s in range(10)])
    ck["decoder_time_embeds"] = te.to(torch.bfloat16).to(device)
    ck["language_embeds"] = language_embeds(seed, prompt_len, device, state_tokens=state_tokens)
    return ck


DM0_VOCAB = 152701


def dm0_checkpoint(seed, device="cpu", vision_layers=23, llm_layers=28, std=0.02, vocab=DM0_VOCAB):
    """Synthetic DM0 checkpoint (keys/shapes of /root/reference/dm0_infer.py:991-1035).  Matrices N(0, std^2); the folded
    LayerNorm column sums are the column sums of the folded weights, as the converter computes them; norm weights
    1 + N(0, 0.1^2); `vocab` rows of token embeddings (the reference table has 152701)."""
    V, L = vision_layers, llm_layers
    shapes = {
        "decoder_attn_qkv_w": (L, 1024, 4096), "decoder_attn_o_w": (L, 2048, 1024),
        "decoder_ffn_gate_w": (L, 1024, 1536), "decoder_ffn_up_w": (L, 1024, 1536), "decoder_ffn_down_w": (L, 1536, 1024),
        "decoder_action_fused_in_proj_w": (32, 1024), "decoder_action_fused_time_biases": (10, 1024),
        "decoder_action_mlp_w": (1024, 1024), "decoder_action_mlp_b": (1024,),
        "decoder_action_fused_out_proj_w": (1024, 32), "decoder_action_fused_out_proj_b": (32,),
        "llm_attn_qkv_w": (L, 2048, 4096), "llm_attn_o_w": (L, 2048, 2048),
        "llm_ffn_gate_w": (L, 2048, 6144), "llm_ffn_up_w": (L, 2048, 6144), "llm_ffn_down_w": (L, 6144, 2048),
        "vision_conv1_w_t": (588, 1024), "vision_class_embedding": (1024,), "vision_pos_emb": (2705, 1024),
        "vision_fused_qkv_w": (V, 1024, 3072), "vision_out_proj_w": (V, 1024, 1024), "vision_out_proj_b": (V, 1024),
        "vision_fused_fc_w": (V, 1024, 4096), "vision_proj_w": (V, 4096, 1024), "vision_proj_b": (V, 1024),
        "vision_ds1_w": (3, 3, 1024, 2048), "vision_ds1_b": (2048,), "vision_ds2_w": (3, 3, 2048, 4096), "vision_ds2_b": (4096,),
        "vision_projector_w_t": (4096, 2048), "vision_embed_tokens_w": (vocab, 2048),
    }
    ck = {k: normal_bf16(seed, k, s, std, device) for k, s in shapes.items()}
    for k in ("decoder_action_fused_out_proj_w", "decoder_action_fused_out_proj_b"):      # dt = -0.1 folded in, as for Pi0
        ck[k] = (ck[k].float() * -0.1).to(torch.bfloat16)
    for k, shape in (("decoder_q_norm_w", (L, 128)), ("decoder_k_norm_w", (L, 128)), ("llm_q_norm_w", (L, 128)), ("llm_k_norm_w", (L, 128)),
                     ("vision_ln_pre_w", (1024,))):
        ck[k] = (1.0 + normal_bf16(seed, k, shape, 0.1, device).float()).to(torch.bfloat16)
    ck["vision_ln_pre_b"] = normal_bf16(seed, "vision_ln_pre_b", (1024,), 0.1, device)
    for name, n in (("qkv", 3072), ("fc", 4096)):                                           # fp32 tensors of the folded LayerNorm
        ck["vision_fused_%s_b" % name] = normal_bf16(seed, "vision_fused_%s_b" % name, (V, n), 0.05, device).float()
        ck["vision_%s_col_sum" % name] = ck["vision_fused_%s_w" % name].float().sum(dim=1)
    return ck


def dm0_observation(seed, num_images, device="cpu", max_lang_len=100, vocab=DM0_VOCAB, draw=0):
    """Seeded DM0 inputs: images [n,3,728,728] uniform[-1,1) bf16, `max_lang_len` token ids, noise [50,32] ~N(0,1) bf16."""
    images = uniform_pm1_bf16(seed, "images", (num_images, 3, 728, 728), device)
    ids = randint(seed, "input_ids", max_lang_len, vocab, device)
    noise = normal_bf16(seed, "diffusion_noise/%d" % draw, (50, 32), 1.0, device)
    return images, ids, noise


def observation(seed, num_views, chunk_size, device="cpu", draw=0):
    """Seeded inputs: images [v,224,224,3] uniform[-1,1), state [32] and noise [chunk,32] ~N(0,1), bf16.
    `draw` selects an independent noise stream (fresh noise per iteration)."""
    images = uniform_pm1_bf16(seed, "observation_images_normalized", (num_views, 224, 224, 3), device)
    state = normal_bf16(seed, "observation_state_normalized", (32,), 1.0, device)
    noise = normal_bf16(seed, "diffusion_noise/%d" % draw, (chunk_size, 32), 1.0, device)
    return images, state, noise
