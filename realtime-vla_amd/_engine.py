"""Shared host logic of Pi0Inference / Pi05Inference: tensor ownership (PyTorch-ROCm), binding
to the C ABI, RoPE tables, graph capture.  PyTorch is used only to own device memory and for
the input staging copies; every kernel of the forward lives in librtvla.so."""
import os

import torch

import rtvla_capi as capi
from tile_cache import TileCache, UNTILED_WEIGHTS, fingerprint

_DTYPES = {2: torch.bfloat16, 4: torch.int32}
_ANY_ROWS = ("vision_embed_tokens_w",)          # tables whose row count is whatever the checkpoint holds


def rope_table(start, count, device):
    """Rows [cos_0, sin_0, cos_1, sin_1, ...] in bf16 for positions start..start+count-1
    (/root/reference/pi0_infer.py:1319-1335)."""
    position_ids = torch.arange(start, start + count, device=device)
    inv_freq = 1.0 / (10000 ** (torch.arange(0, 256, 2, dtype=torch.float32, device=device) / 256))
    phase = inv_freq[None, :] * position_ids[:, None]
    cos = torch.cos(phase).to(torch.bfloat16)
    sin = torch.sin(phase).to(torch.bfloat16)
    return torch.cat([cos[:, :, None], sin[:, :, None]], 2).view(-1, 256)


class Engine:
    def __init__(self, model, checkpoint, num_views, prompt_len, chunk_size, num_steps=10, skip_keys=(), tile_cache=None,
                 vision_layers=None, llm_layers=None):
        if not torch.cuda.is_available():
            raise RuntimeError("realtime-vla_amd needs a ROCm GPU (MI355X / gfx950); there is no CPU path")
        self.device = torch.device("cuda", torch.cuda.current_device())
        if vision_layers is None:
            vision_layers = int(checkpoint["vision_attn_qkv_w"].shape[0]) if "vision_attn_qkv_w" in checkpoint else 27
        if llm_layers is None:
            llm_layers = int(checkpoint["encoder_attn_qkv_w"].shape[0]) if "encoder_attn_qkv_w" in checkpoint else 18
        self.model, self.vision_layers, self.llm_layers, self.num_steps = model, vision_layers, llm_layers, num_steps
        self.prefix_rows = num_views * 256 + prompt_len                       # rows of the prefix pass (as allocated)
        self.suffix_rows = chunk_size + (1 if model == capi.PI0 else 0)       # Pi0: the state token precedes the action rows
        self.tile_cache = TileCache(tile_cache) if isinstance(tile_cache, (str, os.PathLike)) else tile_cache
        self.tile_cache_hit = None                                   # True / False after prepare() when a cache is in use
        self.ctx = capi.Context(model, num_views, prompt_len, chunk_size, num_steps, vision_layers, llm_layers)
        self.weights, self.buffers = {}, {}
        for name, elem, shape, is_weight, required in self.ctx.tensors():
            dtype = torch.float32 if (is_weight and elem == 4) else _DTYPES[elem]      # 4-byte weights are fp32, 4-byte io buffers int32
            if is_weight and (not required or name in _ANY_ROWS):
                # optional weights (Pi05 embedding table, ~1 GB) exist only when the checkpoint brings them; the token
                # embedding tables take their row count from the checkpoint
                if name in checkpoint and name not in skip_keys:
                    v = torch.as_tensor(checkpoint[name])
                    self.weights[name] = torch.zeros(*v.shape, dtype=dtype, device=self.device)
                elif required:
                    self.weights[name] = torch.zeros(1, shape[1], dtype=dtype, device=self.device)
                continue
            # zero-initialised so that a weight the checkpoint omits (the reference leaves it
            # uninitialised, benchmark.py:9-11) can never inject NaN/Inf
            t = torch.zeros(*shape, dtype=dtype, device=self.device)
            (self.weights if is_weight else self.buffers)[name] = t
        for k, v in checkpoint.items():
            if k in skip_keys:
                continue
            if not torch.is_tensor(v):
                v = torch.as_tensor(v)
            self.weights[k].copy_(v)               # KeyError on an unknown key, RuntimeError on a shape mismatch
        for name, t in list(self.weights.items()) + list(self.buffers.items()):
            self.ctx.bind(name, t.data_ptr(), t.numel() * t.element_size())
        nbytes = self.ctx.workspace_bytes()
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self.ctx.bind_workspace(self.workspace.data_ptr(), nbytes)
        # views of the library's internal activations, under the reference's buffer names where one exists
        for name, off, rows, cols, ld, elem in self.ctx.buffers():
            if name.startswith("t_"):
                continue
            flat = self.workspace[off:off + rows * ld * elem].view(torch.bfloat16 if elem == 2 else torch.float32)
            self.buffers.setdefault(name, flat.view(rows, ld)[:, :cols])
        self.stream = torch.cuda.current_stream(self.device)

    def prepare(self):
        """rtvla_prepare; with a tile cache the re-tiled weights come from its file when one matches this checkpoint
        (fingerprint of the weights as they sit on the device), and are saved there after the first re-tiling."""
        if self.tile_cache is None:
            self.ctx.prepare(self.stream.cuda_stream)
            torch.cuda.synchronize(self.device)
            return
        lib = capi.load()
        ident = (lib.rtvla_tile_layout_version(), self.model, self.num_steps, self.vision_layers, self.llm_layers)
        # every weight the tiled region can depend on: for Pi05 it holds W diag(1 + scale) per (flow step, layer), and scale
        # comes from the time embeddings, the time MLP and the norm-modulation weights and biases, not only from the matrices
        # that are re-tiled
        key = fingerprint({k: v for k, v in self.weights.items() if k not in UNTILED_WEIGHTS})
        region = self.workspace[: self.ctx.tiled_bytes()]
        self.tile_cache_hit = self.tile_cache.load_into(key, *ident, region)
        self.ctx.prepare(self.stream.cuda_stream, tiles_loaded=self.tile_cache_hit)
        torch.cuda.synchronize(self.device)
        if not self.tile_cache_hit:
            self.tile_cache.store(key, *ident, region)

    def capture(self):
        """One eager forward, then capture into a HIP graph on a side stream
        (/root/reference/pi0_infer.py:1347-1354)."""
        side = torch.cuda.Stream(self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        self.ctx.graph_capture(side.cuda_stream)
        side.synchronize()
        self.graph_launches = self.ctx.launch_count()      # kernel nodes in the captured graph

    def reference_buffer(self, name):
        """Row-major copy of an internal activation in the shape the reference keeps it in
        (/root/reference/pi0_infer.py:1291-1317, pi05_infer.py:690-730): the MFMA kernels hold these tensors fragment-tiled,
        so `buffers[name]` has other bytes than the reference's tensor of that name.  Pi0 / Pi05 names: encoder_K, encoder_V
        ([layers][prefix + suffix rows][256]), encoder_Q ([prefix rows * 8][256]), vision_QKV ([views][256][3 * 1152]),
        decoder_x, decoder_x_buf, decoder_q_buf, decoder_hidden.  Row-major buffers are returned as they are."""
        B, L = self.buffers, self.llm_layers
        if self.model == capi.DM0:
            raise KeyError("reference_buffer covers the Pi0 / Pi05 buffers")
        if name == "encoder_K":
            kp = B["encoder_K"].numel() // (L * 256)
            return torch.stack([untile_ft(B["encoder_K"].reshape(L, -1)[i], kp, 256) for i in range(L)])[:, : self.prefix_rows + self.suffix_rows]
        if name == "encoder_V":
            kp = B["encoder_Vt"].numel() // (L * 256)
            return torch.stack([untile_vt(B["encoder_Vt"].reshape(L, -1)[i], 256, kp).t() for i in range(L)])[:, : self.prefix_rows + self.suffix_rows].contiguous()
        if name in ("encoder_Q", "decoder_q_buf", "decoder_x", "decoder_x_buf", "decoder_hidden"):
            t = B[name]
            rows = {"encoder_Q": 8 * self.prefix_rows, "decoder_q_buf": 8 * self.suffix_rows, "decoder_x": self.suffix_rows,
                    "decoder_x_buf": self.suffix_rows, "decoder_hidden": self.suffix_rows}[name]
            cols = t.shape[1]
            return untile_ft(t, t.numel() // cols, cols)[:rows]
        if name == "vision_QKV":
            v = B["vision_Q"].shape[0] // 16
            q = torch.stack([untile_ft(x, 256, 96)[:, :72] for x in B["vision_Q"]]).view(v, 16, 256, 72)
            k = torch.stack([untile_ft(x, 256, 96)[:, :72] for x in B["vision_K"]]).view(v, 16, 256, 72)
            vv = torch.stack([untile_vt(x, 80, 256)[:72].t() for x in B["vision_Vt"]]).view(v, 16, 256, 72)
            return torch.stack([q, k, vv], 1).permute(0, 3, 1, 2, 4).reshape(v, 256, 3 * 1152)
        return B[name]

    def replay(self):
        self.ctx.graph_launch(torch.cuda.current_stream(self.device).cuda_stream)

    def run_stage(self, stage, layer=0, step=0):
        self.ctx.forward_stage(stage, layer, step, torch.cuda.current_stream(self.device).cuda_stream)

    def run_eager(self):
        self.ctx.forward(torch.cuda.current_stream(self.device).cuda_stream)


# ---- layout helpers for the library's fragment-tiled activations (taps, tests) -------------------
def untile_ft(flat, rows, cols):
    """Row-major copy of a fragment-tiled [rows][cols] matrix (rows % 16 == 0, cols % 32 == 0):
    tile (row/16, col/32) holds 64 lanes x 8 elements, lane = row%16 + 16*((col%32)/8)."""
    t = flat.reshape(-1)[: rows * cols].view(rows // 16, cols // 32, 4, 16, 8)
    return t.permute(0, 3, 1, 2, 4).reshape(rows, cols)


def tile_ft(mat):
    """Inverse of untile_ft."""
    rows, cols = mat.shape
    t = mat.reshape(rows // 16, 16, cols // 32, 4, 8)
    return t.permute(0, 2, 3, 1, 4).reshape(-1)


def untile_vt(flat, d, keys_pad):
    """Row-major [d][keys_pad] copy of the transposed-V layout: tile (d/16, key/32), lane = d%16 + 16 g,
    register j holding key 32*tile + 4 g + (j & 3) + 16 (j >> 2)."""
    t = flat.reshape(-1)[: d * keys_pad].view(d // 16, keys_pad // 32, 4, 16, 2, 4)     # [dt][kt][g][r][hi][lo]
    return t.permute(0, 3, 1, 4, 2, 5).reshape(d, keys_pad)


def tile_vt(mat):
    """Inverse of untile_vt: row-major [d][keys_pad] -> flat transposed-V tile layout."""
    d, keys_pad = mat.shape
    t = mat.reshape(d // 16, 16, keys_pad // 32, 2, 4, 4)                                # [dt][r][kt][hi][g][lo]
    return t.permute(0, 2, 4, 1, 3, 5).reshape(-1)
