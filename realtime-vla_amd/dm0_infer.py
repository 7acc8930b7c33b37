"""DM0Inference for MI355X: same constructor, forward() and checkpoint layout as
/root/reference/dm0_infer.py:965-1116, backed by hand-written HIP kernels (librtvla.so)."""
import torch

import rtvla_capi as capi
from _engine import Engine


class DB0Config:
    image_size: int = 728
    patch_size: int = 14
    llm_vocab_size: int = 152701
    llm_rope_theta: float = 1000000.0
    chunk_size: int = 50
    diffusion_steps: int = 10


def vision_rope_pairs(device, grid_h=52, grid_w=52, head_dim=64, theta=10000.0):
    """The 2-D rotary table of /root/reference/dm0_infer.py:671-688 (class token first, angles and their cos / sin rounded
    to bf16 as there) as rows [cos_0, sin_0, cos_1, sin_1, ...] of the 32 rotation pairs: the reference's 64 angles repeat
    every frequency twice, once per element of a pair."""
    dim_per_axis = head_dim // 2
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim_per_axis, 2, device=device)[: (dim_per_axis // 2)].float() / dim_per_axis))
    gh = torch.arange(grid_h, dtype=torch.float, device=device) + 1
    gw = torch.arange(grid_w, dtype=torch.float, device=device) + 1
    fh = (gh[:, None] * inv_freq[None, :])[:, None, :].expand(grid_h, grid_w, -1)
    fw = (gw[:, None] * inv_freq[None, :])[None, :, :].expand(grid_h, grid_w, -1)
    freqs = torch.cat([fw, fh], dim=-1).reshape(grid_h * grid_w, -1)                       # one angle per pair: 16 from the column, 16 from the row
    freqs = torch.cat([torch.zeros(1, freqs.shape[-1], device=device), freqs], dim=0).to(torch.bfloat16)
    return torch.stack([freqs.cos(), freqs.sin()], dim=2).reshape(grid_h * grid_w + 1, head_dim)


class DM0Inference:
    def __init__(self, checkpoint, num_images=3, max_lang_len=100, device="cuda", tile_cache=None):
        config = DB0Config()
        self.device = device
        self.num_images = num_images
        self.max_lang_len = max_lang_len
        self.chunk_size = config.chunk_size
        self.diffusion_steps = config.diffusion_steps
        grid_size = config.image_size // config.patch_size
        tokens_per_image = (grid_size // 4) ** 2
        self.prefix_len = num_images * tokens_per_image + max_lang_len
        self.total_keys = self.prefix_len + self.chunk_size
        vision_layers = int(checkpoint["vision_fused_qkv_w"].shape[0]) if "vision_fused_qkv_w" in checkpoint else 23
        llm_layers = int(checkpoint["llm_attn_qkv_w"].shape[0]) if "llm_attn_qkv_w" in checkpoint else 28
        self._engine = Engine(capi.DM0, checkpoint, num_images, max_lang_len, self.chunk_size, num_steps=self.diffusion_steps,
                              tile_cache=tile_cache, vision_layers=vision_layers, llm_layers=llm_layers)
        self.weights = self._engine.weights
        self.buffers = self._engine.buffers
        self._compute_rope_weights(config.llm_rope_theta)
        self.buffers['vision_rope'].copy_(vision_rope_pairs(self._engine.device))
        self._engine.prepare()
        self.graph = None
        self._record_graph()

    def _compute_rope_weights(self, theta):
        dev = self._engine.device
        inv_freq = 1.0 / (theta ** (torch.arange(0, 128, 2, dtype=torch.float32, device=dev) / 128))
        for name, start, count in (('prefix_rope_weights', 0, self.prefix_len), ('decoder_rope_weights', self.prefix_len, self.chunk_size)):
            positions = torch.arange(start, start + count, dtype=torch.float32, device=dev)
            angles = positions[:, None] * inv_freq[None, :]
            rope = torch.stack([torch.cos(angles).to(torch.bfloat16), torch.sin(angles).to(torch.bfloat16)], dim=2).reshape(count, 128)
            self.buffers[name].copy_(rope)

    def _record_run(self):
        """One eager (uncaptured) forward over the bound buffers."""
        self._engine.run_eager()

    def _record_graph(self):
        self._engine.capture()
        self.graph = self._engine.ctx

    def forward(self, images, input_ids, noise):
        self.buffers['images'].copy_(images)
        self.buffers['input_ids'].copy_(input_ids)
        self.buffers['diffusion_noise'].copy_(noise)
        self._engine.replay()
        return self.buffers['diffusion_noise']
