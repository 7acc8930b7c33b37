"""Pi0Inference for MI355X: same constructor, forward() and checkpoint layout as
/root/reference/pi0_infer.py:1238-1361, backed by hand-written HIP kernels (librtvla.so)."""
import torch

import rtvla_capi as capi
from _engine import Engine, rope_table


class Pi0Inference:
    def __init__(self, checkpoint, num_views, chunk_size, tile_cache=None):
        """`tile_cache` (not in the reference): a directory in which the re-tiled weights are kept across processes."""
        self.num_views = num_views
        self.chunk_size = chunk_size
        encoded_prompt = checkpoint['language_embeds']          # KeyError if absent, as in the reference
        self.prompt_len = len(encoded_prompt)
        self._engine = Engine(capi.PI0, checkpoint, num_views, self.prompt_len, chunk_size, tile_cache=tile_cache)
        self.weights = self._engine.weights
        self.buffers = self._engine.buffers

        encoder_seq_len = num_views * 256 + self.prompt_len
        decoder_seq_len = chunk_size + 1
        dev = self._engine.device
        self.buffers['encoder_rope_weights'].copy_(rope_table(0, encoder_seq_len, dev))
        self.buffers['decoder_rope_weights'].copy_(rope_table(encoder_seq_len, decoder_seq_len, dev))

        self._engine.prepare()
        self.infer_graph = None
        self.record_infer_graph()

    def record_run(self):
        """One eager (uncaptured) forward over the bound buffers."""
        self._engine.run_eager()

    def record_infer_graph(self):
        self._engine.capture()
        self.infer_graph = self._engine.ctx

    def forward(self, observation_images_normalized, observation_state_normalized, diffusion_noise):
        self.buffers['observation_images_normalized'].copy_(observation_images_normalized)
        self.buffers['observation_state_normalized'].copy_(observation_state_normalized)
        self.buffers['diffusion_noise'].copy_(diffusion_noise)
        self._engine.replay()
        return self.buffers['diffusion_noise']
