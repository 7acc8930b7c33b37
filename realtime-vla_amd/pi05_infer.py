"""Pi05Inference for MI355X: same constructor, forward() and checkpoint layout as
/root/reference/pi05_infer.py:530-826, backed by hand-written HIP kernels (librtvla.so)."""
import numpy as np
import torch
import torch.nn as nn

import rtvla_capi as capi
from _engine import Engine, rope_table


class Pi05Inference:
    def __init__(
        self,
        checkpoint,
        num_views,
        chunk_size,
        tokenizer_path: str | None = None,
        max_tokenize_len: int = 200,
        discrete_state_input: bool = True,
        max_prompt_text: str | None = None,
        state_dim_for_max_prompt: int | None = None,
        tile_cache=None,                 # not in the reference: directory that keeps the re-tiled weights across processes
    ):
        self.discrete_state_input = discrete_state_input
        self.tokenizer_path = tokenizer_path
        self.checkpoint = checkpoint
        self.num_views = num_views
        self.chunk_size = chunk_size
        self.max_tokenize_len = int(max_tokenize_len)
        self.tokenizer = None
        if discrete_state_input:
            from transformers import AutoTokenizer
            self.tokenizer = AutoTokenizer.from_pretrained(tokenizer_path)
            if max_prompt_text is not None and state_dim_for_max_prompt is not None:
                self.max_prompt_len = self.estimate_max_prompt_len(
                    tokenizer=self.tokenizer,
                    task_prompt=max_prompt_text,
                    state_dim=int(state_dim_for_max_prompt),
                    max_tokenize_len=self.max_tokenize_len,
                    state_token_value=255,
                )
            else:
                self.max_prompt_len = self.max_tokenize_len
            if "embedding_weight" not in checkpoint:
                raise KeyError("checkpoint must contain 'embedding_weight' when discrete_state_input=True")
        elif 'language_embeds' in checkpoint:
            self.max_prompt_len = len(checkpoint['language_embeds'])
        elif 'embedding_weight' in checkpoint:
            self.max_prompt_len = self.max_tokenize_len          # token-id callers (forward_ids), no tokenizer needed
        else:
            self.max_prompt_len = len(checkpoint['language_embeds'])     # KeyError, as in the reference
        print(f"max_prompt_len: {self.max_prompt_len}, max_tokenize_len: {self.max_tokenize_len}")

        # With an embedding table in the checkpoint the prompt is staged ON THE DEVICE, inside the graph: token ids
        # -> embedding rows x sqrt(2048) -> encoder_x, and the decoder's RoPE rows follow valid_encoder_len
        # (the reference does both on the host per call, pi05_infer.py:769-785, :811-822).
        self.device_prompt = "embedding_weight" in checkpoint and (discrete_state_input or 'language_embeds' not in checkpoint)
        self._engine = Engine(capi.PI05, checkpoint, num_views, self.max_prompt_len, chunk_size,
                              skip_keys=("language_embeds",) if self.device_prompt else ("embedding_weight", "language_embeds"),
                              tile_cache=tile_cache)
        self.weights = self._engine.weights
        self.buffers = self._engine.buffers
        dev = self._engine.device
        self.weights['language_embeds'] = torch.as_tensor(checkpoint['language_embeds']).to(device=dev, dtype=torch.bfloat16) \
            if 'language_embeds' in checkpoint else torch.zeros(0, 2048, dtype=torch.bfloat16, device=dev)

        prefix_alloc = self.num_views * 256 + self.max_prompt_len
        max_pos = (self.num_views * 256 + self.max_prompt_len - 1) + self.chunk_size
        self._rope_table = rope_table(0, max_pos + 1, dev)
        self.buffers['rope_table'].copy_(self._rope_table)
        self.buffers['encoder_rope_weights'].copy_(self._rope_table[:prefix_alloc])
        self.buffers['valid_encoder_len'].fill_(self.num_views * 256 + 1)
        self.buffers['decoder_rope_weights'].copy_(self.get_decoder_rope_weights(1))

        self.prompt_embedding = None
        self._prompt_embed_scale = None
        if self.device_prompt:
            # the reference's nn.Embedding, sharing the table the library gathers from
            self.prompt_embedding = nn.Embedding(*self.weights['embedding_weight'].shape, device=dev, dtype=torch.bfloat16,
                                                 _weight=self.weights['embedding_weight'])
            self.prompt_embedding.weight.requires_grad_(False)
            self._prompt_embed_scale = float(self.weights['embedding_weight'].shape[1] ** 0.5)
        self.encoder_seq_len = prefix_alloc

        self._engine.prepare()       # includes the time-conditioning precompute (pi05_infer.py:669-722)
        self.infer_graph = None
        self.record_infer_graph()

    def estimate_max_prompt_len(self, tokenizer, task_prompt: str, state_dim: int, max_tokenize_len: int = 200,
                                state_token_value: int = 255) -> int:
        task_prompt = task_prompt.strip().replace("_", " ")
        state_str = " ".join([str(int(state_token_value))] * int(state_dim))
        full_prompt = f"Task: {task_prompt}, State: {state_str};\nAction: "
        token_ids = tokenizer(full_prompt, return_tensors="pt", truncation=True, max_length=int(max_tokenize_len),
                              padding=False)["input_ids"][0]
        return int(token_ids.shape[0])

    def build_prompt_ids(self, task_prompt: str, state_tokens: np.ndarray) -> torch.Tensor:
        """Host tokenisation of the reference's prompt template (pi05_infer.py:769-781) -> int64 ids on the CPU."""
        task_prompt = task_prompt.strip().replace("_", " ")
        state_str = " ".join(map(str, state_tokens.tolist()))
        full_prompt = f"Task: {task_prompt}, State: {state_str};\nAction: "
        return self.tokenizer(full_prompt, return_tensors="pt", truncation=True, max_length=self.max_tokenize_len,
                              padding=False)["input_ids"][0]

    def build_prompt_embeds(self, task_prompt: str, state_tokens: np.ndarray):
        token_ids = self.build_prompt_ids(task_prompt, state_tokens).to(device=self._engine.device, non_blocking=True)
        embeds = self.prompt_embedding(token_ids) * self._prompt_embed_scale
        return embeds, int(embeds.shape[0])

    def get_decoder_rope_weights(self, prompt_len: int) -> torch.Tensor:
        start = self.num_views * 256 + prompt_len - 1
        end = start + self.chunk_size
        return self._rope_table[start:end]

    def record_run(self):
        self._engine.run_eager()

    def record_infer_graph(self):
        self._engine.capture()
        self.infer_graph = self._engine.ctx

    def stage_token_ids(self, token_ids):
        """Device-side prompt staging: only the ids and the valid length cross to the device; the embedding gather,
        the sqrt(2048) scaling and the decoder RoPE rows are computed by the graph."""
        if not self.device_prompt:
            raise KeyError("checkpoint must contain 'embedding_weight' for token-id input")
        ids = torch.as_tensor(token_ids).reshape(-1)
        n = int(ids.shape[0])
        if n > self.max_prompt_len:
            raise ValueError(f"{n} prompt tokens exceed max_prompt_len {self.max_prompt_len}")
        self.buffers['prompt_token_ids'][:n].copy_(ids)
        self.buffers['valid_encoder_len'].fill_(self.num_views * 256 + n)

    def forward_ids(self, observation_images_normalized, diffusion_noise, token_ids) -> torch.Tensor:
        """forward() for callers that tokenise themselves (no counterpart in the reference, whose tokenizer call is
        inside forward): token_ids is an integer sequence of at most max_prompt_len entries."""
        self.stage_token_ids(token_ids)
        self.buffers['observation_images_normalized'].copy_(observation_images_normalized)
        self.buffers['diffusion_noise'].copy_(diffusion_noise)
        self._engine.replay()
        return self.buffers['diffusion_noise']

    def stage_inputs(self, observation_images_normalized, diffusion_noise, task_prompt=None, state_tokens=None):
        """The host-side staging of forward() without the replay (pi05_infer.py:811-824)."""
        if self.discrete_state_input and self.device_prompt:
            self.stage_token_ids(self.build_prompt_ids(task_prompt, state_tokens))
            self.buffers['observation_images_normalized'].copy_(observation_images_normalized)
            self.buffers['diffusion_noise'].copy_(diffusion_noise)
            return
        if self.discrete_state_input:
            prompt_embeds, prompt_len = self.build_prompt_embeds(task_prompt=task_prompt, state_tokens=state_tokens)
        else:
            prompt_embeds = self.weights['language_embeds']
            prompt_len = self.weights['language_embeds'].shape[0]
        start = self.num_views * 256
        self.buffers['encoder_x'][start: start + prompt_len].copy_(prompt_embeds)
        self.buffers['valid_encoder_len'].fill_(start + prompt_len)
        self.buffers['decoder_rope_weights'].copy_(self.get_decoder_rope_weights(prompt_len))
        self.buffers['observation_images_normalized'].copy_(observation_images_normalized)
        self.buffers['diffusion_noise'].copy_(diffusion_noise)

    def forward(self, observation_images_normalized: torch.Tensor, diffusion_noise: torch.Tensor,
                task_prompt: str = None, state_tokens: np.ndarray = None) -> torch.Tensor:
        self.stage_inputs(observation_images_normalized, diffusion_noise, task_prompt, state_tokens)
        self._engine.replay()
        return self.buffers['diffusion_noise']
