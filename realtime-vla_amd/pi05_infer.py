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
        else:
            self.max_prompt_len = len(checkpoint['language_embeds'])
        print(f"max_prompt_len: {self.max_prompt_len}, max_tokenize_len: {self.max_tokenize_len}")

        self._engine = Engine(capi.PI05, checkpoint, num_views, self.max_prompt_len, chunk_size,
                              skip_keys=("embedding_weight", "language_embeds"))
        self.weights = self._engine.weights
        self.buffers = self._engine.buffers
        dev = self._engine.device
        self.weights['language_embeds'] = torch.as_tensor(checkpoint['language_embeds']).to(device=dev, dtype=torch.bfloat16) \
            if 'language_embeds' in checkpoint else torch.zeros(0, 2048, dtype=torch.bfloat16, device=dev)

        prefix_alloc = self.num_views * 256 + self.max_prompt_len
        max_pos = (self.num_views * 256 + self.max_prompt_len - 1) + self.chunk_size
        self._rope_table = rope_table(0, max_pos + 1, dev)
        self.buffers['encoder_rope_weights'].copy_(self._rope_table[:prefix_alloc])
        self.buffers['valid_encoder_len'].fill_(self.num_views * 256 + 1)
        self.buffers['decoder_rope_weights'].copy_(self.get_decoder_rope_weights(1))

        self.prompt_embedding = None
        self._prompt_embed_scale = None
        if self.discrete_state_input:
            emb_w = checkpoint["embedding_weight"]
            emb_w_t = torch.from_numpy(emb_w) if isinstance(emb_w, np.ndarray) else emb_w
            emb_w_t = emb_w_t.to(device=dev, dtype=torch.bfloat16, non_blocking=True)
            self.prompt_embedding = nn.Embedding(num_embeddings=emb_w_t.shape[0], embedding_dim=emb_w_t.shape[1],
                                                 device=dev, dtype=torch.bfloat16)
            with torch.no_grad():
                self.prompt_embedding.weight.copy_(emb_w_t)
            self._prompt_embed_scale = float(emb_w_t.shape[1] ** 0.5)
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

    def build_prompt_embeds(self, task_prompt: str, state_tokens: np.ndarray):
        task_prompt = task_prompt.strip().replace("_", " ")
        state_str = " ".join(map(str, state_tokens.tolist()))
        full_prompt = f"Task: {task_prompt}, State: {state_str};\nAction: "
        token_ids = self.tokenizer(full_prompt, return_tensors="pt", truncation=True, max_length=self.max_tokenize_len,
                                   padding=False)["input_ids"][0].to(device=self._engine.device, non_blocking=True)
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

    def stage_inputs(self, observation_images_normalized, diffusion_noise, task_prompt=None, state_tokens=None):
        """The host-side staging of forward() without the replay (pi05_infer.py:811-824)."""
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
