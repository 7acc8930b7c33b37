"""Observation pre-/post-processing on the device, with the method names and semantics of the reference's evaluation
harness (/root/reference/test.py:88-201: `_parse_image`, `_resize_with_pad`, `_normalize_image`, `_normalize_state`,
`_digitize_state`, `_unnormalize_actions`, `_apply_input_transforms`, and the action post-processing of `infer`).
The reference runs these in numpy / Pillow on the host for every observation; here each is one or two HIP kernels of
librtvla.so writing straight into the model's input buffers.  PyTorch only owns the memory."""
import ctypes

import numpy as np
import torch

import rtvla_capi as capi

_P = ctypes.c_void_p


class ObservationTransforms:
    def __init__(self, model_version, norm_stats=None, state_len=7, action_dim=7, device=None):
        if model_version not in ("pi0", "pi05"):
            raise ValueError("model_version must be 'pi0' or 'pi05'")
        if not torch.cuda.is_available():
            raise RuntimeError("realtime-vla_amd needs a ROCm GPU (MI355X / gfx950); there is no CPU path")
        self.lib = capi.load()
        self.model_version = model_version
        self.mode = 0 if model_version == "pi0" else 1
        self.norm_stats = norm_stats
        self.state_len, self.action_dim = int(state_len), int(action_dim)
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        keys = ("mean", "std") if model_version == "pi0" else ("q01", "q99")
        self._stats = {}
        for group in ("state", "actions"):
            if norm_stats and group in norm_stats:
                a = torch.tensor(np.asarray(norm_stats[group][keys[0]], dtype=np.float64)[:32], device=self.device)
                b = torch.tensor(np.asarray(norm_stats[group][keys[1]], dtype=np.float64)[:32], device=self.device)
                self._stats[group] = (a, b)
        self._scratch = torch.empty(0, dtype=torch.uint8, device=self.device)

    def _stream(self):
        return _P(torch.cuda.current_stream(self.device).cuda_stream)

    @staticmethod
    def _check(rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with rtvla status %d" % (what, rc))

    # ---- images ----
    def _parse_image(self, image):
        """test.py:88-94, but the result lives on the device as uint8 HWC."""
        image = torch.as_tensor(image)
        if image.is_floating_point():
            image = (255 * image).to(torch.uint8)                 # truncation, as numpy's astype
        if image.shape[0] == 3:
            image = image.permute(1, 2, 0)
        return image.to(self.device).contiguous()

    def resize_pad_normalize_into(self, image, out_view, static_scratch=False):
        """_resize_with_pad + _normalize_image of one image into out_view (bf16 [224, 224, 3], e.g. one view of the
        model's observation_images_normalized buffer).  With static_scratch the library's built-in intermediate buffer
        is used and nothing is allocated (frames of at most 2160 rows at full width; calls on one GPU must not overlap)."""
        img = self._parse_image(image)
        h, w, c = img.shape
        if c != 3 or img.dtype != torch.uint8:
            raise ValueError("expected an RGB uint8 image, got shape %s dtype %s" % (tuple(img.shape), img.dtype))
        if out_view.dtype != torch.bfloat16 or tuple(out_view.shape) != (224, 224, 3) or not out_view.is_contiguous():
            raise ValueError("out_view must be a contiguous bf16 [224, 224, 3] tensor")
        if static_scratch:
            rc = self.lib.rtvla_preprocess_image_static(_P(img.data_ptr()), h, w, _P(out_view.data_ptr()), self._stream())
            if rc == capi.ERR_LIMIT:
                raise ValueError("a %d x %d frame does not fit the library's %d-byte static intermediate buffer (or shrinks by more "
                                 "than a factor of 31)" % (h, w, capi.STATIC_SCRATCH_BYTES))
            self._check(rc, "rtvla_preprocess_image_static")
            self._keep = img
            return out_view
        need = self.lib.rtvla_preprocess_image_scratch(h, w)
        if self._scratch.numel() < need:
            self._scratch = torch.empty(need, dtype=torch.uint8, device=self.device)
        self._check(self.lib.rtvla_preprocess_image(_P(img.data_ptr()), h, w, _P(out_view.data_ptr()), _P(self._scratch.data_ptr()),
                                                    self._scratch.numel(), self._stream()), "rtvla_preprocess_image")
        self._keep = img                                           # alive until the stream has consumed it
        return out_view

    # ---- state ----
    def _normalize_state(self, state, want_bins=False, out_bf16=None):
        """test.py:121-137: returns (normalised float64 [32] on the device, 256-bin indices or None); optionally also
        writes the float32 -> bf16 value into out_bf16 (the model's observation_state_normalized buffer)."""
        if "state" not in self._stats:
            return None, None
        a, b = self._stats["state"]
        st = torch.as_tensor(np.asarray(state, dtype=np.float64)).to(self.device)
        z = torch.empty(32, dtype=torch.float64, device=self.device)
        bins = torch.empty(32, dtype=torch.int32, device=self.device) if want_bins else None
        self._check(self.lib.rtvla_preprocess_state(_P(st.data_ptr()), int(st.numel()), _P(a.data_ptr()), _P(b.data_ptr()), int(a.numel()), self.mode,
                                                    _P(out_bf16.data_ptr()) if out_bf16 is not None else None, _P(z.data_ptr()),
                                                    _P(bins.data_ptr()) if bins is not None else None, self._stream()), "rtvla_preprocess_state")
        return z, bins

    # ---- actions ----
    def postprocess_actions(self, actions_bf16, ori_state):
        """test.py:196-201: un-normalise, add the current state, keep the grippers absolute -> float64 [chunk, action_dim]."""
        if "actions" not in self._stats:
            return None
        a, b = self._stats["actions"]
        if actions_bf16.dtype != torch.bfloat16 or actions_bf16.shape[-1] != 32 or not actions_bf16.is_contiguous():
            raise ValueError("actions must be a contiguous bf16 [chunk, 32] tensor")
        chunk = int(actions_bf16.shape[0])
        st = torch.zeros(32, dtype=torch.float64, device=self.device)
        s_in = torch.as_tensor(np.asarray(ori_state, dtype=np.float64))
        st[: s_in.numel()] = s_in.to(self.device)
        out = torch.empty(chunk, self.action_dim, dtype=torch.float64, device=self.device)
        self._check(self.lib.rtvla_postprocess_actions(_P(actions_bf16.data_ptr()), chunk, _P(a.data_ptr()), _P(b.data_ptr()), int(a.numel()), self.mode,
                                                       _P(st.data_ptr()), self.action_dim, _P(out.data_ptr()), self._stream()), "rtvla_postprocess_actions")
        return out

    # ---- the whole observation, as TritonInference.infer does around policy.forward (test.py:181-205) ----
    def infer(self, policy, inputs, noise):
        """inputs: {"state", "base_0_rgb", "left_wrist_0_rgb", "right_wrist_0_rgb"[, "prompt"]}; returns {"actions": ndarray}."""
        ori_state = np.asarray(inputs["state"]).copy()
        views = ["base_0_rgb", "left_wrist_0_rgb", "right_wrist_0_rgb"][: policy.num_views]
        img_buf = policy.buffers["observation_images_normalized"]
        for v, name in enumerate(views):
            self.resize_pad_normalize_into(inputs[name], img_buf[v])
        noise_t = torch.as_tensor(noise)
        if self.model_version == "pi0":
            self._normalize_state(ori_state, out_bf16=policy.buffers["observation_state_normalized"])
            actions = policy.forward(img_buf, policy.buffers["observation_state_normalized"], noise_t)
        else:
            _, bins = self._normalize_state(ori_state, want_bins=True)
            actions = policy.forward(img_buf, noise_t, inputs.get("prompt"), bins[: self.state_len].cpu().numpy())
        out = self.postprocess_actions(actions, ori_state)
        return {"actions": out.cpu().numpy()}
