"""Converted-checkpoint files for Pi0Inference / Pi05Inference.

The reference's converters write `pickle.dump(dict[str, torch.Tensor(bf16)])` (/root/reference/convert_from_jax.py:279-326,
convert_from_jax_pi05.py, README.md:46-60) and its users `pickle.load` that file, which executes whatever the file says.
This module reads that same format with an unpickler that can build tensors and nothing else, and offers safetensors as
the on-disk format to convert to once: no code execution on load, memory-mapped, loaded straight to the device.

    ck = load_checkpoint("pi0.pkl")            # or .safetensors; dict[str, Tensor], same keys and shapes
    save_safetensors(ck, "pi0.safetensors")
    Pi0Inference(load_checkpoint("pi0.safetensors", device="cuda"), num_views=3, chunk_size=50)
"""
import collections
import io
import pickle

import torch


def _storage_from_bytes(b):
    # what torch.storage._load_from_bytes does, but with the tensor-only loader
    return torch.load(io.BytesIO(b), weights_only=True)


class _TensorOnlyUnpickler(pickle.Unpickler):
    """Resolves only the globals a pickled dict of plain tensors needs; anything else is refused."""

    _ALLOWED = {
        ("collections", "OrderedDict"): collections.OrderedDict,
        ("torch._utils", "_rebuild_tensor_v2"): torch._utils._rebuild_tensor_v2,
        ("torch.storage", "_load_from_bytes"): _storage_from_bytes,
        ("torch", "bfloat16"): torch.bfloat16, ("torch", "float32"): torch.float32, ("torch", "float16"): torch.float16,
        ("torch", "int32"): torch.int32, ("torch", "int64"): torch.int64,
    }
    for _name in ("BFloat16Storage", "FloatStorage", "HalfStorage", "IntStorage", "LongStorage"):
        _ALLOWED[("torch", _name)] = getattr(torch, _name)

    def find_class(self, module, name):
        try:
            return self._ALLOWED[(module, name)]
        except KeyError:
            raise pickle.UnpicklingError("refusing to resolve %s.%s while loading a checkpoint" % (module, name)) from None


def load_pickle(path):
    """The reference's pickle format, without executing anything from the file."""
    with open(path, "rb") as f:
        obj = _TensorOnlyUnpickler(f).load()
    if not isinstance(obj, dict) or not all(isinstance(k, str) and torch.is_tensor(v) for k, v in obj.items()):
        raise ValueError("%s does not hold a dict of tensors" % path)
    return dict(obj)


def save_safetensors(checkpoint, path):
    from safetensors.torch import save_file
    save_file({k: torch.as_tensor(v).detach().cpu().contiguous() for k, v in checkpoint.items()}, path)


def load_safetensors(path, device="cpu"):
    """Memory-mapped read; with a device the tensors go there directly."""
    from safetensors import safe_open
    out = {}
    with safe_open(path, framework="pt", device=str(device)) as f:
        for k in f.keys():
            out[k] = f.get_tensor(k)
    return out


def load_checkpoint(path, device="cpu"):
    if str(path).endswith(".safetensors"):
        return load_safetensors(path, device)
    ck = load_pickle(path)
    return {k: v.to(device) for k, v in ck.items()} if str(device) != "cpu" else ck
