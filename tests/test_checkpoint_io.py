"""Converted-checkpoint files: the reference's pickle format read without code execution, and safetensors."""
import os
import pickle
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "realtime-vla_amd"))
import checkpoint_io as cio          # noqa: E402
import synthetic as syn              # noqa: E402


def _small_checkpoint():
    ck = syn.pi0_checkpoint(3, 2, "cpu", 1, 1)
    return {k: ck[k] for k in ("vision_patch_embedding_w", "vision_attn_qkv_b", "decoder_action_fused_time_biases", "language_embeds")}


def test_reference_pickle_format_loads_bit_exactly(tmp_path):
    ck = _small_checkpoint()
    path = tmp_path / "pi0.pkl"
    with open(path, "wb") as f:                     # exactly what the converter does (convert_from_jax.py:324-325)
        pickle.dump(ck, f)
    got = cio.load_checkpoint(str(path))
    assert set(got) == set(ck)
    for k in ck:
        assert got[k].dtype == torch.bfloat16 and got[k].shape == ck[k].shape and torch.equal(got[k], ck[k])


def test_pickle_loader_refuses_anything_but_tensors(tmp_path):
    class Evil:
        def __reduce__(self):
            return (os.system, ("echo should-never-run",))
    path = tmp_path / "evil.pkl"
    with open(path, "wb") as f:
        pickle.dump({"vision_patch_embedding_b": Evil()}, f)
    with pytest.raises(pickle.UnpicklingError):
        cio.load_pickle(str(path))
    path2 = tmp_path / "notadict.pkl"
    with open(path2, "wb") as f:
        pickle.dump([torch.zeros(2)], f)
    with pytest.raises(ValueError):
        cio.load_pickle(str(path2))


def test_safetensors_round_trip(tmp_path):
    ck = _small_checkpoint()
    ck["strided"] = ck["vision_patch_embedding_w"][:, :, 1]          # non-contiguous view
    path = str(tmp_path / "pi0.safetensors")
    cio.save_safetensors(ck, path)
    got = cio.load_checkpoint(path)
    assert set(got) == set(ck)
    for k in ck:
        assert got[k].dtype == ck[k].dtype and torch.equal(got[k], ck[k])
