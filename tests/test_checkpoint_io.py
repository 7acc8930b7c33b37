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


def test_weight_fingerprint_is_exact_and_order_sensitive():
    import tile_cache as tc
    ck = _small_checkpoint()
    a = tc.fingerprint(ck)
    assert a == tc.fingerprint({k: v.clone() for k, v in reversed(list(ck.items()))}) and len(a) == 32
    flipped = {k: v.clone() for k, v in ck.items()}
    flipped["vision_attn_qkv_b"][0, 5] += 1.0
    assert tc.fingerprint(flipped) != a
    swapped = {k: v.clone() for k, v in ck.items()}
    w = swapped["vision_attn_qkv_b"]
    w[0, 1], w[0, 2] = ck["vision_attn_qkv_b"][0, 2], ck["vision_attn_qkv_b"][0, 1]      # same multiset of values, other order
    assert not torch.equal(w, ck["vision_attn_qkv_b"]) and tc.fingerprint(swapped) != a
    renamed = dict(ck); renamed["other_name"] = renamed.pop("language_embeds")
    assert tc.fingerprint(renamed) != a


def test_tile_cache_file_round_trip_and_header_checks(tmp_path):
    import tile_cache as tc
    cache = tc.TileCache(tmp_path / "tiles")
    key = bytes(range(32))
    region = torch.arange(5000, dtype=torch.int64).to(torch.uint8)
    assert not cache.load_into(key, 2, 0, 10, 27, 18, torch.empty_like(region))               # nothing stored yet
    path = cache.store(key, 2, 0, 10, 27, 18, region)
    assert os.path.getsize(path) == 64 + 5000
    back = torch.zeros_like(region)
    assert cache.load_into(key, 2, 0, 10, 27, 18, back) and torch.equal(back, region)
    for other in ((3, 0, 10, 27, 18), (2, 1, 10, 27, 18), (2, 0, 5, 27, 18), (2, 0, 10, 2, 18), (2, 0, 10, 27, 2)):   # layout version, model, flow steps, layer counts
        assert not cache.load_into(key, *other, torch.zeros_like(region))
    assert not cache.load_into(key, 2, 0, 10, 27, 18, torch.zeros(4999, dtype=torch.uint8))  # another size
    assert not cache.load_into(bytes(32), 2, 0, 10, 27, 18, torch.zeros_like(region))         # another checkpoint
    with open(path, "r+b") as f:                                                           # a truncated / foreign file
        f.write(b"garbage!")
    assert not cache.load_into(key, 2, 0, 10, 27, 18, torch.zeros_like(region))
