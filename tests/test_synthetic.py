"""The seeded generator behind every synthetic checkpoint: integer-exact and device independent."""
import math

import torch

import synthetic as syn


def _ref_normal(key, i):
    tot = 0
    for half in range(2):
        h = syn._splitmix64_int((2 * i + half + key) & syn._M64)
        for f in range(4):
            tot += (h >> (16 * f)) & 0xFFFF
    return (tot - 4 * 65535) * syn._IH_SCALE


def test_splitmix64_known_answers():
    # first outputs of the published splitmix64 sequence seeded with 1234567
    x = 1234567
    got = []
    for _ in range(3):
        got.append(syn._splitmix64_int(x))
        x = (x + syn._GOLD) & syn._M64
    assert got == [6457827717110365317, 3203168211198807973, 9817491932198370423]


def test_tensor_stream_matches_python_integers():
    key = syn.stream_key(11, "vision_attn_qkv_w")
    v = syn._normal_chunk(key, 5, 64, 1.0, "cpu")
    for i in range(64):
        assert abs(v[i].item() - _ref_normal(key, 5 + i)) < 1e-6


def test_chunking_does_not_change_values():
    a = syn.normal_bf16(3, "w", (3, 100003), 0.02)
    old = syn._CHUNK_CPU
    try:
        syn._CHUNK_CPU = 4099
        b = syn.normal_bf16(3, "w", (3, 100003), 0.02)
    finally:
        syn._CHUNK_CPU = old
    assert torch.equal(a, b)


def test_moments_and_ranges():
    x = syn.normal_bf16(1, "a", (1 << 20,), 0.02).float()
    assert abs(x.mean().item()) < 1e-4 and abs(x.std().item() - 0.02) < 2e-4
    u = syn.uniform_pm1_bf16(1, "img", (1 << 20,)).float()
    assert u.min().item() >= -1.0 and u.max().item() <= 1.0 and abs(u.mean().item()) < 5e-3
    ids = syn.randint(1, "ids", 10000, 257152)
    assert ids.min().item() >= 0 and ids.max().item() < 257152 and ids.unique().numel() > 9000


def test_streams_are_keyed_by_name_and_seed():
    a = syn.normal_bf16(1, "a", (1000,))
    assert not torch.equal(a, syn.normal_bf16(1, "b", (1000,)))
    assert not torch.equal(a, syn.normal_bf16(2, "a", (1000,)))
    assert torch.equal(a, syn.normal_bf16(1, "a", (1000,)))


def test_time_embedding_closed_form():
    # /root/reference/convert_from_jax.py:133-140: periods 4e-3 .. 4.0, [sin | cos]
    e = syn._sincos_time(0.3)
    assert e.shape == (1024,)
    assert abs(e[0].item() - math.sin(2 * math.pi / 4e-3 * 0.3)) < 1e-4
    assert abs(e[511].item() - math.sin(2 * math.pi / 4.0 * 0.3)) < 1e-6
    assert abs(e[512 + 511].item() - math.cos(2 * math.pi / 4.0 * 0.3)) < 1e-6
    assert torch.allclose(e[:512] ** 2 + e[512:] ** 2, torch.ones(512), atol=1e-5)


def test_checkpoint_layout_matches_reference_keys():
    ck = syn.pi0_checkpoint(5, 3, vision_layers=1, llm_layers=1)
    assert ck["vision_patch_embedding_w"].shape == (14, 14, 3, 1152)
    assert ck["encoder_attn_qkv_w"].shape == (1, 2048, 2560)
    assert ck["decoder_ffn_down_w"].shape == (1, 4096, 1024)
    assert ck["language_embeds"].shape == (3, 2048)
    assert all(v.dtype == torch.bfloat16 for v in ck.values())
    assert torch.all(ck["vision_pre_attn_norm_w"] == 1) and torch.all(ck["vision_final_norm_b"] == 0)
    ck5 = syn.pi05_checkpoint(5, 3, vision_layers=1, llm_layers=1, state_tokens=2)
    assert ck5["language_embeds"].shape == (5, 2048)
    assert ck5["decoder_time_embeds"].shape == (10, 1024)
    assert ck5["decoder_pre_attn_norm_mod_w"].shape == (1, 1024, 3072)
    # prompt rows are embedding rows scaled by sqrt(2048)
    ids = syn.randint(5, "prompt_ids", 3, syn.VOCAB)
    row = syn.embedding_rows(5, ids[:1])[0].float() * math.sqrt(2048.0)
    assert torch.equal(row.to(torch.bfloat16), ck["language_embeds"][0])
