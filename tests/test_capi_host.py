"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol the
header declares, validates dimensions and bindings, and reports errors as status codes."""
import ctypes
import os
import re

import pytest

import rtvla_capi as capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(capi.LIB_PATH):
        import build
        build.build(force=True)
    return capi.load()


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "rtvla.h")).read()
    declared = set(re.findall(r"\b(rtvla_[a-z_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(capi.SYMBOLS), "binding table and header differ: %s" % (declared ^ set(capi.SYMBOLS))
    for name in declared:
        assert hasattr(lib, name)
    assert lib.rtvla_version() >= 1


def test_the_shipped_library_reads_no_environment(lib):
    """The tuning hooks (forced tiles, graph-branch knobs) exist only in builds made with -DRTVLA_TUNING: the shipped library
    imports no getenv and carries none of the knob names."""
    import subprocess
    syms = subprocess.run(["nm", "-D", "--undefined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    assert "getenv" not in syms
    blob = open(capi.LIB_PATH, "rb").read()
    for knob in (b"RTVLA_FORCE_TILE", b"RTVLA_FORK_GROUP", b"RTVLA_PRINT_TILES"):
        assert knob not in blob


def test_create_validates_dimensions(lib):
    for bad in [(capi.PI0, 0, 0, 50), (capi.PI0, 5, 0, 50), (capi.PI0, 1, -1, 50), (capi.PI0, 1, 0, 0), (3, 1, 0, 50), (capi.DM0, 0, 10, 50), (capi.DM0, 5, 10, 50)]:
        with pytest.raises(capi.RtvlaError):
            capi.Context(*bad)
    with pytest.raises(capi.RtvlaError) as e:
        capi.Context(capi.PI0, 1, 0, 128)         # 129 suffix rows do not fit the two 64-row blocks of the action-expert kernels
    assert e.value.code == 7
    with pytest.raises(capi.RtvlaError) as e:
        capi.Context(capi.DM0, 1, 10, 65)         # DM0's buffers hold one 64-row block
    assert e.value.code == 7
    # the converted Pi0 / DM0 checkpoints are tied to 10 flow steps (dt folded into the output projection, 10 time biases);
    # Pi05 scales by -1/num_steps itself and takes 1..10
    for model, steps in ((capi.PI0, 5), (capi.PI0, 11), (capi.PI0, 20), (capi.DM0, 9), (capi.PI05, 11)):
        with pytest.raises(capi.RtvlaError) as e:
            capi.Context(model, 1, 4, 10, steps)
        assert e.value.code == 7, (model, steps)
    capi.Context(capi.PI05, 1, 4, 10, 4).close()
    capi.Context(capi.PI0, 1, 0, 63).close()
    capi.Context(capi.PI0, 1, 0, 127).close()
    capi.Context(capi.PI05, 3, 52, 128).close()


def test_tensor_table_matches_the_reference_layout(lib):
    c = capi.Context(capi.PI0, 3, 20, 50)
    t = {n: (e, s, w) for n, e, s, w, _ in c.tensors()}
    assert t["vision_patch_embedding_w"] == (2, (14, 14, 3, 1152), True)
    assert t["encoder_ffn_gate_w"] == (2, (18, 2048, 16384), True)
    assert t["decoder_action_fused_time_biases"] == (2, (10, 1024), True)
    assert t["language_embeds"] == (2, (20, 2048), True)
    assert t["diffusion_noise"] == (2, (50, 32), False)
    assert t["encoder_rope_weights"] == (2, (788, 256), False)
    assert t["decoder_rope_weights"] == (2, (51, 256), False)
    assert len([n for n, v in t.items() if v[2]]) == 38      # pi0_infer.py:1245-1287 lists 38 weights
    c5 = capi.Context(capi.PI05, 3, 52, 50)
    t5 = {n: (e, s, w) for n, e, s, w, _ in c5.tensors()}
    assert t5["valid_encoder_len"] == (4, (1,), False)
    assert t5["decoder_pre_attn_norm_mod_w"] == (2, (18, 1024, 3072), True)
    assert t5["decoder_rope_weights"] == (2, (50, 256), False)
    assert "observation_state_normalized" not in t5 and "decoder_state_in_proj_w" not in t5


def test_dm0_tensor_table(lib):
    """dm0_infer.py:986-1026 (weights), 754 (token ids)."""
    c = capi.Context(capi.DM0, 3, 100, 50, 10, 23, 28)
    t = {n: (e, s, w) for n, e, s, w, _ in c.tensors()}
    assert t["images"] == (2, (3, 3, 728, 728), False)
    assert t["input_ids"] == (4, (100,), False)
    assert t["diffusion_noise"] == (2, (50, 32), False)
    assert t["prefix_rope_weights"] == (2, (3 * 169 + 100, 128), False)
    assert t["decoder_rope_weights"] == (2, (50, 128), False)
    assert t["vision_fused_qkv_w"] == (2, (23, 1024, 3072), True)
    assert t["vision_qkv_col_sum"] == (4, (23, 3072), True)          # fp32, as the reference keeps them
    assert t["llm_attn_qkv_w"] == (2, (28, 2048, 4096), True)
    assert t["decoder_attn_qkv_w"] == (2, (28, 1024, 4096), True)
    assert t["vision_ds2_w"] == (2, (3, 3, 2048, 4096), True)
    assert 0 < c.workspace_bytes() < 6 << 30
    c.close()


def test_bind_errors_are_status_codes(lib):
    c = capi.Context(capi.PI0, 1, 0, 50)
    with pytest.raises(capi.RtvlaError) as e:
        c.bind("no_such_tensor", 256, 16)
    assert e.value.code == capi.ERR_NAME and "no_such_tensor" in str(e.value)
    with pytest.raises(capi.RtvlaError) as e:
        c.bind("diffusion_noise", 256, 50 * 32 * 2 + 2)
    assert e.value.code == capi.ERR_SIZE
    with pytest.raises(capi.RtvlaError):
        c.bind("diffusion_noise", 0, 50 * 32 * 2)           # null pointer
    with pytest.raises(capi.RtvlaError):
        c.bind("diffusion_noise", 257, 50 * 32 * 2)         # misaligned
    c.bind("language_embeds", 0, 0)                          # an empty prompt binds a null, zero-byte tensor


def test_calls_out_of_order_are_rejected(lib):
    c = capi.Context(capi.PI0, 1, 0, 50)
    for fn in (c.prepare, c.forward, c.graph_capture):
        with pytest.raises(capi.RtvlaError) as e:
            fn(0)
        assert e.value.code in (4, 5)
    with pytest.raises(capi.RtvlaError):
        c.graph_launch(0)
    with pytest.raises(capi.RtvlaError):
        c.bind_workspace(256, 1024)                          # too small
    assert lib.rtvla_forward(None, None) == 1 and lib.rtvla_destroy(None) == 1


def test_workspace_layout(lib):
    small = capi.Context(capi.PI0, 1, 0, 50, vision_layers=2, llm_layers=2)
    big = capi.Context(capi.PI0, 3, 200, 50)
    assert 0 < small.workspace_bytes() < big.workspace_bytes() < 8 << 30
    bufs = {n: (off, rows, cols, ld, e) for n, off, rows, cols, ld, e in big.buffers()}
    assert bufs["encoder_x"][1:4] == (968, 2048, 2048)
    assert bufs["vision_hidden"][2:4] == (4304, 4352)        # K padded to the 128-wide stage pair
    assert bufs["splitk_partial"][4] == 4
    offs = sorted((v[0], v[0] + v[1] * v[3] * v[4]) for v in bufs.values())
    assert all(a[1] <= b[0] for a, b in zip(offs, offs[1:])), "workspace regions overlap"
    assert all(v[0] % 256 == 0 for v in bufs.values())
    assert lib.rtvla_pretile_elems(588, 1152) == 72 * 20 * 512


def test_unit_and_static_entry_points_check_sizes_before_touching_a_device(lib):
    p = ctypes.c_void_p(4096)
    assert lib.rtvla_linear_workspace_bytes(768, 1152, 3456, -1, 1) > 768 * 1152 * 2
    assert lib.rtvla_linear_workspace_bytes(16, 12, 16, -1, 1) == 0                    # K must be a multiple of 8
    assert lib.rtvla_linear_workspace_bytes(129, 1024, 64, capi.TILE_SKINNY, 1) == 0   # the streaming kernel takes at most 128 rows
    assert lib.rtvla_linear(p, 16, 128, p, 16, None, p, p, 16, -1, 1, None) == capi.ERR_SIZE
    assert lib.rtvla_linear(None, 16, 128, p, 16, None, p, p, 1 << 20, -1, 1, None) == 1
    r, c = ctypes.c_int(), ctypes.c_int()
    assert lib.rtvla_linear_tile_shape(0, ctypes.byref(r), ctypes.byref(c)) == 0 and (r.value, c.value) == (224, 256)
    assert lib.rtvla_linear_tile_shape(99, ctypes.byref(r), ctypes.byref(c)) == 1
    # the allocation-free image entry point: a frame whose intermediate exceeds the static buffer is refused up front
    assert lib.rtvla_preprocess_image_static(p, 2400, 2400, p, None) == capi.ERR_LIMIT
    assert lib.rtvla_preprocess_image_static(p, 8000, 250, p, None) == capi.ERR_LIMIT  # shrink factor above 31
    assert lib.rtvla_preprocess_image_static(None, 10, 10, p, None) == 1
    assert capi.STATIC_SCRATCH_BYTES == 2160 * 224 * 3
