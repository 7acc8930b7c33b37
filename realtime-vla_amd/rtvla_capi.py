"""ctypes binding of librtvla.so (C ABI declared in include/rtvla.h).

The library is the only compute path: there is no eager / CPU fallback, and importing this
module on a machine where the shared library has not been built raises.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librtvla.so")

PI0, PI05, DM0 = 0, 1, 2

STAGE_VISION_EMBED = 0
STAGE_VISION_LAYER = 1
STAGE_PROJECT = 2
STAGE_PREFIX_LAYER = 3
STAGE_SUFFIX_INIT = 4
STAGE_SUFFIX_STEP_BEGIN = 5
STAGE_SUFFIX_LAYER = 6
STAGE_SUFFIX_STEP_END = 7

ERR_NAME, ERR_SIZE, ERR_STATE, ERR_LIMIT = 2, 3, 4, 7
TILE_AUTO, TILE_SKINNY = -1, -2
ACT_BIAS_GELU, ACT_GEGLU, ACT_SWIGLU = 1, 2, 3
NORM_NONE, NORM_RMS, NORM_LAYER = 0, 1, 2
ATTN_GEMMA_PREFIX, ATTN_GEMMA_SUFFIX, ATTN_GQA128_PREFIX, ATTN_GQA128_SUFFIX, ATTN_VIT64, ATTN_SIGLIP = range(6)
STATIC_SCRATCH_BYTES = 2160 * 224 * 3          # RTVLA_STATIC_SCRATCH_BYTES


class Dims(ctypes.Structure):
    _fields_ = [("model", ctypes.c_int32), ("num_views", ctypes.c_int32), ("prompt_len", ctypes.c_int32),
                ("chunk_size", ctypes.c_int32), ("num_steps", ctypes.c_int32), ("vision_layers", ctypes.c_int32),
                ("llm_layers", ctypes.c_int32)]


# every symbol include/rtvla.h declares: name -> (restype, argtypes)
_P = ctypes.c_void_p
SYMBOLS = {
    "rtvla_version": (ctypes.c_int, []),
    "rtvla_create": (ctypes.c_int, [ctypes.POINTER(Dims), ctypes.POINTER(_P)]),
    "rtvla_destroy": (ctypes.c_int, [_P]),
    "rtvla_last_error": (ctypes.c_char_p, [_P]),
    "rtvla_tensor_count": (ctypes.c_int, [_P]),
    "rtvla_tensor_info": (ctypes.c_int, [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_int32),
                                         ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64 * 4),
                                         ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]),
    "rtvla_bind": (ctypes.c_int, [_P, ctypes.c_char_p, _P, ctypes.c_size_t]),
    "rtvla_workspace_bytes": (ctypes.c_size_t, [_P]),
    "rtvla_bind_workspace": (ctypes.c_int, [_P, _P, ctypes.c_size_t]),
    "rtvla_buffer_count": (ctypes.c_int, [_P]),
    "rtvla_buffer_info": (ctypes.c_int, [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_size_t),
                                         ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                                         ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32)]),
    "rtvla_prepare": (ctypes.c_int, [_P, _P]),
    "rtvla_prepare_with_tiles": (ctypes.c_int, [_P, _P]),
    "rtvla_tiled_bytes": (ctypes.c_size_t, [_P]),
    "rtvla_tile_layout_version": (ctypes.c_int, []),
    "rtvla_forward": (ctypes.c_int, [_P, _P]),
    "rtvla_forward_stage": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "rtvla_graph_capture": (ctypes.c_int, [_P, _P]),
    "rtvla_graph_launch": (ctypes.c_int, [_P, _P]),
    "rtvla_launch_count": (ctypes.c_int, [_P]),
    "rtvla_time_stage": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P, ctypes.POINTER(ctypes.c_float)]),
    "rtvla_time_launch": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P,
                                         ctypes.POINTER(ctypes.c_float), ctypes.c_char_p, ctypes.c_size_t]),
    "rtvla_time_forward": (ctypes.c_int, [_P, ctypes.c_int, _P, ctypes.POINTER(ctypes.c_float)]),
    "rtvla_pretile_elems": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int]),
    "rtvla_pretile": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, _P]),
    "rtvla_linear_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 5),
    "rtvla_linear": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, ctypes.c_int, _P, _P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, _P]),
    "rtvla_time_linear": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, ctypes.c_int, _P, _P, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, _P, ctypes.POINTER(ctypes.c_float)]),
    "rtvla_linear_tile_shape": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "rtvla_linear_act_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "rtvla_linear_act": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, _P, ctypes.c_int, _P, ctypes.c_int, _P, _P, ctypes.c_size_t, ctypes.c_int, _P]),
    "rtvla_reduce_norm": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P, _P, ctypes.c_int, _P, _P, ctypes.c_float, _P, _P, _P]),
    "rtvla_attention_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "rtvla_attention": (ctypes.c_int, [ctypes.c_int, _P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int, _P,
                                       ctypes.c_int, _P, ctypes.c_size_t, _P]),
    "rtvla_preprocess_image_scratch": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int]),
    "rtvla_preprocess_image": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, _P, ctypes.c_size_t, _P]),
    "rtvla_preprocess_image_static": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _P, _P]),
    "rtvla_preprocess_state": (ctypes.c_int, [_P, ctypes.c_int, _P, _P, ctypes.c_int, ctypes.c_int, _P, _P, _P, _P]),
    "rtvla_postprocess_actions": (ctypes.c_int, [_P, ctypes.c_int, _P, _P, ctypes.c_int, ctypes.c_int, _P, ctypes.c_int, _P, _P]),
}

_lib = None


def load():
    """Load librtvla.so and declare every entry point; raises if the library is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("librtvla.so is not built (%s); run `python realtime-vla_amd/build.py`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class RtvlaError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("rtvla error %d: %s" % (code, text))
        self.code = code


class Context:
    """Thin owner of one rtvla_ctx."""

    def __init__(self, model, num_views, prompt_len, chunk_size, num_steps=10, vision_layers=27, llm_layers=18):
        self.lib = load()
        self.dims = Dims(model, num_views, prompt_len, chunk_size, num_steps, vision_layers, llm_layers)
        self.handle = _P()
        rc = self.lib.rtvla_create(ctypes.byref(self.dims), ctypes.byref(self.handle))
        if rc != 0:
            self.handle = None
            raise RtvlaError(rc, "rtvla_create rejected the dimensions")

    def close(self):
        if getattr(self, "handle", None):
            self.lib.rtvla_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, rc):
        if rc != 0:
            raise RtvlaError(rc, self.lib.rtvla_last_error(self.handle).decode())

    def tensors(self):
        out = []
        for i in range(self.lib.rtvla_tensor_count(self.handle)):
            name, elem, rank = ctypes.c_char_p(), ctypes.c_int32(), ctypes.c_int32()
            shape, isw, req = (ctypes.c_int64 * 4)(), ctypes.c_int32(), ctypes.c_int32()
            self.check(self.lib.rtvla_tensor_info(self.handle, i, ctypes.byref(name), ctypes.byref(elem), ctypes.byref(rank),
                                                  ctypes.byref(shape), ctypes.byref(isw), ctypes.byref(req)))
            out.append((name.value.decode(), elem.value, tuple(shape[j] for j in range(rank.value)), bool(isw.value), bool(req.value)))
        return out

    def buffers(self):
        out = []
        for i in range(self.lib.rtvla_buffer_count(self.handle)):
            name, off = ctypes.c_char_p(), ctypes.c_size_t()
            rows, cols, ld, elem = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int32()
            self.check(self.lib.rtvla_buffer_info(self.handle, i, ctypes.byref(name), ctypes.byref(off), ctypes.byref(rows),
                                                  ctypes.byref(cols), ctypes.byref(ld), ctypes.byref(elem)))
            out.append((name.value.decode(), off.value, rows.value, cols.value, ld.value, elem.value))
        return out

    def bind(self, name, ptr, nbytes):
        self.check(self.lib.rtvla_bind(self.handle, name.encode(), _P(ptr), nbytes))

    def workspace_bytes(self):
        return self.lib.rtvla_workspace_bytes(self.handle)

    def bind_workspace(self, ptr, nbytes):
        self.check(self.lib.rtvla_bind_workspace(self.handle, _P(ptr), nbytes))

    def prepare(self, stream, tiles_loaded=False):
        fn = self.lib.rtvla_prepare_with_tiles if tiles_loaded else self.lib.rtvla_prepare
        self.check(fn(self.handle, _P(stream)))

    def tiled_bytes(self):
        return self.lib.rtvla_tiled_bytes(self.handle)

    def forward(self, stream):
        self.check(self.lib.rtvla_forward(self.handle, _P(stream)))

    def forward_stage(self, stage, layer, step, stream):
        self.check(self.lib.rtvla_forward_stage(self.handle, stage, layer, step, _P(stream)))

    def graph_capture(self, stream):
        self.check(self.lib.rtvla_graph_capture(self.handle, _P(stream)))

    def graph_launch(self, stream):
        self.check(self.lib.rtvla_graph_launch(self.handle, _P(stream)))

    def launch_count(self):
        return self.lib.rtvla_launch_count(self.handle)

    def time_stage(self, stage, layer, step, iters, stream):
        ms = ctypes.c_float()
        self.check(self.lib.rtvla_time_stage(self.handle, stage, layer, step, iters, _P(stream), ctypes.byref(ms)))
        return ms.value

    def time_launch(self, stage, layer, step, index, iters, stream):
        """(mean ms, launch name) of the index-th kernel of a stage; None past the end."""
        ms = ctypes.c_float()
        name = ctypes.create_string_buffer(64)
        rc = self.lib.rtvla_time_launch(self.handle, stage, layer, step, index, iters, _P(stream), ctypes.byref(ms), name, 64)
        if rc == 1:
            return None
        self.check(rc)
        return ms.value, name.value.decode()

    def time_forward(self, iters, stream):
        arr = (ctypes.c_float * iters)()
        self.check(self.lib.rtvla_time_forward(self.handle, iters, _P(stream), arr))
        return list(arr)
