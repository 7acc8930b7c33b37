"""The allocation-free image entry point (rtvla_preprocess_image_static) against the workspace-taking one
(rtvla_preprocess_image), through the C ABI: bit-identical outputs on two calls in a row, the second on a smaller
frame, so that whatever the first call left in the library's static intermediate buffer must not leak into the second."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
_P = ctypes.c_void_p


def _frame(seed, h, w):
    return torch.from_numpy(np.random.RandomState(seed).randint(0, 256, size=(h, w, 3)).astype(np.uint8)).to("cuda:0")


def _both(lib, frame):
    h, w, _ = frame.shape
    stream = _P(torch.cuda.current_stream().cuda_stream)
    a = torch.full((224, 224, 3), 5.0, dtype=torch.bfloat16, device="cuda:0")
    b = torch.full((224, 224, 3), -5.0, dtype=torch.bfloat16, device="cuda:0")
    ws = torch.empty(lib.rtvla_preprocess_image_scratch(h, w), dtype=torch.uint8, device="cuda:0")
    assert lib.rtvla_preprocess_image(_P(frame.data_ptr()), h, w, _P(a.data_ptr()), _P(ws.data_ptr()), ws.numel(), stream) == 0
    assert lib.rtvla_preprocess_image_static(_P(frame.data_ptr()), h, w, _P(b.data_ptr()), stream) == 0
    torch.cuda.synchronize()
    return a.cpu(), b.cpu()


def test_static_scratch_entry_point_equals_the_workspace_one_on_consecutive_calls():
    import rtvla_capi as capi
    lib = capi.load()
    for seed, (h, w) in enumerate([(1080, 1920), (240, 320), (720, 1280), (37, 53), (224, 224)]):
        a, b = _both(lib, _frame(seed, h, w))
        assert torch.equal(a, b), "%dx%d: %d elements differ" % (h, w, (a != b).sum().item())
        assert a.float().abs().max() <= 1.0
    # beyond the static buffer: rejected, and the destination is left alone
    tall = _frame(9, 2400, 2400)                     # intermediate 2400 x 224 x 3 bytes > RTVLA_STATIC_SCRATCH_BYTES
    out = torch.full((224, 224, 3), 3.0, dtype=torch.bfloat16, device="cuda:0")
    rc = lib.rtvla_preprocess_image_static(_P(tall.data_ptr()), 2400, 2400, _P(out.data_ptr()), _P(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == capi.ERR_LIMIT and torch.all(out == 3.0)
    # the wrapper's route
    from obs_transforms import ObservationTransforms
    tr = ObservationTransforms("pi0")
    f = _frame(11, 480, 640)
    x = tr.resize_pad_normalize_into(f, torch.empty(224, 224, 3, dtype=torch.bfloat16, device="cuda:0")).clone()
    y = tr.resize_pad_normalize_into(f, torch.empty(224, 224, 3, dtype=torch.bfloat16, device="cuda:0"), static_scratch=True)
    torch.cuda.synchronize()
    assert torch.equal(x, y)
    with pytest.raises(ValueError):
        tr.resize_pad_normalize_into(tall, out, static_scratch=True)


def test_static_scratch_entry_point_inside_a_captured_graph():
    """The advertised use: the call recorded into a HIP graph (nothing may allocate there) and replayed on other frames."""
    import rtvla_capi as capi
    lib = capi.load()
    h, w = 480, 640
    frames = [_frame(20 + i, h, w) for i in range(3)]
    src = frames[0].clone()
    out = torch.zeros(224, 224, 3, dtype=torch.bfloat16, device="cuda:0")
    # one eager call first: it resolves the static array's address on this GPU, which a captured call may not do
    assert lib.rtvla_preprocess_image_static(_P(src.data_ptr()), h, w, _P(out.data_ptr()), _P(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.rtvla_preprocess_image_static(_P(src.data_ptr()), h, w, _P(out.data_ptr()), _P(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    for f in frames[1:] + frames[:1]:
        src.copy_(f)
        out.fill_(7.0)
        torch.cuda.synchronize()                       # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        want, _ = _both(lib, f)
        assert torch.equal(out.cpu(), want)
