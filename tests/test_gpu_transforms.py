"""GPU parity of the observation pre-/post-processing kernels against oracle/transforms.py (itself pinned against
Pillow and numpy in tests/test_oracle_transforms.py).  Bit-exact: integer images, IEEE double statistics."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _img(seed, h, w):
    rng = np.random.RandomState(seed)
    img = rng.randint(0, 256, size=(h, w, 3)).astype(np.uint8)
    yy, xx = np.mgrid[0:h, 0:w]
    img[..., 0] = ((xx * 255) // max(1, w - 1)).astype(np.uint8)
    img[h // 4: h // 2, w // 3: w // 2, 2] = 255
    return img


@pytest.mark.parametrize("h,w", [(480, 640), (720, 1280), (224, 224), (100, 150), (640, 480), (250, 224), (224, 300), (37, 53), (1080, 1920)])
def test_image_preprocessing_matches_the_pillow_restatement_bit_exactly(h, w):
    from oracle import transforms as T
    from obs_transforms import ObservationTransforms
    tr = ObservationTransforms("pi0")
    img = _img(h * 7 + w, h, w)
    want = torch.from_numpy(T.normalize_image(T.resize_with_pad(img))).to(torch.bfloat16)
    out = torch.full((224, 224, 3), 7.0, dtype=torch.bfloat16, device="cuda:0")
    tr.resize_pad_normalize_into(img, out)
    torch.cuda.synchronize()
    got = out.cpu()
    assert torch.equal(got, want), "mismatching elements: %d" % (got != want).sum().item()


def test_image_inputs_float_and_chw_and_errors():
    from oracle import transforms as T
    from obs_transforms import ObservationTransforms
    tr = ObservationTransforms("pi05")
    rng = np.random.RandomState(3)
    f = rng.rand(3, 120, 90).astype(np.float32)                          # CHW float in [0, 1]
    want = torch.from_numpy(T.normalize_image(T.resize_with_pad(T.parse_image(f)))).to(torch.bfloat16)
    out = torch.empty(224, 224, 3, dtype=torch.bfloat16, device="cuda:0")
    tr.resize_pad_normalize_into(f, out)
    assert torch.equal(out.cpu(), want)
    with pytest.raises(ValueError):
        tr.resize_pad_normalize_into(np.zeros((10, 10, 4), dtype=np.uint8), out)
    with pytest.raises(ValueError):
        tr.resize_pad_normalize_into(np.zeros((10, 10, 3), dtype=np.uint8), torch.empty(224, 224, 3, device="cuda:0"))
    with pytest.raises(RuntimeError):                                    # shrink factor above the supported 31
        tr.resize_pad_normalize_into(np.zeros((8000, 16, 3), dtype=np.uint8), out)


@pytest.mark.parametrize("version", ["pi0", "pi05"])
def test_state_and_action_transforms_match_numpy_bit_exactly(version):
    from oracle import transforms as T
    from obs_transforms import ObservationTransforms
    rng = np.random.RandomState(11)
    n = 14
    stats = {"state": {"mean": rng.randn(n).tolist(), "std": (rng.rand(n) + 0.1).tolist(),
                       "q01": (-1 - rng.rand(n)).tolist(), "q99": (1 + rng.rand(n)).tolist()},
             "actions": {"mean": rng.randn(n).tolist(), "std": (rng.rand(n) + 0.1).tolist(),
                         "q01": (-1 - rng.rand(n)).tolist(), "q99": (1 + rng.rand(n)).tolist()}}
    tr = ObservationTransforms(version, stats, state_len=n, action_dim=n)
    state = rng.randn(n) * 1.5
    state[0] = stats["state"]["q01"][0] - 3.0                            # far below the first bin edge
    state[1] = stats["state"]["q99"][1] + 3.0                            # far above the last one
    want = T.normalize_state(state, stats["state"], version)
    buf = torch.zeros(32, dtype=torch.bfloat16, device="cuda:0")
    z, bins = tr._normalize_state(state, want_bins=True, out_bf16=buf)
    torch.cuda.synchronize()
    assert np.array_equal(z.cpu().numpy(), want)
    assert torch.equal(buf.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))
    assert np.array_equal(bins.cpu().numpy(), T.digitize_state(want))
    edges = torch.tensor(T.DIGITIZE_BINS)                                # values exactly on bin edges
    a_stats = {"mean": [0.0] * 32, "std": [1.0 - 1e-6] * 32, "q01": [-1.0] * 32, "q99": [1.0 - 1e-6] * 32}
    tr2 = ObservationTransforms(version, {"state": a_stats}, state_len=32)
    for chunk in edges.split(32):
        zz, bb = tr2._normalize_state(chunk.numpy(), want_bins=True)
        assert np.array_equal(bb.cpu().numpy(), T.digitize_state(zz.cpu().numpy()))
    actions = torch.from_numpy(rng.randn(50, 32).astype(np.float32)).to(torch.bfloat16).cuda()
    got = tr.postprocess_actions(actions, state)
    ref = T.postprocess_actions(actions.cpu().float().numpy(), stats["actions"], version, state, n)
    assert got.shape == (50, n) and np.array_equal(got.cpu().numpy(), ref)
    tr7 = ObservationTransforms(version, stats, state_len=n, action_dim=7)
    assert np.array_equal(tr7.postprocess_actions(actions, state).cpu().numpy(),
                          T.postprocess_actions(actions.cpu().float().numpy(), stats["actions"], version, state, 7))


def test_whole_observation_through_the_policy():
    """infer(): camera frames + raw state -> actions, against the oracle transforms wrapped around the same policy."""
    import synthetic as syn
    from oracle import transforms as T
    from obs_transforms import ObservationTransforms
    from pi0_infer import Pi0Inference
    rng = np.random.RandomState(5)
    ck = syn.pi0_checkpoint(31, 2, "cuda:0", 1, 2)
    policy = Pi0Inference(ck, 2, 10)
    stats = {"state": {"mean": rng.randn(7).tolist(), "std": (rng.rand(7) + 0.5).tolist()},
             "actions": {"mean": rng.randn(7).tolist(), "std": (rng.rand(7) + 0.5).tolist()}}
    tr = ObservationTransforms("pi0", stats, state_len=7, action_dim=7)
    frames = {"base_0_rgb": _img(1, 480, 640), "left_wrist_0_rgb": _img(2, 360, 360), "right_wrist_0_rgb": _img(3, 10, 10)}
    state = rng.randn(7)
    noise = rng.randn(10, 32).astype(np.float32)
    out = tr.infer(policy, dict(frames, state=state), noise)["actions"]
    imgs = torch.stack([torch.from_numpy(T.normalize_image(T.resize_with_pad(frames[k]))) for k in ("base_0_rgb", "left_wrist_0_rgb")])
    st = torch.from_numpy(T.normalize_state(state, stats["state"], "pi0").astype(np.float32))
    ref_actions = policy.forward(imgs, st, torch.from_numpy(noise)).cpu().float().numpy()
    ref = T.postprocess_actions(ref_actions, stats["actions"], "pi0", state, 7)
    assert out.shape == (10, 7) and np.array_equal(out, ref)
