"""Pins oracle/transforms.py: the Pillow restatement bit-exactly against Pillow itself, the rest against numpy
routines, closed forms and hand-worked cases.  CPU only."""
import numpy as np
import pytest

from oracle import transforms as T


def _img(seed, h, w, c=3):
    rng = np.random.RandomState(seed)
    base = rng.randint(0, 256, size=(h, w, c)).astype(np.uint8)
    # add structure (gradients, edges) so that a wrong window or weight cannot hide in noise statistics
    yy, xx = np.mgrid[0:h, 0:w]
    base[..., 0] = ((yy * 255) // max(1, h - 1)).astype(np.uint8)
    base[h // 3: h // 2, w // 4: w // 2, 1] = 255
    return base


@pytest.mark.parametrize("h,w,oh,ow", [
    (480, 640, 168, 224),      # 4:3 camera frame shrunk (support > 1: antialiasing path)
    (720, 1280, 126, 224),     # 16:9
    (100, 150, 149, 224),      # enlargement (support = 1)
    (224, 300, 167, 224),      # height already small
    (37, 53, 224, 31),         # odd sizes, one axis up and one down
    (224, 224, 224, 100),      # only the horizontal pass
    (300, 224, 77, 224),       # only the vertical pass
    (2, 3, 5, 7),              # tiny: every window is clamped by both borders
])
def test_resize_matches_pillow_bit_exactly(h, w, oh, ow):
    from PIL import Image
    img = _img(h * 1000 + w, h, w)
    want = np.array(Image.fromarray(img).resize((ow, oh), resample=Image.BILINEAR))
    got = T.pil_bilinear_resize(img, ow, oh)
    assert got.dtype == np.uint8 and got.shape == want.shape
    assert np.array_equal(got, want), "max abs diff %d" % np.abs(got.astype(int) - want.astype(int)).max()


def test_coefficient_tables_have_the_closed_form_properties():
    # the fixed-point weights of every output pixel sum to 1 (within the rounding of each term) and, for an
    # integer shrink factor, are the sampled triangle: a constant image must come out unchanged
    for n_in, n_out in ((640, 224), (224, 640), (448, 224), (7, 3)):
        bounds, coeffs = T.resample_coeffs(n_in, n_out)
        s = coeffs.sum(axis=1)
        assert np.all(np.abs(s - (1 << T.PRECISION_BITS)) <= coeffs.shape[1])
        assert np.all(bounds[:, 0] >= 0) and np.all(bounds[:, 0] + bounds[:, 1] <= n_in)
    const = np.full((50, 70, 3), 173, dtype=np.uint8)
    assert np.all(T.pil_bilinear_resize(const, 31, 22) == 173)
    # shrinking by exactly 2: weights are the triangle (1, 3, 3, 1) / 8 away from the borders
    bounds, coeffs = T.resample_coeffs(448, 224)
    mid = coeffs[100, :4] / float(1 << T.PRECISION_BITS)
    assert np.allclose(mid, [0.125, 0.375, 0.375, 0.125], atol=1e-6) and bounds[100, 0] == 199 and bounds[100, 1] == 4


def test_resize_with_pad_matches_the_reference_recipe_run_with_pillow():
    from PIL import Image
    for h, w in ((480, 640), (640, 480), (224, 224), (100, 100), (1080, 1920), (250, 224)):
        img = _img(h + w, h, w)
        # the recipe of test.py:104-116, written out with Pillow calls
        pil = Image.fromarray(img)
        if (w, h) == (224, 224):
            want = img
        else:
            ratio = max(w / 224, h / 224)
            rh, rw = int(h / ratio), int(w / ratio)
            resized = pil.resize((rw, rh), resample=Image.BILINEAR)
            canvas = Image.new(resized.mode, (224, 224), 0)
            canvas.paste(resized, (max(0, int((224 - rw) / 2)), max(0, int((224 - rh) / 2))))
            want = np.array(canvas)
        got = T.resize_with_pad(img)
        assert got.shape == (224, 224, 3) and np.array_equal(got, want)


def test_parse_and_normalize_image():
    f = np.array([[[0.0, 0.5, 1.0]]], dtype=np.float32)                    # HWC float
    assert T.parse_image(f).tolist() == [[[0, 127, 255]]]                  # truncation, not rounding
    chw = np.zeros((3, 4, 5), dtype=np.uint8)
    assert T.parse_image(chw).shape == (4, 5, 3)
    n = T.normalize_image(np.array([[[0, 255, 128]]], dtype=np.uint8))
    assert n.dtype == np.float32 and n[0, 0, 0] == -1.0 and n[0, 0, 1] == 1.0
    assert n[0, 0, 2] == np.float32(np.float32(128) / np.float32(255.0) * np.float32(2.0) - np.float32(1.0))


def test_state_normalisation_and_digitisation():
    stats = {"mean": [1.0, -2.0], "std": [0.5, 4.0], "q01": [-1.0, 0.0], "q99": [3.0, 10.0]}
    s = np.array([2.0, 2.0])
    z = T.normalize_state(s, stats, "pi0")
    assert z.shape == (32,) and z[0] == (2.0 - 1.0) / (0.5 + 1e-6) and z[1] == (2.0 + 2.0) / (4.0 + 1e-6)
    assert np.all(z[2:] == 0.0)                                           # padded dims: (0 - 0) / (0 + 1e-6)
    q = T.normalize_state(s, stats, "pi05")
    assert q[0] == (2.0 + 1.0) / (4.0 + 1e-6) * 2.0 - 1.0 and q[2] == -1.0
    # digitise: 256 bins of width 2/256 starting at -1; below -1 -> -1, at or above the last edge -> 255
    x = np.array([-1.5, -1.0, -1.0 + 2.0 / 256 - 1e-12, -1.0 + 2.0 / 256, 0.0, 0.999, 1.0, 7.0])
    want = [-1, 0, 0, 1, 128, 255, 255, 255]
    assert T.digitize_state(x).tolist() == want
    # brute force against the definition "number of edges <= x, minus one"
    rng = np.random.RandomState(0)
    y = rng.uniform(-1.2, 1.2, size=2000)
    brute = np.array([(T.DIGITIZE_BINS <= v).sum() - 1 for v in y])
    assert np.array_equal(T.digitize_state(y), brute)


def test_action_postprocessing():
    stats = {"mean": list(range(14)), "std": [2.0] * 14, "q01": [-1.0] * 14, "q99": [1.0] * 14}
    a = np.zeros((3, 32), dtype=np.float32); a[:, :14] = 0.5
    state = np.arange(14, dtype=np.float64) * 10
    out = T.postprocess_actions(a, stats, "pi0", state, 14)
    assert out.shape == (3, 14)
    for d in range(14):
        base = 0.5 * (2.0 + 1e-6) + d
        want = (base + state[d]) - state[d] if d in (6, 13) else base + state[d]   # gripper columns: added, then taken off again
        assert out[1, d] == want
    out5 = T.postprocess_actions(a, stats, "pi05", state, 7)
    assert out5.shape == (3, 7) and out5[0, 0] == 0.75 * (2.0 + 1e-6) + (-1.0) + 0.0
    assert out5[0, 6] == ((0.75 * (2.0 + 1e-6) + (-1.0)) + 60.0) - 60.0
