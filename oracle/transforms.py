"""CPU restatement of the observation pre-/post-processing either side of the forward pass
(/root/reference/test.py:88-201: `_parse_image`, `_resize_with_pad`, `_normalize_image`, `_normalize_state`,
`_digitize_state`, `_unnormalize_actions` and the delta-to-absolute step of `infer`).

TEST INFRASTRUCTURE ONLY, like the rest of this package.

The resize is not the reference's own code: it calls Pillow's `Image.resize(..., resample=Image.BILINEAR)`
(a third-party dependency the reference does not pin; Pillow 12.2.0 is what this image holds).  `pil_bilinear_resize`
restates Pillow's published algorithm (src/libImaging/Resample.c: `precompute_coeffs`, `normalize_coeffs_8bpc`,
`ImagingResampleHorizontal_8bpc`, `ImagingResampleVertical_8bpc`): a triangle filter whose support is stretched by the
scale factor when shrinking, double-precision weights normalised per output pixel, converted to 22-bit fixed point, a
horizontal pass to an 8-bit intermediate and then a vertical pass, each rounding to nearest and clipping to [0, 255].
tests/test_oracle_transforms.py pins it bit-exactly against Pillow itself over up- and down-scaling shapes.
"""
import math

import numpy as np

PRECISION_BITS = 32 - 8 - 2


def resample_coeffs(in_size, out_size):
    """Fixed-point weights and source windows of one axis: (bounds[out_size][2] = (first, count), coeffs[out_size][ksize])."""
    scale = in_size / out_size
    filterscale = scale if scale >= 1.0 else 1.0
    support = 1.0 * filterscale
    ksize = int(math.ceil(support)) * 2 + 1
    bounds = np.zeros((out_size, 2), dtype=np.int64)
    coeffs = np.zeros((out_size, ksize), dtype=np.int64)
    ss = 1.0 / filterscale
    for xx in range(out_size):
        center = 0.0 + (xx + 0.5) * scale
        xmin = int(center - support + 0.5)          # C cast: truncation toward zero
        if xmin < 0:
            xmin = 0
        xmax = int(center + support + 0.5)
        if xmax > in_size:
            xmax = in_size
        xmax -= xmin
        k = [0.0] * ksize
        ww = 0.0
        for x in range(xmax):
            a = abs((x + xmin - center + 0.5) * ss)
            w = 1.0 - a if a < 1.0 else 0.0
            k[x] = w
            ww += w
        for x in range(xmax):
            if ww != 0.0:
                k[x] /= ww
        bounds[xx] = (xmin, xmax)
        for x in range(ksize):
            v = k[x]
            coeffs[xx, x] = int(-0.5 + v * (1 << PRECISION_BITS)) if v < 0 else int(0.5 + v * (1 << PRECISION_BITS))
    return bounds, coeffs


def _resample_axis0(img, out_size):
    """Resample axis 0 of a uint8 array [n, ...] to out_size rows."""
    bounds, coeffs = resample_coeffs(img.shape[0], out_size)
    src = img.astype(np.int64)
    out = np.empty((out_size,) + img.shape[1:], dtype=np.uint8)
    for xx in range(out_size):
        first, count = bounds[xx]
        acc = np.full(img.shape[1:], 1 << (PRECISION_BITS - 1), dtype=np.int64)
        for x in range(count):
            acc += src[first + x] * coeffs[xx, x]
        out[xx] = np.clip(acc >> PRECISION_BITS, 0, 255).astype(np.uint8)
    return out


def pil_bilinear_resize(img, out_w, out_h):
    """uint8 [h, w, c] -> uint8 [out_h, out_w, c], horizontal pass first (skipped when the width is unchanged),
    then the vertical pass (skipped when the height is unchanged), as Pillow does."""
    h, w = img.shape[:2]
    if w != out_w:
        img = np.ascontiguousarray(_resample_axis0(np.swapaxes(img, 0, 1), out_w).swapaxes(0, 1))
    if h != out_h:
        img = _resample_axis0(img, out_h)
    return img


def parse_image(image):
    """test.py:88-94: floats in [0, 1] become uint8 by truncation, CHW becomes HWC."""
    image = np.asarray(image)
    if np.issubdtype(image.dtype, np.floating):
        image = (255 * image).astype(np.uint8)
    if image.shape[0] == 3:
        image = np.transpose(image, (1, 2, 0))
    return image


def resize_geometry(cur_h, cur_w, height=224, width=224):
    """test.py:105-116: (resized_h, resized_w, pad_top, pad_left); an image already at the target size is left alone."""
    if cur_w == width and cur_h == height:
        return height, width, 0, 0
    ratio = max(cur_w / width, cur_h / height)
    resized_h = int(cur_h / ratio)
    resized_w = int(cur_w / ratio)
    pad_h = max(0, int((height - resized_h) / 2))
    pad_w = max(0, int((width - resized_w) / 2))
    return resized_h, resized_w, pad_h, pad_w


def resize_with_pad(image, height=224, width=224):
    """test.py:104-116 on a uint8 HWC image: aspect-preserving bilinear resize pasted centred on a black canvas."""
    cur_h, cur_w = image.shape[:2]
    rh, rw, ph, pw = resize_geometry(cur_h, cur_w, height, width)
    if (rh, rw) == (cur_h, cur_w):
        resized = image
    else:
        resized = pil_bilinear_resize(image, rw, rh)
    out = np.zeros((height, width, image.shape[2]), dtype=np.uint8)
    out[ph:ph + rh, pw:pw + rw] = resized[:height - ph, :width - pw]
    return out


def normalize_image(image):
    """test.py:118-119."""
    return image.astype(np.float32) / 255.0 * 2.0 - 1.0


def pad_to_dim(x, target_dim):
    x = np.asarray(x, dtype=np.float64)
    if x.shape[-1] < target_dim:
        x = np.concatenate([x, np.zeros(x.shape[:-1] + (target_dim - x.shape[-1],))], axis=-1)
    return x


def normalize_state(state, stats, model_version, target_dim=32):
    """test.py:121-134 in float64, as numpy computes it: Pi0 (x - mean) / (std + 1e-6); Pi05 quantile scaling to [-1, 1]."""
    state = pad_to_dim(state, target_dim)
    if model_version == "pi05":
        q01, q99 = pad_to_dim(stats["q01"], target_dim), pad_to_dim(stats["q99"], target_dim)
        return (state - q01) / (q99 - q01 + 1e-6) * 2.0 - 1.0
    mean, std = pad_to_dim(stats["mean"], target_dim), pad_to_dim(stats["std"], target_dim)
    return (state - mean) / (std + 1e-6)


DIGITIZE_BINS = np.linspace(-1, 1, 256 + 1)[:-1]


def digitize_state(state_normed):
    """test.py:136-137: index of the last bin edge <= x, minus nothing for x below -1 gives -1."""
    return np.digitize(state_normed, bins=DIGITIZE_BINS) - 1


def unnormalize_actions(actions, stats, model_version, target_dim=32):
    """test.py:139-151 on float32 actions [chunk, 32] (numpy promotes to float64 through the statistics)."""
    actions = np.asarray(actions, dtype=np.float32)
    if model_version == "pi05":
        q01, q99 = pad_to_dim(stats["q01"], target_dim), pad_to_dim(stats["q99"], target_dim)
        return (actions + 1.0) / 2.0 * (q99 - q01 + 1e-6) + q01
    mean, std = pad_to_dim(stats["mean"], target_dim), pad_to_dim(stats["std"], target_dim)
    return actions * (std + 1e-6) + mean


def postprocess_actions(actions, stats, model_version, ori_state, action_dim):
    """test.py:196-201: un-normalise, keep `action_dim` columns, add the current state (deltas become absolute
    targets) except for every 7th column (the gripper), which stays absolute."""
    a = unnormalize_actions(actions, stats, model_version, 32)[:, :action_dim]
    ori_state = np.asarray(ori_state, dtype=np.float64)
    a[..., :action_dim] = a[..., :action_dim] + ori_state[..., :action_dim]
    for i in range(action_dim // 7):
        a[..., (i + 1) * 7 - 1] = a[..., (i + 1) * 7 - 1] - ori_state[..., (i + 1) * 7 - 1]
    return a
