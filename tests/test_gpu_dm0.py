"""GPU parity of the DM0 path (through the C ABI) against the CPU oracle (oracle/dm0.py, pinned in
tests/test_oracle_dm0.py).  Same tolerances as the Pi0 / Pi05 tests: action MAE <= 1e-2, layer-local relative L2 <= 2e-2
with every layer fed the oracle's input, free-running drift bounded by 1.5 x the oracle's own bf16-vs-fp32 drift."""
import pytest
import torch

import synthetic as syn

pytestmark = pytest.mark.gpu
MAE_TOL, LAYER_TOL, DRIFT_FACTOR, DRIFT_FLOOR = 1e-2, 2e-2, 1.5, 1e-2


def rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).norm() / (b.norm() + 1e-30)).item()


def bf(x):
    return x.to(torch.bfloat16).to("cuda")


class Case:
    def __init__(self, seed, n_img, lang, vision_layers, llm_layers, vocab=300, fp32_taps=True):
        import rtvla_capi as capi
        from oracle import dm0 as o, ops
        from dm0_infer import DM0Inference
        self.capi, self.o, self.ops = capi, o, ops
        self.n, self.VL, self.LL = n_img, vision_layers, llm_layers
        self.ck = syn.dm0_checkpoint(seed, "cuda:0", vision_layers, llm_layers, vocab=vocab)
        self.img, self.ids, self.noise = syn.dm0_observation(seed, n_img, "cuda:0", max_lang_len=lang, vocab=vocab)
        self.m = DM0Inference(self.ck, num_images=n_img, max_lang_len=lang)
        self.P = self.m.prefix_len
        self.ckc = {k: v.cpu() for k, v in self.ck.items()}
        self.taps, self.taps32 = {}, {}
        self.ref = o.forward(self.ckc, self.img.cpu(), self.ids.cpu(), self.noise.cpu(), taps=self.taps)
        if fp32_taps:
            o.forward(self.ckc, self.img.cpu(), self.ids.cpu(), self.noise.cpu(), bf16_boundaries=False, taps=self.taps32)
        self.e, self.B = self.m._engine, self.m.buffers
        self.kp = self.B["kv_K"].shape[1] // 128

    def stage_inputs(self):
        self.B["images"].copy_(self.img); self.B["input_ids"].copy_(self.ids); self.B["diffusion_noise"].copy_(self.noise)

    def run(self, stage, layer=0, step=0):
        self.e.run_stage(stage, layer, step)
        torch.cuda.synchronize()

    def vit(self, name):
        """The valid rows of a row-major ViT buffer (every image owns 2720 rows, 2705 of them tokens)."""
        b = self.B[name]
        return b.view(self.n, 2720, b.shape[1])[:, :2705].reshape(self.n * 2705, b.shape[1])

    def set_vit(self, name, x):
        b = self.B[name]
        b.view(self.n, 2720, b.shape[1])[:, :2705].copy_(bf(x).view(self.n, 2705, b.shape[1]))

    def dec_x(self):
        from _engine import untile_ft
        return untile_ft(self.B["decoder_x"], 64, 1024)[:50]

    def set_dec_x(self, x):
        from _engine import tile_ft
        full = torch.zeros(64, 1024, dtype=torch.bfloat16, device="cuda")
        full[:50] = bf(x)
        self.B["decoder_x"].reshape(-1).copy_(tile_ft(full))

    def cache(self, i):
        """K, V of layer i as [keys_pad, 8, 128]."""
        from _engine import untile_ft, untile_vt
        K = torch.stack([untile_ft(self.B["kv_K"][i * 8 + h], self.kp, 128) for h in range(8)], dim=1)
        V = torch.stack([untile_vt(self.B["kv_Vt"][i * 8 + h], 128, self.kp).t() for h in range(8)], dim=1)
        return K, V

    def set_cache_prefix(self, i, k, v):
        from _engine import tile_ft, tile_vt
        K, V = self.cache(i)
        K = K.clone(); V = V.clone()
        K[: self.P] = bf(k); V[: self.P] = bf(v)
        for h in range(8):
            self.B["kv_K"][i * 8 + h].copy_(tile_ft(K[:, h].contiguous()))
            self.B["kv_Vt"][i * 8 + h].copy_(tile_vt(V[:, h].t().contiguous()))

    def free_running(self):
        c, t, t32 = self.capi, self.taps, self.taps32
        self.stage_inputs()
        drift, odrift = {}, {}

        def note(name, got, tap, rows=None):
            a = t[tap]
            if rows is not None:
                got, a = got[:rows], a[:rows]
            drift[name] = rel(got, a.reshape(got.shape))
            if t32:
                b = t32[tap][:rows] if rows is not None else t32[tap]
                odrift[name] = rel(a, b)
        self.run(c.STAGE_VISION_EMBED)
        note("vision_embed", self.vit("vision_x_2d"), "vision_embed")
        for i in range(self.VL):
            self.run(c.STAGE_VISION_LAYER, i)
            note("vision_x/%d" % i, self.vit("vision_x_2d"), "vision_x/%d" % i)
        self.run(c.STAGE_PROJECT)
        note("prefix_x0", self.B["prefix_x"], "prefix_x0")
        for i in range(self.LL):
            self.run(c.STAGE_PREFIX_LAYER, i)
            if i < self.LL - 1:                      # the last prefix layer only fills the K / V cache: nothing reads its output stream
                note("prefix_x/%d" % i, self.B["prefix_x"], "prefix_x/%d" % i)
            K, V = self.cache(i)
            note("prefix_K/%d" % i, K, "prefix_K/%d" % i, self.P)
            note("prefix_V/%d" % i, V, "prefix_V/%d" % i, self.P)
        for s in range(10):
            self.run(c.STAGE_SUFFIX_STEP_BEGIN, 0, s)
            for i in range(self.LL):
                self.run(c.STAGE_SUFFIX_LAYER, i, s)
            note("decoder_x/%d" % s, self.dec_x(), "decoder_x/%d/%d" % (s, self.LL - 1))
            self.run(c.STAGE_SUFFIX_STEP_END, 0, s)
            note("noise/%d" % s, self.B["diffusion_noise"], "noise/%d" % s)
        return drift, odrift, self.B["diffusion_noise"].float().cpu().clone()

    def teacher_forced(self, steps=(0, 9)):
        c, t, o, ops, w = self.capi, self.taps, self.o, self.ops, self.ckc
        errs = {}
        self.stage_inputs()
        self.run(c.STAGE_VISION_EMBED)
        errs["vision_embed"] = rel(self.vit("vision_x_2d"), t["vision_embed"])
        for i in range(self.VL):
            x = t["vision_embed"] if i == 0 else t["vision_x/%d" % (i - 1)]
            mean, rstd = o.ln_stats(x)
            self.set_vit("vision_x_2d", x); self.set_vit("vision_x_norm", (x - mean) * rstd)
            self.run(c.STAGE_VISION_LAYER, i)
            errs["vision_layer/%d" % i] = rel(self.vit("vision_x_2d"), t["vision_x/%d" % i])
        self.set_vit("vision_x_2d", t["vision_x/%d" % (self.VL - 1)])
        self.run(c.STAGE_PROJECT)
        errs["project"] = rel(self.B["prefix_x"], t["prefix_x0"])
        for i in range(self.LL):
            x = t["prefix_x0"] if i == 0 else t["prefix_x/%d" % (i - 1)]
            self.B["prefix_x"].copy_(bf(x)); self.B["prefix_norm_factor"].reshape(-1).copy_(ops.rms_factor(x)[:, 0].to("cuda"))
            self.run(c.STAGE_PREFIX_LAYER, i)
            K, V = self.cache(i)
            errs["prefix_K/%d" % i] = rel(K[: self.P], t["prefix_K/%d" % i])
            errs["prefix_V/%d" % i] = rel(V[: self.P], t["prefix_V/%d" % i])
            if i < self.LL - 1:
                errs["prefix_layer/%d" % i] = rel(self.B["prefix_x"], t["prefix_x/%d" % i])
        for i in range(self.LL):
            self.set_cache_prefix(i, t["prefix_K/%d" % i], t["prefix_V/%d" % i])
        for s in steps:
            noise_in = self.noise.float().cpu() if s == 0 else t["noise/%d" % (s - 1)]
            self.B["diffusion_noise"].copy_(bf(noise_in))
            self.run(c.STAGE_SUFFIX_STEP_BEGIN, 0, s)
            errs["suffix_in/%d" % s] = rel(self.dec_x(), t["decoder_in/%d" % s])
            for i in range(self.LL):
                self.set_dec_x(t["decoder_in/%d" % s] if i == 0 else t["decoder_x/%d/%d" % (s, i - 1)])
                self.run(c.STAGE_SUFFIX_LAYER, i, s)
                errs["suffix_layer/%d/%d" % (s, i)] = rel(self.dec_x(), t["decoder_x/%d/%d" % (s, i)])
            self.set_dec_x(t["decoder_x/%d/%d" % (s, self.LL - 1)])
            self.B["diffusion_noise"].copy_(bf(noise_in))
            self.run(c.STAGE_SUFFIX_STEP_END, 0, s)
            errs["euler/%d" % s] = (self.B["diffusion_noise"].float().cpu() - t["noise/%d" % s]).abs().mean().item()
        return errs


def check_case(case, tag):
    drift, odrift, staged = case.free_running()
    mae = (staged - case.ref).abs().mean().item()
    worst = max(drift, key=drift.get)
    print("\n[%s] free-running: action MAE %.5f, largest cumulative rel-L2 %.4f at %s" % (tag, mae, drift[worst], worst))
    assert torch.isfinite(staged).all() and mae <= MAE_TOL
    if odrift:
        bound = {k: max(DRIFT_FACTOR * odrift[k], DRIFT_FLOOR) for k in drift}
        tight = max(drift, key=lambda k: drift[k] / bound[k])
        print("[%s] closest to its drift bound: %s at %.2f of it" % (tag, tight, drift[tight] / bound[tight]))
        assert drift[tight] <= bound[tight], (tight, drift[tight], bound[tight])
    out = case.m.forward(case.img, case.ids, case.noise).float().cpu()
    assert torch.equal(out, staged), "graph replay differs from the staged eager run"
    assert torch.equal(case.m.forward(case.img, case.ids, case.noise).float().cpu(), out), "two replays differ"
    errs = case.teacher_forced()
    layer = {k: v for k, v in errs.items() if not k.startswith("euler")}
    worst = max(layer, key=layer.get)
    print("[%s] teacher-forced: worst layer-local rel-L2 %.5f at %s; Euler MAE %.5f" % (tag, layer[worst], worst, max(v for k, v in errs.items() if k.startswith("euler"))))
    assert layer[worst] <= LAYER_TOL, (worst, layer[worst])
    assert all(v <= MAE_TOL for k, v in errs.items() if k.startswith("euler"))


def test_dm0_reduced_depth_staged_and_graph():
    check_case(Case(61, 1, 6, 2, 2), "dm0_small")


def test_dm0_two_images_odd_prompt():
    check_case(Case(62, 2, 37, 1, 2), "dm0_2img")


def test_dm0_full_size_three_images():
    """The reference benchmark's shape: 3 images, 100 language tokens, 23 + 28 + 28 layers (benchmark.py:61-62)."""
    case = Case(1234, 3, 100, 23, 28, vocab=4096, fp32_taps=False)
    case.stage_inputs()
    out = case.m.forward(case.img, case.ids, case.noise).float().cpu()
    mae = (out - case.ref).abs().mean().item()
    print("\n[dm0 full] action MAE vs oracle %.5f" % mae)
    assert torch.isfinite(out).all() and mae <= MAE_TOL
    assert torch.equal(case.m.forward(case.img, case.ids, case.noise).float().cpu(), out)


def test_dm0_contract():
    from dm0_infer import DM0Inference
    ck = syn.dm0_checkpoint(63, "cuda:0", 1, 1, vocab=64)
    img, ids, noise = syn.dm0_observation(63, 1, "cuda:0", max_lang_len=4, vocab=64)
    m = DM0Inference({k: v.cpu() for k, v in ck.items()}, num_images=1, max_lang_len=4)
    a = m.forward(img, ids, noise).clone()
    b = m.forward(img.float().cpu(), ids.cpu(), noise.float())               # other dtypes / devices are converted by copy_
    assert b.dtype == torch.bfloat16 and b.shape == (50, 32) and b.is_cuda and torch.equal(a, b)
    assert b.data_ptr() == m.buffers["diffusion_noise"].data_ptr()
    assert m.prefix_len == 169 + 4 and m.total_keys == 169 + 4 + 50 and m.chunk_size == 50
    with pytest.raises(KeyError):
        DM0Inference(dict(ck, not_a_weight=torch.zeros(1)), num_images=1, max_lang_len=4)
