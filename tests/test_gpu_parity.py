"""GPU parity: the HIP path (through the C ABI) against the CPU oracle and the golden fixtures.

Tolerances are the ones the task states for this floating-point path: action MAE <= 1e-2 against
the bf16-boundary oracle, per-layer relative L2 <= 2e-2.  "Per layer" is measured layer-locally:
each stage is fed the oracle's input for that layer (teacher forcing) so that the bf16 drift two
independent pipelines accumulate over 45 layers is not charged to any single kernel.  The
free-running cumulative drift is bounded as well: at every tap it may not exceed DRIFT_FACTOR times
the drift between the oracle's own bf16-boundary and all-fp32 variants at that tap (two bf16
pipelines that round at different places differ from each other by about sqrt(2) times what each
differs from exact arithmetic), with DRIFT_FLOOR for taps where that figure is a single rounding.

The golden files are written by the oracle itself (tests/golden/make_golden.py): they guard against
the oracle drifting, they are not an independent anchor.  The oracle's independent pins are
tests/test_oracle_ops.py and tests/test_oracle_layers.py.  Except for the BASELINE configurations
C1-C4 (which specify LayerNorm weights of 1), every case here uses random LayerNorm weights and
biases that differ per layer.
"""
import os

import pytest
import torch

import synthetic as syn

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
MAE_TOL = 1e-2
LAYER_TOL = 2e-2
DRIFT_FACTOR = 1.5
DRIFT_FLOOR = 1e-2


def rel(a, b):
    a, b = a.float().cpu(), b.float().cpu()
    return ((a - b).norm() / (b.norm() + 1e-30)).item()


def bf(x, dev="cuda"):
    return x.to(torch.bfloat16).to(dev)


class Case:
    """One model instance + its oracle run with taps."""

    def __init__(self, model, seed, views, prompt, chunk, vision_layers=27, llm_layers=18, state_tokens=0, max_prompt=None,
                 norms="random"):
        import rtvla_capi as capi
        from oracle import pi0 as o0, pi05 as o5, ops
        self.capi, self.ops = capi, ops
        self.model_name, self.views, self.chunk = model, views, chunk
        self.VL, self.LL = vision_layers, llm_layers
        dev = "cuda:0"
        if model == "pi0":
            from pi0_infer import Pi0Inference
            self.ck = syn.pi0_checkpoint(seed, prompt, dev, vision_layers, llm_layers, norms=norms)
            self.img, self.state, self.noise = syn.observation(seed, views, chunk, dev)
            self.m = Pi0Inference(self.ck, views, chunk)
            self.S_e = 256 * views + prompt
            self.S_d = chunk + 1
            self.valid = self.S_e
        else:
            from pi05_infer import Pi05Inference
            self.ck = syn.pi05_checkpoint(seed, prompt, dev, vision_layers, llm_layers, state_tokens=state_tokens, norms=norms)
            self.img, self.state, self.noise = syn.observation(seed, views, chunk, dev)
            plen = prompt + state_tokens
            if max_prompt is not None and max_prompt != plen:
                # allocate a longer prefix than the prompt: pad the checkpoint's prompt, then shorten it per call
                pad = torch.zeros(max_prompt - plen, 2048, dtype=torch.bfloat16, device=dev)
                ck2 = dict(self.ck); ck2["language_embeds"] = torch.cat([self.ck["language_embeds"], pad])
                self.m = Pi05Inference(ck2, views, chunk, discrete_state_input=False)
                self.m.weights["language_embeds"] = self.ck["language_embeds"].clone()
            else:
                self.m = Pi05Inference(self.ck, views, chunk, discrete_state_input=False)
            self.S_e = 256 * views + (max_prompt if max_prompt is not None else plen)
            self.S_d = chunk
            self.valid = 256 * views + plen
        self.ckc = {k: v.cpu() for k, v in self.ck.items()}
        self.taps, self.taps32 = {}, {}
        if model == "pi0":
            self.ref = o0.forward(self.ckc, self.img.cpu(), self.state.cpu(), self.noise.cpu(), taps=self.taps)
            o0.forward(self.ckc, self.img.cpu(), self.state.cpu(), self.noise.cpu(), bf16_boundaries=False, taps=self.taps32)
        else:
            self.ref = o5.forward(self.ckc, self.img.cpu(), self.noise.cpu(), max_prompt_len=max_prompt, taps=self.taps)
            o5.forward(self.ckc, self.img.cpu(), self.noise.cpu(), max_prompt_len=max_prompt, bf16_boundaries=False, taps=self.taps32)
        self.e, self.B = self.m._engine, self.m.buffers
        self.keys_pad = self.B["encoder_Vt"].shape[1]

    # ---- input staging (what forward() does before the replay) ----
    def stage_inputs(self):
        if self.model_name == "pi0":
            self.B["observation_images_normalized"].copy_(self.img)
            self.B["observation_state_normalized"].copy_(self.state)
            self.B["diffusion_noise"].copy_(self.noise)
        else:
            self.m.stage_inputs(self.img, self.noise)

    def forward(self):
        if self.model_name == "pi0":
            return self.m.forward(self.img, self.state, self.noise)
        return self.m.forward(self.img, self.noise)

    def run(self, stage, layer=0, step=0):
        self.e.run_stage(stage, layer, step)
        torch.cuda.synchronize()

    # ---- buffer access in the library's layouts ----
    def dec_x(self):
        from _engine import untile_ft
        return untile_ft(self.B["decoder_x"], self.B["decoder_x"].numel() // 1024, 1024)[: self.S_d]

    def set_dec_x(self, x):
        from _engine import tile_ft
        full = torch.zeros(self.B["decoder_x"].numel() // 1024, 1024, dtype=torch.bfloat16, device="cuda")
        full[: self.S_d] = bf(x)
        self.B["decoder_x"].reshape(-1).copy_(tile_ft(full))

    def cache(self, i):
        from _engine import untile_ft, untile_vt
        K = untile_ft(self.B["encoder_K"].reshape(self.LL, -1)[i], self.keys_pad, 256)
        V = untile_vt(self.B["encoder_Vt"].reshape(self.LL, -1)[i], 256, self.keys_pad).t()
        return K, V

    def set_cache_prefix(self, i, k, v):
        from _engine import tile_ft, tile_vt
        K, V = self.cache(i)
        K = K.clone(); V = V.clone()
        K[: self.S_e] = bf(k); V[: self.S_e] = bf(v)
        self.B["encoder_K"].reshape(self.LL, -1)[i].copy_(tile_ft(K))
        self.B["encoder_Vt"].reshape(self.LL, -1)[i].copy_(tile_vt(V.t().contiguous()))

    # ---- the checks ----
    def free_running(self):
        """Whole forward stage by stage; returns the drift per tap and the final MAE."""
        c, t, t32 = self.capi, self.taps, self.taps32
        self.stage_inputs()
        drift, self.oracle_drift = {}, {}

        def note(name, got, tap, rows=None):
            a, b = t[tap], t32[tap]
            if rows is not None:
                got, a, b = got[:rows], a[:rows], b[:rows]
            drift[name] = rel(got, a)
            self.oracle_drift[name] = rel(a, b)
        self.run(c.STAGE_VISION_EMBED)
        note("vision_embed", self.B["vision_x"], "vision_embed")
        for i in range(self.VL):
            self.run(c.STAGE_VISION_LAYER, i)
            note("vision_x/%d" % i, self.B["vision_x"], "vision_x/%d" % i)
        self.run(c.STAGE_PROJECT)
        note("encoder_x0", self.B["encoder_x"], "encoder_x0", self.valid)
        for i in range(self.LL):
            self.run(c.STAGE_PREFIX_LAYER, i)
            K, V = self.cache(i)
            note("encoder_K/%d" % i, K, "encoder_K/%d" % i, self.valid)
            note("encoder_V/%d" % i, V, "encoder_V/%d" % i, self.valid)
        self.run(c.STAGE_SUFFIX_INIT)
        for s in range(10):
            self.run(c.STAGE_SUFFIX_STEP_BEGIN, 0, s)
            for i in range(self.LL):
                self.run(c.STAGE_SUFFIX_LAYER, i, s)
            note("decoder_x/%d" % s, self.dec_x(), "decoder_x/%d/%d" % (s, self.LL - 1))
            self.run(c.STAGE_SUFFIX_STEP_END, 0, s)
            note("noise/%d" % s, self.B["diffusion_noise"], "noise/%d" % s)
        out = self.B["diffusion_noise"].float().cpu().clone()
        return drift, out

    def teacher_forced(self, steps=(0, 9)):
        """Every layer fed the oracle's input; returns the layer-local relative L2 per layer."""
        c, t, ops, w = self.capi, self.taps, self.ops, self.ckc
        errs = {}
        self.stage_inputs()
        self.run(c.STAGE_VISION_EMBED)
        errs["vision_embed"] = rel(self.B["vision_x"], t["vision_embed"])
        for i in range(self.VL):
            x = t["vision_embed"] if i == 0 else t["vision_x/%d" % (i - 1)]
            self.B["vision_x"].copy_(bf(x))
            self.B["vision_x_norm"].copy_(bf(ops.layer_norm(x, w["vision_pre_attn_norm_w"][i], w["vision_pre_attn_norm_b"][i])))
            self.run(c.STAGE_VISION_LAYER, i)
            errs["vision_layer/%d" % i] = rel(self.B["vision_x"], t["vision_x/%d" % i])
        x = t["vision_x/%d" % (self.VL - 1)]
        self.B["vision_x_norm"].copy_(bf(ops.layer_norm(x, w["vision_final_norm_w"], w["vision_final_norm_b"])))
        self.run(c.STAGE_PROJECT)
        errs["project"] = rel(self.B["encoder_x"][: self.valid], t["encoder_x0"][: self.valid])
        for i in range(self.LL):
            x = t["encoder_x0"] if i == 0 else t["encoder_x/%d" % (i - 1)]
            self.B["encoder_x"].copy_(bf(x))
            self.B["encoder_x_norm"].copy_(bf(x * ops.rms_factor(x)))
            self.run(c.STAGE_PREFIX_LAYER, i)
            K, V = self.cache(i)
            errs["prefix_K/%d" % i] = rel(K[: self.valid], t["encoder_K/%d" % i][: self.valid])
            errs["prefix_V/%d" % i] = rel(V[: self.valid], t["encoder_V/%d" % i][: self.valid])
            if i != self.LL - 1:
                errs["prefix_layer/%d" % i] = rel(self.B["encoder_x"][: self.valid], t["encoder_x/%d" % i][: self.valid])
        for i in range(self.LL):
            self.set_cache_prefix(i, t["encoder_K/%d" % i], t["encoder_V/%d" % i])
        self.run(c.STAGE_SUFFIX_INIT)
        for s in steps:
            noise_in = self.noise.float().cpu() if s == 0 else t["noise/%d" % (s - 1)]
            self.B["diffusion_noise"].copy_(bf(noise_in))
            self.run(c.STAGE_SUFFIX_STEP_BEGIN, 0, s)
            errs["suffix_in/%d" % s] = rel(self.dec_x(), t["decoder_in/%d" % s])
            for i in range(self.LL):
                x = t["decoder_in/%d" % s] if i == 0 else t["decoder_x/%d/%d" % (s, i - 1)]
                self.set_dec_x(x)
                self.run(c.STAGE_SUFFIX_LAYER, i, s)
                errs["suffix_layer/%d/%d" % (s, i)] = rel(self.dec_x(), t["decoder_x/%d/%d" % (s, i)])
            self.set_dec_x(t["decoder_x/%d/%d" % (s, self.LL - 1)])
            self.B["diffusion_noise"].copy_(bf(noise_in))
            self.run(c.STAGE_SUFFIX_STEP_END, 0, s)
            errs["euler/%d" % s] = (self.B["diffusion_noise"].float().cpu() - t["noise/%d" % s]).abs().mean().item()
        return errs


def check_case(case, gold_key=None, gold_file="golden_small.pt"):
    drift, staged = case.free_running()
    mae = (staged - case.ref).abs().mean().item()
    worst = max(drift, key=drift.get)
    bound = {k: max(DRIFT_FACTOR * case.oracle_drift[k], DRIFT_FLOOR) for k in drift}
    tight = max(drift, key=lambda k: drift[k] / bound[k])
    print("\n[%s] free-running: action MAE %.5f, largest cumulative rel-L2 %.4f at %s (oracle bf16 vs fp32 there: %.4f); "
          "closest to its bound: %s at %.2f of it" % (gold_key, mae, drift[worst], worst, case.oracle_drift[worst], tight, drift[tight] / bound[tight]))
    if os.environ.get("RTVLA_PRINT_DRIFT"):            # the whole table (pytest -s), e.g. for profiles/free_running_drift_*.md
        print("| tap | HIP vs bf16-boundary oracle, rel-L2 | oracle bf16 vs fp32, rel-L2 | bound |\n|---|---|---|---|")
        for k in drift:
            print("| %s | %.5f | %.5f | %.5f |" % (k, drift[k], case.oracle_drift[k], bound[k]))
    assert torch.isfinite(staged).all()
    assert mae <= MAE_TOL
    assert drift[tight] <= bound[tight], (tight, drift[tight], bound[tight])
    per_dim = (staged - case.ref).abs().mean(0)
    assert per_dim.max().item() <= 3 * MAE_TOL          # per-dimension MAE, the second statistic of test.py:282-287
    out = case.forward().float().cpu()                    # the captured graph, same inputs
    assert torch.equal(out, staged), "graph replay differs from the staged eager run"
    assert torch.equal(case.forward().float().cpu(), out), "two replays differ"
    if gold_key:
        g = torch.load(os.path.join(GOLD, gold_file), weights_only=True)
        assert (out - g[gold_key + "/actions"].float()).abs().mean().item() <= MAE_TOL
        assert (out - g[gold_key + "/actions_fp32"]).abs().mean().item() <= MAE_TOL
        # the oracle re-run on this host's CPU agrees with the committed vector up to the BLAS summation order
        assert (case.ref - g[gold_key + "/actions"].float()).abs().mean().item() <= 0.5 * MAE_TOL
    errs = case.teacher_forced()
    layer = {k: v for k, v in errs.items() if not k.startswith("euler")}
    worst = max(layer, key=layer.get)
    print("[%s] teacher-forced: worst layer-local rel-L2 %.5f at %s; Euler MAE %.5f" %
          (gold_key, layer[worst], worst, max(v for k, v in errs.items() if k.startswith("euler"))))
    assert layer[worst] <= LAYER_TOL, (worst, layer[worst])
    assert all(v <= MAE_TOL for k, v in errs.items() if k.startswith("euler"))
    return mae


def test_pi0_reduced_depth_staged_and_graph():
    check_case(Case("pi0", 7, 1, 4, 10, 2, 2), "pi0_small")


def test_pi0_empty_prompt_max_chunk():
    check_case(Case("pi0", 8, 1, 0, 63, 1, 2), "pi0_small_noprompt_c63")


def test_pi05_reduced_depth_with_padded_prefix():
    check_case(Case("pi05", 9, 1, 4, 10, 2, 2, state_tokens=3, max_prompt=12), "pi05_small")


def test_pi0_two_views_ragged_prefix():
    check_case(Case("pi0", 21, 2, 7, 17, 1, 2))


@pytest.mark.parametrize("model,views,prompt,chunk,state_tokens", [
    ("pi0", 1, 1, 1, 0),        # one action row, one prompt token: 258 prefix rows, 2 suffix rows
    ("pi0", 3, 37, 33, 0),      # odd everything: 805 prefix rows (GEMM row tiles with a ragged tail), 34 suffix rows
    ("pi0", 2, 200, 50, 0),     # long prompt on two views: 712 prefix rows, 763 keys (6 key splits)
    ("pi05", 2, 5, 64, 9),      # Pi05 with exactly one 64-row block of the action-expert kernels
    ("pi0", 1, 3, 100, 0),      # 101 suffix rows: two 64-row blocks, 51 attention row blocks
    ("pi05", 1, 5, 128, 4),     # Pi05 at the 128-row limit
    ("pi0", 1, 2000, 20, 0),    # 2277 keys: more than four 32-key blocks per key split, i.e. the suffix pass on the general attention kernel
    ("pi05", 3, 100, 7, 0),     # Pi05, long prompt, short chunk
])
def test_shape_sweep_against_the_oracle(model, views, prompt, chunk, state_tokens):
    """Shapes between and beyond the BASELINE configurations at reduced depth: every tile choice, split count and
    ragged tail they select must still agree with the oracle (and replay must equal the eager run)."""
    check_case(Case(model, 100 + views * 7 + prompt, views, prompt, chunk, 1, 2, state_tokens=state_tokens))


@pytest.mark.parametrize("name,spec", [
    ("c1", ("pi0", 1234, 1, 0, 50)),
    ("c2", ("pi0", 1234, 2, 20, 50)),
    ("c3", ("pi0", 1234, 3, 0, 63)),
])
def test_pi0_full_size_configs(name, spec):
    check_case(Case(*spec, norms="ones"), name, "golden_full.pt")         # the BASELINE configurations specify norms = 1


def test_pi05_full_size_c4():
    check_case(Case("pi05", 1234, 3, 20, 50, state_tokens=32, norms="ones"), "c4", "golden_full.pt")


def test_pi0_full_size_headline_shape_with_random_norms():
    """The shape the headline metric is quoted on (3 views, 20-token prompt, chunk 50) at full depth, with LayerNorm
    weights and biases that are random and distinct per layer: every per-layer parameter pick of the 27 SigLIP layers
    and the final norm shows in the taps."""
    check_case(Case("pi0", 1234, 3, 20, 50, norms="random"), "headline", "golden_full.pt")


def test_c5_prefix_stress_sustained_replay():
    """BASELINE configuration 5 as specified: 968-token prefix (1019 keys), a sustained loop of 1000 replays of the captured
    graph, fresh N(0,1) noise every iteration, p50 / p99 of the wall-clock forward reported (method of
    /root/reference/benchmark.py:17-33).  Every 100th iteration is re-run eagerly and must agree bit for bit; the
    latency bound is loose (twice the 15 ms target of the smaller headline shape) so that a busy box cannot fail the test."""
    import time
    from pi0_infer import Pi0Inference
    from oracle import pi0 as o0
    ck = syn.pi0_checkpoint(1234, 200, "cuda:0")
    img, state, noise = syn.observation(1234, 3, 50, "cuda:0")
    m = Pi0Inference(ck, 3, 50)
    ref = o0.forward({k: v.cpu() for k, v in ck.items()}, img.cpu(), state.cpu(), noise.cpu())
    out = m.forward(img, state, noise).float().cpu()
    assert (out - ref).abs().mean().item() <= MAE_TOL
    times, finite = [], torch.ones((), dtype=torch.bool, device="cuda:0")
    for it in range(1000):
        nz = syn.normal_bf16(1234, "diffusion_noise/%d" % it, (50, 32), 1.0, "cuda:0")     # a fresh draw, made before the clock starts
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        got = m.forward(img, state, nz)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
        finite &= torch.isfinite(got.float()).all()
        if it % 100 == 0:
            got = got.clone()
            m.buffers["diffusion_noise"].copy_(nz)
            m.record_run()
            torch.cuda.synchronize()
            assert torch.equal(got, m.buffers["diffusion_noise"]), "replay %d differs from the eager run" % it
    assert bool(finite)
    st = sorted(times)
    p50, p99 = st[len(st) // 2], st[int(0.99 * len(st))]
    print("\n[c5] 1000 sustained replays, fresh noise each: p50 %.3f ms, p99 %.3f ms, max %.3f ms" % (p50, p99, st[-1]))
    assert p50 <= 30.0
    assert torch.equal(m.forward(img, state, noise).float().cpu(), out)


def test_reference_buffer_gives_the_reference_layout_of_the_internal_activations():
    """`Engine.reference_buffer` un-tiles the activations the MFMA kernels keep in fragment order into the tensors the reference
    keeps under the same names (/root/reference/pi0_infer.py:1291-1317): shapes as there, prefix K / V equal to the oracle's,
    vision_QKV consistent with the attention output it produced (torch SDPA over it, pi0_infer.py:588-596), and a row-major
    buffer passed through unchanged."""
    c = Case("pi0", 7, views=2, prompt=5, chunk=9, vision_layers=2, llm_layers=3)
    c.forward(); torch.cuda.synchronize()
    e = c.e
    S_e, S_d = c.S_e, c.S_d
    K, V = e.reference_buffer("encoder_K"), e.reference_buffer("encoder_V")
    assert K.shape == (3, S_e + S_d, 256) and V.shape == (3, S_e + S_d, 256)
    for i in range(3):
        for got, name in ((K, "encoder_K/%d"), (V, "encoder_V/%d")):
            want = c.taps[name % i][:S_e].float()
            err = (got[i, :S_e].float().cpu() - want).norm() / want.norm()
            assert err < 2e-2, (name % i, err.item())
    assert e.reference_buffer("encoder_Q").shape == (S_e * 8, 256)
    assert e.reference_buffer("decoder_x").shape == (S_d, 1024)
    assert e.reference_buffer("decoder_x_buf").shape == (S_d, 1024)
    assert e.reference_buffer("decoder_q_buf").shape == (S_d * 8, 256)
    assert e.reference_buffer("decoder_hidden").shape == (S_d, 4096)
    assert torch.equal(e.reference_buffer("decoder_x"), c.dec_x())
    assert e.reference_buffer("encoder_x").data_ptr() == c.B["encoder_x"].data_ptr()
    # the last vision layer's Q, K, V in the reference's packing reproduce that layer's attention output
    c.run(c.capi.STAGE_VISION_EMBED)
    c.run(c.capi.STAGE_VISION_LAYER, 0)
    qkv = e.reference_buffer("vision_QKV")
    assert qkv.shape == (2, 256, 3 * 1152)
    t = qkv.float().view(-1, 256, 3, 16, 72).permute(0, 2, 3, 1, 4)
    attn = torch.nn.functional.scaled_dot_product_attention(t[:, 0], t[:, 1], t[:, 2]).transpose(1, 2).reshape(2 * 256, 1152)
    got = c.B["vision_attn"].float()
    assert ((got - attn).norm() / attn.norm()).item() < 1e-2


def test_zero_output_projection_returns_the_noise_bit_exactly():
    from pi0_infer import Pi0Inference
    ck = syn.pi0_checkpoint(3, 2, "cuda:0", 1, 2)
    ck["decoder_action_fused_out_proj_w"].zero_(); ck["decoder_action_fused_out_proj_b"].zero_()
    img, state, noise = syn.observation(3, 1, 12, "cuda:0")
    out = Pi0Inference(ck, 1, 12).forward(img, state, noise)
    assert torch.equal(out, noise)


def test_forward_contract_dtypes_devices_and_aliasing():
    from pi0_infer import Pi0Inference
    ck = syn.pi0_checkpoint(4, 3, "cuda:0", 1, 2)
    img, state, noise = syn.observation(4, 1, 10, "cuda:0")
    m = Pi0Inference({k: v.cpu() for k, v in ck.items()}, 1, 10)        # CPU checkpoint tensors are copied in
    a = m.forward(img, state, noise).clone()
    b = m.forward(img.float().cpu(), state.float().cpu(), noise.float())    # fp32 / CPU inputs, test.py:188-190
    assert b.dtype == torch.bfloat16 and b.shape == (10, 32) and b.is_cuda
    assert torch.equal(a, b)
    assert b.data_ptr() == m.buffers["diffusion_noise"].data_ptr()        # the live internal buffer, pi0_infer.py:1361
    assert m.prompt_len == 3 and m.num_views == 1 and m.chunk_size == 10
    assert set(ck) <= set(m.weights)


def test_pi05_device_side_prompt_equals_host_staged_prompt():
    """Token ids staged on the device (embedding gather x sqrt(2048) and decoder RoPE rows inside the graph) give
    bit-identical actions to the reference's host route (embeds copied into encoder_x, RoPE slice copied per call,
    pi05_infer.py:811-822), for prompts of different length on the same instance."""
    from pi05_infer import Pi05Inference
    dev, views, chunk, max_len, vocab = "cuda:0", 1, 10, 12, 640
    ck = syn.pi05_checkpoint(21, 0, dev, 1, 2, state_tokens=0)
    del ck["language_embeds"]
    table = syn.normal_bf16(21, "embedding_weight_small", (vocab, 2048), 0.02, dev)
    img, _, noise = syn.observation(21, views, chunk, dev)
    m_ids = Pi05Inference(dict(ck, embedding_weight=table), views, chunk, max_tokenize_len=max_len, discrete_state_input=False)
    assert m_ids.device_prompt and m_ids.max_prompt_len == max_len
    m_emb = Pi05Inference(dict(ck, language_embeds=torch.zeros(max_len, 2048, dtype=torch.bfloat16, device=dev)), views, chunk,
                          discrete_state_input=False)
    for n in (9, 4, 12):
        ids = syn.randint(21, "ids%d" % n, n, vocab)
        m_emb.weights["language_embeds"] = (table[ids.to(dev)].float() * (2048.0 ** 0.5)).to(torch.bfloat16)
        a = m_ids.forward_ids(img, noise, ids).float().clone()
        b = m_emb.forward(img, noise).float().clone()
        torch.cuda.synchronize()
        assert torch.isfinite(a).all()
        assert torch.equal(a, b), "prompt of %d tokens: max diff %g" % (n, (a - b).abs().max().item())
    with pytest.raises(ValueError):
        m_ids.forward_ids(img, noise, torch.zeros(max_len + 1, dtype=torch.int64))
    with pytest.raises(KeyError):
        m_emb.forward_ids(img, noise, torch.zeros(3, dtype=torch.int64))


def _word_tokenizer_dir(path):
    """A local tokenizer directory AutoTokenizer can load offline: whitespace / punctuation split, one id per word of the
    reference's prompt template and per state bin (stands in for the PaliGemma tokenizer, which does not ship here)."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    from transformers import PreTrainedTokenizerFast
    words = ["[UNK]", "Task", ":", ",", ";", "State", "Action", "pick", "up", "the", "red", "cube"] + [str(i) for i in range(256)]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="[UNK]"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    PreTrainedTokenizerFast(tokenizer_object=tok, unk_token="[UNK]").save_pretrained(str(path))
    return len(words)


def test_pi05_discrete_state_prompt_through_a_tokenizer(tmp_path):
    """discrete_state_input=True (pi05_infer.py:539-562, :769-785): the prompt template is tokenised on the host per call,
    max_prompt_len comes from the longest prompt, and forward(images, noise, task_prompt, state_tokens) must equal (a) the
    same ids handed to forward_ids, bit for bit, and (b) the CPU oracle fed with embedding[ids] * sqrt(2048)."""
    import numpy as np
    from pi05_infer import Pi05Inference
    from oracle import pi05 as oracle_pi05
    dev, views, chunk, state_dim = "cuda:0", 1, 10, 5
    vocab = _word_tokenizer_dir(tmp_path)
    ck = syn.pi05_checkpoint(33, 0, dev, 1, 2, state_tokens=0, norms="random")
    del ck["language_embeds"]
    ck["embedding_weight"] = syn.normal_bf16(33, "embedding_weight_words", (vocab, 2048), 0.02, dev)
    img, _, noise = syn.observation(33, views, chunk, dev)
    with pytest.raises(KeyError):                                         # the reference's check, pi05_infer.py:559-560
        Pi05Inference({k: v for k, v in ck.items() if k != "embedding_weight"}, views, chunk, tokenizer_path=str(tmp_path))
    m = Pi05Inference(ck, views, chunk, tokenizer_path=str(tmp_path), max_tokenize_len=64, discrete_state_input=True,
                      max_prompt_text="pick_up the red cube", state_dim_for_max_prompt=state_dim)
    # "Task : pick up the red cube , State : <5 bins> ; Action :" = 2 + 5 + 3 + 5 + 3 words
    assert m.max_prompt_len == 18 and m.device_prompt
    for prompt, bins in (("pick_up the red cube", np.array([3, 255, 17, 0, 128])), ("pick up", np.array([9, 8]))):
        ids = m.build_prompt_ids(prompt, bins)
        assert ids.dtype == torch.int64 and int(ids.max()) < vocab and (ids != 0).all()      # no unknown word
        a = m.forward(img, noise, task_prompt=prompt, state_tokens=bins).float().clone()
        b = m.forward_ids(img, noise, ids).float().clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b)
        embeds = (ck["embedding_weight"][ids.to(dev)].float() * (2048.0 ** 0.5)).to(torch.bfloat16).cpu()
        ref = oracle_pi05.forward({k: v.cpu() for k, v in ck.items() if k != "embedding_weight"}, img.cpu(), noise.cpu(),
                                  prompt_embeds=embeds.float(), max_prompt_len=m.max_prompt_len)
        mae = (a.cpu() - ref.float()).abs().mean().item()
        assert mae <= 1e-2, (prompt, mae)


def test_constructor_errors_match_the_reference():
    from pi0_infer import Pi0Inference
    ck = syn.pi0_checkpoint(4, 1, "cuda:0", 1, 1)
    no_prompt = {k: v for k, v in ck.items() if k != "language_embeds"}
    with pytest.raises(KeyError):
        Pi0Inference(no_prompt, 1, 10)
    with pytest.raises(KeyError):
        Pi0Inference(dict(ck, not_a_weight=torch.zeros(1)), 1, 10)
    with pytest.raises(RuntimeError):
        Pi0Inference(dict(ck, vision_final_norm_w=torch.zeros(7)), 1, 10)
    with pytest.raises(RuntimeError):
        Pi0Inference(ck, 1, 128)                                           # 129 suffix rows exceed the two 64-row blocks
    m = Pi0Inference(ck, 1, 10)
    with pytest.raises(RuntimeError):
        m.forward(torch.zeros(2, 224, 224, 3), torch.zeros(32), torch.zeros(10, 32))


def test_start_from_the_tile_cache_gives_bit_identical_actions(tmp_path):
    """Second construction on the same checkpoint loads the re-tiled weights from the cache file instead of
    re-tiling; a changed weight misses the cache."""
    from pi0_infer import Pi0Inference
    from pi05_infer import Pi05Inference
    ck = syn.pi0_checkpoint(41, 3, "cuda:0", 2, 2, norms="random")
    img, state, noise = syn.observation(41, 1, 9, "cuda:0")
    plain = Pi0Inference(ck, 1, 9).forward(img, state, noise).clone()
    first = Pi0Inference(ck, 1, 9, tile_cache=tmp_path)
    assert first._engine.tile_cache_hit is False and len(list(tmp_path.iterdir())) == 1
    second = Pi0Inference(ck, 1, 9, tile_cache=str(tmp_path))
    assert second._engine.tile_cache_hit is True
    assert torch.equal(first.forward(img, state, noise), plain) and torch.equal(second.forward(img, state, noise), plain)
    # another prompt re-uses the tiles (the prompt is not re-tiled), another weight does not
    ck2 = dict(ck, language_embeds=syn.language_embeds(42, 5, "cuda:0"))
    assert Pi0Inference(ck2, 1, 9, tile_cache=tmp_path)._engine.tile_cache_hit is True
    ck3 = dict(ck); ck3["decoder_ffn_up_w"] = ck["decoder_ffn_up_w"].clone(); ck3["decoder_ffn_up_w"][1, 7, 9] += 0.5
    third = Pi0Inference(ck3, 1, 9, tile_cache=tmp_path)
    assert third._engine.tile_cache_hit is False and len(list(tmp_path.iterdir())) == 2
    assert not torch.equal(third.forward(img, state, noise), plain)
    # Pi05: the scaled output projection and the conditioning are rebuilt around the cached tiles
    ck5 = syn.pi05_checkpoint(43, 4, "cuda:0", 1, 2, state_tokens=2, norms="random")
    img5, _, noise5 = syn.observation(43, 1, 6, "cuda:0")
    a = Pi05Inference(ck5, 1, 6, discrete_state_input=False, tile_cache=tmp_path)
    b = Pi05Inference(ck5, 1, 6, discrete_state_input=False, tile_cache=tmp_path)
    assert (a._engine.tile_cache_hit, b._engine.tile_cache_hit) == (False, True)
    assert torch.equal(a.forward(img5, noise5), b.forward(img5, noise5))
    # the cached region holds W diag(1 + scale) per (flow step, layer): a checkpoint that differs only in a tensor the scale
    # is computed from (here a norm-modulation bias, which is not itself re-tiled) must miss the cache
    ck6 = dict(ck5); ck6["decoder_pre_attn_norm_mod_b"] = ck5["decoder_pre_attn_norm_mod_b"].clone()
    ck6["decoder_pre_attn_norm_mod_b"][0, :1024] += 0.25
    files = len(list(tmp_path.iterdir()))
    c = Pi05Inference(ck6, 1, 6, discrete_state_input=False, tile_cache=tmp_path)
    assert c._engine.tile_cache_hit is False and len(list(tmp_path.iterdir())) == files + 1
    uncached = Pi05Inference(ck6, 1, 6, discrete_state_input=False).forward(img5, noise5).clone()
    assert torch.equal(c.forward(img5, noise5), uncached) and not torch.equal(uncached, a.forward(img5, noise5))
