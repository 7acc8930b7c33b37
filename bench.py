"""Latency benchmark of the Pi0 / Pi05 single-observation forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config headline|c1|c2|c3|c4|c5|dm0] [--no-cpu]

A "step" is one forward (vision encoder + prefix pass + 10 flow steps) on synthetic inputs that are
already resident in HBM.  Prints ONE JSON line: p50 latency (ms) as `value`, the live roofline of the
dominant kernel, and the CPU oracle timed on the host cores as a reported baseline.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "realtime-vla_amd"))

CONFIGS = {
    # name: (model, views, prompt_len, chunk, state_tokens, description)
    "headline": ("pi0", 3, 20, 50, 0, "Pi0, 3 views, 20-token prompt, chunk 50, 10 flow steps"),
    "c1": ("pi0", 1, 0, 50, 0, "Pi0, 1 view, empty prompt, chunk 50, 10 flow steps"),
    "c2": ("pi0", 2, 20, 50, 0, "Pi0, 2 views, 20-token prompt, chunk 50, 10 flow steps"),
    "c3": ("pi0", 3, 0, 63, 0, "Pi0, 3 views, empty prompt, chunk 63, 10 flow steps"),
    "c4": ("pi05", 3, 20, 50, 32, "Pi05, 3 views, 20 prompt + 32 state tokens, chunk 50, 10 flow steps"),
    "c5": ("pi0", 3, 200, 50, 0, "Pi0, 3 views, 200-token prompt (968-token prefix), chunk 50, 10 flow steps"),
    "dm0": ("dm0", 3, 100, 50, 0, "DM0, 3 images of 728x728, 100 language tokens, chunk 50, 10 flow steps"),
}
MFMA_PEAK_TFLOPS = 2500.0      # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
COPY_PROBE_BYTES = 256 << 20   # size of the calibration copy of --traffic-probe
PROFILES = os.path.join(ROOT, "profiles")
PROFILE_TAGS = {"headline": "pi0_3view_p20_c50"}      # workloads that have counter summaries under profiles/


def profiled_traffic(file_name, kernel_desc, workload, lib_version):
    """HBM bytes per launch as recorded in a rocprofv3 counter summary under profiles/ (a line `facts: {json}`), or None
    when no summary exists for exactly this kernel variant (tile and split as the library reports them), workload and
    library version: a counter reading of an older kernel says nothing about the current one."""
    path = os.path.join(PROFILES, file_name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("facts:"):
            try:
                f = json.loads(line[len("facts:"):])
            except ValueError:
                return None
            if f.get("kernel") == kernel_desc and f.get("workload") == workload and f.get("rtvla_version") == lib_version:
                return f.get("traffic_bytes_per_launch")
    return None


def bench_transforms(args, dev):
    """One observation's pre- and post-processing: 3 uint8 frames of 480x640 already in HBM -> bf16 model buffers, raw
    state -> normalised state, bf16 actions -> absolute float64 actions.  CPU baseline: the same steps as the reference
    runs them (Pillow + numpy on the host, /root/reference/test.py:88-201), via the oracle's restatement."""
    import numpy as np
    import torch
    from obs_transforms import ObservationTransforms
    rng = np.random.RandomState(0)
    frames = [rng.randint(0, 256, size=(480, 640, 3)).astype(np.uint8) for _ in range(3)]
    stats = {g: {"mean": rng.randn(7).tolist(), "std": (rng.rand(7) + 0.5).tolist()} for g in ("state", "actions")}
    tr = ObservationTransforms("pi0", stats, state_len=7, action_dim=7)
    dframes = [torch.from_numpy(f).to(dev) for f in frames]
    out = torch.empty(3, 224, 224, 3, dtype=torch.bfloat16, device=dev)
    sbuf = torch.empty(32, dtype=torch.bfloat16, device=dev)
    actions = torch.randn(50, 32, device=dev).to(torch.bfloat16)
    state = rng.randn(7)

    def step():
        for v in range(3):
            tr.resize_pad_normalize_into(dframes[v], out[v])
        tr._normalize_state(state, out_bf16=sbuf)
        return tr.postprocess_actions(actions, state)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    times = []
    for _ in range(args.steps):
        torch.cuda.synchronize(); t0 = time.perf_counter(); step(); torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e6)
    times.sort()
    # kernel time alone (HIP events around the three image launches)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        for v in range(3):
            tr.resize_pad_normalize_into(dframes[v], out[v])
    e1.record(); torch.cuda.synchronize()
    img_us = e0.elapsed_time(e1) * 1e3 / 20
    alg_bytes = 3 * (480 * 640 * 3 + 2 * 480 * 224 * 3 + 224 * 224 * 3 * 2)        # frame read, 8-bit intermediate write+read, bf16 write
    result = {"metric": "us per observation pre+post-processing (3 frames 480x640 -> 224x224 bf16, state, 50x7 actions)",
              "value": round(times[len(times) // 2], 1), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "higher_is_better": False, "dtype": "u8/f64", "data": "synthetic",
              "roofline": {"bound": "hbm", "kernel": "resample_h_kernel + resample_v_pad_norm_kernel x 3 frames", "achieved": round(alg_bytes / img_us / 1e3, 2),
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg_bytes / img_us / 1e3 / HBM_PEAK_GBS, 5), "launch_ms": round(img_us / 1e3, 4),
                           "traffic": None}}
    if not args.no_cpu:
        from oracle import transforms as T
        from PIL import Image
        t0 = time.perf_counter()
        for _ in range(20):
            for f in frames:                                     # the reference's own recipe: Pillow resize + numpy
                pil = Image.fromarray(f).resize((224, 168), resample=Image.BILINEAR)
                canvas = Image.new(pil.mode, (224, 224), 0); canvas.paste(pil, (0, 28))
                T.normalize_image(np.array(canvas))
            T.normalize_state(state, stats["state"], "pi0")
            T.postprocess_actions(actions.cpu().float().numpy(), stats["actions"], "pi0", state, 7)
        result["cpu_baseline"] = {"value": round((time.perf_counter() - t0) / 20 * 1e6, 1), "unit": "us", "cores": 1, "kind": "port",
                                  "sample": "20 observations, Pillow resize + numpy on one host core"}
    print(json.dumps(result))


def vendor_gemm(dev):
    """torch.matmul (hipBLASLt / rocBLAS) against this library's GEMM on the same shapes and the same box.  A comparator for the
    roofline fractions only: nothing in the product calls a library GEMM."""
    import ctypes
    import torch
    import rtvla_capi as capi
    lib, P = capi.load(), ctypes.c_void_p
    shapes = [(788, 2048, 32768, "prefix gate+up as one GEMM (the library fuses GELU(gate) * up: N = 2 x 16384)"), (788, 2048, 16384, "prefix gate alone"),
              (788, 16384, 2048, "prefix down"), (788, 2048, 2560, "prefix qkv"), (768, 1152, 3456, "SigLIP qkv"), (768, 1152, 4304, "SigLIP up"),
              (768, 4304, 1152, "SigLIP down"), (8115, 1024, 4096, "DM0 ViT up-projection"), (8115, 4096, 1024, "DM0 ViT projection"),
              (8115, 1024, 3072, "DM0 ViT qkv"), (51, 1024, 8192, "action-expert gate+up (M = 51)")]
    st = torch.cuda.Stream()
    rows = []
    for M, K, N, what in shapes:
        x = torch.randn(M, K, device=dev).bfloat16(); w = (torch.randn(K, N, device=dev) * 0.05).bfloat16()
        out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
        for _ in range(5):
            torch.matmul(x, w, out=out)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(20):
                torch.matmul(x, w, out=out)
        g.replay(); torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); g.replay(); e1.record(); torch.cuda.synchronize()
        vendor_us = e0.elapsed_time(e1) * 1e3 / 20
        mine = None
        for tile, ns in ((capi.TILE_SKINNY, 1),) if M <= 64 else ((capi.TILE_AUTO, 1), (capi.TILE_AUTO, 0)):
            need = lib.rtvla_linear_workspace_bytes(M, K, N, tile, ns)
            if not need:
                continue
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            ms = ctypes.c_float()
            with torch.cuda.stream(st):
                rc = lib.rtvla_time_linear(P(x.data_ptr()), M, K, P(w.data_ptr()), N, P(out.data_ptr()), P(ws.data_ptr()), need, tile, ns, 20, P(st.cuda_stream), ctypes.byref(ms))
            torch.cuda.synchronize()
            if rc == 0 and (mine is None or ms.value * 1e3 < mine):
                mine = ms.value * 1e3
        rows.append({"gemm": what, "M": M, "K": K, "N": N, "vendor_us": round(vendor_us, 1), "vendor_tflops": round(2.0 * M * K * N / vendor_us / 1e6),
                     "rtvla_linear_us": round(mine, 1) if mine else None, "rtvla_tflops": round(2.0 * M * K * N / mine / 1e6) if mine else None})
    print(json.dumps({"vendor_gemm": rows, "rtvla_version": lib.rtvla_version()}))


def bench_dm0(args, dev, desc, views, lang, chunk):
    """The reference's third model at its own benchmark shape (/root/reference/benchmark.py:61-62, README.md:35)."""
    import torch
    import synthetic as syn
    import rtvla_capi as capi
    from dm0_infer import DM0Inference
    seed = 1234
    ck = syn.dm0_checkpoint(seed, dev)
    img, ids, noise = syn.dm0_observation(seed, views, dev, max_lang_len=lang)
    model = DM0Inference(ck, num_images=views, max_lang_len=lang)
    ctx, stream = model._engine.ctx, torch.cuda.current_stream().cuda_stream
    lib_version = capi.load().rtvla_version()
    draws = [syn.dm0_observation(seed, views, dev, max_lang_len=lang, draw=i)[2] for i in range(16)]
    for i in range(args.warmup):
        model.forward(img, ids, draws[i % 16])
    torch.cuda.synchronize()
    times = []
    t_all0 = time.perf_counter()
    for i in range(args.steps):
        torch.cuda.synchronize(); t0 = time.perf_counter()
        model.forward(img, ids, draws[i % 16])
        torch.cuda.synchronize(); times.append((time.perf_counter() - t0) * 1e3)
    t_all = (time.perf_counter() - t_all0) * 1e3
    st = sorted(times)
    p50, p99 = st[len(st) // 2], st[min(len(st) - 1, int(0.99 * len(st)))]
    # every launch of one ViT / prefix / action-expert layer (weights cold: cycled over the layers)
    launches = {}
    for label, stage in (("vit", capi.STAGE_VISION_LAYER), ("prefix", capi.STAGE_PREFIX_LAYER), ("action", capi.STAGE_SUFFIX_LAYER)):
        rows = []
        for idx in range(16):
            r = ctx.time_launch(stage, -1, 0, idx, 3, stream)
            if r is None:
                break
            rows.append((r[1], round(r[0] * 1e3, 2)))
        launches[label] = {"launches_us": rows, "layer_us": round(ctx.time_stage(stage, -1, 0, 3, stream) * 1e3, 2)}
    stages = {name: round(ctx.time_stage(stage, 0, 0, 5, stream) * 1e3, 2) for name, stage in
              (("patch_embed_us", capi.STAGE_VISION_EMBED), ("downsample_project_us", capi.STAGE_PROJECT))}
    M, P = views * 2705, views * 169 + lang
    fc = next((r for r in launches["vit"]["launches_us"] if "fc" in r[0]), None)
    fc_flop = 2.0 * M * 1024 * 4096
    roofline = None
    if fc:
        tf = fc_flop / (fc[1] * 1e-6) / 1e12
        roofline = {"bound": "mfma", "kernel": "ViT MLP up-projection with folded LayerNorm and GELU (gemm8_kernel), M=%d K=1024 N=4096" % M,
                    "achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS, 4),
                    "launch_ms": round(fc[1] / 1e3, 4), "traffic": None, "kernel_variant": fc[0],
                    "algorithmic_bytes": 2.0 * (M * 1024 + 1024 * 4096 + M * 4096)}
    d_l = 1024 * 4096 + 2048 * 1024 + 3 * 1024 * 1536
    layer_bytes = 2.0 * d_l + 2.0 * (P + chunk) * 8 * 128 * 2
    hbm = layer_bytes / (launches["action"]["layer_us"] * 1e-6) / 1e9
    roofline_hbm = {"bound": "hbm", "kernel": "one DM0 action-expert layer", "achieved": round(hbm, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(hbm / HBM_PEAK_GBS, 4), "launch_ms": round(launches["action"]["layer_us"] / 1e3, 4), "traffic": None,
                    "algorithmic_bytes": layer_bytes}
    v_l = 1024 * 3072 + 1024 * 1024 + 2 * 1024 * 4096
    e_l = 2048 * 4096 + 2048 * 2048 + 3 * 2048 * 6144
    f_vis = 2.0 * M * (588 * 1024 + 23 * v_l) + 23 * views * 16 * 4.0 * 2705 * 2705 * 64 \
        + 2.0 * views * (676 * 9216 * 2048 + 169 * 18432 * 4096 + 169 * 4096 * 2048)
    f_pre = 2.0 * P * 28 * e_l + 28 * 16 * 4.0 * P * P * 128 / 2
    b_dec = 10 * 28 * layer_bytes
    ideal_ms = ((f_vis + f_pre) / (MFMA_PEAK_TFLOPS * 1e12) + b_dec / (HBM_PEAK_GBS * 1e9)) * 1e3
    result = {"metric": "p50 ms per DM0 forward (%d images, chunk %d, 10 steps); %% roofline" % (views, chunk),
              "value": round(p50, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": round(t_all / args.steps, 4), "p99_ms": round(p99, 4), "higher_is_better": False, "scaling": "weak",
              "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
              "config": {"workload": desc, "config_id": "dm0", "vit_tokens": M, "prefix_len": P, "graph_launches": model._engine.graph_launches,
                         "weights": "seeded N(0, 0.02^2) bf16, random norm weights", "rtvla_version": lib_version},
              "roofline": roofline, "roofline_hbm": roofline_hbm, "layers": launches, "stages": stages,
              "forward_roofline_frac": round(ideal_ms / p50, 4), "forward_ideal_ms": round(ideal_ms, 4),
              "reference_published": {"value_ms": 55.8, "hardware": "RTX 5090, Triton", "source": "README.md:35"}}
    if not args.no_cpu:
        from oracle import dm0 as od                      # the checker, timed as a baseline only
        cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or os.cpu_count()
        torch.set_num_threads(cores)
        ckc = {k: v.cpu() for k, v in ck.items()}
        cpu_times = []
        for it in range(1 + args.cpu_runs):
            t0 = time.perf_counter()
            ref = od.forward(ckc, img.cpu(), ids.cpu(), draws[0].cpu())
            if it:
                cpu_times.append((time.perf_counter() - t0) * 1e3)
        out = model.forward(img, ids, draws[0]).float().cpu()
        result["cpu_baseline"] = {"value": round(sorted(cpu_times)[len(cpu_times) // 2], 1), "unit": "ms", "cores": cores, "kind": "port",
                                  "sample": "median of %d forwards of the same workload after 1 warm-up, PyTorch CPU eager oracle" % args.cpu_runs,
                                  "runs_ms": [round(t, 1) for t in cpu_times]}
        result["action_mae_vs_oracle"] = round((out - ref).abs().mean().item(), 5)
    print(json.dumps(result))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="headline", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--cpu-runs", type=int, default=3, help="timed CPU-oracle forwards after one warm-up (median reported)")
    ap.add_argument("--transforms", action="store_true",
                    help="measure the observation pre-/post-processing kernels (3 camera frames of 480x640, state, actions) instead of the forward")
    ap.add_argument("--launch-times", action="store_true",
                    help="print the mean duration of every kernel launch of one SigLIP, prefix and action-expert layer (weights cache-warm "
                         "and cold), measured in temporary graphs, and exit")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="comparator, not part of the product: time torch.matmul (the vendor GEMM library) on the GEMM shapes of the "
                         "three models, 20 launches in a graph each, and the library's own kernel for the same shape through rtvla_time_linear")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs: launch the roofline kernel a few times, then a "
                         "plain 256 MiB device copy whose counter reading calibrates the unit, and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one observation on ONE GPU; --gpus %d is not supported "
              "(one observation is latency-bound work for a single device)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import synthetic as syn
    import rtvla_capi as capi
    capi.load()                                   # no fallback: fail loudly if the HIP library is missing
    model_name, views, prompt, chunk, state_tokens, desc = CONFIGS[args.config]
    dev = "cuda:0"
    seed = 1234
    if args.transforms:
        return bench_transforms(args, dev)
    if args.vendor_gemm:
        return vendor_gemm(dev)
    if model_name == "dm0":
        return bench_dm0(args, dev, desc, views, prompt, chunk)
    if model_name == "pi0":
        from pi0_infer import Pi0Inference
        ck = syn.pi0_checkpoint(seed, prompt, device=dev)
        img, state, noise = syn.observation(seed, views, chunk, device=dev)
        model = Pi0Inference(ck, views, chunk)
        run = lambda nz: model.forward(img, state, nz)
    else:
        from pi05_infer import Pi05Inference
        ck = syn.pi05_checkpoint(seed, prompt, device=dev, state_tokens=state_tokens)
        img, state, noise = syn.observation(seed, views, chunk, device=dev)
        model = Pi05Inference(ck, views, chunk, discrete_state_input=False)
        run = lambda nz: model.forward(img, nz)
    ctx = model._engine.ctx
    stream = torch.cuda.current_stream().cuda_stream
    lib_version = capi.load().rtvla_version()
    # index of the gate/up GEMM among the launches of one prefix layer, found by its name
    GEGLU_LAUNCH = next(i for i in range(16) if (ctx.time_launch(capi.STAGE_PREFIX_LAYER, 0, 0, i, 1, stream) or (0, "prefix geglu"))[1].startswith("prefix geglu"))
    if args.launch_times:
        for i in range(3):
            run(noise)
        torch.cuda.synchronize()
        rows = []
        for label, stage in (("siglip", capi.STAGE_VISION_LAYER), ("prefix", capi.STAGE_PREFIX_LAYER), ("action", capi.STAGE_SUFFIX_LAYER)):
            for idx in range(16):
                r = ctx.time_launch(stage, 3, 0, idx, 50, stream)
                if r is None:
                    break
                rows.append({"layer": label, "launch": r[1], "warm_us": round(r[0] * 1e3, 2),
                             "cold_us": round(ctx.time_launch(stage, -1, 0, idx, 3, stream)[0] * 1e3, 2)})
            rows.append({"layer": label, "launch": "whole layer", "warm_us": round(ctx.time_stage(stage, 3, 0, 50, stream) * 1e3, 2),
                         "cold_us": round(ctx.time_stage(stage, -1, 0, 3, stream) * 1e3, 2)})
        out = {"workload": desc, "rtvla_version": lib_version, "launches": rows}
        print(json.dumps(out))
        return
    if args.traffic_probe:
        ms, name = ctx.time_launch(capi.STAGE_PREFIX_LAYER, 3, 0, GEGLU_LAUNCH, 5, stream)
        ctx.time_stage(capi.STAGE_SUFFIX_LAYER, -1, 0, 2, stream)          # every action-expert layer, weights cold
        src = torch.ones(COPY_PROBE_BYTES // 2, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"probe": name, "launch_ms": ms, "copy_bytes": COPY_PROBE_BYTES, "rtvla_version": lib_version,
                          "workload": args.config}))
        return
    # fresh noise every iteration (BASELINE config 5); drawn up front so the timed region holds only forward()
    draws = [syn.observation(seed, views, chunk, device=dev, draw=i % 16)[2] for i in range(16)]

    for i in range(args.warmup):
        run(draws[i % 16])
    torch.cuda.synchronize()
    times = []
    t_all0 = time.perf_counter()
    for i in range(args.steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(draws[i % 16])
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    t_all = (time.perf_counter() - t_all0) * 1e3
    st = sorted(times)
    p50 = st[len(st) // 2]
    p99 = st[min(len(st) - 1, int(0.99 * len(st)))]

    # ---- roofline of the dominant kernel, measured live with HIP events on its own stream ----------
    S_v = 256 * views
    S_e = S_v + prompt + state_tokens
    S_d = chunk + (1 if model_name == "pi0" else 0)
    keys = S_e + S_d
    # dominant kernel: the Gemma-prefix GeGLU GEMM (gate and up, 2048 -> 16384 each): launch index 4 of a prefix layer
    # (cycled over the layers, so that each launch streams its 134 MB of weights from HBM as it does inside the forward;
    # repeated on one layer the weights stay in the memory-side cache and the launch is ~8 % shorter)
    geglu_ms, geglu_name = ctx.time_launch(capi.STAGE_PREFIX_LAYER, -1, 0, GEGLU_LAUNCH, 3, stream)
    geglu_warm_ms, _ = ctx.time_launch(capi.STAGE_PREFIX_LAYER, 3, 0, GEGLU_LAUNCH, 20, stream)
    assert geglu_name.startswith("prefix geglu"), geglu_name
    geglu_flop = 2.0 * 2.0 * S_e * 2048 * 16384
    mfma = geglu_flop / (geglu_ms * 1e-3) / 1e12
    # bytes the launch pulls from L2 into the CUs, fixed by its block tile (no operand is reused out of L1): every column block
    # reads the (32-row padded) activations once, every row block the gate and up weights once
    import re
    bm, bn = (int(v) for v in re.search(r"\[(\d+)x(\d+)", geglu_name).groups())
    m_pad = 32 * ((S_e + 31) // 32)
    l2_bytes = 2.0 * 2048 * ((2 * 16384 // bn) * m_pad + ((m_pad + bm - 1) // bm) * 2 * 16384)
    roofline = {"bound": "mfma", "kernel": "prefix GeGLU GEMM (gemm_mfma_kernel, EPI_GEGLU), M=%d K=2048 N=2x16384" % S_e,
                "achieved": round(mfma, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(mfma / MFMA_PEAK_TFLOPS, 4),
                "launch_ms": round(geglu_ms, 4), "launch_ms_cache_warm": round(geglu_warm_ms, 4),
                # HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each calibrated on a 256 MiB copy, as recorded in
                # profiles/ for exactly this kernel variant and library version (null otherwise)
                "traffic": profiled_traffic("gemm_geglu_%s_hbm_traffic.md" % PROFILE_TAGS.get(args.config), geglu_name, args.config, lib_version),
                "kernel_variant": geglu_name,
                "algorithmic_bytes": 2.0 * (S_e * 2048 + 2 * 2048 * 16384 + S_e * 16384),
                # informational: the rate at which the launch draws its operand tiles from L2 (the kernels here top out near 10 TB/s)
                "l2_to_cu": {"bytes": l2_bytes, "tb_per_s": round(l2_bytes / (geglu_ms * 1e-3) / 1e12, 2)}}
    # the action-expert side: one suffix layer (5 launches) streams 18 D_L-sized weight sets per step
    layer_ms = ctx.time_stage(capi.STAGE_SUFFIX_LAYER, -1, 0, 5, stream)          # all 18 layers in turn: weights cold, as in the forward
    layer_warm_ms = ctx.time_stage(capi.STAGE_SUFFIX_LAYER, 3, 0, 20, stream)
    d_l = 1024 * 2560 + 2048 * 1024 + 3 * 1024 * 4096
    layer_bytes = 2.0 * d_l + 2.0 * keys * 256 * 2
    hbm = layer_bytes / (layer_ms * 1e-3) / 1e9
    roofline_hbm = {"bound": "hbm", "kernel": "one action-expert layer (qkv, attention, o, geglu, down)",
                    "achieved": round(hbm, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(hbm / HBM_PEAK_GBS, 4),
                    "launch_ms": round(layer_ms, 4), "launch_ms_cache_warm": round(layer_warm_ms, 4),
                    # HBM bytes per layer from rocprofv3 FETCH_SIZE + WRITE_SIZE summed over the layer's kernels (profiles/)
                    "traffic": profiled_traffic("action_expert_layer_%s_hbm_traffic.md" % PROFILE_TAGS.get(args.config), "action-expert layer", args.config, lib_version),
                    "algorithmic_bytes": layer_bytes}
    # whole-forward roofline fraction: (F_vis + F_pre) / P_mfma + B_dec / BW  over the measured p50
    v_l = 1152 * 3456 + 1152 * 1152 + 2 * 1152 * 4304
    e_l = 2048 * 2560 + 2048 * 2048 + 3 * 2048 * 16384
    f_vis = 2.0 * S_v * (588 * 1152 + 27 * v_l + 1152 * 2048) + 27 * views * 16 * 4 * 256 * 256 * 72
    f_pre = 2.0 * S_e * (17 * e_l + 2048 * 512) + 17 * 8 * 4 * S_e * S_e * 256
    x_bytes = (32 * 1024 + 1024 * 1024 + 1024 * 32) if model_name == "pi0" else (32 * 1024 + 1024 * 32)
    b_dec = 10 * (2.0 * (18 * d_l + x_bytes) + 18 * 2 * keys * 256 * 2 + (37 * 3072 * 2 if model_name == "pi05" else 0))
    ideal_ms = ((f_vis + f_pre) / (MFMA_PEAK_TFLOPS * 1e12) + b_dec / (HBM_PEAK_GBS * 1e9)) * 1e3

    result = {
        "metric": "p50 ms per %s forward (%d views, chunk %d, 10 steps); %% roofline" % ("Pi0" if model_name == "pi0" else "Pi05", views, chunk),
        "value": round(p50, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(t_all / args.steps, 4), "p99_ms": round(p99, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": desc, "config_id": args.config, "S_v": S_v, "S_e": S_e, "S_d": S_d, "keys": keys,
                   "graph_launches": model._engine.graph_launches, "weights": "seeded N(0, 0.02^2) bf16, norms = 1",
                   "rtvla_version": lib_version},
        "roofline": roofline, "roofline_hbm": roofline_hbm,
        "forward_roofline_frac": round(ideal_ms / p50, 4), "forward_ideal_ms": round(ideal_ms, 4),
        "reference_published": {"value_ms": 39.2, "hardware": "RTX 4090, Triton", "source": "README.md:18"} if args.config == "headline" else None,
    }

    # ---- CPU baseline: the oracle (a port of the reference math) on the host cores: 1 warm-up + 3 timed forwards, median ----
    if not args.no_cpu:
        from oracle import pi0 as o0, pi05 as o5          # the checker, timed as a baseline only
        cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or os.cpu_count()
        torch.set_num_threads(cores)
        ckc = {k: v.cpu() for k, v in ck.items()}
        imgc, statec, noisec = img.cpu(), state.cpu(), draws[0].cpu()
        cpu_times = []
        for it in range(1 + args.cpu_runs):
            t0 = time.perf_counter()
            ref = o0.forward(ckc, imgc, statec, noisec) if model_name == "pi0" else o5.forward(ckc, imgc, noisec)
            if it:
                cpu_times.append((time.perf_counter() - t0) * 1e3)
        cpu_ms = sorted(cpu_times)[len(cpu_times) // 2]
        out = run(draws[0]).float().cpu()
        result["cpu_baseline"] = {"value": round(cpu_ms, 1), "unit": "ms", "cores": cores, "kind": "port",
                                  "sample": "median of %d forwards of the same workload after 1 warm-up, PyTorch CPU eager oracle" % args.cpu_runs,
                                  "runs_ms": [round(t, 1) for t in cpu_times]}
        result["action_mae_vs_oracle"] = round((out - ref).abs().mean().item(), 5)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
