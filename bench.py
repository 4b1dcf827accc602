#!/usr/bin/env python3
"""Benchmark of the PhysicsAttention forward path on one MI355X.

Default workload (the configuration the headline metric is quoted on): one PhysicsAttentionIrregularMesh layer,
bf16, B=1, N=1,048,576 points, C=256, 8 heads (D=32), slice_num=64, synthetic N(0,1) input (seed 1234),
seeded random weights (seed 0, orthogonal slice projection).  A "step" is one full layer forward through
the C ABI (parameter repack + kernels a+b fused, combine/attention, d), inputs resident in HBM.

Prints ONE JSON line: whole-layer Mpoints/s, the roofline of the dominant kernel (measured live with events on
the launch stream), per-kernel figures, and the CPU baseline (the oracle's ATen op sequence timed on the host
cores on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TOP_CLOCK_GHZ = 2.4  # the clock the published peaks are quoted at
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16, published


TRACE_KERNELS = True


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed run-in of the same call before the warm-up steps: after an idle spell the engine clock "
                         "overshoots, is throttled and takes some 20 ms of load to converge")
    ap.add_argument("--points", type=int, default=1 << 20)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--hidden", type=int, default=256)
    ap.add_argument("--slices", type=int, default=64)
    ap.add_argument("--kernel-reps", type=int, default=20, help="launches per kernel for the per-kernel timing")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-models", action="store_true", help="skip the per-full-model throughput lines")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic) so FETCH_SIZE / WRITE_SIZE can be scaled")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU time of the baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the slice_num sweep of the layer workload")
    ap.add_argument("--no-kernel-trace", action="store_true",
                    help="skip the in-process kernel trace (torch.profiler) of the layer calls without stage entry "
                         "points; use it when the script itself runs under rocprofv3 (one tracer at a time)")
    ap.add_argument("--mlp-only", action="store_true",
                    help="only the two stand-alone block-MLP legs (for counter runs of those kernels)")
    ap.add_argument("--conv-only", action="store_true",
                    help="only the structured-grid legs: bf16 layers with Conv2d (1024 x 1024) and Conv3d (64^3) "
                         "projections (for counter runs of the convolution kernel)")
    ap.add_argument("--write-traffic", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="no GPU work: read the counter files of two rocprofv3 --pmc runs of this script (FETCH_SIZE, "
                         "WRITE_SIZE, both with --calibrate-copy) and write profiles/hbm_traffic.json")
    return ap.parse_args()


def algorithmic_bytes_per_point(C, H, S, b=2):
    """Bytes each kernel must move per point when every tensor is read / written once (bf16)."""
    return {
        "project_softmax_reduce": (C + H * S) * b,  # read x; write w (fx_mid stays on chip)
        "project_softmax": (C + C + H * S) * b,   # read x; write fx_mid, w
        "slice_reduce": (H * S + C) * b,          # read w, fx_mid
        "deslice_project": (H * S + C) * b,       # read w; write y   (+C*b per extra residual / LayerNorm tensor)
    }


def mfma_flops_per_point(C, S):
    return {
        "project_softmax_reduce": 4 * C * C + 4 * C * S,  # two projections + slice logits + aggregation
        "project_softmax": 4 * C * C + 2 * C * S,  # two projections + slice logits
        "slice_reduce": 2 * C * S,                 # aggregation
        "deslice_project": 2 * C * S + 2 * C * C,  # deslice + out_linear
    }


SETTLE_MS = 150.0  # set from --settle-ms


def run_in(fn):
    """Untimed run-in before a timed region: keeps the GPU under the very load that is about to be timed until the
    clock governor has converged (after an idle spell the engine clock overshoots, is throttled, and takes some 20 ms
    of load to settle: the first twenty calls of the layer run up to 35 % longer than the rest)."""
    import torch

    fn()  # the first call may carry one-time set-up (parameter repacking, library initialisation): not part of the run-in
    torch.cuda.synchronize()
    t_end = time.perf_counter() + SETTLE_MS * 1e-3
    while time.perf_counter() < t_end:
        fn()
        torch.cuda.synchronize()


def time_kernel(fn, reps):
    import torch

    run_in(fn)
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()  # recorded on torch's current stream, the stream the library launches on
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps  # ms per launch


def cpu_baseline(state_dict, x_cpu_f32, C, H, S, target_seconds):
    """The oracle (the reference's ATen op sequence) on the host cores, fp32, on a prefix of the same points."""
    import torch

    from oracle import torch_oracle as to

    ref = to.OraclePhysicsAttentionIrregularMesh(C, heads=H, dim_head=C // H, slice_num=S).eval()
    ref.load_state_dict(state_dict)
    threads = torch.get_num_threads()
    n_total = x_cpu_f32.shape[1]
    probe = min(16384, n_total)
    with torch.no_grad():
        ref(x_cpu_f32[:, :probe])
        t0 = time.perf_counter()
        ref(x_cpu_f32[:, :probe])
        per_point = (time.perf_counter() - t0) / probe
        # 2 warm-ups + 5 timed runs within the budget
        n = int(min(n_total, max(probe, target_seconds / 7.0 / per_point)))
        xs = x_cpu_f32[:, :n].contiguous()
        for _ in range(2):
            ref(xs)
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            ref(xs)
            times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {
        "value": round(xs.shape[0] * n / med / 1e6, 4), "unit": "Mpoints/s", "cores": threads, "kind": "port",
        "sample": f"first {n} of {n_total} points of the same input, fp32, median of 5 runs after 2 warm-ups, "
                  f"torch {torch.__version__} CPU ATen ops, {threads} threads",
    }


def time_block_mlp(rows, C, hidden, reps=10):
    """The fused block MLP kernel alone (LN'd rows -> Linear -> GELU -> Linear -> + residual -> LayerNorm), bf16."""
    import torch

    from physicsnemo_amd import functional as PF

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(4321)
    u = torch.randn(1, rows, C, generator=g).to(dev).bfloat16()
    res = torch.randn(1, rows, C, generator=g).to(dev).bfloat16()
    w1 = (torch.randn(hidden, C, generator=g) * C ** -0.5).to(dev).bfloat16()
    w2 = (torch.randn(C, hidden, generator=g) * hidden ** -0.5).to(dev).bfloat16()
    b1, b2 = torch.zeros(hidden, device=dev), torch.zeros(C, device=dev)
    gam, bet = torch.ones(C, device=dev), torch.zeros(C, device=dev)
    ms = time_kernel(lambda: PF.mlp_forward(u, w1, b1, w2, b2, residual=res, ln_weight=gam, ln_bias=bet), reps)
    flops = 4.0 * C * hidden * rows
    return {"rows": rows, "hidden": C, "mlp_hidden": hidden, "ms": round(ms, 4),
            "mfma_tflops": round(flops / (ms * 1e-3) / 1e12, 1),
            "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TF, 4),
            "algorithmic_bytes": 4 * rows * C * 2,  # read rows and residual, write the sum and its LayerNorm
            "hbm_frac": round(4 * rows * C * 2 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}


def time_yardsticks(reps=20):
    """What this card sustains on two textbook kernels, timed like every other leg (run-in first): the GEMM library
    behind torch.matmul on a large square bf16 product, and a device-to-device copy of 1 GiB.  They are not part of
    the product; they put a practical ceiling next to the published peaks the fractions above are priced at."""
    import torch

    n = 8192
    a = torch.randn(n, n, device="cuda").bfloat16()
    b = torch.randn(n, n, device="cuda").bfloat16()
    src = torch.empty(1 << 28, device="cuda", dtype=torch.float32).normal_()
    dst = torch.empty_like(src)
    out = {}
    for name, fn, work, unit, peak in (
            ("library_gemm_bf16_8192", lambda: torch.matmul(a, b), 2.0 * n ** 3 / 1e12, "TFLOP/s", MFMA_BF16_PEAK_TF),
            ("device_copy_1gib", lambda: dst.copy_(src), 2.0 * src.numel() * 4 / 1e9, "GB/s", HBM_PEAK_GBS)):
        run_in(fn)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t0) / reps
        out[name] = {"ms": round(sec * 1e3, 4), "achieved": round(work / sec, 1), "unit": unit,
                     "frac_of_peak": round(work / sec / peak, 4)}
    del a, b, src, dst
    torch.cuda.empty_cache()
    return out


def time_structured_layers(C, S, reps=5):
    """bf16 structured-grid layers at the layer workload's width: a 1024 x 1024 grid with 3 x 3 Conv2d projections and a
    64^3 grid with 3 x 3 x 3 Conv3d projections; per leg the layer time and the convolutions' share of the MFMA peak
    (FLOPs of both projections over the time of the whole layer call: a lower bound for the kernel itself)."""
    import torch

    import physicsnemo_amd as pn

    out = []
    H = C // 32
    for name, grid, layer_cls in (("structured-2D", (1024, 1024), pn.PhysicsAttentionStructuredMesh2D),
                                  ("structured-3D", (64, 64, 64), pn.PhysicsAttentionStructuredMesh3D)):
        n = 1
        for gdim in grid:
            n *= gdim
        layer = layer_cls(C, grid, heads=H, dim_head=32, slice_num=S, kernel=3, use_te=False).cuda().eval()
        x = torch.randn(1, n, C, device="cuda").bfloat16()
        with torch.no_grad():
            run_in(lambda: layer(x))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                layer(x)
            torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / reps * 1e3
        taps = 3 ** len(grid)
        conv_tflop = 2.0 * taps * C * 2 * C * n / 1e12
        out.append({"workload": f"{name} layer bf16, grid {'x'.join(map(str, grid))}, kernel 3, C={C}, S={S}", "points": n,
                    "ms_forward": round(ms, 3), "mpoints_per_s": round(n / (ms * 1e-3) / 1e6, 2),
                    "conv_tflop": round(conv_tflop, 3),
                    "conv_mfma_frac_lower_bound": round(conv_tflop / (ms * 1e-3) / MFMA_BF16_PEAK_TF, 4)})
        del layer, x
        torch.cuda.empty_cache()
    return out


def time_training_step(points, C, S, reps=10):
    """Forward + backward of one layer under bf16 autocast at the layer workload's size (gradients w.r.t. the input
    and all ten parameters)."""
    import torch

    import physicsnemo_amd as pn

    torch.manual_seed(0)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=C // 32, dim_head=32, slice_num=S, use_te=False).cuda().train()
    x = torch.randn(1, points, C, device="cuda").bfloat16().requires_grad_(True)
    dy = torch.ones(1, points, C, device="cuda", dtype=torch.bfloat16)

    def step():
        layer.zero_grad(set_to_none=True)
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = layer(x)
        y.backward(dy)

    run_in(step)
    for _ in range(2):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / reps * 1e3
    assert torch.isfinite(x.grad[:, :1024].float()).all()
    return {"workload": f"layer forward + backward, {points} points, C={C}, S={S}, bf16 autocast",
            "ms_per_step": round(ms, 3), "mpoints_per_s": round(points / (ms * 1e-3) / 1e6, 2),
            "kernels": "MFMA forward kernels; backward: weights-stationary row GEMMs, packed slice sum, per-point MFMA "
                       "backward kernel, split-row MFMA weight-gradient kernel"}


def time_variants(points, C, S, reps=5):
    """The neighbouring layer variants at the layer workload's size where they fit, each forward (no_grad) and, where
    served, forward + backward: Transolver++, the structured 3-D and 2-D layers (implicit-GEMM projections + the
    packed-tile stages), a GALE layer with a projected context (MFMA kernels + the cross-attention stage), the context
    projector itself and a FLARE layer."""
    import torch

    import physicsnemo_amd as pn

    H = C // 32
    out = []

    def timed(fn, n=reps):
        run_in(fn)
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    def entry(name, pts, fwd_ms, train_ms=None):
        e = {"workload": name, "points": pts, "ms_forward": round(fwd_ms, 3),
             "mpoints_per_s": round(pts / (fwd_ms * 1e-3) / 1e6, 2)}
        if train_ms is not None:
            e["ms_forward_backward"] = round(train_ms, 3)
        out.append(e)

    def train_step(module, call, x):
        def step():
            module.zero_grad(set_to_none=True)
            x.grad = None
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y = call()
            y.backward(torch.ones_like(y))
        return step

    torch.manual_seed(0)
    # GALE + context projector, bf16, MFMA kernels
    geom = torch.randn(1, points // 4, C, device="cuda").bfloat16()
    proj = pn.ContextProjector(C, heads=H, dim_head=32, slice_num=S).cuda()
    gale = pn.GALE(C, heads=H, dim_head=32, slice_num=S, context_dim=32, use_te=False).cuda()
    x = torch.randn(1, points, C, device="cuda").bfloat16()
    with torch.no_grad():
        ctx = proj(geom)
        entry(f"ContextProjector bf16, C={C}, S={S}", points // 4, timed(lambda: proj(geom)))
        entry(f"GALE layer bf16 with context ({S} x 32), C={C}, S={S}", points, timed(lambda: gale((x,), ctx)))
    xg = x.clone().requires_grad_(True)
    out[-1]["ms_forward_backward"] = round(timed(train_step(gale, lambda: gale((xg,), ctx)[0], xg), 3), 3)
    del geom, x, xg
    # Transolver++ (inference on the staged MFMA kernels, training on the general kernels): a quarter of the points
    pts = points // 4
    plus = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False, plus=True).cuda()
    xp = torch.randn(1, pts, C, device="cuda").bfloat16()
    with torch.no_grad():
        fwd = timed(lambda: plus(xp), 3)
    xpg = xp.clone().requires_grad_(True)
    entry(f"Transolver++ layer bf16 (staged MFMA forward; training on the general kernels), C={C}, S={S}", pts, fwd,
          timed(train_step(plus, lambda: plus(xpg), xpg), 2))
    del xp, xpg
    # FLARE (two composed row GEMMs + the MFMA slice kernels), bf16
    flare = pn.FLARE(C, heads=H, dim_head=32, n_global_queries=S).cuda()
    xf = torch.randn(1, pts, C, device="cuda").bfloat16()
    with torch.no_grad():
        entry(f"FLARE layer bf16 (MFMA kernels), C={C}, {S} global queries", pts, timed(lambda: flare(xf), 3))
    del xf
    # GeoTransolver: context projectors + 4 GALE blocks (fused attention kernels, block-MLP kernel), bf16 autocast
    geo = pn.GeoTransolver(functional_dim=8, out_dim=4, geometry_dim=3, global_dim=16, n_layers=4, n_hidden=C,
                           n_head=H, slice_num=S).cuda().eval()
    ge, gg, gl = (torch.randn(1, pts, 8, device="cuda"), torch.randn(1, pts // 4, 3, device="cuda"),
                  torch.randn(1, 8, 16, device="cuda"))
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        entry(f"GeoTransolver bf16, 4 GALE blocks, hidden {C}, S={S}, geometry {pts // 4} points", pts,
              timed(lambda: geo(ge, None, gl, gg), 3))
    del ge, gg, gl, geo
    # whole models of the two variants, 4 layers, bf16 autocast: blocks chained through the same kernels
    for label, model in (("FLARE model", pn.FLAREModel(functional_dim=8, out_dim=4, embedding_dim=3, n_layers=4, n_hidden=C,
                                                       n_head=H, slice_num=S, use_te=False)),
                         ("Transolver++ model", pn.Transolver(functional_dim=8, out_dim=4, embedding_dim=3, n_layers=4,
                                                              n_hidden=C, n_head=H, slice_num=S, plus=True,
                                                              use_te=False))):
        model = model.cuda().eval()
        mf, me = torch.randn(1, pts, 8, device="cuda"), torch.randn(1, pts, 3, device="cuda")
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            entry(f"{label} bf16, 4 layers, hidden {C}, S={S}", pts, timed(lambda: model(mf, me), 3))
        del model, mf, me
    # ball query of the GeoTransolver local features: 8 nearest within a radius that holds about 8 points
    from physicsnemo_amd import functional as PF
    cloud, probes = torch.rand(1, pts, 3, device="cuda"), torch.rand(1, pts, 3, device="cuda")
    radius = (8 / pts * 3 / (4 * math.pi)) ** (1 / 3)
    entry(f"ball query (cell list), {pts} points, K=8, radius {radius:.4f}", pts,
          timed(lambda: PF.ball_query(cloud, probes, radius, 8), 3))
    del cloud, probes
    # structured 3-D, 64^3 grid, Conv3d k=3 projections
    g = 64
    s3 = pn.PhysicsAttentionStructuredMesh3D(C, (g, g, g), heads=H, dim_head=32, slice_num=S, kernel=3,
                                             use_te=False).cuda()
    x3 = torch.randn(1, g ** 3, C, device="cuda").bfloat16()
    with torch.no_grad():
        entry(f"structured-3D layer bf16, {g}^3 grid, Conv3d k=3, C={C}, S={S}", g ** 3, timed(lambda: s3(x3), 3))
    del s3, x3
    # structured 2-D at the layer workload's point count: 1024 x 1024 grid, Conv2d k=3 projections
    g2 = 1024
    s2 = pn.PhysicsAttentionStructuredMesh2D(C, (g2, g2), heads=H, dim_head=32, slice_num=S, kernel=3, use_te=False).cuda()
    x2 = torch.randn(1, g2 * g2, C, device="cuda").bfloat16()
    with torch.no_grad():
        entry(f"structured-2D layer bf16, {g2}x{g2} grid, Conv2d k=3, C={C}, S={S}", g2 * g2, timed(lambda: s2(x2), 3))
    return out


def synthetic_points(kind, B, N, gen):
    """Point coordinates of the full-model workloads (CPU, float32): "annulus" -- uniform in the annulus 0.5 <= r <= 1
    (2 coordinates); "surface" -- an ellipsoid (1, 0.6, 0.4) perturbed by two low-order harmonics, with unit normals
    (3 + 3); "box" -- uniform in the unit cube (3)."""
    import torch

    if kind == "annulus":
        r = torch.sqrt(torch.empty(B, N).uniform_(0.25, 1.0, generator=gen))
        th = torch.empty(B, N).uniform_(0, 2 * math.pi, generator=gen)
        return torch.stack((r * torch.cos(th), r * torch.sin(th)), -1)
    if kind == "surface":
        th = torch.acos(torch.empty(B, N).uniform_(-1, 1, generator=gen))
        ph = torch.empty(B, N).uniform_(0, 2 * math.pi, generator=gen)
        rad = 1 + 0.1 * (3 * torch.cos(th) ** 2 - 1) / 2 + 0.05 * torch.sin(th) ** 2 * torch.cos(th) * torch.cos(2 * ph)
        xyz = torch.stack((1.0 * rad * torch.sin(th) * torch.cos(ph), 0.6 * rad * torch.sin(th) * torch.sin(ph),
                           0.4 * rad * torch.cos(th)), -1)
        nrm = torch.nn.functional.normalize(xyz / torch.tensor([1.0, 0.36, 0.16]), dim=-1)
        return torch.cat((xyz, nrm), -1)
    if kind == "box":
        return torch.rand(B, N, 3, generator=gen)
    raise ValueError(kind)


def time_full_model(name, B, N, functional_dim, points, slice_num, n_layers, steps=5, warmup=2, n_hidden=256,
                    fp8_weights=False, graph=True):
    """Forward of a whole Transolver (bf16 autocast, random-init weights, synthetic inputs: coordinates from
    `synthetic_points(points, ...)`, N(0,1) fields) -> Mpoints/s.

    The PhysicsAttention layers, the block MLPs, their residual adds and the LayerNorms between them, the preprocess
    MLP, the first LayerNorm and the output Linear run in the HIP library; PyTorch-ROCm only concatenates the inputs.
    `fp8_weights`: every block's large weights (attention projections and MLP Linears) as fp8-e4m3 with
    per-output-channel scales.
    """
    import torch

    import physicsnemo_amd as pn

    torch.manual_seed(0)
    g = torch.Generator().manual_seed(1234)
    emb = synthetic_points(points, B, N, g)
    fx = torch.randn(B, N, functional_dim, generator=g)
    model = pn.Transolver(functional_dim=functional_dim, embedding_dim=emb.shape[-1], out_dim=4, n_layers=n_layers,
                          n_hidden=n_hidden, n_head=n_hidden // 32, slice_num=slice_num, use_te=False).eval().cuda()
    if fp8_weights:
        model.use_fp8_weights(True)
    fx, emb = fx.cuda(), emb.cuda()
    def fwd(a, b):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return model(a, b)

    def timed(fn):
        run_in(lambda: fn(fx, emb))
        for _ in range(warmup):
            o = fn(fx, emb)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            o = fn(fx, emb)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, o

    with torch.no_grad():
        dt, out = timed(fwd)
        assert torch.isfinite(out.float()).all()
        res = {"workload": name, "batch": B, "points": N, "layers": n_layers, "hidden": n_hidden, "slice_num": slice_num,
               "inputs": f"{points} coordinates + {functional_dim} N(0,1) field(s)",
               "weights": "fp8-e4m3 per-output-channel (attention projections + MLP Linears)" if fp8_weights else "bf16",
               "ms_per_forward": round(dt * 1e3, 3), "mpoints_per_s": round(B * N / dt / 1e6, 2)}
        if TRACE_KERNELS:
            res["kernels"] = trace_forward_kernels(lambda: fwd(fx, emb))
        if graph:
            graphed = pn.GraphedForward(fwd, fx, emb)  # the same forward replayed from a HIP graph
            dt_graph, out = timed(lambda a, b: graphed.replay())
            assert torch.isfinite(out.float()).all()
            res.update({"ms_per_forward_graph": round(dt_graph * 1e3, 3),
                        "mpoints_per_s_graph": round(B * N / dt_graph / 1e6, 2)})
            del graphed
    del model, fx, emb, out
    torch.cuda.empty_cache()
    return res


def time_structured_model(steps=5, warmup=2):
    """cfg1: Transolver on a structured 85 x 85 grid (Conv2d k = 3 projections), fp32, 4 layers, hidden 128, 8 heads,
    32 slices, mlp_ratio 1, batch 4 -> Mpoints/s.  Served by the float32 kernels of this shape class: the structured
    front end, the row kernels (hand-back + out_linear + tail, block MLP, preprocess MLP) and the general combine /
    slice-attention kernels."""
    import torch

    import physicsnemo_amd as pn

    torch.manual_seed(0)
    model = pn.Transolver(functional_dim=1, embedding_dim=2, out_dim=1, n_layers=4, n_hidden=128, n_head=8, mlp_ratio=1,
                          slice_num=32, structured_shape=(85, 85), unified_pos=False, use_te=False).eval().cuda()
    g = torch.Generator().manual_seed(1234)
    lin = torch.linspace(0, 1, 85)
    pos = torch.stack(torch.meshgrid(lin, lin, indexing="ij"), -1).reshape(1, 7225, 2).repeat(4, 1, 1).cuda()
    fx = torch.randn(4, 7225, 1, generator=g).cuda()
    def timed(fn):
        run_in(fn)
        for _ in range(warmup):
            o = fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            o = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps, o

    with torch.no_grad():
        dt, out = timed(lambda: model(fx, pos))
        assert torch.isfinite(out).all()
        # 28 900 points per forward in 23 kernel submissions; the same forward replayed from a HIP graph is one
        graphed = pn.GraphedForward(model, fx, pos)
        dt_graph, out = timed(graphed.replay)
        assert torch.isfinite(out).all()
        # one block of the model on its own (pa_block_forward: front end, combine + slice attention, per-point tail)
        block = model.blocks[1]
        hx = torch.randn(4, 7225, 128, generator=g).cuda()
        dt_block, o = timed(lambda: block(hx))
        assert torch.isfinite(o).all()
    # float32 FLOPs of a block: both 3 x 3 convolutions, slice logits, token sums, hand-back, out_linear, two MLP Linears
    pts, C, H, D, S = 4 * 7225, 128, 8, 16, 32
    block_flop = 2.0 * pts * (2 * 9 * C * C + H * D * S + 2 * H * S * D + C * C + 2 * C * C)
    structured_block = {"ms": round(dt_block * 1e3, 4), "gflop": round(block_flop / 1e9, 2),
                        "tflops": round(block_flop / dt_block / 1e12, 1),
                        "frac_of_fp32_mfma_peak": round(block_flop / dt_block / 157.3e12, 3),
                        "note": "float32-accurate FLOPs per second; the products run as bf16 MFMA pieces, so the float32 "
                                "MFMA peak (157.3 TFLOP/s) is a yardstick here, not a bound"}
    return {"workload": "cfg1: Transolver structured 2D 85x85 (conv k=3), fp32, 4 layers", "batch": 4, "points": 7225,
            "layers": 4, "slice_num": 32,
            "arithmetic": "float32 storage and accumulation; matrix products as six bf16 MFMA products of three-way "
                          "split operands (error vs float64 as small as with float32 matrix instructions)",
            "ms_per_forward": round(dt * 1e3, 3),
            "mpoints_per_s": round(4 * 7225 / dt / 1e6, 2), "ms_per_forward_graph": round(dt_graph * 1e3, 3),
            "mpoints_per_s_graph": round(4 * 7225 / dt_graph / 1e6, 2), "block": structured_block}


def source_stamp():
    """Hash of the kernel sources the traffic figures were measured with (the snapshot on the GPU box has no git
    metadata, so the stamp is taken from the files themselves)."""
    import hashlib

    h = hashlib.sha256()
    for name in ("pa_mfma.hip", "pa_mfma_ops.h"):
        with open(os.path.join(ROOT, "physicsnemo_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(kernel, B, N, C, S):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary, or None when
    the summary was taken with other kernel sources or another workload than the ones running now."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("source_stamp") != source_stamp():
        return None
    key = f"{kernel}:B{B}:N{N}:C{C}:S{S}"
    ent = rec.get("kernels", {}).get(key)
    return None if ent is None else int(ent["hbm_bytes"])


def write_traffic(fetch_dir, write_dir, B, N, C, S):
    """Turns two rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE; --calibrate-copy adds a plain 1 GiB
    copy of known traffic that fixes the scale of each counter) into profiles/hbm_traffic.json."""
    import csv
    import glob

    def per_kernel(d, counter):
        acc = {}
        for fn in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
            with open(fn) as f:
                for r in csv.DictReader(f):
                    if r["Counter_Name"] == counter:
                        acc.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        # the runtime's copy kernel also serves small transfers: the 1 GiB calibration copy is its largest dispatch
        return {k: (max(v) if "copyBuffer" in k else sum(v[-10:]) / len(v[-10:])) for k, v in acc.items()}

    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")
    copy = [k for k in fetch if "copyBuffer" in k]
    if not copy or fetch[copy[0]] < (1 << 18) or write.get(copy[0], 0) < (1 << 18):
        raise SystemExit("no calibration copy in the counter files: run the profiled command with --calibrate-copy")
    f_scale = (1 << 20) / fetch[copy[0]]   # KiB the copy really read / KiB the counter reports
    w_scale = (1 << 20) / write[copy[0]]
    names = {"project_softmax_reduce": ("project_softmax_kernel", ", true>"), "project_softmax": ("project_softmax_kernel", ", false>"),
             "slice_reduce": ("slice_reduce_kernel", ""), "deslice_project": ("deslice_project_kernel", "")}
    out = {"source_stamp": source_stamp(), "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4),
           "kernels": {}}
    for short, (frag, tail) in names.items():
        hits = [k for k in fetch if frag in k and tail in k]
        if not hits:
            continue
        k = hits[0]
        rd, wr = fetch[k] * f_scale * 1024, write.get(k, 0.0) * w_scale * 1024
        out["kernels"][f"{short}:B{B}:N{N}:C{C}:S{S}"] = {"kernel": k, "hbm_read_bytes": int(rd), "hbm_write_bytes": int(wr),
                                                          "hbm_bytes": int(rd + wr)}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(out, f, indent=1)
    print(json.dumps(out, indent=1))


# kernels of the packed-tile sequence (S = 128, and every 512-wide layer): algorithmic bytes and MFMA flops per point
def staged_kernel_model(C, H, S, b=2):
    return {
        "project_rows_kernel": {"bytes": 3 * C * b, "flops": 4 * C * C},                  # x -> x_mid, fx_mid tiles
        "slice_softmax_reduce_kernel": {"bytes": 2 * C * b, "flops": 4 * C * S},          # logits + token sums
        "deslice_recompute_kernel": {"bytes": 2 * C * b, "flops": 4 * C * S},             # logits again + deslice
        "linear_rows_kernel": {"bytes": 2 * C * b, "flops": 2 * C * C},                   # out_linear
    }


def trace_layer_kernels(layer, x, B, N, C, S, reps=10):
    """Per-kernel GPU time of one layer call, from the profiler's kernel records (for the kernel sequences that have no
    stage entry points of their own).  Averages over `reps` calls behind a run-in."""
    import collections

    import torch
    from torch.profiler import ProfilerActivity, profile

    H = C // 32
    run_in(lambda: layer(x))
    with torch.no_grad(), profile(activities=[ProfilerActivity.CUDA]) as prof:
        for _ in range(reps):
            layer(x)
        torch.cuda.synchronize()
    acc = collections.defaultdict(float)
    for ev in prof.events():
        if ev.device_type == torch.autograd.DeviceType.CUDA:
            acc[ev.name] += ev.device_time  # microseconds
    model, out = staged_kernel_model(C, H, S), {}
    for name, us in sorted(acc.items(), key=lambda kv: -kv[1]):
        ms = us / reps * 1e-3
        short = name.split("(")[0].split("::")[-1].split("<")[0]
        e = {"ms": round(ms, 4)}
        if short in model and ms > 0:
            gbs = model[short]["bytes"] * B * N / (ms * 1e-3) / 1e9
            tf = model[short]["flops"] * B * N / (ms * 1e-3) / 1e12
            e.update({"hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "mfma_frac": round(tf / MFMA_BF16_PEAK_TF, 4)})
        out[short] = e
    return out


def trace_forward_kernels(fn, top=6):
    """One call of `fn` under the in-process tracer: share of GPU time by kernel (the `top` largest), the share spent in
    this library's kernels, and how many launches went to a GEMM library (hipBLASLt / rocBLAS tile kernels)."""
    import collections

    import torch
    from torch.profiler import ProfilerActivity, profile

    with torch.no_grad(), profile(activities=[ProfilerActivity.CUDA]) as prof:
        fn()
        torch.cuda.synchronize()
    acc, calls = collections.defaultdict(float), collections.defaultdict(int)
    for ev in prof.events():
        if ev.device_type == torch.autograd.DeviceType.CUDA:
            acc[ev.name] += ev.device_time
            calls[ev.name] += 1
    total = sum(acc.values()) or 1.0
    short = lambda n: n.split("(")[0].replace("void ", "")
    return {"gpu_ms": round(total * 1e-3, 3),
            "library_share": round(sum(v for k, v in acc.items() if short(k).startswith("pa::")) / total, 4),
            "gemm_library_launches": sum(c for k, c in calls.items() if k.startswith(("Cijk_", "rocblas", "void rocblas"))),
            "top": [{"kernel": short(k), "calls": calls[k], "share": round(v / total, 4)}
                    for k, v in sorted(acc.items(), key=lambda kv: -kv[1])[:top]]}


def occupancy_sweep(x, layer, counts=(256, 192, 128, 64)):
    """Kernel (a+b) restricted to n workgroups (= n compute units busy, the rest of the chip idle): time of the launch
    and the shader clock the chip holds under it (the kernel's clock-reporting twin).  The cycles the kernel needs per
    tile do not depend on n; the clock does."""
    import torch

    from physicsnemo_amd import _lib
    from physicsnemo_amd import functional as PF

    lib, out = _lib.load(), []
    dev = x.device
    try:
        for n in counts:
            _lib.check(lib.pa_set_compute_units(int(n)), "pa_set_compute_units")
            st = PF.MfmaStages(layer.kernel_params(torch.bfloat16, dev), layer.layer_dims(x), dev)
            st.pack_params()
            run_in(lambda: st.project_softmax_reduce(x))
            ms = time_kernel(lambda: st.project_softmax_reduce(x), 20)
            ghz = []
            for _ in range(5):
                for _ in range(10):
                    st.project_softmax_reduce(x)
                ghz.append(st.project_softmax_reduce_clocked(x))
            g = sorted(ghz)[2]
            tiles = (x.shape[1] + 31) // 32 * x.shape[0]
            out.append({"compute_units": int(n), "ms": round(ms, 4), "shader_clock_ghz": round(g[0], 3),
                        "cycles_per_tile": round(g[1] / (tiles / n), 1)})
            del st
    finally:
        lib.pa_set_compute_units(0)
    return out


def measure_layer(B, N, C, S, steps, warmup, kernel_reps, x_cpu=None, cold=False, occupancy=False):
    """One PhysicsAttentionIrregularMesh layer at (B, N, C, S), bf16: whole-layer time through the module and the C ABI,
    the same call replayed from a HIP graph, and every kernel of the layer timed on its own."""
    import torch

    import physicsnemo_amd as pn
    from physicsnemo_amd import functional as PF

    dev = torch.device("cuda:0")
    H = C // 32
    torch.manual_seed(0)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False).eval()
    state = {k: v.clone() for k, v in layer.state_dict().items()}
    layer = layer.to(dev)
    if x_cpu is None:
        x_cpu = torch.randn(B, N, C, generator=torch.Generator().manual_seed(1234))
    x = x_cpu.to(dev).bfloat16().contiguous()
    dims = layer.layer_dims(x)
    path = PF.query_path(torch.bfloat16, dims)
    res = {"state": state, "path": path}

    def timed_steps():
        for _ in range(warmup):
            y = layer(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            y = layer(x)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3, y

    with torch.no_grad():
        if cold:
            # the plain procedure -- `warmup` untimed calls, then `steps` timed ones -- straight after an idle spell:
            # it includes the clock governor's transient of the first ~20 ms of load
            layer(x)
            torch.cuda.synchronize()
            time.sleep(0.5)
            res["ms_per_step_cold"], _ = timed_steps()
        run_in(lambda: layer(x))
        res["ms_per_step"], y = timed_steps()
    assert torch.isfinite(y[:, :1024].float()).all()

    graphed = pn.GraphedForward(layer, x)  # the same call recorded once into a HIP graph and replayed
    run_in(graphed.replay)
    for _ in range(warmup):
        graphed.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graphed.replay()
    torch.cuda.synchronize()
    res["ms_graph"] = (time.perf_counter() - t0) / steps * 1e3
    del graphed

    kernels, roofline = {}, None
    if path == 1:
        params = layer.kernel_params(torch.bfloat16, dev)
        st = PF.MfmaStages(params, dims, dev)
        yk = torch.empty_like(x)
        st.pack_params()
        fused = st.fused_groups > 0  # the layer call runs kernels (a)+(b) as one launch
        stage_fns = {"project_softmax": lambda: st.project_softmax(x), "slice_reduce": st.slice_reduce}
        if fused:  # the separate kernels first, so that the later stages time on the layer path's partials
            stage_fns["project_softmax_reduce"] = lambda: st.project_softmax_reduce(x)
        stage_fns.update({"combine_attention": st.combine_attention, "deslice_project": lambda: st.deslice_project(yk),
                          "pack_params": st.pack_params})
        # S = 128: the layer call runs the packed-tile kernels of the staged family (no stage entry points of their own:
        # their times are in profiles/); the stage kernels timed here are then not on the layer's path
        on_path = {"project_softmax_reduce", "deslice_project"} if fused else set()
        bytes_pp = algorithmic_bytes_per_point(C, H, S)
        flops_pp = mfma_flops_per_point(C, S)
        for name, fn in stage_fns.items():
            ms = time_kernel(fn, kernel_reps)
            entry = {"ms": round(ms, 4)}
            if name in bytes_pp:
                gbs = bytes_pp[name] * B * N / (ms * 1e-3) / 1e9
                tf = flops_pp[name] * B * N / (ms * 1e-3) / 1e12
                entry.update({"algorithmic_bytes": bytes_pp[name] * B * N, "hbm_gbs": round(gbs, 1),
                              "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "mfma_tflops": round(tf, 1),
                              "mfma_frac": round(tf / MFMA_BF16_PEAK_TF, 4)})
            # the parameter repack runs once per parameter set (the module keeps the packed copy), not per layer call
            entry["on_layer_path"] = name in on_path or (fused and name == "combine_attention")
            kernels[name] = entry
        if on_path:
            dominant = max(on_path, key=lambda k: kernels[k]["ms"])
            roofline = {"kernel": dominant, "bound": "hbm", "achieved": kernels[dominant]["hbm_gbs"], "peak": HBM_PEAK_GBS,
                        "unit": "GB/s", "frac": kernels[dominant]["hbm_frac"],
                        "traffic": measured_traffic(dominant, B, N, C, S)}
            if dominant == "project_softmax_reduce" and C == 256:
                # the shader clock the chip holds under this kernel, read inside the kernel's clock-reporting twin
                # (shader cycles against the 100 MHz wall clock over one workgroup's run) after the same run-in
                run_in(lambda: st.project_softmax_reduce(x))
                ghz = []
                for _ in range(5):
                    for _ in range(kernel_reps):  # the clocked launch queues behind these: no idle gap before it
                        st.project_softmax_reduce(x)
                    ghz.append(st.project_softmax_reduce_clocked(x)[0])
                roofline["shader_clock_ghz"] = round(sorted(ghz)[2], 3)
                roofline["top_clock_ghz"] = TOP_CLOCK_GHZ
                # the MFMA fraction priced at the clock the chip actually holds under this kernel
                roofline["mfma_frac_at_held_clock"] = round(
                    kernels[dominant]["mfma_frac"] * TOP_CLOCK_GHZ / roofline["shader_clock_ghz"], 4)
        del st, yk
        if occupancy and fused and C == 256:
            res["occupancy_sweep"] = occupancy_sweep(x, layer)
    if TRACE_KERNELS and not any(k.get("on_layer_path") for k in kernels.values()):
        # no stage entry points on this layer's path (packed-tile sequence): per-kernel times from the profiler
        res["traced_kernels"] = trace_layer_kernels(layer, x, B, N, C, S)
    res.update({"kernels": kernels, "roofline": roofline, "H": H})
    del layer, x
    torch.cuda.empty_cache()
    return res


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}): this build has no multi-GPU path; "
              "run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    B, N, C, S = args.batch, args.points, args.hidden, args.slices
    if args.write_traffic:
        write_traffic(args.write_traffic[0], args.write_traffic[1], B, N, C, S)
        return
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU path exists for the product)", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    H = C // 32
    if args.mlp_only:
        print(json.dumps({"block_mlp": time_block_mlp(1 << 20, 256, 1024, reps=3),
                          "block_mlp_c512": time_block_mlp(1 << 20, 512, 2048, reps=3)}), flush=True)
        return
    if args.conv_only:
        print(json.dumps({"structured_layers": time_structured_layers(C, S)}), flush=True)
        return
    global SETTLE_MS, TRACE_KERNELS
    SETTLE_MS = args.settle_ms
    TRACE_KERNELS = not args.no_kernel_trace
    gen = torch.Generator().manual_seed(1234)
    x_cpu = torch.randn(B, N, C, generator=gen)
    m = measure_layer(B, N, C, S, args.steps, args.warmup, args.kernel_reps, x_cpu=x_cpu, cold=True,
                      occupancy=not args.no_sweep)
    ms_per_step, path, kernels = m["ms_per_step"], m["path"], m["kernels"]
    mpoints = B * N / (ms_per_step * 1e-3) / 1e6

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def layer_fracs(bn, c, s, ms):
        """Whole-layer HBM fractions: against the fused floor (x read twice, y written once: 3 C b bytes per point) and
        against the four-kernel contract dataflow ((3 H S + 5 C) b bytes per point)."""
        floor_b, contract_b = 3 * c * 2, (3 * (c // 32) * s + 5 * c) * 2
        t = ms * 1e-3
        return {"roofline_vs_floor": round(floor_b * bn / t / 1e9 / HBM_PEAK_GBS, 4),
                "vs_contract": round(contract_b * bn / t / 1e9 / HBM_PEAK_GBS, 4),
                "floor_bytes_per_point": floor_b, "contract_bytes_per_point": contract_b}

    out = {
        "metric": "Mpoints/s per PhysicsAttention layer at 1M pts bf16; % HBM/MFMA roofline",
        "value": round(mpoints, 2), "unit": "Mpoints/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_cold": round(m["ms_per_step_cold"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3: single PhysicsAttentionIrregularMesh layer forward", "batch": B, "points": N,
                   "hidden": C, "heads": H, "dim_head": 32, "slice_num": S,
                   "kernel_path": {0: "general", 1: "mfma", 2: "mfma-staged"}[path]},
        "roofline": m["roofline"], "kernels": kernels, "layer": layer_fracs(B * N, C, S, ms_per_step),
        "graph_replay": {"ms_per_step": round(m["ms_graph"], 4),
                         "mpoints_per_s": round(B * N / (m["ms_graph"] * 1e-3) / 1e6, 2)},
    }
    if "occupancy_sweep" in m:
        out["occupancy_sweep"] = {"kernel": "project_softmax_reduce", "points": B * N, "rows": m["occupancy_sweep"]}
    if not args.no_sweep:
        # cfg3's slice sweep: the same layer and points at every slice count (the headline count taken from above)
        sweep = []
        for s_k in (16, 32, 64, 128):
            mk = m if s_k == S else measure_layer(B, N, C, s_k, args.steps, args.warmup, max(5, args.kernel_reps // 2))
            e = {"slice_num": s_k, "ms_per_step": round(mk["ms_per_step"], 4),
                 "mpoints_per_s": round(B * N / (mk["ms_per_step"] * 1e-3) / 1e6, 2),
                 "kernels": {k: {f: v[f] for f in ("ms", "hbm_frac", "mfma_frac") if f in v}
                             for k, v in mk["kernels"].items() if v.get("on_layer_path")}}
            e.update(layer_fracs(B * N, C, s_k, mk["ms_per_step"]))
            if not e["kernels"]:
                # packed-tile sequence (slice weights recomputed, never stored): per-kernel times from the profiler
                e["kernels"] = mk.get("traced_kernels", {})
            sweep.append(e)
        out["slice_sweep"] = sweep
    if not args.no_models:
        out["block_mlp"] = time_block_mlp(1 << 20, 256, 1024)
        out["block_mlp_c512"] = time_block_mlp(1 << 20, 512, 2048)
        # the cfg5 layer shape at the layer workload's point count (staged MFMA kernels on packed tiles)
        m5 = measure_layer(1, N, 512, 128, 5, 2, 5)
        out["layer_c512_s128"] = dict({"points": N, "hidden": 512, "heads": 16, "slice_num": 128,
                                       "ms_per_step": round(m5["ms_per_step"], 4),
                                       "mpoints_per_s": round(N / (m5["ms_per_step"] * 1e-3) / 1e6, 2),
                                       "kernel_path": {0: "general", 1: "mfma", 2: "mfma-staged"}[m5["path"]],
                                       "kernels": m5.get("traced_kernels", {})},
                                      **layer_fracs(N, 512, 128, m5["ms_per_step"]))
        out["yardsticks"] = time_yardsticks()
        out["training_step"] = time_training_step(N, C, S)
        out["variants"] = time_variants(N, C, S)
        out["full_model"] = [
            time_structured_model(),
            time_full_model("cfg2: Transolver irregular 2D, 8 layers", 8, 32768, 3, "annulus", 64, 8),
            time_full_model("cfg4: Transolver 3D surface cloud, 8 layers", 1, 1000000, 1, "surface", 32, 8),
            time_full_model("cfg5: Transolver 3D volume, 12 layers, hidden 512, fp8-e4m3 weights", 1, 4194304,
                            4, "box", 128, 12, steps=2, warmup=1, n_hidden=512, fp8_weights=True, graph=False),
        ]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(m["state"], x_cpu, C, H, S, args.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
