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

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16, published


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
    served, forward + backward: Transolver++ (general kernels), the structured-3D layer (implicit-GEMM projections +
    general stages), a GALE layer with a projected context (MFMA kernels + the cross-attention stage), the context
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
    return out


def time_full_model(name, B, N, functional_dim, embedding_dim, slice_num, n_layers, steps=5, warmup=2, n_hidden=256,
                    fp8_weights=False, graph=True):
    """Forward of a whole Transolver (bf16 autocast, random-init weights, synthetic N(0,1) inputs) -> Mpoints/s.

    The PhysicsAttention layers, the block MLPs, their residual adds and the LayerNorms between them run in the HIP
    library; the remaining glue (preprocess MLP, first LayerNorm, output Linear) is PyTorch-ROCm.
    """
    import torch

    import physicsnemo_amd as pn

    torch.manual_seed(0)
    model = pn.Transolver(functional_dim=functional_dim, embedding_dim=embedding_dim, out_dim=4, n_layers=n_layers,
                          n_hidden=n_hidden, n_head=n_hidden // 32, slice_num=slice_num, use_te=False).eval().cuda()
    if fp8_weights:  # the layers' three large weights as fp8-e4m3 bytes with per-output-channel scales
        for blk in model.blocks:
            blk.Attn.use_fp8_weights(True)
    g = torch.Generator().manual_seed(1234)
    fx = torch.randn(B, N, functional_dim, generator=g).cuda()
    emb = torch.randn(B, N, embedding_dim, generator=g).cuda()
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
               "ms_per_forward": round(dt * 1e3, 3), "mpoints_per_s": round(B * N / dt / 1e6, 2)}
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
    32 slices, mlp_ratio 1, batch 4 -> Mpoints/s.  Served by the general (fp32) kernels."""
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
        # 28 900 points per forward: the eager call is bound by its ~50 kernel submissions; the same forward replayed
        # from a HIP graph is one submission
        graphed = pn.GraphedForward(model, fx, pos)
        dt_graph, out = timed(graphed.replay)
        assert torch.isfinite(out).all()
    return {"workload": "cfg1: Transolver structured 2D 85x85 (conv k=3), fp32, 4 layers", "batch": 4, "points": 7225,
            "layers": 4, "slice_num": 32, "ms_per_forward": round(dt * 1e3, 3),
            "mpoints_per_s": round(4 * 7225 / dt / 1e6, 2), "ms_per_forward_graph": round(dt_graph * 1e3, 3),
            "mpoints_per_s_graph": round(4 * 7225 / dt_graph / 1e6, 2)}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}): this build has no multi-GPU path; "
              "run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch

    import physicsnemo_amd as pn
    from physicsnemo_amd import functional as PF

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU path exists for the product)", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    B, N, C, S = args.batch, args.points, args.hidden, args.slices
    H = C // 32
    torch.manual_seed(0)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False).eval()
    state = {k: v.clone() for k, v in layer.state_dict().items()}
    layer = layer.to(dev)
    gen = torch.Generator().manual_seed(1234)
    x_cpu = torch.randn(B, N, C, generator=gen)
    x = x_cpu.to(dev).bfloat16().contiguous()
    dims = layer.layer_dims(x)
    path = PF.query_path(torch.bfloat16, dims)

    global SETTLE_MS
    SETTLE_MS = args.settle_ms
    with torch.no_grad():
        run_in(lambda: layer(x))
        for _ in range(args.warmup):
            y = layer(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = layer(x)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    mpoints = B * N / (ms_per_step * 1e-3) / 1e6
    assert torch.isfinite(y[:, :1024].float()).all()

    # the same call recorded once into a HIP graph and replayed (same kernels, one submission per step)
    graphed = pn.GraphedForward(layer, x)  # its static input holds a copy of x
    run_in(graphed.replay)
    for _ in range(args.warmup):
        graphed.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graphed.replay()
    torch.cuda.synchronize()
    ms_graph = (time.perf_counter() - t0) / args.steps * 1e3
    del graphed

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    kernels = {}
    roofline = None
    if path == 1:
        params = layer.kernel_params(torch.bfloat16, dev)
        st = PF.MfmaStages(params, dims, dev)
        yk = torch.empty_like(x)
        st.pack_params()
        fused = st.fused_groups > 0  # the layer call runs kernels (a)+(b) as one launch
        stage_fns = {}
        if fused:  # the separate kernels first, so that the later stages time on the layer path's partials
            stage_fns["project_softmax"] = lambda: st.project_softmax(x)
            stage_fns["slice_reduce"] = st.slice_reduce
            stage_fns["project_softmax_reduce"] = lambda: st.project_softmax_reduce(x)
        else:
            stage_fns["project_softmax"] = lambda: st.project_softmax(x)
            stage_fns["slice_reduce"] = st.slice_reduce
        stage_fns.update({
            "combine_attention": st.combine_attention,
            "deslice_project": lambda: st.deslice_project(yk),
            "pack_params": st.pack_params,
        })
        on_path = ({"project_softmax_reduce", "deslice_project"} if fused else
                   {"project_softmax", "slice_reduce", "deslice_project"})
        bytes_pp = algorithmic_bytes_per_point(C, H, S)
        flops_pp = mfma_flops_per_point(C, S)
        for name, fn in stage_fns.items():
            ms = time_kernel(fn, args.kernel_reps)
            entry = {"ms": round(ms, 4)}
            if name in bytes_pp:
                gbs = bytes_pp[name] * B * N / (ms * 1e-3) / 1e9
                tf = flops_pp[name] * B * N / (ms * 1e-3) / 1e12
                entry.update({"algorithmic_bytes": bytes_pp[name] * B * N, "hbm_gbs": round(gbs, 1),
                              "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "mfma_tflops": round(tf, 1),
                              "mfma_frac": round(tf / MFMA_BF16_PEAK_TF, 4)})
            # the parameter repack runs once per parameter set (the module keeps the packed copy), not per layer call
            entry["on_layer_path"] = name in on_path or name == "combine_attention"
            kernels[name] = entry
        dominant = max(on_path, key=lambda k: kernels[k]["ms"])
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 1 GiB copy (x2.0 / x1.0);
        # measured for the default workload only (profiles/layer_cfg3_s64_hbm_traffic.md)
        measured_traffic = {"project_softmax_reduce": (517 + 1041) << 20, "project_softmax": (542 + 1536) << 20, "slice_reduce": (1536 + 8) << 20,
                            "deslice_project": (1025 + 512) << 20}
        default_workload = (B, N, C, S) == (1, 1 << 20, 256, 64)
        roofline = {"kernel": dominant, "bound": "hbm", "achieved": kernels[dominant]["hbm_gbs"], "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": kernels[dominant]["hbm_frac"],
                    "traffic": measured_traffic[dominant] if default_workload else None}

    out = {
        "metric": "Mpoints/s per PhysicsAttention layer at 1M pts bf16; % HBM/MFMA roofline",
        "value": round(mpoints, 2), "unit": "Mpoints/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3: single PhysicsAttentionIrregularMesh layer forward", "batch": B, "points": N,
                   "hidden": C, "heads": H, "dim_head": 32, "slice_num": S,
                   "kernel_path": {0: "general", 1: "mfma", 2: "mfma-staged"}[path]},
        "roofline": roofline, "kernels": kernels,
        "graph_replay": {"ms_per_step": round(ms_graph, 4), "mpoints_per_s": round(B * N / (ms_graph * 1e-3) / 1e6, 2)},
    }
    if not args.no_models:
        out["block_mlp"] = time_block_mlp(1 << 20, 256, 1024)
        out["training_step"] = time_training_step(N, C, S)
        out["variants"] = time_variants(N, C, S)
        out["full_model"] = [
            time_structured_model(),
            time_full_model("cfg2: Transolver irregular 2D, 8 layers", 8, 32768, 3, 2, 64, 8),
            time_full_model("cfg4: Transolver 3D surface cloud, 8 layers", 1, 1000000, 1, 6, 32, 8),
            time_full_model("cfg5: Transolver 3D volume, 12 layers, hidden 512, fp8-e4m3 projection weights", 1, 4194304,
                            4, 3, 128, 12, steps=2, warmup=1, n_hidden=512, fp8_weights=True, graph=False),
        ]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(state, x_cpu, C, H, S, args.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
