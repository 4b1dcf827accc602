"""Full-model GPU parity at the BASELINE configurations (HIP layer inside the Transolver glue) against the CPU oracle."""
import math

import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _pair(**kw):
    torch.manual_seed(0)
    ref = to.OracleTransolver(**kw).eval()
    hip = pn.Transolver(use_te=False, **kw).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.cuda()


def test_cfg1_structured2d_fp32_full_size():
    # cfg1: grid 85 x 85 (N = 7225), batch 4, n_hidden 128, 8 heads (D = 16), 32 slices, 4 layers, mlp_ratio 1, fp32
    announce("cfg1 structured 2D fp32")
    ref, hip = _pair(functional_dim=1, embedding_dim=2, out_dim=1, n_layers=4, n_hidden=128, n_head=8, mlp_ratio=1,
                     slice_num=32, structured_shape=(85, 85), unified_pos=False)
    g = torch.Generator().manual_seed(1234)
    lin = torch.linspace(0, 1, 85)
    pos = torch.stack(torch.meshgrid(lin, lin, indexing="ij"), -1).reshape(1, 7225, 2).repeat(4, 1, 1)
    fx = torch.randn(4, 7225, 1, generator=g)
    with torch.no_grad():
        want = ref(fx, pos)
        got = hip(fx.cuda(), pos.cuda())
    assert got.shape == (4, 7225, 1)
    assert_fp32_close(got, want, "cfg1 model output")


def test_cfg2_irregular_bf16_autocast():
    # cfg2: 32768 annulus points, n_hidden 256, 8 heads, 64 slices, 8 layers (batch 2 of the 8 to bound CPU time)
    announce("cfg2 irregular bf16")
    ref, hip = _pair(functional_dim=3, embedding_dim=2, out_dim=4, n_layers=8, n_hidden=256, n_head=8, slice_num=64)
    g = torch.Generator().manual_seed(1234)
    B, N = 2, 32768
    r = torch.sqrt(torch.empty(B, N).uniform_(0.25, 1.0, generator=g))
    th = torch.empty(B, N).uniform_(0, 2 * math.pi, generator=g)
    pos = torch.stack((r * torch.cos(th), r * torch.sin(th)), -1)
    fx = torch.randn(B, N, 3, generator=g)
    with torch.no_grad():
        want = ref(fx, pos)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip(fx.cuda(), pos.cuda())
    assert got.shape == (B, N, 4)
    # for scale: the oracle itself under bf16 autocast on the CPU (the reference's own mixed-precision recipe: fp32
    # parameters, bf16 matrix products, fp32 softmax / LayerNorm / residual stream) against its fp32 run
    with torch.no_grad(), torch.autocast("cpu", dtype=torch.bfloat16):
        ref_bf16 = ref(fx[:1, :8192], pos[:1, :8192]).float()
    with torch.no_grad():
        want_sub = ref(fx[:1, :8192], pos[:1, :8192])
    import conftest

    conftest.MEASURED.append(("(oracle only) cfg2 model under CPU bf16 autocast vs its fp32 run, 8192 points",
                              to.rel_l2(ref_bf16, want_sub), 1.0))
    # eight bf16 blocks deep with a bf16 residual stream: measured 1.0e-2 .. 1.1e-2 (the single-layer bar is 1e-2); the
    # measured figure is listed in the test summary
    assert_rel_l2(got, want, "cfg2 model output (8 blocks, bf16 autocast)", tol=1.2e-2, report=True)


def test_cfg4_surface_bf16_layer_stack_reduced():
    # cfg4 shape class: 3 coords + 3 normals + 1 field, n_hidden 256, 8 heads, 32 slices, 8 layers; 20000 points
    # (not a multiple of 32: exercises the ragged tile) on an ellipsoid perturbed by low-order harmonics
    announce("cfg4 surface bf16")
    ref, hip = _pair(functional_dim=1, embedding_dim=6, out_dim=4, n_layers=8, n_hidden=256, n_head=8, slice_num=32)
    g = torch.Generator().manual_seed(1234)
    N = 20000
    th = torch.acos(torch.empty(N).uniform_(-1, 1, generator=g))
    ph = torch.empty(N).uniform_(0, 2 * math.pi, generator=g)
    rad = 1 + 0.1 * (3 * torch.cos(th) ** 2 - 1) / 2 + 0.05 * torch.sin(th) ** 2 * torch.cos(th) * torch.cos(2 * ph)
    xyz = torch.stack((1.0 * rad * torch.sin(th) * torch.cos(ph), 0.6 * rad * torch.sin(th) * torch.sin(ph),
                       0.4 * rad * torch.cos(th)), -1)
    nrm = torch.nn.functional.normalize(xyz / torch.tensor([1.0, 0.36, 0.16]), dim=-1)
    emb = torch.cat((xyz, nrm), -1)[None]
    fx = torch.randn(1, N, 1, generator=g)
    with torch.no_grad():
        want = ref(fx, emb)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip(fx.cuda(), emb.cuda())
    assert_rel_l2(got, want, "cfg4-class model output (8 blocks, bf16 autocast)", tol=1.2e-2, report=True)


@pytest.mark.parametrize("fp8", [False, True])
def test_cfg5_volume_model_reduced_points(fp8):
    # cfg5 as configured -- 12 layers, n_hidden 512, 16 heads (D = 32), 128 slices, 3 coordinates + 4 fields -> 4
    # channels, bf16 activations, optionally fp8-e4m3 per-channel-scaled projection and MLP weights -- at 8192 points
    # (the oracle's budget) against the fp32 oracle holding the ORIGINAL weights
    announce("cfg5 volume model", "fp8" if fp8 else "bf16")
    ref, hip = _pair(functional_dim=4, embedding_dim=3, out_dim=4, n_layers=12, n_hidden=512, n_head=16, slice_num=128)
    g = torch.Generator().manual_seed(1234)
    N = 8192
    pos = torch.rand(1, N, 3, generator=g)
    fx = torch.randn(1, N, 4, generator=g)
    with torch.no_grad():
        want = ref(fx, pos)
        if fp8:
            hip.use_fp8_weights(True)
            # the same rounding applied to the oracle's weights: isolates the kernels from the number format
            for blk in ref.blocks:
                for lin in (blk.Attn.in_project_x, blk.Attn.in_project_fx, blk.Attn.out_linear, blk.ln_mlp1[1].layers[0],
                            blk.ln_mlp1[1].layers[2]):
                    lin.weight.copy_(PF.dequantize_e4m3_per_channel(*PF.quantize_e4m3_per_channel(lin.weight)))
            want_q = ref(fx, pos)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip(fx.cuda(), pos.cuda())
    assert got.shape == (1, N, 4)
    if not fp8:
        # twelve bf16 blocks deep (the residual stream is rounded to bf16 twice per block): measured 1.2e-2
        assert_rel_l2(got, want, "cfg5 model output (12 blocks, bf16) vs the fp32 oracle", tol=1.5e-2, report=True)
        return
    # e4m3 keeps 3 mantissa bits: rounding the 60 large weight matrices of the model ALONE moves the fp32 oracle's
    # output by the first figure below; the kernels are held to the bf16 bar against the oracle with the same weights
    import conftest

    conftest.MEASURED.append(("(oracle only) e4m3 rounding of the cfg5 model's weights alone", to.rel_l2(want_q, want), 1.0))
    assert_rel_l2(got, want_q, "cfg5 model output (12 blocks, fp8 weights) vs the fp32 oracle with the dequantised weights",
                  tol=1.5e-2, report=True)
    assert_rel_l2(got, want, "cfg5 model output (12 blocks, fp8 weights) vs the fp32 oracle with the ORIGINAL weights",
                  tol=9e-2, report=True)


def _surface_points(n, g):
    th = torch.acos(torch.empty(n).uniform_(-1, 1, generator=g))
    ph = torch.empty(n).uniform_(0, 2 * math.pi, generator=g)
    rad = 1 + 0.1 * (3 * torch.cos(th) ** 2 - 1) / 2 + 0.05 * torch.sin(th) ** 2 * torch.cos(th) * torch.cos(2 * ph)
    xyz = torch.stack((1.0 * rad * torch.sin(th) * torch.cos(ph), 0.6 * rad * torch.sin(th) * torch.sin(ph),
                       0.4 * rad * torch.cos(th)), -1)
    nrm = torch.nn.functional.normalize(xyz / torch.tensor([1.0, 0.36, 0.16]), dim=-1)
    return torch.cat((xyz, nrm), -1)[None]


# The full-size multi-block paths, pinned to the oracle in two steps.  (1) One copy of a point set goes through the
# HIP model and through the fp32 oracle: the usual bound.  (2) The full-size input is COPIES copies of that point set:
# every slice token is a weighted mean over the points, so the copies leave the tokens unchanged (up to the 1e-2 the
# reference adds to the slice norms -- 1e-6 relative at these sizes -- and the order of the float32 partial sums), the
# row-local stages (LayerNorms, MLPs, projections) see each copy as they saw the original, and every copy of a point
# must come out as the original did, to within the bf16 rounding that a changed summation order can flip.
@pytest.mark.parametrize("name", ["cfg4", "cfg5-fp8"])
def test_full_size_models_by_replication(name):
    g = torch.Generator().manual_seed(1234)
    if name == "cfg4":
        # cfg4: 1 000 000 surface points, n_hidden 256, 8 heads, 32 slices, 8 layers = 32 copies of 31 250 points
        n0, copies, tol = 31250, 32, 1.3e-2  # 8 bf16 blocks deep: measured 1.17e-2 for one copy
        kw = dict(functional_dim=1, embedding_dim=6, out_dim=4, n_layers=8, n_hidden=256, n_head=8, slice_num=32)
        emb0, fx0 = _surface_points(n0, g), torch.randn(1, n0, 1, generator=g)
    else:
        # cfg5: 4 194 304 box points, n_hidden 512, 16 heads, 128 slices, 12 layers, fp8-e4m3 weights = 64 x 65 536
        n0, copies, tol = 65536, 64, 1.5e-2
        kw = dict(functional_dim=4, embedding_dim=3, out_dim=4, n_layers=12, n_hidden=512, n_head=16, slice_num=128)
        emb0, fx0 = torch.rand(1, n0, 3, generator=g), torch.randn(1, n0, 4, generator=g)
    announce("full-size model by replication", name, copies * n0)
    ref, hip = _pair(**kw)
    with torch.no_grad():
        if name != "cfg4":
            hip.use_fp8_weights(True)
            for blk in ref.blocks:  # the oracle holds the dequantised weights: the kernels, not the format, are tested
                for lin in (blk.Attn.in_project_x, blk.Attn.in_project_fx, blk.Attn.out_linear, blk.ln_mlp1[1].layers[0],
                            blk.ln_mlp1[1].layers[2]):
                    lin.weight.copy_(PF.dequantize_e4m3_per_channel(*PF.quantize_e4m3_per_channel(lin.weight)))
        want0 = ref(fx0, emb0)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got0 = hip(fx0.cuda(), emb0.cuda())
            full = hip(fx0.cuda().repeat(1, copies, 1), emb0.cuda().repeat(1, copies, 1))
    assert full.shape == (1, copies * n0, 4) and torch.isfinite(full.float()).all()
    assert_rel_l2(got0, want0, f"{name}: one copy ({n0} points) vs the fp32 oracle", tol=tol, report=True)
    # every copy of the full-size output against the ORACLE's output for the point set (the bar itself), and against
    # the HIP model's output for one copy: two bf16 evaluations whose slice tokens were summed in different orders
    # differ by about as much as each differs from the fp32 result, so that second figure is reported, bounded loosely
    want_gpu, got_gpu = want0.cuda(), got0.float()
    worst_oracle = worst_copy = 0.0
    for k in range(copies):
        part = full[:, k * n0:(k + 1) * n0].float()
        worst_oracle = max(worst_oracle, float((part - want_gpu).norm() / want_gpu.norm()))
        worst_copy = max(worst_copy, float((part - got_gpu).norm() / got_gpu.norm()))
    import conftest

    conftest.MEASURED.append((f"{name}: worst copy of the full-size output ({copies * n0} points) vs the fp32 oracle",
                              worst_oracle, tol))
    conftest.MEASURED.append((f"{name}: worst copy of the full-size output vs the HIP output for one copy", worst_copy,
                              1.5 * tol))
    assert worst_oracle <= tol, worst_oracle
    assert worst_copy <= 1.5 * tol, worst_copy
