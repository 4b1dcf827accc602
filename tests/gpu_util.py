"""Helpers shared by the GPU parity tests."""
import sys

import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def make_pair(variant, dim, heads, dim_head, slice_num, spatial=None, kernel=3, seed=0, sharpen=1.0, temps=None):
    """Oracle module (CPU, fp32) and HIP module (cuda:0) holding identical parameters."""
    torch.manual_seed(seed)
    if variant == "irregular":
        ref = to.OraclePhysicsAttentionIrregularMesh(dim, heads=heads, dim_head=dim_head, slice_num=slice_num)
        hip = pn.PhysicsAttentionIrregularMesh(dim, heads=heads, dim_head=dim_head, slice_num=slice_num, use_te=False)
    elif variant == "structured3d":
        ref = to.OraclePhysicsAttentionStructuredMesh3D(dim, spatial, heads=heads, dim_head=dim_head,
                                                        slice_num=slice_num, kernel=kernel)
        hip = pn.PhysicsAttentionStructuredMesh3D(dim, spatial, heads=heads, dim_head=dim_head, slice_num=slice_num,
                                                  kernel=kernel, use_te=False)
    else:
        ref = to.OraclePhysicsAttentionStructuredMesh2D(dim, spatial, heads=heads, dim_head=dim_head,
                                                        slice_num=slice_num, kernel=kernel)
        hip = pn.PhysicsAttentionStructuredMesh2D(dim, spatial, heads=heads, dim_head=dim_head, slice_num=slice_num,
                                                  kernel=kernel, use_te=False)
    with torch.no_grad():
        ref.in_project_slice.weight.mul_(sharpen)
        if temps is not None:
            ref.temperature.copy_(torch.tensor(temps, dtype=torch.float32).view(1, 1, heads, 1))
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


def assert_fp32_close(got, want, what, rtol=1e-4):
    """north-star fp32 bar: rtol 1e-4 with atol = 1e-4 * max|ref|."""
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    atol = rtol * float(want.abs().max())
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bool(bad.any()), f"{what}: max err {float(err.max()):.3e} (atol {atol:.3e}), rel-L2 {to.rel_l2(got, want):.3e}"


def assert_rel_l2(got, want, what, tol=1e-2, report=False):
    """`report`: also list the measured figure in the terminal summary of the test run."""
    r = to.rel_l2(got.detach().float().cpu(), want.detach().float().cpu())
    if report:
        import conftest

        conftest.MEASURED.append((what, r, tol))
    assert r <= tol, f"{what}: rel-L2 {r:.3e} > {tol}"
    return r
