"""Transolver++ (plus=True) forward of the HIP layer against the oracle, with the uniform samples behind the Gumbel
noise handed to both sides (deterministic parity), plus a distributional check of the self-drawn noise path."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _pair(variant, dim, heads, dim_head, slice_num, grid=None, kernel=3, seed=0):
    torch.manual_seed(seed)
    if variant == "irregular":
        ref = to.OraclePhysicsAttentionIrregularMesh(dim, heads=heads, dim_head=dim_head, slice_num=slice_num, plus=True)
        hip = pn.PhysicsAttentionIrregularMesh(dim, heads=heads, dim_head=dim_head, slice_num=slice_num, plus=True,
                                               use_te=False)
    else:
        ref = to.OraclePhysicsAttentionStructuredMesh2D(dim, grid, heads=heads, dim_head=dim_head, slice_num=slice_num,
                                                        kernel=kernel, plus=True)
        hip = pn.PhysicsAttentionStructuredMesh2D(dim, grid, heads=heads, dim_head=dim_head, slice_num=slice_num,
                                                  kernel=kernel, plus=True, use_te=False)
    with torch.no_grad():
        # make the learned temperature offset matter: spread the per-point temperatures over (0.01, ~2)
        ref.proj_temperature[2].weight.mul_(3.0)
        ref.temperature.copy_(torch.linspace(-0.2, 1.2, heads).view(1, 1, heads, 1))
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


@pytest.mark.parametrize("variant,dim,heads,dim_head,S,B,N,grid", [
    ("irregular", 32, 4, 8, 8, 2, 300, None),
    ("irregular", 64, 2, 32, 64, 1, 1000, None),
    ("structured2d", 32, 4, 8, 16, 2, 63, (7, 9)),
])
def test_fp32_plus_layer_matches_oracle_given_the_noise(variant, dim, heads, dim_head, S, B, N, grid):
    announce("fp32 plus", variant, dim, heads, dim_head, S, B, N, grid)
    ref, hip = _pair(variant, dim, heads, dim_head, S, grid)
    x = torch.randn(B, N, dim)
    u = torch.rand(B, N, heads, S)
    with torch.no_grad():
        want = ref.stages(x, u)
        got = hip.forward_with_noise(x.cuda(), u.cuda(), stages=True)
    for k in ("x_mid", "w", "tok", "norm", "tok_out", "y"):
        assert_fp32_close(got[k], want[k], k)


def test_bf16_plus_layer():
    announce("bf16 plus")
    ref, hip = _pair("irregular", 256, 8, 32, 64)
    x = torch.randn(1, 4096, 256)
    u = torch.rand(1, 4096, 8, 64).bfloat16()  # what rand_like draws for bf16 logits
    with torch.no_grad():
        want = ref.forward_with_noise(x, u.float())
        got = hip.forward_with_noise(x.cuda().bfloat16(), u.cuda())
    assert got.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 plus y", tol=2e-2)


def test_plus_forward_draws_its_own_noise_reproducibly():
    announce("plus self-drawn noise")
    ref, hip = _pair("irregular", 32, 4, 8, 8)
    x = torch.randn(2, 500, 32, device="cuda")
    with torch.no_grad():
        torch.manual_seed(77)
        a = hip(x)
        torch.manual_seed(77)
        u = torch.rand(2, 500, 4, 8, device="cuda")  # the draw forward() makes: rand_like(slice_projections)
        b = hip.forward_with_noise(x, u)
        c = hip(x)  # generator advanced: different noise
    assert torch.equal(a, b)
    assert not torch.equal(a, c)
    # block / model construction accepts plus=True (reference transolver.py:213-250)
    blk = pn.TransolverBlock(4, 32, 0.0, mlp_ratio=2, slice_num=8, use_te=False, plus=True).eval().cuda()
    with torch.no_grad():
        out = blk(x)
    assert out.shape == x.shape and torch.isfinite(out).all()
    with pytest.raises(NotImplementedError):
        hip(x.requires_grad_(True))
