"""Transolver++ (plus=True) forward and backward of the HIP layer against the oracle (and autograd over it), with the
uniform samples behind the Gumbel noise handed to both sides (deterministic parity), plus a distributional check of the
self-drawn noise path.  Bars: fp32 rtol 1e-4 (2e-4 for gradients) with atol = rtol * max|ref| per tensor; bf16 output
rel-L2 2e-2, bf16 gradients rel-L2 5e-2 (1e-1 for the scalar proj_temperature.2.bias) against the fp32 reference."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _pair(variant, dim, heads, dim_head, slice_num, grid=None, kernel=3, seed=0, spread=True):
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
    if spread:
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


@pytest.mark.parametrize("dim,heads,S,B,N", [(256, 8, 64, 1, 5000), (128, 4, 16, 3, 1777), (256, 8, 32, 2, 4096),
                                             (512, 16, 128, 1, 4100), (256, 8, 128, 1, 4097)])
def test_bf16_plus_layer_on_the_mfma_kernels(dim, heads, S, B, N):
    """The whole Transolver++ layer on the staged bf16 MFMA kernels: against the fp32 oracle with the same samples, and
    against the stage-by-stage general kernels on the same bf16 inputs."""
    from physicsnemo_amd import functional as PF

    announce("bf16 plus MFMA", dim, heads, S, B, N)
    ref, hip = _pair("irregular", dim, heads, 32, S, seed=S + B)
    x = torch.randn(B, N, dim)
    u = torch.rand(B, N, heads, S).bfloat16()
    xb = x.cuda().bfloat16()
    assert PF.layer_forward_plus_supported(torch.bfloat16, hip.layer_dims(xb))
    with torch.no_grad():
        want = ref.forward_with_noise(x, u.float())
        got = hip.forward_with_noise(xb, u.cuda())
        general = hip.forward_with_noise(xb, u.cuda(), stages=True)["y"]
    assert got.dtype == torch.bfloat16 and torch.isfinite(got.float()).all()
    assert_rel_l2(got, want, "bf16 plus y (MFMA) vs fp32 oracle", tol=2e-2)
    assert_rel_l2(got, general, "bf16 plus y: MFMA vs general kernels", tol=1e-2)


def test_bf16_plus_block_tail_on_the_mfma_kernels():
    announce("bf16 plus forward_block")
    ref, hip = _pair("irregular", 256, 8, 32, 64, seed=5)
    ln = torch.nn.LayerNorm(256).cuda()
    x, res = torch.randn(1, 4500, 256).cuda().bfloat16(), torch.randn(1, 4500, 256).cuda().bfloat16()
    with torch.no_grad():
        torch.manual_seed(3)
        fx_new, normed = hip.forward_block(x, res, ln)
        torch.manual_seed(3)
        u = torch.rand(1, 4500, 8, 64, dtype=torch.bfloat16, device="cuda")
        y = hip.forward_with_noise(x, u)
    want = y.float() + res.float()
    assert_rel_l2(fx_new, want, "fx_new", tol=1e-2)
    assert_rel_l2(normed, torch.nn.functional.layer_norm(want, (256,), ln.weight, ln.bias, ln.eps), "LayerNorm", tol=1e-2)


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


def _plus_grads(module, x, u, probe):
    module.zero_grad(set_to_none=True)
    x = x.clone().requires_grad_(True)
    y = module.forward_with_noise(x, u)
    (y.float() * probe.to(y.device)).sum().backward()
    out = {"x": x.grad}
    out.update({name: p.grad for name, p in module.named_parameters()})
    return y, out


@pytest.mark.parametrize("variant,dim,heads,dim_head,S,B,N,grid", [
    ("irregular", 32, 4, 8, 8, 2, 300, None),
    ("irregular", 64, 2, 32, 64, 1, 1000, None),
    ("irregular", 48, 3, 16, 20, 3, 77, None),
    ("structured2d", 32, 4, 8, 16, 2, 63, (7, 9)),
])
def test_fp32_plus_gradients(variant, dim, heads, dim_head, S, B, N, grid):
    announce("fp32 plus backward", variant, dim, heads, dim_head, S, B, N, grid)
    ref, hip = _pair(variant, dim, heads, dim_head, S, grid)
    ref.train(), hip.train()
    with torch.no_grad():  # one head whose temperature sits below the clamp for every point: no gradient through it
        t = ref.temperature.clone()
        t[0, 0, 0, 0] = -5.0
        ref.temperature.copy_(t)
        hip.temperature.copy_(t)
    x, probe = torch.randn(B, N, dim), torch.randn(B, N, dim)
    u = torch.rand(B, N, heads, S)
    y_ref, want = _plus_grads(ref, x, u, probe)
    y_hip, got = _plus_grads(hip, x.cuda(), u.cuda(), probe)
    assert_fp32_close(y_hip, y_ref, "forward y (training path)")
    assert set(got) == set(want) and "proj_temperature.0.weight" in want and "in_project_fx.weight" not in want
    for name in want:
        assert got[name] is not None and got[name].shape == want[name].shape, name
        assert_fp32_close(got[name], want[name], f"grad {name}", rtol=2e-4)
    assert got["temperature"].flatten()[0] == 0.0 and got["temperature"].flatten()[1] != 0.0
    assert got["proj_temperature.2.weight"].abs().max() > 0


def test_bf16_plus_gradients():
    announce("bf16 plus backward (autocast)")
    ref, hip = _pair("irregular", 256, 8, 32, 64, spread=False)  # temperatures near 0.5, as initialised
    ref.train(), hip.train()
    torch.manual_seed(7)
    x, probe = torch.randn(1, 4096, 256), torch.randn(1, 4096, 256)
    u = torch.rand(1, 4096, 8, 64).bfloat16()
    _, want = _plus_grads(ref, x, u.float(), probe)
    hip.zero_grad(set_to_none=True)
    xc = x.cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip.forward_with_noise(xc, u.cuda())
    assert y.dtype == torch.bfloat16
    (y.float() * probe.cuda()).sum().backward()
    got = {"x": xc.grad}
    got.update({name: p.grad for name, p in hip.named_parameters()})
    for name in want:
        assert got[name].dtype == torch.float32 and torch.isfinite(got[name]).all(), name
        # proj_temperature.2.bias is one scalar, the sum of d a2 over every (point, head): cancelling terms of bf16 data
        assert_rel_l2(got[name], want[name], f"bf16 plus grad {name}",
                      tol=1e-1 if name == "proj_temperature.2.bias" else 5e-2)


def test_plus_training_forward_draws_noise_and_backpropagates():
    announce("plus training, self-drawn noise")
    _, hip = _pair("irregular", 32, 4, 8, 8)
    hip.train()
    x = torch.randn(2, 300, 32, device="cuda", requires_grad=True)
    torch.manual_seed(11)
    y1 = hip(x)
    y1.square().mean().backward()
    g1 = x.grad.clone()
    x.grad = None
    torch.manual_seed(11)
    y2 = hip(x)
    y2.square().mean().backward()
    assert torch.equal(y1, y2) and torch.equal(g1, x.grad)  # same generator state: same noise, same gradient
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in hip.parameters())
