"""Sizes whose element and byte offsets pass 2^32: index arithmetic of the kernels at the top of the size range.

No oracle run is affordable there; the checks use properties that hold at any size:
  * row-local kernels (block MLP with residual and LayerNorm): a tensor made of k copies of a small one gives k copies
    of the small result, bit for bit;
  * the attention layer: the slice tokens are weighted means over the points, so k copies of a point set give the
    tokens of one copy (up to the 1e-2 the reference adds to the slice norms, 1e-6 relative here, and the order of the
    float32 partial sums), and every copy of a point gets the output of the original.
"""
import pytest
import torch

import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_rel_l2

pytestmark = pytest.mark.gpu

N0 = (1 << 20) + 37  # ragged against every tile size
COPIES = 17          # 17 * N0 * 256 elements = 4.56e9 > 2^32


def test_block_mlp_rows_beyond_2_32_elements():
    announce("large mlp", COPIES * N0)
    C, Fh = 256, 1024
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(7)
    u0 = torch.randn(1, N0, C, generator=g).bfloat16().to(dev)
    r0 = torch.randn(1, N0, C, generator=g).bfloat16().to(dev)
    w1 = (torch.randn(Fh, C, generator=g) * 0.06).bfloat16().to(dev)
    w2 = (torch.randn(C, Fh, generator=g) * 0.03).bfloat16().to(dev)
    b1, b2 = (torch.randn(Fh, generator=g) * 0.1).to(dev), (torch.randn(C, generator=g) * 0.1).to(dev)
    gam, bet = (torch.rand(C, generator=g) + 0.5).to(dev), (torch.randn(C, generator=g) * 0.1).to(dev)
    with torch.no_grad():
        y0, ln0 = PF.mlp_forward(u0, w1, b1, w2, b2, residual=r0, ln_weight=gam, ln_bias=bet)
        u = u0.repeat(1, COPIES, 1)
        r = r0.repeat(1, COPIES, 1)
        assert u.numel() > 1 << 32
        y, ln = PF.mlp_forward(u, w1, b1, w2, b2, residual=r, ln_weight=gam, ln_bias=bet)
    del u, r
    for k in (0, 1, COPIES // 2, COPIES - 1):  # the last copy lies wholly beyond 2^32 elements
        assert torch.equal(y[:, k * N0:(k + 1) * N0], y0), f"copy {k}"
        assert torch.equal(ln[:, k * N0:(k + 1) * N0], ln0), f"copy {k} (LayerNorm)"
    assert torch.isfinite(y0.float()).all()


@pytest.mark.parametrize("C,S,COPIES", [(256, 64, 17), (256, 128, 17), (512, 128, 9)])
def test_layer_points_beyond_2_32_elements(C, S, COPIES):
    # C = 256, S = 64: the fused kernels of the headline path; S = 128: the packed-tile sequence with recomputed slice
    # weights; C = 512: the staged kernels of the 512-wide layers
    announce("large layer", C, S, COPIES * N0)
    H = C // 32
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False).eval().to(dev)
    g = torch.Generator().manual_seed(11)
    x0 = torch.randn(1, N0, C, generator=g).bfloat16().to(dev)
    p = layer.kernel_params(torch.bfloat16, dev)
    with torch.no_grad():
        y0, tok0 = PF.layer_forward(x0, p, layer.layer_dims(x0), return_slice_tokens=True)
        x = x0.repeat(1, COPIES, 1)
        assert x.numel() > 1 << 32
        y, tok = PF.layer_forward(x, p, layer.layer_dims(x), return_slice_tokens=True)
    del x
    assert torch.isfinite(y.float()).all()
    assert_rel_l2(tok, tok0, f"S={S}: slice tokens of {COPIES} copies vs one copy", tol=1e-4)
    for k in (0, COPIES // 2, COPIES - 1):
        assert_rel_l2(y[:, k * N0:(k + 1) * N0], y0, f"S={S}: outputs of copy {k}", tol=3e-3)


def test_general_fp32_layer_beyond_2_32_elements():
    # the general (float32) kernels: 71 M points of 64 channels, two heads, 16 slices -- x, x_mid, fx_mid and the output
    # hold 4.6e9 elements each, the slice weights 2.3e9
    n0, copies = (1 << 22) + 37, 17
    announce("large general fp32", copies * n0)
    C, H, S = 64, 2, 16
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False).eval().to(dev)
    g = torch.Generator().manual_seed(13)
    x0 = torch.randn(1, n0, C, generator=g).to(dev)
    p = layer.kernel_params(torch.float32, dev)
    assert PF.query_path(torch.float32, layer.layer_dims(x0)) == 0
    with torch.no_grad():
        y0, tok0 = PF.layer_forward(x0, p, layer.layer_dims(x0), return_slice_tokens=True)
        x = x0.repeat(1, copies, 1)
        assert x.numel() > 1 << 32
        y, tok = PF.layer_forward(x, p, layer.layer_dims(x), return_slice_tokens=True)
    del x
    assert_rel_l2(tok, tok0, f"fp32: slice tokens of {copies} copies vs one copy", tol=1e-5)
    for k in (0, copies // 2, copies - 1):
        assert_rel_l2(y[:, k * n0:(k + 1) * n0], y0, f"fp32: outputs of copy {k}", tol=1e-5)


@pytest.mark.parametrize("dtype,C,H,D,S,grid,B", [
    (torch.bfloat16, 256, 8, 32, 64, (512, 513), 70),   # staged MFMA kernels behind the implicit-GEMM projections
    (torch.float32, 128, 8, 16, 32, (256, 257), 515),   # fused float32 front end and row kernels
])
def test_structured2d_batches_beyond_2_32_elements(dtype, C, H, D, S, grid, B):
    # batch elements are independent: a batch of B copies of one grid gives B copies of its output
    n = grid[0] * grid[1]
    announce("large structured2d", dtype, C, grid, B)
    assert B * n * C > 1 << 32
    dev = torch.device("cuda:0")
    torch.manual_seed(9)
    layer = pn.PhysicsAttentionStructuredMesh2D(C, grid, heads=H, dim_head=D, slice_num=S, kernel=3,
                                                use_te=False).eval().to(dev)
    g = torch.Generator().manual_seed(17)
    x0 = torch.randn(1, n, C, generator=g).to(dtype).to(dev)
    with torch.no_grad():
        y0 = layer(x0)
        x = x0.repeat(B, 1, 1)
        y = layer(x)
    del x
    assert y.shape == (B, n, C) and torch.isfinite(y.float()).all()
    tol = 2e-3 if dtype == torch.bfloat16 else 1e-5
    for b in (0, 1, B // 2, B - 1):
        assert_rel_l2(y[b:b + 1], y0, f"{dtype}: batch element {b} of {B}", tol=tol)


def test_layer_training_step_beyond_2_32_elements():
    # forward + backward of the bf16 layer on 17 copies of a point set, probed with 17 copies of one cotangent: the slice
    # tokens are those of one copy, so every parameter gradient is 17 times that of one copy and every copy of a point
    # gets the input gradient of the original
    announce("large training step", COPIES * N0)
    C, H, S = 256, 8, 64
    dev = torch.device("cuda:0")
    torch.manual_seed(21)
    layer = pn.PhysicsAttentionIrregularMesh(C, heads=H, dim_head=32, slice_num=S, use_te=False).to(dev)
    g = torch.Generator().manual_seed(23)
    x0 = torch.randn(1, N0, C, generator=g).bfloat16().to(dev)
    probe0 = torch.randn(1, N0, C, generator=g).bfloat16().to(dev)

    def step(x, probe):
        layer.zero_grad(set_to_none=True)
        xc = x.clone().requires_grad_(True)
        y = layer(xc)
        assert y.dtype == torch.bfloat16
        (y.float() * probe.float()).sum().backward()
        return xc.grad, {name: p.grad.clone() for name, p in layer.named_parameters()}

    dx0, grads0 = step(x0, probe0)
    dx, grads = step(x0.repeat(1, COPIES, 1), probe0.repeat(1, COPIES, 1))
    assert dx.numel() > 1 << 32
    for name, g0 in grads0.items():
        assert torch.isfinite(grads[name]).all(), name
        assert_rel_l2(grads[name], COPIES * g0, f"grad {name}: {COPIES} copies vs {COPIES} x one copy", tol=1e-2)
    for k in (0, COPIES // 2, COPIES - 1):
        assert_rel_l2(dx[:, k * N0:(k + 1) * N0], dx0, f"input gradient of copy {k}", tol=1e-2)
