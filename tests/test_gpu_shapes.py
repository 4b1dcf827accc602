"""Shapes that fall on and off the 16-byte fast paths of the general kernels (slice counts and head widths that are,
or are not, whole numbers of 16-byte units in float32 and bf16), ragged point counts, batches: forward stages and all
gradients against the oracle.  Bars: fp32 rtol 1e-4 (gradients 2e-4), bf16 rel-L2 1e-2 (gradients 3e-2; the scalar
temperature sums 1e-1)."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2, make_pair

pytestmark = pytest.mark.gpu

STAGES = ("x_mid", "fx_mid", "w", "tok", "norm", "tok_out", "y")
#          dim heads dim_head  S    B   N
SHAPES = [(40, 2, 20, 20, 2, 131),    # S = 20: units of four only;  D = 20
          (36, 3, 12, 6, 1, 257),     # S = 6: no vector path at all; D = 12
          (80, 2, 40, 24, 3, 65),     # D = 40, S = 24: whole 16-byte units in both types
          (64, 8, 8, 40, 1, 1000),    # many heads, narrow
          (64, 2, 32, 128, 2, 300),   # S = 128
          (32, 1, 32, 10, 2, 33),     # one head, S = 10
          (24, 2, 12, 4, 4, 7)]       # a handful of points


@pytest.mark.parametrize("dim,heads,dim_head,S,B,N", SHAPES)
def test_fp32_forward_stages_and_gradients(dim, heads, dim_head, S, B, N):
    announce("shape sweep fp32", dim, heads, dim_head, S, B, N)
    ref, hip = make_pair("irregular", dim, heads, dim_head, S, seed=S + N, sharpen=2.0)
    x, probe = torch.randn(B, N, dim), torch.randn(B, N, dim)
    with torch.no_grad():
        want = ref.stages(x)
        got = hip.forward_stages(x.cuda())
    for k in STAGES:
        assert_fp32_close(got[k], want[k], k)
    ref.train(), hip.train()
    xr, xh = x.clone().requires_grad_(), x.clone().cuda().requires_grad_()
    (ref(xr) * probe).sum().backward()
    (hip(xh) * probe.cuda()).sum().backward()
    assert_fp32_close(xh.grad, xr.grad, "d x", rtol=2e-4)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=2e-4)


@pytest.mark.parametrize("dim,heads,dim_head,S,B,N", SHAPES)
def test_bf16_forward_and_gradients(dim, heads, dim_head, S, B, N):
    announce("shape sweep bf16", dim, heads, dim_head, S, B, N)
    ref, hip = make_pair("irregular", dim, heads, dim_head, S, seed=S + N)
    x, probe = torch.randn(B, N, dim), torch.randn(B, N, dim)
    ref.train(), hip.train()
    xr = x.clone().requires_grad_()
    yr = ref(xr)
    (yr * probe).sum().backward()
    xh = x.clone().cuda().bfloat16().requires_grad_()
    yh = hip(xh)
    assert yh.dtype == torch.bfloat16
    assert_rel_l2(yh, yr, "bf16 y", tol=1e-2)
    (yh.float() * probe.cuda()).sum().backward()
    assert_rel_l2(xh.grad, xr.grad, "bf16 d x", tol=3e-2)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        tol = 1e-1 if name in ("temperature", "in_project_slice.bias") else 3e-2
        assert_rel_l2(grads[name].grad, p.grad, f"bf16 grad {name}", tol=tol)


def test_backward_refuses_slice_tables_beyond_lds_with_a_clear_error():
    """The slice-attention backward keeps seven S x (D + 1) float32 tables in LDS: S = 128 with D = 48 does not fit.
    The forward serves the shape; asking for gradients raises instead of computing something else."""
    announce("backward LDS limit")
    ref, hip = make_pair("irregular", 96, 2, 48, 128)
    x = torch.randn(1, 200, 96)
    with torch.no_grad():
        assert_fp32_close(hip(x.cuda()), ref(x), "forward y")
    with pytest.raises(RuntimeError, match="backward kernels do not serve this shape"):
        hip(x.cuda().requires_grad_())


@pytest.mark.parametrize("variant,grid,kernel,dim,heads,S,B", [
    ("structured2d", (64, 64), 3, 128, 4, 32, 1),
    ("structured2d", (48, 50), 5, 256, 8, 64, 2),
    ("structured3d", (16, 16, 16), 3, 256, 8, 64, 1),
    ("structured3d", (12, 10, 9), 3, 128, 4, 16, 4),
    # 256 / 512 channels: the implicit-GEMM kernel that writes packed tiles; grids whose rows straddle the 32-point tiles,
    # ragged last tiles, a grid narrower than the kernel's reach, one slice tile and four
    ("structured2d", (37, 29), 3, 256, 8, 32, 4),
    ("structured2d", (2050, 2), 3, 256, 8, 16, 1),
    ("structured2d", (1, 4100), 5, 256, 8, 64, 1),
    ("structured3d", (11, 9, 13), 3, 256, 8, 128, 4),
    ("structured3d", (3, 70, 20), 5, 256, 8, 32, 1),
    # 512 channels on the same kernel: reduction steps of 256 channels, two passes of 256 outputs per projection
    ("structured2d", (40, 37), 3, 512, 16, 64, 3),
    ("structured3d", (9, 8, 10), 3, 512, 16, 128, 6),
])
def test_bf16_structured_layers_on_the_staged_mfma_kernels(variant, grid, kernel, dim, heads, S, B):
    """Grid-convolution projections feeding the staged bf16 MFMA kernels (the implicit-GEMM kernels write fx_mid in the
    packed operand layout and x_mid either in natural layout or, at 256 / 512 channels, as packed tiles too), against the
    fp32 oracle; with the block tail."""
    announce("bf16 structured staged MFMA", variant, grid, kernel, dim, heads, S, B)
    ref, hip = make_pair(variant, dim, heads, 32, S, spatial=grid, kernel=kernel, seed=S)
    n = 1
    for g in grid:
        n *= g
    x = torch.randn(B, n, dim)
    xb = x.cuda().bfloat16()
    assert PF.query_path(torch.bfloat16, hip.layer_dims(xb)) == 2
    with torch.no_grad():
        want = ref(x)
        got = hip(xb)
        ln = torch.nn.LayerNorm(dim).cuda()
        res = torch.randn(B, n, dim, device="cuda").bfloat16()
        fx_new, normed = hip.forward_block(xb, res, ln)
    assert got.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 structured y vs fp32 oracle", tol=1e-2)
    tail = got.float() + res.float()
    assert_rel_l2(fx_new, tail, "fx_new", tol=1e-2)
    assert_rel_l2(normed, torch.nn.functional.layer_norm(tail, (dim,), ln.weight, ln.bias, ln.eps), "LayerNorm", tol=1e-2)


def test_bf16_structured_plus_layer_on_the_staged_mfma_kernels():
    announce("bf16 structured plus staged MFMA")
    torch.manual_seed(0)
    grid, dim, heads, S = (64, 64), 128, 4, 32
    ref = to.OraclePhysicsAttentionStructuredMesh2D(dim, grid, heads=heads, dim_head=32, slice_num=S, kernel=3, plus=True)
    hip = pn.PhysicsAttentionStructuredMesh2D(dim, grid, heads=heads, dim_head=32, slice_num=S, kernel=3, plus=True,
                                              use_te=False)
    hip.load_state_dict(ref.state_dict())
    ref.eval(), hip.eval().cuda()
    x = torch.randn(1, 4096, dim)
    u = torch.rand(1, 4096, heads, S).bfloat16()
    xb = x.cuda().bfloat16()
    assert PF.layer_forward_plus_supported(torch.bfloat16, hip.layer_dims(xb))
    with torch.no_grad():
        want = ref.forward_with_noise(x, u.float())
        got = hip.forward_with_noise(xb, u.cuda())
    assert_rel_l2(got, want, "bf16 structured plus y vs fp32 oracle", tol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_empty_inputs_give_empty_outputs(dtype):
    """No points, or an empty batch: the reference's tensor ops return the empty (B, N, C) tensor; so do the modules
    (nothing is launched)."""
    announce("empty inputs", dtype)
    layer = pn.PhysicsAttentionIrregularMesh(128, heads=4, dim_head=32, slice_num=16, use_te=False).eval().cuda()
    grid = pn.PhysicsAttentionStructuredMesh2D(128, (6, 5), heads=4, dim_head=32, slice_num=16, kernel=3,
                                               use_te=False).eval().cuda()
    ln = torch.nn.LayerNorm(128).cuda()
    with torch.no_grad():
        for shape in ((2, 0, 128), (0, 7, 128)):
            x = torch.empty(shape, dtype=dtype, device="cuda")
            y = layer(x)
            assert y.shape == shape and y.dtype == dtype
            fx, normed = layer.forward_block(x, torch.empty(shape, dtype=dtype, device="cuda"), ln)
            assert fx.shape == shape and normed.shape == shape
        y = grid(torch.empty((0, 30, 128), dtype=dtype, device="cuda"))
        assert y.shape == (0, 30, 128)
        with pytest.raises(RuntimeError):  # a token count that is not the grid's: the reference's view() fails too
            grid(torch.empty((2, 0, 128), dtype=dtype, device="cuda"))
        model = pn.Transolver(functional_dim=2, out_dim=3, embedding_dim=2, n_layers=2, n_hidden=64, n_head=2,
                              slice_num=8, use_te=False).eval().cuda().to(dtype)
        for shape in ((2, 0), (0, 9)):
            out = model(torch.empty(shape + (2,), dtype=dtype, device="cuda"),
                        torch.empty(shape + (2,), dtype=dtype, device="cuda"))
            assert out.shape == shape + (3,)
