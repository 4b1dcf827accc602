"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs and weights.

Bars: fp32 within rtol 1e-4 (atol = 1e-4 * max|ref|); bf16 within relative L2 error 1e-2 of the fp32 oracle.
"""
import os

import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2, make_pair

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
STAGES = ("x_mid", "fx_mid", "w", "tok", "norm", "tok_out", "y")


@pytest.mark.parametrize("B,N,dim,heads,dim_head,S", [
    (1, 100, 64, 4, 16, 4), (2, 500, 128, 8, 16, 16), (4, 1000, 256, 8, 32, 64), (2, 333, 96, 3, 32, 32),
    (1, 257, 64, 2, 64, 16), (2, 129, 128, 4, 16, 32),  # inner_dim != dim, as the reference layer tests allow
    (1, 1, 32, 2, 16, 8),  # single point: exposes the 1e-2 epsilon
])
def test_fp32_irregular_stages_and_layer(B, N, dim, heads, dim_head, S):
    announce("fp32 irregular", B, N, dim, heads, dim_head, S)
    ref, hip = make_pair("irregular", dim, heads, dim_head, S, sharpen=2.0,
                         temps=[0.3 + 5.7 * i / max(1, heads - 1) for i in range(heads)])
    x = torch.randn(B, N, dim)
    with torch.no_grad():
        want = ref.stages(x)
        got = hip.forward_stages(x.cuda())
        y = hip(x.cuda())
    for k in STAGES:
        assert_fp32_close(got[k], want[k], k)
    assert_fp32_close(y, want["y"], "layer y")
    assert y.shape == (B, N, dim) and y.dtype == torch.float32


@pytest.mark.parametrize("kernel,grid", [(1, (8, 8)), (3, (16, 16)), (3, (9, 14)), (5, (12, 7)), (7, (10, 10))])
def test_fp32_structured2d_stages_and_layer(kernel, grid):
    announce("fp32 structured2d", kernel, grid)
    B, dim, heads, dim_head, S = 2, 32, 4, 8, 16
    ref, hip = make_pair("structured2d", dim, heads, dim_head, S, spatial=grid, kernel=kernel, sharpen=2.0)
    x = torch.randn(B, grid[0] * grid[1], dim)
    with torch.no_grad():
        want = ref.stages(x)
        got = hip.forward_stages(x.cuda())
        y = hip(x.cuda())
    for k in STAGES:
        assert_fp32_close(got[k], want[k], k)
    assert_fp32_close(y, want["y"], "layer y")


@pytest.mark.parametrize("kernel,grid,B", [(1, (9, 14), 2), (3, (13, 11), 3), (3, (40, 37), 2), (5, (16, 23), 1),
                                           (3, (85, 85), 1)])
def test_fp32_structured2d_fused_front_end(kernel, grid, B):
    # C = 128, 8 heads of 16, 32 slices: the layer call runs the fused front end (both convolutions as split-bf16 MFMA
    # products, slice softmax and partial token sums in one launch); the stage API runs the float32-MFMA kernels.
    # Grids with ragged last tiles (126, 143 points), workgroups with idle waves (143 points: 5 tiles) and cfg1's grid.
    announce("fp32 structured2d fused front end", kernel, grid, B)
    dim, heads, dim_head, S = 128, 8, 16, 32
    ref, hip = make_pair("structured2d", dim, heads, dim_head, S, spatial=grid, kernel=kernel, sharpen=2.0,
                         temps=[0.3 + 5.7 * i / 7 for i in range(8)])
    x = torch.randn(B, grid[0] * grid[1], dim)
    with torch.no_grad():
        want = ref.stages(x)
        want64 = ref.double().stages(x.double())["y"]
        staged = hip.forward_stages(x.cuda())["y"]
        y = hip(x.cuda())
    assert_fp32_close(y, want["y"], "layer y")
    # against the float64 run of the oracle the split products are as close as the float32 matrix instructions
    e_fused, e_staged = to.rel_l2(y.double().cpu(), want64), to.rel_l2(staged.double().cpu(), want64)
    import conftest

    conftest.MEASURED.append((f"structured 2D fp32 layer vs float64 oracle, k={kernel} grid={grid}: fused front end "
                              f"(split-bf16 products); stage kernels (fp32 MFMA) {e_staged:.2e}", e_fused, 2e-6))
    assert e_fused < 2e-6 and e_fused < 4 * e_staged + 2e-7


@pytest.mark.parametrize("B,N", [(2, 500), (1, 33), (3, 4100)])
def test_fp32_irregular_row_kernel_back_end(B, N):
    # C = 128, 8 heads of 16, 32 slices, irregular mesh: the layer call runs the fused front end (Linear projections as
    # its 1 x 1 case) and hands back to the points, applies out_linear and the block tail in the float32 row kernel
    announce("fp32 irregular, row-kernel back end", B, N)
    dim, heads, dim_head, S = 128, 8, 16, 32
    ref, hip = make_pair("irregular", dim, heads, dim_head, S, sharpen=2.0, temps=[0.3 + 5.7 * i / 7 for i in range(8)])
    ln = torch.nn.LayerNorm(dim)
    with torch.no_grad():
        ln.weight.add_(0.2 * torch.randn(dim))
        ln.bias.add_(0.2 * torch.randn(dim))
    x, res = torch.randn(B, N, dim), torch.randn(B, N, dim)
    with torch.no_grad():
        want = ref(x)
        want_fx = want + res
        want_ln = ln(want_fx)
        y = hip(x.cuda())
        fx, normed = hip.forward_block(x.cuda(), res.cuda(), ln.cuda())
    assert_fp32_close(y, want, "layer y")
    assert_fp32_close(fx, want_fx, "fx_new")
    assert_fp32_close(normed, want_ln, "LayerNorm(fx_new)")


@pytest.mark.parametrize("spatial,B,mlp_ratio,last", [(None, 2, 1, False), ((13, 11), 3, 4, False), ((85, 85), 1, 1, True),
                                                      (None, 1, 2, True)])
def test_fp32_whole_block_in_one_call(spatial, B, mlp_ratio, last):
    # hidden 128, 8 heads of 16, 32 slices: TransolverBlock.forward runs pa_block_forward (front end, combine + slice
    # attention, then hand-back, out_linear, both residuals, the MLP and the LayerNorms in one launch); irregular and
    # structured layers, ragged tiles, several chunks of hidden features, the last block with its output head
    announce("fp32 whole block", spatial, B, mlp_ratio, last)
    torch.manual_seed(3)
    kw = dict(mlp_ratio=mlp_ratio, last_layer=last, out_dim=3, slice_num=32, spatial_shape=spatial)
    ref = to.OracleTransolverBlock(8, 128, **kw).eval()
    hip = pn.TransolverBlock(8, 128, 0.0, use_te=False, **kw).eval()
    with torch.no_grad():
        for ln in (ref.ln_1, ref.ln_mlp1[0]):
            ln.weight.add_(0.2 * torch.randn(128))
            ln.bias.add_(0.2 * torch.randn(128))
        ref.Attn.in_project_slice.weight.mul_(2.0)
    hip.load_state_dict(ref.state_dict())
    hip = hip.cuda()
    N = 333 if spatial is None else spatial[0] * spatial[1]
    fx = torch.randn(B, N, 128)
    calls = []
    orig = PF.block_forward
    PF.block_forward = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        with torch.no_grad():
            want = ref(fx)
            got = hip(fx.cuda())
    finally:
        PF.block_forward = orig
    assert calls, "the whole-block entry point did not run"
    assert_fp32_close(got, want, "block output")
    if last:  # the output head inside the same call (what the model's last block runs)
        with torch.no_grad():
            xc = fx.cuda()
            whole = hip._whole_block(hip.ln_1(xc), xc, hip.ln_mlp2[0], head=hip.ln_mlp2[1])
        assert whole is not None
        assert_fp32_close(whole[1], want, "block output, head in the call")


def test_fp32_fused_path_is_bit_reproducible():
    # the float32 kernels stream weights and rows through LDS rings with asynchronous loads and reduce the token sums
    # in a fixed order: repeated calls on the same inputs must agree to the bit (a race would show up here first);
    # model, block and layer level, cfg1's shape
    announce("fp32 fused path: run-to-run bit equality")
    torch.manual_seed(5)
    m = pn.Transolver(functional_dim=1, embedding_dim=2, out_dim=1, n_layers=4, n_hidden=128, n_head=8, mlp_ratio=1,
                      slice_num=32, structured_shape=(85, 85), unified_pos=False, use_te=False).eval().cuda()
    lin = torch.linspace(0, 1, 85)
    pos = torch.stack(torch.meshgrid(lin, lin, indexing="ij"), -1).reshape(1, 7225, 2).repeat(4, 1, 1).cuda()
    fx = torch.randn(4, 7225, 1).cuda()
    x = torch.randn(4, 7225, 128).cuda()
    with torch.no_grad():
        first = (m(fx, pos), m.blocks[1](x), m.blocks[1].Attn(x))
        for _ in range(5):
            again = (m(fx, pos), m.blocks[1](x), m.blocks[1].Attn(x))
            for a, b in zip(first, again):
                assert torch.equal(a, b)


@pytest.mark.parametrize("kernel,grid", [(3, (4, 4, 4)), (3, (8, 8, 8)), (5, (8, 8, 8)), (3, (3, 5, 7)), (1, (4, 6, 5))])
def test_fp32_structured3d_stages_and_layer(kernel, grid):
    announce("fp32 structured3d", kernel, grid)
    B, dim, heads, dim_head, S = 2, 32, 4, 8, 8
    ref, hip = make_pair("structured3d", dim, heads, dim_head, S, spatial=grid, kernel=kernel, sharpen=2.0)
    x = torch.randn(B, grid[0] * grid[1] * grid[2], dim)
    with torch.no_grad():
        want = ref.stages(x)
        got = hip.forward_stages(x.cuda())
        y = hip(x.cuda())
        yb = hip(x.cuda().bfloat16())
    for k in STAGES:
        assert_fp32_close(got[k], want[k], k)
    assert_fp32_close(y, want["y"], "layer y")
    assert_rel_l2(yb, want["y"], "bf16 layer y", tol=2e-2)
    with pytest.raises(RuntimeError):
        hip(x.cuda()[:, :-1])  # the token count must match the grid, as in the reference's view()


def test_structured3d_model_flatten_equivalence():
    announce("structured3d model: (B, H, W, D, C) input == flattened input")
    torch.manual_seed(0)
    grid = (6, 5, 4)
    m = pn.Transolver(functional_dim=2, out_dim=3, embedding_dim=3, structured_shape=grid, n_layers=2, n_hidden=32,
                      n_head=4, slice_num=8, mlp_ratio=2, use_te=False).eval().cuda()
    ref = to.OracleTransolver(functional_dim=2, out_dim=3, embedding_dim=3, structured_shape=grid, n_layers=2, n_hidden=32,
                              n_head=4, slice_num=8, mlp_ratio=2).eval()
    ref.load_state_dict(m.state_dict())
    fx, emb = torch.randn(2, *grid, 2), torch.randn(2, *grid, 3)
    with torch.no_grad():
        out5 = m(fx.cuda(), emb.cuda())
        outf = m(fx.reshape(2, -1, 2).cuda(), emb.reshape(2, -1, 3).cuda())
        want = ref(fx, emb)
    assert out5.shape == (2, *grid, 3)
    assert torch.equal(out5.reshape(2, -1, 3), outf)
    assert_fp32_close(out5, want, "structured3d model")


def test_fp32_block_tail_residual_and_layernorm():
    announce("fp32 block tail")
    B, N, dim, heads, S = 2, 300, 128, 8, 32
    ref, hip = make_pair("irregular", dim, heads, dim // heads, S)
    ln = torch.nn.LayerNorm(dim)
    with torch.no_grad():
        ln.weight.add_(0.2 * torch.randn(dim))
        ln.bias.add_(0.2 * torch.randn(dim))
    x, res = torch.randn(B, N, dim), torch.randn(B, N, dim)
    with torch.no_grad():
        want_fx = ref(x) + res
        want_ln = ln(want_fx)
        fx, normed = hip.forward_block(x.cuda(), res.cuda(), ln.cuda())
    assert_fp32_close(fx, want_fx, "fx_new")
    assert_fp32_close(normed, want_ln, "LayerNorm(fx_new)")


def test_fp32_closed_form_zero_slice_projection():
    # w = 1/S everywhere -> every point gets Wout tile_H(Wv sum_n fx_mid / (N + 0.01 S)) + bout
    announce("fp32 closed form")
    B, N, C, H, D, S = 2, 77, 64, 4, 16, 8
    ref, hip = make_pair("irregular", C, H, D, S)
    with torch.no_grad():
        for m in (ref, hip):
            m.in_project_slice.weight.zero_()
            m.in_project_slice.bias.zero_()
    x = torch.randn(B, N, C)
    sd = {k: v.double() for k, v in ref.state_dict().items()}
    fm = x.double() @ sd["in_project_fx.weight"].T + sd["in_project_fx.bias"]
    tok = (fm.sum(1) / (N + 0.01 * S)).reshape(B, H, D)
    o = torch.einsum("bhd,ed->bhe", tok, sd["qkv_project.weight"][2 * D:]).reshape(B, H * D)
    want = (o @ sd["out_linear.weight"].T + sd["out_linear.bias"])[:, None, :].expand(B, N, C)
    with torch.no_grad():
        y = hip(x.cuda())
    assert_fp32_close(y, want.float(), "closed form")


def test_bf16_layer_against_fp32_oracle():
    announce("bf16 general shapes")
    for (B, N, dim, heads, dim_head, S) in [(2, 1000, 128, 8, 16, 32), (1, 515, 64, 2, 32, 4)]:
        ref, hip = make_pair("irregular", dim, heads, dim_head, S)
        x = torch.randn(B, N, dim)
        with torch.no_grad():
            want = ref(x)
            y = hip(x.cuda().bfloat16())
        assert y.dtype == torch.bfloat16
        assert_rel_l2(y, want, f"bf16 y {B, N, dim, heads, dim_head, S}")


def test_autocast_bf16_and_errors_on_gpu():
    announce("autocast + error paths")
    ref, hip = make_pair("irregular", 64, 4, 16, 8)
    x = torch.randn(2, 200, 64)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip(x.cuda())
    assert y.dtype == torch.bfloat16
    with torch.no_grad():
        assert_rel_l2(y, ref(x), "autocast y")
    y_grad = hip(x.cuda())  # grad enabled, parameters require grad: the differentiable path
    assert y_grad.requires_grad and y_grad.grad_fn is not None
    assert_fp32_close(y_grad, ref(x), "differentiable-path y")
    hip.use_fp8_weights(True)
    with pytest.raises(RuntimeError, match="no gradients"):
        hip(x.cuda().bfloat16())
    hip.use_fp8_weights(False)
    with torch.no_grad(), pytest.raises(ValueError, match="Expected 3D input"):
        hip(x.cuda()[0])
    _, hip2 = make_pair("structured2d", 16, 2, 8, 4, spatial=(4, 4))
    with torch.no_grad(), pytest.raises(RuntimeError):
        hip2(torch.randn(1, 15, 16).cuda())  # 15 tokens cannot be viewed as a 4 x 4 grid


def test_run_to_run_determinism():
    announce("determinism")
    ref, hip = make_pair("irregular", 128, 8, 16, 32)
    x = torch.randn(2, 5000, 128).cuda()
    with torch.no_grad():
        a = hip(x)
        for _ in range(5):
            assert torch.equal(hip(x), a)


def _golden_model(kind):
    torch.manual_seed(0)
    if kind == "2d":
        kw = dict(structured_shape=(85, 85), n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1, functional_dim=1,
                  out_dim=1, slice_num=32, ref=1, unified_pos=True)
        ref = to.OracleTransolver(init="rejection", **kw)
        args = (torch.randn(4, 85 * 85, 1), torch.randn(4, 85, 85))
        gold, atol = "transolver2d_output.pth", 2e-3
    else:
        kw = dict(structured_shape=None, n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1, functional_dim=2,
                  embedding_dim=3, out_dim=1, slice_num=32, unified_pos=False)
        ref = to.OracleTransolver(init="rejection", **kw)
        args = (torch.randn(4, 12345, 3), torch.randn(4, 12345, 2))
        gold, atol = "transolver_irregular_output.pth", 1e-3
    hip = pn.Transolver(use_te=False, **kw)
    hip.load_state_dict(ref.state_dict())
    return hip.cuda().eval(), args, torch.load(os.path.join(GOLD, gold), weights_only=True)[0], atol


@pytest.mark.parametrize("kind", ["2d", "irregular"])
def test_full_model_reproduces_reference_golden_output(kind):
    # the reference's own non-regression vectors (test/models/transolver/test_transolver.py:97-169), its tolerances
    announce("golden", kind)
    hip, args, gold, atol = _golden_model(kind)
    with torch.no_grad():
        out = hip(*[a.cuda() for a in args]).cpu()
    assert out.shape == gold.shape
    assert torch.allclose(out, gold, rtol=1e-3, atol=atol), float((out - gold).abs().max())
    assert float((out - gold).abs().max()) < 1e-4


def test_model_flatten_equivalence_on_gpu():
    announce("flatten equivalence")
    torch.manual_seed(0)
    m = pn.Transolver(functional_dim=3, out_dim=2, embedding_dim=4, structured_shape=(16, 16), n_layers=2,
                      n_hidden=32, n_head=4, slice_num=8, use_te=False).cuda().eval()
    fx, emb = torch.randn(2, 16, 16, 3).cuda(), torch.randn(2, 16, 16, 4).cuda()
    with torch.no_grad():
        a = m(fx, embedding=emb)
        b = m(fx.reshape(2, -1, 3), embedding=emb.reshape(2, -1, 4))
    assert a.shape == (2, 16, 16, 2)
    assert torch.allclose(a.reshape(2, -1, 2), b, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,C", [(1000, 512), (37, 48), (5000, 256), (300, 1024), (64, 36)])
def test_residual_layernorm_entry_point(dtype, rows, C):
    announce("pa_residual_layernorm", dtype, rows, C)
    from physicsnemo_amd import functional as PF
    torch.manual_seed(rows + C)
    y, res = torch.randn(rows, C), torch.randn(rows, C)
    gamma, beta = torch.rand(C) + 0.5, torch.randn(C)
    yq, rq = y.to(dtype), res.to(dtype)
    want_sum = (yq.float() + rq.float()).to(dtype).float()  # the sum is stored in the activation type first
    want_ln = torch.nn.functional.layer_norm(want_sum, (C,), gamma, beta, 1e-5)
    got_sum, got_ln = PF.residual_layernorm(yq.cuda().clone(), residual=rq.cuda(), ln_weight=gamma.cuda(),
                                            ln_bias=beta.cuda(), ln_eps=1e-5)
    assert torch.equal(got_sum.float().cpu(), want_sum)
    if dtype == torch.float32:
        assert_fp32_close(got_ln, want_ln, "LayerNorm(y + residual)")
    else:
        assert_rel_l2(got_ln, want_ln, "LayerNorm(y + residual)", tol=5e-3)
    only_ln = PF.residual_layernorm(yq.cuda().clone(), ln_weight=gamma.cuda(), ln_bias=beta.cuda())[1]
    want = torch.nn.functional.layer_norm(yq.float(), (C,), gamma, beta, 1e-5)
    (assert_fp32_close if dtype == torch.float32 else assert_rel_l2)(only_ln, want, "LayerNorm(y)")
    only_sum = PF.residual_layernorm(yq.cuda().clone(), residual=rq.cuda())
    assert torch.equal(only_sum.float().cpu(), want_sum)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,N,cin,cout,grid,k", [
    (2, 300, 64, 96, None, 0), (1, 5000, 256, 256, None, 0), (1, 6000, 512, 256, None, 0), (3, 50, 20, 7, None, 0),
    (2, 63, 32, 48, (7, 9), 3), (1, 60, 16, 40, (3, 4, 5), 3), (1, 30, 12, 8, (5, 6), 5),
])
def test_rows_gemm_entry_point(dtype, B, N, cin, cout, grid, k):
    # every kernel behind pa_rows_gemm: scalar FMA (odd widths), fp32 / bf16 MFMA tiles, weights-stationary bf16 Linear
    announce("pa_rows_gemm", dtype, B, N, cin, cout, grid, k)
    from physicsnemo_amd import functional as PF
    torch.manual_seed(N + cin)
    x = torch.randn(B, N, cin).to(dtype)
    bias = torch.randn(cout)
    if grid is None:
        w = (torch.randn(cout, cin) / cin ** 0.5).to(dtype)
        want = x.float() @ w.float().t() + bias
        dims = PF.LayerDims(B, N, cin, 1, 1, 1)
    else:
        w = (torch.randn(cout, cin, *([k] * len(grid))) / (cin * k ** len(grid)) ** 0.5).to(dtype)
        img = x.float().reshape(B, *grid, cin).movedim(-1, 1)
        conv = torch.nn.functional.conv2d if len(grid) == 2 else torch.nn.functional.conv3d
        want = conv(img, w.float(), bias, padding=k // 2).flatten(2).transpose(1, 2)
        dims = PF.LayerDims(B, N, cin, 1, 1, 1, grid[0], grid[1], k, grid[2] if len(grid) == 3 else 0)
    got = PF.rows_gemm(x.cuda(), w.cuda().contiguous(), bias.cuda(), dims, cin, cout)
    assert got.shape == (B, N, cout) and got.dtype == dtype
    if dtype == torch.float32:
        assert_fp32_close(got, want, "rows gemm")
    else:
        assert_rel_l2(got, want, "rows gemm", tol=5e-3)


def test_time_input_model_forward():
    announce("Transolver with time_input")
    torch.manual_seed(0)
    kw = dict(functional_dim=2, out_dim=3, embedding_dim=3, n_layers=2, n_hidden=64, n_head=4, slice_num=8, mlp_ratio=2)
    m = pn.Transolver(time_input=True, use_te=False, **kw).eval().cuda()
    ref = to.OracleTransolver(time_input=True, **kw).eval()
    ref.load_state_dict(m.state_dict())
    fx, emb, t = torch.randn(3, 150, 2), torch.randn(3, 150, 3), torch.tensor([0.0, 12.5, 400.0])
    with torch.no_grad():
        want = ref(fx, emb, time=t)
        got = m(fx.cuda(), emb.cuda(), time=t.cuda())
        assert_fp32_close(got, want, "model with time")
        assert not torch.allclose(got.cpu(), ref(fx, emb), atol=1e-3)  # the time input matters
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got16 = m(fx.cuda(), emb.cuda(), time=t.cuda())
        assert_rel_l2(got16, want, "model with time, bf16 autocast", tol=3e-2)


def test_fp16_autocast_is_served_and_memory_does_not_grow():
    """The reference's optimisation smoke tests run AMP with float16 on GPUs, and its layer tests bound the memory
    growth over repeated forwards (test_physics_attention.py:745-781): both must hold for the drop-in."""
    announce("fp16 autocast + memory growth")
    ref, hip = make_pair("irregular", 64, 4, 16, 8)
    x = torch.randn(2, 300, 64)
    with torch.no_grad():
        want = ref(x)
        with torch.autocast("cuda", dtype=torch.float16):
            y = hip(x.cuda())
        assert y.dtype == torch.float16
        assert_rel_l2(y, want, "fp16 autocast y", tol=2e-3)
        assert hip(x.cuda().half()).dtype == torch.float16
    torch.manual_seed(0)
    m = pn.Transolver(functional_dim=2, out_dim=1, embedding_dim=2, n_layers=2, n_hidden=64, n_head=4, slice_num=8,
                      mlp_ratio=2, use_te=False).eval().cuda()
    o = to.OracleTransolver(functional_dim=2, out_dim=1, embedding_dim=2, n_layers=2, n_hidden=64, n_head=4, slice_num=8,
                            mlp_ratio=2).eval()
    o.load_state_dict(m.state_dict())
    fx, emb = torch.randn(2, 300, 2), torch.randn(2, 300, 2)
    with torch.no_grad():
        with torch.autocast("cuda", dtype=torch.float16):
            out = m(fx.cuda(), emb.cuda())
        assert_rel_l2(out, o(fx, emb), "fp16 autocast model", tol=1e-2)
        xb = x.cuda()
        for _ in range(3):
            hip(xb)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        for _ in range(10):
            hip(xb)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() - before < 1 << 20
