"""Backward pass of the HIP layer against autograd over the fp32 oracle (the oracle's own gradient is pinned by
finite differences in test_oracle_closed_forms.py).  Bars: fp32 gradients rtol 1e-4 with atol = 1e-4 * max|ref|
per tensor; bf16 gradients rel-L2 <= 3e-2 against the fp32 reference gradients."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2, make_pair

pytestmark = pytest.mark.gpu


def _grads(module, x, probe):
    """Gradients of sum(module(x) * probe) w.r.t. x and every parameter."""
    module.zero_grad(set_to_none=True)
    x = x.clone().requires_grad_(True)
    y = module(x)
    (y.float() * probe.to(y.device)).sum().backward()
    out = {"x": x.grad}
    out.update({name: p.grad for name, p in module.named_parameters()})
    return y, out


CASES = [
    ("irregular", dict(dim=32, heads=4, dim_head=8, slice_num=8), 2, 300, None, 3),
    ("irregular", dict(dim=64, heads=2, dim_head=32, slice_num=64), 1, 1000, None, 3),
    ("irregular", dict(dim=48, heads=3, dim_head=16, slice_num=20), 3, 77, None, 3),
    ("structured2d", dict(dim=32, heads=4, dim_head=8, slice_num=8), 2, 63, (7, 9), 3),
    ("structured2d", dict(dim=16, heads=2, dim_head=8, slice_num=8), 1, 30, (5, 6), 5),
    ("structured3d", dict(dim=16, heads=2, dim_head=8, slice_num=8), 2, 60, (3, 4, 5), 3),
]


@pytest.mark.parametrize("variant,kw,B,N,grid,kernel", CASES)
def test_fp32_layer_gradients(variant, kw, B, N, grid, kernel):
    announce("fp32 backward", variant, kw, B, N, grid, kernel)
    heads = kw["heads"]
    temps = [0.3, 1.0, 2.5, 7.0][:heads] if heads <= 4 else None  # heads outside [0.5, 5] get zero temperature grad
    ref, hip = make_pair(variant, kw["dim"], heads, kw["dim_head"], kw["slice_num"], spatial=grid, kernel=kernel,
                         sharpen=2.0, temps=temps)
    ref.train(), hip.train()
    x = torch.randn(B, N, kw["dim"])
    probe = torch.randn(B, N, kw["dim"])
    y_ref, want = _grads(ref, x, probe)
    y_hip, got = _grads(hip, x.cuda(), probe)
    assert_fp32_close(y_hip, y_ref, "forward y (training path)")
    assert set(got) == set(want)
    for name in want:
        assert got[name] is not None and got[name].shape == want[name].shape, name
        assert_fp32_close(got[name], want[name], f"grad {name}", rtol=2e-4)
    if temps is not None:
        t = got["temperature"].flatten().cpu()
        assert t[0] == 0.0 and (heads < 4 or t[3] == 0.0)
        assert t[1] != 0.0


def test_slice_attention_backward_stage():
    announce("slice attention backward stage")
    B, H, S, D = 2, 3, 24, 16
    torch.manual_seed(3)
    tok = torch.randn(B, H, S, D)
    wqkv = torch.randn(3 * D, D) / D ** 0.5
    d_out = torch.randn(B, H, S, D)
    tok_r, w_r = tok.clone().requires_grad_(True), wqkv.clone().requires_grad_(True)
    q, k, v = (tok_r @ w_r.t()).chunk(3, dim=-1)
    out = torch.softmax(q @ k.transpose(-1, -2) / D ** 0.5, dim=-1) @ v
    (out * d_out).sum().backward()
    dims = PF.LayerDims(B, 100, H * D, H, D, S)
    params = {"qkv_project_weight": wqkv.cuda().contiguous()}
    d_tok, d_norm, d_w = PF.slice_attention_backward(tok.cuda(), None, d_out.cuda(), params, dims)
    assert d_norm is None
    assert_fp32_close(d_tok, tok_r.grad, "d slice_token")
    assert_fp32_close(d_w, w_r.grad, "d qkv weight")


def test_bf16_layer_gradients():
    announce("bf16 backward (autocast)")
    ref, hip = make_pair("irregular", 256, 8, 32, 64, sharpen=2.0)
    ref.train(), hip.train()
    torch.manual_seed(5)
    x = torch.randn(2, 2048, 256)
    probe = torch.randn(2, 2048, 256)
    _, want = _grads(ref, x, probe)
    hip.zero_grad(set_to_none=True)
    xc = x.cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip(xc)
    assert y.dtype == torch.bfloat16
    (y.float() * probe.cuda()).sum().backward()
    got = {"x": xc.grad}
    got.update({name: p.grad for name, p in hip.named_parameters()})
    for name in want:
        assert got[name].dtype == torch.float32 and torch.isfinite(got[name]).all(), name
        assert_rel_l2(got[name], want[name], f"bf16 grad {name}", tol=3e-2)


def test_model_training_step_matches_oracle():
    announce("Transolver training step fp32")
    torch.manual_seed(0)
    kw = dict(functional_dim=2, out_dim=3, embedding_dim=3, n_layers=2, n_hidden=32, n_head=4, slice_num=8, mlp_ratio=2)
    m = pn.Transolver(use_te=False, **kw).cuda().train()
    ref = to.OracleTransolver(**kw).train()
    ref.load_state_dict(m.state_dict())
    fx, emb, target = torch.randn(2, 200, 2), torch.randn(2, 200, 3), torch.randn(2, 200, 3)
    loss_ref = ((ref(fx, emb) - target) ** 2).mean()
    loss_ref.backward()
    loss = ((m(fx.cuda(), emb.cuda()) - target.cuda()) ** 2).mean()
    loss.backward()
    assert abs(float(loss.detach()) - float(loss_ref.detach())) <= 1e-4 * abs(float(loss_ref.detach()))
    want = dict(ref.named_parameters())
    for name, p in m.named_parameters():
        assert p.grad is not None, name
        assert_fp32_close(p.grad, want[name].grad, f"grad {name}", rtol=5e-4)
    # the same optimiser step on both sides leads to the same new loss
    torch.optim.SGD(m.parameters(), lr=0.01).step()
    torch.optim.SGD(ref.parameters(), lr=0.01).step()
    with torch.no_grad():
        loss2 = float(((m(fx.cuda(), emb.cuda()) - target.cuda()) ** 2).mean())
        loss2_ref = float(((ref(fx, emb) - target) ** 2).mean())
    assert abs(loss2 - loss2_ref) <= 1e-4 * abs(loss2_ref)
    assert loss2_ref >= float(loss_ref.detach()) or loss2 < float(loss.detach())


def test_gradients_reach_the_input_only_when_asked():
    announce("needs_input_grad handling")
    _, hip = make_pair("irregular", 32, 4, 8, 8)
    for p in hip.parameters():
        p.requires_grad_(False)
    x = torch.randn(1, 50, 32, device="cuda", requires_grad=True)
    hip(x).sum().backward()
    assert x.grad is not None and torch.isfinite(x.grad).all()
    assert all(p.grad is None for p in hip.parameters())


@pytest.mark.parametrize("B,N,C,S", [(2, 2048, 256, 64), (3, 1000, 128, 32), (1, 77, 128, 16), (2, 333, 256, 32),
                                     (2, 1500, 256, 128), (1, 999, 128, 128)])
def test_bf16_mfma_backward_matches_oracle_and_general_path(B, N, C, S):
    """Shapes the bf16 MFMA backward serves (ragged N, B > 1, every S <= 64): gradients against the fp32 oracle and
    against the general-kernel backward run on the same bf16 inputs."""
    announce("bf16 MFMA backward", B, N, C, S)
    from physicsnemo_amd import autograd as PA
    H = C // 32
    ref, hip = make_pair("irregular", C, H, 32, S, sharpen=2.0, temps=[0.3 + 0.4 * k for k in range(H)])
    ref.train(), hip.train()
    torch.manual_seed(9)
    x, probe = torch.randn(B, N, C), torch.randn(B, N, C)
    _, want = _grads(ref, x, probe)
    xb = x.cuda().bfloat16()
    dims = hip.layer_dims(xb)
    assert PF.mfma_backward_supported(torch.bfloat16, dims)

    def run(fn):
        hip.zero_grad(set_to_none=True)
        xc = xb.clone().requires_grad_(True)
        params = (hip.in_project_x.weight, hip.in_project_x.bias, hip.in_project_fx.weight, hip.in_project_fx.bias,
                  hip.in_project_slice.weight, hip.in_project_slice.bias, hip.temperature, hip.qkv_project.weight,
                  hip.out_linear.weight, hip.out_linear.bias)
        y = fn.apply(xc, dims, hip.kernel_params(torch.bfloat16, xc.device), *params)
        (y.float() * probe.cuda()).sum().backward()
        out = {"x": xc.grad.float()}
        out.update({name: p.grad.clone() for name, p in hip.named_parameters()})
        return out

    got = run(PA.PhysicsAttentionMfmaFunction)
    general = run(PA.PhysicsAttentionFunction)
    for name in want:
        assert torch.isfinite(got[name]).all(), name
        # d temperature is H scalars, each a sum of cancelling terms d l * logit over all points and slices; both
        # kernels keep sum_s d l = 0 per point (weights renormalised / softmax re-formed in float32), which holds it
        # to the bar of the tensor-valued gradients
        assert_rel_l2(got[name], want[name], f"MFMA bf16 grad {name} vs fp32 oracle", tol=3e-2)
        # two bf16 paths, each within 3e-2 of the oracle: their mutual distance may reach the sum for the H scalars
        assert_rel_l2(got[name], general[name], f"MFMA vs general bf16 grad {name}",
                      tol=6e-2 if name == "temperature" else 3e-2)
    t = got["temperature"].flatten().cpu()
    assert t[0] == 0.0  # 0.3 is below the clamp: no gradient


def test_mfma_deslice_natural_layout():
    announce("MFMA deslice to natural layout")
    ref, hip = make_pair("irregular", 256, 8, 32, 64, sharpen=2.0)
    x = torch.randn(2, 500, 256)
    xb = x.cuda().bfloat16()
    dims = hip.layer_dims(xb)
    with torch.no_grad():
        st = PF.MfmaStages(hip.kernel_params(torch.bfloat16, xb.device), dims, xb.device)
        st.pack_params()
        st.project_softmax_reduce(xb)
        st.combine_attention()
        out_x = st.deslice()
        stages = ref.stages(x)
        want = torch.einsum("bths,bhsd->bthd", stages["w"], stages["tok_out"]).reshape(2, 500, 256)
        assert_rel_l2(out_x, want, "out_x")
        # packed and natural outputs of the row GEMM agree: the packed copy feeds the slice sum, compare through it
        w = hip.out_linear.weight.detach().bfloat16().t().contiguous()  # any (256, 256) weight
        nat, pack = st.rows_gemm_packed(xb, w, None)
        assert_rel_l2(nat, x @ w.float().cpu().t(), "natural GEMM output")
        sums = st.slice_weighted_sum(pack)
        want_sums = torch.einsum("bnhs,bnhd->bhsd", stages["w"], (x @ w.float().cpu().t()).reshape(2, 500, 8, 32))
        assert_rel_l2(sums[..., :32], want_sums, "slice sums of the packed GEMM output")
        assert_rel_l2(sums[..., 32], stages["w"].sum(1), "slice counts")


@pytest.mark.parametrize("rows,ca,cb", [(5000, 64, 32), (1000, 256, 256), (333, 512, 256), (31, 32, 32), (70000, 256, 128)])
def test_cols_gemm_weight_gradient_product(rows, ca, cb):
    announce("cols_gemm", rows, ca, cb)
    torch.manual_seed(rows)
    a = torch.randn(rows, ca, device="cuda").bfloat16()
    b = torch.randn(rows, cb, device="cuda").bfloat16()
    assert PF.cols_gemm_supported(a, b)
    got, sums = PF.cols_gemm(a, b, col_sums=True)
    assert_fp32_close(sums, a.double().sum(0).float(), "column sums of a", rtol=1e-4)
    want = a.double().t() @ b.double()  # exact products of the bf16 inputs; the kernel accumulates them in fp32
    assert got.shape == (ca, cb) and got.dtype == torch.float32
    assert_fp32_close(got, want.float(), "a^T b", rtol=1e-4)
    assert torch.equal(got, PF.cols_gemm(a, b))  # fixed summation order


@pytest.mark.parametrize("rows,ca,cb", [(5000, 64, 32), (4099, 256, 256), (8192, 512, 132), (70001, 4, 260), (300000, 128, 256)])
def test_cols_gemm_float32(rows, ca, cb):
    announce("cols_gemm float32", rows, ca, cb)
    torch.manual_seed(rows)
    a = torch.randn(rows, ca, device="cuda") + 0.25
    b = torch.randn(rows, cb, device="cuda")
    assert PF.cols_gemm_supported(a, b)
    got, sums = PF.cols_gemm(a, b, col_sums=True)
    assert_fp32_close(sums, a.double().sum(0).float(), "column sums of a", rtol=1e-4)
    want = a.double().t() @ b.double()
    assert got.shape == (ca, cb) and got.dtype == torch.float32
    assert_fp32_close(got, want.float(), "a^T b", rtol=1e-4)
    assert torch.equal(got, PF.cols_gemm(a, b))  # fixed summation order


def test_bf16_model_training_step_runs_the_mfma_backward():
    announce("Transolver training step, bf16 autocast, MFMA backward inside the blocks")
    torch.manual_seed(1)
    kw = dict(functional_dim=3, out_dim=2, embedding_dim=2, n_layers=2, n_hidden=128, n_head=4, slice_num=32, mlp_ratio=2)
    m = pn.Transolver(use_te=False, **kw).cuda().train()
    ref = to.OracleTransolver(**kw).train()
    ref.load_state_dict(m.state_dict())
    fx, emb, target = torch.randn(2, 700, 3), torch.randn(2, 700, 2), torch.randn(2, 700, 2)
    ((ref(fx, emb) - target) ** 2).mean().backward()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = m(fx.cuda(), emb.cuda())
    ((out.float() - target.cuda()) ** 2).mean().backward()
    want = dict(ref.named_parameters())
    for name, p in m.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), name
        if "temperature" in name or want[name].grad.abs().max() < 1e-6:
            continue
        assert_rel_l2(p.grad, want[name].grad, f"bf16 model grad {name}", tol=8e-2)


def test_mfma_backward_at_scale_agrees_with_general_path():
    """200 000 points (more than any CPU-oracle case): the MFMA backward and the general backward, two independent
    implementations of the same gradient, agree on the same bf16 inputs; the input gradient is finite everywhere."""
    announce("MFMA vs general backward at 200k points")
    from physicsnemo_amd import autograd as PA
    _, hip = make_pair("irregular", 256, 8, 32, 64, sharpen=2.0)
    hip.train()
    torch.manual_seed(2)
    N = 200_000
    xb = torch.randn(1, N, 256, device="cuda").bfloat16()
    probe = torch.randn(1, N, 256, device="cuda").bfloat16()
    dims = hip.layer_dims(xb)
    params = (hip.in_project_x.weight, hip.in_project_x.bias, hip.in_project_fx.weight, hip.in_project_fx.bias,
              hip.in_project_slice.weight, hip.in_project_slice.bias, hip.temperature, hip.qkv_project.weight,
              hip.out_linear.weight, hip.out_linear.bias)
    res = []
    for fn in (PA.PhysicsAttentionMfmaFunction, PA.PhysicsAttentionFunction):
        hip.zero_grad(set_to_none=True)
        xc = xb.clone().requires_grad_(True)
        y = fn.apply(xc, dims, hip.kernel_params(torch.bfloat16, xc.device), *params)
        y.backward(probe)
        g = {"x": xc.grad.float()}
        g.update({n: p.grad.clone() for n, p in hip.named_parameters()})
        res.append(g)
    assert torch.isfinite(res[0]["x"]).all()
    for name in res[0]:
        if name != "temperature":
            assert_rel_l2(res[0][name], res[1][name], f"grad {name}", tol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,C", [(1000, 256), (37, 48), (4096, 512), (300, 1024)])
def test_layernorm_and_linear_autograd_functions(dtype, rows, C):
    announce("LayerNormFunction / LinearFunction", dtype, rows, C)
    from physicsnemo_amd import autograd as PA
    torch.manual_seed(rows)
    ln = torch.nn.LayerNorm(C)
    with torch.no_grad():
        ln.weight.uniform_(0.5, 1.5)
        ln.bias.uniform_(-0.5, 0.5)
    x, probe = torch.randn(2, rows, C), torch.randn(2, rows, C)
    xr = x.to(dtype).float().clone().requires_grad_(True)  # reference: fp32 arithmetic on the same (rounded) input
    (ln(xr) * probe).sum().backward()
    want = (xr.grad, ln.weight.grad.clone(), ln.bias.grad.clone())
    ln.zero_grad()
    lng = ln.cuda()
    xg = x.detach().to(dtype).cuda().requires_grad_(True)
    y = PA.layer_norm(xg, lng)
    assert y.dtype == dtype and y.grad_fn is not None
    (y.float() * probe.cuda()).sum().backward()
    got = (xg.grad, lng.weight.grad, lng.bias.grad)
    for name, g, w in zip(("dx", "d gamma", "d beta"), got, want):
        if dtype == torch.float32:
            assert_fp32_close(g, w, name, rtol=2e-4)
        else:
            assert_rel_l2(g, w, name, tol=1e-2)
    if dtype == torch.bfloat16:
        lin = torch.nn.Linear(C, 256)
        xr = x.detach().bfloat16().float().requires_grad_(True)
        p2 = torch.randn(2, rows, 256)
        (torch.nn.functional.linear(xr, lin.weight.bfloat16().float(), lin.bias) * p2).sum().backward()
        wx = xr.grad
        lin.zero_grad(set_to_none=True)  # the reference pass above left gradients on the parameters
        lin = lin.cuda()
        xg = x.detach().bfloat16().cuda().requires_grad_(True)
        out = PA.linear(xg, lin.weight, lin.bias)
        (out.float() * p2.cuda()).sum().backward()
        assert lin.weight.grad.dtype == torch.float32
        assert_rel_l2(xg.grad, wx, "linear dx", tol=1e-2)
        ref_dw = (p2.bfloat16().float().reshape(-1, 256).t() @ x.bfloat16().float().reshape(-1, C))
        assert_rel_l2(lin.weight.grad, ref_dw, "linear dW", tol=1e-2)
        assert_rel_l2(lin.bias.grad, p2.bfloat16().float().reshape(-1, 256).sum(0), "linear db", tol=1e-2)


def test_output_dropout_in_training_matches_the_reference_site():
    """The reference applies nn.Dropout to the layer output in training mode (physics_attention.py:499): kept entries
    are y / (1 - p), the rest zero, gradients flow through the kept entries only; eval mode is the identity."""
    announce("output dropout in training")
    torch.manual_seed(0)
    layer = pn.PhysicsAttentionIrregularMesh(64, heads=2, dim_head=32, dropout=0.25, slice_num=16, use_te=False).cuda()
    x = torch.randn(2, 2000, 64, device="cuda")
    layer.eval()
    with torch.no_grad():
        y_eval = layer(x)
    layer.train()
    xg = x.clone().requires_grad_(True)
    y = layer(xg)
    kept = y != 0
    frac = kept.float().mean().item()
    assert abs(frac - 0.75) < 0.01, frac
    assert_fp32_close(y[kept], (y_eval / 0.75)[kept], "kept entries")
    y.sum().backward()
    assert xg.grad is not None and torch.isfinite(xg.grad).all()
    blk = pn.TransolverBlock(2, 64, 0.25, mlp_ratio=2, slice_num=16, use_te=False).cuda().train()
    out = blk(x)
    assert out.shape == x.shape and torch.isfinite(out).all()
