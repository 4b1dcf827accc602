"""FLARE attention layer on the HIP kernels against the oracle (and autograd over it).  Bars: fp32 rtol 1e-4 (gradients
2e-4) with atol = rtol * max|ref|; bf16 output rel-L2 <= 1e-2, bf16 gradients <= 5e-2 against the fp32 oracle."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _pair(dim, heads, dim_head, S, seed=0):
    torch.manual_seed(seed)
    ref = to.OracleFLARE(dim, heads=heads, dim_head=dim_head, n_global_queries=S)
    hip = pn.FLARE(dim, heads=heads, dim_head=dim_head, n_global_queries=S)
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


@pytest.mark.parametrize("dim,heads,dim_head,S,B,N", [
    (32, 4, 8, 8, 2, 300),
    (64, 2, 32, 64, 1, 1000),
    (48, 3, 16, 20, 3, 77),
    (24, 2, 8, 5, 2, 1),       # one point: both softmaxes degenerate on the point axis
    (32, 4, 8, 1, 2, 515),     # one global query
])
def test_fp32_flare_matches_oracle(dim, heads, dim_head, S, B, N):
    announce("fp32 FLARE", dim, heads, dim_head, S, B, N)
    ref, hip = _pair(dim, heads, dim_head, S)
    x = torch.randn(B, N, dim)
    with torch.no_grad():
        want = ref(x)
        got = hip(x.cuda())
    assert got.shape == want.shape
    assert_fp32_close(got, want, "FLARE y")


def test_flare_stages_against_closed_forms():
    announce("FLARE stage kernels")
    B, N, H, S = 2, 700, 3, 20
    dims = PF.LayerDims(B, N, 48, H, 16, S)
    a = torch.randn(B, N, H, S, device="cuda") * 3
    w, colmax = PF.flare_column_weights(a, dims)
    want_max = a.amax(dim=1)
    assert torch.equal(colmax, want_max)
    assert_fp32_close(w, torch.exp(a - want_max[:, None]), "exp(A - column max)")
    rows = PF.flare_softmax_rows_(a.clone(), dims)
    assert_fp32_close(rows, torch.softmax(a, dim=-1), "row softmax")


@pytest.mark.parametrize("S,N", [(64, 8192), (32, 5000)])
def test_bf16_flare(S, N):
    announce("bf16 FLARE", S, N)
    ref, hip = _pair(256, 8, 32, S)
    x = torch.randn(2, N, 256)
    with torch.no_grad():
        want = ref(x)
        got = hip(x.cuda().bfloat16())
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got_ac = hip(x.cuda())
    assert got.dtype == torch.bfloat16 and got_ac.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 FLARE y", tol=1e-2)
    assert torch.equal(got, got_ac)


def test_flare_errors():
    announce("FLARE errors")
    _, hip = _pair(32, 4, 8, 8)
    x = torch.randn(2, 50, 32, device="cuda")
    with pytest.raises(ValueError, match="Expected 3D input tensor"), torch.no_grad():
        hip(x[0])
    with pytest.raises(ValueError, match="feature dimension"), torch.no_grad():
        hip(x[..., :16])
    with pytest.raises(RuntimeError, match="GPU"), torch.no_grad():
        hip.cpu()(x.cpu())


def _flare_grads(module, x, probe):
    module.zero_grad(set_to_none=True)
    x = x.clone().requires_grad_(True)
    y = module(x)
    (y.float() * probe.to(y.device)).sum().backward()
    out = {"x": x.grad}
    out.update({name: p.grad for name, p in module.named_parameters()})
    return y, out


@pytest.mark.parametrize("dim,heads,dim_head,S,B,N", [(32, 4, 8, 8, 2, 300), (64, 2, 32, 64, 1, 1000), (48, 3, 16, 20, 3, 77)])
def test_fp32_flare_gradients(dim, heads, dim_head, S, B, N):
    announce("fp32 FLARE backward", dim, heads, dim_head, S, B, N)
    ref, hip = _pair(dim, heads, dim_head, S)
    ref.train(), hip.train()
    x, probe = torch.randn(B, N, dim), torch.randn(B, N, dim)
    y_ref, want = _flare_grads(ref, x, probe)
    y_hip, got = _flare_grads(hip, x.cuda(), probe)
    assert_fp32_close(y_hip, y_ref, "forward y (training path)")
    assert set(got) == set(want)
    for name in want:
        assert got[name] is not None and got[name].shape == want[name].shape, name
        assert_fp32_close(got[name], want[name], f"grad {name}", rtol=2e-4)


def test_bf16_flare_gradients():
    announce("bf16 FLARE backward (autocast)")
    ref, hip = _pair(256, 8, 32, 64)
    ref.train(), hip.train()
    torch.manual_seed(5)
    x, probe = torch.randn(2, 2048, 256), torch.randn(2, 2048, 256)
    _, want = _flare_grads(ref, x, probe)
    hip.zero_grad(set_to_none=True)
    xc = x.cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip(xc)
    assert y.dtype == torch.bfloat16
    (y.float() * probe.cuda()).sum().backward()
    got = {"x": xc.grad}
    got.update({name: p.grad for name, p in hip.named_parameters()})
    for name in want:
        assert got[name] is not None and torch.isfinite(got[name]).all(), name
        assert_rel_l2(got[name], want[name], f"bf16 FLARE grad {name}", tol=5e-2)


@pytest.mark.parametrize("dim,heads,S,B,N", [(256, 8, 64, 1, 5000), (128, 4, 16, 3, 1777), (256, 8, 32, 2, 4096),
                                             (256, 8, 128, 1, 4097), (128, 4, 64, 2, 2500)])
def test_bf16_flare_on_the_mfma_kernels(dim, heads, S, B, N):
    """The whole FLARE layer on the bf16 MFMA kernels: against the fp32 oracle and against the general kernels on the
    same bf16 input; with the block tail."""
    from physicsnemo_amd import functional as PF

    announce("bf16 FLARE MFMA", dim, heads, S, B, N)
    torch.manual_seed(S + B)
    kw = dict(heads=heads, dim_head=32, n_global_queries=S)
    ref, hip = to.OracleFLARE(dim, **kw).eval(), pn.FLARE(dim, **kw).eval()
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    x = torch.randn(B, N, dim)
    xb = x.cuda().bfloat16()
    assert PF.flare_forward_mfma_supported(torch.bfloat16, PF.LayerDims(B, N, dim, heads, 32, S))
    with torch.no_grad():
        want = ref(x)
        got = hip(xb)
        hip.use_mfma = False
        general = hip(xb)
        hip.use_mfma = True
        ln = torch.nn.LayerNorm(dim).cuda()
        res = torch.randn(B, N, dim, device="cuda").bfloat16()
        fx_new, normed = hip.forward_block(xb, res, ln)
    assert got.dtype == torch.bfloat16 and torch.isfinite(got.float()).all()
    assert_rel_l2(got, want, "bf16 FLARE y (MFMA) vs fp32 oracle", tol=1e-2)
    assert_rel_l2(got, general, "bf16 FLARE y: MFMA vs general kernels", tol=1e-2)
    tail = got.float() + res.float()
    assert_rel_l2(fx_new, tail, "fx_new", tol=1e-2)
    assert_rel_l2(normed, torch.nn.functional.layer_norm(tail, (dim,), ln.weight, ln.bias, ln.eps), "LayerNorm", tol=1e-2)


@pytest.mark.parametrize("mode,dim,heads,dim_head,S,B,N,Sc,Dc", [
    ("weighted", 32, 4, 8, 8, 2, 300, 5, 7),
    ("concat_project", 48, 3, 16, 20, 3, 77, 9, 4),
    ("weighted", 64, 2, 32, 64, 1, 1000, 1, 16),
])
def test_fp32_gale_fa_matches_oracle(mode, dim, heads, dim_head, S, B, N, Sc, Dc):
    announce("fp32 GALE_FA", mode, dim, heads, dim_head, S, B, N, Sc, Dc)
    torch.manual_seed(0)
    kw = dict(heads=heads, dim_head=dim_head, n_global_queries=S, context_dim=Dc, state_mixing_mode=mode)
    ref, hip = to.OracleGALE_FA(dim, **kw).eval(), pn.GALE_FA(dim, **kw).eval()
    if mode == "weighted":
        with torch.no_grad():
            ref.state_mixing.fill_(0.3)
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    x1, x2, ctx = torch.randn(B, N, dim), torch.randn(B, N, dim), torch.randn(B, heads, Sc, Dc)
    with torch.no_grad():
        want = ref((x1, x2), ctx)
        got = hip((x1.cuda(), x2.cuda()), ctx.cuda())
        for g, w in zip(got, want):
            assert_fp32_close(g, w, "GALE_FA y")
        assert_fp32_close(hip((x1.cuda(),))[0], ref((x1,))[0], "GALE_FA y without context")


def test_bf16_gale_fa():
    announce("bf16 GALE_FA")
    torch.manual_seed(0)
    kw = dict(heads=8, dim_head=32, n_global_queries=64, context_dim=32)
    ref, hip = to.OracleGALE_FA(256, **kw).eval(), pn.GALE_FA(256, **kw).eval()
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    x, ctx = torch.randn(2, 4096, 256), torch.randn(2, 8, 48, 32)
    with torch.no_grad():
        want = ref((x,), ctx)[0]
        got = hip((x.cuda().bfloat16(),), ctx.cuda())[0]
    assert got.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 GALE_FA y", tol=1e-2)


@pytest.mark.parametrize("mode,dim,heads,dim_head,S,B,N,Sc,Dc,with_ctx", [
    ("weighted", 32, 4, 8, 8, 2, 300, 5, 7, True),
    ("concat_project", 48, 3, 16, 20, 3, 77, 9, 4, True),
    ("weighted", 64, 2, 32, 64, 1, 1000, 1, 16, True),
    ("weighted", 64, 2, 32, 16, 2, 500, 6, 16, False),
])
def test_fp32_gale_fa_gradients_match_autograd_over_the_oracle(mode, dim, heads, dim_head, S, B, N, Sc, Dc, with_ctx):
    announce("fp32 GALE_FA gradients", mode, dim, heads, dim_head, S, B, N, Sc, Dc, with_ctx)
    torch.manual_seed(1)
    kw = dict(heads=heads, dim_head=dim_head, n_global_queries=S, context_dim=Dc, state_mixing_mode=mode)
    ref, hip = to.OracleGALE_FA(dim, **kw).train(), pn.GALE_FA(dim, **kw).train()
    if mode == "weighted":
        with torch.no_grad():
            ref.state_mixing.fill_(-0.4)
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    x, ctx, dy = torch.randn(B, N, dim), torch.randn(B, heads, Sc, Dc), torch.randn(B, N, dim)
    xr, cr = x.clone().requires_grad_(), ctx.clone().requires_grad_()
    xh, ch = x.clone().cuda().requires_grad_(), ctx.clone().cuda().requires_grad_()
    yr = ref((xr,), cr if with_ctx else None)[0]
    yh = hip((xh,), ch if with_ctx else None)[0]
    assert_fp32_close(yh, yr, "GALE_FA y (training path)")
    yr.backward(dy)
    yh.backward(dy.cuda())
    assert_fp32_close(xh.grad, xr.grad, "d x", rtol=5e-4)
    if with_ctx:
        assert_fp32_close(ch.grad, cr.grad, "d context", rtol=5e-4)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if p.grad is None:
            assert grads[name].grad is None, name  # the cross-attention parameters without a context
            continue
        if name == "cross_k.bias":
            continue  # zero in exact arithmetic: a shift of all keys leaves the softmax unchanged
        if Sc == 1 and name.startswith(("cross_q", "cross_k")):
            assert float(grads[name].grad.abs().max()) < 1e-4  # one context token: its softmax weight is 1 whatever q, k
            continue
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=5e-4)


def test_bf16_gale_fa_gradients_and_geotransolver_training_with_gale_fa():
    announce("bf16 GALE_FA gradients")
    torch.manual_seed(2)
    kw = dict(heads=8, dim_head=32, n_global_queries=32, context_dim=32)
    ref, hip = to.OracleGALE_FA(256, **kw).train(), pn.GALE_FA(256, **kw).train()
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    x, ctx, dy = torch.randn(1, 6000, 256), torch.randn(1, 8, 16, 32), torch.randn(1, 6000, 256)
    xr = x.clone().requires_grad_()
    ref((xr,), ctx)[0].backward(dy)
    xh = x.clone().cuda().requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        yh = hip((xh,), ctx.cuda())[0]
    assert yh.dtype == torch.bfloat16
    yh.backward(dy.cuda().bfloat16())
    assert_rel_l2(xh.grad, xr.grad, "bf16 d x", tol=5e-2)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if name == "cross_k.bias":
            continue
        assert_rel_l2(grads[name].grad, p.grad, f"bf16 grad {name}", tol=6e-2)

    announce("GeoTransolver with GALE_FA blocks: training step")
    model = pn.GeoTransolver(functional_dim=6, out_dim=3, geometry_dim=3, global_dim=5, n_layers=2, n_hidden=32, n_head=4,
                             mlp_ratio=2, slice_num=8, attention_type="GALE_FA", use_te=False).cuda().train()
    e, geom, glob = torch.randn(2, 150, 6).cuda(), torch.randn(2, 90, 3).cuda(), torch.randn(2, 4, 5).cuda()
    opt = torch.optim.SGD(model.parameters(), lr=1e-2)
    losses = []
    for _ in range(3):
        opt.zero_grad()
        loss = (model(e, None, glob, geom) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())
    assert losses[-1] < losses[0]


# ---------------------------------------------------------------------------------------------------
# FLARE model (Transolver with FLARE blocks) against the reference's golden outputs
# ---------------------------------------------------------------------------------------------------
import os

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("kind", ["structured2d", "irregular"])
def test_flare_model_reproduces_reference_golden_output(kind):
    """reference test/models/flare/test_flare.py:124-193: seed 0, the same inputs, its own atol; the weights come from
    the oracle model (whose seeded construction reproduces the golden files on the CPU)."""
    announce("FLARE model golden", kind)
    torch.manual_seed(0)
    if kind == "structured2d":
        kw = dict(structured_shape=(85, 85), n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1, functional_dim=1, out_dim=1,
                  slice_num=32, ref=1, unified_pos=True)
        ref = to.OracleFLAREModel(init="rejection", **kw)
        a, b = torch.randn(4, 85 * 85, 1), torch.randn(4, 85, 85)
        name, atol = "flare_2d_output.pth", 2e-3
    else:
        kw = dict(structured_shape=None, n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1, functional_dim=2,
                  embedding_dim=3, out_dim=1, slice_num=32, unified_pos=False)
        ref = to.OracleFLAREModel(init="rejection", **kw)
        a, b = torch.randn(4, 12345, 3), torch.randn(4, 12345, 2)
        name, atol = "flare_irregular_output.pth", 1e-3
    gold = torch.load(os.path.join(GOLD, name), weights_only=True)[0]
    hip = pn.FLAREModel(use_te=False, **kw)
    hip.load_state_dict(ref.state_dict())
    hip = hip.eval().cuda()
    with torch.no_grad():
        out = hip(a.cuda(), b.cuda()).cpu()
    assert out.shape == gold.shape
    assert torch.allclose(out, gold, rtol=1e-3, atol=atol)
    assert_fp32_close(out, gold, "FLARE model vs golden", rtol=2e-4)


def test_flare_model_training_step_and_checkpoint(tmp_path):
    announce("FLARE model training step")
    torch.manual_seed(0)
    kw = dict(functional_dim=2, out_dim=3, embedding_dim=3, n_layers=2, n_hidden=32, n_head=4, slice_num=8, mlp_ratio=2)
    m = pn.FLAREModel(use_te=False, **kw).cuda().train()
    ref = to.OracleFLAREModel(**kw).train()
    ref.load_state_dict(m.state_dict())
    fx, emb, target = torch.randn(2, 200, 2), torch.randn(2, 200, 3), torch.randn(2, 200, 3)
    ((ref(fx, emb) - target) ** 2).mean().backward()
    ((m(fx.cuda(), emb.cuda()) - target.cuda()) ** 2).mean().backward()
    grads = dict(m.named_parameters())
    for name, p in ref.named_parameters():
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=5e-4)
    path = str(tmp_path / "flare.mdlus")
    m.save(path)
    again = pn.FLAREModel.from_checkpoint(path).cuda().eval()
    m.eval()
    with torch.no_grad():
        assert torch.equal(again(fx.cuda(), emb.cuda()), m(fx.cuda(), emb.cuda()))
