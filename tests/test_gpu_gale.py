"""GALE layers (PhysicsAttention + cross-attention of the slice tokens to a context) on the HIP kernels against the
oracle.  Bars: fp32 rtol 1e-4 (gradients 2e-4) with atol = rtol * max|ref|; bf16 output rel-L2 <= 1e-2 and bf16
gradients rel-L2 <= 5e-2 (d temperature 6e-2; measured: 3.3e-2 for the gradients through the slice softmax, under 1e-2
for the rest) against the fp32 oracle."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _pair(variant, mode, dim, heads, dim_head, S, context_dim, grid=None, plus=False, seed=0):
    torch.manual_seed(seed)
    kw = dict(heads=heads, dim_head=dim_head, slice_num=S, context_dim=context_dim, state_mixing_mode=mode, plus=plus)
    if variant == "irregular":
        ref, hip = to.OracleGALE(dim, **kw), pn.GALE(dim, use_te=False, **kw)
    elif variant == "structured2d":
        ref = to.OracleGALEStructuredMesh2D(dim, grid, kernel=3, **kw)
        hip = pn.GALEStructuredMesh2D(dim, grid, kernel=3, use_te=False, **kw)
    else:
        raise ValueError(variant)
    with torch.no_grad():
        ref.in_project_slice.weight.mul_(2.0)
        if mode == "weighted":
            ref.state_mixing.fill_(0.6)
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


@pytest.mark.parametrize("variant,mode,dim,heads,dim_head,S,B,N,Sc,Dc,grid", [
    ("irregular", "weighted", 32, 4, 8, 8, 2, 300, 5, 7, None),
    ("irregular", "concat_project", 32, 4, 8, 8, 2, 300, 5, 7, None),
    ("irregular", "weighted", 64, 2, 32, 64, 1, 1000, 1, 16, None),
    ("irregular", "concat_project", 48, 3, 16, 20, 3, 77, 130, 3, None),
    ("structured2d", "weighted", 32, 4, 8, 16, 2, 63, 9, 12, (7, 9)),
])
def test_fp32_gale_matches_oracle(variant, mode, dim, heads, dim_head, S, B, N, Sc, Dc, grid):
    announce("fp32 GALE", variant, mode, dim, heads, dim_head, S, B, N, Sc, Dc, grid)
    ref, hip = _pair(variant, mode, dim, heads, dim_head, S, Dc, grid)
    x1, x2 = torch.randn(B, N, dim), torch.randn(B, N, dim)
    ctx = torch.randn(B, heads, Sc, Dc)
    with torch.no_grad():
        want = ref((x1, x2), ctx)
        got = hip((x1.cuda(), x2.cuda()), ctx.cuda())
        assert isinstance(got, list) and len(got) == 2
        for g, w in zip(got, want):
            assert_fp32_close(g, w, "GALE y")
        # no context: the plain layer (fused path)
        assert_fp32_close(hip((x1.cuda(),))[0], ref((x1,))[0], "GALE y without context")


def test_cross_mix_stage_against_oracle_functions():
    announce("GALE cross-attention + blend stage")
    B, H, S, D, Sc, Dc = 2, 3, 24, 16, 11, 5
    for mode in ("weighted", "concat_project"):
        torch.manual_seed(4)
        ref = to.OracleGALE(H * D, heads=H, dim_head=D, slice_num=S, context_dim=Dc, state_mixing_mode=mode)
        hip = pn.GALE(H * D, heads=H, dim_head=D, slice_num=S, context_dim=Dc, state_mixing_mode=mode, use_te=False)
        hip.load_state_dict(ref.state_dict())
        tok, self_out, ctx = torch.randn(B, H, S, D), torch.randn(B, H, S, D), torch.randn(B, H, Sc, Dc)
        with torch.no_grad():
            cross = to.gale_cross_attention(tok, ctx, ref.cross_q, ref.cross_k, ref.cross_v)
            want = to.gale_mix(self_out, cross, mode, getattr(ref, "state_mixing", None),
                               getattr(ref, "concat_project", None))
        dims = PF.LayerDims(B, 100, H * D, H, D, S)
        got = PF.slice_cross_attention_mix(tok.cuda(), self_out.cuda(), ctx.cuda(), hip.gale_params(torch.device("cuda")),
                                           dims)
        assert_fp32_close(got, want, f"blend {mode}")


@pytest.mark.parametrize("mode,S,N", [("weighted", 64, 4096), ("concat_project", 32, 5000), ("weighted", 128, 3000)])
def test_bf16_gale_on_the_mfma_kernels(mode, S, N):
    announce("bf16 GALE MFMA", mode, S, N)
    ref, hip = _pair("irregular", mode, 256, 8, 32, S, 32)
    x = torch.randn(2, N, 256)
    ctx = torch.randn(2, 8, 48, 32)
    xb = x.cuda().bfloat16()
    assert PF.query_path(torch.bfloat16, hip.layer_dims(xb)) == 1
    with torch.no_grad():
        want = ref((x,), ctx)[0]
        got = hip((xb,), ctx.cuda())[0]
        plain = hip((xb,))[0]
    assert got.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 GALE y", tol=1e-2)
    assert to.rel_l2(plain.float().cpu(), want) > 5e-2  # the context matters in this case


def test_gale_plus_and_errors():
    announce("GALE plus / errors")
    ref, hip = _pair("irregular", "weighted", 32, 4, 8, 8, 7, plus=True)
    x = torch.randn(2, 200, 32, device="cuda")
    ctx = torch.randn(2, 4, 5, 7, device="cuda")
    with torch.no_grad():
        torch.manual_seed(5)
        a = hip((x,), ctx)[0]
        torch.manual_seed(5)
        b = hip((x,), ctx)[0]
    assert torch.equal(a, b) and torch.isfinite(a).all()
    with pytest.raises(ValueError, match="non-empty"):
        hip(())
    with pytest.raises(ValueError, match="Expected 3D input tensor"):
        hip((x[0],), ctx)
    with pytest.raises(ValueError, match="Expected context"):
        hip((x,), ctx[:, :2])
    with pytest.raises(TypeError):
        hip(x, ctx)


@pytest.mark.parametrize("mode", ["weighted", "concat_project"])
def test_gale_plus_gradients_with_context_match_autograd_over_the_oracle(mode):
    """plus=True with a context, training: the layer draws its Gumbel samples on the device; the same seed and shape
    give the test the same samples for the oracle."""
    announce("GALE plus gradients with context", mode)
    ref, hip = _pair("irregular", mode, 32, 4, 8, 8, 7, plus=True, seed=3)
    ref.train(), hip.train()
    B, N = 2, 300
    x, ctx, probe = torch.randn(B, N, 32), torch.randn(B, 4, 5, 7), torch.randn(B, N, 32)
    torch.manual_seed(11)
    u = torch.rand((B, N, 4, 8), dtype=torch.float32, device="cuda")
    xr, cr = x.clone().requires_grad_(), ctx.clone().requires_grad_()
    yr = ref.stages(xr, noise_u=u.cpu(), context=cr)["y"]
    (yr * probe).sum().backward()
    xh, ch = x.clone().cuda().requires_grad_(), ctx.clone().cuda().requires_grad_()
    torch.manual_seed(11)
    yh = hip((xh,), ch)[0]
    assert_fp32_close(yh, yr, "GALE plus y (training path)")
    (yh * probe.cuda()).sum().backward()
    assert_fp32_close(xh.grad, xr.grad, "d x", rtol=5e-4)
    assert_fp32_close(ch.grad, cr.grad, "d context", rtol=5e-4)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if name == "cross_k.bias" or p.grad is None:
            continue  # zero in exact arithmetic / in_project_fx, which plus=True does not use
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=5e-4)


def _gale_grads(module, x, ctx, probe):
    module.zero_grad(set_to_none=True)
    x = x.clone().requires_grad_(True)
    ctx = ctx.clone().requires_grad_(True)
    y = module((x,), ctx)[0]
    (y.float() * probe.to(y.device)).sum().backward()
    out = {"x": x.grad, "context": ctx.grad}
    out.update({name: p.grad for name, p in module.named_parameters()})
    return y, out


@pytest.mark.parametrize("variant,mode,dim,heads,dim_head,S,B,N,Sc,Dc,grid", [
    ("irregular", "weighted", 32, 4, 8, 8, 2, 300, 5, 7, None),
    ("irregular", "concat_project", 64, 2, 32, 64, 1, 1000, 9, 16, None),
    ("structured2d", "weighted", 32, 4, 8, 16, 2, 63, 9, 12, (7, 9)),
])
def test_fp32_gale_gradients(variant, mode, dim, heads, dim_head, S, B, N, Sc, Dc, grid):
    announce("fp32 GALE backward", variant, mode, dim, heads, dim_head, S, B, N, Sc, Dc, grid)
    ref, hip = _pair(variant, mode, dim, heads, dim_head, S, Dc, grid)
    ref.train(), hip.train()
    x, probe, ctx = torch.randn(B, N, dim), torch.randn(B, N, dim), torch.randn(B, heads, Sc, Dc)
    y_ref, want = _gale_grads(ref, x, ctx, probe)
    y_hip, got = _gale_grads(hip, x.cuda(), ctx.cuda(), probe)
    assert_fp32_close(y_hip, y_ref, "forward y (training path)")
    assert set(got) == set(want)
    for name in want:
        assert got[name] is not None and got[name].shape == want[name].shape, name
        if name == "cross_k.bias":  # shifts every score of a query alike: the gradient is zero in exact arithmetic
            assert got[name].abs().max() < 1e-5 and want[name].abs().max() < 1e-5
            continue
        assert_fp32_close(got[name], want[name], f"grad {name}", rtol=2e-4)


def test_bf16_gale_gradients_on_the_mfma_kernels():
    announce("bf16 GALE backward (autocast, MFMA)")
    ref, hip = _pair("irregular", "weighted", 256, 8, 32, 64, 32)
    ref.train(), hip.train()
    torch.manual_seed(5)
    x, probe, ctx = torch.randn(2, 2048, 256), torch.randn(2, 2048, 256), torch.randn(2, 8, 48, 32)
    _, want = _gale_grads(ref, x, ctx, probe)
    hip.zero_grad(set_to_none=True)
    xc, cc = x.cuda().requires_grad_(True), ctx.cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip((xc,), cc)[0]
    assert y.dtype == torch.bfloat16
    (y.float() * probe.cuda()).sum().backward()
    got = {"x": xc.grad, "context": cc.grad}
    got.update({name: p.grad for name, p in hip.named_parameters()})
    for name in want:
        assert got[name] is not None and torch.isfinite(got[name]).all(), name
        if name != "cross_k.bias":
            # d temperature: 8 scalars, each a sum of cancelling terms over 4096 points of bf16 activations
            assert_rel_l2(got[name], want[name], f"bf16 GALE grad {name}", tol=6e-2 if name == "temperature" else 5e-2)


# ---------------------------------------------------------------------------------------------------
# context projectors (GeoTransolver): the encoding half of the layer, returning slice tokens
# ---------------------------------------------------------------------------------------------------
def _projector_pair(variant, dim, heads, dim_head, S, grid=None, plus=False, seed=0):
    torch.manual_seed(seed)
    if variant == "irregular":
        ref = to.OracleContextProjector(dim, heads=heads, dim_head=dim_head, slice_num=S, plus=plus)
        hip = pn.ContextProjector(dim, heads=heads, dim_head=dim_head, slice_num=S, plus=plus)
    else:
        ref = to.OracleStructuredContextProjector(dim, grid, heads=heads, dim_head=dim_head, slice_num=S, kernel=3)
        hip = pn.StructuredContextProjector(dim, grid, heads=heads, dim_head=dim_head, slice_num=S, kernel=3)
    with torch.no_grad():
        ref.in_project_slice.weight.mul_(4.0)
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


@pytest.mark.parametrize("variant,dim,heads,dim_head,S,B,N,grid", [
    ("irregular", 6, 4, 8, 8, 2, 300, None),         # input width differs from heads * dim_head
    ("irregular", 64, 2, 32, 64, 1, 1000, None),
    ("structured2d", 5, 4, 8, 16, 2, 63, (7, 9)),
    ("structured3d", 3, 2, 8, 8, 2, 60, (3, 4, 5)),
])
def test_fp32_context_projector_tokens_and_gradients(variant, dim, heads, dim_head, S, B, N, grid):
    announce("fp32 context projector", variant, dim, heads, dim_head, S, B, N, grid)
    ref, hip = _projector_pair("irregular" if variant == "irregular" else "structured", dim, heads, dim_head, S, grid)
    x = torch.randn(B, N, dim)
    with torch.no_grad():
        want = ref(x)
        got = hip(x.cuda())
    assert got.shape == (B, heads, S, dim_head) and got.dtype == torch.float32
    assert_fp32_close(got, want, "slice tokens")
    probe = torch.randn(B, heads, S, dim_head)
    ref.train(), hip.train()
    xr = x.clone().requires_grad_(True)
    (ref(xr) * probe).sum().backward()
    xh = x.cuda().requires_grad_(True)
    tok = hip(xh)
    assert_fp32_close(tok, want, "slice tokens (training path)")
    (tok * probe.cuda()).sum().backward()
    assert_fp32_close(xh.grad, xr.grad, "grad x", rtol=2e-4)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=2e-4)


def test_bf16_context_projector_feeds_gale_on_the_mfma_kernels():
    announce("bf16 context projector -> GALE")
    ref_p, hip_p = _projector_pair("irregular", 256, 8, 32, 64)
    ref_g, hip_g = _pair("irregular", "weighted", 256, 8, 32, 64, 32)
    geom, x = torch.randn(2, 3000, 256), torch.randn(2, 4096, 256)
    with torch.no_grad():
        ctx_ref = ref_p(geom)
        want = ref_g((x,), ctx_ref)[0]
        gb = geom.cuda().bfloat16()
        assert PF.query_path(torch.bfloat16, hip_p.layer_dims(gb)) == 1
        ctx_hip = hip_p(gb)
        got = hip_g((x.cuda().bfloat16(),), ctx_hip)[0]
    assert_rel_l2(ctx_hip, ctx_ref, "bf16 context tokens", tol=1e-2)
    assert_rel_l2(got, want, "bf16 GALE y from projected context", tol=1e-2)
    # training through both, bf16 autocast
    ref_p.train(), hip_p.train(), ref_g.train(), hip_g.train()
    probe = torch.randn(2, 4096, 256)
    (ref_g((x,), ref_p(geom))[0] * probe).sum().backward()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = hip_g((x.cuda(),), hip_p(geom.cuda()))[0]
    (y.float() * probe.cuda()).sum().backward()
    for name, p in ref_p.named_parameters():
        g = dict(hip_p.named_parameters())[name].grad
        assert g is not None and torch.isfinite(g).all(), name
        assert_rel_l2(g, p.grad, f"bf16 projector grad {name}", tol=1e-1 if name == "temperature" else 5e-2)


def test_context_projector_plus_and_errors():
    announce("context projector plus / errors")
    ref, hip = _projector_pair("irregular", 16, 4, 8, 8, plus=True)
    x = torch.randn(2, 200, 16, device="cuda")
    with torch.no_grad():
        torch.manual_seed(3)
        a = hip(x)
        torch.manual_seed(3)
        b = hip(x)
    assert a.shape == (2, 4, 8, 8) and torch.equal(a, b) and torch.isfinite(a).all()
    with pytest.raises(ValueError, match="Expected 3D input tensor"):
        hip(x[0])
    with pytest.raises(NotImplementedError):
        hip(x.requires_grad_(True))
    with pytest.raises(ValueError, match="length 2 or 3"):
        pn.StructuredContextProjector(4, (3,), heads=2, dim_head=8)
    sp = pn.StructuredContextProjector(4, (3, 4), heads=2, dim_head=8, slice_num=4).cuda()
    with pytest.raises(ValueError, match="Expected N=12 tokens"), torch.no_grad():
        sp(torch.randn(1, 13, 4, device="cuda"))


# ---------------------------------------------------------------------------------------------------
# GALE block
# ---------------------------------------------------------------------------------------------------
def _block_pair(hidden, heads, S, Dc, grid=None, mlp_ratio=2, seed=0):
    torch.manual_seed(seed)
    ref = to.OracleGALEBlock(heads, hidden, mlp_ratio=mlp_ratio, slice_num=S, context_dim=Dc, spatial_shape=grid)
    hip = pn.GALEBlock(heads, hidden, 0.0, mlp_ratio=mlp_ratio, slice_num=S, context_dim=Dc, spatial_shape=grid)
    with torch.no_grad():
        ref.Attn.in_project_slice.weight.mul_(2.0)
        ref.Attn.state_mixing.fill_(0.4)
    hip.load_state_dict(ref.state_dict())
    return ref.eval(), hip.eval().cuda()


@pytest.mark.parametrize("hidden,heads,S,B,N,Sc,Dc,grid", [
    (32, 4, 8, 2, 300, 5, 7, None),
    (32, 4, 16, 2, 63, 9, 12, (7, 9)),
])
def test_fp32_gale_block_forward_and_gradients(hidden, heads, S, B, N, Sc, Dc, grid):
    announce("fp32 GALE block", hidden, heads, S, B, N, Sc, Dc, grid)
    ref, hip = _block_pair(hidden, heads, S, Dc, grid)
    x1, x2, ctx = torch.randn(B, N, hidden), torch.randn(B, N, hidden), torch.randn(B, heads, Sc, Dc)
    with torch.no_grad():
        want = ref((x1, x2), ctx)
        got = hip((x1.cuda(), x2.cuda()), ctx.cuda())
    for g, w in zip(got, want):
        assert_fp32_close(g, w, "GALE block y")
    probe = torch.randn(B, N, hidden)
    ref.train(), hip.train()
    xr = x1.clone().requires_grad_(True)
    (ref((xr,), ctx)[0] * probe).sum().backward()
    xh = x1.cuda().requires_grad_(True)
    (hip((xh,), ctx.cuda())[0] * probe.cuda()).sum().backward()
    assert_fp32_close(xh.grad, xr.grad, "grad x", rtol=2e-4)
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if name == "Attn.cross_k.bias":
            continue  # zero in exact arithmetic
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=2e-4)


def test_bf16_gale_block_on_the_fused_kernels():
    announce("bf16 GALE block")
    ref, hip = _block_pair(256, 8, 64, 32, mlp_ratio=4)
    x, ctx = torch.randn(2, 4096, 256), torch.randn(2, 8, 48, 32)
    with torch.no_grad():
        want = ref((x,), ctx)[0]
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip((x.cuda(),), ctx.cuda())[0]
    assert got.dtype == torch.bfloat16
    assert_rel_l2(got, want, "bf16 GALE block y", tol=1e-2)
    fa = pn.GALEBlock(8, 256, 0.0, attention_type="GALE_FA", slice_num=32, context_dim=32).eval().cuda()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        out = fa((x.cuda(),), ctx.cuda())[0]
    assert isinstance(fa.Attn, pn.GALE_FA) and out.shape == x.shape and torch.isfinite(out).all()
    with pytest.raises(ValueError, match="Invalid attention type"):
        pn.GALEBlock(8, 256, 0.0, attention_type="other")
