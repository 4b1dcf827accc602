"""Pins for the oracle that do not retype its formulas: an independent float64 NumPy restatement,
library special cases, invariants and hand-computable closed forms.  Each check is chosen so that a
plausible slip (wrong split order, transposed operand, dropped eps, wrong clamp, normalised-vs-raw
weights in the deslice) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import numpy_oracle as no
from oracle import torch_oracle as to


def _sd_np(m):
    return {k: v.detach().double().numpy() for k, v in m.state_dict().items()}


def _mk_irregular(dim=16, heads=2, dim_head=8, slice_num=4, dtype=torch.float64):
    m = to.OraclePhysicsAttentionIrregularMesh(dim, heads=heads, dim_head=dim_head, slice_num=slice_num).to(dtype)
    with torch.no_grad():
        m.temperature.copy_(torch.linspace(0.3, 6.0, heads).view(1, 1, heads, 1))  # exercises both clamps
        m.in_project_slice.weight.mul_(3.0)
    return m


@pytest.mark.parametrize("shape", [(2, 17, 16, 2, 8, 4), (1, 33, 24, 3, 4, 5), (3, 8, 8, 1, 8, 16)])
def test_torch_oracle_equals_numpy_oracle_irregular(shape):
    B, N, C, H, D, S = shape
    m = _mk_irregular(C, H, D, S)
    x = torch.randn(B, N, C, dtype=torch.float64)
    with torch.no_grad():
        st = m.stages(x)
    ref = no.layer_forward(_sd_np(m), x.numpy(), H, D)
    for key in ("x_mid", "fx_mid", "logits", "w", "norm", "tok", "tok_out", "y"):
        np.testing.assert_allclose(st[key].numpy(), ref[key], rtol=1e-10, atol=1e-12, err_msg=key)


@pytest.mark.parametrize("kernel", [1, 3, 5])
def test_torch_oracle_equals_numpy_oracle_structured(kernel):
    B, gh, gw, C, H, D, S = 2, 5, 7, 12, 3, 4, 6
    m = to.OraclePhysicsAttentionStructuredMesh2D(C, (gh, gw), heads=H, dim_head=D, slice_num=S, kernel=kernel).double()
    x = torch.randn(B, gh * gw, C, dtype=torch.float64)
    with torch.no_grad():
        st = m.stages(x)
    ref = no.layer_forward(_sd_np(m), x.numpy(), H, D, variant="structured2d", spatial_shape=(gh, gw))
    for key in ("x_mid", "fx_mid", "w", "tok", "tok_out", "y"):
        np.testing.assert_allclose(st[key].numpy(), ref[key], rtol=1e-10, atol=1e-12, err_msg=key)


def test_conv_kernel1_is_the_linear_variant():
    # k = 1 conv == per-point linear: the 2D layer must equal the irregular layer with W[:, :, 0, 0]
    B, gh, gw, C, H, D, S = 2, 4, 6, 8, 2, 4, 3
    m2 = to.OraclePhysicsAttentionStructuredMesh2D(C, (gh, gw), heads=H, dim_head=D, slice_num=S, kernel=1).double()
    m1 = to.OraclePhysicsAttentionIrregularMesh(C, heads=H, dim_head=D, slice_num=S).double()
    sd = dict(m2.state_dict())
    sd["in_project_x.weight"] = sd["in_project_x.weight"][:, :, 0, 0]
    sd["in_project_fx.weight"] = sd["in_project_fx.weight"][:, :, 0, 0]
    m1.load_state_dict(sd)
    x = torch.randn(B, gh * gw, C, dtype=torch.float64)
    with torch.no_grad():
        assert torch.allclose(m1(x), m2(x), rtol=1e-12, atol=1e-13)


def test_conv_token_order_and_zero_padding():
    # a delta at grid (i0, j0) with an all-ones 3x3 kernel lights up exactly its 3x3 neighbourhood in
    # row-major token order n = i*W + j, clipped at the border (zero padding)
    gh, gw = 4, 5
    x = torch.zeros(1, gh * gw, 1, dtype=torch.float64)
    i0, j0 = 0, 4
    x[0, i0 * gw + j0, 0] = 1.0
    w = torch.ones(1, 1, 3, 3, dtype=torch.float64)
    zero = torch.zeros(1, dtype=torch.float64)
    xm, _ = to.project_conv2d(x, w, zero, w, zero, 1, 1, gh, gw)
    got = xm.reshape(gh, gw)
    want = torch.zeros(gh, gw, dtype=torch.float64)
    want[0:2, 3:5] = 1.0
    assert torch.equal(got, want)
    # cross-correlation orientation: weight tap (u, v) multiplies x[i+u-1, j+v-1]
    w2 = torch.zeros(1, 1, 3, 3, dtype=torch.float64)
    w2[0, 0, 0, 2] = 1.0  # reads the neighbour one row up, one column right
    xm2, _ = to.project_conv2d(x, w2, zero, w2, zero, 1, 1, gh, gw)
    got2 = xm2.reshape(gh, gw)
    assert got2[1, 3] == 1.0 and got2.sum() == 1.0
    np.testing.assert_allclose(no.conv2d_projection(x.numpy(), w2.numpy(), zero.numpy(), gh, gw).reshape(gh, gw), got2.numpy())


@pytest.mark.parametrize("kernel", [1, 3])
def test_torch_oracle_equals_numpy_oracle_structured3d(kernel):
    B, grid, C, H, D, S = 2, (3, 4, 5), 6, 2, 4, 5
    m = to.OraclePhysicsAttentionStructuredMesh3D(C, grid, heads=H, dim_head=D, slice_num=S, kernel=kernel).double()
    x = torch.randn(B, grid[0] * grid[1] * grid[2], C, dtype=torch.float64)
    with torch.no_grad():
        st = m.stages(x)
    ref = no.layer_forward(_sd_np(m), x.numpy(), H, D, variant="structured3d", spatial_shape=grid)
    for key in ("x_mid", "fx_mid", "w", "tok", "tok_out", "y"):
        np.testing.assert_allclose(st[key].numpy(), ref[key], rtol=1e-10, atol=1e-12, err_msg=key)


def test_conv3d_special_cases_pin_token_order_and_orientation():
    gh, gw, gd = 3, 4, 5
    zero = torch.zeros(1, dtype=torch.float64)
    # (a) a grid of depth 1 with weights confined to the central depth tap is the 2-D variant
    x2 = torch.randn(2, gh * gw, 3, dtype=torch.float64)
    w2 = torch.randn(4, 3, 3, 3, dtype=torch.float64)
    b2 = torch.randn(4, dtype=torch.float64)
    w3 = torch.zeros(4, 3, 3, 3, 3, dtype=torch.float64)
    w3[:, :, :, :, 1] = w2
    a, _ = to.project_conv2d(x2, w2, b2, w2, b2, 1, 4, gh, gw)
    c, _ = to.project_conv3d(x2, w3, b2, w3, b2, 1, 4, gh, gw, 1)
    assert torch.allclose(a, c, rtol=1e-12, atol=1e-13)
    # (b) k = 1 is the per-point linear map
    xl = torch.randn(2, gh * gw * gd, 3, dtype=torch.float64)
    w1 = torch.randn(4, 3, 1, 1, 1, dtype=torch.float64)
    c1, _ = to.project_conv3d(xl, w1, b2, w1, b2, 1, 4, gh, gw, gd)
    l1, _ = to.project_linear(xl, w1[:, :, 0, 0, 0], b2, w1[:, :, 0, 0, 0], b2, 1, 4)
    assert torch.allclose(c1, l1, rtol=1e-12, atol=1e-13)
    # (c) token order n = (i*W + j)*Dg + l and cross-correlation orientation: tap (u, v, z) reads x[i+u-1, j+v-1, l+z-1]
    x = torch.zeros(1, gh * gw * gd, 1, dtype=torch.float64)
    i0, j0, l0 = 1, 3, 4
    x[0, (i0 * gw + j0) * gd + l0, 0] = 1.0
    w = torch.zeros(1, 1, 3, 3, 3, dtype=torch.float64)
    w[0, 0, 0, 2, 1] = 1.0  # reads one step back in i, one step forward in j, same l
    out, _ = to.project_conv3d(x, w, zero, w, zero, 1, 1, gh, gw, gd)
    vol = out.reshape(gh, gw, gd)
    assert vol[i0 + 1, j0 - 1, l0] == 1.0 and vol.sum() == 1.0
    ones = torch.ones(1, 1, 3, 3, 3, dtype=torch.float64)
    full, _ = to.project_conv3d(x, ones, zero, ones, zero, 1, 1, gh, gw, gd)
    want = torch.zeros(gh, gw, gd, dtype=torch.float64)
    want[0:3, 2:4, 3:5] = 1.0  # the 3x3x3 neighbourhood clipped at the faces (zero padding)
    assert torch.equal(full.reshape(gh, gw, gd), want)
    np.testing.assert_allclose(
        no.conv3d_projection(x.numpy(), w.numpy(), zero.numpy(), gh, gw, gd).reshape(gh, gw, gd), vol.numpy())


@pytest.mark.parametrize("variant", ["irregular", "structured2d"])
def test_oracle_gradient_matches_finite_differences(variant):
    """The GPU backward tests compare against autograd over the torch oracle; here that gradient is pinned by
    central finite differences in float64 (torch.autograd.gradcheck), w.r.t. the input and every parameter."""
    torch.manual_seed(11)
    if variant == "irregular":
        m = to.OraclePhysicsAttentionIrregularMesh(6, heads=2, dim_head=3, slice_num=4).double()
        n = 7
    else:
        m = to.OraclePhysicsAttentionStructuredMesh2D(6, (3, 4), heads=2, dim_head=3, slice_num=4, kernel=3).double()
        n = 12
    with torch.no_grad():
        m.temperature.copy_(torch.tensor([0.8, 2.0], dtype=torch.float64).view(1, 1, 2, 1))
    names = [k for k, _ in m.named_parameters()]
    params = [p.detach().clone().requires_grad_(True) for _, p in m.named_parameters()]
    x = torch.randn(2, n, 6, dtype=torch.float64, requires_grad=True)

    def fn(x, *ps):
        return torch.func.functional_call(m, dict(zip(names, ps)), (x,))

    assert torch.autograd.gradcheck(fn, (x, *params), eps=1e-6, atol=1e-6, rtol=1e-5)


def test_oracle_plus_gradient_matches_finite_differences():
    """Gradient of the Transolver++ branch of the oracle (given the uniform samples), pinned the same way; the
    per-point temperatures are kept away from the clamp at 0.01, where the function has a kink."""
    torch.manual_seed(12)
    m = to.OraclePhysicsAttentionIrregularMesh(6, heads=2, dim_head=3, slice_num=4, plus=True).double()
    with torch.no_grad():
        m.temperature.copy_(torch.tensor([0.8, 1.5], dtype=torch.float64).view(1, 1, 2, 1))
    u = torch.rand(2, 7, 2, 4, dtype=torch.float64)

    class GivenNoise(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.m = m

        def forward(self, x):
            return self.m.forward_with_noise(x, u)

    wrapped = GivenNoise()
    names = [k for k, _ in wrapped.named_parameters()]
    params = [p.detach().clone().requires_grad_(True) for _, p in wrapped.named_parameters()]
    x = torch.randn(2, 7, 6, dtype=torch.float64, requires_grad=True)

    def fn(x, *ps):
        return torch.func.functional_call(wrapped, dict(zip(names, ps)), (x,))

    assert "m.proj_temperature.2.weight" in names
    assert torch.autograd.gradcheck(fn, (x, *params), eps=1e-6, atol=1e-6, rtol=1e-5)


def test_plus_branch_numpy_vs_torch_and_special_cases():
    torch.manual_seed(21)
    B, N, C, H, D, S = 2, 9, 6, 2, 4, 5
    m = to.OraclePhysicsAttentionIrregularMesh(C, heads=H, dim_head=D, slice_num=S, plus=True).double()
    assert "in_project_fx.weight" not in m.state_dict()
    assert list(m.state_dict())[:5] == ["temperature", "proj_temperature.0.weight", "proj_temperature.0.bias",
                                        "proj_temperature.2.weight", "proj_temperature.2.bias"]
    x = torch.randn(B, N, C, dtype=torch.float64)
    u = torch.rand(B, N, H, S, dtype=torch.float64)
    with torch.no_grad():
        st = m.stages(x, u)
    ref = no.layer_forward(_sd_np(m), x.numpy(), H, D, noise_u=u.numpy())
    for key in ("x_mid", "w", "tok", "tok_out", "y"):
        np.testing.assert_allclose(st[key].numpy(), ref[key], rtol=1e-10, atol=1e-12, err_msg=key)
    # noise that is the same for every slice of a point cancels in the softmax, and a proj_temperature whose last
    # Linear is zero adds GELU(0) = 0: the layer is then the plain one with in_project_fx := in_project_x
    # (temperatures inside [0.5, 5], where both clamps are inactive)
    plain = to.OraclePhysicsAttentionIrregularMesh(C, heads=H, dim_head=D, slice_num=S).double()
    sd = {k: v for k, v in m.state_dict().items() if not k.startswith("proj_temperature")}
    sd["in_project_fx.weight"], sd["in_project_fx.bias"] = sd["in_project_x.weight"], sd["in_project_x.bias"]
    plain.load_state_dict(sd)
    with torch.no_grad():
        m.proj_temperature[2].weight.zero_()
        m.proj_temperature[2].bias.zero_()
        m.temperature.copy_(torch.tensor([0.7, 3.0], dtype=torch.float64).view(1, 1, 2, 1))
        plain.temperature.copy_(m.temperature)
        u_const = torch.rand(B, N, H, 1, dtype=torch.float64).expand(B, N, H, S)
        assert torch.allclose(m.forward_with_noise(x, u_const), plain(x), rtol=1e-11, atol=1e-12)
        # below the plain clamp's floor the plus branch keeps the small temperature (floor 0.01, not 0.5)
        m.temperature.fill_(0.1)
        w_small = m.stages(x, u_const)["w"]
        want = torch.softmax(m.stages(x, u_const)["logits"] / 0.1, dim=-1)
        assert torch.allclose(w_small, want, rtol=1e-10, atol=1e-12)
        m.temperature.fill_(-3.0)  # clamps to 0.01
        want = torch.softmax(m.stages(x, u_const)["logits"] / 0.01, dim=-1)
        assert torch.allclose(m.stages(x, u_const)["w"], want, rtol=1e-10, atol=1e-12)
    # the noise is Gumbel(0, 1): mean = Euler-Mascheroni, variance = pi^2 / 6
    g = to.gumbel_from_uniform(torch.rand(400000, dtype=torch.float64))
    assert abs(float(g.mean()) - 0.5772156649) < 0.01 and abs(float(g.var()) - math.pi ** 2 / 6) < 0.03


def test_softmax_rows_and_temperature_clamp():
    B, N, H, D, S = 2, 11, 3, 4, 5
    logits = torch.randn(B, N, H, S, dtype=torch.float64) * 4
    fx = torch.randn(B, N, H, D, dtype=torch.float64)

    def run(tvals):
        t = torch.tensor(tvals, dtype=torch.float64).view(1, 1, H, 1)
        return to.slice_weights_and_tokens(logits, fx, t)

    w, tok, norm = run([0.5, 1.0, 5.0])
    assert torch.allclose(w.sum(-1), torch.ones(B, N, H, dtype=torch.float64), atol=1e-14)
    # clamp: 0.1 behaves as 0.5, 10 behaves as 5 (physics_attention.py:173)
    w2, tok2, _ = run([0.1, 1.0, 10.0])
    assert torch.equal(w, w2) and torch.equal(tok, tok2)
    # T = 0.5 doubles the logits; T = 1 is the plain softmax
    assert torch.allclose(w[:, :, 0], F.softmax(2.0 * logits[:, :, 0], -1), atol=1e-15)
    assert torch.allclose(w[:, :, 1], F.softmax(logits[:, :, 1], -1), atol=1e-15)
    assert torch.allclose(w[:, :, 2], F.softmax(logits[:, :, 2] / 5.0, -1), atol=1e-15)
    # shift invariance of the softmax over S
    w3, _, _ = to.slice_weights_and_tokens(logits + 7.25, fx, torch.tensor([0.5, 1.0, 5.0], dtype=torch.float64).view(1, 1, H, 1))
    assert torch.allclose(w, w3, atol=1e-14)
    # sum_s norm = N + 0.01 S  (eps is 1e-2, added once per slice)
    assert torch.allclose(norm.sum(-1), torch.full((B, H), N + 0.01 * S, dtype=torch.float64), atol=1e-12)


def test_aggregation_constant_field_single_point_and_permutation():
    B, N, H, D, S = 1, 9, 2, 3, 4
    logits = torch.randn(B, N, H, S, dtype=torch.float64)
    t = torch.full((1, 1, H, 1), 1.0, dtype=torch.float64)
    # constant fx = c  =>  tok[s] = c (norm_s - 0.01) / norm_s
    c = 2.5
    w, tok, norm = to.slice_weights_and_tokens(logits, torch.full((B, N, H, D), c, dtype=torch.float64), t)
    want = c * (norm - 0.01) / norm
    assert torch.allclose(tok, want[..., None].expand_as(tok), atol=1e-13)
    # N = 1 exposes the eps: tok = w fx / (w + 0.01)
    l1 = logits[:, :1]
    f1 = torch.randn(B, 1, H, D, dtype=torch.float64)
    w1, tok1, _ = to.slice_weights_and_tokens(l1, f1, t)
    want1 = (w1[0, 0] / (w1[0, 0] + 0.01))[:, :, None] * f1[0, 0][:, None, :]
    assert torch.allclose(tok1[0], want1, atol=1e-14)
    # permutation invariance over points
    fx = torch.randn(B, N, H, D, dtype=torch.float64)
    perm = torch.randperm(N)
    _, ta, _ = to.slice_weights_and_tokens(logits, fx, t)
    _, tb, _ = to.slice_weights_and_tokens(logits[:, perm], fx[:, perm], t)
    assert torch.allclose(ta, tb, atol=1e-13)


def test_slice_attention_split_order_and_textbook():
    B, H, S, D = 2, 3, 5, 4
    tok = torch.randn(B, H, S, D, dtype=torch.float64)
    eye, zero = torch.eye(D, dtype=torch.float64), torch.zeros(D, D, dtype=torch.float64)
    # Wqkv = [0; 0; I]: q = k = 0 -> uniform attention -> every output row is the mean token
    out = to.slice_attention(tok, torch.cat([zero, zero, eye]), D)
    assert torch.allclose(out, tok.mean(2, keepdim=True).expand_as(tok), atol=1e-14)
    # Wqkv = [A; I; 2I]: q = tok A^T, k = tok, v = 2 tok, textbook softmax(q k^T / sqrt D) v
    A = torch.randn(D, D, dtype=torch.float64)
    out = to.slice_attention(tok, torch.cat([A, eye, 2 * eye]), D)
    q = tok @ A.T
    p = torch.softmax(q @ tok.transpose(-1, -2) / math.sqrt(D), -1)
    assert torch.allclose(out, p @ (2 * tok), atol=1e-13)


def test_deslice_uses_raw_weights_and_head_merge_order():
    B, N, H, D, S = 1, 6, 2, 3, 4
    w = torch.softmax(torch.randn(B, N, H, S, dtype=torch.float64), -1)
    v = torch.randn(H, D, dtype=torch.float64)
    tok_out = v[None, :, None, :].expand(B, H, S, D).contiguous()
    ident = torch.eye(H * D, dtype=torch.float64)
    y = to.deslice_and_project(w, tok_out, ident, torch.zeros(H * D, dtype=torch.float64))
    # sum_s w = 1  =>  every point gets v, heads concatenated as c = h*D + d
    assert torch.allclose(y, v.reshape(1, 1, H * D).expand(B, N, H * D), atol=1e-14)


def test_whole_layer_closed_form_with_zero_slice_weight():
    # in_project_slice.weight = 0 and bias = 0  =>  w = 1/S everywhere; tok[s] = sum_n fx_mid / (N + 0.01 S);
    # identical tokens => attention returns Wv tok; y = Wout tile_H(Wv tok) + bout for every point.
    B, N, C, H, D, S = 2, 13, 12, 3, 4, 5
    m = to.OraclePhysicsAttentionIrregularMesh(C, heads=H, dim_head=D, slice_num=S).double()
    with torch.no_grad():
        m.in_project_slice.weight.zero_()
        m.in_project_slice.bias.zero_()
    x = torch.randn(B, N, C, dtype=torch.float64)
    with torch.no_grad():
        y = m(x)
    sd = _sd_np(m)
    xn = x.numpy()
    fm = xn @ sd["in_project_fx.weight"].T + sd["in_project_fx.bias"]  # (B, N, H*D)
    tok = fm.sum(1) / (N + 0.01 * S)  # (B, H*D): same for every s
    wv = sd["qkv_project.weight"][2 * D:3 * D]
    o = np.einsum("bhd,ed->bhe", tok.reshape(B, H, D), wv).reshape(B, H * D)
    want = o @ sd["out_linear.weight"].T + sd["out_linear.bias"]
    np.testing.assert_allclose(y.numpy(), np.broadcast_to(want[:, None, :], (B, N, C)), rtol=1e-11, atol=1e-13)


def test_block_and_model_glue_against_numpy():
    B, N, C, H, S = 2, 10, 16, 4, 6
    torch.manual_seed(3)
    blk = to.OracleTransolverBlock(H, C, mlp_ratio=2, last_layer=True, out_dim=3, slice_num=S).double()
    with torch.no_grad():
        for n_, p_ in blk.named_parameters():  # make LN affine non-trivial
            if "ln" in n_ and p_.ndim == 1:
                p_.add_(0.1 * torch.randn_like(p_))
    x = torch.randn(B, N, C, dtype=torch.float64)
    with torch.no_grad():
        y = blk(x)
    ref = no.block_forward(_sd_np(blk), x.numpy(), H, C // H, last_layer=True)
    np.testing.assert_allclose(y.numpy(), ref, rtol=1e-9, atol=1e-11)


def test_model_flatten_equivalence_and_concat_order():
    # reference test_transolver.py:172-216: spatial and pre-flattened inputs agree (row-major flatten)
    torch.manual_seed(0)
    m = to.OracleTransolver(functional_dim=3, out_dim=2, embedding_dim=4, structured_shape=(6, 5), n_layers=2,
                            n_hidden=32, n_head=4, slice_num=8).eval()
    fx = torch.randn(2, 6, 5, 3)
    emb = torch.randn(2, 6, 5, 4)
    with torch.no_grad():
        a = m(fx, emb)
        b = m(fx.reshape(2, -1, 3), emb.reshape(2, -1, 4))
    assert a.shape == (2, 6, 5, 2) and torch.allclose(a.reshape(2, -1, 2), b, atol=1e-6)
    # concat order is [embedding, fx]: zeroing the first 4 preprocess input columns removes the embedding
    with torch.no_grad():
        m.preprocess.layers[0].weight[:, :4] = 0
        c = m(fx, emb)
        d = m(fx, torch.randn_like(emb))
    assert torch.allclose(c, d, atol=1e-6)


def test_unified_pos_grid_values():
    g = to.unified_pos_grid((3, 2), ref=2)  # points (i/2, j/1), lattice {0,1}^2
    assert g.shape == (1, 6, 4)
    # point (i=1,j=1) -> (0.5, 1.0); lattice order (0,0),(0,1),(1,0),(1,1)
    want = [math.hypot(0.5, 1.0), math.hypot(0.5, 0.0), math.hypot(0.5, 1.0), math.hypot(0.5, 0.0)]
    np.testing.assert_allclose(g[0, 1 * 2 + 1].numpy(), want, rtol=1e-6)


def test_validation_errors():
    m = to.OraclePhysicsAttentionIrregularMesh(8, heads=2, dim_head=4, slice_num=3)
    with pytest.raises(ValueError, match="Expected 3D input"):
        m(torch.randn(4, 8))
    with pytest.raises(ValueError, match="Expected input feature dimension 8, got 6"):
        m(torch.randn(1, 4, 6))


def test_state_dict_keys_and_shapes_match_reference_contract():
    m = to.OracleTransolver(functional_dim=1, out_dim=1, embedding_dim=2, n_layers=2, n_hidden=32, n_head=4,
                            slice_num=8, structured_shape=(4, 4), mlp_ratio=1)
    sd = m.state_dict()
    want = {
        "preprocess.layers.0.weight": (64, 3), "preprocess.layers.2.weight": (32, 64),
        "blocks.0.ln_1.weight": (32,), "blocks.0.Attn.temperature": (1, 1, 4, 1),
        "blocks.0.Attn.in_project_slice.weight": (8, 8), "blocks.0.Attn.in_project_slice.bias": (8,),
        "blocks.0.Attn.qkv_project.weight": (24, 8), "blocks.0.Attn.out_linear.weight": (32, 32),
        "blocks.0.Attn.in_project_x.weight": (32, 32, 3, 3), "blocks.0.Attn.in_project_fx.bias": (32,),
        "blocks.0.ln_mlp1.0.weight": (32,), "blocks.0.ln_mlp1.1.layers.0.weight": (32, 32),
        "blocks.0.ln_mlp1.1.layers.2.bias": (32,), "blocks.1.ln_mlp2.0.bias": (32,), "blocks.1.ln_mlp2.1.weight": (1, 32),
    }
    for k, shp in want.items():
        assert tuple(sd[k].shape) == shp, k
    assert "blocks.0.Attn.qkv_project.bias" not in sd and "blocks.0.ln_mlp2.0.weight" not in sd
    # registration order inside the attention module (drives RNG consumption)
    keys = [k for k in sd if k.startswith("blocks.0.Attn.")]
    assert [k.split(".", 3)[3] for k in keys] == [
        "temperature", "in_project_slice.weight", "in_project_slice.bias", "qkv_project.weight",
        "out_linear.weight", "out_linear.bias", "in_project_x.weight", "in_project_x.bias",
        "in_project_fx.weight", "in_project_fx.bias"]


def test_mlp_kernel_gelu_constants_against_exact_erf():
    """The fused MLP kernel evaluates GELU as x / (1 + exp2(x * P(min(x^2, 81)))) with the three constants found in
    physicsnemo_amd/csrc/pa_common.h (gelu_logistic).  Evaluate that form (float32, constants parsed from the source) against the
    exact erf form on a dense grid: a wrong or mistyped constant moves the error far above the bound."""
    import math
    import os
    import re

    import numpy as np

    src = open(os.path.join(os.path.dirname(__file__), "..", "physicsnemo_amd", "csrc", "pa_common.h")).read()
    body = src[src.index("__device__ __forceinline__ float gelu_logistic(float x)"):]
    body = body[:body.index("}")]
    consts = [float(c) for c in re.findall(r"(-?\d\.\d+e-?\d+)f \* -2\.f \* kLog2e", body)]
    assert len(consts) == 3, consts
    c2, c1, c0 = consts  # order of appearance: x^4, x^2, constant term
    clamp = float(re.search(r"fminf\(x \* x, (\d+)\.f\)", body).group(1))
    x = np.linspace(-30, 30, 1200001, dtype=np.float32)
    x2 = np.minimum(x * x, np.float32(clamp))
    k = np.float32(-2.0 * 1.4426950408889634)
    p = (np.float32(c2) * k * x2 + np.float32(c1) * k) * x2 + np.float32(c0) * k
    with np.errstate(over="ignore"):
        got = x / (np.float32(1) + np.exp2(x * p, dtype=np.float32))
    want = np.array([0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))) for v in x[::40].astype(np.float64)])
    err = np.abs(got[::40].astype(np.float64) - want)
    assert err.max() < 3e-5, err.max()
    # saturation ends: exactly x for large x, exactly 0 (up to sign) for large negative x
    assert got[-1] == x[-1] and abs(got[0]) == 0.0
