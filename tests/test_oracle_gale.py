"""Pins of the GALE restatement in oracle/ (reference physicsnemo/nn/module/gale.py:43-239): the torch oracle against the
independent NumPy one, and special cases that fix what a plausible mistake would change -- which operand feeds q and
which k / v, the SDPA scale, the direction of the sigmoid gate, the order of the concatenation, and that no context
means the plain PhysicsAttention layer."""
import math

import numpy as np
import pytest
import torch

from oracle import numpy_oracle as no
from oracle import torch_oracle as to


def _sd_np(m):
    return {k: v.detach().double().numpy() for k, v in m.state_dict().items()}


def _gale(mode="weighted", dim=12, heads=2, dim_head=6, slice_num=5, context_dim=7, variant="irregular", seed=3):
    torch.manual_seed(seed)
    if variant == "irregular":
        m = to.OracleGALE(dim, heads=heads, dim_head=dim_head, slice_num=slice_num, context_dim=context_dim,
                          state_mixing_mode=mode)
    else:
        m = to.OracleGALEStructuredMesh2D(dim, (3, 4), heads=heads, dim_head=dim_head, slice_num=slice_num, kernel=3,
                                          context_dim=context_dim, state_mixing_mode=mode)
    m = m.double()
    if mode == "weighted":
        with torch.no_grad():
            m.state_mixing.fill_(0.7)
    return m.eval()


@pytest.mark.parametrize("mode", ["weighted", "concat_project"])
@pytest.mark.parametrize("variant", ["irregular", "structured2d"])
def test_torch_gale_equals_numpy_gale(mode, variant):
    m = _gale(mode, variant=variant)
    x = torch.randn(2, 12, 12, dtype=torch.float64)
    ctx = torch.randn(2, 2, 9, 7, dtype=torch.float64)
    with torch.no_grad():
        y = m((x,), ctx)[0]
    ref = no.layer_forward(_sd_np(m), x.numpy(), 2, 6, variant=variant,
                           spatial_shape=None if variant == "irregular" else (3, 4), context=ctx.numpy())
    np.testing.assert_allclose(y.numpy(), ref["y"], rtol=1e-10, atol=1e-12)


def test_no_context_is_the_plain_layer_and_tuple_inputs_are_independent():
    m = _gale("weighted")
    plain = to.OraclePhysicsAttentionIrregularMesh(12, heads=2, dim_head=6, slice_num=5).double()
    plain.load_state_dict({k: v for k, v in m.state_dict().items() if k in plain.state_dict()})
    x1, x2 = torch.randn(2, 9, 12, dtype=torch.float64), torch.randn(2, 4, 12, dtype=torch.float64)
    ctx = torch.randn(2, 2, 3, 7, dtype=torch.float64)
    with torch.no_grad():
        out = m((x1, x2))
        assert len(out) == 2
        torch.testing.assert_close(out[0], plain(x1))
        torch.testing.assert_close(out[1], plain(x2))
        both = m((x1, x2), ctx)
        torch.testing.assert_close(both[1], m((x2,), ctx)[0])


def test_gate_direction_and_single_context_token_closed_form():
    """sigmoid(m) weighs the SELF-attention result (gale.py:78-79).  With one context token the cross-attention
    returns cross_v(context) for every slice whatever q and k are; the deslice then gives every point the same row
    (the slice weights of a point sum to one), so the layer output is Wout . concat_h(cross_v(ctx_h)) + bout."""
    m = _gale("weighted")
    x = torch.randn(2, 9, 12, dtype=torch.float64)
    ctx = torch.randn(2, 2, 1, 7, dtype=torch.float64)
    plain = to.OraclePhysicsAttentionIrregularMesh(12, heads=2, dim_head=6, slice_num=5).double()
    plain.load_state_dict({k: v for k, v in m.state_dict().items() if k in plain.state_dict()})
    with torch.no_grad():
        m.state_mixing.fill_(40.0)  # gate -> 1: self only
        torch.testing.assert_close(m((x,), ctx)[0], plain(x))
        m.state_mixing.fill_(-40.0)  # gate -> 0: cross only
        y = m((x,), ctx)[0]
        v = ctx[:, :, 0, :] @ m.cross_v.weight.t() + m.cross_v.bias  # (B, H, D)
        want = v.reshape(2, 1, 12) @ m.out_linear.weight.t() + m.out_linear.bias
        torch.testing.assert_close(y, want.expand(2, 9, 12))
        m.state_mixing.fill_(0.0)  # balanced: the mean of the two
        torch.testing.assert_close(m((x,), ctx)[0], 0.5 * (plain(x) + want.expand(2, 9, 12)))


def test_keys_come_from_the_context_and_scale_is_inverse_sqrt_d():
    """Zero cross_k gives uniform attention = the mean of cross_v(context) over the context tokens.  A context whose
    first token's key is c q-aligned and the rest zero gives softmax weights [e^{c|q|^2/sqrt(D)}, 1, 1, ...]: checked
    for one slice token through the stage function."""
    m = _gale("weighted")
    B, H, S, D, Sc, Dc = 1, 2, 5, 6, 4, 7
    tok = torch.randn(B, H, S, D, dtype=torch.float64)
    ctx = torch.randn(B, H, Sc, Dc, dtype=torch.float64)
    with torch.no_grad():
        m.cross_k.weight.zero_()
        m.cross_k.bias.zero_()
        got = to.gale_cross_attention(tok, ctx, m.cross_q, m.cross_k, m.cross_v)
        v = ctx @ m.cross_v.weight.t() + m.cross_v.bias
        torch.testing.assert_close(got, v.mean(dim=2, keepdim=True).expand(B, H, S, D))
        # explicit softmax with the 1/sqrt(D) scale
        m.cross_k.weight.normal_()
        q = tok @ m.cross_q.weight.t() + m.cross_q.bias
        k = ctx @ m.cross_k.weight.t() + m.cross_k.bias
        a = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(D), dim=-1)
        torch.testing.assert_close(to.gale_cross_attention(tok, ctx, m.cross_q, m.cross_k, m.cross_v), a @ v)


def test_concat_order_is_self_then_cross():
    m = _gale("concat_project")
    B, H, S, D = 1, 2, 5, 6
    a, b = torch.randn(B, H, S, D, dtype=torch.float64), torch.randn(B, H, S, D, dtype=torch.float64)
    eye, zero = torch.eye(D, dtype=torch.float64), torch.zeros(D, D, dtype=torch.float64)
    with torch.no_grad():
        m.concat_project[0].bias.zero_()
        m.concat_project[0].weight.copy_(torch.cat([eye, zero], dim=1))
        torch.testing.assert_close(to.gale_mix(a, b, "concat_project", concat_project=m.concat_project),
                                   torch.nn.functional.gelu(a))
        m.concat_project[0].weight.copy_(torch.cat([zero, eye], dim=1))
        torch.testing.assert_close(to.gale_mix(a, b, "concat_project", concat_project=m.concat_project),
                                   torch.nn.functional.gelu(b))
    with pytest.raises(ValueError):
        to.gale_mix(a, b, "other")


def test_gale_state_dict_contract_and_validation():
    """Parameter names, shapes and registration order of gale.py:401-429 on top of the PhysicsAttention ones."""
    m = to.OracleGALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5)
    keys = list(m.state_dict())
    assert keys == ["temperature", "state_mixing", "in_project_slice.weight", "in_project_slice.bias",
                    "qkv_project.weight", "out_linear.weight", "out_linear.bias", "in_project_x.weight",
                    "in_project_x.bias", "in_project_fx.weight", "in_project_fx.bias", "cross_q.weight", "cross_q.bias",
                    "cross_k.weight", "cross_k.bias", "cross_v.weight", "cross_v.bias"]
    sd = m.state_dict()
    assert sd["state_mixing"].shape == () and float(sd["state_mixing"]) == 0.0
    assert sd["cross_q.weight"].shape == (8, 8) and sd["cross_k.weight"].shape == (8, 5)
    c = to.OracleGALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5, state_mixing_mode="concat_project")
    assert "state_mixing" not in c.state_dict() and c.state_dict()["concat_project.0.weight"].shape == (8, 16)
    with pytest.raises(ValueError, match="Invalid state_mixing_mode"):
        to.OracleGALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5, state_mixing_mode="sum")
    with pytest.raises(ValueError, match="non-empty"):
        m(())
    with pytest.raises(ValueError, match="Expected 3D input tensor"):
        m((torch.randn(3, 16),))


def test_context_projector_is_the_encoding_half_of_the_layer():
    """context_projector.py:338-378 computes exactly the slice tokens of a PhysicsAttention layer with the same
    projection / slice parameters (physics_attention.py:529-540); state_dict order as registered in :283-300."""
    torch.manual_seed(2)
    proj = to.OracleContextProjector(10, heads=2, dim_head=6, slice_num=5).double()
    assert list(proj.state_dict()) == ["temperature", "in_project_x.weight", "in_project_x.bias", "in_project_fx.weight",
                                       "in_project_fx.bias", "in_project_slice.weight", "in_project_slice.bias"]
    layer = to.OraclePhysicsAttentionIrregularMesh(10, heads=2, dim_head=6, slice_num=5).double()
    layer.load_state_dict(proj.state_dict(), strict=False)
    x = torch.randn(2, 9, 10, dtype=torch.float64)
    with torch.no_grad():
        tok = proj(x)
        assert tok.shape == (2, 2, 5, 6)
        torch.testing.assert_close(tok, layer.stages(x)["tok"])
    ref = no.layer_forward({**_sd_np(layer)}, x.numpy(), 2, 6)
    np.testing.assert_allclose(tok.numpy(), ref["tok"], rtol=1e-10, atol=1e-12)
    # structured: same statement with the convolutions
    sp = to.OracleStructuredContextProjector(4, (3, 4), heads=2, dim_head=6, slice_num=5).double()
    sl = to.OraclePhysicsAttentionStructuredMesh2D(4, (3, 4), heads=2, dim_head=6, slice_num=5, kernel=3).double()
    sl.load_state_dict(sp.state_dict(), strict=False)
    xs = torch.randn(2, 12, 4, dtype=torch.float64)
    with torch.no_grad():
        torch.testing.assert_close(sp(xs), sl.stages(xs)["tok"])
    with pytest.raises(ValueError, match="length 2 or 3"):
        to.OracleStructuredContextProjector(4, (3,), heads=2, dim_head=6)
    # plus: one projection, given noise
    pp = to.OracleContextProjector(10, heads=2, dim_head=6, slice_num=5, plus=True).double()
    lp = to.OraclePhysicsAttentionIrregularMesh(10, heads=2, dim_head=6, slice_num=5, plus=True).double()
    lp.load_state_dict(pp.state_dict(), strict=False)
    u = torch.rand(2, 9, 2, 5, dtype=torch.float64)
    with torch.no_grad():
        torch.testing.assert_close(pp(x, u), lp.stages(x, u)["tok"])


def test_gale_block_against_numpy_pieces():
    """OracleGALEBlock = LayerNorm, GALE layer, residual, LayerNorm, MLP, residual (gale.py:1018-1028), checked against
    the NumPy restatements of each piece."""
    torch.manual_seed(6)
    blk = to.OracleGALEBlock(2, 12, mlp_ratio=2, slice_num=5, context_dim=7).double().eval()
    x = torch.randn(2, 9, 12, dtype=torch.float64)
    ctx = torch.randn(2, 2, 4, 7, dtype=torch.float64)
    with torch.no_grad():
        got = blk((x,), ctx)[0].numpy()
    p = _sd_np(blk)
    attn_p = {k[len("Attn."):]: v for k, v in p.items() if k.startswith("Attn.")}
    h1 = no.layer_norm(x.numpy(), p["ln_1.weight"], p["ln_1.bias"])
    fx = no.layer_forward(attn_p, h1, 2, 6, context=ctx.numpy())["y"] + x.numpy()
    h2 = no.layer_norm(fx, p["ln_mlp1.0.weight"], p["ln_mlp1.0.bias"])
    want = no.mlp(p, "ln_mlp1.1.", h2) + fx
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
