"""Pins of the FLARE restatement in oracle/ (reference physicsnemo/nn/module/flare_attention.py:38-72, :222-255): the torch
oracle against the independent NumPy one, and special cases that fix what a plausible mistake would change -- which
axis each softmax runs over, the scale (1, not 1/sqrt(D)), which operand is query / key / value in each pass."""
import numpy as np
import pytest
import torch

from oracle import numpy_oracle as no
from oracle import torch_oracle as to


def _sd_np(m):
    return {k: v.detach().double().numpy() for k, v in m.state_dict().items()}


def _flare(dim=12, heads=2, dim_head=6, S=5, seed=1):
    torch.manual_seed(seed)
    return to.OracleFLARE(dim, heads=heads, dim_head=dim_head, n_global_queries=S).double().eval()


@pytest.mark.parametrize("B,N", [(2, 9), (1, 1), (3, 40)])
def test_torch_flare_equals_numpy_flare(B, N):
    m = _flare()
    x = torch.randn(B, N, 12, dtype=torch.float64)
    with torch.no_grad():
        y = m(x)
    np.testing.assert_allclose(y.numpy(), no.flare_forward(_sd_np(m), x.numpy(), 2, 6), rtol=1e-10, atol=1e-12)


def test_zero_queries_give_the_mean_value_everywhere():
    """q_global = 0: all scores are zero, both softmaxes are uniform, so z[s] = mean_n v[n] for every s and
    y[n] = mean_n v[n] for every point: the output is constant over the points."""
    m = _flare()
    x = torch.randn(2, 9, 12, dtype=torch.float64)
    with torch.no_grad():
        m.q_global.zero_()
        y = m(x)
        xm = m.in_project_x(x).reshape(2, 9, 2, 6)
        v = m.self_v(xm).mean(dim=1)  # (B, H, D)
        want = v.reshape(2, 1, 12) @ m.out_linear.weight.t() + m.out_linear.bias
    torch.testing.assert_close(y, want.expand(2, 9, 12))


def test_one_query_gathers_with_a_softmax_over_the_points_at_scale_one():
    """S = 1: the hand-back softmax is over a single query (weight 1), so y[n] = z = sum_n softmax_n(k_n . g) v_n,
    with the scores NOT divided by sqrt(D)."""
    m = _flare(S=1)
    x = torch.randn(1, 7, 12, dtype=torch.float64)
    with torch.no_grad():
        y = m(x)
        xm = m.in_project_x(x).reshape(1, 7, 2, 6)
        k, v = m.self_k(xm), m.self_v(xm)
        a = torch.einsum("bnhd,hd->bnh", k, m.q_global[0, :, 0, :])
        z = torch.einsum("bnh,bnhd->bhd", torch.softmax(a, dim=1), v)
        want = z.reshape(1, 1, 12) @ m.out_linear.weight.t() + m.out_linear.bias
    torch.testing.assert_close(y, want.expand(1, 7, 12))


def test_flare_is_equivariant_under_point_permutations_and_keeps_its_contract():
    m = _flare()
    x = torch.randn(2, 11, 12, dtype=torch.float64)
    perm = torch.randperm(11)
    with torch.no_grad():
        torch.testing.assert_close(m(x[:, perm]), m(x)[:, perm])
    assert list(m.state_dict()) == ["q_global", "in_project_x.weight", "in_project_x.bias", "self_k.weight",
                                    "self_k.bias", "self_v.weight", "self_v.bias", "out_linear.weight",
                                    "out_linear.bias"]
    assert m.state_dict()["q_global"].shape == (1, 2, 5, 6) and m.scale == 1.0


def test_oracle_flare_gradient_matches_finite_differences():
    """The GPU backward test compares against autograd over the torch oracle; here that gradient is pinned by central
    finite differences in float64."""
    m = _flare(dim=6, heads=2, dim_head=3, S=4)
    names = [k for k, _ in m.named_parameters()]
    params = [p.detach().clone().requires_grad_(True) for _, p in m.named_parameters()]
    x = torch.randn(2, 7, 6, dtype=torch.float64, requires_grad=True)

    def fn(x, *ps):
        return torch.func.functional_call(m, dict(zip(names, ps)), (x,))

    assert torch.autograd.gradcheck(fn, (x, *params), eps=1e-6, atol=1e-6, rtol=1e-5)


def test_gale_fa_special_cases():
    """GALE_FA (gale.py:654-762): no context = the FLARE layer; gate -> 1 / 0 = self only / cross only; with one
    context token the per-point cross-attention returns cross_v(context) whatever the queries are (scale 1 plays no
    role then), so the cross-only output is W_out . concat_h(cross_v(ctx_h)) + b_out at every point."""
    torch.manual_seed(8)
    m = to.OracleGALE_FA(12, heads=2, dim_head=6, n_global_queries=5, context_dim=7).double().eval()
    flare = to.OracleFLARE(12, heads=2, dim_head=6, n_global_queries=5).double().eval()
    flare.load_state_dict({k: v for k, v in m.state_dict().items() if k in flare.state_dict()})
    assert list(m.state_dict())[:2] == ["q_global", "state_mixing"] and list(m.state_dict())[-2:] == [
        "out_linear.weight", "out_linear.bias"]
    x = torch.randn(2, 9, 12, dtype=torch.float64)
    ctx = torch.randn(2, 2, 1, 7, dtype=torch.float64)
    with torch.no_grad():
        torch.testing.assert_close(m((x,))[0], flare(x))
        m.state_mixing.fill_(40.0)
        torch.testing.assert_close(m((x,), ctx)[0], flare(x))
        m.state_mixing.fill_(-40.0)
        v = ctx[:, :, 0, :] @ m.cross_v.weight.t() + m.cross_v.bias
        want = v.reshape(2, 1, 12) @ m.out_linear.weight.t() + m.out_linear.bias
        torch.testing.assert_close(m((x,), ctx)[0], want.expand(2, 9, 12))
        # several context tokens: explicit softmax at scale 1 over the context axis
        ctx4 = torch.randn(2, 2, 4, 7, dtype=torch.float64)
        xm = m.in_project_x(x).reshape(2, 9, 2, 6).permute(0, 2, 1, 3)
        q, k, vv = m.cross_q(xm), m.cross_k(ctx4), m.cross_v(ctx4)
        cross = torch.softmax(q @ k.transpose(-1, -2), dim=-1) @ vv
        want4 = cross.permute(0, 2, 1, 3).reshape(2, 9, 12) @ m.out_linear.weight.t() + m.out_linear.bias
        torch.testing.assert_close(m((x,), ctx4)[0], want4)
