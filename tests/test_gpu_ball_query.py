"""Ball query on the HIP kernel and the GeoTransolver local features built on it, against the oracle.  Bars: neighbour
indices identical (integer work; clouds without exactly equal distances), distances rtol 1e-6, model outputs rtol 2e-4,
gradients rtol 5e-4, bf16 rel-L2 <= 1e-2."""
import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _check(points, queries, radius, K, method=None):
    idx, out, counts, dist = PF.ball_query(points.cuda(), queries.cuda(), radius, K, return_dists=True, method=method)
    ridx, rout, rdist = to.radius_search_nearest(points, queries, radius, K)
    assert idx.dtype == torch.int64 and idx.shape == ridx.shape
    assert torch.equal(idx.cpu(), ridx)
    assert torch.equal(out.cpu(), rout)
    assert torch.allclose(dist.cpu(), rdist, rtol=1e-6, atol=1e-7)
    within = torch.cdist(points, queries, compute_mode="donot_use_mm_for_euclid_dist") <= radius  # (B, Np, Nq)
    assert torch.equal(counts.cpu().long(), within.sum(1).clamp(max=K))
    return counts.cpu()


def test_lattice_problem_of_the_reference():
    """reference test/nn/functional/neighbors/test_radius_search.py:28-47; the construction fixes the answer."""
    announce("ball query lattice")
    base = torch.linspace(0, 10, 11)
    x, y, z = torch.meshgrid(base, base, base, indexing="ij")
    queries = torch.stack([x.flatten(), y.flatten(), z.flatten()], dim=1)
    disp = torch.tensor([[-0.05, 0, 0], [0.1, 0, 0], [0, 0.15, 0], [0, -0.2, 0], [0, 0, 0.25], [0, 0, -0.3]])
    points = (queries[None] + disp[:, None]).reshape(-1, 3)
    Q = queries.shape[0]
    idx, out, counts = PF.ball_query(points[None].cuda(), queries[None].cuda(), 0.17, 5)
    q = torch.arange(Q)
    want = torch.stack([q, Q + q, 2 * Q + q, torch.zeros_like(q), torch.zeros_like(q)], dim=1)
    assert torch.equal(idx[0].cpu(), want)
    assert torch.equal(counts[0].cpu(), torch.full((Q,), 3, dtype=torch.int32))
    assert torch.equal(out[0, :, :3].cpu(), points[want[:, :3]]) and not out[0, :, 3:].any()


@pytest.mark.parametrize("B,Np,Nq,K,radius", [(2, 3000, 1777, 8, 0.25), (1, 5000, 4096, 32, 0.4), (3, 235, 100, 32, 0.6),
                                               (1, 1025, 63, 1, 0.2), (2, 50, 300, 64, 5.0), (1, 7, 5, 16, 10.0)])
@pytest.mark.parametrize("method", ["pairs", "cells"])
def test_against_the_oracle(B, Np, Nq, K, radius, method):
    announce("ball query", B, Np, Nq, K, radius, method)
    torch.manual_seed(Np + K)
    counts = _check(torch.randn(B, Np, 3), torch.randn(B, Nq, 3), radius, K, method)
    if Np > 1000:
        assert counts.min() < K and counts.max() == K  # both partly and fully used lists occur


def test_points_as_their_own_queries_and_radius_zero():
    announce("ball query self")
    torch.manual_seed(3)
    pts = torch.randn(2, 500, 3)
    idx, out, counts, dist = PF.ball_query(pts.cuda(), pts.cuda(), 0.0, 4, return_dists=True)
    assert torch.equal(counts.cpu(), torch.ones(2, 500, dtype=torch.int32))  # every point finds itself, nothing else
    assert torch.equal(idx[..., 0].cpu(), torch.arange(500).expand(2, -1)) and not idx[..., 1:].any()
    assert torch.equal(out[..., 0, :].cpu(), pts) and not dist.any()
    with pytest.raises(RuntimeError):
        PF.ball_query(pts.cuda(), pts.cuda(), 0.1, 65)  # more slots than the kernel keeps
    with pytest.raises(ValueError):
        PF.ball_query(pts.cuda(), pts[:1].cuda(), 0.1, 4)


def test_cell_list_equals_all_pairs_with_ties_flat_clouds_and_far_queries():
    announce("ball query cells vs pairs")
    torch.manual_seed(6)
    half = torch.rand(2, 6000, 3)
    pts = torch.cat([half, half], dim=1).cuda()          # every point twice: equal distances, ordered by index
    pts[1, :, 2] = 0.25                                  # a flat cloud (no extent along z)
    qs = torch.cat([torch.rand(2, 3000, 3), torch.rand(2, 500, 3) * 6 - 3], dim=1).cuda()  # some far outside the box
    for K, radius in ((6, 0.04), (32, 0.08), (8, 0.0)):
        a = PF.ball_query(pts, qs, radius, K, return_dists=True, method="pairs")
        c = PF.ball_query(pts, qs, radius, K, return_dists=True, method="cells")
        for x, y in zip(a, c):
            assert torch.equal(x, y)
        if radius > 0:
            assert int(a[2].max()) == K and int(a[2].min()) == 0
    same = PF.ball_query(pts, pts, 0.0, 4, method="cells")
    assert torch.equal(same[2], torch.full((2, 12000), 2, dtype=torch.int32, device="cuda"))  # itself and its twin


def test_large_cloud_properties():
    """131 072 points: every list ascending and within the radius, counts equal to the brute-force counts on a sample."""
    announce("ball query 131072 points")
    torch.manual_seed(4)
    pts = torch.rand(1, 131072, 3, device="cuda")
    K, radius = 16, 0.03
    idx, out, counts, dist = PF.ball_query(pts, pts, radius, K, return_dists=True)
    used = torch.arange(K, device="cuda") < counts[..., None]
    assert (dist[used] <= radius).all() and not dist[~used].any() and not idx[~used].any()
    assert ((dist[..., 1:] >= dist[..., :-1]) | ~used[..., 1:]).all()
    assert torch.equal(idx[..., 0], torch.arange(131072, device="cuda")[None])  # nearest is the point itself
    recomputed = (out - pts[:, :, None]).norm(dim=-1)
    assert torch.allclose(recomputed[used], dist[used], rtol=1e-5, atol=1e-7)
    sample = torch.arange(0, 131072, 1031, device="cuda")
    within = (((pts[0, sample][:, None] - pts[0][None]) ** 2).sum(-1).sqrt() <= radius).sum(-1)
    assert torch.equal(counts[0, sample].long(), within.clamp(max=K))


def _models(**kw):
    ref = to.OracleGeoTransolver(**kw)
    hip = pn.GeoTransolver(use_te=False, **kw)
    hip.load_state_dict(ref.state_dict())
    return ref, hip.cuda()


def test_bqwarp_module_and_feature_processor():
    announce("BQWarp / GeometricFeatureProcessor")
    torch.manual_seed(5)
    x, grid = torch.randn(2, 400, 3), torch.randn(2, 6, 7, 3)
    ref = to.OracleGeometricFeatureProcessor(0.5, 6, 3, 16)
    hip = pn.GeometricFeatureProcessor(0.5, 6, 3, 16)
    hip.load_state_dict(ref.state_dict())
    hip.cuda()
    assert_fp32_close(hip(x.cuda(), grid.reshape(2, 42, 3).cuda()), ref(x, grid.reshape(2, 42, 3)), "features", rtol=1e-4)
    ridx, rout = ref.bq_warp(x, grid.reshape(2, 42, 3))
    idx, out = hip.bq_warp(x.cuda(), grid.cuda())  # 4-D grids are flattened
    assert torch.equal(idx.cpu(), ridx) and torch.equal(out.cpu(), rout)
    # gradients reach the gathered coordinates
    xg = x.clone().cuda().requires_grad_()
    _, o = hip.bq_warp(xg, grid.reshape(2, 42, 3).cuda())
    o.sum().backward()
    xr = x.clone().requires_grad_()
    ref.bq_warp(xr, grid.reshape(2, 42, 3))[1].sum().backward()
    assert torch.equal(xg.grad.cpu(), xr.grad)
    with pytest.raises(ValueError):
        hip.bq_warp(x.cuda()[..., :2], grid.cuda()[..., :2])


def test_geotransolver_with_local_features_matches_the_oracle():
    """Configuration of reference test/models/geotransolver/test_geotransolver.py:347-395 (radii scaled to clouds that
    have neighbours) and the batch > 1 case of :1120-1165."""
    announce("GeoTransolver local features forward")
    torch.manual_seed(42)
    kw = dict(functional_dim=32, out_dim=4, geometry_dim=3, global_dim=16, n_layers=2, n_hidden=64, n_head=4, mlp_ratio=2,
              slice_num=8, include_local_features=True, radii=[0.3, 0.8], neighbors_in_radius=[8, 32], n_hidden_local=32)
    ref, hip = _models(**kw)
    ref.eval(), hip.eval()
    e, geom, glob = torch.randn(2, 100, 32), torch.randn(2, 235, 3), torch.randn(2, 5, 16)
    with torch.no_grad():
        want = ref(e, e[:, :, :3], glob, geom)
        got, feats = hip(e.cuda(), e[:, :, :3].cuda(), glob.cuda(), geom.cuda(), return_point_features=True)
    assert got.shape == (2, 100, 4) and feats.shape == (2, 100, 64 + 32 * 2)
    assert_fp32_close(got, want, "GeoTransolver with local features", rtol=2e-4)
    with pytest.raises(ValueError, match="Local positions are required"):
        hip(e.cuda(), None, glob.cuda(), geom.cuda())

    announce("GeoTransolver local features, two streams, default radii")
    kw = dict(functional_dim=(16, 12), out_dim=(4, 2), geometry_dim=3, global_dim=8, n_layers=1, n_hidden=32, n_head=4,
              mlp_ratio=1, slice_num=4, include_local_features=True, n_hidden_local=16)
    ref, hip = _models(**kw)
    ref.eval(), hip.eval()
    e1, e2 = torch.randn(2, 64, 16) * 0.2, torch.randn(2, 40, 12) * 0.2
    geom, glob = torch.randn(2, 50, 3) * 0.2, torch.randn(2, 2, 8)
    with torch.no_grad():
        want = ref((e1, e2), (e1[..., :3], e2[..., :3]), glob, geom)
        got = hip((e1.cuda(), e2.cuda()), (e1[..., :3].cuda(), e2[..., :3].cuda()), glob.cuda(), geom.cuda())
    for i in range(2):
        assert_fp32_close(got[i], want[i], f"stream {i}", rtol=2e-4)


def test_geotransolver_with_local_features_trains():
    announce("GeoTransolver local features training step")
    torch.manual_seed(7)
    kw = dict(functional_dim=6, out_dim=3, geometry_dim=3, global_dim=5, n_layers=2, n_hidden=32, n_head=4, mlp_ratio=2,
              slice_num=8, include_local_features=True, radii=[0.5], neighbors_in_radius=[6], n_hidden_local=16)
    ref, hip = _models(**kw)
    ref.train(), hip.train()
    e, geom, glob, target = torch.randn(2, 150, 6), torch.randn(2, 90, 3), torch.randn(2, 4, 5), torch.randn(2, 150, 3)
    ((ref(e, e[..., :3], glob, geom) - target) ** 2).mean().backward()
    ((hip(e.cuda(), e[..., :3].cuda(), glob.cuda(), geom.cuda()) - target.cuda()) ** 2).mean().backward()
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if name.endswith("cross_k.bias"):
            continue  # zero in exact arithmetic
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=5e-4)

    announce("GeoTransolver local features, bf16 autocast")
    hip.eval(), ref.eval()
    with torch.no_grad():
        want = ref(e, e[..., :3], glob, geom)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip(e.cuda(), e[..., :3].cuda(), glob.cuda(), geom.cuda())
    assert_rel_l2(got.float(), want, "bf16 autocast")
