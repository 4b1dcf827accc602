"""Pins the oracle's ball query (`radius_search_nearest`) and the local-feature modules built on it: the reference's
lattice problem, whose construction fixes the answer; brute-force loops on small clouds; the shapes the reference's
GeoTransolver tests state for include_local_features=True."""
import math

import torch

from oracle import torch_oracle as to


def _lattice_problem():
    """reference test/nn/functional/neighbors/test_radius_search.py:28-47: queries on the 11^3 integer lattice, points =
    every query displaced by one of six axis offsets of lengths 0.05 ... 0.3."""
    base = torch.linspace(0, 10, 11)
    x, y, z = torch.meshgrid(base, base, base, indexing="ij")
    queries = torch.stack([x.flatten(), y.flatten(), z.flatten()], dim=1)
    disp = torch.tensor([[-0.05, 0, 0], [0.1, 0, 0], [0, 0.15, 0], [0, -0.2, 0], [0, 0, 0.25], [0, 0, -0.3]])
    points = (queries[None] + disp[:, None]).reshape(-1, 3)
    return points, queries


def test_lattice_problem_has_the_neighbours_its_construction_fixes():
    points, queries = _lattice_problem()
    Q = queries.shape[0]
    idx, out, dist = to.radius_search_nearest(points[None], queries[None], 0.17, 5)
    assert idx.shape == (1, Q, 5) and out.shape == (1, Q, 5, 3) and dist.shape == (1, Q, 5)
    q = torch.arange(Q)
    want = torch.stack([q, Q + q, 2 * Q + q, torch.zeros_like(q), torch.zeros_like(q)], dim=1)
    assert torch.equal(idx[0], want)  # displacements 0.05 < 0.1 < 0.15 <= 0.17 < 0.2: three neighbours, nearest first
    assert torch.allclose(dist[0], torch.tensor([0.05, 0.1, 0.15, 0.0, 0.0]).expand(Q, 5), atol=1e-5)
    assert torch.equal(out[0, :, :3], points[want[:, :3]])
    assert torch.equal(out[0, :, 3:], torch.zeros(Q, 2, 3))
    # a radius that takes in all six displaced copies, capped at four
    idx4, _, dist4 = to.radius_search_nearest(points[None], queries[None], 0.31, 4)
    assert torch.equal(idx4[0], torch.stack([q, Q + q, 2 * Q + q, 3 * Q + q], dim=1))
    assert torch.allclose(dist4[0], torch.tensor([0.05, 0.1, 0.15, 0.2]).expand(Q, 4), atol=1e-5)


def test_against_brute_force_loops():
    torch.manual_seed(0)
    B, N, Q, K, radius = 2, 40, 25, 4, 0.9
    points, queries = torch.randn(B, N, 3), torch.randn(B, Q, 3)
    idx, out, dist = to.radius_search_nearest(points, queries, radius, K)
    seen_partial = seen_full = False
    for b in range(B):
        for q in range(Q):
            cand = []
            for n in range(N):
                d = math.sqrt(sum((float(points[b, n, c]) - float(queries[b, q, c])) ** 2 for c in range(3)))
                if d <= radius:
                    cand.append((d, n))
            cand.sort()
            cand = cand[:K]
            seen_partial |= 0 < len(cand) < K
            seen_full |= len(cand) == K
            for k in range(K):
                if k < len(cand):
                    assert int(idx[b, q, k]) == cand[k][1]
                    assert abs(float(dist[b, q, k]) - cand[k][0]) < 1e-5
                    assert torch.equal(out[b, q, k], points[b, cand[k][1]])
                else:
                    assert int(idx[b, q, k]) == 0 and float(dist[b, q, k]) == 0.0
                    assert torch.equal(out[b, q, k], torch.zeros(3))
    assert seen_partial and seen_full  # the case exercises both partly and fully used lists


def test_fewer_points_than_slots_leaves_the_spare_slots_unused():
    torch.manual_seed(1)
    points, queries = torch.rand(1, 3, 3), torch.rand(1, 7, 3)
    idx, out, dist = to.radius_search_nearest(points, queries, 10.0, 5)
    assert idx.shape == (1, 7, 5)
    assert torch.equal(idx[..., 3:], torch.zeros(1, 7, 2, dtype=torch.int64))
    assert torch.equal(out[..., 3:, :], torch.zeros(1, 7, 2, 3))
    assert (dist[..., :3] > 0).all() and torch.equal(dist[..., 3:], torch.zeros(1, 7, 2))


def test_feature_processor_and_extractor_shapes_and_argument_roles():
    """context_projector.py:722-763: context features come from the geometry points' neighbourhoods among the mesh
    points (one token set per radius), local features from the mesh points' neighbourhoods among the geometry points."""
    torch.manual_seed(2)
    ext = to.OracleMultiScaleFeatureExtractor(3, [0.5, 1.0], [4, 6], hidden_dim=16, n_head=2, dim_head=8, slice_num=5)
    coords, geometry = torch.randn(2, 30, 3), torch.randn(2, 45, 3)
    ctx = ext.extract_context_features(coords, geometry)
    assert len(ctx) == 2 and all(c.shape == (2, 2, 5, 8) for c in ctx)
    local = ext.extract_local_features(coords, geometry)
    assert local.shape == (2, 30, 32) and float(local.detach().abs().max()) <= 1.0  # tanh-bounded
    # a mesh point with no geometry point in reach sees all-zero neighbours: its feature is tanh(Mlp(0))
    far = coords.clone()
    far[:, 0] = 100.0
    proc = ext.processors[0]
    zero_feature = torch.tanh(proc.mlp(torch.zeros(1, 12)))
    assert torch.allclose(proc(geometry, far)[:, 0], zero_feature.expand(2, -1), atol=1e-6)


def test_geotransolver_with_local_features_has_the_shapes_the_reference_states():
    """reference test/models/geotransolver/test_geotransolver.py:220-256 and :347-395."""
    torch.manual_seed(42)
    m = to.OracleGeoTransolver(functional_dim=32, out_dim=4, geometry_dim=3, global_dim=16, n_layers=2, n_hidden=64,
                               n_head=4, mlp_ratio=2, slice_num=8, include_local_features=True, radii=[0.05, 0.25],
                               neighbors_in_radius=[8, 32], n_hidden_local=32).eval()
    e = torch.randn(1, 100, 32)
    with torch.no_grad():
        out = m(e, e[:, :, :3], torch.randn(1, 5, 16), torch.randn(1, 235, 3))
    assert out.shape == (1, 100, 4) and torch.isfinite(out).all()
    assert m.blocks[0].ln_1.normalized_shape == (64 + 32 * 2,)
    assert m.context_builder.get_context_dim() == 16 * 2 + 16 + 16
