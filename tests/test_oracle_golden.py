"""The oracle against the reference's own golden output files (whole model, both variants)."""
import os

import torch

from oracle.torch_oracle import OracleTransolver

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _load(name):
    return torch.load(os.path.join(GOLD, name), weights_only=True)[0]


def test_structured2d_model_matches_reference_golden():
    # reference: test/models/transolver/test_transolver.py:97-131 (atol 2e-3, rtol 1e-3)
    torch.manual_seed(0)
    model = OracleTransolver(structured_shape=(85, 85), n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1,
                             functional_dim=1, out_dim=1, slice_num=32, ref=1, unified_pos=True,
                             init="rejection")
    fx = torch.randn(4, 85 * 85, 1)
    embedding = torch.randn(4, 85, 85)  # drawn (RNG order) and then replaced by the unified-pos buffer
    with torch.no_grad():
        out = model(fx, embedding)
    gold = _load("transolver2d_output.pth")
    assert out.shape == gold.shape == (4, 7225, 1)
    assert torch.allclose(out, gold, rtol=1e-3, atol=2e-3)
    # far tighter than the reference's own tolerance: the init stream and op order are right
    assert (out - gold).abs().max().item() < 5e-6


def test_irregular_model_matches_reference_golden():
    # reference: test_transolver.py:134-169 (atol 1e-3); the 3-wide tensor goes in as fx, the 2-wide as embedding
    torch.manual_seed(0)
    model = OracleTransolver(structured_shape=None, n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1,
                             functional_dim=2, embedding_dim=3, out_dim=1, slice_num=32, unified_pos=False,
                             init="rejection")
    a = torch.randn(4, 12345, 3)
    b = torch.randn(4, 12345, 2)
    with torch.no_grad():
        out = model(a, b)
    gold = _load("transolver_irregular_output.pth")
    assert out.shape == gold.shape == (4, 12345, 1)
    assert torch.allclose(out, gold, rtol=1e-3, atol=1e-3)
    assert (out - gold).abs().max().item() < 5e-6


def test_flare_structured2d_model_matches_reference_golden():
    # reference: test/models/flare/test_flare.py:124-158 (atol 2e-3)
    from oracle.torch_oracle import OracleFLAREModel
    torch.manual_seed(0)
    model = OracleFLAREModel(structured_shape=(85, 85), n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1,
                             functional_dim=1, out_dim=1, slice_num=32, ref=1, unified_pos=True, init="rejection")
    fx = torch.randn(4, 85 * 85, 1)
    embedding = torch.randn(4, 85, 85)
    with torch.no_grad():
        out = model(fx, embedding)
    gold = _load("flare_2d_output.pth")
    assert out.shape == gold.shape == (4, 7225, 1)
    print("flare 2d max abs diff", (out - gold).abs().max().item())
    assert torch.allclose(out, gold, rtol=1e-3, atol=2e-3)
    assert (out - gold).abs().max().item() < 5e-6


def test_flare_irregular_model_matches_reference_golden():
    # reference: test/models/flare/test_flare.py:161-193 (atol 1e-3)
    from oracle.torch_oracle import OracleFLAREModel
    torch.manual_seed(0)
    model = OracleFLAREModel(structured_shape=None, n_layers=8, n_hidden=64, n_head=4, mlp_ratio=1, functional_dim=2,
                             embedding_dim=3, out_dim=1, slice_num=32, unified_pos=False, init="rejection")
    a = torch.randn(4, 12345, 3)
    b = torch.randn(4, 12345, 2)
    with torch.no_grad():
        out = model(a, b)
    gold = _load("flare_irregular_output.pth")
    assert out.shape == gold.shape == (4, 12345, 1)
    print("flare irregular max abs diff", (out - gold).abs().max().item())
    assert torch.allclose(out, gold, rtol=1e-3, atol=1e-3)
    assert (out - gold).abs().max().item() < 5e-6


def test_geotransolver_basic_matches_reference_golden():
    # reference: test/models/geotransolver/test_geotransolver.py:400-437 (seed 42, atol 1e-3)
    from oracle.torch_oracle import OracleGeoTransolver
    torch.manual_seed(42)
    model = OracleGeoTransolver(functional_dim=32, out_dim=4, geometry_dim=3, global_dim=16, n_layers=2, n_hidden=64,
                                n_head=4, mlp_ratio=2, slice_num=8)
    local_emb = torch.randn(2, 100, 32)
    geometry = torch.randn(2, 235, 3)
    global_emb = torch.randn(2, 5, 16)
    with torch.no_grad():
        out = model(local_emb, local_emb[:, :, :3], global_emb, geometry)
    gold = _load("geotransolver_basic_output.pth")
    assert out.shape == gold.shape == (2, 100, 4)
    print("geotransolver basic max abs diff", (out - gold).abs().max().item())
    assert torch.allclose(out, gold, rtol=1e-3, atol=1e-3)
    assert (out - gold).abs().max().item() < 5e-6


def test_geotransolver_tuple_matches_reference_golden():
    # reference: test_geotransolver.py:440-490 (seed 42, two input streams, atol 2e-3)
    from oracle.torch_oracle import OracleGeoTransolver
    torch.manual_seed(42)
    model = OracleGeoTransolver(functional_dim=(32, 48), out_dim=(4, 6), geometry_dim=3, global_dim=16, n_layers=2,
                                n_hidden=64, n_head=4, mlp_ratio=2, slice_num=8)
    e1, e2 = torch.randn(2, 100, 32), torch.randn(2, 150, 48)
    geometry = torch.randn(2, 235, 3)
    global_emb = torch.randn(2, 5, 16)
    with torch.no_grad():
        out = model((e1, e2), (e1[:, :, :3], e2[:, :, :3]), global_emb, geometry)
    gold = torch.load(os.path.join(GOLD, "geotransolver_tuple_output.pth"), weights_only=True)
    print("golden keys", type(gold), list(gold.keys()) if isinstance(gold, dict) else None)
    for i, o in enumerate(out):
        g = gold[i]
        assert o.shape == g.shape
        print("geotransolver tuple", i, "max abs diff", (o - g).abs().max().item())
        assert torch.allclose(o, g, rtol=1e-3, atol=2e-3)
        assert (o - g).abs().max().item() < 5e-6
