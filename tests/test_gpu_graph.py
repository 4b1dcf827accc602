"""HIP-graph replay of the layer and of a whole model gives the eager results, replay after replay.

Each graph is replayed several times with new inputs and with eager work and synchronisations in between; every
replay is compared bit for bit with the eager call on the same input.
"""
import pytest
import torch

import physicsnemo_amd as pn
from gpu_util import announce

pytestmark = pytest.mark.gpu


def test_graph_replay_of_a_layer_equals_eager():
    announce("graph replay: layer")
    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    layer = pn.PhysicsAttentionIrregularMesh(256, heads=8, dim_head=32, slice_num=64, use_te=False).eval().to(dev)
    xs = [torch.randn(2, 3000, 256, device=dev).bfloat16() for _ in range(4)]
    graphed = pn.GraphedForward(layer, xs[0])
    with torch.no_grad():
        for x in xs + xs[:2]:
            got = graphed(x).clone()
            torch.cuda.synchronize()
            want = layer(x)  # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(got, want)
    with pytest.raises(ValueError):
        graphed(xs[0][:, :100])


def test_graph_replay_of_a_model_equals_eager():
    announce("graph replay: model under bf16 autocast")
    torch.manual_seed(1)
    dev = torch.device("cuda:0")
    model = pn.Transolver(functional_dim=3, embedding_dim=2, out_dim=4, n_layers=3, n_hidden=256, n_head=8,
                          slice_num=32, use_te=False).eval().to(dev)

    def fwd(fx, emb):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return model(fx, emb)

    inputs = [(torch.randn(2, 2500, 3, device=dev), torch.randn(2, 2500, 2, device=dev)) for _ in range(3)]
    graphed = pn.GraphedForward(fwd, *inputs[0])
    with torch.no_grad():
        for fx, emb in inputs + inputs[:1]:
            got = graphed(fx, emb).clone()
            torch.cuda.synchronize()
            want = fwd(fx, emb)
            torch.cuda.synchronize()
            assert torch.equal(got, want)


def test_graph_replay_of_flare_and_geotransolver_models_equals_eager():
    """The reference validates CUDA-graph capture of these models (test_flare.py, test_geotransolver.py
    ``validate_cuda_graphs``); here every replay must equal the eager call bit for bit."""
    announce("graph replay: FLARE model and GeoTransolver")
    torch.manual_seed(2)
    dev = torch.device("cuda:0")
    flare = pn.FLAREModel(functional_dim=2, embedding_dim=3, out_dim=1, n_layers=2, n_hidden=64, n_head=4, mlp_ratio=1,
                          slice_num=32, use_te=False).eval().to(dev)
    geo = pn.GeoTransolver(functional_dim=6, out_dim=3, geometry_dim=3, global_dim=5, n_layers=2, n_hidden=64, n_head=4,
                           mlp_ratio=2, slice_num=8).eval().to(dev)

    def run_geo(e, glob, geom):
        return geo(e, None, glob, geom)

    cases = [
        (flare, [(torch.randn(2, 1234, 2, device=dev), torch.randn(2, 1234, 3, device=dev)) for _ in range(3)]),
        (run_geo, [(torch.randn(2, 700, 6, device=dev), torch.randn(2, 4, 5, device=dev),
                    torch.randn(2, 300, 3, device=dev)) for _ in range(3)]),
    ]
    with torch.no_grad():
        for fn, inputs in cases:
            graphed = pn.GraphedForward(fn, *inputs[0])
            for args in inputs + inputs[:1]:
                got = graphed(*args).clone()
                torch.cuda.synchronize()
                want = fn(*args)
                torch.cuda.synchronize()
                assert torch.equal(got, want)
