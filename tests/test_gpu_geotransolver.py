"""GeoTransolver (context projectors + GALE blocks) on the HIP kernels: the reference's own golden outputs, the fp32
oracle, gradients.  Bars: the reference's atol for its golden files (1e-3 / 2e-3) and rtol 2e-4 against them and the
oracle; gradients rtol 5e-4; bf16 rel-L2 <= 1e-2."""
import os

import pytest
import torch

from oracle import torch_oracle as to
import physicsnemo_amd as pn
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _hip_from(ref, **kw):
    """The HIP model with the oracle's weights; its own construction draws from the generator, so the golden tests
    build it only after the inputs are drawn."""
    hip = pn.GeoTransolver(use_te=False, **kw)
    hip.load_state_dict(ref.state_dict())
    return hip.cuda()


def _models(**kw):
    ref = to.OracleGeoTransolver(**kw)
    return ref, _hip_from(ref, **kw)


def test_geotransolver_reproduces_reference_golden_outputs():
    """reference test/models/geotransolver/test_geotransolver.py:400-490: seed 42, same construction and input draws."""
    announce("GeoTransolver golden basic")
    torch.manual_seed(42)
    kw = dict(functional_dim=32, out_dim=4, geometry_dim=3, global_dim=16, n_layers=2, n_hidden=64, n_head=4,
              mlp_ratio=2, slice_num=8)
    ref = to.OracleGeoTransolver(**kw)
    e, geom, glob = torch.randn(2, 100, 32), torch.randn(2, 235, 3), torch.randn(2, 5, 16)
    hip = _hip_from(ref, **kw)
    gold = torch.load(os.path.join(GOLD, "geotransolver_basic_output.pth"), weights_only=True)[0]
    hip.eval()
    with torch.no_grad():
        out = hip(e.cuda(), e[:, :, :3].cuda(), glob.cuda(), geom.cuda()).cpu()
    assert torch.allclose(out, gold, rtol=1e-3, atol=1e-3)
    assert_fp32_close(out, gold, "GeoTransolver vs golden", rtol=2e-4)

    announce("GeoTransolver golden tuple")
    torch.manual_seed(42)
    kw = dict(functional_dim=(32, 48), out_dim=(4, 6), geometry_dim=3, global_dim=16, n_layers=2, n_hidden=64, n_head=4,
              mlp_ratio=2, slice_num=8)
    ref = to.OracleGeoTransolver(**kw)
    e1, e2 = torch.randn(2, 100, 32), torch.randn(2, 150, 48)
    geom, glob = torch.randn(2, 235, 3), torch.randn(2, 5, 16)
    hip = _hip_from(ref, **kw)
    gold = torch.load(os.path.join(GOLD, "geotransolver_tuple_output.pth"), weights_only=True)
    hip.eval()
    with torch.no_grad():
        outs = hip((e1.cuda(), e2.cuda()), (e1[:, :, :3].cuda(), e2[:, :, :3].cuda()), glob.cuda(), geom.cuda())
    assert isinstance(outs, tuple) and len(outs) == 2
    for i, o in enumerate(outs):
        assert torch.allclose(o.cpu(), gold[i], rtol=1e-3, atol=2e-3)
        assert_fp32_close(o, gold[i], f"GeoTransolver stream {i} vs golden", rtol=2e-4)


def test_geotransolver_training_step_return_options_and_checkpoint(tmp_path):
    announce("GeoTransolver training step")
    torch.manual_seed(1)
    kw = dict(functional_dim=6, out_dim=3, geometry_dim=3, global_dim=5, n_layers=2, n_hidden=32, n_head=4, mlp_ratio=2,
              slice_num=8)
    ref, hip = _models(**kw)
    ref.train(), hip.train()
    e, geom, glob, target = torch.randn(2, 150, 6), torch.randn(2, 90, 3), torch.randn(2, 4, 5), torch.randn(2, 150, 3)
    ((ref(e, None, glob, geom) - target) ** 2).mean().backward()
    ((hip(e.cuda(), None, glob.cuda(), geom.cuda()) - target.cuda()) ** 2).mean().backward()
    grads = dict(hip.named_parameters())
    for name, p in ref.named_parameters():
        if name.endswith("cross_k.bias"):
            continue  # zero in exact arithmetic
        assert grads[name].grad is not None, name
        assert_fp32_close(grads[name].grad, p.grad, f"grad {name}", rtol=5e-4)
    hip.eval()
    with torch.no_grad():
        out, states, feats = hip(e.cuda(), None, glob.cuda(), geom.cuda(), return_embedding_states=True,
                                 return_point_features=True)
    assert out.shape == (2, 150, 3) and states.shape == (2, 4, 8, 16) and feats.shape == (2, 150, 32)
    with pytest.raises(NotImplementedError):
        hip(e.cuda(), None, glob.cuda(), geom.cuda(), time=torch.zeros(2))
    with pytest.raises(ValueError, match="Expected 1 local_embedding"):
        hip((e.cuda(), e.cuda()), None, glob.cuda(), geom.cuda())
    path = str(tmp_path / "geo.mdlus")
    hip.save(path)
    again = pn.GeoTransolver.from_checkpoint(path).cuda().eval()
    with torch.no_grad():
        assert torch.equal(again(e.cuda(), None, glob.cuda(), geom.cuda()), out)


def test_bf16_geotransolver_on_the_fused_kernels():
    announce("bf16 GeoTransolver")
    torch.manual_seed(2)
    ref, hip = _models(functional_dim=8, out_dim=2, geometry_dim=3, global_dim=6, n_layers=2, n_hidden=256, n_head=8,
                       mlp_ratio=4, slice_num=32)
    e, geom, glob = torch.randn(1, 5000, 8), torch.randn(1, 3000, 3), torch.randn(1, 7, 6)
    hip.eval()
    with torch.no_grad():
        want = ref(e, None, glob, geom)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = hip(e.cuda(), None, glob.cuda(), geom.cuda())
    assert_rel_l2(got, want, "bf16 GeoTransolver", tol=1e-2)


def test_float16_autocast_is_served_in_float32():
    """The reference's AMP checks run these models under float16 autocast; there are no float16 kernels, the layers
    then compute in float32 (at least the precision asked for)."""
    announce("fp16 autocast: GeoTransolver, FLARE model")
    torch.manual_seed(3)
    geo = pn.GeoTransolver(functional_dim=6, out_dim=3, geometry_dim=3, global_dim=5, n_layers=2, n_hidden=32, n_head=4,
                           mlp_ratio=2, slice_num=8).eval().cuda()
    flare = pn.FLAREModel(functional_dim=2, embedding_dim=3, out_dim=1, n_layers=2, n_hidden=32, n_head=4, mlp_ratio=1,
                          slice_num=8, use_te=False).eval().cuda()
    e, glob, geom = torch.randn(2, 300, 6).cuda(), torch.randn(2, 4, 5).cuda(), torch.randn(2, 100, 3).cuda()
    a, b = torch.randn(2, 300, 2).cuda(), torch.randn(2, 300, 3).cuda()
    with torch.no_grad():
        want_g, want_f = geo(e, None, glob, geom), flare(a, b)
        with torch.autocast("cuda", dtype=torch.float16):
            got_g, got_f = geo(e, None, glob, geom), flare(a, b)
    assert torch.isfinite(got_g).all() and torch.isfinite(got_f).all()
    assert_rel_l2(got_g, want_g, "GeoTransolver under fp16 autocast", tol=5e-3)
    assert_rel_l2(got_f, want_f, "FLARE model under fp16 autocast", tol=5e-3)
