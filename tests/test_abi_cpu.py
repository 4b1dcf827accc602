"""CPU-side checks of the C-ABI library and the host modules (no kernel is launched)."""
import ctypes
import os
import re

import pytest
import torch

import physicsnemo_amd as pn
from physicsnemo_amd import _lib
from physicsnemo_amd import functional as PF

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "physattn.h")).read()
    declared = set(re.findall(r"\b(pa_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations parsed"
    assert declared == set(_lib.EXPORTED)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.pa_version() >= 100
    assert lib.pa_status_string(0) == b"ok"


def test_marker_ranges_follow_the_environment():
    """PA_ROCTX=1 turns the roctx ranges on (the marker library is opened at run time); without it they are off."""
    import subprocess
    import sys
    code = "from physicsnemo_amd import _lib; print(_lib.load().pa_markers_enabled())"
    for value, expected in ((None, "0"), ("0", "0"), ("1", "1")):
        env = {k: v for k, v in os.environ.items() if k != "PA_ROCTX"}
        if value is not None:
            env["PA_ROCTX"] = value
        out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == expected, (value, out.stdout, out.stderr)


def _shape(**kw):
    base = dict(B=1, N=64, C=64, H=2, D=32, S=16, grid_h=0, grid_w=0, conv_k=0)
    base.update(kw)
    return _lib.PaShape(**base)


def test_argument_errors_are_codes_not_crashes():
    lib = _lib.load()
    assert lib.pa_workspace_bytes(0, None) == -1
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(N=0))) == -2
    assert lib.pa_workspace_bytes(7, ctypes.byref(_shape())) == -3
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(D=4096))) == -3
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(conv_k=3, grid_h=8, grid_w=9))) == -2  # 72 != 64
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(conv_k=2, grid_h=8, grid_w=8))) == -3
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(conv_k=3, grid_h=4, grid_w=4, grid_d=4))) > 0  # 64 points
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape(conv_k=3, grid_h=4, grid_w=4, grid_d=5))) == -2
    assert lib.pa_workspace_bytes(0, ctypes.byref(_shape())) > 0
    # null tensors / params are rejected before anything touches a device
    s = _shape()
    assert lib.pa_layer_forward(0, ctypes.byref(s), None, None, None, None, None, None, 0, None) == -1
    p = _lib.PaParams(*([256] * 10))
    assert lib.pa_layer_forward(0, ctypes.byref(s), ctypes.byref(p), None, None, None, None, None, 0, None) == -1
    assert lib.pa_layer_forward(0, ctypes.byref(s), ctypes.byref(p), 256, 256, None, None, 256, 1, None) == -5
    assert lib.pa_layer_forward(0, ctypes.byref(s), ctypes.byref(p), 260, 256, None, None, 256, 1 << 40, None) == -4
    assert lib.pa_status_string(-5) == b"workspace too small"


def test_mfma_layer_forward_rejects_missing_biases_and_mixed_scales():
    """The fused kernels sum fx_mid without its bias and the combine step adds it from `p`: a parameter set without
    in_project_fx_bias is an error, not a silently bias-free result.  Scales are all set (e4m3 weights) or all NULL."""
    lib = _lib.load()
    assert lib.pa_version() >= 110
    s = _shape(B=1, N=4096, C=256, H=8, D=32, S=64)
    names = [n for n, _ in _lib.PaParams._fields_]

    def params(**null):
        vals = {n: (256 if not n.endswith("_scale") else None) for n in names}
        vals.update(null)
        return _lib.PaParams(*[vals[n] for n in names])

    big = 1 << 40
    ok_args = (256, 256, 256, None, None, 256, big, None)  # blob, x, y, tail, tokens, workspace, bytes, stream
    p = params(in_project_fx_bias=None)
    assert lib.pa_mfma_layer_forward(ctypes.byref(s), ctypes.byref(p), *ok_args) == -1
    p = params(qkv_project_weight=None)
    assert lib.pa_mfma_layer_forward(ctypes.byref(s), ctypes.byref(p), *ok_args) == -1
    # S = 128 runs the packed-tile sequence, which reads every parameter itself
    s128 = _shape(B=1, N=4096, C=256, H=8, D=32, S=128)
    for missing in ("in_project_x_bias", "in_project_fx_bias", "out_linear_bias", "in_project_x_weight"):
        p = params(**{missing: None})
        assert lib.pa_mfma_layer_forward(ctypes.byref(s128), ctypes.byref(p), *ok_args) == -1, missing
    # repacking: one or two of the three scales is a malformed parameter set
    p = params(in_project_x_scale=256)
    assert lib.pa_mfma_pack_params(ctypes.byref(s), ctypes.byref(p), 256, None) == -1
    p = params(in_project_x_scale=256, in_project_fx_scale=256)
    assert lib.pa_mfma_pack_params(ctypes.byref(s), ctypes.byref(p), 256, None) == -1
    # the e4m3 repack of the MLP weights: argument errors are codes
    assert lib.pa_mlp_pack_e4m3(256, 1024, None, 256, 256, 256, 256, big, None) == -1
    assert lib.pa_mlp_pack_e4m3(256, 1024, 256, None, 256, 256, 256, big, None) == -1
    assert lib.pa_mlp_pack_e4m3(256, 1024, 260, 256, 256, 256, 256, big, None) == -4   # bytes must be 8-byte aligned
    assert lib.pa_mlp_pack_e4m3(256, 1024, 256, 256, 256, 256, 256, 16, None) == -5
    assert lib.pa_mlp_pack_e4m3(200, 1024, 256, 256, 256, 256, 256, big, None) == -3
    assert lib.pa_mlp_pack_e4m3(0, 1024, 256, 256, 256, 256, 256, big, None) == -2


def test_module_signatures_state_dict_and_seeded_init_match_oracle():
    from oracle import torch_oracle as to
    torch.manual_seed(7)
    a = pn.PhysicsAttentionIrregularMesh(64, heads=4, dim_head=16, slice_num=8, use_te=False)
    torch.manual_seed(7)
    b = to.OraclePhysicsAttentionIrregularMesh(64, heads=4, dim_head=16, slice_num=8)
    sa, sb = a.state_dict(), b.state_dict()
    assert list(sa) == list(sb)
    for k in sa:
        assert torch.equal(sa[k], sb[k]), k
    torch.manual_seed(7)
    a2 = pn.PhysicsAttentionStructuredMesh2D(32, (5, 6), heads=2, dim_head=16, slice_num=8, kernel=3, use_te=False)
    torch.manual_seed(7)
    b2 = to.OraclePhysicsAttentionStructuredMesh2D(32, (5, 6), heads=2, dim_head=16, slice_num=8, kernel=3)
    assert list(a2.state_dict()) == list(b2.state_dict())
    assert all(torch.equal(a2.state_dict()[k], b2.state_dict()[k]) for k in a2.state_dict())
    assert (a2.H, a2.W) == (5, 6)
    torch.manual_seed(7)
    a3 = pn.PhysicsAttentionStructuredMesh3D(32, (3, 4, 5), heads=2, dim_head=16, slice_num=8, kernel=3, use_te=False)
    torch.manual_seed(7)
    b3 = to.OraclePhysicsAttentionStructuredMesh3D(32, (3, 4, 5), heads=2, dim_head=16, slice_num=8, kernel=3)
    assert list(a3.state_dict()) == list(b3.state_dict())
    assert all(torch.equal(a3.state_dict()[k], b3.state_dict()[k]) for k in a3.state_dict())
    assert (a3.H, a3.W, a3.D) == (3, 4, 5) and tuple(a3.in_project_x.weight.shape) == (32, 32, 3, 3, 3)
    # reference defaults: heads=8, dim_head=64, slice_num=64, use_te=True accepted
    d = pn.PhysicsAttentionIrregularMesh(128)
    assert (d.heads, d.dim_head, d.in_project_slice.out_features) == (8, 64, 64)
    assert isinstance(d.temperature, torch.nn.Parameter) and tuple(d.temperature.shape) == (1, 1, 8, 1)
    assert torch.all(d.temperature == 0.5)
    # orthogonal slice projection: rows of a (16, 32) weight are orthonormal (reference test_physics_attention.py:667-685)
    o = pn.PhysicsAttentionIrregularMesh(64, heads=2, dim_head=32, slice_num=16)
    wwt = o.in_project_slice.weight @ o.in_project_slice.weight.T
    assert torch.allclose(wwt, torch.eye(16), atol=1e-5)


def test_model_state_dict_matches_oracle_and_loads_legacy_keys():
    from oracle import torch_oracle as to
    kw = dict(functional_dim=2, out_dim=3, embedding_dim=3, n_layers=2, n_hidden=32, n_head=4, slice_num=8, mlp_ratio=2)
    torch.manual_seed(1)
    m = pn.Transolver(use_te=False, **kw)
    torch.manual_seed(1)
    o = to.OracleTransolver(**kw)
    assert list(m.state_dict()) == list(o.state_dict())
    assert all(torch.equal(m.state_dict()[k], o.state_dict()[k]) for k in m.state_dict())
    sd = {k.replace("layers.0", "linear_pre").replace("layers.2", "linear_post"): v for k, v in o.state_dict().items()}
    assert any("linear_pre" in k for k in sd)
    m.load_state_dict(sd)  # legacy MLP key names (reference transolver.py:92-97)
    s2 = pn.Transolver(functional_dim=1, out_dim=1, n_layers=1, n_hidden=16, n_head=2, structured_shape=(4, 5),
                       unified_pos=True, ref=2, use_te=False)
    assert tuple(s2.embedding.shape) == (1, 20, 4)
    assert torch.equal(s2.embedding, to.unified_pos_grid((4, 5), 2))


def test_validation_messages_and_no_cpu_fallback():
    from oracle import torch_oracle as to
    m = pn.PhysicsAttentionIrregularMesh(8, heads=2, dim_head=4, slice_num=3, use_te=False)
    with pytest.raises(ValueError, match="Expected 3D input"):
        m(torch.randn(4, 8))
    with pytest.raises(ValueError, match="Expected input feature dimension 8, got 6"):
        m(torch.randn(1, 4, 6))
    with torch.no_grad(), pytest.raises(RuntimeError, match="GPU tensors only"):
        m(torch.randn(1, 4, 8))
    with pytest.raises(RuntimeError, match="GPU tensors only"):
        m(torch.randn(1, 4, 8))  # gradients enabled: still no CPU path
    # Transolver++: no in_project_fx, proj_temperature registered right after temperature (reference :285-295, :622-627)
    torch.manual_seed(3)
    mp = pn.PhysicsAttentionIrregularMesh(8, heads=2, dim_head=4, slice_num=3, plus=True, use_te=False)
    torch.manual_seed(3)
    op = to.OraclePhysicsAttentionIrregularMesh(8, heads=2, dim_head=4, slice_num=3, plus=True)
    assert list(mp.state_dict()) == list(op.state_dict())
    assert all(torch.equal(mp.state_dict()[k], op.state_dict()[k]) for k in mp.state_dict())
    assert "in_project_fx.weight" not in mp.state_dict()
    with pytest.raises(ValueError, match="n_hidden % n_head"):
        pn.Transolver(functional_dim=1, out_dim=1, embedding_dim=1, n_hidden=30, n_head=4)
    with pytest.raises(ValueError, match="structured_shape when using unified_pos"):
        pn.Transolver(functional_dim=1, out_dim=1, unified_pos=True)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libphysattn.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "physicsnemo_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f


def test_integration_stub_structs_match_the_binding():
    """The ctypes stub printed in the integration guide must lay out pa_shape / pa_params / pa_block_tail like the header."""
    import re
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()

    def fields(cls):
        body = text[text.index(f"class {cls}(Structure):"):]
        body = body[:body.index("\nclass ", 1) if "\nclass " in body[1:] else None]
        body = body[:body.index("\n\n")] if "\n\n" in body else body
        return re.findall(r'"([a-z_A-Z0-9]+)"', body)

    assert fields("pa_shape") == [n for n, _ in _lib.PaShape._fields_]
    assert fields("pa_params") == [n for n, _ in _lib.PaParams._fields_]
    assert fields("pa_block_tail") == [n for n, _ in _lib.PaBlockTail._fields_]
    assert fields("pa_mlp_params") == [n for n, _ in _lib.PaMlpParams._fields_]


def test_mdlus_checkpoints_round_trip_and_legacy_tar(tmp_path):
    """.mdlus ingestion (reference core/module.py:446-1070): the zip format the reference writes by default, its legacy
    tar format, constructor arguments from args.json, weights via a loader that executes nothing."""
    import io
    import json
    import tarfile
    from physicsnemo_amd import checkpoint as ck
    torch.manual_seed(4)
    kw = dict(functional_dim=2, out_dim=3, embedding_dim=2, n_layers=2, n_hidden=32, n_head=4, slice_num=8, mlp_ratio=2,
              structured_shape=(4, 5), use_te=False)
    m = pn.Transolver(**kw)
    path = str(tmp_path / "model.mdlus")
    m.save(path)
    args, meta, state = ck.read_mdlus(path)
    assert args["__name__"] == "Transolver" and args["__module__"] == "physicsnemo.models.transolver.transolver"
    assert args["__args__"]["n_hidden"] == 32 and args["__args__"]["structured_shape"] == [4, 5]
    assert "mdlus_file_version" in meta and list(state) == list(m.state_dict())
    m2 = pn.Transolver.from_checkpoint(path)
    assert m2.structured_shape == (4, 5)
    assert all(torch.equal(a, b) for a, b in zip(m.state_dict().values(), m2.state_dict().values()))
    with pytest.raises(ValueError, match="cannot be overridden"):
        pn.Transolver.from_checkpoint(path, override_args={"n_hidden": 64})
    # the legacy tar layout, assembled by hand as the reference's save(legacy_format=True) lays it out
    tar_path = str(tmp_path / "legacy.mdlus")
    buf = io.BytesIO()
    torch.save(m.state_dict(), buf)
    with tarfile.open(tar_path, "w") as tar:
        for name, data in (("model.pt", buf.getvalue()), ("args.json", json.dumps(args).encode()),
                           ("metadata.json", json.dumps(meta).encode())):
            info = tarfile.TarInfo(name)
            info.size = len(data)
            tar.addfile(info, io.BytesIO(data))
    m3 = pn.Transolver(**kw)
    m3.load(tar_path)
    assert all(torch.equal(a, b) for a, b in zip(m.state_dict().values(), m3.state_dict().values()))
    with pytest.raises(ValueError, match=".mdlus"):
        m.save(str(tmp_path / "model.pt"))
    bad = tmp_path / "bad.mdlus"
    bad.write_bytes(b"not an archive")
    with pytest.raises(IOError):
        ck.read_mdlus(str(bad))


def test_time_input_model_matches_oracle_layout_and_embedding_closed_forms():
    from oracle import torch_oracle as to
    kw = dict(functional_dim=2, out_dim=1, embedding_dim=2, n_layers=2, n_hidden=32, n_head=4, slice_num=8, mlp_ratio=2)
    torch.manual_seed(5)
    m = pn.Transolver(time_input=True, use_te=False, **kw)
    torch.manual_seed(5)
    o = to.OracleTransolver(time_input=True, **kw)
    assert list(m.state_dict()) == list(o.state_dict())
    assert all(torch.equal(m.state_dict()[k], o.state_dict()[k]) for k in m.state_dict())
    assert "time_embed.freqs" in m.state_dict() and "time_fc.2.bias" in m.state_dict()
    # the embedding: f_k = 10000^(-k/16) for 32 channels; t = 0 gives [1..1 | 0..0]; cos first, then sin
    emb = o.time_embed
    k = torch.arange(16, dtype=torch.float64)
    assert torch.allclose(emb.freqs.double(), 10000.0 ** (-k / 16), rtol=1e-6)
    e0 = emb(torch.zeros(3))
    assert torch.equal(e0[:, :16], torch.ones(3, 16)) and torch.equal(e0[:, 16:], torch.zeros(3, 16))
    t = torch.tensor([0.3, 7.0])
    e = emb(t).double()
    assert torch.allclose(e[:, 0], torch.cos(t.double()), atol=1e-6) and torch.allclose(e[:, 16], torch.sin(t.double()), atol=1e-6)
    assert torch.allclose(e[:, :16] ** 2 + e[:, 16:] ** 2, torch.ones(2, 16, dtype=torch.float64), atol=1e-6)
    # a time_fc whose last Linear is zero leaves the model equal to the one evaluated without time
    fx, pos = torch.randn(2, 20, 2), torch.randn(2, 20, 2)
    with torch.no_grad():
        o.time_fc[2].weight.zero_()
        o.time_fc[2].bias.zero_()
        assert torch.equal(o(fx, pos, time=t), o(fx, pos))
    # old checkpoints without the freqs buffer still load (reference embedding_layers.py:135-140)
    sd = {k: v for k, v in o.state_dict().items() if k != "time_embed.freqs"}
    m.load_state_dict(sd)
    with pytest.raises(ValueError, match="time_input=False"):
        pn.Transolver(use_te=False, **kw)(fx, pos, time=t)


def test_gale_modules_share_the_reference_state_dict_contract():
    """GALE variants: constructor arguments, parameter names / order / shapes as in gale.py:242-512 (the oracle holds
    the same contract, pinned against the reference's registration order in test_oracle_gale.py)."""
    from oracle import torch_oracle as to
    for mode in ("weighted", "concat_project"):
        torch.manual_seed(0)
        ref = to.OracleGALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5, state_mixing_mode=mode)
        torch.manual_seed(0)
        hip = pn.GALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5, state_mixing_mode=mode, use_te=False)
        assert list(hip.state_dict()) == list(ref.state_dict())
        for k, v in ref.state_dict().items():  # same seed, same construction order: same initial values
            assert torch.equal(hip.state_dict()[k], v), k
        hip.load_state_dict(ref.state_dict())
    g2 = pn.GALEStructuredMesh2D(16, (3, 4), heads=2, dim_head=8, slice_num=4, kernel=3, context_dim=5)
    assert g2.in_project_x.weight.shape == (16, 16, 3, 3) and g2.cross_k.weight.shape == (8, 5)
    g3 = pn.GALEStructuredMesh3D(16, (2, 3, 4), heads=2, dim_head=8, slice_num=4, kernel=3, context_dim=5,
                                 state_mixing_mode="concat_project")
    assert g3.in_project_x.weight.ndim == 5 and g3.concat_project[0].weight.shape == (8, 16)
    with pytest.raises(ValueError, match="Invalid state_mixing_mode"):
        pn.GALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5, state_mixing_mode="sum")
    with pytest.raises(RuntimeError, match="GPU"), torch.no_grad():
        pn.GALE(16, heads=2, dim_head=8, slice_num=4, context_dim=5)((torch.randn(1, 7, 16),), torch.randn(1, 2, 3, 5))
