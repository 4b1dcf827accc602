"""GPU parity of the fused block MLP (pa_mlp_forward, through the C ABI) against the fp32 CPU oracle.

Bar for bf16: relative L2 error <= 1e-2 against the fp32 oracle evaluated on the same bf16-rounded inputs/weights.
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_oracle as to
from physicsnemo_amd import functional as PF
from gpu_util import announce, assert_fp32_close, assert_rel_l2

pytestmark = pytest.mark.gpu


def _case(rows_shape, C, Fh, seed=0, scale=1.0):
    torch.manual_seed(seed)
    ref = to.OracleMlp(C, Fh, C).eval()
    with torch.no_grad():
        for p in ref.parameters():  # bf16-representable weights: both sides compute with the same numbers
            p.mul_(scale)
        ref.layers[0].weight.copy_(ref.layers[0].weight.bfloat16().float())
        ref.layers[2].weight.copy_(ref.layers[2].weight.bfloat16().float())
    u = torch.randn(*rows_shape, C).bfloat16()
    res = torch.randn(*rows_shape, C).bfloat16()
    gamma, beta = torch.rand(C) + 0.5, torch.randn(C) * 0.1
    dev = torch.device("cuda:0")
    args = dict(
        u=u.to(dev), w1=ref.layers[0].weight.detach().bfloat16().to(dev).contiguous(),
        b1=ref.layers[0].bias.detach().float().to(dev), w2=ref.layers[2].weight.detach().bfloat16().to(dev).contiguous(),
        b2=ref.layers[2].bias.detach().float().to(dev))
    return ref, u, res, gamma, beta, args


@pytest.mark.parametrize("rows_shape,C,Fh", [
    ((1, 4096), 256, 1024), ((2, 1000), 256, 1024), ((1, 257), 256, 256), ((3, 77), 128, 512), ((1, 1), 256, 1024),
    ((1, 5000), 128, 128), ((1, 20000), 256, 512),
    ((1, 4096), 512, 2048), ((2, 777), 512, 2048), ((1, 1), 512, 64), ((1, 33000), 512, 512),
    ((1, 300), 512, 5632), ((1, 300), 256, 6912), ((1, 300), 128, 8192),  # the widest hidden layers that fit LDS
])
def test_mlp_matches_fp32_oracle(rows_shape, C, Fh):
    announce("mlp", rows_shape, C, Fh)
    ref, u, res, gamma, beta, args = _case(rows_shape, C, Fh)
    assert PF.mlp_supported(torch.bfloat16, u.numel() // C, C, Fh)
    dev = args["u"].device
    with torch.no_grad():
        want = ref(u.float())
        want_sum = want + res.float()
        want_ln = F.layer_norm(want_sum, (C,), gamma, beta, 1e-5)
        y = PF.mlp_forward(**args)
        y2, ln2 = PF.mlp_forward(**args, residual=res.to(dev), ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
        y3 = PF.mlp_forward(**args, residual=res.to(dev))
        y4, ln4 = PF.mlp_forward(**args, ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
    assert y.dtype == torch.bfloat16 and y.shape == u.shape
    assert torch.isfinite(y.float()).all()
    assert_rel_l2(y, want, "mlp output")
    assert_rel_l2(y2, want_sum, "mlp + residual")
    assert_rel_l2(ln2, want_ln, "LayerNorm(mlp + residual)")
    assert torch.equal(y3, y2)
    assert torch.equal(y4, y)
    assert_rel_l2(ln4, F.layer_norm(want, (C,), gamma, beta, 1e-5), "LayerNorm(mlp)")


def test_mlp_gelu_tails_and_determinism():
    announce("mlp large activations / determinism")
    # large pre-activations exercise both saturated ends of the erf and the sign handling
    ref, u, res, gamma, beta, args = _case((1, 3000), 256, 1024, seed=3, scale=6.0)
    with torch.no_grad():
        want = ref(u.float())
        y = PF.mlp_forward(**args)
        y_again = PF.mlp_forward(**args)
    assert_rel_l2(y, want, "mlp output, large activations")
    assert torch.equal(y, y_again)
    # rows are independent: a prefix gives the same bits
    args_prefix = dict(args, u=args["u"][:, :777].contiguous())
    with torch.no_grad():
        y_prefix = PF.mlp_forward(**args_prefix)
    assert torch.equal(y_prefix, y[:, :777])


def test_mlp_packed_weights_give_the_same_bits():
    announce("mlp, weights packed once")
    for C, Fh in ((256, 1024), (512, 2048), (128, 256)):
        ref, u, res, gamma, beta, args = _case((1, 1500), C, Fh, seed=5)
        dev = args["u"].device
        with torch.no_grad():
            y, ln = PF.mlp_forward(**args, residual=res.to(dev), ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
            packed = PF.mlp_pack(args["w1"], args["w2"])
            for _ in range(2):  # the packed buffer is read only
                y2, ln2 = PF.mlp_forward_packed(args["u"], packed, args["b1"], args["b2"], residual=res.to(dev),
                                                ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
                assert torch.equal(y, y2) and torch.equal(ln, ln2)


def test_mlp_rejects_unsupported():
    assert not PF.mlp_supported(torch.float32, 100, 256, 1024)
    assert not PF.mlp_supported(torch.bfloat16, 100, 384, 1536)
    assert not PF.mlp_supported(torch.bfloat16, 100, 512, 8192)
    assert not PF.mlp_supported(torch.bfloat16, 100, 256, 8192)
    assert not PF.mlp_supported(torch.bfloat16, 100, 256, 1000)


@pytest.mark.parametrize("rows_shape,Fh", [((1, 4096), 128), ((2, 1000), 512), ((1, 1), 128), ((3, 77), 256),
                                           ((4, 7225), 128), ((1, 300), 1024)])
def test_mlp_fp32_matches_oracle(rows_shape, Fh):
    # float32 at C = 128: the row kernel on split-bf16 products; ragged row counts, idle waves (77 rows: 3 tiles),
    # several chunks of 128 hidden features, cfg1's shape (4 x 7225 rows, mlp_ratio 1)
    announce("mlp fp32", rows_shape, Fh)
    C = 128
    torch.manual_seed(1)
    ref = to.OracleMlp(C, Fh, C).eval()
    u, res = torch.randn(*rows_shape, C), torch.randn(*rows_shape, C)
    gamma, beta = torch.rand(C) + 0.5, torch.randn(C) * 0.1
    dev = torch.device("cuda:0")
    args = dict(u=u.to(dev), w1=ref.layers[0].weight.detach().to(dev).contiguous(), b1=ref.layers[0].bias.detach().to(dev),
                w2=ref.layers[2].weight.detach().to(dev).contiguous(), b2=ref.layers[2].bias.detach().to(dev))
    assert PF.mlp_supported(torch.float32, u.numel() // C, C, Fh)
    with torch.no_grad():
        want = ref(u)
        want_sum = want + res
        want_ln = F.layer_norm(want_sum, (C,), gamma, beta, 1e-5)
        want64 = ref.double()(u.double())
        y = PF.mlp_forward(**args)
        y2, ln2 = PF.mlp_forward(**args, residual=res.to(dev), ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
        y3 = PF.mlp_forward(**args, residual=res.to(dev))
        y4, ln4 = PF.mlp_forward(**args, ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
        packed = PF.mlp_pack(args["w1"], args["w2"])
        y5 = PF.mlp_forward_packed(args["u"], packed, args["b1"], args["b2"])
    assert y.dtype == torch.float32 and y.shape == u.shape
    assert_fp32_close(y, want, "mlp output")
    assert_fp32_close(y2, want_sum, "mlp + residual")
    assert_fp32_close(ln2, want_ln, "LayerNorm(mlp + residual)")
    assert_fp32_close(ln4, F.layer_norm(want, (C,), gamma, beta, 1e-5), "LayerNorm(mlp)")
    assert torch.equal(y3, y2) and torch.equal(y4, y) and torch.equal(y5, y)
    # float32 accuracy of the split products: as close to the float64 result as float32 tensor ops are
    e_hip, e_f32 = to.rel_l2(y.double().cpu(), want64), to.rel_l2(want.double(), want64)
    assert e_hip < 4 * e_f32 + 2e-7, (e_hip, e_f32)


def test_mlp_fp32_unsupported_shapes():
    assert not PF.mlp_supported(torch.float32, 100, 256, 1024)  # float32 is served at C = 128 only
    assert not PF.mlp_supported(torch.float32, 100, 128, 192)   # hidden features in chunks of 128


@pytest.mark.parametrize("rows_shape,c_in,Fh", [((4, 7225), 3, 256), ((1, 100), 1, 128), ((2, 333), 7, 256), ((1, 5000), 8, 384)])
def test_preprocess_mlp_fp32_matches_oracle(rows_shape, c_in, Fh):
    # the model's preprocess Mlp (a few input features per point -> F -> 128) and the first LayerNorm in one launch
    announce("preprocess mlp fp32", rows_shape, c_in, Fh)
    C = 128
    torch.manual_seed(2)
    ref = to.OracleMlp(c_in, Fh, C).eval()
    u = torch.randn(*rows_shape, c_in)
    gamma, beta = torch.rand(C) + 0.5, torch.randn(C) * 0.1
    dev = torch.device("cuda:0")
    args = dict(u=u.to(dev), w1=ref.layers[0].weight.detach().to(dev).contiguous(), b1=ref.layers[0].bias.detach().to(dev),
                w2=ref.layers[2].weight.detach().to(dev).contiguous(), b2=ref.layers[2].bias.detach().to(dev))
    assert PF.preprocess_supported(torch.float32, u.numel() // c_in, c_in, Fh, C)
    with torch.no_grad():
        want = ref(u)
        want_ln = F.layer_norm(want, (C,), gamma, beta, 1e-5)
        y = PF.preprocess_forward(**args)
        y2, ln2 = PF.preprocess_forward(**args, ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
    assert y.shape == (*rows_shape, C) and y.dtype == torch.float32
    assert_fp32_close(y, want, "preprocess mlp output")
    assert_fp32_close(ln2, want_ln, "LayerNorm(preprocess mlp)")
    assert torch.equal(y2, y)
    assert not PF.preprocess_supported(torch.float32, 100, 9, 256, C)
    assert not PF.preprocess_supported(torch.float32, 100, 8, 512, C)  # the first Linear no longer fits beside the ring
    assert not PF.preprocess_supported(torch.float32, 100, 3, 256, 256)


@pytest.mark.parametrize("rows_shape,c_in,Fh,C", [
    ((8, 32768), 5, 512, 256), ((1, 20000), 7, 512, 256), ((1, 8192), 7, 1024, 512), ((2, 333), 1, 32, 256),
    ((1, 1), 16, 64, 512), ((1, 70001), 9, 1024, 512), ((3, 257), 3, 1728, 256),  # the widest hidden layer whose first Linear fits LDS
])
def test_preprocess_mlp_bf16_matches_oracle(rows_shape, c_in, Fh, C):
    # the model's preprocess Mlp at the bf16 configurations (cfg2 / cfg4: 5 or 7 inputs -> 512 -> 256; cfg5: 7 -> 1024
    # -> 512) with the hidden layer kept on chip, and the first LayerNorm (in the kernel's epilogue at 256 channels)
    announce("preprocess mlp bf16", rows_shape, c_in, Fh, C)
    torch.manual_seed(5)
    ref = to.OracleMlp(c_in, Fh, C).eval()
    with torch.no_grad():
        for lin in (ref.layers[0], ref.layers[2]):  # bf16-representable weights: both sides compute with the same numbers
            lin.weight.copy_(lin.weight.bfloat16().float())
    u = torch.randn(*rows_shape, c_in).bfloat16()
    gamma, beta = torch.rand(C) + 0.5, torch.randn(C) * 0.1
    dev = torch.device("cuda:0")
    args = dict(u=u.to(dev), w1=ref.layers[0].weight.detach().bfloat16().to(dev).contiguous(),
                b1=ref.layers[0].bias.detach().to(dev), w2=ref.layers[2].weight.detach().bfloat16().to(dev).contiguous(),
                b2=ref.layers[2].bias.detach().to(dev))
    assert PF.preprocess_supported(torch.bfloat16, u.numel() // c_in, c_in, Fh, C)
    with torch.no_grad():
        want = ref(u.float())
        want_ln = F.layer_norm(want, (C,), gamma, beta, 1e-5)
        y = PF.preprocess_forward(**args)
        y2, ln2 = PF.preprocess_forward(**args, ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
    assert y.shape == (*rows_shape, C) and y.dtype == torch.bfloat16
    assert torch.isfinite(y.float()).all()
    assert_rel_l2(y, want, "bf16 preprocess mlp output", report=True)
    assert_rel_l2(ln2, want_ln, "LayerNorm(bf16 preprocess mlp)")
    assert torch.equal(y2, y)
    assert not PF.preprocess_supported(torch.bfloat16, 100, 17, 512, 256)
    assert not PF.preprocess_supported(torch.bfloat16, 100, 7, 500, 256)
    assert not PF.preprocess_supported(torch.bfloat16, 100, 7, 1760, 256)  # W1 no longer fits beside the stream
    assert not PF.preprocess_supported(torch.bfloat16, 100, 7, 512, 128)


@pytest.mark.parametrize("rows_shape,C,Fh", [((1, 4096), 256, 1024), ((2, 1001), 256, 512), ((1, 1), 256, 1024),
                                             ((1, 4097), 512, 2048), ((3, 300), 512, 512)])
def test_mlp_normalises_its_input_rows(rows_shape, C, Fh):
    """pa_mlp_forward_packed_ln: y = u + Mlp(LayerNorm(u)) with the LayerNorm applied inside the kernel, against the
    oracle's op sequence (transolver.py:303) and against the two-call sequence (LayerNorm kernel, then the MLP kernel)."""
    announce("mlp with input LayerNorm", rows_shape, C, Fh)
    ref, _, _, gamma, beta, args = _case(rows_shape, C, Fh, seed=3)
    dev = args["u"].device
    torch.manual_seed(9)
    u = (torch.randn(*rows_shape, C) * 1.7 + 0.4).bfloat16()  # a residual stream: not centred, not unit variance
    g_in, b_in = torch.rand(C) + 0.5, torch.randn(C) * 0.2
    assert PF.mlp_input_ln_supported(torch.bfloat16, u.numel() // C, C, Fh)
    assert not PF.mlp_input_ln_supported(torch.bfloat16, 100, 128, 512)
    with torch.no_grad():
        normed = F.layer_norm(u.float(), (C,), g_in, b_in, 1e-5)
        want = u.float() + ref(normed)
        want_ln = F.layer_norm(want, (C,), gamma, beta, 1e-5)
        packed = PF.mlp_pack(args["w1"], args["w2"])
        ud = u.to(dev)
        in_ln = (g_in.to(dev), b_in.to(dev), 1e-5)
        y, ln = PF.mlp_forward_packed(ud, packed, args["b1"], args["b2"], residual=ud, in_ln=in_ln,
                                      ln_weight=gamma.to(dev), ln_bias=beta.to(dev))
        y_plain = PF.mlp_forward_packed(ud, packed, args["b1"], args["b2"], residual=ud, in_ln=in_ln)
        # the two-call sequence the fused form replaces
        _, normed_dev = PF.residual_layernorm(ud.clone(), ln_weight=in_ln[0], ln_bias=in_ln[1], ln_eps=1e-5)
        y2 = PF.mlp_forward_packed(normed_dev, packed, args["b1"], args["b2"], residual=ud)
    assert_rel_l2(y, want, "u + Mlp(LayerNorm(u)), LayerNorm inside the kernel", report=True)
    assert_rel_l2(ln, want_ln, "next LayerNorm of the same")
    assert torch.equal(y_plain, y)
    assert_rel_l2(y, y2.float().cpu(), "against the LayerNorm kernel followed by the MLP kernel", tol=3e-3)


@pytest.mark.parametrize("C,Fh", [(128, 512), (256, 1024), (512, 2048)])
def test_mlp_repack_reads_e4m3_weights(C, Fh):
    """pa_mlp_pack_e4m3 (the repacking kernel fed e4m3 bytes + per-row scales) writes the very fragments pa_mlp_pack
    writes for the dequantised weights rounded to bf16: fp8 weights cost one expansion per parameter set, in the repack."""
    announce("mlp e4m3 repack", C, Fh)
    torch.manual_seed(C)
    dev = torch.device("cuda:0")
    w1, w2 = (torch.randn(Fh, C) / C ** 0.5).to(dev), (torch.randn(C, Fh) / Fh ** 0.5).to(dev)
    w1[3] = 0  # an all-zero row: scale floor, zero bytes
    q1, s1 = PF.quantize_e4m3_per_channel(w1)
    q2, s2 = PF.quantize_e4m3_per_channel(w2)
    d1, d2 = PF.dequantize_e4m3_per_channel(q1, s1), PF.dequantize_e4m3_per_channel(q2, s2)
    # the searched scale never does worse than max|row| / 448
    q1p, s1p = PF.quantize_e4m3_per_channel(w1, search=0)
    err = lambda d, w: float((d - w).norm() / w.norm())
    assert err(d1, w1) <= err(PF.dequantize_e4m3_per_channel(q1p, s1p), w1) + 1e-9
    assert err(d1, w1) < 2.6e-2 and err(d2, w2) < 2.6e-2  # 3 mantissa bits: 2.2e-2 .. 2.55e-2 whatever the scale
    want = PF.mlp_pack(d1.bfloat16().contiguous(), d2.bfloat16().contiguous())
    got = PF.mlp_pack_e4m3(q1, s1, q2, s2)
    assert torch.equal(got, want)
    u = torch.randn(1, 999, C).bfloat16().to(dev)
    b1, b2 = torch.randn(Fh).to(dev) * 0.1, torch.randn(C).to(dev) * 0.1
    y8 = PF.mlp_forward_packed(u, got, b1, b2)
    y16 = PF.mlp_forward(u, d1.bfloat16().contiguous(), b1, d2.bfloat16().contiguous(), b2)
    assert torch.equal(y8, y16)
