"""pa_slice_reduce_static (the entry point that allocates nothing) against pa_slice_reduce, through the C ABI.

Both run the same two kernels with the same chunking, so the results are required to be bit-identical; the static
variant keeps its partial sums in a device array that outlives the call, hence two calls in a row, the second on a
smaller input (stale partials of the first call must not leak into it).
"""
import pytest
import torch

from ctypes import byref

from physicsnemo_amd import _lib
from physicsnemo_amd import functional as PF
from gpu_util import announce

pytestmark = pytest.mark.gpu


def _inputs(B, N, H, D, S, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.softmax(torch.randn(B, N, H, S, generator=g) * 2.0, dim=-1).to(dtype).cuda().contiguous()
    fx = torch.randn(B, N, H * D, generator=g).to(dtype).cuda().contiguous()
    return w, fx


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_slice_reduce_matches_workspace_variant(dtype):
    first = (2, 20000, 8, 32, 64)
    second = (1, 777, 4, 16, 32)  # smaller in every dimension: reuses a prefix of the scratch the first call filled
    for seed, (B, N, H, D, S) in enumerate((first, second)):
        announce("static-scratch slice reduce", dtype, B, N, H, D, S)
        dims = PF.LayerDims(B, N, H * D, H, D, S)
        w, fx = _inputs(B, N, H, D, S, dtype, seed)
        want_tok, want_norm = PF.slice_reduce(w, fx, dims)
        tok = torch.full((B, H, S, D), float("nan"), device="cuda")
        norm = torch.full((B, H, S), float("nan"), device="cuda")
        base = torch.cuda.memory_allocated()
        PF.slice_reduce_static(w, fx, dims, out=(tok, norm))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == base  # nothing went through torch's allocator
        assert torch.equal(tok, want_tok)
        assert torch.equal(norm, want_norm)
        # closed form: the norms of a (batch, head) add up to the number of points + 0.01 per slice
        total = (norm.double() - 0.01).sum(-1)
        assert torch.allclose(total, torch.full_like(total, float(N)), rtol=2e-3 if dtype == torch.bfloat16 else 1e-5)


def test_static_scratch_rejects_oversized_problems():
    announce("static-scratch limit")
    lib = _lib.load()
    limit = int(lib.pa_static_scratch_bytes())
    assert limit == 64 << 20
    B, N, H, D, S = 1, 1 << 20, 8, 32, 128  # (512 chunks + 1) x 8 heads x 128 x 33 floats = 69.3 MB > 64 MiB
    dims = PF.LayerDims(B, N, H * D, H, D, S)
    need = (int(lib.pa_reduce_partial_count(byref(dims.c()))) + 1) * B * H * S * (D + 1) * 4  # chunks + their total
    assert need > limit
    dummy = torch.zeros(64, device="cuda")
    with pytest.raises(RuntimeError, match="static scratch"):
        PF.slice_reduce_static(dummy, dummy, dims, out=(dummy, dummy))
