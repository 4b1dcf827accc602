"""Drop-in PhysicsAttention modules whose forward runs hand-written HIP kernels (libphysattn.so).

Mirrors the constructor signatures, parameter names / registration order and input validation of the
reference classes in physicsnemo/nn/module/physics_attention.py:
  PhysicsAttentionBase            :209-558
  PhysicsAttentionIrregularMesh   :561-660
  PhysicsAttentionStructuredMesh2D:663-783
  PhysicsAttentionStructuredMesh3D:786-907
so that a reference ``state_dict`` loads unchanged and seeded construction consumes the RNG identically.

``plus=True`` (Transolver++) runs through the stage-level kernels, forward and backward.  ``use_te`` is accepted for
signature compatibility and ignored: the HIP kernels are the only backend and there is no CPU path.  Under ``torch.no_grad()`` the fused inference kernels run; with gradients
enabled on tensors that require them the stage-level kernels run and the backward pass is served by the library's
backward kernels (see ``autograd.py``).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as PF
from .autograd import PhysicsAttentionFunction, PhysicsAttentionMfmaFunction, PhysicsAttentionPlusFunction

__all__ = ["PhysicsAttentionBase", "PhysicsAttentionIrregularMesh", "PhysicsAttentionStructuredMesh2D",
           "PhysicsAttentionStructuredMesh3D"]


def _kernel_layout(p: torch.Tensor) -> torch.Tensor:
    """Convolution weights (O, C, k, k[, k]) -> tap-major (O, k, k[, k], C), the order in which the implicit GEMM
    walks its reduction index (`conv_tap_major` of the shape); everything else unchanged."""
    return p.movedim(1, -1) if p.ndim > 2 else p


class PhysicsAttentionBase(nn.Module):
    """Parameters shared by the variants plus the HIP forward (reference base class: :262-327, :501-558)."""

    def __init__(self, dim: int, heads: int, dim_head: int, dropout: float, slice_num: int, use_te: bool, plus: bool):
        super().__init__()
        self.dim = dim
        self.dim_head = dim_head
        self.heads = heads
        self.slice_num = slice_num
        self.plus = plus
        self.scale = dim_head ** -0.5
        self.use_te = use_te

        # registration order follows the reference so state_dict order and RNG draws agree
        self.softmax = nn.Softmax(dim=-1)
        self.dropout = nn.Dropout(dropout)
        self.temperature = nn.Parameter(torch.ones([1, 1, heads, 1]) * 0.5)
        if plus:  # Transolver++: learned per-point temperature offset (reference :287-295)
            self.proj_temperature = nn.Sequential(nn.Linear(dim_head, slice_num), nn.GELU(),
                                                  nn.Linear(slice_num, 1), nn.GELU())
        self.in_project_slice = nn.Linear(dim_head, slice_num)
        torch.nn.init.orthogonal_(self.in_project_slice.weight)
        self.qkv_project = nn.Linear(dim_head, 3 * dim_head, bias=False)
        self.out_linear = nn.Linear(dim_head * heads, dim)
        self.out_dropout = nn.Dropout(dropout)
        self._kernel_param_cache: dict = {}
        self.fp8_weights = False  # see use_fp8_weights()

    def use_fp8_weights(self, enabled: bool = True):
        """Serve bf16 inputs with the three large weights quantised to fp8-e4m3, one scale per output channel
        (scale = max|row| / 448).  The kernels expand them to bf16 MFMA operands; activations stay bf16.
        Irregular-mesh variant only.  No counterpart in the reference."""
        if enabled and (self._conv_geometry()[2] != 0 or self.plus):
            raise NotImplementedError("fp8 weights are served for the irregular-mesh variant with plus=False only")
        self.fp8_weights = bool(enabled)
        self._kernel_param_cache = {}
        return self

    # ---------------------------------------------------------------- parameters in kernel form
    def _conv_geometry(self):
        """(grid_h, grid_w, kernel, grid_d): all zero for the irregular variant, grid_d = 0 for a 2-D grid."""
        return 0, 0, 0, 0

    def layer_dims(self, x: torch.Tensor) -> PF.LayerDims:
        gh, gw, k, gd = self._conv_geometry()
        return PF.LayerDims(x.shape[0], x.shape[1], self.dim, self.heads, self.dim_head, self.slice_num, gh, gw, k, gd,
                            1 if k > 0 else 0)  # kernel_params() hands convolution weights over tap-major

    def kernel_params(self, dtype: torch.dtype, device: torch.device) -> dict:
        """Parameters as the C ABI wants them: the three large weights in ``dtype``, everything else float32,
        contiguous.  Cached until a parameter is modified in place, replaced or moved."""
        named = [
            ("in_project_x_weight", self.in_project_x.weight, True),
            ("in_project_x_bias", self.in_project_x.bias, False),
        ]
        if self.plus:
            named += [("proj_temperature_0_weight", self.proj_temperature[0].weight, False),
                      ("proj_temperature_0_bias", self.proj_temperature[0].bias, False),
                      ("proj_temperature_2_weight", self.proj_temperature[2].weight, False),
                      ("proj_temperature_2_bias", self.proj_temperature[2].bias, False)]
        else:
            named += [("in_project_fx_weight", self.in_project_fx.weight, True),
                      ("in_project_fx_bias", self.in_project_fx.bias, False)]
        named += [
            ("in_project_slice_weight", self.in_project_slice.weight, False),
            ("in_project_slice_bias", self.in_project_slice.bias, False),
            ("temperature", self.temperature, False),
            ("qkv_project_weight", self.qkv_project.weight, False),
            ("out_linear_weight", self.out_linear.weight, True),
            ("out_linear_bias", self.out_linear.bias, False),
        ]
        fp8 = self.fp8_weights and dtype == torch.bfloat16
        stamp = (dtype, device, fp8) + tuple((p.data_ptr(), p._version, p.dtype) for _, p, _ in named)
        hit = self._kernel_param_cache.get("stamp")
        if hit == stamp:
            return self._kernel_param_cache["params"]
        with torch.no_grad():
            params = {
                name: _kernel_layout(p.detach()).to(device=device, dtype=dtype if big else torch.float32)
                .contiguous().reshape(-1).clone()
                for name, p, big in named
            }
            if fp8:
                for name, p, big in named:
                    if big:
                        q, scale = PF.quantize_e4m3_per_channel(p.detach().reshape(p.shape[0], -1))
                        params[name] = q.to(device).reshape(-1)
                        params[name.replace("_weight", "_scale")] = scale.to(device)
        self._kernel_param_cache = {"stamp": stamp, "params": params}
        return params

    # ---------------------------------------------------------------- forward
    def _validate(self, x: torch.Tensor) -> None:
        # same checks and messages as the reference forward (:516-526)
        if x.ndim != 3:
            raise ValueError(
                f"Expected 3D input tensor (B, N, C), got {x.ndim}D tensor with shape {tuple(x.shape)}")
        if x.shape[-1] != self.dim:
            raise ValueError(f"Expected input feature dimension {self.dim}, got {x.shape[-1]}")

    def _check_spatial(self, x: torch.Tensor) -> None:
        pass

    def _needs_grad(self, x: torch.Tensor) -> bool:
        return torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))

    def _prepare_input(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_cuda:
            raise RuntimeError("physicsnemo_amd PhysicsAttention runs on GPU tensors only (no CPU fallback)")
        if torch.is_autocast_enabled("cuda"):
            ac = torch.get_autocast_dtype("cuda")
            if ac != torch.bfloat16:
                raise TypeError(f"autocast dtype {ac} is not supported (bfloat16, or float16 served in float32)")
            x = x.to(torch.bfloat16)
        if x.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"expected float32 or bfloat16 input, got {x.dtype}")
        self._check_spatial(x)
        return x.contiguous()

    def _forward_with_grad(self, x: torch.Tensor) -> torch.Tensor:
        """Training path: stage-level kernels forward, backward kernels in `autograd.PhysicsAttentionFunction`."""
        if self.fp8_weights:
            raise RuntimeError("fp8 weights are an inference format: no gradients flow through them")
        if self.plus:
            return self._forward_plus_with_grad(x, None)
        dims = self.layer_dims(x)
        if not PF.backward_supported(x.dtype, dims):
            raise RuntimeError(f"the backward kernels do not serve this shape: {dims}")
        fn = PhysicsAttentionMfmaFunction if PF.mfma_backward_supported(x.dtype, dims) else PhysicsAttentionFunction
        return fn.apply(
            x, dims, self.kernel_params(x.dtype, x.device), self.in_project_x.weight, self.in_project_x.bias,
            self.in_project_fx.weight, self.in_project_fx.bias, self.in_project_slice.weight,
            self.in_project_slice.bias, self.temperature, self.qkv_project.weight, self.out_linear.weight,
            self.out_linear.bias)

    def _forward_plus_with_grad(self, x: torch.Tensor, noise_u: torch.Tensor | None) -> torch.Tensor:
        """Training path of Transolver++: `autograd.PhysicsAttentionPlusFunction` on the general kernels."""
        dims = self.layer_dims(x)
        if not PF.plus_backward_supported(x.dtype, dims):
            raise RuntimeError(f"the backward kernels do not serve this shape: {dims}")
        if noise_u is None:
            noise_u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=x.dtype, device=x.device)
        pt = self.proj_temperature
        return PhysicsAttentionPlusFunction.apply(
            x, noise_u.detach().to(x.dtype).contiguous(), dims, self.kernel_params(x.dtype, x.device),
            self.in_project_x.weight, self.in_project_x.bias, self.in_project_slice.weight, self.in_project_slice.bias,
            self.temperature, pt[0].weight, pt[0].bias, pt[2].weight, pt[2].bias, self.qkv_project.weight,
            self.out_linear.weight, self.out_linear.bias)

    @staticmethod
    def _wants_fp16(x: torch.Tensor) -> bool:
        """float16 inputs / float16 autocast (the reference's AMP smoke tests): there are no float16 kernels; the layer
        then computes in float32 with autocast off and hands back float16, i.e. at least the precision asked for."""
        if x.dtype == torch.float16:
            return True
        return torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.float16

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """(B, N, C) -> (B, N, C); replaces reference forward :501-558.  With gradients enabled on tensors that
        require them the differentiable path runs (stage-level kernels + backward kernels)."""
        if x.is_cuda and self._wants_fp16(x):
            with torch.autocast("cuda", enabled=False):
                return self.forward(x.float()).to(torch.float16)
        self._validate(x)
        if x.numel() == 0:
            # no points (or an empty batch): the reference's tensor ops return the empty (B, N, C) result
            self._check_spatial(x)
            return self._prepare_input(x).clone()
        needs_grad = self._needs_grad(x)
        x = self._prepare_input(x)
        if needs_grad:
            y = self._forward_with_grad(x)
        elif self.plus:
            return self.forward_with_noise(x, None)
        else:
            y = PF.layer_forward(x, self.kernel_params(x.dtype, x.device), self.layer_dims(x))
        return self.out_dropout(y)  # identity unless training with dropout > 0 (reference :499)

    def forward_with_noise(self, x: torch.Tensor, noise_u: torch.Tensor | None, stages: bool = False):
        """Transolver++ forward (reference :166-170, :530-532) through the stage-level kernels.  ``noise_u``
        (B, N, H, S): the uniform samples behind the Gumbel noise; ``None`` draws them from torch's generator of the
        input's device exactly as the reference's ``torch.rand_like(slice_projections)`` does."""
        if not self.plus:
            raise RuntimeError("forward_with_noise is the plus=True path")
        self._validate(x)
        if self._needs_grad(x) and not stages:
            return self.out_dropout(self._forward_plus_with_grad(self._prepare_input(x), noise_u))
        x = self._prepare_input(x)
        dims = self.layer_dims(x)
        p = self.kernel_params(x.dtype, x.device)
        if noise_u is None:
            noise_u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=x.dtype, device=x.device)
        noise_u = noise_u.to(x.dtype).contiguous()
        if not stages and not self.fp8_weights and PF.layer_forward_plus_supported(x.dtype, dims):
            return self.out_dropout(PF.layer_forward_plus(x, noise_u, p, dims))  # staged bf16 MFMA kernels
        x_mid, fx_mid = PF.project_inputs(x, p, dims)
        w = PF.slice_softmax_plus(x_mid, noise_u, p, dims)
        tok, norm = PF.slice_reduce(w, fx_mid, dims)
        tok_out = PF.slice_attention(tok, p, dims)
        y = PF.deslice_project(w, tok_out, p, dims)
        if stages:
            H, D = self.heads, self.dim_head
            return dict(x_mid=x_mid.view(dims.B, dims.N, H, D), w=w, tok=tok, norm=norm, tok_out=tok_out, y=y)
        return self.out_dropout(y)

    def forward_block(self, x: torch.Tensor, residual: torch.Tensor, ln: nn.LayerNorm):
        """Layer + the caller block's ``+ residual`` and following LayerNorm in one pass
        (physicsnemo/models/transolver/transolver.py:300-303).  Returns (fx_new, LayerNorm(fx_new)); with ln = None
        (inference on the library kernels only) just fx_new."""
        if x.is_cuda and self._wants_fp16(x):
            with torch.autocast("cuda", enabled=False):  # float32 inside, as the residual stream of the caller is
                return self.forward_block(x.float(), residual.float(), ln)
        self._validate(x)
        if x.numel() == 0:
            y = self.forward(x)
            return (y + residual.to(y.dtype), y.clone()) if ln is not None else y + residual.to(y.dtype)
        if ln is None and (self.plus or (self.training and self.out_dropout.p > 0) or self._needs_grad(x)):
            return self.forward(x) + residual
        if self.plus and not self._needs_grad(x) and not self.fp8_weights and not (self.training and self.out_dropout.p > 0):
            xp = self._prepare_input(x)
            dims = self.layer_dims(xp)
            if PF.layer_forward_plus_supported(xp.dtype, dims):
                u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=xp.dtype, device=xp.device)
                return PF.layer_forward_plus(
                    xp, u, self.kernel_params(xp.dtype, xp.device), dims, residual=residual.to(xp.dtype).contiguous(),
                    ln_weight=ln.weight.detach().float().contiguous(), ln_bias=ln.bias.detach().float().contiguous(),
                    ln_eps=ln.eps)
        # dropout sits between the layer and the residual add; with gradients required the differentiable layer path
        # runs and the tail is formed by tensor ops, so the result carries a grad_fn
        if self.plus or (self.training and self.out_dropout.p > 0) or self._needs_grad(x):
            y = self.forward(x)
            fx_new = y + residual.to(y.dtype)
            normed = torch.nn.functional.layer_norm(fx_new.float(), ln.normalized_shape, ln.weight, ln.bias, ln.eps)
            return fx_new, normed.to(y.dtype)
        x = self._prepare_input(x)
        residual = residual.to(x.dtype).contiguous()
        if ln is None:
            return PF.layer_forward(x, self.kernel_params(x.dtype, x.device), self.layer_dims(x), residual=residual)[0]
        return PF.layer_forward(
            x, self.kernel_params(x.dtype, x.device), self.layer_dims(x), residual=residual,
            ln_weight=ln.weight.detach().float().contiguous(), ln_bias=ln.bias.detach().float().contiguous(),
            ln_eps=ln.eps)

    def forward_stages(self, x: torch.Tensor) -> dict:
        """Stage-by-stage forward through the natural-layout entry points; returns every intermediate."""
        self._validate(x)
        x = self._prepare_input(x)
        dims = self.layer_dims(x)
        p = self.kernel_params(x.dtype, x.device)
        x_mid, fx_mid = PF.project_inputs(x, p, dims)
        w = PF.slice_softmax(x_mid, p, dims)
        tok, norm = PF.slice_reduce(w, fx_mid, dims)
        tok_out = PF.slice_attention(tok, p, dims)
        y = PF.deslice_project(w, tok_out, p, dims)
        H, D = self.heads, self.dim_head
        return dict(x_mid=x_mid.view(dims.B, dims.N, H, D), fx_mid=fx_mid.view(dims.B, dims.N, H, D), w=w, tok=tok,
                    norm=norm, tok_out=tok_out, y=y)


class PhysicsAttentionIrregularMesh(PhysicsAttentionBase):
    """Unstructured point clouds: nn.Linear projections (reference :606-627)."""

    def __init__(self, dim: int, heads: int = 8, dim_head: int = 64, dropout: float = 0.0, slice_num: int = 64,
                 use_te: bool = True, plus: bool = False):
        super().__init__(dim, heads, dim_head, dropout, slice_num, use_te, plus)
        inner_dim = dim_head * heads
        self.in_project_x = nn.Linear(dim, inner_dim)
        if not plus:
            self.in_project_fx = nn.Linear(dim, inner_dim)


class PhysicsAttentionStructuredMesh2D(PhysicsAttentionBase):
    """Row-major 2D grids: k x k Conv2d projections, stride 1, zero padding k//2 (reference :721-742).

    ``forward`` takes the flattened ``(B, H_s*W_s, C)`` tensor with token n = i*W_s + j (:768-783).
    """

    def __init__(self, dim: int, spatial_shape: tuple[int, int], heads: int = 8, dim_head: int = 64,
                 dropout: float = 0.0, slice_num: int = 64, kernel: int = 3, use_te: bool = True, plus: bool = False):
        super().__init__(dim, heads, dim_head, dropout, slice_num, use_te, plus)
        inner_dim = dim_head * heads
        self.H = spatial_shape[0]
        self.W = spatial_shape[1]
        self.kernel = kernel
        self.in_project_x = nn.Conv2d(dim, inner_dim, kernel, 1, kernel // 2)
        if not plus:
            self.in_project_fx = nn.Conv2d(dim, inner_dim, kernel, 1, kernel // 2)

    def _conv_geometry(self):
        return self.H, self.W, self.kernel, 0

    def _check_spatial(self, x: torch.Tensor) -> None:
        # the reference reshapes with x.view(B, H, W, C) (:772): same failure for a wrong token count
        x.view(x.shape[0], self.H, self.W, x.shape[-1])


class PhysicsAttentionStructuredMesh3D(PhysicsAttentionBase):
    """Row-major 3D grids: k x k x k Conv3d projections, stride 1, zero padding k//2 (reference :857-867).

    ``forward`` takes the flattened ``(B, H_s*W_s*D_s, C)`` tensor with token n = (i*W_s + j)*D_s + l (:896-907).
    """

    def __init__(self, dim: int, spatial_shape: tuple[int, int, int], heads: int = 8, dim_head: int = 64,
                 dropout: float = 0.0, slice_num: int = 32, kernel: int = 3, use_te: bool = True, plus: bool = False):
        super().__init__(dim, heads, dim_head, dropout, slice_num, use_te, plus)
        inner_dim = dim_head * heads
        self.H = spatial_shape[0]
        self.W = spatial_shape[1]
        self.D = spatial_shape[2]
        self.kernel = kernel
        self.in_project_x = nn.Conv3d(dim, inner_dim, kernel, 1, kernel // 2)
        if not plus:
            self.in_project_fx = nn.Conv3d(dim, inner_dim, kernel, 1, kernel // 2)

    def _conv_geometry(self):
        return self.H, self.W, self.kernel, self.D

    def _check_spatial(self, x: torch.Tensor) -> None:
        # the reference reshapes with x.view(B, H, W, D, C) (:896): same failure for a wrong token count
        x.view(x.shape[0], self.H, self.W, self.D, x.shape[-1])
