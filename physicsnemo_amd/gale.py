"""GALE (Geometry-Aware Latent Embeddings) attention layers on the PhysicsAttention HIP kernels.

Mirrors ``physicsnemo/nn/module/gale.py``:
  GALE:242-398 (irregular), GALEStructuredMesh2D:447-478, GALEStructuredMesh3D:480-512, ``_gale_cross_init``:401-429,
  ``_gale_forward_impl``:148-239, ``_gale_compute_slice_attention_cross``:87-145, ``_mix_self_and_cross``:43-84,
  GALEBlock:764-1030.

A GALE layer is a PhysicsAttention layer whose slice tokens, besides attending to each other, attend to a context
``(B, H, S_c, D_c)``; the two results are blended (learned sigmoid gate, or concatenation + Linear + GELU) before the
deslice.  Same constructor arguments, parameter names and ``forward(x: tuple, context=None) -> list`` as the
reference, so a reference ``state_dict`` loads unchanged.  Every per-point stage runs on the layer's own kernels (the
fused bf16 MFMA kernels where they serve the shape); the cross-attention + blend is one small kernel per (batch, head).
With gradients required the per-point stages run on the layer's forward / backward kernels and the slice-token stage
(S x D work per (batch, head)) is evaluated with PyTorch ops under autograd (``autograd.GALEFunction``).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as PF
from . import autograd as PA
from .autograd import GALEFunction, GALEPlusFunction
from .transolver import Mlp, TransolverBlock
from .physics_attention import (
    PhysicsAttentionIrregularMesh,
    PhysicsAttentionStructuredMesh2D,
    PhysicsAttentionStructuredMesh3D,
)

_MODES = ("weighted", "concat_project")


def _gale_cross_init(self: nn.Module, dim_head: int, context_dim: int, state_mixing_mode: str) -> None:
    """Cross-attention parameters in the reference's registration order (gale.py:401-429)."""
    self.cross_q = nn.Linear(dim_head, dim_head)
    self.cross_k = nn.Linear(context_dim, dim_head)
    self.cross_v = nn.Linear(context_dim, dim_head)
    self.state_mixing_mode = state_mixing_mode
    if state_mixing_mode == "weighted":
        self.state_mixing = nn.Parameter(torch.tensor(0.0))
    elif state_mixing_mode == "concat_project":
        self.concat_project = nn.Sequential(nn.Linear(2 * dim_head, dim_head), nn.GELU())
    else:
        raise ValueError(f"Invalid state_mixing_mode: {state_mixing_mode!r}. Expected 'weighted' or 'concat_project'.")
    self.context_dim = context_dim


class _GALEForwardMixin:
    """``forward`` shared by the three variants (reference ``_gale_forward_impl``)."""

    def gale_params(self, device: torch.device) -> dict:
        """The cross-attention / blend parameters as float32 contiguous tensors on `device`."""
        def f32(t):
            return t.detach().to(device=device, dtype=torch.float32).contiguous()

        p = {f"cross_{n}_{kind}": f32(getattr(getattr(self, f"cross_{n}"), kind))
             for n in "qkv" for kind in ("weight", "bias")}
        if self.state_mixing_mode == "weighted":
            p["state_mixing"] = f32(self.state_mixing).reshape(1)
        else:
            p["concat_project_weight"] = f32(self.concat_project[0].weight)
            p["concat_project_bias"] = f32(self.concat_project[0].bias)
        return p

    def _check_context(self, context: torch.Tensor, batch: int) -> None:
        if context.ndim != 4 or context.shape[0] != batch or context.shape[1] != self.heads or \
                context.shape[3] != self.context_dim:
            raise ValueError(f"Expected context of shape (B, H, S_c, D_c) = ({batch}, {self.heads}, S_c, "
                             f"{self.context_dim}), got {tuple(context.shape)}")

    def _stage_params(self) -> list:
        p = [self.qkv_project.weight, self.cross_q.weight, self.cross_q.bias, self.cross_k.weight, self.cross_k.bias,
             self.cross_v.weight, self.cross_v.bias]
        if self.state_mixing_mode == "weighted":
            return p + [self.state_mixing]
        return p + [self.concat_project[0].weight, self.concat_project[0].bias]

    def _token_stage(self, tok: torch.Tensor, context: torch.Tensor) -> torch.Tensor:
        """Slice tokens (B,H,S,D) -> blended attended tokens with PyTorch ops in float32 (reference :207-229)."""
        sdpa = torch.nn.functional.scaled_dot_product_attention
        with torch.autocast("cuda", enabled=False):
            tok, context = tok.float(), context.float()
            B, H, S, D = tok.shape
            q, k, v = torch.nn.functional.linear(tok, self.qkv_project.weight.float()).reshape(B, H, S, 3, D).unbind(3)
            self_out = sdpa(q, k, v, is_causal=False)
            cross = sdpa(self.cross_q(tok), self.cross_k(context), self.cross_v(context), is_causal=False)
            if self.state_mixing_mode == "weighted":
                m = torch.sigmoid(self.state_mixing)
                return m * self_out + (1 - m) * cross
            return self.concat_project(torch.cat([self_out, cross], dim=-1))

    def _forward_one_with_grad(self, x: torch.Tensor, context: torch.Tensor) -> torch.Tensor:
        if self.fp8_weights:
            raise NotImplementedError("GALE training with a context is not served with fp8 weights")
        if x.is_cuda and self._wants_fp16(x):
            with torch.autocast("cuda", enabled=False):
                return self._forward_one_with_grad(x.float(), context).to(torch.float16)
        x = self._prepare_input(x)
        dims = self.layer_dims(x)
        if self.plus:
            if not PF.plus_backward_supported(x.dtype, dims):
                raise RuntimeError(f"the backward kernels do not serve this shape: {dims}")
            stage, pt = self._stage_params(), self.proj_temperature
            u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=x.dtype, device=x.device)
            return GALEPlusFunction.apply(
                x, u, context, dims, self.kernel_params(x.dtype, x.device), self._token_stage, len(stage),
                self.in_project_x.weight, self.in_project_x.bias, self.in_project_slice.weight,
                self.in_project_slice.bias, self.temperature, pt[0].weight, pt[0].bias, pt[2].weight, pt[2].bias,
                self.qkv_project.weight, self.out_linear.weight, self.out_linear.bias, *stage)
        if not PF.backward_supported(x.dtype, dims):
            raise RuntimeError(f"the backward kernels do not serve this shape: {dims}")
        stage = self._stage_params()
        return GALEFunction.apply(
            x, context, dims, self.kernel_params(x.dtype, x.device), self._token_stage, len(stage),
            self.in_project_x.weight, self.in_project_x.bias, self.in_project_fx.weight, self.in_project_fx.bias,
            self.in_project_slice.weight, self.in_project_slice.bias, self.temperature, self.qkv_project.weight,
            self.out_linear.weight, self.out_linear.bias, *stage)

    def _forward_one(self, x: torch.Tensor, context: torch.Tensor | None, gp: dict | None) -> torch.Tensor:
        if context is None:  # self-attention only: the plain layer (reference :226-228)
            return super().forward(x)
        if x.is_cuda and self._wants_fp16(x):
            with torch.autocast("cuda", enabled=False):
                return self._forward_one(x.float(), context, gp).to(torch.float16)
        x = self._prepare_input(x)
        dims = self.layer_dims(x)
        p = self.kernel_params(x.dtype, x.device)
        if not self.plus and not self.fp8_weights and PF.query_path(x.dtype, dims) == 1:
            st = PF.MfmaStages(p, dims, x.device)
            st.pack_params()
            if st.fused_groups > 0:
                st.project_softmax_reduce(x)
            else:
                st.project_softmax(x)
                st.slice_reduce()
            st.combine_attention()
            PF.slice_cross_attention_mix(st.tok, st.tok_out, context, gp, dims, tokp=st.tokp)
            y = torch.empty_like(x)
            st.deslice_project(y)
            return y
        if self.fp8_weights:
            raise NotImplementedError("fp8 weights are served by the plain layer only")
        x_mid, fx_mid = PF.project_inputs(x, p, dims)
        if self.plus:
            u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=x.dtype, device=x.device)
            w = PF.slice_softmax_plus(x_mid, u, p, dims)
        else:
            w = PF.slice_softmax(x_mid, p, dims)
        tok, _ = PF.slice_reduce(w, fx_mid, dims)
        self_out = PF.slice_attention(tok, p, dims)
        out_tok = PF.slice_cross_attention_mix(tok, self_out, context, gp, dims)
        return PF.deslice_project(w, out_tok, p, dims)

    def forward_block(self, x: torch.Tensor, residual: torch.Tensor, ln: nn.LayerNorm,
                      context: torch.Tensor | None = None, gp: dict | None = None):
        """One input tensor: layer (with the context) + the caller block's ``+ residual`` and following LayerNorm
        (reference gale.py:1019-1024) -> (fx_new, LayerNorm(fx_new)); inference only.  On the MFMA shapes the add and
        the LayerNorm are the tail of the deslice kernel, as in the plain layer."""
        if context is None:
            return super().forward_block(x, residual, ln)
        if x.is_cuda and self._wants_fp16(x):
            with torch.autocast("cuda", enabled=False):
                return self.forward_block(x.float(), residual.float(), ln, context, gp)
        self._validate(x)
        x = self._prepare_input(x)
        residual = residual.to(x.dtype).contiguous()
        ln_w, ln_b = ln.weight.detach().float().contiguous(), ln.bias.detach().float().contiguous()
        dims = self.layer_dims(x)
        fused = (not self.plus and not self.fp8_weights and not (self.training and self.out_dropout.p > 0)
                 and PF.query_path(x.dtype, dims) == 1)
        if not fused:
            y = self.out_dropout(self._forward_one(x, context, gp)).contiguous()
            return PF.residual_layernorm(y, residual=residual, ln_weight=ln_w, ln_bias=ln_b, ln_eps=ln.eps)
        st = PF.MfmaStages(self.kernel_params(x.dtype, x.device), dims, x.device)
        st.pack_params()
        if st.fused_groups > 0:
            st.project_softmax_reduce(x)
        else:
            st.project_softmax(x)
            st.slice_reduce()
        st.combine_attention()
        PF.slice_cross_attention_mix(st.tok, st.tok_out, context, gp, dims, tokp=st.tokp)
        fx_new, normed = torch.empty_like(x), torch.empty_like(x)
        st.deslice_project(fx_new, residual=residual, ln_weight=ln_w, ln_bias=ln_b, ln_eps=ln.eps, ln_out=normed)
        return fx_new, normed

    def forward(self, x: tuple, context: torch.Tensor | None = None) -> list:
        """x: tuple of (B, N, C) tensors; context (B, H, S_c, D_c) or None -> list of (B, N, C) tensors."""
        if isinstance(x, torch.Tensor):
            raise TypeError("GALE takes a tuple of input tensors (reference gale.py:352-356)")
        if len(x) == 0:
            raise ValueError("Expected non-empty tuple of input tensors")
        for i, t in enumerate(x):
            if t.ndim != 3:
                raise ValueError(f"Expected 3D input tensor (B, N, C) at index {i}, "
                                 f"got {t.ndim}D tensor with shape {tuple(t.shape)}")
        gp = None
        if context is not None:
            for t in x:
                self._validate(t)
            self._check_context(context, x[0].shape[0])
            if torch.is_grad_enabled() and (context.requires_grad or any(self._needs_grad(t) for t in x)):
                return [self.out_dropout(self._forward_one_with_grad(t, context)) for t in x]
            context = context.detach().float().contiguous()
            gp = self.gale_params(context.device)
        return [self.out_dropout(self._forward_one(t, context, gp)) if context is not None
                else self._forward_one(t, None, None) for t in x]  # without a context the plain layer applies it


class GALE(_GALEForwardMixin, PhysicsAttentionIrregularMesh):
    """Irregular-mesh GALE layer (reference gale.py:242-398)."""

    def __init__(self, dim: int, heads: int = 8, dim_head: int = 64, dropout: float = 0.0, slice_num: int = 64,
                 use_te: bool = False, plus: bool = False, context_dim: int = 0, concrete_dropout: bool = False,
                 state_mixing_mode: str = "weighted"):
        super().__init__(dim, heads, dim_head, dropout, slice_num, use_te, plus)
        _gale_cross_init(self, dim_head, context_dim, state_mixing_mode)
        if concrete_dropout:
            raise NotImplementedError("ConcreteDropout is a training-time regulariser; the HIP layer has none")


class GALEStructuredMesh2D(_GALEForwardMixin, PhysicsAttentionStructuredMesh2D):
    """GALE with Conv2d projections on a 2-D grid (reference gale.py:447-478)."""

    def __init__(self, dim: int, spatial_shape: tuple[int, int], heads: int = 8, dim_head: int = 64,
                 dropout: float = 0.0, slice_num: int = 64, kernel: int = 3, use_te: bool = False, plus: bool = False,
                 context_dim: int = 0, state_mixing_mode: str = "weighted"):
        super().__init__(dim, spatial_shape, heads, dim_head, dropout, slice_num, kernel, use_te, plus)
        _gale_cross_init(self, dim_head, context_dim, state_mixing_mode)


class GALEStructuredMesh3D(_GALEForwardMixin, PhysicsAttentionStructuredMesh3D):
    """GALE with Conv3d projections on a 3-D grid (reference gale.py:480-512)."""

    def __init__(self, dim: int, spatial_shape: tuple[int, int, int], heads: int = 8, dim_head: int = 64,
                 dropout: float = 0.0, slice_num: int = 64, kernel: int = 3, use_te: bool = False, plus: bool = False,
                 context_dim: int = 0, state_mixing_mode: str = "weighted"):
        super().__init__(dim, spatial_shape, heads, dim_head, dropout, slice_num, kernel, use_te, plus)
        _gale_cross_init(self, dim_head, context_dim, state_mixing_mode)


class GALEBlock(nn.Module):
    """LayerNorm -> GALE attention (with the shared context) -> +residual -> LayerNorm -> MLP -> +residual, for every
    tensor of the input tuple (reference gale.py:764-1030).  ``attention_type="GALE_FA"`` builds the FLARE form of the
    attention (inference only); ``concrete_dropout`` is not served.  The LayerNorms, the block MLP and its residual add run on the library kernels of the Transolver block."""

    def __init__(self, num_heads: int, hidden_dim: int, dropout: float, act: str = "gelu", mlp_ratio: int = 4,
                 last_layer: bool = False, out_dim: int = 1, slice_num: int = 32, use_te: bool = False,
                 plus: bool = False, context_dim: int = 0, spatial_shape: tuple | None = None,
                 attention_type: str = "GALE", concrete_dropout: bool = False, state_mixing_mode: str = "weighted"):
        super().__init__()
        self.last_layer = last_layer
        self.ln_1 = nn.LayerNorm(hidden_dim)
        if attention_type not in ("GALE", "GALE_FA"):
            raise ValueError(f"Invalid attention type: {attention_type}. Expected 'GALE' or 'GALE_FA'.")
        if concrete_dropout:
            raise NotImplementedError("ConcreteDropout is a training-time regulariser; the HIP block has none")
        common = dict(heads=num_heads, dim_head=hidden_dim // num_heads, dropout=dropout, slice_num=slice_num,
                      use_te=use_te, plus=plus, context_dim=context_dim, state_mixing_mode=state_mixing_mode)
        if attention_type == "GALE_FA":  # FLARE self-attention; inference only (reference :932-943)
            from .flare import GALE_FA

            self.Attn = GALE_FA(hidden_dim, heads=num_heads, dim_head=hidden_dim // num_heads, dropout=dropout,
                                n_global_queries=slice_num, use_te=use_te, context_dim=context_dim,
                                state_mixing_mode=state_mixing_mode)
        elif spatial_shape is None:
            self.Attn = GALE(hidden_dim, **common)
        elif len(spatial_shape) == 2:
            self.Attn = GALEStructuredMesh2D(hidden_dim, spatial_shape=tuple(int(v) for v in spatial_shape), **common)
        elif len(spatial_shape) == 3:
            self.Attn = GALEStructuredMesh3D(hidden_dim, spatial_shape=tuple(int(v) for v in spatial_shape), **common)
        else:
            raise ValueError(f"spatial_shape must be None, length-2, or length-3; got {spatial_shape!r}")
        self.ln_mlp1 = nn.Sequential(nn.LayerNorm(hidden_dim), Mlp(hidden_dim, hidden_dim * mlp_ratio, hidden_dim, act))
        self.attn_dropout = None
        self.ffn_dropout = None
        self._mlp_cache: dict = {}

    # the block MLP (reference mlp_layers.py:101-173) and its kernels are the Transolver block's
    fp8_weights = False  # the shared MLP helpers read it; GALE blocks are served in bf16 / float32 only
    _mlp_kernel_params = TransolverBlock._mlp_kernel_params
    _mlp_kernel_packed = TransolverBlock._mlp_kernel_packed
    _mlp_kernel_serves = TransolverBlock._mlp_kernel_serves
    _mlp_with_grad = TransolverBlock._mlp_with_grad
    _mlp_residual = TransolverBlock._mlp_residual

    def _one(self, fx: torch.Tensor, attn: torch.Tensor, needs_grad: bool) -> torch.Tensor:
        fx1 = attn + fx
        normed = PA.layer_norm(fx1, self.ln_mlp1[0])
        if not needs_grad and self._mlp_kernel_serves(normed):
            packed, b1, b2 = self._mlp_kernel_packed(normed.device, normed.dtype)
            return PF.mlp_forward_packed(normed, packed, b1, b2, residual=fx1.to(normed.dtype).contiguous())
        return self._mlp_with_grad(normed) + fx1

    def forward_chain(self, fx: tuple, normed_in, global_context: torch.Tensor | None, next_ln: nn.LayerNorm | None):
        """Inference, one block inside a chain: takes LayerNorm_1 of every stream if the previous block produced it and
        returns (outputs, next_ln(outputs) or None).  The residual adds and LayerNorms ride on the deslice and block-MLP
        kernels (same arithmetic as `forward`)."""
        attn = self.Attn
        gp = None
        if global_context is not None:
            attn._check_context(global_context, fx[0].shape[0])
            global_context = global_context.detach().float().contiguous()
            gp = attn.gale_params(global_context.device)
        outs, normed_out = [], []
        for i, t in enumerate(fx):
            x_in = normed_in[i] if normed_in is not None else PA.layer_norm(t, self.ln_1)
            fx1, normed = attn.forward_block(x_in, t, self.ln_mlp1[0], global_context, gp)
            out, nxt = self._mlp_residual(fx1, normed, next_ln)
            outs.append(out)
            normed_out.append(nxt)
        return outs, (normed_out if next_ln is not None and all(n is not None for n in normed_out) else None)

    def forward(self, fx: tuple, global_context: torch.Tensor | None) -> list:
        if isinstance(fx, torch.Tensor):
            raise TypeError("GALEBlock takes a tuple of input tensors")
        if len(fx) == 0:
            raise ValueError("Expected non-empty tuple of input tensors")
        for i, t in enumerate(fx):
            if t.ndim != 3:
                raise ValueError(f"Expected 3D input tensor (B, N, C) at index {i}, "
                                 f"got {t.ndim}D tensor with shape {tuple(t.shape)}")
        needs_grad = torch.is_grad_enabled() and (any(t.requires_grad for t in fx) or
                                                  any(p.requires_grad for p in self.parameters()))
        if not needs_grad and torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16:
            fx = tuple(t.to(torch.bfloat16) for t in fx)  # inference: the residual stream in the compute type
        attn = self.Attn(tuple(PA.layer_norm(t, self.ln_1) for t in fx), global_context)
        return [self._one(t, a, needs_grad) for t, a in zip(fx, attn)]
