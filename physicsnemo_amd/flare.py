"""FLARE (Fast Low-rank Attention Routing Engine) attention layer on the HIP kernels.

Mirrors ``physicsnemo/nn/module/flare_attention.py``: FLARE:118-255, ``_flare_self_attention``:38-72.  Same constructor
arguments, parameter names and ``forward(x) -> (B, N, C)``, so a reference ``state_dict`` loads unchanged.

The layer is two attention passes through S learned global queries per head, with scores
``A[b,n,h,s] = k[b,n,h,:] . q_global[h,s,:]`` (scale 1): the queries gather ``z = softmax_n(A)^T v`` from all points,
then every point reads ``y = softmax_s(A) z`` back.  That is the slice aggregation and the deslice of the
PhysicsAttention layer with two normalisations of one score matrix, so it runs on the same kernels:

  A, v   two row GEMMs straight from x: in_project_x, self_k / self_v and q_global are linear maps applied one after
         the other, composed once per parameter set into two weight matrices (H*S x C and H*D x C)
  z      exp(A - max_n A) (``pa_flare_column_weights``), then the slice aggregation kernels
  y      row softmax of A in place (``pa_flare_softmax_rows``), then deslice + out_linear

With gradients required ``autograd.FlareFunction`` runs the same kernels forward and, backward, the per-point FLARE
kernel plus the layer family's row / weight-gradient GEMMs; the weight composition is then done with tensor ops under
autograd so the gradients reach q_global, self_k, self_v and in_project_x.  ``use_te`` is accepted and ignored.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as PF
from .autograd import FlareFunction
from .transolver import Mlp, Transolver, TransolverBlock


class FLARE(nn.Module):
    def __init__(self, dim: int, heads: int = 8, dim_head: int = 64, dropout: float = 0.0,
                 n_global_queries: int = 64, use_te: bool = False):
        super().__init__()
        self.use_te = use_te
        self.dim, self.heads, self.dim_head, self.n_global_queries = dim, heads, dim_head, n_global_queries
        self.scale = 1.0
        inner_dim = dim_head * heads
        # registration order follows the reference so state_dict order and RNG draws agree
        self.q_global = nn.Parameter(torch.randn(1, heads, n_global_queries, dim_head))
        self.in_project_x = nn.Linear(dim, inner_dim)
        self.self_k = nn.Linear(dim_head, dim_head)
        self.self_v = nn.Linear(dim_head, dim_head)
        self.out_linear = nn.Linear(inner_dim, dim)
        self.out_dropout = nn.Dropout(dropout)
        self._cache: dict = {}
        self.use_mfma = True  # bf16 inference on the MFMA kernels where they serve the shape (False: general kernels)

    def kernel_params(self, dtype: torch.dtype, device: torch.device) -> dict:
        """The composed GEMM weights (in `dtype`; biases float32) and out_linear, cached per parameter version."""
        ps = [self.q_global, self.in_project_x.weight, self.in_project_x.bias, self.self_k.weight, self.self_k.bias,
              self.self_v.weight, self.self_v.bias, self.out_linear.weight, self.out_linear.bias]
        stamp = (dtype, device) + tuple((p.data_ptr(), p._version) for p in ps)
        if self._cache.get("stamp") == stamp:
            return self._cache["params"]
        H, D, S, C = self.heads, self.dim_head, self.n_global_queries, self.dim
        with torch.no_grad():
            g, wx, bx, wk, bk, wv, bv, wo, bo = (p.detach().to(device=device, dtype=torch.float64) for p in ps)
            wx_h, bx_h = wx.view(H, D, C), bx.view(H, D)
            gk = g.view(H, S, D) @ wk                                     # (H, S, D): q_global . W_k
            w_a = torch.einsum("hsd,hdc->hsc", gk, wx_h).reshape(H * S, C)
            b_a = torch.einsum("hsd,hd->hs", gk, bx_h) + g.view(H, S, D) @ bk
            w_v = torch.einsum("ed,hdc->hec", wv, wx_h).reshape(H * D, C)
            b_v = torch.einsum("ed,hd->he", wv, bx_h) + bv
            params = {
                "scores_weight": w_a.to(dtype).contiguous(), "scores_bias": b_a.reshape(-1).float().contiguous(),
                "values_weight": w_v.to(dtype).contiguous(), "values_bias": b_v.reshape(-1).float().contiguous(),
                "out_linear_weight": wo.to(dtype).contiguous().reshape(-1),
                "out_linear_bias": bo.float().contiguous(),
            }
        self._cache = {"stamp": stamp, "params": params}
        return params

    def forward_block(self, x: torch.Tensor, residual: torch.Tensor, ln: nn.LayerNorm):
        """Layer + the caller block's ``+ residual`` and following LayerNorm (flare.py:98-99): (fx_new, LayerNorm(fx_new))
        with the add and the LayerNorm in one library kernel."""
        fp16 = x.dtype == torch.float16 or (torch.is_autocast_enabled("cuda")
                                            and torch.get_autocast_dtype("cuda") == torch.float16)
        if fp16:  # float32 inside, as the residual stream of the caller is
            with torch.autocast("cuda", enabled=False):
                return self.forward_block(x.float(), residual.float(), ln)
        if (not self._needs_grad(x) and x.is_cuda and self.use_mfma and x.ndim == 3
                and not (self.training and self.out_dropout.p > 0)):
            xb = x.to(torch.get_autocast_dtype("cuda")) if torch.is_autocast_enabled("cuda") else x
            if xb.dtype == torch.bfloat16:
                xb = xb.contiguous()
                dims = PF.LayerDims(xb.shape[0], xb.shape[1], xb.shape[2], self.heads, self.dim_head, self.n_global_queries)
                if xb.shape[2] == self.dim and PF.flare_forward_mfma_supported(xb.dtype, dims):
                    return PF.flare_forward_mfma(
                        xb, self.kernel_params(xb.dtype, xb.device), dims, residual=residual.to(xb.dtype).contiguous(),
                        ln_weight=ln.weight.detach().float().contiguous(), ln_bias=ln.bias.detach().float().contiguous(),
                        ln_eps=ln.eps)
        y = self.forward(x).contiguous()
        return PF.residual_layernorm(y, residual=residual.to(y.dtype).contiguous(),
                                     ln_weight=ln.weight.detach().float().contiguous(),
                                     ln_bias=ln.bias.detach().float().contiguous(), ln_eps=ln.eps)

    def _needs_grad(self, x: torch.Tensor) -> bool:
        return torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))

    def _composed(self, device: torch.device):
        """(scores weight (H*S, C), scores bias, values weight (H*D, C), values bias) as differentiable float32
        functions of the parameters."""
        H, D, S, C = self.heads, self.dim_head, self.n_global_queries, self.dim
        g = self.q_global.to(device=device, dtype=torch.float32).view(H, S, D)
        wx_h = self.in_project_x.weight.float().view(H, D, C)
        bx_h = self.in_project_x.bias.float().view(H, D)
        gk = g @ self.self_k.weight.float()
        w_a = torch.einsum("hsd,hdc->hsc", gk, wx_h).reshape(H * S, C)
        b_a = (torch.einsum("hsd,hd->hs", gk, bx_h) + g @ self.self_k.bias.float()).reshape(-1)
        w_v = torch.einsum("ed,hdc->hec", self.self_v.weight.float(), wx_h).reshape(H * D, C)
        b_v = (torch.einsum("ed,hd->he", self.self_v.weight.float(), bx_h) + self.self_v.bias.float()).reshape(-1)
        return w_a, b_a, w_v, b_v

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.ndim != 3:
            raise ValueError(f"Expected 3D input tensor (B, N, C), got {x.ndim}D tensor with shape {tuple(x.shape)}")
        if x.shape[-1] != self.dim:
            raise ValueError(f"Expected input feature dimension {self.dim}, got {x.shape[-1]}")
        if not x.is_cuda:
            raise RuntimeError("physicsnemo_amd FLARE runs on GPU tensors only (no CPU fallback)")
        needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        out_dtype = None
        if torch.is_autocast_enabled("cuda"):
            ac = torch.get_autocast_dtype("cuda")
            if ac == torch.float16:
                out_dtype, ac = torch.float16, torch.float32
            x = x.to(ac)
        elif x.dtype == torch.float16:
            out_dtype, x = torch.float16, x.float()
        if x.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"expected float32 or bfloat16 input, got {x.dtype}")
        x = x.contiguous()
        B, N, C = x.shape
        H, D, S = self.heads, self.dim_head, self.n_global_queries
        dims = PF.LayerDims(B, N, C, H, D, S)
        if needs_grad:
            with torch.autocast("cuda", enabled=False):
                w_a, b_a, w_v, b_v = self._composed(x.device)
            y = FlareFunction.apply(x, dims, w_a, b_a, w_v, b_v, self.out_linear.weight, self.out_linear.bias)
            return self.out_dropout(y if out_dtype is None else y.to(out_dtype))
        p = self.kernel_params(x.dtype, x.device)
        if self.use_mfma and PF.flare_forward_mfma_supported(x.dtype, dims):
            y = PF.flare_forward_mfma(x, p, dims)
            return self.out_dropout(y if out_dtype is None else y.to(out_dtype))
        scores = PF.rows_gemm(x, p["scores_weight"], p["scores_bias"], dims, C, H * S).view(B, N, H, S)
        values = PF.rows_gemm(x, p["values_weight"], p["values_bias"], dims, C, H * D)
        weights, _ = PF.flare_column_weights(scores, dims)
        tok, norm = PF.slice_reduce(weights, values, dims)
        # the aggregation kernel divides by (sum + 1e-2), the slice norm of PhysicsAttention; FLARE's softmax has no such
        # term (the sum is >= 1: the column maximum contributes exp(0))
        z = (tok * (norm / (norm - 1e-2)).unsqueeze(-1)).contiguous()
        PF.flare_softmax_rows_(scores, dims)
        y = PF.deslice_project(scores, z, p, dims)
        return self.out_dropout(y if out_dtype is None else y.to(out_dtype))


class GALE_FA(nn.Module):
    """GALE with FLARE self-attention (reference gale.py:513-762): the FLARE two-pass self-attention of every point,
    optionally blended with a per-point cross-attention to a context (B, H, S_c, D_c), then out_linear.  Same
    constructor arguments, parameter names and ``forward(x: tuple, context=None) -> list`` as the reference.

    Every stage is a row GEMM or a slice-weight kernel of the layer family: the cross-attention of a point is
    ``softmax_u(q_n . k_u) v_u`` with scale 1 -- scores from a row GEMM whose weight folds in_project_x, cross_q and the
    context's keys (one weight per batch element), an in-place row softmax, and the deslice kernel with the context's
    values as slice tokens.  With gradients required the same kernels run inside `FlareFunction` (self-attention) and
    `PointCrossFunction` (cross-attention); the weight compositions and the blend are PyTorch ops under autograd."""

    def __init__(self, dim: int, heads: int = 8, dim_head: int = 64, dropout: float = 0.0, n_global_queries: int = 64,
                 use_te: bool = False, context_dim: int = 0, concrete_dropout: bool = False,
                 state_mixing_mode: str = "weighted"):
        super().__init__()
        from .gale import _gale_cross_init

        if concrete_dropout:
            raise NotImplementedError("ConcreteDropout is a training-time regulariser; the HIP layer has none")
        self.use_te = use_te
        self.dim, self.heads, self.dim_head, self.n_global_queries = dim, heads, dim_head, n_global_queries
        self.scale = 1.0
        inner_dim = dim_head * heads
        self.q_global = nn.Parameter(torch.randn(1, heads, n_global_queries, dim_head))
        self.in_project_x = nn.Linear(dim, inner_dim)
        self.self_k = nn.Linear(dim_head, dim_head)
        self.self_v = nn.Linear(dim_head, dim_head)
        if context_dim > 0:
            _gale_cross_init(self, dim_head, context_dim, state_mixing_mode)
        self.context_dim = context_dim
        self.out_linear = nn.Linear(inner_dim, dim)
        self.out_dropout = nn.Dropout(dropout)
        self._cache: dict = {}

    kernel_params = FLARE.kernel_params
    _composed = FLARE._composed

    def _cross_composed(self, context: torch.Tensor):
        """(score weight (B, H*Sc, C), score bias (B, H*Sc), values (B, H, Sc, D)) as differentiable float32 functions of
        the parameters and the context."""
        H, D, C = self.heads, self.dim_head, self.dim
        ctx = context.float()
        B, Sc = ctx.shape[0], ctx.shape[2]
        k = torch.nn.functional.linear(ctx, self.cross_k.weight.float(), self.cross_k.bias.float())  # (B, H, Sc, D)
        v = torch.nn.functional.linear(ctx, self.cross_v.weight.float(), self.cross_v.bias.float())
        wx_h, bx_h = self.in_project_x.weight.float().view(H, D, C), self.in_project_x.bias.float().view(H, D)
        kq = k @ self.cross_q.weight.float()
        w_c = torch.einsum("bhud,hdc->bhuc", kq, wx_h).reshape(B, H * Sc, C)
        b_c = (torch.einsum("bhud,hd->bhu", kq, bx_h) + k @ self.cross_q.bias.float()).reshape(B, H * Sc)
        return w_c, b_c, v

    def _forward_one_with_grad(self, t: torch.Tensor, context: torch.Tensor | None, dims: PF.LayerDims) -> torch.Tensor:
        from .autograd import FlareFunction, PointCrossFunction, linear

        B, N, H, D = dims.B, dims.N, dims.H, dims.D
        with torch.autocast("cuda", enabled=False):
            w_a, b_a, w_v, b_v = self._composed(t.device)
            y = FlareFunction.apply(t, dims, w_a, b_a, w_v, b_v, None, None)
            if context is not None:
                w_c, b_c, v = self._cross_composed(context.to(t.device))
                cdims = PF.LayerDims(B, N, dims.C, H, D, context.shape[2])
                cross = PointCrossFunction.apply(t, cdims, w_c, b_c, v)
                if self.state_mixing_mode == "weighted":
                    m = torch.sigmoid(self.state_mixing.float())
                    y = (m * y.float() + (1 - m) * cross.float()).to(t.dtype)
                else:
                    lin = self.concat_project[0]
                    cat = torch.cat([y.view(B, N, H, D), cross.view(B, N, H, D)], dim=-1)
                    y = torch.nn.functional.gelu(linear(cat, lin.weight, lin.bias)).reshape(B, N, H * D)
            return linear(y, self.out_linear.weight, self.out_linear.bias)

    def _self_attention(self, x: torch.Tensor, p: dict, dims: PF.LayerDims) -> torch.Tensor:
        """FLARE two-pass attention -> (B, N, H*D), before out_linear."""
        B, N, C, H, D, S = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
        scores = PF.rows_gemm(x, p["scores_weight"], p["scores_bias"], dims, C, H * S).view(B, N, H, S)
        values = PF.rows_gemm(x, p["values_weight"], p["values_bias"], dims, C, H * D)
        weights, _ = PF.flare_column_weights(scores, dims)
        tok, norm = PF.slice_reduce(weights, values, dims)
        z = (tok * (norm / (norm - 1e-2)).unsqueeze(-1)).contiguous()
        return PF.deslice(PF.flare_softmax_rows_(scores, dims), z, dims)

    def _cross_attention(self, x: torch.Tensor, context: torch.Tensor, dims: PF.LayerDims) -> torch.Tensor:
        """Per-point cross-attention to the context (reference :735-744) -> (B, N, H*D)."""
        B, N, C, H, D = dims.B, dims.N, dims.C, dims.H, dims.D
        Sc = context.shape[2]
        with torch.no_grad():
            ctx = context.double()
            k = ctx @ self.cross_k.weight.double().t() + self.cross_k.bias.double()      # (B, H, Sc, D)
            v = (ctx @ self.cross_v.weight.double().t() + self.cross_v.bias.double()).float().contiguous()
            wx_h = self.in_project_x.weight.double().view(H, D, C)
            bx_h = self.in_project_x.bias.double().view(H, D)
            kq = k @ self.cross_q.weight.double()                                        # k_u . W_q: (B, H, Sc, D)
            w_c = torch.einsum("bhud,hdc->bhuc", kq, wx_h).reshape(B, H * Sc, C)
            b_c = (torch.einsum("bhud,hd->bhu", kq, bx_h) + k @ self.cross_q.bias.double()).reshape(B, H * Sc)
        cdims = PF.LayerDims(B, N, C, H, D, Sc)
        one = PF.LayerDims(1, N, C, H, D, Sc)
        scores = torch.empty(B, N, H, Sc, dtype=x.dtype, device=x.device)
        for b in range(B):  # the score weight holds the batch element's keys
            xb = x[b:b + 1] if x[b].data_ptr() % 16 == 0 else x[b:b + 1].clone()
            scores[b] = PF.rows_gemm(xb, w_c[b].to(x.dtype).contiguous(), b_c[b].float().contiguous(), one, C,
                                     H * Sc).view(N, H, Sc)
        return PF.deslice(PF.flare_softmax_rows_(scores, cdims), v, cdims)

    def _mix(self, self_x: torch.Tensor, cross_x: torch.Tensor, dims: PF.LayerDims) -> torch.Tensor:
        if self.state_mixing_mode == "weighted":
            m = torch.sigmoid(self.state_mixing.detach().float())
            return (m * self_x.float() + (1 - m) * cross_x.float()).to(self_x.dtype)
        B, N, H, D = dims.B, dims.N, dims.H, dims.D
        cat = torch.cat([self_x.view(B, N, H, D), cross_x.view(B, N, H, D)], dim=-1).reshape(B, N * H, 2 * D).contiguous()
        lin = self.concat_project[0]
        out = PF.rows_gemm(cat, lin.weight.detach().to(cat.dtype).contiguous(), lin.bias.detach().float().contiguous(),
                           PF.LayerDims(B, N * H, 2 * D, 1, 1, 1), 2 * D, D, gelu=True)
        return out.view(B, N, H * D)

    def forward(self, x: tuple, context: torch.Tensor | None = None) -> list:
        if isinstance(x, torch.Tensor):
            raise TypeError("GALE_FA takes a tuple of input tensors")
        if len(x) == 0:
            raise ValueError("Expected non-empty tuple of input tensors")
        outs = []
        for i, t in enumerate(x):
            if t.ndim != 3:
                raise ValueError(f"Expected 3D input tensor (B, N, C) at index {i}, "
                                 f"got {t.ndim}D tensor with shape {tuple(t.shape)}")
            if not t.is_cuda:
                raise RuntimeError("physicsnemo_amd GALE_FA runs on GPU tensors only (no CPU fallback)")
            needs_grad = torch.is_grad_enabled() and (t.requires_grad or (context is not None and context.requires_grad)
                                                      or any(p.requires_grad for p in self.parameters()))
            if torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16:
                t = t.to(torch.bfloat16)
            if t.dtype not in (torch.float32, torch.bfloat16):
                t = t.float()
            t = t.contiguous()
            B, N, C = t.shape
            dims = PF.LayerDims(B, N, C, self.heads, self.dim_head, self.n_global_queries)
            if context is not None and self.context_dim <= 0:
                raise ValueError("this GALE_FA was built without cross-attention (context_dim = 0)")
            if needs_grad:
                outs.append(self.out_dropout(self._forward_one_with_grad(t, context, dims)))
                continue
            p = self.kernel_params(t.dtype, t.device)
            if PF.flare_forward_mfma_supported(t.dtype, dims):
                y = PF.flare_forward_mfma(t, p, dims, project=False)  # bf16: the self-attention on the MFMA kernels
            else:
                y = self._self_attention(t, p, dims)
            if context is not None:
                y = self._mix(y, self._cross_attention(t, context.to(t.device), dims), dims)
            out = PF.rows_gemm(y, p["out_linear_weight"].view(C, -1), p["out_linear_bias"],
                               PF.LayerDims(B, N, y.shape[-1], 1, 1, 1), y.shape[-1], C)
            outs.append(self.out_dropout(out))
        return outs


# ---------------------------------------------------------------------------------------------------
# the FLARE model (physicsnemo/models/flare/flare.py): Transolver with FLARE blocks
# ---------------------------------------------------------------------------------------------------
class FLAREBlock(TransolverBlock):
    """LayerNorm -> FLARE attention -> +residual -> LayerNorm -> MLP -> +residual [-> LayerNorm -> Linear]
    (reference flare.py:37-104); the chaining, LayerNorm and block-MLP kernels are the Transolver block's."""

    def __init__(self, num_heads: int, hidden_dim: int, dropout: float, act: str = "gelu", mlp_ratio: int = 4,
                 last_layer: bool = False, out_dim: int = 1, n_global_queries: int = 32, use_te: bool = False):
        nn.Module.__init__(self)
        self.last_layer = last_layer
        self.ln_1 = nn.LayerNorm(hidden_dim)
        self.Attn = FLARE(hidden_dim, heads=num_heads, dim_head=hidden_dim // num_heads, dropout=dropout,
                          n_global_queries=n_global_queries, use_te=use_te)
        self.ln_mlp1 = nn.Sequential(nn.LayerNorm(hidden_dim),
                                     Mlp(hidden_dim, hidden_dim * mlp_ratio, hidden_dim, act))
        if last_layer:
            self.ln_mlp2 = nn.Sequential(nn.LayerNorm(hidden_dim), nn.Linear(hidden_dim, out_dim))
        self._mlp_cache = {}

class FLAREModel(Transolver):
    """Transolver with FLARE attention (reference flare.py:107-213, class ``FLARE`` there): same constructor
    (without ``plus``), inputs and outputs as `Transolver`.  As in the reference the Transolver is built first, then
    its blocks are replaced and the weight init runs again, so seeded construction consumes the generator alike."""

    _mdlus_class = ("FLARE", "physicsnemo.models.flare.flare")

    def __init__(self, functional_dim: int, out_dim: int, embedding_dim: int | None = None, n_layers: int = 4,
                 n_hidden: int = 256, dropout: float = 0.0, n_head: int = 8, act: str = "gelu", mlp_ratio: int = 4,
                 slice_num: int = 32, unified_pos: bool = False, ref: int = 8,
                 structured_shape: tuple | None = None, time_input: bool = False, use_te: bool = False):
        super().__init__(functional_dim=functional_dim, out_dim=out_dim, embedding_dim=embedding_dim,
                         n_layers=n_layers, n_hidden=n_hidden, dropout=dropout, n_head=n_head, act=act,
                         mlp_ratio=mlp_ratio, slice_num=slice_num, unified_pos=unified_pos, ref=ref,
                         structured_shape=structured_shape, use_te=use_te, time_input=time_input, plus=False)
        self._args.pop("plus", None)
        self.blocks = nn.ModuleList([
            FLAREBlock(num_heads=n_head, hidden_dim=n_hidden, dropout=dropout, act=act, mlp_ratio=mlp_ratio,
                       last_layer=(i == n_layers - 1), out_dim=out_dim, n_global_queries=slice_num, use_te=use_te)
            for i in range(n_layers)
        ])
        self.initialize_weights()

