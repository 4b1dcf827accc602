"""Context projectors of GeoTransolver on the PhysicsAttention HIP kernels.

Mirrors ``physicsnemo/models/geotransolver/context_projector.py``: ContextProjector:190-378 (Linear projections),
StructuredContextProjector:380-486 (Conv2d / Conv3d projections), ``_SliceToContextMixin``:108-187,
GeometricFeatureProcessor:491-606 and MultiScaleFeatureExtractor:609-763 (ball-query local features; the ball query
is ``BQWarp`` of ``physicsnemo/nn/module/ball_query.py:32-140`` on the library's HIP kernel).

A context projector is the encoding half of a PhysicsAttention layer -- projections, slice softmax, aggregation --
and returns the slice tokens ``(B, H, S, D)`` that GALE layers cross-attend to; it never projects back to the points.
It therefore runs on stages (a) and (b) of the layer: the fused bf16 MFMA kernel where it serves the shape (its slice
self-attention and deslice operands are simply not used), the natural-layout kernels otherwise.  Same constructor
arguments and parameter names as the reference; ``concrete_dropout=True`` is not served.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as PF
from .autograd import SliceTokensFunction
from .physics_attention import _kernel_layout


class _SliceToContextMixin:
    """Shared slice components and forward (reference :108-187, :338-378, :466-486)."""

    def _init_slice_components(self, dim_head: int, slice_num: int, heads: int, plus: bool) -> None:
        self.in_project_slice = nn.Linear(dim_head, slice_num)
        self.temperature = nn.Parameter(torch.ones([1, 1, heads, 1]) * 0.5)
        if plus:
            self.proj_temperature = nn.Sequential(nn.Linear(dim_head, slice_num), nn.GELU(),
                                                  nn.Linear(slice_num, 1), nn.GELU())
        self.slice_num = slice_num
        self._kernel_param_cache: dict = {}

    def _conv_geometry(self):
        return 0, 0, 0, 0

    def layer_dims(self, x: torch.Tensor) -> PF.LayerDims:
        gh, gw, k, gd = self._conv_geometry()
        return PF.LayerDims(x.shape[0], x.shape[1], self.dim, self.heads, self.dim_head, self.slice_num, gh, gw, k, gd,
                            1 if k > 0 else 0)

    def kernel_params(self, dtype: torch.dtype, device: torch.device) -> dict:
        """Parameters as the C ABI wants them (projection weights in `dtype`, the rest float32).  The layer's
        qkv_project / out_linear, which a projector does not have, are zero tensors: the fused kernels' parameter pack
        reads them, nothing a projector returns depends on them."""
        named = [("in_project_x_weight", self.in_project_x.weight, True),
                 ("in_project_x_bias", self.in_project_x.bias, False)]
        if self.plus:
            named += [(f"proj_temperature_{i}_{kind}", getattr(self.proj_temperature[i], kind), False)
                      for i in (0, 2) for kind in ("weight", "bias")]
        else:
            named += [("in_project_fx_weight", self.in_project_fx.weight, True),
                      ("in_project_fx_bias", self.in_project_fx.bias, False)]
        named += [("in_project_slice_weight", self.in_project_slice.weight, False),
                  ("in_project_slice_bias", self.in_project_slice.bias, False),
                  ("temperature", self.temperature, False)]
        stamp = (dtype, device) + tuple((p.data_ptr(), p._version, p.dtype) for _, p, _ in named)
        if self._kernel_param_cache.get("stamp") == stamp:
            return self._kernel_param_cache["params"]
        with torch.no_grad():
            params = {name: _kernel_layout(p.detach()).to(device=device, dtype=dtype if big else torch.float32)
                      .contiguous().reshape(-1).clone() for name, p, big in named}
            HD, D = self.heads * self.dim_head, self.dim_head
            params["qkv_project_weight"] = torch.zeros(3 * D * D, dtype=torch.float32, device=device)
            params["out_linear_weight"] = torch.zeros(self.dim * HD, dtype=dtype, device=device)
            params["out_linear_bias"] = torch.zeros(self.dim, dtype=torch.float32, device=device)
        self._kernel_param_cache = {"stamp": stamp, "params": params}
        return params

    def _check_spatial(self, x: torch.Tensor) -> None:
        pass

    def _prepare_input(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_cuda:
            raise RuntimeError("physicsnemo_amd context projectors run on GPU tensors only (no CPU fallback)")
        if torch.is_autocast_enabled("cuda"):
            ac = torch.get_autocast_dtype("cuda")
            x = x.to(torch.float32 if ac == torch.float16 else ac)
        elif x.dtype == torch.float16:
            x = x.float()
        if x.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"expected float32 or bfloat16 input, got {x.dtype}")
        self._check_spatial(x)
        return x.contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """(B, N, C) -> slice tokens (B, H, S, D), float32."""
        if x.ndim != 3:
            raise ValueError(f"Expected 3D input tensor (B, N, C), got {x.ndim}D tensor with shape {tuple(x.shape)}")
        if x.shape[-1] != self.dim:
            raise ValueError(f"Expected input feature dimension {self.dim}, got {x.shape[-1]}")
        needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        x = self._prepare_input(x)
        dims = self.layer_dims(x)
        p = self.kernel_params(x.dtype, x.device)
        if needs_grad:
            if self.plus:
                raise NotImplementedError("training a plus=True context projector is not served")
            if not PF.backward_supported(x.dtype, dims):
                raise RuntimeError(f"the backward kernels do not serve this shape: {dims}")
            return SliceTokensFunction.apply(x, dims, p, self.in_project_x.weight, self.in_project_x.bias,
                                             self.in_project_fx.weight, self.in_project_fx.bias,
                                             self.in_project_slice.weight, self.in_project_slice.bias, self.temperature)
        if not self.plus and PF.query_path(x.dtype, dims) == 1:
            st = PF.MfmaStages(p, dims, x.device)
            st.pack_params()
            if st.fused_groups > 0:
                st.project_softmax_reduce(x)
            else:
                st.project_softmax(x)
                st.slice_reduce()
            st.combine_attention()
            return st.tok
        x_mid, fx_mid = PF.project_inputs(x, p, dims)
        if self.plus:
            u = torch.rand((dims.B, dims.N, dims.H, dims.S), dtype=x.dtype, device=x.device)
            w = PF.slice_softmax_plus(x_mid, u, p, dims)
        else:
            w = PF.slice_softmax(x_mid, p, dims)
        return PF.slice_reduce(w, fx_mid, dims)[0]


class ContextProjector(_SliceToContextMixin, nn.Module):
    """Irregular point sets: nn.Linear projections (reference :190-378)."""

    def __init__(self, dim: int, heads: int = 8, dim_head: int = 64, dropout: float = 0.0, slice_num: int = 64,
                 use_te: bool = False, plus: bool = False, concrete_dropout: bool = False):
        super().__init__()
        if concrete_dropout:
            raise NotImplementedError("ConcreteDropout is a training-time regulariser; the HIP projector has none")
        inner_dim = dim_head * heads
        self.dim, self.dim_head, self.heads, self.plus = dim, dim_head, heads, plus
        self.scale = dim_head ** -0.5
        self.use_te = use_te
        # registration order follows the reference so state_dict order and RNG draws agree
        self.in_project_x = nn.Linear(dim, inner_dim)
        if not plus:
            self.in_project_fx = nn.Linear(dim, inner_dim)
        self.softmax = nn.Softmax(dim=-1)
        self._init_slice_components(dim_head, slice_num, heads, plus)
        self.output_dropout = None


class StructuredContextProjector(_SliceToContextMixin, nn.Module):
    """2-D / 3-D grids: Conv2d / Conv3d projections (reference :380-486)."""

    def __init__(self, dim: int, spatial_shape: tuple, heads: int = 8, dim_head: int = 64, dropout: float = 0.0,
                 slice_num: int = 64, kernel: int = 3, use_te: bool = False, plus: bool = False,
                 concrete_dropout: bool = False):
        super().__init__()
        if len(spatial_shape) not in (2, 3):
            raise ValueError(f"StructuredContextProjector expects spatial_shape of length 2 or 3, got {spatial_shape!r}")
        if concrete_dropout:
            raise NotImplementedError("ConcreteDropout is a training-time regulariser; the HIP projector has none")
        inner_dim = dim_head * heads
        self.dim, self.dim_head, self.heads, self.plus = dim, dim_head, heads, plus
        self.use_te = use_te
        self.spatial_shape = tuple(int(s) for s in spatial_shape)
        self._nd = len(self.spatial_shape)
        self.kernel = kernel
        conv = nn.Conv2d if self._nd == 2 else nn.Conv3d
        self.in_project_x = conv(dim, inner_dim, kernel, 1, kernel // 2)
        if not plus:
            self.in_project_fx = conv(dim, inner_dim, kernel, 1, kernel // 2)
        self.softmax = nn.Softmax(dim=-1)
        self.dropout = nn.Dropout(dropout)
        self._init_slice_components(dim_head, slice_num, heads, plus)
        self.output_dropout = None

    def _conv_geometry(self):
        s = self.spatial_shape
        return s[0], s[1], self.kernel, (s[2] if self._nd == 3 else 0)

    def _check_spatial(self, x: torch.Tensor) -> None:
        n = 1
        for s in self.spatial_shape:
            n *= s
        if x.shape[1] != n:
            raise ValueError(f"Expected N={n} tokens for {self._nd}D grid, got N={x.shape[1]}")


class BQWarp(nn.Module):
    """Ball-query layer (reference physicsnemo/nn/module/ball_query.py:32-140; the name is the reference's, the search
    runs on the library's HIP kernel).  With ``reverse_mapping`` (the default) it returns, for every point of ``p_grid``,
    the up to ``neighbors_in_radius`` nearest points of ``x`` within ``radius``: (indices (B, Q, K), coordinates
    (B, Q, K, 3)), nearest first, index 0 / zero coordinates in unused slots -- the order of the reference's torch
    backend (radius_search/_torch_impl.py:96-160); its Warp backend keeps the first K it meets in hash-grid order, an
    order that is not specified.  Gradients flow to the coordinates that were gathered, as in the reference."""

    def __init__(self, radius: float = 0.25, neighbors_in_radius: int | None = 10):
        super().__init__()
        if neighbors_in_radius is None:
            raise NotImplementedError("the variable-length form (neighbors_in_radius=None) is not served")
        self.radius = radius
        self.neighbors_in_radius = neighbors_in_radius

    def forward(self, x: torch.Tensor, p_grid: torch.Tensor, reverse_mapping: bool = True):
        if p_grid.shape[-1] != x.shape[-1] or x.shape[-1] != 3:
            raise ValueError("The last dimension of p_grid and x must be 3")
        if p_grid.ndim in (4, 5):
            p_grid = p_grid.reshape(p_grid.shape[0], -1, 3)
        elif p_grid.ndim != 3:
            raise ValueError("p_grid must be 3D, 4D, 5D only")
        points, queries = (x, p_grid) if reverse_mapping else (p_grid, x)
        idx, out, counts = PF.ball_query(points, queries, self.radius, self.neighbors_in_radius)
        if torch.is_grad_enabled() and points.requires_grad:
            K = self.neighbors_in_radius
            used = torch.arange(K, device=idx.device) < counts[..., None]
            flat = idx.reshape(idx.shape[0], -1, 1).expand(-1, -1, 3)
            out = points.gather(1, flat).reshape(*idx.shape, 3) * used[..., None].to(points.dtype)
        else:
            out = out.to(points.dtype)
        return idx, out


class GeometricFeatureProcessor(nn.Module):
    """One radius of the local geometric features (reference :491-606): ball query, the neighbours' coordinates
    flattened, a three-layer GELU Mlp (``mlp.layers.0/2/4``), tanh."""

    def __init__(self, radius: float, neighbors_in_radius: int, feature_dim: int, hidden_dim: int):
        super().__init__()
        self.bq_warp = BQWarp(radius=radius, neighbors_in_radius=neighbors_in_radius)
        self.mlp = nn.Module()
        self.mlp.layers = nn.Sequential(nn.Linear(feature_dim * neighbors_in_radius, hidden_dim), nn.GELU(),
                                        nn.Linear(hidden_dim, hidden_dim // 2), nn.GELU(),
                                        nn.Linear(hidden_dim // 2, hidden_dim))

    def forward(self, query_points: torch.Tensor, key_features: torch.Tensor) -> torch.Tensor:
        if query_points.ndim != 3:
            raise ValueError(f"Expected 3D query_points tensor (B, N, 3), got {query_points.ndim}D tensor with shape "
                             f"{tuple(query_points.shape)}")
        if key_features.ndim != 3:
            raise ValueError(f"Expected 3D key_features tensor (B, N, C), got {key_features.ndim}D tensor with shape "
                             f"{tuple(key_features.shape)}")
        _, neighbors = self.bq_warp(query_points, key_features)
        return torch.tanh(self.mlp.layers(neighbors.flatten(2)))


class MultiScaleFeatureExtractor(nn.Module):
    """Local geometric features at several radii (reference :609-763): per radius one processor and one context
    projector that turns its features into slice tokens."""

    def __init__(self, geometry_dim: int, radii: list, neighbors_in_radius: list, hidden_dim: int, n_head: int,
                 dim_head: int, dropout: float = 0.0, slice_num: int = 64, use_te: bool = False, plus: bool = False,
                 concrete_dropout: bool = False):
        super().__init__()
        self.num_scales = len(radii)
        self.processors = nn.ModuleList([GeometricFeatureProcessor(radii[i], neighbors_in_radius[i], geometry_dim,
                                                                   hidden_dim) for i in range(self.num_scales)])
        self.tokenizers = nn.ModuleList([ContextProjector(hidden_dim, n_head, dim_head, dropout, slice_num, use_te, plus,
                                                          concrete_dropout=concrete_dropout)
                                         for _ in range(self.num_scales)])

    def extract_context_features(self, spatial_coords: torch.Tensor, geometry: torch.Tensor) -> list:
        """One (B, H, S, D) context per radius: the geometry points' neighbourhoods among the mesh points."""
        return [tok(proc(spatial_coords, geometry)) for proc, tok in zip(self.processors, self.tokenizers)]

    def extract_local_features(self, spatial_coords: torch.Tensor, geometry: torch.Tensor) -> torch.Tensor:
        """(B, N, hidden_dim * num_scales): the mesh points' neighbourhoods among the geometry points."""
        return torch.cat([proc(geometry, spatial_coords) for proc in self.processors], dim=-1)
