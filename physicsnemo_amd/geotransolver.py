"""GeoTransolver on the PhysicsAttention / GALE HIP kernels.

Mirrors ``physicsnemo/models/geotransolver/geotransolver.py`` (GeoTransolver:390-766) and the context builder of
``context_projector.py`` (GlobalContextBuilder:766-1069): geometry and global embeddings are projected onto slice
tokens by context projectors and concatenated into the context every GALE block cross-attends to; with
``include_local_features=True`` ball-query neighbourhoods at several radii add further contexts and widen every
point's hidden state; each input stream has its own preprocess Mlp and LayerNorm + Linear head.  Same constructor
arguments, parameter names and forward signature as the reference, so its checkpoints load unchanged.  The
not-yet-implemented ``time`` input of the reference is refused as it is there.
"""
from __future__ import annotations

import math
from collections.abc import Sequence

import torch
import torch.nn as nn

from . import autograd as PA
from .context_projector import ContextProjector, MultiScaleFeatureExtractor, StructuredContextProjector
from .gale import GALEBlock
from .transolver import Mlp, Transolver


def _normalize_dim(x) -> tuple:
    if isinstance(x, int):
        return (x,)
    if isinstance(x, Sequence) and not isinstance(x, (str, bytes)):
        return tuple(int(v) for v in x)
    raise TypeError(f"Invalid dim specifier {x!r}")


class GlobalContextBuilder(nn.Module):
    """Context (B, H, S, D_c) from geometry and global embeddings and, optionally, the multi-scale ball-query features
    (reference context_projector.py:766-1069): one context projector each, concatenated along the feature axis."""

    def __init__(self, functional_dims: tuple, geometry_dim: int | None = None, global_dim: int | None = None,
                 radii=None, neighbors_in_radius=None, n_hidden_local: int = 32, n_hidden: int = 256, n_head: int = 8,
                 dropout: float = 0.0, slice_num: int = 32, use_te: bool = False, plus: bool = False,
                 include_local_features: bool = False, structured_shape: tuple | None = None,
                 concrete_dropout: bool = False):
        super().__init__()
        radii = [0.05, 0.25] if radii is None else radii
        neighbors_in_radius = [8, 32] if neighbors_in_radius is None else neighbors_in_radius
        dim_head = n_hidden // n_head
        self.structured_shape = structured_shape
        self._context_dim = 0
        kw = dict(use_te=use_te, plus=plus, concrete_dropout=concrete_dropout)
        if geometry_dim is not None and include_local_features and structured_shape is None:
            self.local_extractors = nn.ModuleList([
                MultiScaleFeatureExtractor(geometry_dim, radii, neighbors_in_radius, n_hidden_local, n_head, dim_head,
                                           dropout, slice_num, **kw) for _ in functional_dims])
            self._context_dim += dim_head * len(radii) * len(functional_dims)
        else:
            self.local_extractors = None
        if geometry_dim is not None:
            if structured_shape is not None:
                self.geometry_tokenizer = StructuredContextProjector(geometry_dim, structured_shape, n_head, dim_head,
                                                                     dropout, slice_num, **kw)
            else:
                self.geometry_tokenizer = ContextProjector(geometry_dim, n_head, dim_head, dropout, slice_num, **kw)
            self._context_dim += dim_head
        else:
            self.geometry_tokenizer = None
        if global_dim is not None:
            self.global_tokenizer = ContextProjector(global_dim, n_head, dim_head, dropout, slice_num, **kw)
            self._context_dim += dim_head
        else:
            self.global_tokenizer = None

    def get_context_dim(self) -> int:
        return self._context_dim

    def build_context(self, local_embeddings, local_positions, geometry=None, global_embedding=None):
        """Returns (context or None, per-stream local features or None, detached geometry context or None), as the
        reference does."""
        if len(local_embeddings) == 0:
            raise ValueError("Expected non-empty tuple of local embeddings")
        parts, geometry_context, local_features = [], None, None
        if local_positions is None and self.local_extractors is not None:
            raise ValueError("Local positions are required if local features are enabled.")
        if self.local_extractors is not None and geometry is not None:
            local_features = []
            for i in range(len(local_embeddings)):
                parts.extend(self.local_extractors[i].extract_context_features(local_positions[i], geometry))
                local_features.append(self.local_extractors[i].extract_local_features(local_positions[i], geometry))
        if self.geometry_tokenizer is not None and geometry is not None:
            geometry_context = self.geometry_tokenizer(geometry)
            parts.append(geometry_context)
        if self.global_tokenizer is not None and global_embedding is not None:
            parts.append(self.global_tokenizer(global_embedding))
        context = torch.cat(parts, dim=-1) if parts else None
        return context, local_features, (geometry_context.detach() if geometry_context is not None else None)


class GeoTransolver(nn.Module):
    """GALE blocks over one or several input streams with a shared geometry / global context (reference :390-766)."""

    _mdlus_class = ("GeoTransolver", "physicsnemo.models.geotransolver.geotransolver")
    save = Transolver.save
    load = Transolver.load
    from_checkpoint = classmethod(Transolver.from_checkpoint.__func__)

    def __init__(self, functional_dim, out_dim, geometry_dim: int | None = None, global_dim: int | None = None,
                 n_layers: int = 4, n_hidden: int = 256, dropout: float = 0.0, n_head: int = 8, act: str = "gelu",
                 mlp_ratio: int = 4, slice_num: int = 32, use_te: bool = False, time_input: bool = False,
                 plus: bool = False, include_local_features: bool = False, radii=None, neighbors_in_radius=None,
                 n_hidden_local: int = 32, structured_shape: tuple | None = None, attention_type: str = "GALE",
                 concrete_dropout: bool = False, state_mixing_mode: str = "weighted"):
        super().__init__()
        self._args = dict(functional_dim=functional_dim, out_dim=out_dim, geometry_dim=geometry_dim,
                          global_dim=global_dim, n_layers=n_layers, n_hidden=n_hidden, dropout=dropout, n_head=n_head,
                          act=act, mlp_ratio=mlp_ratio, slice_num=slice_num, use_te=use_te, time_input=time_input,
                          plus=plus, include_local_features=include_local_features, radii=radii,
                          neighbors_in_radius=neighbors_in_radius, n_hidden_local=n_hidden_local,
                          structured_shape=structured_shape, attention_type=attention_type,
                          concrete_dropout=concrete_dropout, state_mixing_mode=state_mixing_mode)
        if structured_shape is not None:
            if include_local_features:
                raise ValueError("include_local_features=True is not supported with structured_shape "
                                 "(ball-query path is mesh-only).")
            if len(structured_shape) not in (2, 3):
                raise ValueError(f"structured_shape must have length 2 or 3, got {structured_shape!r}")
            if not all(int(s) > 0 for s in structured_shape):
                raise ValueError(f"structured_shape must be positive ints, got {structured_shape!r}")
            structured_shape = tuple(int(s) for s in structured_shape)
        self.include_local_features = include_local_features
        self.use_te = use_te
        self.structured_shape = structured_shape
        if n_head <= 0:
            raise ValueError(f"GeoTransolver requires n_head > 0, got {n_head}")
        if n_hidden % n_head != 0:
            raise ValueError(f"GeoTransolver requires n_hidden % n_head == 0, got n_hidden={n_hidden}, n_head={n_head}")
        functional_dims, out_dims = _normalize_dim(functional_dim), _normalize_dim(out_dim)
        radii = [0.05, 0.25] if radii is None else radii
        neighbors_in_radius = [8, 32] if neighbors_in_radius is None else neighbors_in_radius
        self.radii = radii if include_local_features else []
        self.context_builder = GlobalContextBuilder(
            functional_dims=functional_dims, geometry_dim=geometry_dim, global_dim=global_dim, radii=radii,
            neighbors_in_radius=neighbors_in_radius, n_hidden_local=n_hidden_local, n_hidden=n_hidden, n_head=n_head,
            dropout=dropout, slice_num=slice_num, use_te=use_te, plus=plus,
            include_local_features=include_local_features, structured_shape=structured_shape,
            concrete_dropout=concrete_dropout)
        context_dim = self.context_builder.get_context_dim()
        if len(functional_dims) != len(out_dims):
            raise ValueError(f"functional_dim and out_dim must be the same length, but instead got "
                             f"{len(functional_dims)} and {len(out_dims)}")
        self.preprocess = nn.ModuleList([Mlp(f, n_hidden * 2, n_hidden, act) for f in functional_dims])
        self.n_hidden = n_hidden
        effective_hidden = n_hidden + n_hidden_local * len(self.radii) if include_local_features else n_hidden
        self.blocks = nn.ModuleList([
            GALEBlock(num_heads=n_head, hidden_dim=effective_hidden, dropout=dropout, act=act, mlp_ratio=mlp_ratio,
                      slice_num=slice_num, last_layer=(i == n_layers - 1), use_te=use_te, plus=plus,
                      context_dim=context_dim, spatial_shape=structured_shape, attention_type=attention_type,
                      concrete_dropout=concrete_dropout, state_mixing_mode=state_mixing_mode)
            for i in range(n_layers)
        ])
        self.ln_mlp_out = nn.ModuleList([nn.Sequential(nn.LayerNorm(effective_hidden), nn.Linear(effective_hidden, o))
                                         for o in out_dims])
        self.time_input = time_input
        if time_input:
            self.time_fc = nn.Sequential(nn.Linear(n_hidden, n_hidden), nn.SiLU(), nn.Linear(n_hidden, n_hidden))

    def _flatten(self, t: torch.Tensor, name: str) -> torch.Tensor:
        n = int(math.prod(self.structured_shape))
        if t.ndim == 3:
            if t.shape[1] != n:
                raise ValueError(f"{name} token count {t.shape[1]} != structured grid size {n}")
            return t
        if t.ndim == len(self.structured_shape) + 2:
            if tuple(t.shape[1:-1]) != self.structured_shape:
                raise ValueError(f"{name} spatial dims {tuple(t.shape[1:-1])} != structured_shape {self.structured_shape}")
            return t.reshape(t.shape[0], n, t.shape[-1])
        raise ValueError(f"{name} must be (B, N, C) or (B, *structured_shape, C), got shape {tuple(t.shape)}")

    def forward(self, local_embedding, local_positions=None, global_embedding: torch.Tensor | None = None,
                geometry: torch.Tensor | None = None, time: torch.Tensor | None = None, *,
                return_embedding_states: bool = False, return_point_features: bool = False):
        single_input = isinstance(local_embedding, torch.Tensor)
        if time is not None:
            raise NotImplementedError("Time input is not implemented yet. Error rather than silently ignoring it.")
        streams = (local_embedding,) if single_input else tuple(local_embedding)
        if local_positions is not None:
            local_positions = (local_positions,) if isinstance(local_positions, torch.Tensor) else tuple(local_positions)
        unflatten_output = False
        if self.structured_shape is not None:
            unflatten_output = any(t.ndim in (4, 5) for t in streams)
            streams = tuple(self._flatten(t, f"local_embedding[{i}]") for i, t in enumerate(streams))
            if geometry is not None:
                geometry = self._flatten(geometry, "geometry")
        if len(streams) == 0:
            raise ValueError("Expected non-empty local_embedding")
        if len(streams) != len(self.preprocess):
            raise ValueError(f"Expected {len(self.preprocess)} local_embedding stream(s) to match the model's configured "
                             f"functional_dim/out_dim, got {len(streams)}")
        if local_positions is not None and len(local_positions) != len(streams):
            raise ValueError(f"Expected local_positions to provide the same number of streams as local_embedding "
                             f"({len(streams)}), got {len(local_positions)}")
        for i, t in enumerate(streams):
            if t.ndim != 3:
                raise ValueError(f"Expected 3D local_embedding tensor (B, N, C) at index {i}, "
                                 f"got {t.ndim}D tensor with shape {tuple(t.shape)}")
        if geometry is not None and geometry.ndim != 3:
            raise ValueError(f"Expected 3D geometry tensor (B, N, C_geo), got {geometry.ndim}D tensor with shape "
                             f"{tuple(geometry.shape)}")
        if global_embedding is not None and global_embedding.ndim != 3:
            raise ValueError(f"Expected 3D global_embedding tensor (B, N_g, C_g), got {global_embedding.ndim}D tensor "
                             f"with shape {tuple(global_embedding.shape)}")
        embedding_states, local_bq, _ = self.context_builder.build_context(streams, local_positions, geometry,
                                                                           global_embedding)
        x = [self.preprocess[i](t) for i, t in enumerate(streams)]
        if self.include_local_features and local_bq is not None:
            x = [torch.cat([x[i], local_bq[i].to(x[i].dtype)], dim=-1) for i in range(len(x))]
        needs_grad = torch.is_grad_enabled() and (any(t.requires_grad for t in x)
                                                  or any(p.requires_grad for p in self.parameters()))
        chain = not needs_grad and all(t.is_cuda for t in x) and all(hasattr(b.Attn, "gale_params") for b in self.blocks)
        if chain:
            # inference: each block hands the next one LayerNorm_1 of its outputs (computed in its MLP kernel's tail)
            if torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16:
                x = [t.to(torch.bfloat16) for t in x]
            normed = None
            for k, block in enumerate(self.blocks):
                next_ln = self.blocks[k + 1].ln_1 if k + 1 < len(self.blocks) else None
                x, normed = block.forward_chain(tuple(x), normed, embedding_states, next_ln)
        else:
            for block in self.blocks:
                x = block(tuple(x), embedding_states)
        point_features = list(x)
        # per-stream head: LayerNorm on the library kernel (forward and backward), then the output Linear
        x = [self.ln_mlp_out[i][1](PA.layer_norm(t, self.ln_mlp_out[i][0])) for i, t in enumerate(x)]
        if self.structured_shape is not None and unflatten_output:
            x = [t.reshape(t.shape[0], *self.structured_shape, -1) for t in x]
        out = x[0] if single_input else tuple(x)
        feats = point_features[0] if single_input else tuple(point_features)
        if return_embedding_states and return_point_features:
            return out, embedding_states, feats
        if return_embedding_states:
            return out, embedding_states
        if return_point_features:
            return out, feats
        return out
