"""Host-side mirror of the caller of the hot path: TransolverBlock and Transolver
(physicsnemo/models/transolver/transolver.py:137-309 and :447-736, use_te=False).

Inference (no gradients required): the PhysicsAttention layer, its residual add and the LayerNorm that follows it
run in the HIP library, and so does
the block MLP with its residual add and the LayerNorm the next block starts with whenever the fused kernel serves
the shape (bf16, hidden 128 / 256, GELU); the preprocess MLP, the first LayerNorm and the output Linear run on the
library's row GEMM / LayerNorm kernels; what is left to PyTorch-ROCm tensor ops is the concatenation of the inputs
and every block MLP the fused kernel does not serve.
Module names, registration order and state_dict keys match the reference so its checkpoints load unchanged,
including the legacy ``linear_pre`` / ``linear_post`` MLP keys (:92-97).
Training (gradients required): the layer runs its differentiable path (stage-level kernels forward, the library's
backward kernels backward); LayerNorms, MLPs and residual adds are differentiable PyTorch-ROCm tensor ops.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn

from . import autograd as PA
from . import checkpoint as _ckpt
from . import functional as PF
from .physics_attention import (PhysicsAttentionIrregularMesh, PhysicsAttentionStructuredMesh2D,
                                PhysicsAttentionStructuredMesh3D)

__all__ = ["Mlp", "TransolverBlock", "Transolver"]

_LEGACY_MLP_KEYS = {
    "linear_pre.weight": "layers.0.weight",
    "linear_pre.bias": "layers.0.bias",
    "linear_post.weight": "layers.2.weight",
    "linear_post.bias": "layers.2.bias",
}

_ACTIVATIONS = {"gelu": nn.GELU, "relu": nn.ReLU, "silu": nn.SiLU, "tanh": nn.Tanh, "sigmoid": nn.Sigmoid}


class Mlp(nn.Module):
    """Linear -> activation -> Linear under ``layers.{0,2}`` (physicsnemo/nn/module/mlp_layers.py:139-173)."""

    def __init__(self, in_features: int, hidden_features: int, out_features: int, act_layer: str = "gelu"):
        super().__init__()
        try:
            act = _ACTIVATIONS[act_layer.lower()]()
        except KeyError:
            raise KeyError(f"Activation function {act_layer} not found. Available options are: {list(_ACTIVATIONS)}")
        self.layers = nn.Sequential(nn.Linear(in_features, hidden_features), act, nn.Linear(hidden_features, out_features))

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        for old, new in _LEGACY_MLP_KEYS.items():
            if prefix + old in state_dict and prefix + new not in state_dict:
                state_dict[prefix + new] = state_dict.pop(prefix + old)
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _kernel_params(self, dtype: torch.dtype, device: torch.device):
        """Both weights in the activation dtype and both biases in float32, cached until a parameter changes."""
        lin1, lin2 = self.layers[0], self.layers[2]
        named = (lin1.weight, lin1.bias, lin2.weight, lin2.bias)
        stamp = (dtype, device) + tuple((t.data_ptr(), t._version, t.dtype) for t in named)
        cache = self.__dict__.setdefault("_kernel_cache", {})
        if cache.get("stamp") != stamp:
            with torch.no_grad():
                cache["params"] = (lin1.weight.detach().to(device=device, dtype=dtype).contiguous().clone(),
                                   lin1.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone(),
                                   lin2.weight.detach().to(device=device, dtype=dtype).contiguous().clone(),
                                   lin2.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone())
            cache["stamp"] = stamp
        return cache["params"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lin1, lin2 = self.layers[0], self.layers[2]
        act = self.layers[1]
        needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        if (x.is_cuda and not needs_grad and x.numel() > 0 and isinstance(act, nn.GELU) and act.approximate == "none"
                and lin1.bias is not None and lin2.bias is not None):
            # inference with a few input features per row: both Linears and the GELU in one library launch with the
            # hidden layer kept on chip
            dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else x.dtype
            rows = x.numel() // x.shape[-1]
            if (dtype in (torch.float32, torch.bfloat16) and
                    PF.preprocess_supported(dtype, rows, lin1.in_features, lin1.out_features, lin2.out_features)):
                w1, b1, w2, b2 = self._kernel_params(dtype, x.device)
                return PF.preprocess_forward(x.to(dtype).contiguous(), w1, b1, w2, b2)
        return self.layers(x)


class PositionalEmbedding(nn.Module):
    """Timestep features [cos(t f_k) | sin(t f_k)], f_k = max_positions^(-k / (C/2)) (reference
    physicsnemo/nn/module/embedding_layers.py:67-152 with the arguments Transolver passes, transolver.py:532-538)."""

    def __init__(self, num_channels: int, max_positions: int = 10000):
        super().__init__()
        freqs = torch.arange(start=0, end=num_channels // 2, dtype=torch.float32) / (num_channels // 2)
        self.register_buffer("freqs", (1 / max_positions) ** freqs)
        self.register_load_state_dict_pre_hook(self._fill_missing_freqs)

    @staticmethod
    def _fill_missing_freqs(module, state_dict, prefix, *_args, **_kwargs):
        if prefix + "freqs" not in state_dict:  # older checkpoints kept freqs out of the state dict (:135-140)
            state_dict[prefix + "freqs"] = module.freqs.clone()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = torch.outer(x, self.freqs)
        return torch.cat([x.cos(), x.sin()], dim=1)


class TransolverBlock(nn.Module):
    """LayerNorm -> PhysicsAttention -> +residual -> LayerNorm -> MLP -> +residual [-> LayerNorm -> Linear]."""

    fp8_weights = False  # class default for subclasses with constructors of their own; see use_fp8_weights()

    def __init__(self, num_heads: int, hidden_dim: int, dropout: float, act: str = "gelu", mlp_ratio: int = 4,
                 last_layer: bool = False, out_dim: int = 1, slice_num: int = 32,
                 spatial_shape: tuple[int, ...] | None = None, use_te: bool = True, plus: bool = False):
        super().__init__()
        self.last_layer = last_layer
        self.ln_1 = nn.LayerNorm(hidden_dim)
        common = dict(heads=num_heads, dim_head=hidden_dim // num_heads, dropout=dropout, slice_num=slice_num,
                      use_te=use_te, plus=plus)
        if spatial_shape is None:
            self.Attn = PhysicsAttentionIrregularMesh(hidden_dim, **common)
        elif len(spatial_shape) == 2:
            self.Attn = PhysicsAttentionStructuredMesh2D(hidden_dim, spatial_shape=spatial_shape, **common)
        elif len(spatial_shape) == 3:
            self.Attn = PhysicsAttentionStructuredMesh3D(hidden_dim, spatial_shape=spatial_shape, **common)
        else:
            raise ValueError(
                f"Unexpected length of spatial shape encountered in Transolver_block: {len(spatial_shape)}. Expected 2 or 3.")
        self.ln_mlp1 = nn.Sequential(nn.LayerNorm(hidden_dim), Mlp(hidden_dim, hidden_dim * mlp_ratio, hidden_dim, act))
        if last_layer:
            self.ln_mlp2 = nn.Sequential(nn.LayerNorm(hidden_dim), nn.Linear(hidden_dim, out_dim))
        self._mlp_cache: dict = {}
        self.fp8_weights = False  # see use_fp8_weights()

    def use_fp8_weights(self, enabled: bool = True):
        """Inference with the block's large weights held as fp8-e4m3 with one scale per output channel
        (scale = max|row| / 448): the attention layer's three projections (`PhysicsAttentionBase.use_fp8_weights`)
        and the two Linears of the MLP.  The kernels expand them to bf16 operands; activations stay bf16.  No
        counterpart in the reference."""
        self.Attn.use_fp8_weights(enabled)
        self.fp8_weights = bool(enabled)
        self._mlp_cache = {}
        return self

    # ---------------------------------------------------------------- fused MLP (pa_mlp_forward)
    def _mlp_kernel_params(self, device, dtype=torch.bfloat16):
        """Weights (in the activation dtype: bf16, or float32) / fp32 biases of ln_mlp1's Mlp for the fused kernel;
        cached until a parameter changes.  With fp8 weights enabled the bf16 values are the dequantised e4m3 weights."""
        lin1, lin2 = self.ln_mlp1[1].layers[0], self.ln_mlp1[1].layers[2]
        named = (lin1.weight, lin1.bias, lin2.weight, lin2.bias)
        stamp = (device, dtype, self.fp8_weights) + tuple((t.data_ptr(), t._version, t.dtype) for t in named)
        if self._mlp_cache.get("stamp") != stamp:
            def big(w):
                w = w.detach().to(device=device, dtype=torch.float32)
                if self.fp8_weights:
                    w = PF.dequantize_e4m3_per_channel(*PF.quantize_e4m3_per_channel(w))
                return w.to(dtype).contiguous().clone()

            with torch.no_grad():
                params = (big(lin1.weight), lin1.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone(),
                          big(lin2.weight), lin2.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone())
            self._mlp_cache = {"stamp": stamp, "params": params}
        return self._mlp_cache["params"]

    def _mlp_kernel_packed(self, device, dtype=torch.bfloat16):
        """(packed weights, b1, b2) for pa_mlp_forward_packed: the weights repacked once per parameter set."""
        w1, b1, w2, b2 = self._mlp_kernel_params(device, dtype)
        if "packed" not in self._mlp_cache:
            if self.fp8_weights and dtype == torch.bfloat16:
                # the e4m3 bytes and scales go to the repacking kernel as they are: expanded once per parameter set
                lin1, lin2 = self.ln_mlp1[1].layers[0], self.ln_mlp1[1].layers[2]
                with torch.no_grad():
                    q1, s1 = PF.quantize_e4m3_per_channel(lin1.weight.detach().to(device))
                    q2, s2 = PF.quantize_e4m3_per_channel(lin2.weight.detach().to(device))
                self._mlp_cache["packed"] = PF.mlp_pack_e4m3(q1, s1, q2, s2)
            else:
                self._mlp_cache["packed"] = PF.mlp_pack(w1, w2)
        return self._mlp_cache["packed"], b1, b2

    def _mlp_kernel_serves(self, normed: torch.Tensor) -> bool:
        mlp = self.ln_mlp1[1]
        if not (normed.is_cuda and normed.dtype in (torch.bfloat16, torch.float32) and isinstance(mlp.layers[1], nn.GELU)
                and mlp.layers[1].approximate == "none"):
            return False
        if normed.dtype == torch.float32 and self.fp8_weights:
            return False
        hidden = mlp.layers[0].out_features
        return PF.mlp_supported(normed.dtype, normed.numel() // normed.shape[-1], normed.shape[-1], hidden)

    def _mlp_normalises_its_input(self, x_in: torch.Tensor) -> bool:
        """True where the block runs as layer call (+ residual) -> MLP kernel with ln_mlp1[0] applied on the way in:
        bf16 rows of 256 / 512 channels on the plain attention layer's fused tail."""
        attn = self.Attn
        if not (x_in.is_cuda and hasattr(attn, "layer_dims") and not getattr(attn, "plus", False)):
            return False
        if attn.training and attn.out_dropout.p > 0:
            return False
        dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else x_in.dtype
        if dtype != torch.bfloat16:
            return False
        mlp = self.ln_mlp1[1]
        if not (isinstance(mlp.layers[1], nn.GELU) and mlp.layers[1].approximate == "none"):
            return False
        rows, C = x_in.numel() // x_in.shape[-1], x_in.shape[-1]
        if C != 256:
            # at 512 channels the MLP kernel runs one wave per SIMD and nothing hides the normalisation of its rows:
            # measured on the 12-block model, it costs that kernel more than the layer's tail saves
            return False
        return PF.mlp_input_ln_supported(torch.bfloat16, rows, C, mlp.layers[0].out_features)

    def _needs_grad(self, fx: torch.Tensor) -> bool:
        return torch.is_grad_enabled() and (fx.requires_grad or any(p.requires_grad for p in self.parameters()))

    def _mlp_with_grad(self, normed: torch.Tensor) -> torch.Tensor:
        """ln_mlp1[1] in training; under bf16 autocast its Linears use `autograd.linear` (weight gradients on the
        library's row-axis kernel), otherwise the module as it is."""
        mlp = self.ln_mlp1[1]
        if normed.is_cuda and torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16:
            lin1, act, lin2 = mlp.layers[0], mlp.layers[1], mlp.layers[2]
            with torch.autocast("cuda", enabled=False):
                h = PA.linear(normed.to(torch.bfloat16), lin1.weight, lin1.bias)
                return PA.linear(act(h), lin2.weight, lin2.bias)
        return mlp(normed)

    def forward_chain(self, fx: torch.Tensor, normed_in: torch.Tensor | None, next_ln: nn.LayerNorm | None):
        """One block inside a chain of blocks: takes LayerNorm_1(fx) if the previous stage already produced it and
        returns (fx_out, next_ln(fx_out) or None).  Same arithmetic as `forward` (reference :300-303)."""
        if self._needs_grad(fx):
            # training: the layer's autograd path, LayerNorms / MLP as differentiable tensor ops (reference :300-303)
            x_in = normed_in if normed_in is not None else PA.layer_norm(fx, self.ln_1)
            fx1 = self.Attn(x_in) + fx
            return self._mlp_with_grad(PA.layer_norm(fx1, self.ln_mlp1[0])) + fx1, None
        x_in = normed_in if normed_in is not None else self.ln_1(fx)
        whole = self._whole_block(x_in, fx, next_ln)
        if whole is not None:
            return whole
        ln2 = self.ln_mlp1[0]
        if self._mlp_normalises_its_input(x_in):
            # fx1 = Attn(ln_1(fx)) + fx from the layer call; the MLP kernel applies ln_mlp1[0] to its rows itself, so
            # no normalised copy of fx1 is written or read (reference :300, :303)
            fx1 = self.Attn.forward_block(x_in, fx, None)
            packed, b1, b2 = self._mlp_kernel_packed(fx1.device, fx1.dtype)
            in_ln = (ln2.weight.detach().float().contiguous(), ln2.bias.detach().float().contiguous(), ln2.eps)
            if next_ln is None:
                return PF.mlp_forward_packed(fx1, packed, b1, b2, residual=fx1, in_ln=in_ln), None
            return PF.mlp_forward_packed(fx1, packed, b1, b2, residual=fx1, in_ln=in_ln,
                                         ln_weight=next_ln.weight.detach().float().contiguous(),
                                         ln_bias=next_ln.bias.detach().float().contiguous(), ln_eps=next_ln.eps)
        # fx1 = Attn(ln_1(fx)) + fx and LayerNorm(fx1) come out of one fused library call (reference :300, :303)
        fx1, normed = self.Attn.forward_block(x_in, fx, ln2)
        return self._mlp_residual(fx1, normed, next_ln)

    def _whole_block(self, x_in: torch.Tensor, fx: torch.Tensor, next_ln: nn.LayerNorm | None,
                     head: nn.Linear | None = None):
        """The block behind ln_1 in one library call (pa_block_forward) where the shape is served (float32, hidden 128,
        8 heads of 16, 32 slices), else None.  With `head` (the last block's ln_mlp2[1], up to 4 outputs) the second
        element of the result is the head's output instead of the LayerNorm."""
        attn, mlp = self.Attn, self.ln_mlp1[1]
        if not (x_in.is_cuda and x_in.dtype == torch.float32 and fx.dtype == torch.float32 and not self.fp8_weights
                and not getattr(attn, "plus", False) and isinstance(mlp.layers[1], nn.GELU)
                and mlp.layers[1].approximate == "none" and hasattr(attn, "layer_dims")):
            return None
        if (attn.training and attn.out_dropout.p > 0) or torch.is_autocast_enabled("cuda"):
            return None  # autocast runs the layer in its own dtype: the separate calls handle that
        x = attn._prepare_input(x_in)
        attn._validate(x_in)
        dims = attn.layer_dims(x)
        if not PF.block_supported(x.dtype, dims, mlp.layers[0].out_features):
            return None
        w1, b1, w2, b2 = self._mlp_kernel_params(x.device, torch.float32)
        ln2 = self.ln_mlp1[0]
        f32 = lambda t: t.detach().float().contiguous()
        nxt = {} if next_ln is None else dict(next_ln_weight=f32(next_ln.weight), next_ln_bias=f32(next_ln.bias),
                                              next_ln_eps=next_ln.eps)
        if head is not None:
            if next_ln is None or head.out_features > 4:
                return None
            nxt.update(head_weight=f32(head.weight), head_bias=None if head.bias is None else f32(head.bias))
        out = PF.block_forward(x, fx.contiguous(), attn.kernel_params(x.dtype, x.device), dims, f32(ln2.weight),
                               f32(ln2.bias), ln2.eps, w1, b1, w2, b2, **nxt)
        return (out, None) if next_ln is None else out

    def _mlp_residual(self, fx1: torch.Tensor, normed: torch.Tensor, next_ln: nn.LayerNorm | None):
        """fx1 + Mlp(normed) and, with `next_ln`, its LayerNorm (reference :303, and :300 of the next block): the fused
        block-MLP kernel where it serves the shape, else the tensor-op MLP followed by one add (+ LayerNorm) kernel."""
        if self._mlp_kernel_serves(normed):
            packed, b1, b2 = self._mlp_kernel_packed(normed.device, normed.dtype)
            if next_ln is None:
                return PF.mlp_forward_packed(normed, packed, b1, b2, residual=fx1), None
            return PF.mlp_forward_packed(normed, packed, b1, b2, residual=fx1,
                                         ln_weight=next_ln.weight.detach().float().contiguous(),
                                         ln_bias=next_ln.bias.detach().float().contiguous(), ln_eps=next_ln.eps)
        # MLP shapes the fused kernel does not serve: tensor-op MLP, then residual add (+ the next LayerNorm) in one pass
        if self.fp8_weights and normed.is_cuda and normed.dtype == torch.bfloat16:
            w1, b1, w2, b2 = self._mlp_kernel_params(normed.device)
            F = torch.nn.functional
            h = F.linear(self.ln_mlp1[1].layers[1](F.linear(normed, w1, b1.to(normed.dtype))), w2, b2.to(normed.dtype))
        else:
            h = self.ln_mlp1[1](normed)
        if h.is_cuda and h.dtype == fx1.dtype and h.dtype in (torch.float32, torch.bfloat16):
            h = h.contiguous()
            if next_ln is None:
                return PF.residual_layernorm(h, residual=fx1.contiguous()), None
            return PF.residual_layernorm(h, residual=fx1.contiguous(),
                                         ln_weight=next_ln.weight.detach().float().contiguous(),
                                         ln_bias=next_ln.bias.detach().float().contiguous(), ln_eps=next_ln.eps)
        return h + fx1, None

    def forward(self, fx: torch.Tensor) -> torch.Tensor:
        if self.last_layer:
            fx2, normed = self.forward_chain(fx, None, self.ln_mlp2[0])
            return self.ln_mlp2[1](normed) if normed is not None else self.ln_mlp2(fx2)
        return self.forward_chain(fx, None, None)[0]


class Transolver(nn.Module):
    """Transolver model (reference :447-736) built on the HIP PhysicsAttention layer."""

    def __init__(self, functional_dim: int, out_dim: int, embedding_dim: int | None = None, n_layers: int = 4,
                 n_hidden: int = 256, dropout: float = 0.0, n_head: int = 8, act: str = "gelu", mlp_ratio: int = 4,
                 slice_num: int = 32, unified_pos: bool = False, ref: int = 8,
                 structured_shape: None | tuple[int, ...] = None, use_te: bool = True, time_input: bool = False,
                 plus: bool = False) -> None:
        super().__init__()
        # constructor arguments as the reference records them for its checkpoints (core/module.py:196-223)
        self._args = dict(functional_dim=functional_dim, out_dim=out_dim, embedding_dim=embedding_dim, n_layers=n_layers,
                          n_hidden=n_hidden, dropout=dropout, n_head=n_head, act=act, mlp_ratio=mlp_ratio,
                          slice_num=slice_num, unified_pos=unified_pos, ref=ref,
                          structured_shape=list(structured_shape) if structured_shape is not None else None,
                          use_te=use_te, time_input=time_input, plus=plus)
        self.use_te = use_te
        if not n_hidden % n_head == 0:
            raise ValueError(
                f"Transolver requires n_hidden % n_head == 0, but got n_hidden={n_hidden}, n_head={n_head} "
                f"(remainder={n_hidden % n_head})")
        if structured_shape is not None:
            if len(structured_shape) not in [2, 3]:
                raise ValueError(
                    f"Transolver only supports 2D or 3D structured data, got shape with {len(structured_shape)} dimensions")
            if not all([s > 0 and s == int(s) for s in structured_shape]):
                raise ValueError(f"Transolver requires positive integer shapes, got {structured_shape}")
        elif unified_pos:
            raise ValueError("Transolver requires structured_shape when using unified_pos=True")
        self.structured_shape = structured_shape
        self.unified_pos = unified_pos
        if unified_pos:
            self.register_buffer("embedding", self.get_grid(ref))
            self.embedding_dim = ref * ref
        else:
            if embedding_dim is None:
                raise ValueError("Transolver requires embedding_dim when unified_pos=False")
            self.embedding_dim = embedding_dim
        self.preprocess = Mlp(functional_dim + self.embedding_dim, n_hidden * 2, n_hidden, act)
        self.time_input = time_input
        self.n_hidden = n_hidden
        if time_input:  # timestep embedding and its projection (reference :531-543)
            self.time_embed = PositionalEmbedding(n_hidden)
            self.time_fc = nn.Sequential(nn.Linear(n_hidden, n_hidden), nn.SiLU(), nn.Linear(n_hidden, n_hidden))
        self.blocks = nn.ModuleList([
            TransolverBlock(num_heads=n_head, hidden_dim=n_hidden, dropout=dropout, act=act, mlp_ratio=mlp_ratio,
                            out_dim=out_dim, slice_num=slice_num, spatial_shape=structured_shape,
                            last_layer=(i == n_layers - 1), use_te=use_te, plus=plus)
            for i in range(n_layers)
        ])
        self.initialize_weights()

    # ---------------------------------------------------------------- .mdlus checkpoints (core/module.py:446-1070)
    _mdlus_class = ("Transolver", "physicsnemo.models.transolver.transolver")  # class name and module in args.json

    def save(self, file_name: str | None = None) -> None:
        """Writes a ``.mdlus`` checkpoint the reference's ``Module.from_checkpoint`` / ``load`` accept."""
        name, module = self._mdlus_class
        _ckpt.write_mdlus(file_name or f"{name}.mdlus", name, module, self._args, self.state_dict())

    def load(self, file_name: str, map_location=None, strict: bool = True) -> None:
        """Loads the weights of a ``.mdlus`` checkpoint (zip or legacy tar) into this model."""
        device = map_location if map_location is not None else next(self.parameters()).device
        _, _, state = _ckpt.read_mdlus(file_name, map_location=device)
        self.load_state_dict(state, strict=strict)

    @classmethod
    def from_checkpoint(cls, file_name: str, override_args: dict | None = None, strict: bool = True) -> "Transolver":
        """Builds the model from the constructor arguments stored in a ``.mdlus`` checkpoint and loads its weights.
        ``use_te`` is the one argument the reference lets a caller override (transolver.py ``_overridable_args``)."""
        args, _, state = _ckpt.read_mdlus(file_name)
        if args.get("__name__") != cls._mdlus_class[0]:
            raise IOError(f"checkpoint holds a {args.get('__name__')!r}, not a {cls._mdlus_class[0]}")
        ctor = dict(args["__args__"])
        for key, value in (override_args or {}).items():
            if key != "use_te":
                raise ValueError(f"Argument '{key}' cannot be overridden for Transolver.")
            ctor[key] = value
        if ctor.get("structured_shape") is not None:
            ctor["structured_shape"] = tuple(ctor["structured_shape"])
        model = cls(**ctor)
        model.load_state_dict(state, strict=strict)
        return model

    # ---------------------------------------------------------------- glue layers on the library kernels
    def _glue_on_library(self, fx: torch.Tensor) -> bool:
        """Inference on a GPU with a GELU preprocess Mlp: the preprocess Mlp, the first LayerNorm and the output Linear
        run on the library's row kernels; otherwise (training, other activations) they are PyTorch-ROCm tensor ops."""
        if not fx.is_cuda or (torch.is_grad_enabled() and (fx.requires_grad or any(p.requires_grad
                                                                                   for p in self.parameters()))):
            return False
        act = self.preprocess.layers[1]
        if not (isinstance(act, nn.GELU) and act.approximate == "none"):
            return False
        dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else fx.dtype
        return dtype in (torch.float32, torch.bfloat16)

    def _library_linear(self, x: torch.Tensor, lin: nn.Linear, gelu: bool = False) -> torch.Tensor:
        cache = self.__dict__.setdefault("_linear_cache", {})
        stamp = (x.dtype, x.device, lin.weight.data_ptr(), lin.weight._version, lin.bias.data_ptr(), lin.bias._version)
        hit = cache.get(id(lin))
        if hit is None or hit[0] != stamp:
            with torch.no_grad():
                hit = (stamp, lin.weight.detach().to(device=x.device, dtype=x.dtype).contiguous().clone(),
                       lin.bias.detach().to(device=x.device, dtype=torch.float32).contiguous().clone())
            cache[id(lin)] = hit
        return PF.linear(x, hit[1], hit[2], gelu=gelu)

    def _preprocess_params(self, dtype, device):
        """The preprocess Mlp's weights in the activation dtype and its biases in float32, cached until one changes."""
        lin1, lin2 = self.preprocess.layers[0], self.preprocess.layers[2]
        named = (lin1.weight, lin1.bias, lin2.weight, lin2.bias)
        stamp = (dtype, device) + tuple((t.data_ptr(), t._version, t.dtype) for t in named)
        cache = self.__dict__.setdefault("_preprocess_cache", {})
        if cache.get("stamp") != stamp:
            with torch.no_grad():
                cache["params"] = (lin1.weight.detach().to(device=device, dtype=dtype).contiguous().clone(),
                                   lin1.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone(),
                                   lin2.weight.detach().to(device=device, dtype=dtype).contiguous().clone(),
                                   lin2.bias.detach().to(device=device, dtype=torch.float32).contiguous().clone())
            cache["stamp"] = stamp
        return cache["params"]

    def use_fp8_weights(self, enabled: bool = True):
        """Every block's large weights as fp8-e4m3 with per-output-channel scales (`TransolverBlock.use_fp8_weights`);
        the preprocess Mlp, the LayerNorms, the slice / qkv projections and the output head stay in higher precision."""
        for block in self.blocks:
            block.use_fp8_weights(enabled)
        return self

    def initialize_weights(self) -> None:
        self.apply(self._init_weights)

    def _init_weights(self, m: nn.Module) -> None:
        # every nn.Linear (the slice projection included) is redrawn; Conv2d keeps its default init (:579-593)
        if isinstance(m, nn.Linear):
            nn.init.trunc_normal_(m.weight, std=0.02)
            if m.bias is not None:
                nn.init.constant_(m.bias, 0)
        if isinstance(m, (nn.LayerNorm, nn.BatchNorm1d)):
            nn.init.constant_(m.bias, 0)
            nn.init.constant_(m.weight, 1.0)

    def get_grid(self, ref: int, batchsize: int = 1) -> torch.Tensor:
        """Distances from every grid point to a ref x ref lattice on the unit square, (B, H*W, ref*ref) (:595-645)."""
        if self.structured_shape is None:
            raise ValueError("Cannot generate positional encoding grid: structured_shape is None. "
                             "This method requires structured_shape to be set.")
        size_x, size_y = self.structured_shape
        px = torch.tensor(np.linspace(0, 1, size_x), dtype=torch.float)
        py = torch.tensor(np.linspace(0, 1, size_y), dtype=torch.float)
        pts = torch.stack(torch.meshgrid(px, py, indexing="ij"), dim=-1).reshape(-1, 1, 2)
        lr = torch.tensor(np.linspace(0, 1, ref), dtype=torch.float)
        lattice = torch.stack(torch.meshgrid(lr, lr, indexing="ij"), dim=-1).reshape(1, -1, 2)
        pos = torch.sqrt(((pts - lattice) ** 2).sum(-1))
        return pos.unsqueeze(0).repeat(batchsize, 1, 1).contiguous()

    def forward(self, fx: torch.Tensor, embedding: torch.Tensor | None = None, time: torch.Tensor | None = None):
        if fx.ndim < 2:
            raise ValueError(
                f"Expected input tensor with at least 2 dimensions, got {fx.ndim}D tensor with shape {tuple(fx.shape)}")
        if not self.unified_pos and embedding is None:
            raise ValueError("Embedding is required when unified_pos=False")
        if time is not None and not self.time_input:
            raise ValueError("time was given but the model was built with time_input=False")
        unflatten_output = False
        if self.unified_pos:
            embedding = self.embedding.repeat(fx.shape[0], 1, 1)
        if self.structured_shape is not None:
            if fx.ndim != 3:
                unflatten_output = True
                fx = fx.reshape(fx.shape[0], -1, fx.shape[-1])
            if embedding is not None and embedding.ndim != 3:
                embedding = embedding.reshape(embedding.shape[0], -1, embedding.shape[-1])
        fx = torch.cat((embedding.to(fx.dtype), fx), -1)  # embedding first, then the functional input (:716)
        if fx.numel() == 0 and self.structured_shape is None:
            # no points or an empty batch: the reference's tensor ops return the empty (B, N, out_dim) result
            return fx.new_zeros(fx.shape[:-1] + (self.blocks[-1].ln_mlp2[1].out_features,))
        on_library = self._glue_on_library(fx)
        normed = None
        first_ln_done = False
        if on_library:
            # preprocess Mlp (Linear -> GELU -> Linear, :519-525) and the first block's LayerNorm on the library kernels
            if torch.is_autocast_enabled("cuda"):
                fx = fx.to(torch.get_autocast_dtype("cuda"))
            lin1, lin2 = self.preprocess.layers[0], self.preprocess.layers[2]
            rows = fx.numel() // fx.shape[-1]
            if (time is None and len(self.preprocess.layers) == 3 and
                    PF.preprocess_supported(fx.dtype, rows, lin1.in_features, lin1.out_features, lin2.out_features)):
                # both Linears, the GELU and the first block's LayerNorm in one library call with the hidden layer kept
                # on chip (float32 at hidden 128; bfloat16 at hidden 256 / 512)
                ln = self.blocks[0].ln_1
                w1, b1, w2, b2 = self._preprocess_params(fx.dtype, fx.device)
                fx, normed = PF.preprocess_forward(
                    fx.contiguous(), w1, b1, w2, b2, ln_weight=ln.weight.detach().float().contiguous(),
                    ln_bias=ln.bias.detach().float().contiguous(), ln_eps=ln.eps)
                first_ln_done = True
            elif lin2.in_features <= 512:  # the weights-stationary row kernel holds up to 512 input features
                fx = self._library_linear(self._library_linear(fx.contiguous(), lin1, gelu=True), lin2)
            else:
                fx = self.preprocess(fx).contiguous()
        else:
            fx = self.preprocess(fx)
        if time is not None:
            # every token of a batch gets the same vector, so time_fc runs on (B, C) and is broadcast (reference
            # :721-725 repeats first; the arithmetic per token is the same)
            time_emb = self.time_fc(self.time_embed(time.to(torch.float32)))
            fx = (fx + time_emb.to(fx.dtype).unsqueeze(1)).contiguous()
        if on_library and not first_ln_done:
            ln = self.blocks[0].ln_1
            fx, normed = PF.residual_layernorm(fx, ln_weight=ln.weight.detach().float().contiguous(),
                                               ln_bias=ln.bias.detach().float().contiguous(), ln_eps=ln.eps)
        # each block hands the next one its residual stream and, when the fused MLP kernel ran, LayerNorm_1 of it
        for k, block in enumerate(self.blocks):
            if block.last_layer:
                if not block._needs_grad(fx):
                    x_in = normed if normed is not None else block.ln_1(fx)
                    whole = block._whole_block(x_in, fx, block.ln_mlp2[0], head=block.ln_mlp2[1])
                    if whole is not None:  # the block and its output head in one library call
                        fx = whole[1]
                        continue
                    normed = x_in
                fx, normed = block.forward_chain(fx, normed, block.ln_mlp2[0])
                if normed is not None and on_library:
                    fx = self._library_linear(normed, block.ln_mlp2[1])  # output head (:305-307)
                else:
                    fx = block.ln_mlp2[1](normed) if normed is not None else block.ln_mlp2(fx)
            else:
                fx, normed = block.forward_chain(fx, normed, self.blocks[k + 1].ln_1)
        if unflatten_output:
            fx = fx.reshape(fx.shape[0], *self.structured_shape, -1)
        return fx
