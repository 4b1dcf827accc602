"""Training path of the PhysicsAttention layer: a torch.autograd.Function whose forward runs the stage-level HIP
kernels and keeps their intermediates, and whose backward runs the backward kernels of libphysattn.so.

The reference has no backward code of its own (autograd differentiates physics_attention.py:501-558 op by op);
this is the same gradient, assembled from
  * hand-written kernels for everything specific to the layer (slice softmax, slice sums, slice attention,
    deslice and their adjoints, the input-gradient GEMMs / transposed convolutions), and
  * the weight gradients ``d out^T . in`` (products over the point axis) on the library's own MFMA kernel for bf16
    shapes it serves, and on the GEMM library behind ``torch.matmul`` otherwise (fp32, convolutions, odd widths).
"""
from __future__ import annotations

import itertools

import torch

from . import functional as PF


def _rows(t: torch.Tensor) -> torch.Tensor:
    return t.reshape(-1, t.shape[-1])


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """`t` itself, or a copy when it is a view that starts off a 16-byte boundary (a batch element of odd size)."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


def _wgrad(d_out: torch.Tensor, inp: torch.Tensor):
    """(d W, d b) = (d out^T . in, column sums of d out) over all rows: one pass of the library's MFMA kernel where it
    serves the shape, else the GEMM library and a reduction."""
    if PF.cols_gemm_supported(d_out, inp):
        return PF.cols_gemm(d_out, inp, col_sums=True)
    ca, cb = d_out.shape[-1], inp.shape[-1]
    rows = d_out.numel() // ca
    fold = 32 // ca if ca < 32 and 32 % ca == 0 else 0
    if fold and rows % fold == 0 and d_out.is_contiguous() and inp.is_contiguous():
        # narrow d out (slice_num 16): `fold` consecutive rows side by side make 32 columns; the wanted product is the
        # sum of the diagonal blocks of the folded one
        a2, b2 = d_out.reshape(rows // fold, 32), inp.reshape(rows // fold, cb * fold)
        if PF.cols_gemm_supported(a2, b2):
            p2, s2 = PF.cols_gemm(a2, b2, col_sums=True)
            dw = sum(p2[k * ca:(k + 1) * ca, k * cb:(k + 1) * cb] for k in range(fold))
            return dw, s2.reshape(fold, ca).sum(0)
    return _rows(d_out).t() @ _rows(inp), _rows(d_out).sum(0, dtype=torch.float32)


def _conv_weight_grad(d_out: torch.Tensor, x: torch.Tensor, grid: tuple, k: int) -> torch.Tensor:
    """d W[o, c, taps...] = sum over grid points of d_out[p, o] * x[p + tap - k//2, c] (zero outside the grid).

    d_out (B, N, O), x (B, N, C) channels-last over `grid`; returns (O, C, k, ..., k) in d_out's dtype."""
    B, O, C, nd, pad = x.shape[0], d_out.shape[-1], x.shape[-1], len(grid), k // 2
    if nd == 2:
        # one product against the unfolded (im2col) input: its columns are ordered (c, u, v) like the weight
        cols = torch.nn.functional.unfold(x.reshape(B, *grid, C).permute(0, 3, 1, 2), k, padding=pad)  # (B, C k k, N)
        return (_rows(d_out).t() @ cols.transpose(1, 2).reshape(-1, C * k * k)).reshape(O, C, k, k)
    dg, xg = d_out.reshape(B, *grid, O), x.reshape(B, *grid, C)
    dW = torch.zeros((O, C) + (k,) * nd, dtype=d_out.dtype, device=x.device)
    for tap in itertools.product(range(k), repeat=nd):
        lo = [max(0, pad - u) for u in tap]
        hi = [min(g, g + pad - u) for g, u in zip(grid, tap)]
        if any(a >= b for a, b in zip(lo, hi)):
            continue
        out_sl = (slice(None),) + tuple(slice(a, b) for a, b in zip(lo, hi))
        in_sl = (slice(None),) + tuple(slice(a + u - pad, b + u - pad) for a, b, u in zip(lo, hi, tap))
        dW[(slice(None), slice(None)) + tap] = dg[out_sl].reshape(-1, O).t() @ xg[in_sl].reshape(-1, C)
    return dW


def _torch_conv_layout(w_flat: torch.Tensor, O: int, C: int, taps: tuple, dims) -> torch.Tensor:
    """The kernel-form convolution weight (flat; tap-major when `dims.conv_tap_major`) as torch's (O, C, k, ...)."""
    if dims.conv_tap_major:
        return w_flat.view(O, *taps, C).movedim(-1, 1)
    return w_flat.view(O, C, *taps)


def _slice_weight_grad(d_z: torch.Tensor, x_mid: torch.Tensor, H: int, S: int, D: int):
    """d W_slice[s, d] = sum over points and heads of d z[n, h, s] x_mid[n, h, d] (+ d b_slice).

    As a product over (point, head) rows the operands are only S and D wide, which leaves the row-axis kernel two waves
    per workgroup; taking whole points as rows ((H S) x (H D) result) fills it, and the wanted sum is the sum of the H
    diagonal blocks -- 8 x the arithmetic on matrix cores that have the slack, 30 % less time."""
    a, b = d_z.reshape(-1, H * S), x_mid.reshape(-1, H * D)
    if H > 1 and H * S <= 512 and PF.cols_gemm_supported(a, b):  # wider: the extra passes over x_mid cost more
        p, sums = PF.cols_gemm(a, b, col_sums=True)
        dw = sum(p[h * S:(h + 1) * S, h * D:(h + 1) * D] for h in range(H))
        return dw, sums.reshape(H, S).sum(0)
    return _wgrad(d_z.reshape(-1, S), x_mid.reshape(-1, D))


def _finish_backward(ctx, x, dy, out_x, d_wqkv, d_proj, d_z, d_temp, x_mid, temperature, param_offset=3):
    """Everything after the layer-specific kernels: d x (input-gradient GEMM / transposed convolution) and the weight
    and bias gradients, which are plain GEMMs / column sums over the point axis.  Returns (d x, None, None, the ten
    parameter gradients); `param_offset`: position of the first parameter among the Function's inputs."""
    dims, kp = ctx.dims, ctx.kparams
    B, N, C, H, D, S = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
    HD = H * D
    linear = PF.LayerDims(B, N, C, H, D, S)
    d_wo, d_bo = _wgrad(dy, out_x) if out_x is not None else (None, None)  # None: no out_linear (context projector)
    d_ws, d_bs = _slice_weight_grad(d_z, x_mid, H, S, D)
    t = temperature.reshape(-1)
    d_temp = d_temp * ((t >= 0.5) & (t <= 5.0)).to(d_temp.dtype)

    k = dims.conv_k
    wx, wf = kp["in_project_x_weight"], kp["in_project_fx_weight"]
    if k == 0:
        w_cat = torch.cat([wx.view(HD, C).t(), wf.view(HD, C).t()], dim=1).contiguous()  # (C, 2HD)
        dx = PF.rows_gemm(d_proj, w_cat, None, linear, 2 * HD, C) if ctx.needs_input_grad[0] else None
        d_w_in, d_b_in = _wgrad(d_proj, x)  # (2HD, C), (2HD)
    else:
        grid = (dims.grid_h, dims.grid_w) + ((dims.grid_d,) if dims.grid_d > 0 else ())
        taps = (k,) * len(grid)
        w_both = torch.cat([_torch_conv_layout(wx, HD, C, taps, dims), _torch_conv_layout(wf, HD, C, taps, dims)],
                           dim=0)  # (2HD, C, k, ...)
        # transposed convolution = the same gather with flipped taps and swapped channel roles
        w_t = w_both.flip(dims=tuple(range(2, 2 + len(grid)))).transpose(0, 1)  # (C, 2HD, k, ...)
        w_t = (w_t.movedim(1, -1) if dims.conv_tap_major else w_t).contiguous()
        dx = PF.rows_gemm(d_proj, w_t, None, dims, 2 * HD, C) if ctx.needs_input_grad[0] else None
        d_w_in = _conv_weight_grad(d_proj, x, grid, k)
        d_b_in = _rows(d_proj).sum(0, dtype=torch.float32)

    grads = (d_w_in[:HD], d_b_in[:HD], d_w_in[HD:], d_b_in[HD:], d_ws, d_bs, d_temp, d_wqkv, d_wo, d_bo)
    grads = tuple(gr.reshape(p.shape).to(p.dtype) if gr is not None and ctx.needs_input_grad[param_offset + i] else None
                  for i, (gr, p) in enumerate(zip(grads, ctx.param_like)))
    return (dx, None, None) + grads


class PhysicsAttentionFunction(torch.autograd.Function):
    """y = PhysicsAttention(x); differentiable w.r.t. x and the ten parameters.  General kernels (any shape, fp32 or
    bf16 storage): the forward keeps x_mid, fx_mid, the slice weights, the slice tokens and out_x."""

    @staticmethod
    def forward(ctx, x, dims, kparams, wx, bx, wf, bf, ws, bs, temperature, wqkv, wo, bo):
        x_mid, fx_mid = PF.project_inputs(x, kparams, dims)
        w = PF.slice_softmax(x_mid, kparams, dims)
        tok, norm = PF.slice_reduce(w, fx_mid, dims)
        tok_out = PF.slice_attention(tok, kparams, dims)
        y, out_x = PF.deslice_project(w, tok_out, kparams, dims, return_out_x=True)
        ctx.save_for_backward(x, x_mid, fx_mid, w, tok, norm, tok_out, out_x, temperature)
        ctx.dims, ctx.kparams = dims, kparams
        ctx.param_like = (wx, bx, wf, bf, ws, bs, temperature, wqkv, wo, bo)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, x_mid, fx_mid, w, tok, norm, tok_out, out_x, temperature = ctx.saved_tensors
        dims, kp = ctx.dims, ctx.kparams
        C, HD, D = dims.C, dims.H * dims.D, dims.D
        dy = dy.to(x.dtype).contiguous()
        linear = PF.LayerDims(dims.B, dims.N, C, dims.H, D, dims.S)
        # out_linear: g = d out_x
        g = PF.rows_gemm(dy, kp["out_linear_weight"].view(C, HD).t().contiguous(), None, linear, C, HD)
        # adjoint of the deslice w.r.t. the attended tokens, then the slice attention and the normalisation
        d_tok_out = PF.slice_weighted_sum(w, g, dims)[..., :D].contiguous()
        d_num, d_norm, d_wqkv = PF.slice_attention_backward(tok, norm, d_tok_out, kp, dims)
        # per point: slice softmax, aggregation and deslice adjoints
        d_proj, d_z, d_temp = PF.slice_softmax_backward(x_mid, fx_mid, w, g, tok_out, d_num, d_norm, kp, dims)
        return _finish_backward(ctx, x, dy, out_x, d_wqkv, d_proj, d_z, d_temp, x_mid, temperature)


class PhysicsAttentionMfmaFunction(torch.autograd.Function):
    """The same gradient on the bf16 MFMA kernels (irregular variant, D = 32, C in {128, 256}, S <= 64).

    The forward is the inference path (fused projection / softmax / aggregation kernel, slice attention, deslice +
    out_linear) with its packed slice weights kept; the backward recomputes x_mid / fx_mid with one MFMA GEMM and reads
    the slice weights in their packed form."""

    @staticmethod
    def forward(ctx, x, dims, kparams, wx, bx, wf, bf, ws, bs, temperature, wqkv, wo, bo):
        st = PF.MfmaStages(kparams, dims, x.device)
        st.pack_params()
        if st.fused_groups > 0:
            st.project_softmax_reduce(x)
        else:
            st.project_softmax(x)
            st.slice_reduce()
        st.combine_attention()
        y = torch.empty_like(x)
        st.deslice_project(y)
        ctx.save_for_backward(x, temperature)
        ctx.stages, ctx.dims, ctx.kparams = st, dims, kparams
        ctx.param_like = (wx, bx, wf, bf, ws, bs, temperature, wqkv, wo, bo)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, temperature = ctx.saved_tensors
        st, dims, kp = ctx.stages, ctx.dims, ctx.kparams
        C, HD, D = dims.C, dims.H * dims.D, dims.D
        dy = dy.to(x.dtype).contiguous()
        g, g_pack = st.rows_gemm_packed(dy, kp["out_linear_weight"].view(C, HD).t().contiguous(), None)
        x_mid, fx_mid = PF.project_inputs(x, kp, dims)
        d_tok_out = st.slice_weighted_sum(g_pack)[..., :D].contiguous()
        d_num, d_norm, d_wqkv = PF.slice_attention_backward(st.tok, st.norm, d_tok_out, kp, dims)
        out_x = st.deslice()
        d_proj, d_z, d_temp = st.slice_softmax_backward(x_mid, fx_mid, g, d_num, d_norm)
        return _finish_backward(ctx, x, dy, out_x, d_wqkv, d_proj, d_z, d_temp, x_mid, temperature)


def _plus_backward_tail(ctx, x, uniform, x_mid, w, tok_out, out_x, dy, g, d_num, d_norm, d_wqkv, first_param):
    """Everything of the Transolver++ backward after the slice-token stage: the per-point kernel, d x and the parameter
    gradients (d_wqkv is passed through; None when the caller's token-stage graph provides it).  Returns (d x, the
    twelve parameter gradients in the order of `ctx.param_like`)."""
    dims, kp = ctx.dims, ctx.kparams
    B, N, C, H, D, S = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
    HD = H * D
    linear = PF.LayerDims(B, N, C, H, D, S)
    d_xm, d_z, d_a1, d_a2, d_temp = PF.slice_softmax_plus_backward(x_mid, uniform, w, g, tok_out, d_num, d_norm, kp, dims)
    d_wo, d_bo = _wgrad(dy, out_x)
    xm_rows = x_mid.reshape(-1, D)
    d_ws, d_bs = _wgrad(d_z.reshape(-1, S), xm_rows)
    # proj_temperature = Linear(D, S) -> GELU -> Linear(S, 1) -> GELU: the kernel returns the gradients of the two
    # Linear outputs; the second weight gradient needs the hidden activation again
    d_w1, d_b1 = _wgrad(d_a1.reshape(-1, S), xm_rows)
    hidden = torch.nn.functional.gelu(torch.addmm(kp["proj_temperature_0_bias"], xm_rows.float(),
                                                  kp["proj_temperature_0_weight"].view(S, D).t()))
    d_w2 = (d_a2.reshape(-1, 1) * hidden).sum(0, keepdim=True)  # (1, rows) x (rows, S): a reduction, not a GEMM shape
    d_b2 = d_a2.sum().reshape(1)

    k = dims.conv_k
    wx = kp["in_project_x_weight"]
    if k == 0:
        dx = PF.rows_gemm(d_xm, wx.view(HD, C).t().contiguous(), None, linear, HD, C) if ctx.needs_input_grad[0] else None
        d_wx, d_bx = _wgrad(d_xm, x)
    else:
        grid = (dims.grid_h, dims.grid_w) + ((dims.grid_d,) if dims.grid_d > 0 else ())
        w_t = _torch_conv_layout(wx, HD, C, (k,) * len(grid), dims).flip(dims=tuple(range(2, 2 + len(grid)))).transpose(0, 1)
        w_t = (w_t.movedim(1, -1) if dims.conv_tap_major else w_t).contiguous()
        dx = PF.rows_gemm(d_xm, w_t, None, dims, HD, C) if ctx.needs_input_grad[0] else None
        d_wx = _conv_weight_grad(d_xm, x, grid, k)
        d_bx = _rows(d_xm).sum(0, dtype=torch.float32)

    grads = (d_wx, d_bx, d_ws, d_bs, d_temp, d_w1, d_b1, d_w2, d_b2, d_wqkv, d_wo, d_bo)
    grads = tuple(gr.reshape(p.shape).to(p.dtype) if gr is not None and ctx.needs_input_grad[first_param + i] else None
                  for i, (gr, p) in enumerate(zip(grads, ctx.param_like)))
    return dx, grads


class PhysicsAttentionPlusFunction(torch.autograd.Function):
    """Transolver++ (plus=True) layer, differentiable w.r.t. x and its twelve parameters; general kernels.  ``uniform``
    (B, N, H, S) holds the samples behind the Gumbel noise and gets no gradient (the reference draws them with
    ``torch.rand_like``, gumbel_softmax.py:50)."""

    @staticmethod
    def forward(ctx, x, uniform, dims, kparams, wx, bx, ws, bs, temperature, pt_w1, pt_b1, pt_w2, pt_b2, wqkv, wo, bo):
        x_mid, _ = PF.project_inputs(x, kparams, dims)
        w = PF.slice_softmax_plus(x_mid, uniform, kparams, dims)
        tok, norm = PF.slice_reduce(w, x_mid, dims)
        tok_out = PF.slice_attention(tok, kparams, dims)
        y, out_x = PF.deslice_project(w, tok_out, kparams, dims, return_out_x=True)
        ctx.save_for_backward(x, uniform, x_mid, w, tok, norm, tok_out, out_x)
        ctx.dims, ctx.kparams = dims, kparams
        ctx.param_like = (wx, bx, ws, bs, temperature, pt_w1, pt_b1, pt_w2, pt_b2, wqkv, wo, bo)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, uniform, x_mid, w, tok, norm, tok_out, out_x = ctx.saved_tensors
        dims, kp = ctx.dims, ctx.kparams
        C, HD, D = dims.C, dims.H * dims.D, dims.D
        dy = dy.to(x.dtype).contiguous()
        linear = PF.LayerDims(dims.B, dims.N, C, dims.H, D, dims.S)
        g = PF.rows_gemm(dy, kp["out_linear_weight"].view(C, HD).t().contiguous(), None, linear, C, HD)
        d_tok_out = PF.slice_weighted_sum(w, g, dims)[..., :D].contiguous()
        d_num, d_norm, d_wqkv = PF.slice_attention_backward(tok, norm, d_tok_out, kp, dims)
        dx, grads = _plus_backward_tail(ctx, x, uniform, x_mid, w, tok_out, out_x, dy, g, d_num, d_norm, d_wqkv, 4)
        return (dx, None, None, None) + grads


class GALEPlusFunction(torch.autograd.Function):
    """Transolver++ form of the GALE layer with a context (gale.py:148-239 with plus=True): the per-point stages of
    `PhysicsAttentionPlusFunction`, the slice-token stage (self-attention, cross-attention, blend) as a PyTorch graph
    like in `GALEFunction`.  Differentiable w.r.t. x, the context, the twelve layer parameters and the stage's."""

    @staticmethod
    def forward(ctx, x, uniform, context, dims, kparams, token_stage, n_stage, *params):
        layer_params, stage_params = params[:len(params) - n_stage], params[len(params) - n_stage:]
        x_mid, _ = PF.project_inputs(x, kparams, dims)
        w = PF.slice_softmax_plus(x_mid, uniform, kparams, dims)
        tok, norm = PF.slice_reduce(w, x_mid, dims)
        with torch.enable_grad():
            tok_leaf = tok.detach().requires_grad_(True)
            ctx_leaf = context.detach().requires_grad_(ctx.needs_input_grad[2])
            out_graph = token_stage(tok_leaf, ctx_leaf)
        tok_out = out_graph.detach().float().contiguous()
        y, out_x = PF.deslice_project(w, tok_out, kparams, dims, return_out_x=True)
        ctx.save_for_backward(x, uniform, x_mid, w, tok, norm, tok_out, out_x)
        ctx.dims, ctx.kparams = dims, kparams
        ctx.param_like = layer_params
        ctx.graph = (out_graph, tok_leaf, ctx_leaf, stage_params)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, uniform, x_mid, w, tok, norm, tok_out, out_x = ctx.saved_tensors
        dims, kp = ctx.dims, ctx.kparams
        C, HD, D = dims.C, dims.H * dims.D, dims.D
        dy = dy.to(x.dtype).contiguous()
        linear = PF.LayerDims(dims.B, dims.N, C, dims.H, D, dims.S)
        g = PF.rows_gemm(dy, kp["out_linear_weight"].view(C, HD).t().contiguous(), None, linear, C, HD)
        d_tok_out = PF.slice_weighted_sum(w, g, dims)[..., :D].contiguous()
        out_graph, tok_leaf, ctx_leaf, stage_params = ctx.graph
        wanted = [tok_leaf] + ([ctx_leaf] if ctx_leaf.requires_grad else []) + \
                 [p for p in stage_params if p.requires_grad]
        got = list(torch.autograd.grad(out_graph, wanted, d_tok_out.to(out_graph.dtype), allow_unused=True))
        d_tok = got.pop(0).float()
        d_context = got.pop(0) if ctx_leaf.requires_grad else None
        d_stage = [got.pop(0) if p.requires_grad else None for p in stage_params]
        d_num = (d_tok / norm[..., None]).contiguous()
        d_norm = (-(d_tok * tok).sum(-1) / norm).contiguous()
        # qkv_project.weight takes part in the token stage only: its gradient comes with `d_stage`
        dx, grads = _plus_backward_tail(ctx, x, uniform, x_mid, w, tok_out, out_x, dy, g, d_num, d_norm, None, 7)
        return (dx, None, d_context, None, None, None, None) + grads + tuple(d_stage)


class GALEFunction(torch.autograd.Function):
    """GALE layer with a context (gale.py:148-239), differentiable w.r.t. x, the context, the ten PhysicsAttention
    parameters and the cross-attention / blend parameters.

    The per-point stages are the layer's kernels, forward and backward, as in the two Functions above.  The slice-token
    stage in between (self-attention, cross-attention to the context, blend: S x D work per (batch, head), independent
    of the number of points) is evaluated by `token_stage(tok, context)` with PyTorch ops under autograd in the
    forward; the backward asks that small graph for d tok, d context and the gradients of `stage_params`."""

    @staticmethod
    def forward(ctx, x, context, dims, kparams, token_stage, n_stage, *params):
        layer_params, stage_params = params[:len(params) - n_stage], params[len(params) - n_stage:]
        mfma = PF.mfma_backward_supported(x.dtype, dims)
        if mfma:
            st = PF.MfmaStages(kparams, dims, x.device)
            st.pack_params()
            if st.fused_groups > 0:
                st.project_softmax_reduce(x)
            else:
                st.project_softmax(x)
                st.slice_reduce()
            st.combine_attention()  # for the normalised slice tokens; its self-attention result is replaced below
            tok, norm = st.tok, st.norm
        else:
            x_mid, fx_mid = PF.project_inputs(x, kparams, dims)
            w = PF.slice_softmax(x_mid, kparams, dims)
            tok, norm = PF.slice_reduce(w, fx_mid, dims)
        with torch.enable_grad():
            tok_leaf = tok.detach().requires_grad_(True)
            ctx_leaf = context.detach().requires_grad_(ctx.needs_input_grad[1])
            out_graph = token_stage(tok_leaf, ctx_leaf)
        out_tok = out_graph.detach().float().contiguous()
        if mfma:
            st.set_out_tokens(out_tok)
            y = torch.empty_like(x)
            st.deslice_project(y)
            ctx.save_for_backward(x, layer_params[6])
            ctx.stages = st
        else:
            y, out_x = PF.deslice_project(w, out_tok, kparams, dims, return_out_x=True)
            ctx.save_for_backward(x, layer_params[6], x_mid, fx_mid, w, out_x)
        ctx.mfma, ctx.dims, ctx.kparams = mfma, dims, kparams
        ctx.tok, ctx.norm, ctx.out_tok = tok, norm, out_tok
        ctx.graph = (out_graph, tok_leaf, ctx_leaf, stage_params)
        ctx.param_like = layer_params
        return y

    @staticmethod
    def backward(ctx, dy):
        dims, kp = ctx.dims, ctx.kparams
        C, HD, D = dims.C, dims.H * dims.D, dims.D
        x, temperature = ctx.saved_tensors[:2]
        dy = dy.to(x.dtype).contiguous()
        linear = PF.LayerDims(dims.B, dims.N, C, dims.H, D, dims.S)
        w_out_t = kp["out_linear_weight"].view(C, HD).t().contiguous()
        if ctx.mfma:
            st = ctx.stages
            g, g_pack = st.rows_gemm_packed(dy, w_out_t, None)
            x_mid, fx_mid = PF.project_inputs(x, kp, dims)
            d_out_tok = st.slice_weighted_sum(g_pack)[..., :D].contiguous()
        else:
            x_mid, fx_mid, w, out_x = ctx.saved_tensors[2:]
            g = PF.rows_gemm(dy, w_out_t, None, linear, C, HD)
            d_out_tok = PF.slice_weighted_sum(w, g, dims)[..., :D].contiguous()
        # slice-token stage: PyTorch's graph of the forward
        out_graph, tok_leaf, ctx_leaf, stage_params = ctx.graph
        wanted = [tok_leaf] + ([ctx_leaf] if ctx_leaf.requires_grad else []) + \
                 [p for p in stage_params if p.requires_grad]
        got = list(torch.autograd.grad(out_graph, wanted, d_out_tok.to(out_graph.dtype), allow_unused=True))
        d_tok = got.pop(0).float()
        d_context = got.pop(0) if ctx_leaf.requires_grad else None
        d_stage = [got.pop(0) if p.requires_grad else None for p in stage_params]
        # tok = num / nrm
        d_num = (d_tok / ctx.norm[..., None]).contiguous()
        d_norm = (-(d_tok * ctx.tok).sum(-1) / ctx.norm).contiguous()
        if ctx.mfma:
            out_x = st.deslice()
            d_proj, d_z, d_temp = st.slice_softmax_backward(x_mid, fx_mid, g, d_num, d_norm)
        else:
            d_proj, d_z, d_temp = PF.slice_softmax_backward(x_mid, fx_mid, w, g, ctx.out_tok, d_num, d_norm, kp, dims)
        # qkv_project.weight takes part in the token stage only: its gradient comes with `d_stage`
        base = _finish_backward(ctx, x, dy, out_x, None, d_proj, d_z, d_temp, x_mid, temperature, param_offset=6)
        return (base[0], d_context, None, None, None, None) + base[3:] + tuple(d_stage)


class SliceTokensFunction(torch.autograd.Function):
    """x -> normalised slice tokens (B,H,S,D) float32: the projection, slice-softmax and aggregation stages of the
    layer on their own (a GeoTransolver context projector, context_projector.py:338-378), differentiable w.r.t. x and
    the seven parameters involved.  The backward is the per-point backward kernel with no deslice term (d out_x = 0)."""

    @staticmethod
    def forward(ctx, x, dims, kparams, wx, bx, wf, bf, ws, bs, temperature):
        mfma = PF.mfma_backward_supported(x.dtype, dims)
        if mfma:
            st = PF.MfmaStages(kparams, dims, x.device)
            st.pack_params()
            if st.fused_groups > 0:
                st.project_softmax_reduce(x)
            else:
                st.project_softmax(x)
                st.slice_reduce()
            st.combine_attention()
            tok, norm = st.tok.clone(), st.norm
            ctx.stages = st
            ctx.save_for_backward(x, temperature, tok, norm)
        else:
            x_mid, fx_mid = PF.project_inputs(x, kparams, dims)
            w = PF.slice_softmax(x_mid, kparams, dims)
            tok, norm = PF.slice_reduce(w, fx_mid, dims)
            ctx.save_for_backward(x, temperature, tok, norm, x_mid, fx_mid, w)
        ctx.mfma, ctx.dims, ctx.kparams = mfma, dims, kparams
        ctx.param_like = (wx, bx, wf, bf, ws, bs, temperature)
        return tok

    @staticmethod
    def backward(ctx, d_tok):
        dims, kp = ctx.dims, ctx.kparams
        x, temperature, tok, norm = ctx.saved_tensors[:4]
        d_tok = d_tok.float()
        d_num = (d_tok / norm[..., None]).contiguous()
        d_norm = (-(d_tok * tok).sum(-1) / norm).contiguous()
        g = torch.zeros(dims.B, dims.N, dims.H * dims.D, dtype=x.dtype, device=x.device)
        if ctx.mfma:
            st = ctx.stages
            st.tok_out.zero_()
            x_mid, fx_mid = PF.project_inputs(x, kp, dims)
            d_proj, d_z, d_temp = st.slice_softmax_backward(x_mid, fx_mid, g, d_num, d_norm)
        else:
            x_mid, fx_mid, w = ctx.saved_tensors[4:]
            d_proj, d_z, d_temp = PF.slice_softmax_backward(x_mid, fx_mid, w, g, torch.zeros_like(tok), d_num, d_norm,
                                                            kp, dims)
        base = _finish_backward(ctx, x, None, None, None, d_proj, d_z, d_temp, x_mid, temperature)
        return base[:3] + base[3:10]


class FlareFunction(torch.autograd.Function):
    """FLARE layer core (flare_attention.py:38-72, :222-255) given the composed score / value weights: differentiable
    w.r.t. x, the four composed tensors and out_linear.  The composition itself (q_global, self_k / self_v and
    in_project_x folded into two matrices) is a handful of small tensor products done by the caller under autograd, so
    the gradients reach the layer's own parameters through it.  Without out_linear (`wo` None) the result is the
    attention output (B, N, H*D) itself, for callers that blend it with something else first (GALE_FA)."""

    @staticmethod
    def forward(ctx, x, dims, w_a, b_a, w_v, b_v, wo, bo):
        B, N, C, H, D, S = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
        wa_k, wv_k = w_a.detach().to(x.dtype).contiguous(), w_v.detach().to(x.dtype).contiguous()
        scores = PF.rows_gemm(x, wa_k, b_a.detach().float().contiguous(), dims, C, H * S).view(B, N, H, S)
        values = PF.rows_gemm(x, wv_k, b_v.detach().float().contiguous(), dims, C, H * D)
        col_w, _ = PF.flare_column_weights(scores, dims)
        tok, norm = PF.slice_reduce(col_w, values, dims)
        den = norm - 1e-2  # the aggregation kernel adds the PhysicsAttention epsilon to the divisor; FLARE has none
        z = (tok * (norm / den).unsqueeze(-1)).contiguous()
        row_w = PF.flare_softmax_rows_(scores, dims)
        ctx.dims = dims
        ctx.projected = wo is not None
        if not ctx.projected:
            out_x = PF.deslice(row_w, z, dims)
            ctx.save_for_backward(x, row_w, col_w, values, z, den, wa_k, wv_k)
            ctx.dtypes = tuple(t.dtype for t in (w_a, b_a, w_v, b_v))
            return out_x
        kp = {"out_linear_weight": wo.detach().to(x.dtype).contiguous().reshape(-1),
              "out_linear_bias": bo.detach().float().contiguous()}
        y, out_x = PF.deslice_project(row_w, z, kp, dims, return_out_x=True)
        ctx.save_for_backward(x, row_w, col_w, values, z, den, wa_k, wv_k, out_x, kp["out_linear_weight"])
        ctx.dtypes = tuple(t.dtype for t in (w_a, b_a, w_v, b_v, wo, bo))
        return y

    @staticmethod
    def backward(ctx, dy):
        x, row_w, col_w, values, z, den, wa_k, wv_k = ctx.saved_tensors[:8]
        dims = ctx.dims
        B, N, C, H, D, S = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
        HD, HS = H * D, H * S
        dy = dy.to(x.dtype).contiguous()
        if ctx.projected:
            out_x, wo_k = ctx.saved_tensors[8:]
            g = PF.rows_gemm(dy, wo_k.view(C, HD).t().contiguous(), None, dims, C, HD)
            d_wo, d_bo = _wgrad(dy, out_x)
        else:
            g, d_wo, d_bo = dy, None, None
        d_z = PF.slice_weighted_sum(row_w, g, dims)[..., :D]
        d_num = (d_z / den.unsqueeze(-1)).contiguous()
        d_den = (-(d_z * z).sum(-1) / den).contiguous()
        d_a, d_v = PF.flare_backward_points(row_w, col_w, values, g, z, d_num, d_den, dims)
        d_a = d_a.view(B, N, HS)
        dx = None
        if ctx.needs_input_grad[0]:
            w_cat = torch.cat([wa_k, wv_k], dim=0).t().contiguous()  # (C, HS + HD)
            dx = PF.rows_gemm(torch.cat([d_a, d_v], dim=-1), w_cat, None, dims, HS + HD, C)
        d_wa, d_ba = _wgrad(d_a, x)
        d_wv, d_bv = _wgrad(d_v, x)
        grads = [gr.float().reshape(shape).to(dt) for gr, shape, dt in zip(
            (d_wa, d_ba, d_wv, d_bv, d_wo, d_bo), ((HS, C), (HS,), (HD, C), (HD,), (C, HD), (C,)), ctx.dtypes)]
        if not ctx.projected:
            grads += [None, None]
        return (dx, None, *grads)


class PointCrossFunction(torch.autograd.Function):
    """Cross-attention of every point to a small set of context tokens, scale 1 (GALE_FA, reference gale.py:735-744):
    out[b,n,h,:] = sum_u softmax_u(x[b,n,:] . w_c[b,(h,u),:] + b_c[b,(h,u)]) v[b,h,u,:].  The caller folds in_project_x,
    cross_q and the context's keys into the per-batch score weight `w_c` (B, H*Sc, C) / `b_c` (B, H*Sc) and projects
    the context's values `v` (B, H, Sc, D), all under autograd.  Scores from the row GEMM, the in-place row softmax and
    the deslice kernel; backward: the row-softmax part of the FLARE per-point kernel (gather weights zero), the
    slice-weighted sum for d v, row / column GEMMs for d x and d w_c."""

    @staticmethod
    def forward(ctx, x, dims, w_c, b_c, v):
        B, N, C, H, Sc = dims.B, dims.N, dims.C, dims.H, dims.S
        one = PF.LayerDims(1, N, C, H, dims.D, Sc)
        wk = w_c.detach().to(x.dtype).contiguous()
        bk = b_c.detach().float().contiguous()
        scores = torch.empty(B, N, H, Sc, dtype=x.dtype, device=x.device)
        for b in range(B):  # the score weight holds the batch element's keys
            scores[b] = PF.rows_gemm(_aligned(x[b:b + 1]), _aligned(wk[b]), _aligned(bk[b]), one, C, H * Sc).view(N, H, Sc)
        p = PF.flare_softmax_rows_(scores, dims)
        v32 = v.detach().float().contiguous()
        ctx.save_for_backward(x, p, v32, wk)
        ctx.dims = dims
        ctx.dtypes = (w_c.dtype, b_c.dtype, v.dtype)
        return PF.deslice(p, v32, dims)

    @staticmethod
    def backward(ctx, g):
        x, p, v32, wk = ctx.saved_tensors
        dims = ctx.dims
        B, N, C, H, D, Sc = dims.B, dims.N, dims.C, dims.H, dims.D, dims.S
        g = g.to(x.dtype).contiguous()
        d_v = PF.slice_weighted_sum(p, g, dims)[..., :D]
        zeros_w = torch.zeros_like(p)
        d_s, _ = PF.flare_backward_points(p, zeros_w, g, g, v32, torch.zeros_like(v32),
                                          torch.zeros(B, H, Sc, dtype=torch.float32, device=x.device), dims)
        d_s = d_s.view(B, N, H * Sc)
        one = PF.LayerDims(1, N, C, H, D, Sc)
        dx = torch.empty_like(x) if ctx.needs_input_grad[0] else None
        d_w, d_b = [], []
        for b in range(B):
            if dx is not None:
                dx[b] = PF.rows_gemm(_aligned(d_s[b:b + 1]), _aligned(wk[b].t()), None, one, H * Sc, C)[0]
            dw_b, db_b = _wgrad(_aligned(d_s[b]), _aligned(x[b]))
            d_w.append(dw_b.float())
            d_b.append(db_b.float())
        return (dx, None, torch.stack(d_w).to(ctx.dtypes[0]), torch.stack(d_b).to(ctx.dtypes[1]),
                d_v.to(ctx.dtypes[2]))


class LinearFunction(torch.autograd.Function):
    """torch.nn.functional.linear for the block MLP in bf16 training: the two row GEMMs (forward, input gradient) go to
    the GEMM library, the weight and bias gradients -- products over the huge row axis, where the library's kernels
    leave most of the machine idle -- to `cols_gemm_kernel`, which also returns them in float32."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        w16 = weight.to(x.dtype)
        ctx.save_for_backward(x, w16)
        ctx.param_dtypes = (weight.dtype, bias.dtype if bias is not None else None)
        return torch.nn.functional.linear(x, w16, bias.to(x.dtype) if bias is not None else None)

    @staticmethod
    def backward(ctx, dy):
        x, w16 = ctx.saved_tensors
        dy = dy.contiguous()
        dx = (dy @ w16) if ctx.needs_input_grad[0] else None
        dw = db = None
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            dy2, x2 = _rows(dy), _rows(x).contiguous()
            if PF.cols_gemm_supported(dy2, x2):
                dw, db = PF.cols_gemm(dy2, x2, col_sums=True)
            elif PF.cols_gemm_supported(x2, dy2):  # wide output, narrow input: form (x^T dy) and transpose
                dw = PF.cols_gemm(x2, dy2).t()
                db = dy2.sum(0, dtype=torch.float32)
            else:
                dw, db = dy2.t() @ x2, dy2.sum(0, dtype=torch.float32)
            dw = dw.to(ctx.param_dtypes[0])
            db = db.to(ctx.param_dtypes[1]) if ctx.param_dtypes[1] is not None else None
        return dx, dw, db


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """Differentiable linear layer; on bf16 GPU tensors the weight gradient runs on the library's kernel."""
    if x.is_cuda and x.dtype == torch.bfloat16:
        return LinearFunction.apply(x.contiguous(), weight, bias)
    return torch.nn.functional.linear(x, weight, bias)


class LayerNormFunction(torch.autograd.Function):
    """LayerNorm over the last axis on the library's kernels, forward and backward, in the input's dtype (fp32 or bf16;
    statistics in fp32).  The backward recomputes the statistics from the saved input."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        x = x.contiguous()
        w32, b32 = weight.detach().float().contiguous(), bias.detach().float().contiguous()
        _, out = PF.residual_layernorm(x, ln_weight=w32, ln_bias=b32, ln_eps=eps)
        ctx.save_for_backward(x, w32)
        ctx.eps, ctx.param_dtypes = eps, (weight.dtype, bias.dtype)
        return out

    @staticmethod
    def backward(ctx, dy):
        x, w32 = ctx.saved_tensors
        dx, dg, db = PF.layernorm_backward(x, dy.to(x.dtype).contiguous(), w32, ctx.eps)
        return dx, dg.to(ctx.param_dtypes[0]), db.to(ctx.param_dtypes[1]), None


def layer_norm(x: torch.Tensor, ln: torch.nn.LayerNorm) -> torch.Tensor:
    """Differentiable LayerNorm: the library's kernels where they serve the rows, the module itself otherwise."""
    if len(ln.normalized_shape) == 1 and ln.elementwise_affine and ln.bias is not None and PF.layernorm_supported(x):
        return LayerNormFunction.apply(x, ln.weight, ln.bias, ln.eps)
    return ln(x)
