"""Float64 NumPy restatement of one PhysicsAttention layer / Transolver block, written from the formulas.

TEST INFRASTRUCTURE ONLY (see oracle/torch_oracle.py for the rule on who may import oracle/).

This file deliberately shares no code with ``torch_oracle.py``: it uses index-explicit einsum / loops in
float64 so that a transposed operand, a wrong head split or a dropped term in either restatement makes the
two disagree.  Each step cites the reference lines (relative to the reference checkout) it follows.
Inputs are plain ``dict[str, np.ndarray]`` keyed like the reference ``state_dict``.
"""

from __future__ import annotations

import math

import numpy as np

_erf = np.vectorize(math.erf, otypes=[np.float64])


def _f64(a):
    return np.asarray(a, dtype=np.float64)


def linear_projection(x, weight, bias):
    """y[b,n,o] = sum_c x[b,n,c] W[o,c] + bias[o]  (nn.Linear; physics_attention.py:625-627)."""
    return np.einsum("bnc,oc->bno", _f64(x), _f64(weight)) + _f64(bias)


def conv2d_projection(x, weight, bias, grid_h, grid_w):
    """Zero-padded stride-1 cross-correlation on tokens n = i*grid_w + j (physics_attention.py:740,772-783).

    y[b, i*W+j, o] = bias[o] + sum_{c,u,v} W[o,c,u,v] * x[b, (i+u-p)*W + (j+v-p), c], p = k//2, out-of-grid terms are 0.
    Direct loops over the k*k taps.
    """
    x = _f64(x)
    weight = _f64(weight)
    b, n, c = x.shape
    o, c2, k, k2 = weight.shape
    assert n == grid_h * grid_w and c == c2 and k == k2
    p = k // 2
    img = x.reshape(b, grid_h, grid_w, c)
    out = np.zeros((b, grid_h, grid_w, o))
    for u in range(k):
        for v in range(k):
            di, dj = u - p, v - p
            i0, i1 = max(0, -di), min(grid_h, grid_h - di)
            j0, j1 = max(0, -dj), min(grid_w, grid_w - dj)
            if i0 >= i1 or j0 >= j1:
                continue
            src = img[:, i0 + di:i1 + di, j0 + dj:j1 + dj, :]
            out[:, i0:i1, j0:j1, :] += np.einsum("bijc,oc->bijo", src, weight[:, :, u, v])
    return out.reshape(b, n, o) + _f64(bias)


def conv3d_projection(x, weight, bias, grid_h, grid_w, grid_d):
    """Zero-padded stride-1 cross-correlation on tokens n = (i*W + j)*Dg + l (physics_attention.py:865-867,892-907).

    y[b, n(i,j,l), o] = bias[o] + sum_{c,u,v,z} W[o,c,u,v,z] * x[b, n(i+u-p, j+v-p, l+z-p), c], p = k//2,
    out-of-grid terms are 0.  Direct loops over the k^3 taps.
    """
    x = _f64(x)
    weight = _f64(weight)
    b, n, c = x.shape
    o, c2, k, k2, k3 = weight.shape
    assert n == grid_h * grid_w * grid_d and c == c2 and k == k2 == k3
    p = k // 2
    vol = x.reshape(b, grid_h, grid_w, grid_d, c)
    out = np.zeros((b, grid_h, grid_w, grid_d, o))
    for u in range(k):
        for v in range(k):
            for z in range(k):
                di, dj, dl = u - p, v - p, z - p
                i0, i1 = max(0, -di), min(grid_h, grid_h - di)
                j0, j1 = max(0, -dj), min(grid_w, grid_w - dj)
                l0, l1 = max(0, -dl), min(grid_d, grid_d - dl)
                if i0 >= i1 or j0 >= j1 or l0 >= l1:
                    continue
                src = vol[:, i0 + di:i1 + di, j0 + dj:j1 + dj, l0 + dl:l1 + dl, :]
                out[:, i0:i1, j0:j1, l0:l1, :] += np.einsum("bijlc,oc->bijlo", src, weight[:, :, u, v, z])
    return out.reshape(b, n, o) + _f64(bias)


def layer_forward(p, x, heads, dim_head, variant="irregular", spatial_shape=None, noise_u=None, context=None):
    """All intermediates of one layer in float64 (steps 1-9 below follow physics_attention.py:529-558).

    p: in_project_x.{weight,bias}, in_project_fx.{weight,bias}, in_project_slice.{weight,bias},
       temperature, qkv_project.weight, out_linear.{weight,bias}
    Transolver++ (plus=True) is selected by the absence of in_project_fx.weight: then fx_mid = x_mid (:530-532),
    p also holds proj_temperature.{0,2}.{weight,bias} and noise_u (B, N, H, S) holds the uniform samples behind
    the Gumbel noise (gumbel_softmax.py:50).
    GALE (gale.py:148-239): with `context` (B, H, Sc, Dc) and cross_{q,k,v}.{weight,bias} plus either state_mixing or
    concat_project.0.{weight,bias} in p, the attended slice tokens are blended with their cross-attention to the context.
    """
    plus = "in_project_fx.weight" not in p
    if plus:
        p = dict(p)
        p["in_project_fx.weight"], p["in_project_fx.bias"] = p["in_project_x.weight"], p["in_project_x.bias"]
    x = _f64(x)
    B, N, C = x.shape
    H, D = heads, dim_head
    # 1. projections, channel c = h*D + d (:114-117, :652-660 / :768-783)
    if variant == "irregular":
        xm = linear_projection(x, p["in_project_x.weight"], p["in_project_x.bias"])
        fm = linear_projection(x, p["in_project_fx.weight"], p["in_project_fx.bias"])
    elif len(spatial_shape) == 3:
        gh, gw, gd = spatial_shape
        xm = conv3d_projection(x, p["in_project_x.weight"], p["in_project_x.bias"], gh, gw, gd)
        fm = conv3d_projection(x, p["in_project_fx.weight"], p["in_project_fx.bias"], gh, gw, gd)
    else:
        gh, gw = spatial_shape
        xm = conv2d_projection(x, p["in_project_x.weight"], p["in_project_x.bias"], gh, gw)
        fm = conv2d_projection(x, p["in_project_fx.weight"], p["in_project_fx.bias"], gh, gw)
    xm = xm.reshape(B, N, H, D)
    fm = fm.reshape(B, N, H, D)
    # 2. slice logits, one (S, D) weight shared by all heads (:537)
    ws, bs = _f64(p["in_project_slice.weight"]), _f64(p["in_project_slice.bias"])
    S = ws.shape[0]
    logits = np.einsum("bnhd,sd->bnhs", xm, ws) + bs
    # 3. clamp temperature to [0.5, 5], softmax over S (:173-178)
    if plus:
        # per-point temperature, clamped from below only (:168-169); noise added before the division
        # (gumbel_softmax.py:50-55)
        h1 = gelu_erf(np.einsum("bnhd,sd->bnhs", xm, _f64(p["proj_temperature.0.weight"]))
                      + _f64(p["proj_temperature.0.bias"]))
        h2 = gelu_erf(np.einsum("bnhs,os->bnho", h1, _f64(p["proj_temperature.2.weight"]))
                      + _f64(p["proj_temperature.2.bias"]))
        t = np.maximum(_f64(p["temperature"]).reshape(1, 1, H, 1) + h2, 0.01)
        u = _f64(noise_u)
        z = (logits + -np.log(-np.log(u + 1e-8) + 1e-8)) / t
    else:
        t = np.clip(_f64(p["temperature"]).reshape(H), 0.5, 5.0)
        z = logits / t[None, None, :, None]
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    w = e / e.sum(axis=-1, keepdims=True)
    # 4. norm over points + 1e-2 (:185)
    norm = w.sum(axis=1) + 1e-2  # (B, H, S)
    # 5. slice tokens = sum_n (w / norm) fx_mid (:188-203)
    tok = np.einsum("bnhs,bnhd->bhsd", w / norm[:, None, :, :], fm)
    # 6. qkv = tok Wqkv^T (no bias, :309,:448); q | k | v split in that order (:450,:458)
    wqkv = _f64(p["qkv_project.weight"])
    q = np.einsum("bhsd,ed->bhse", tok, wqkv[0:D])
    k = np.einsum("bhsd,ed->bhse", tok, wqkv[D:2 * D])
    v = np.einsum("bhsd,ed->bhse", tok, wqkv[2 * D:3 * D])
    # 7. softmax(q k^T / sqrt(D)) v (:461-463, default SDPA scale)
    sc = np.einsum("bhse,bhte->bhst", q, k) / math.sqrt(D)
    sc = sc - sc.max(axis=-1, keepdims=True)
    a = np.exp(sc)
    a = a / a.sum(axis=-1, keepdims=True)
    tok_out = np.einsum("bhst,bhte->bhse", a, v)
    if context is not None:
        tok_out = gale_blend(p, tok, tok_out, context)
    # 8. deslice with the un-normalised w, merge heads (:492-495)
    o = np.einsum("bnhs,bhsd->bnhd", w, tok_out).reshape(B, N, H * D)
    # 9. output projection (:498)
    y = np.einsum("bnk,ok->bno", o, _f64(p["out_linear.weight"])) + _f64(p["out_linear.bias"])
    return dict(x_mid=xm, fx_mid=fm, logits=logits, w=w, norm=norm, tok=tok, tok_out=tok_out, y=y)


def gale_blend(p, tok, self_out, context):
    """GALE slice-token stage: cross-attention to the context (gale.py:112-144) and the blend (gale.py:76-84)."""
    ctx = _f64(context)
    D = tok.shape[-1]
    q = np.einsum("bhsd,ed->bhse", tok, _f64(p["cross_q.weight"])) + _f64(p["cross_q.bias"])
    k = np.einsum("bhuc,ec->bhue", ctx, _f64(p["cross_k.weight"])) + _f64(p["cross_k.bias"])
    v = np.einsum("bhuc,ec->bhue", ctx, _f64(p["cross_v.weight"])) + _f64(p["cross_v.bias"])
    sc = np.einsum("bhse,bhue->bhsu", q, k) / math.sqrt(D)
    sc = sc - sc.max(axis=-1, keepdims=True)
    a = np.exp(sc)
    a = a / a.sum(axis=-1, keepdims=True)
    cross = np.einsum("bhsu,bhue->bhse", a, v)
    if "state_mixing" in p:
        m = 1.0 / (1.0 + np.exp(-float(np.asarray(p["state_mixing"]).reshape(-1)[0])))
        return m * self_out + (1.0 - m) * cross
    cat = np.concatenate([self_out, cross], axis=-1)
    return gelu_erf(np.einsum("bhsk,ek->bhse", cat, _f64(p["concat_project.0.weight"])) + _f64(p["concat_project.0.bias"]))


def flare_forward(p, x, heads, dim_head):
    """FLARE layer in float64 (flare_attention.py:38-72, :222-255): scores A = k G^T with scale 1, softmax over the
    points for the gather, softmax over the global queries for the hand-back."""
    x = _f64(x)
    B, N, C = x.shape
    H, D = heads, dim_head
    xm = (np.einsum("bnc,oc->bno", x, _f64(p["in_project_x.weight"])) + _f64(p["in_project_x.bias"])).reshape(B, N, H, D)
    k = np.einsum("bnhd,ed->bnhe", xm, _f64(p["self_k.weight"])) + _f64(p["self_k.bias"])
    v = np.einsum("bnhd,ed->bnhe", xm, _f64(p["self_v.weight"])) + _f64(p["self_v.bias"])
    g = _f64(p["q_global"])[0]  # (H, S, D)
    a = np.einsum("bnhe,hse->bnhs", k, g)
    col = np.exp(a - a.max(axis=1, keepdims=True))
    col = col / col.sum(axis=1, keepdims=True)          # softmax over the points, per (b, h, s)
    z = np.einsum("bnhs,bnhe->bhse", col, v)
    row = np.exp(a - a.max(axis=-1, keepdims=True))
    row = row / row.sum(axis=-1, keepdims=True)         # softmax over the global queries, per (b, n, h)
    y = np.einsum("bnhs,bhse->bnhe", row, z).reshape(B, N, H * D)
    return np.einsum("bnk,ok->bno", y, _f64(p["out_linear.weight"])) + _f64(p["out_linear.bias"])


def layer_norm(x, gamma, beta, eps=1e-5):
    """Biased-variance LayerNorm over the last axis (torch.nn.LayerNorm default eps; transolver.py:210)."""
    x = _f64(x)
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * _f64(gamma) + _f64(beta)


def gelu_erf(x):
    """Exact GELU: 0.5 x (1 + erf(x / sqrt 2)) (activations.py:198 'gelu' -> nn.GELU())."""
    x = _f64(x)
    return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))


def mlp(p, prefix, x):
    """Linear -> GELU -> Linear with keys layers.0 / layers.2 (mlp_layers.py:139-156)."""
    h = np.einsum("bnc,oc->bno", _f64(x), _f64(p[prefix + "layers.0.weight"])) + _f64(p[prefix + "layers.0.bias"])
    h = gelu_erf(h)
    return np.einsum("bnc,oc->bno", h, _f64(p[prefix + "layers.2.weight"])) + _f64(p[prefix + "layers.2.bias"])


def block_forward(p, fx, heads, dim_head, last_layer, variant="irregular", spatial_shape=None):
    """One Transolver block (transolver.py:300-309); p holds the block's state_dict (keys 'ln_1.weight', 'Attn.*', ...)."""
    fx = _f64(fx)
    attn_p = {k[len("Attn."):]: v for k, v in p.items() if k.startswith("Attn.")}
    h1 = layer_norm(fx, p["ln_1.weight"], p["ln_1.bias"])
    fx = layer_forward(attn_p, h1, heads, dim_head, variant, spatial_shape)["y"] + fx
    h2 = layer_norm(fx, p["ln_mlp1.0.weight"], p["ln_mlp1.0.bias"])
    fx = mlp(p, "ln_mlp1.1.", h2) + fx
    if last_layer:
        h3 = layer_norm(fx, p["ln_mlp2.0.weight"], p["ln_mlp2.0.bias"])
        return np.einsum("bnc,oc->bno", h3, _f64(p["ln_mlp2.1.weight"])) + _f64(p["ln_mlp2.1.bias"])
    return fx
