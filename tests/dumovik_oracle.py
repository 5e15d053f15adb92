"""A plain float64 model of the Dumovik design: one function per mechanism,
whole sequences at once, no cache, no batching. It shares no code with the
package; the tests compare the engine against it.

A configuration is the dict a checkpoint's config.json holds; `t` maps
tensor names to tensors.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def rotate_half(v, positions, dims, base):
    """v [T, ..., n]: entry i of the first `dims` is paired with i + dims/2."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)],
                     dtype=F64)
    ang = positions.to(F64)[:, None] * f[None, :]            # [T, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    co, si = ang.cos().view(shape), ang.sin().view(shape)
    a, b = v[..., :half], v[..., half:dims]
    out = v.clone()
    out[..., :half] = a * co - b * si
    out[..., half:dims] = b * co + a * si
    return out


def softmax_rows(score, visible):
    score = score.masked_fill(~visible, float("-inf"))
    return torch.softmax(score, -1)


def chunked_attention(h, t, p, m, eps, shared=None):
    """-> (output [T, W], (k, v) as a sharing layer reads them)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ t[p + "q"].to(F64).T
    q = unit_rms(q, eps) * t[p + "q.norm"].to(F64)
    if shared is None:
        k = h @ t[p + "k"].to(F64).T
        k = unit_rms(k, eps) * t[p + "k.norm"].to(F64)
        v = h @ t[p + "v"].to(F64).T
    else:
        k, v = shared
    q = q.view(T, H, d)
    kk = k.view(T, G, d)
    vv = v.view(T, G, dv)
    i = torch.arange(T)
    vis = (i[None, :] <= i[:, None])
    size = (m.get("mask") or {}).get("size")
    if size:
        vis = vis & ((i[None, :] // size) == (i[:, None] // size))
    cap = m.get("softcap")
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ kk[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        out[:, hd] = softmax_rows(s, vis) @ vv[:, g]
    return out.reshape(T, H * dv) @ t[p + "o"].to(F64).T, (k, v)


def latent_attention(h, t, p, m, eps):
    T = h.shape[0]
    H, d, dr, dv, R = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                       m["kv_rank"])
    pos = torch.arange(T)
    q = (h @ t[p + "q"].to(F64).T).view(T, H, d + dr)
    kv = h @ t[p + "dkv"].to(F64).T
    c = unit_rms(kv[:, :R], eps) * t[p + "dkv.norm"].to(F64)
    k_rot = rotate_half(kv[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])
    q_rot = rotate_half(q[..., d:], pos, m["rot"]["dims"], m["rot"]["base"])
    k_n = (c @ t[p + "uk"].to(F64).T).view(T, H, d)
    v = (c @ t[p + "uv"].to(F64).T).view(T, H, dv)
    vis = pos[None, :] <= pos[:, None]
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :d] @ k_n[:, hd].T + q_rot[:, hd] @ k_rot.T) * m["scale"]
        out[:, hd] = softmax_rows(s, vis) @ v[:, hd]
    gate = torch.sigmoid(h @ t[p + "g"].to(F64).T)
    return (out.reshape(T, H * dv) * gate) @ t[p + "o"].to(F64).T


def lightning(h, t, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    silu = lambda z: z * torch.sigmoid(z)
    q = silu(h @ t[p + "q"].to(F64).T).view(T, H, d)
    k = silu(h @ t[p + "k"].to(F64).T).view(T, H, d)
    v = silu(h @ t[p + "v"].to(F64).T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(H, d, dv, dtype=F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        S = decay[:, None, None] * S + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hde,hd->he", S, q[i])
    o = unit_rms(out.reshape(T, H * dv), eps) * t[p + "norm"].to(F64)
    o = o * torch.sigmoid(h @ t[p + "g"].to(F64).T)
    return o @ t[p + "o"].to(F64).T


def dense_ff(h, t, p):
    g = gelu_tanh(h @ t[p + "gate"].to(F64).T)
    return (g * (h @ t[p + "up"].to(F64).T)) @ t[p + "down"].to(F64).T


def expert(h, t, p, limit):
    g = torch.clamp(h @ t[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ t[p + "up"].to(F64).T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[p + "down"].to(F64).T


def moe_ff(h, t, p, f):
    top = f["router"]["top"]
    z = h @ t[p + "router"].to(F64).T                        # [T, E]
    val, idx = z.topk(top, -1)
    w = torch.softmax(val, -1)
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for j in range(top):
            e = int(idx[r, j])
            out[r] += w[r, j] * expert(h[r:r + 1], t, p + f"e{e}.",
                                       f["expert"]["limit"])[0]
    return out


MIXERS = {"attention": chunked_attention, "latent_attention": latent_attention,
          "lightning": lightning}


def forward(config, t, tokens):
    """-> (logits [T, vocab], residual stream after every layer
    [layers, T, width]), float64."""
    eps = config["norm"]["eps"]
    x = t["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    kept = {}
    taps = []
    for i, L in enumerate(config["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        if L["type"] == "attention":
            src = m.get("kv_from")
            y, kept[i] = chunked_attention(
                x, t, p + "mix.", m, eps,
                shared=None if src is None else kept[src])
        elif L["type"] in MIXERS:
            y = MIXERS[L["type"]](x, t, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + layer_norm(y, t[p + "norm1"].to(F64), eps)
        f = L.get("mlp")
        if f:
            if f["kind"] == "dense":
                y = dense_ff(x, t, p + "mlp.")
            elif f["kind"] == "moe":
                y = moe_ff(x, t, p + "mlp.", f)
            else:
                raise ValueError(f["kind"])
            x = x + layer_norm(y, t[p + "norm2"].to(F64), eps)
        taps.append(x.clone())
    xn = layer_norm(x, t["final.norm"].to(F64), eps)
    return xn @ t["embed"].to(F64).T, torch.stack(taps)
