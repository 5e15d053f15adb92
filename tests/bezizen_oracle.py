"""A plain, slow float64 model of the Bezizen design: one function per
mechanism, whole sequences only (no cache, no state, no batching), written
from the equations and sharing no code with the package.

Notation: h [T, W] is a sublayer's input for positions 0 .. T-1 of one
sequence, `t` the dict of checkpoint tensors (float64), `p` a tensor-name
prefix, `m` the part of config.json that describes the mechanism.
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def lin(x, w):
    return x @ w.T


# ---- embedding, streams, output ---------------------------------------------
def embed(tokens, t, cfg):
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = t["embed"][ids] * float((cfg.get("embedding") or {}).get("scale", 1))
    if "pos" in t:
        x = x + t["pos"][: len(tokens)]
    return x


def streams_read(xs, coef):
    """u = sum_s coef[s] xs[s]."""
    return sum(coef[s] * xs[s] for s in range(len(xs)))


def streams_write(xs, y, mix, out):
    """new[j] = sum_s mix[s, j] xs[s] + out[j] y, all from the old xs."""
    n = len(xs)
    return [sum(mix[s, j] * xs[s] for s in range(n)) + out[j] * y
            for j in range(n)]


def logits(x, t, cfg):
    eps = float(cfg["norm"]["eps"])
    return lin(unit_rms(x, eps) * t["final.norm"], t["head"]) * \
        float(cfg.get("logit_scale", 1.0))


# ---- time mixing with a data-dependent decay and a bonus --------------------
def wkv_mixer(h, t, p, m, eps):
    T, W = h.shape
    H, D = int(m["heads"]), int(m["dim"])
    before = torch.cat([torch.zeros(1, W, dtype=F64), h[:-1]], 0)

    def shifted(n):
        return h + (before - h) * t[p + "mu." + n]

    r = lin(shifted("r"), t[p + "r"]).view(T, H, D)
    k = lin(shifted("k"), t[p + "k"]).view(T, H, D)
    v = lin(shifted("v"), t[p + "v"]).view(T, H, D)
    gate = silu(lin(shifted("g"), t[p + "g"]))
    z = lin(torch.tanh(lin(shifted("w"), t[p + "w1"])), t[p + "w2"]) + \
        t[p + "w0"]
    w = torch.exp(-torch.exp(z)).view(T, H, D)
    u = t[p + "u"].view(H, D)
    o = torch.zeros(T, H, D, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, D, dtype=F64)           # [key channel, value]
        for i in range(T):
            kv = torch.outer(k[i, hd], v[i, hd])
            o[i, hd] = (S + u[hd][:, None] * kv).T @ r[i, hd]
            S = w[i, hd][:, None] * S + kv
    o = unit_rms(o, eps).reshape(T, H * D) * t[p + "norm"] * gate
    return lin(o, t[p + "o"])


# ---- short causal convolution -----------------------------------------------
def short_conv(u, w):
    """y[i] = sum_j w[:, j] u[i - taps + 1 + j], zeros before row 0.
    u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), u], 0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        y = y + w[:, j] * pad[j: j + T]
    return y


# ---- windowed softmax attention whose values are its keys -------------------
def window_attention(h, t, p, m):
    T = h.shape[0]
    H, G = int(m["heads"]), int(m["kv_heads"])
    D = int(m["dim"])
    q = lin(h, t[p + "q"])
    k = lin(h, t[p + "k"])
    if m.get("conv"):
        q = short_conv(q, t[p + "q.conv"])
        k = short_conv(k, t[p + "k.conv"])
    q = q.view(T, H, D)
    k = k.view(T, G, D)
    if m.get("q_temp"):
        coef, every = float(m["q_temp"]["coef"]), int(m["q_temp"]["every"])
        temp = torch.tensor([1.0 + coef * math.log((i + 1) // every + 1)
                             for i in range(T)], dtype=F64)
        q = q * temp[:, None, None]
    size = int(m["mask"]["size"]) if m.get("mask") else 0
    o = torch.zeros(T, H, D, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        slope = 2.0 ** (-8.0 * (hd + 1) / H)
        for i in range(T):
            lo = max(0, i - size + 1) if size > 0 else 0
            js = torch.arange(lo, i + 1)
            sc = (k[lo: i + 1, g] @ q[i, hd]) * float(m["scale"]) - \
                slope * (i - js).to(F64)
            o[i, hd] = torch.softmax(sc, 0) @ k[lo: i + 1, g]
    o = o.reshape(T, H * D) * torch.sigmoid(lin(h, t[p + "g"]))
    return lin(o, t[p + "o"])


# ---- linear attention with a gate on every key channel ----------------------
def gated_linear_attention(h, t, p, m, eps):
    T = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (lin(h, t[p + "q"]) * D ** -0.5).view(T, H, D)
    k = lin(h, t[p + "k"]).view(T, H, D)
    v = lin(h, t[p + "v"]).view(T, H, V)
    z = lin(lin(h, t[p + "a1"]), t[p + "a2"]) + t[p + "a2.b"]
    a = (torch.sigmoid(z) ** (1.0 / float(m["tau"]))).view(T, H, D)
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for i in range(T):
            S = a[i, hd][:, None] * S + torch.outer(k[i, hd], v[i, hd])
            o[i, hd] = S.T @ q[i, hd]
    o = (unit_rms(o, eps) * t[p + "norm"]).reshape(T, H * V)
    return lin(o * silu(lin(h, t[p + "g"])), t[p + "o"])


def parallel_mixer(h, t, p, m, eps):
    left = window_attention(h, t, p + "left.", m["left"])
    right = gated_linear_attention(h, t, p + "right.", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ---- mixture of experts -----------------------------------------------------
def gated_ff(h, t, p):
    return lin(silu(lin(h, t[p + "gate"])) * lin(h, t[p + "up"]),
               t[p + "down"])


def route(h, t, p, r):
    """-> (chosen experts [T, top], their weights [T, top])."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(lin(h, t[p + "router"]), -1)
    allowed = s.clone()
    if r.get("groups"):
        n, keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
        best = s.view(-1, n, E // n).max(-1).values
        kept = torch.sort(best, dim=-1, descending=True, stable=True).indices
        mask = torch.zeros_like(best, dtype=torch.bool)
        mask.scatter_(1, kept[:, :keep], True)
        allowed = torch.where(mask.repeat_interleave(E // n, 1), s,
                              torch.full_like(s, -1.0))
    pick = torch.sort(allowed, dim=-1, descending=True,
                      stable=True).indices[:, :top]
    w = s.gather(1, pick)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))
    return pick, w


def moe(h, t, p, f):
    pick, w = route(h, t, p, f["router"])
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, we in zip(pick[i].tolist(), w[i]):
            out[i] += we * gated_ff(h[i: i + 1], t, p + f"e{e}.")[0]
    if f.get("shared"):
        out = out + gated_ff(h, t, p + "shared.")
    return out


# ---- the whole model --------------------------------------------------------
def forward(tokens, tensors, cfg, taps=None):
    """-> logits [T, vocab]; `taps`, if a list, receives the stream (summed
    over its copies) after every layer."""
    t = {k: v.to(F64) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    n = int(cfg.get("streams") or 0)
    x0 = embed(tokens, t, cfg)
    xs = [x0.clone() for _ in range(max(n, 1))]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        subs = [("norm1", "hc1.", lambda a: (
            wkv_mixer(a, t, p + "mix.", L["mixer"], eps)
            if L["type"] == "wkv" else
            parallel_mixer(a, t, p + "mix.", L["mixer"], eps)))]
        if L.get("mlp"):
            subs.append(("norm2", "hc2.",
                         lambda a: moe(a, t, p + "mlp.", L["mlp"])))
        for norm, hc, fn in subs:
            if n:
                u = streams_read(xs, t[p + hc + "in"])
            else:
                u = xs[0]
            y = fn(unit_rms(u, eps) * t[p + norm])
            if n:
                xs = streams_write(xs, y, t[p + hc + "mix"], t[p + hc + "out"])
            else:
                xs = [xs[0] + y]
        if taps is not None:
            taps.append(sum(xs))
    return logits(sum(xs), t, cfg)
