"""Sequence mixers that carry their own kind of memory: a selective
state-space mixer (fixed-size recurrent state per sequence), a latent
attention mixer (one low-rank row per token in the paged cache), a
grouped-query attention mixer with chunk-local keys and capped scores, and a
linear-attention mixer with a fixed decay per head (a state matrix per
sequence). All take the layer input [T, W] of a packed batch plus the
engine's row maps and return the mixer output [T, W]; all sizes and constants
are arguments, so any model family can stack them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn as nn

from kukeon_amd import ops
from kukeon_amd.engine.kv_cache import LayerKVSpec


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


def pad_rank(w1: torch.Tensor, w2: torch.Tensor, multiple: int = 16):
    """A low-rank pair w2 f(w1 x) with f(0) = 0, its inner size brought up
    to a multiple of `multiple` with zero rows of w1 and zero columns of w2:
    the same function, and the first product is never narrower than the
    matrix cores' tiles."""
    n = -w1.shape[0] % multiple
    if n:
        w1 = torch.cat([w1, torch.zeros(n, w1.shape[1], dtype=w1.dtype,
                                        device=w1.device)], 0)
        w2 = torch.cat([w2, torch.zeros(w2.shape[0], n, dtype=w2.dtype,
                                        device=w2.device)], 1)
    return w1.contiguous(), w2.contiguous()


def fuse_rows(segs, width: int, dtype, device):
    """Stack projection weights [rows_i, width] into one matrix whose
    segments each start on a multiple of 8 output columns.
    -> ({name: first column}, parameter)."""
    col, rows, at = {}, [], 0
    for name, wt in segs:
        col[name] = at
        n = wt.shape[0]
        rows.append(wt.to(device=device, dtype=dtype))
        pad = _pad8(n) - n
        if pad:
            rows.append(torch.zeros(pad, width, dtype=dtype, device=device))
        at += _pad8(n)
    return col, nn.Parameter(torch.cat(rows, 0).contiguous(),
                             requires_grad=False)


# ---------------------------------------------------------------------------
@dataclass
class StateSpaceCfg:
    heads: int
    vdim: int                # channels per head
    state: int               # rows of a head's state matrix
    groups: int              # B/C groups; head h reads group h // (heads/groups)
    conv: int                # taps of the short convolution
    norm_groups: int         # parts of the gated output normed separately

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


class StateSpaceMixer(nn.Module):
    """Selective state-space mixer (the recurrent form of state-space
    duality). The input projection yields [z | x | B | C | dt]; x, B and C
    pass a short causal convolution and silu; per head
    S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x with
    dt = softplus(dt + dt_bias); y is gated by silu(z), normed in
    `norm_groups` parts and projected out. The state matrix and the last
    taps-1 convolution inputs live in the engine's state slots (fp32).

    Tensors (prefix p): in [2*inner + 2*G*N + H, W], conv [C, taps],
    conv.b [C], dt_bias, A_log, D [H], norm [inner], o [W, inner]."""

    def __init__(self, m: StateSpaceCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        if m.heads % m.groups:
            raise ValueError(f"{p}: heads not a multiple of groups")
        if m.inner % m.norm_groups:
            raise ValueError(f"{p}: inner size not divisible by norm_groups")
        self.m = m
        self.eps = eps
        C = m.conv_channels
        w_in = t[p + "in"]
        if w_in.shape[0] != 2 * m.inner + 2 * m.groups * m.state + m.heads:
            raise ValueError(f"{p}in: rows do not fit the mixer's sizes")
        self.w_in = nn.Parameter(w_in.to(device=device, dtype=dtype)
                                 .contiguous(), requires_grad=False)
        cw = t[p + "conv"]
        if tuple(cw.shape) != (C, m.conv):
            raise ValueError(f"{p}conv: shape {tuple(cw.shape)}")
        f32 = dict(device=device, dtype=torch.float32)
        self.conv_w = cw.to(**f32).t().contiguous()          # [taps, C]
        self.conv_b = t[p + "conv.b"].to(**f32).contiguous()
        self.zero_b = torch.zeros(C, **f32)
        self.dt_bias = t[p + "dt_bias"].to(**f32).contiguous()
        self.rate = torch.exp(t[p + "A_log"].to(**f32)).contiguous()
        self.skip = t[p + "D"].to(**f32).contiguous()
        self.norm_w = t[p + "norm"].to(**f32).contiguous()
        self.w_o = nn.Parameter(t[p + "o"].to(device=device, dtype=dtype)
                                .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(m: StateSpaceCfg, width: int) -> Dict[str, tuple]:
        C = m.conv_channels
        return {"in": (2 * m.inner + 2 * m.groups * m.state + m.heads, width),
                "conv": (C, m.conv), "conv.b": (C,), "dt_bias": (m.heads,),
                "A_log": (m.heads,), "D": (m.heads,), "norm": (m.inner,),
                "o": (width, m.inner)}

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return None

    def state_shape(self):
        m = self.m
        return [(m.conv - 1, m.conv_channels), (m.heads, m.vdim, m.state)]

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        m = self.m
        T = h.shape[0]
        conv_state, ssm_state = state
        proj = ops.linear(h, self.w_in)
        inner, C = m.inner, m.conv_channels
        xbc = torch.empty(T, C, dtype=h.dtype, device=h.device)
        # a step of single tokens shifts the slots in the same launch
        one = meta.max_rows == 1 and T == meta.cu_rows.numel() - 1
        ops.conv_act(xbc, proj, inner, self.conv_w, self.conv_b, conv_state,
                     meta.positions, meta.row_seq, meta.cu_rows,
                     meta.state_slots, 1, one)
        if not one:
            ops.conv_tail_update(conv_state, proj, inner, self.zero_b,
                                 meta.positions, meta.cu_rows,
                                 meta.state_slots)
        y = torch.empty(T, inner, dtype=torch.float32, device=h.device)
        ops.ssm_scan(y, xbc, proj[:, inner + C:inner + C + m.heads],
                     self.dt_bias, self.rate, self.skip, ssm_state,
                     meta.positions, meta.cu_rows, meta.state_slots,
                     m.heads, m.vdim, m.state, m.groups)
        g = torch.empty(T, inner, dtype=h.dtype, device=h.device)
        ops.gated_group_rmsnorm(g, y, proj[:, :inner], self.norm_w,
                                m.norm_groups, self.eps)
        return ops.linear(g, self.w_o)


# ---------------------------------------------------------------------------
@dataclass
class LatentAttnCfg:
    heads: int
    dim: int                 # unrotated query/key entries per head
    rot_dim: int             # rotated entries per head (one shared key part)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int              # position i sees i-window+1 .. i (0: all)
    rot_dims: int            # leading entries of the rotated part that turn
    rot_base: float
    # "pairs": entries (2i, 2i+1) turn together; "half": entry i turns with
    # entry i + rot_dims/2
    rot_layout: str = "pairs"
    # "head": one gate per head (g [H, W]); "element": one per output entry
    # (g [H*vdim, W])
    gate: str = "head"


def _pairs_from_half(dims: int, n: int) -> torch.Tensor:
    """Row order that turns the half layout of a rotated part of n entries
    into the pair layout: new[2i] = old[i], new[2i+1] = old[i + dims/2]."""
    half = dims // 2
    order = []
    for i in range(half):
        order += [i, i + half]
    return torch.tensor(order + list(range(dims, n)), dtype=torch.long)


class LatentAttention(nn.Module):
    """Attention over a low-rank latent. Per token the cache holds ONE row
    [c | k_rot]: the normed latent c (kv_rank) from which every head's
    unrotated keys (W_uk c) and values (W_uv c) derive, and one rotated key
    part shared by all heads. The products with W_uk and W_uv are moved to
    the query and the output side,

        score_h(i, j) = ((W_uk_h^T q_h)(i) . c(j) + rot(q_rot_h)(i) . k_rot(j)) scale
        out_h(i)      = W_uv_h  sum_j softmax_j(score_h)(i, j) c(j)

    so the kernel reads each cache row once for all heads. Queries pass
    their own normed latent (q_rank), or come straight from the input when
    q_rank is 0. A sliding window may bound the keys, and the output is
    scaled by sigmoid of a gate projected from the mixer's input, per head
    or per entry.

    The kernels turn pairs (2i, 2i+1). A checkpoint in the half layout
    (entry i with i + rot_dims/2) has the rows of the rotated parts of its
    query and key projections reordered at load; a score is a dot product
    over those rows, so only its order of summation changes.

    Tensors (prefix p): dq [q_rank, W], dq.norm, uq [H*(dim+rot_dim), q_rank]
    (or q [H*(dim+rot_dim), W] when q_rank is 0), dkv [kv_rank+rot_dim, W],
    dkv.norm, uk [H*dim, kv_rank], uv [H*vdim, kv_rank], g [H or H*vdim, W],
    o [W, H*vdim]."""

    def __init__(self, m: LatentAttnCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        if m.rot_dims % 2 or m.rot_dims > m.rot_dim:
            raise ValueError(f"{p}: bad rotary dims")
        if m.rot_layout not in ("pairs", "half"):
            raise ValueError(f"{p}: unknown rotary layout {m.rot_layout!r}")
        if m.gate not in ("head", "element"):
            raise ValueError(f"{p}: unknown gate kind {m.gate!r}")
        self.m = m
        self.eps = eps
        H, R = m.heads, m.kv_rank
        hd = m.dim + m.rot_dim
        w_q = t[p + ("uq" if m.q_rank else "q")]
        w_dkv = t[p + "dkv"]
        if m.rot_layout == "half":
            order = _pairs_from_half(m.rot_dims, m.rot_dim)
            w_q = w_q.view(H, hd, -1)
            w_q = torch.cat([w_q[:, :m.dim], w_q[:, m.dim:][:, order]],
                            1).reshape(H * hd, -1)
            w_dkv = torch.cat([w_dkv[:R], w_dkv[R:][order]], 0)
        first = ("q", t[p + "dq"] if m.q_rank else w_q)
        self.col, self.w_down = fuse_rows(
            [first, ("kv", w_dkv), ("g", t[p + "g"])], width, dtype, device)
        f32 = dict(device=device, dtype=torch.float32)
        self.q_norm = (t[p + "dq.norm"].to(**f32).contiguous() if m.q_rank
                       else torch.empty(0, **f32))
        self.kv_norm = t[p + "dkv.norm"].to(**f32).contiguous()
        dev = dict(device=device, dtype=dtype)
        self.w_uq = None
        if m.q_rank:
            self.w_uq = nn.Parameter(w_q.to(**dev).contiguous(),
                                     requires_grad=False)
        self.gate_cols = H if m.gate == "head" else H * m.vdim
        # [H, dim, R]: q_abs_h = q_h W_uk_h;  [H, R, vdim]: o_h = l_h W_uv_h^T
        self.w_uk = nn.Parameter(t[p + "uk"].to(**dev).view(H, m.dim, R)
                                 .contiguous(), requires_grad=False)
        self.w_uv = nn.Parameter(t[p + "uv"].to(**dev).view(H, m.vdim, R)
                                 .transpose(1, 2).contiguous(),
                                 requires_grad=False)
        self.w_o = nn.Parameter(t[p + "o"].to(**dev).contiguous(),
                                requires_grad=False)
        self.cs = None       # angle table [positions, rot_dims], set by the model

    @staticmethod
    def tensor_shapes(m: LatentAttnCfg, width: int) -> Dict[str, tuple]:
        H = m.heads
        out = {"dkv": (m.kv_rank + m.rot_dim, width),
               "dkv.norm": (m.kv_rank,), "uk": (H * m.dim, m.kv_rank),
               "uv": (H * m.vdim, m.kv_rank),
               "g": (H if m.gate == "head" else H * m.vdim, width),
               "o": (width, H * m.vdim)}
        if m.q_rank:
            out.update({"dq": (m.q_rank, width), "dq.norm": (m.q_rank,),
                        "uq": (H * (m.dim + m.rot_dim), m.q_rank)})
        else:
            out["q"] = (H * (m.dim + m.rot_dim), width)
        return out

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return LayerKVSpec(1, self.m.kv_rank + self.m.rot_dim, 0)

    def state_shape(self):
        return None

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        m = self.m
        T = h.shape[0]
        H, R = m.heads, m.kv_rank
        hd = m.dim + m.rot_dim
        proj = ops.linear(h, self.w_down)
        cq = torch.empty(T, m.q_rank, dtype=h.dtype, device=h.device)
        ops.latent_kv_append(cq, cache, proj, self.col["q"], self.col["kv"],
                             self.q_norm, self.kv_norm, self.eps, self.cs,
                             meta.positions, meta.row_seq, meta.block_table)
        if m.q_rank:
            q = ops.linear(cq, self.w_uq)              # [T, H*(dim+rot)]
        else:
            q = proj[:, self.col["q"]: self.col["q"] + H * hd]
        q_n = q.unflatten(1, (H, hd))[:, :, :m.dim].transpose(0, 1)
        q_abs = torch.bmm(q_n, self.w_uk)              # [H, T, R]
        lat = torch.empty(H, T, R, dtype=h.dtype, device=h.device)
        ops.latent_attention(lat, q_abs, q, cache, self.cs, meta.positions,
                             meta.row_seq, meta.block_table, H, m.dim,
                             m.rot_dim, m.window, m.scale)
        o = torch.bmm(lat, self.w_uv)                  # [H, T, vdim]
        og = torch.empty(T, H * m.vdim, dtype=h.dtype, device=h.device)
        ops.head_gate(og, o, proj[:, self.col["g"]:
                                  self.col["g"] + self.gate_cols])
        return ops.linear(og, self.w_o)


# ---------------------------------------------------------------------------
@dataclass
class ChunkAttnCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0     # scores become cap tanh(score / cap) (0: off)
    chunk: int = 0           # keys of the query's own chunk only (0: all)
    kv_from: Optional[int] = None    # read this earlier layer's pages


class ChunkedAttention(nn.Module):
    """Grouped-query softmax attention without positions in the scores.
    Queries and keys are RMS-normed over their WHOLE projection (all heads
    at once, one weight entry per row of the projection) before they are cut
    into heads; scores are scaled, optionally capped with tanh, and position
    i sees j <= i of its own chunk, floor(i / chunk) == floor(j / chunk).
    A mixer with `kv_from` projects no keys or values and reads the pages
    of that earlier layer with its own queries.

    Tensors (prefix p): q [H*dim, W], q.norm [H*dim], o [W, H*vdim] and, for
    a layer with pages of its own, k [G*dim, W], k.norm [G*dim],
    v [G*vdim, W]."""

    def __init__(self, m: ChunkAttnCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        if m.heads % m.kv_heads:
            raise ValueError(f"{p}: heads not a multiple of kv_heads")
        self.m = m
        self.eps = eps
        self.owns_kv = m.kv_from is None
        segs = [("q", t[p + "q"])]
        if self.owns_kv:
            segs += [("k", t[p + "k"]), ("v", t[p + "v"])]
        self.col, self.w_in = fuse_rows(segs, width, dtype, device)
        f32 = dict(device=device, dtype=torch.float32)
        self.q_norm = t[p + "q.norm"].to(**f32).contiguous()
        self.k_norm = (t[p + "k.norm"].to(**f32).contiguous()
                       if self.owns_kv else None)
        self.w_o = nn.Parameter(t[p + "o"].to(device=device, dtype=dtype)
                                .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(m: ChunkAttnCfg, width: int) -> Dict[str, tuple]:
        out = {"q": (m.heads * m.dim, width), "q.norm": (m.heads * m.dim,),
               "o": (width, m.heads * m.vdim)}
        if m.kv_from is None:
            out.update({"k": (m.kv_heads * m.dim, width),
                        "k.norm": (m.kv_heads * m.dim,),
                        "v": (m.kv_heads * m.vdim, width)})
        return out

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return LayerKVSpec(self.m.kv_heads, self.m.dim, self.m.vdim,
                           share_from=self.m.kv_from)

    def state_shape(self):
        return None

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        m = self.m
        T = h.shape[0]
        proj = ops.linear(h, self.w_in)
        q = torch.empty(T, m.heads * m.dim, dtype=h.dtype, device=h.device)
        c = self.col
        ops.qk_norm_append(q, cache if self.owns_kv else None,
                           cache_v if self.owns_kv else None, proj, c["q"],
                           c.get("k", 0), c.get("v", 0), self.q_norm,
                           self.k_norm, self.eps, meta.positions,
                           meta.row_seq, meta.block_table)
        o = torch.empty(T, m.heads * m.vdim, dtype=h.dtype, device=h.device)
        if (meta.mode == "prefill" and meta.max_rows >= 16 and
                meta.qb_seq is not None and
                ops.chunk_tiles_supported(q, m.dim, m.vdim, cache.shape[2])):
            # prompt portions on the matrix cores
            ops.chunk_attention_tiles(o, q, cache, cache_v, meta.block_table,
                                      meta.seq_lens, meta.q_starts,
                                      meta.qb_seq, meta.qb_start, m.scale,
                                      m.softcap, m.chunk)
        else:
            ops.chunk_attention(o, q, cache, cache_v, meta.positions,
                                meta.row_seq, meta.block_table, m.heads,
                                m.scale, m.softcap, m.chunk)
        return ops.linear(o, self.w_o)


# ---------------------------------------------------------------------------
@dataclass
class LightningCfg:
    heads: int
    dim: int
    vdim: int
    decay: tuple             # one factor per head


class LightningMixer(nn.Module):
    """Linear attention with a fixed decay per head. q, k and v are silu of
    their projections, head by head; per head the state matrix follows
    S_t = decay_h S_(t-1) + k_t v_t^T and the output is S_t^T q_t, with no
    other scale. The heads' outputs are RMS-normed together, multiplied by
    sigmoid of a gate projected from the mixer's input, and projected out.
    The state (fp32, stored transposed as [H, vdim, dim]) lives in the
    engine's state slots.

    Tensors (prefix p): q, k [H*dim, W], v, g [H*vdim, W], norm [H*vdim],
    o [W, H*vdim]."""

    def __init__(self, m: LightningCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        if len(m.decay) != m.heads:
            raise ValueError(f"{p}: one decay per head is needed")
        self.m = m
        self.eps = eps
        self.col, self.w_in = fuse_rows(
            [("q", t[p + "q"]), ("k", t[p + "k"]), ("v", t[p + "v"]),
             ("g", t[p + "g"])], width, dtype, device)
        f32 = dict(device=device, dtype=torch.float32)
        self.decay = torch.tensor([float(d) for d in m.decay],
                                  dtype=torch.float64).to(**f32).contiguous()
        self.norm_w = t[p + "norm"].to(**f32).contiguous()
        self.w_o = nn.Parameter(t[p + "o"].to(device=device, dtype=dtype)
                                .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(m: LightningCfg, width: int) -> Dict[str, tuple]:
        H = m.heads
        return {"q": (H * m.dim, width), "k": (H * m.dim, width),
                "v": (H * m.vdim, width), "g": (H * m.vdim, width),
                "norm": (H * m.vdim,), "o": (width, H * m.vdim)}

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return None

    def state_shape(self):
        # the slot holds S^T: a column of S is one contiguous run
        return (self.m.heads, self.m.vdim, self.m.dim)

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        m = self.m
        T = h.shape[0]
        inner = m.heads * m.vdim
        proj = ops.linear(h, self.w_in)
        c = self.col
        y = torch.empty(T, inner, dtype=torch.float32, device=h.device)
        ops.lightning_scan(y, proj, c["q"], c["k"], c["v"], self.decay, state,
                           meta.positions, meta.cu_rows, meta.state_slots,
                           m.heads, m.dim, m.vdim)
        g = torch.empty(T, inner, dtype=h.dtype, device=h.device)
        ops.gated_rmsnorm(g, y, proj[:, c["g"]: c["g"] + inner], self.norm_w,
                          self.eps)
        return ops.linear(g, self.w_o)


# ---------------------------------------------------------------------------
@dataclass
class WkvCfg:
    heads: int
    dim: int                 # key channels = value channels per head


class WkvMixer(nn.Module):
    """Time mixing with a data-dependent decay per key channel and a bonus
    for the current token. Each of r, k, v, g, w reads its own blend of the
    input h and the previous token's input h', h + (h' - h) mu; r, k, v are
    projections of their blends, the output gate is silu of g's projection,
    and the decay is exp(-exp(W2 tanh(W1 blend_w) + w0)). Per head, with the
    state S [key channel, value channel]:

        o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t
        S_t = diag(decay_t) S_(t-1) + k_t v_t^T

    Each head's o is divided by its root mean square, then weight, gate and
    output projection. Carried per sequence (fp32 state slots): h' and S^T.

    Tensors (prefix p): mu.{r,k,v,g,w} [W], r, k, v, g [H*dim, W],
    w1 [rank, W], w2 [H*dim, rank], w0 [H*dim], u [H, dim], norm [H*dim],
    o [W, H*dim]."""

    BLENDS = ("r", "k", "v", "g", "w")

    def __init__(self, m: WkvCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        self.m = m
        self.eps = eps
        f32 = dict(device=device, dtype=torch.float32)
        dev = dict(device=device, dtype=dtype)
        self.mu = torch.stack([t[p + "mu." + n] for n in self.BLENDS]).to(
            **f32).contiguous()
        # r, k, v, g have one shape: their matrices are kept stacked
        self.w_rkvg = nn.Parameter(torch.stack(
            [t[p + n] for n in ("r", "k", "v", "g")]).to(**dev).contiguous(),
            requires_grad=False)
        # the second, tiny product of the decay runs inside the scan (fp32)
        w1, self.w2 = pad_rank(t[p + "w1"].to(**dev), t[p + "w2"].to(**f32))
        self.w1 = nn.Parameter(w1, requires_grad=False)
        self.w0 = t[p + "w0"].to(**f32).contiguous()
        self.bonus = t[p + "u"].to(**f32).reshape(-1).contiguous()
        self.norm_w = t[p + "norm"].to(**f32).contiguous()
        self.w_o = nn.Parameter(t[p + "o"].to(**dev).contiguous(),
                                requires_grad=False)

    @staticmethod
    def tensor_shapes(m: WkvCfg, width: int, rank: int = 16):
        C = m.heads * m.dim
        out = {"mu." + n: (width,) for n in WkvMixer.BLENDS}
        out.update({n: (C, width) for n in ("r", "k", "v", "g")})
        out.update({"w1": (rank, width), "w2": (C, rank), "w0": (C,),
                    "u": (m.heads, m.dim), "norm": (C,), "o": (width, C)})
        return out

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return None

    def state_shape(self):
        m = self.m
        return [(self.mu.shape[1],), (m.heads, m.dim, m.dim)]

    @property
    def out_width(self) -> int:
        return self.m.heads * self.m.dim

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        g = torch.empty(h.shape[0], self.out_width, dtype=h.dtype,
                        device=h.device)
        self.pre_output(h, cache, state, meta, cache_v, g, 1.0)
        return ops.linear(g, self.w_o)

    def pre_output(self, h, cache, state, meta, cache_v, out,
                   scale: float) -> None:
        """The input of the output projection, times `scale`, into `out`."""
        m = self.m
        T, W = h.shape
        C = m.heads * m.dim
        prev, S = state
        one = meta.max_rows == 1 and T == meta.cu_rows.numel() - 1
        blends = torch.empty(5, T, W, dtype=h.dtype, device=h.device)
        ops.token_shift(blends, h, self.mu, prev, meta.positions,
                        meta.row_seq, meta.cu_rows, meta.state_slots, one)
        if not one:
            ops.token_shift_tail(prev, h, meta.positions, meta.cu_rows,
                                 meta.state_slots)
        # four plain products into one buffer (each blend has its own matrix)
        rkvg = torch.empty(4, T, C, dtype=h.dtype, device=h.device)
        for i in range(4):
            torch.mm(blends[i], self.w_rkvg[i].t(), out=rkvg[i])
        lo = ops.linear_f32(blends[4], self.w1)                    # [T, R]
        y = torch.empty(T, C, dtype=torch.float32, device=h.device)
        ops.decay_scan(y, rkvg[0], rkvg[1], rkvg[2], lo, self.w2, self.w0,
                       self.bonus, S, meta.positions, meta.cu_rows,
                       meta.state_slots, m.heads, m.dim, m.dim, 0)
        ops.head_rmsnorm_gate(out, y, rkvg[3], self.norm_w, m.heads,
                              self.eps, 0, scale)


# ---------------------------------------------------------------------------
@dataclass
class WindowAttnCfg:
    heads: int
    kv_heads: int
    dim: int                 # query/key entries per head; values = keys
    scale: float
    window: int = 0          # position i sees i-window+1 .. i (0: all)
    conv: int = 0            # taps of the convolution on q and k (0: none)
    temp_coef: float = 0.0   # queries times 1 + coef ln(floor((p+1)/every)+1)
    temp_every: int = 0      # (0: no temperature)
    bias: bool = True        # slope_h (i - j) off the scores


def distance_slopes(heads: int) -> torch.Tensor:
    """slope_h = 2^(-8 (h + 1) / heads)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads)
                         for h in range(heads)], dtype=torch.float64)


class WindowAttention(nn.Module):
    """Grouped-query softmax attention over a sliding window whose values
    are its keys (one cache row per token and kv head). q and k pass a short
    causal convolution per channel straight after their projections; there
    is no rotation: positions enter through a query temperature that grows
    with the logarithm of the position, and through a bias slope_h (i - j)
    taken off the scaled scores. The concatenated heads are multiplied by
    sigmoid of a gate projected from the mixer's input, then projected out.
    Carried per sequence: the last taps-1 projected q and k rows (fp32).

    Tensors (prefix p): q [H*dim, W], k [G*dim, W], q.conv [H*dim, taps],
    k.conv [G*dim, taps], g [H*dim, W], o [W, H*dim]."""

    def __init__(self, m: WindowAttnCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        if m.heads % m.kv_heads:
            raise ValueError(f"{p}: heads not a multiple of kv_heads")
        self.m = m
        self.Cq, self.Ck = m.heads * m.dim, m.kv_heads * m.dim
        self.col, self.w_in = fuse_rows(
            [("q", t[p + "q"]), ("k", t[p + "k"]), ("g", t[p + "g"])], width,
            dtype, device)
        f32 = dict(device=device, dtype=torch.float32)
        taps = max(1, m.conv)
        if m.conv:
            cw = torch.cat([t[p + "q.conv"], t[p + "k.conv"]], 0)
            if tuple(cw.shape) != (self.Cq + self.Ck, taps):
                raise ValueError(f"{p}: convolution shape {tuple(cw.shape)}")
            self.conv_w = cw.to(**f32).t().contiguous()       # [taps, C]
        else:
            self.conv_w = torch.ones(1, self.Cq + self.Ck, **f32)
        self.taps = taps
        self.zero_b = torch.zeros(self.Cq + self.Ck, **f32)
        self.slopes = (distance_slopes(m.heads).to(**f32).contiguous()
                       if m.bias else None)
        self.w_o = nn.Parameter(t[p + "o"].to(device=device, dtype=dtype)
                                .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(m: WindowAttnCfg, width: int) -> Dict[str, tuple]:
        Cq, Ck = m.heads * m.dim, m.kv_heads * m.dim
        out = {"q": (Cq, width), "k": (Ck, width), "g": (Cq, width),
               "o": (width, Cq)}
        if m.conv:
            out.update({"q.conv": (Cq, m.conv), "k.conv": (Ck, m.conv)})
        return out

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return LayerKVSpec(self.m.kv_heads, self.m.dim, 0)

    def state_shape(self):
        return (self.taps - 1, self.Cq + self.Ck)

    @property
    def out_width(self) -> int:
        return self.Cq

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        og = torch.empty(h.shape[0], self.Cq, dtype=h.dtype, device=h.device)
        self.pre_output(h, cache, state, meta, cache_v, og, 1.0)
        return ops.linear(og, self.w_o)

    def pre_output(self, h, cache, state, meta, cache_v, out,
                   scale: float) -> None:
        m = self.m
        T = h.shape[0]
        c = self.col
        proj = ops.linear(h, self.w_in)
        q = torch.empty(T, self.Cq, dtype=h.dtype, device=h.device)
        one = meta.max_rows == 1 and T == meta.cu_rows.numel() - 1
        ops.conv_scale_append(q, cache, proj, c["q"], c["k"], self.conv_w,
                              state, m.temp_coef, m.temp_every,
                              meta.positions, meta.row_seq, meta.cu_rows,
                              meta.state_slots, meta.block_table, one)
        if not one and self.taps > 1:
            ops.conv_pair_tail_update(state, proj, c["q"], c["k"], self.Cq,
                                      self.Ck, self.zero_b, meta.positions,
                                      meta.cu_rows, meta.state_slots)
        o = torch.empty(T, self.Cq, dtype=h.dtype, device=h.device)
        if (meta.mode == "prefill" and meta.max_rows >= 16 and
                meta.qb_seq is not None and
                ops.window_tiles_supported(q, m.dim, cache.shape[2])):
            # prompt portions on the matrix cores
            ops.window_attention_tiles(o, q, cache, self.slopes,
                                       meta.block_table, meta.seq_lens,
                                       meta.q_starts, meta.qb_seq,
                                       meta.qb_start, m.scale, m.window)
        else:
            ops.window_attention(o, q, cache, None, self.slopes,
                                 meta.positions, meta.row_seq,
                                 meta.block_table, m.heads, m.scale, m.window)
        ops.scaled_gate(out, o, proj[:, c["g"]: c["g"] + self.Cq], 1, scale)


# ---------------------------------------------------------------------------
@dataclass
class GatedLinearCfg:
    heads: int
    dim: int
    vdim: int
    tau: float               # decay = sigmoid(z)^(1/tau)


class GatedLinearAttention(nn.Module):
    """Linear attention with a learned decay per key channel:
    q = W_q h dim^(-1/2), k = W_k h, v = W_v h,
    decay_t = sigmoid(W_a2 (W_a1 h) + b)^(1/tau), and per head

        S_t = diag(decay_t) S_(t-1) + k_t v_t^T ,  o_t = S_t^T q_t .

    Each head's o is RMS-normed over its value entries with one weight
    vector shared by the heads, the concatenation is multiplied by
    silu(W_g h) and projected out. Carried per sequence: S^T (fp32).

    Tensors (prefix p): q, k [H*dim, W], v, g [H*vdim, W], a1 [rank, W],
    a2 [H*dim, rank], a2.b [H*dim], norm [vdim], o [W, H*vdim]."""

    def __init__(self, m: GatedLinearCfg, width: int, eps: float,
                 t: Dict[str, torch.Tensor], p: str, device, dtype):
        super().__init__()
        self.m = m
        self.eps = eps
        self.col, self.w_in = fuse_rows(
            [("q", t[p + "q"]), ("k", t[p + "k"]), ("v", t[p + "v"]),
             ("g", t[p + "g"])], width, dtype, device)
        f32 = dict(device=device, dtype=torch.float32)
        # the decay's low-rank pair: the first product keeps its fp32 sums,
        # the second, tiny one runs inside the scan
        w1, self.w_a2 = pad_rank(t[p + "a1"].to(device=device, dtype=dtype),
                                 t[p + "a2"].to(**f32))
        self.w_a1 = nn.Parameter(w1, requires_grad=False)
        self.a_bias = t[p + "a2.b"].to(**f32).contiguous()
        self.norm_w = t[p + "norm"].to(**f32).repeat(m.heads).contiguous()
        self.w_o = nn.Parameter(t[p + "o"].to(device=device, dtype=dtype)
                                .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(m: GatedLinearCfg, width: int, rank: int = 16):
        H = m.heads
        return {"q": (H * m.dim, width), "k": (H * m.dim, width),
                "v": (H * m.vdim, width), "g": (H * m.vdim, width),
                "a1": (rank, width), "a2": (H * m.dim, rank),
                "a2.b": (H * m.dim,), "norm": (m.vdim,),
                "o": (width, H * m.vdim)}

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return None

    def state_shape(self):
        return (self.m.heads, self.m.vdim, self.m.dim)

    @property
    def out_width(self) -> int:
        return self.m.heads * self.m.vdim

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        g = torch.empty(h.shape[0], self.out_width, dtype=h.dtype,
                        device=h.device)
        self.pre_output(h, cache, state, meta, cache_v, g, 1.0)
        return ops.linear(g, self.w_o)

    def pre_output(self, h, cache, state, meta, cache_v, out,
                   scale: float) -> None:
        m = self.m
        T = h.shape[0]
        c = self.col
        Cq, Cv = m.heads * m.dim, m.heads * m.vdim
        proj = ops.linear(h, self.w_in)
        lo = ops.linear_f32(h, self.w_a1)                          # [T, R]
        y = torch.empty(T, Cv, dtype=torch.float32, device=h.device)
        ops.decay_scan(y, proj[:, c["q"]: c["q"] + Cq],
                       proj[:, c["k"]: c["k"] + Cq],
                       proj[:, c["v"]: c["v"] + Cv], lo, self.w_a2,
                       self.a_bias, None, state, meta.positions, meta.cu_rows, meta.state_slots,
                       m.heads, m.dim, m.vdim, 1, m.tau, m.dim ** -0.5)
        ops.head_rmsnorm_gate(out, y, proj[:, c["g"]: c["g"] + Cv],
                              self.norm_w, m.heads, self.eps, 0, scale)


# ---------------------------------------------------------------------------
class ParallelMixer(nn.Module):
    """Two mixers side by side on the same input; the result is
    left_scale * left + right_scale * right. Each side writes the input of
    its output projection, already times its scale (applied in fp32 before
    the value is rounded), into its half of one buffer, and ONE GEMM over
    [left | right] with the two projections' columns side by side makes the
    sum. At most one side keeps pages; the layer's state is the list of
    both sides' pieces."""

    def __init__(self, left: nn.Module, right: nn.Module, left_scale: float,
                 right_scale: float):
        super().__init__()
        if left.kv_spec() is not None and right.kv_spec() is not None:
            raise ValueError("only one side of a parallel mixer may keep "
                             "pages")
        self.left, self.right = left, right
        self.left_scale, self.right_scale = left_scale, right_scale
        # the right half starts on a multiple of 8 columns
        self.split = _pad8(left.out_width)
        wl, wr = left.w_o.data, right.w_o.data
        pad = torch.zeros(wl.shape[0], self.split - wl.shape[1],
                          dtype=wl.dtype, device=wl.device)
        self.w_o = nn.Parameter(torch.cat([wl, pad, wr], 1).contiguous(),
                                requires_grad=False)
        left.w_o = right.w_o = None       # held once, in the fused matrix
        self.nleft = len(self._pieces(left.state_shape()))

    def kv_spec(self) -> Optional[LayerKVSpec]:
        return self.left.kv_spec() or self.right.kv_spec()

    @staticmethod
    def _pieces(shape):
        if shape is None:
            return []
        if len(shape) and isinstance(shape[0], (tuple, list)):
            return list(shape)
        return [shape]

    def state_shape(self):
        return (self._pieces(self.left.state_shape()) +
                self._pieces(self.right.state_shape()))

    @staticmethod
    def _part(side, pieces):
        kind = side.state_shape()
        if kind is None:
            return None
        if len(kind) and isinstance(kind[0], (tuple, list)):
            return tuple(pieces)
        return pieces[0]

    def forward(self, h: torch.Tensor, cache, state, meta,
                cache_v=None) -> torch.Tensor:
        T = h.shape[0]
        lw, rw = self.left.out_width, self.right.out_width
        buf = torch.empty(T, self.split + rw, dtype=h.dtype, device=h.device)
        if self.split != lw:
            buf[:, lw: self.split] = 0
        n = self.nleft
        self.left.pre_output(h, cache, self._part(self.left, state[:n]), meta,
                             cache_v, buf[:, :lw], self.left_scale)
        self.right.pre_output(h, cache, self._part(self.right, state[n:]),
                              meta, cache_v, buf[:, self.split:],
                              self.right_scale)
        return ops.linear(buf, self.w_o)
