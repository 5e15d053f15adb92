"""Feed-forward sublayers beyond the SwiGLU of the Llama family: a dense
layer with the xIELU activation, a mixture of small experts chosen by a
per-token-id table (no learned router at run time), a gated dense layer with
the tanh form of gelu, and a mixture of clamped gated experts chosen by a
learned router."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict

import torch
import torch.nn as nn

from kukeon_amd import ops
from kukeon_amd.models.mixers import fuse_rows


@dataclass
class FFCfg:
    kind: str                # "dense" | "moe"
    ff: int                  # hidden size (of one expert for "moe")
    experts: int = 0
    top: int = 0
    limit: float = 0.0       # clamp of the routed experts' gate and up
    # routed experts: "clamp" is g sigmoid(1.702 g) (u + 1) with g and u
    # clamped to `limit`; "silu" is silu(g) u
    act: str = "clamp"
    # "top": weights = softmax over the chosen logits; "all": scores =
    # softmax over all logits, the chosen scores divided by their sum and
    # multiplied by route_scale
    score: str = "top"
    groups: int = 0          # experts in this many equal runs of neighbours,
    keep: int = 0            # of which only the best `keep` can be chosen
    route_scale: float = 1.0
    shared_ff: int = 0       # hidden size of an always-on expert (0: none)


def pad_rows(w: torch.Tensor, multiple: int) -> torch.Tensor:
    """w with zero rows appended up to a multiple of `multiple` rows."""
    n = -w.shape[0] % multiple
    if not n:
        return w
    return torch.cat([w, torch.zeros(n, w.shape[1], dtype=w.dtype,
                                     device=w.device)], 0).contiguous()


def _softplus(x: float) -> float:
    return x if x > 30 else math.log1p(math.exp(x))


class XieluFF(nn.Module):
    """down(act(up h)) with act(z) = softplus(p) z^2 + z/2 for z > 0 and
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 otherwise; (p, q) is the
    two-entry tensor `act`."""

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        dev = dict(device=device, dtype=dtype)
        self.w_up = nn.Parameter(t[p + "up"].to(**dev).contiguous(),
                                 requires_grad=False)
        self.w_down = nn.Parameter(t[p + "down"].to(**dev).contiguous(),
                                   requires_grad=False)
        pq = t[p + "act"].double()
        self.ap = _softplus(float(pq[0]))
        self.aq = 0.5 + _softplus(float(pq[1]))

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        return {"up": (f.ff, width), "down": (width, f.ff), "act": (2,)}

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        z = ops.linear(h, self.w_up)
        a = torch.empty_like(z)
        ops.xielu(a, z, self.ap, self.aq)
        return ops.linear(a, self.w_down)


class TableMoE(nn.Module):
    """`experts` small feed-forward layers down(relu(up h)^2) without
    biases; token id v uses the `top` experts table[v] with weight 1/top
    each. The expert weights are stacked [E, ff, W] and [E, W, ff]."""

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        dev = dict(device=device, dtype=dtype)
        self.f = f
        self.w_up = nn.Parameter(torch.stack(
            [t[p + f"e{e}.up"] for e in range(f.experts)]).to(**dev)
            .contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(torch.stack(
            [t[p + f"e{e}.down"] for e in range(f.experts)]).to(**dev)
            .contiguous(), requires_grad=False)
        table = t[p + "table"].to(torch.int32)
        if table.dim() != 2 or table.shape[1] != f.top:
            raise ValueError(f"{p}table: shape {tuple(table.shape)}")
        if int(table.min()) < 0 or int(table.max()) >= f.experts:
            raise ValueError(f"{p}table names an expert that does not exist")
        self.table = table.to(device).contiguous()
        self.table_host = table.cpu().numpy()

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        out = {"table": (vocab, f.top)}
        for e in range(f.experts):
            out[f"e{e}.up"] = (f.ff, width)
            out[f"e{e}.down"] = (width, f.ff)
        return out

    # portions of at least this many rows take the grouped form when the
    # step's token ids are known on the host
    grouped_min_rows = 64

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        out = torch.empty_like(h)
        host_ids = getattr(meta, "host_ids", None)
        if host_ids is not None and h.shape[0] >= self.grouped_min_rows:
            return self._forward_grouped(out, h, host_ids, meta)
        ops.table_moe(out, h, ids, self.table, self.w_up, self.w_down)
        return out

    def _forward_grouped(self, out, h, host_ids, meta) -> torch.Tensor:
        """Rows sorted by expert on the host (the routing is a function of
        the token id, which the scheduler knows): no device round trip to
        learn the group sizes, and every expert runs plain GEMMs over its
        contiguous rows."""
        import numpy as np
        T, W = h.shape
        top, E = self.f.top, self.f.experts
        key = ("table_moe", id(self))
        maps = meta.tile_maps.get(key)
        if maps is None:
            flat = self.table_host[np.asarray(host_ids)].reshape(-1)
            order = np.argsort(flat, kind="stable")
            counts = np.bincount(flat, minlength=E)
            inv = np.empty_like(order)
            inv[order] = np.arange(order.size)
            dev = h.device
            maps = (torch.from_numpy((order // top).astype(np.int32)).to(dev),
                    torch.from_numpy(inv.astype(np.int32).reshape(T, top))
                    .to(dev), counts.tolist())
            meta.tile_maps[key] = maps
        row_map, inv, counts = maps
        rows = torch.empty(T * top, W, dtype=h.dtype, device=h.device)
        ops.gather_rows(rows, h, row_map)
        done = torch.empty_like(rows)
        at = 0
        for e in range(E):
            n = counts[e]
            if n == 0:
                continue
            a = ops.linear(rows[at: at + n], self.w_up[e])
            ops.relu_square_(a)
            done[at: at + n] = ops.linear(a, self.w_down[e])
            at += n
        ops.combine_rows(out, done, inv)
        return out


class GeluGatedFF(nn.Module):
    """down(gelu_tanh(gate h) * (up h)); gate and up are one fused GEMM."""

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        self.ff = f.ff
        self.col, self.w_in = fuse_rows(
            [("gate", t[p + "gate"]), ("up", t[p + "up"])], width, dtype,
            device)
        self.w_down = nn.Parameter(t[p + "down"].to(device=device,
                                                    dtype=dtype)
                                   .contiguous(), requires_grad=False)

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        return {"gate": (f.ff, width), "up": (f.ff, width),
                "down": (width, f.ff)}

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        z = ops.linear(h, self.w_in)
        a = torch.empty(h.shape[0], self.ff, dtype=h.dtype, device=h.device)
        c = self.col
        ops.gelu_glu(a, z[:, c["gate"]: c["gate"] + self.ff],
                     z[:, c["up"]: c["up"] + self.ff])
        return ops.linear(a, self.w_down)


class RoutedMoE(nn.Module):
    """`experts` small gated feed-forward layers without biases; a token
    uses the `top` experts with the largest router logits, weighted by the
    softmax over those logits only. Expert: g = min(gate h, limit),
    u = clamp(up h, +-limit), y = g sigmoid(1.702 g) (u + 1), out = down y.
    The router's logits, the choice and the weights are fp32.

    Variants by configuration: experts of the form down(silu(gate h) up h)
    (`act`); scores from a softmax over ALL logits, the chosen ones divided
    by their sum and scaled, the choice limited to the best `keep` of
    `groups` runs of neighbouring experts (`score`, `groups`); an always-on
    shared expert of the same form (`shared_ff`), which enters the fold as
    one more chosen row with weight 1. Weights are stacked [E, 2 ff', W] (gate rows,
    then up rows, each padded to a multiple of 8) and [E, W, ff].

    Two forms behind one call. Few rows (decode steps; nothing leaves the
    device, so the step can sit in a captured graph): every expert runs on
    every row as one batched GEMM pair — a batch of a few dozen rows
    touches nearly every expert anyway, so the weights stream once — and
    the fold picks each row's chosen results. Many rows (prompt portions):
    the (row, expert) pairs are sorted by expert, the group sizes come to
    the host, and each expert runs plain GEMMs over its contiguous rows."""

    sorted_min_rows = 64
    alpha = 1.702

    def __init__(self, f: FFCfg, width: int, t: Dict[str, torch.Tensor],
                 p: str, device, dtype):
        super().__init__()
        if not (0 < f.top <= f.experts):
            raise ValueError(f"{p}: top must be within 1 .. experts")
        if f.act not in ("clamp", "silu") or f.score not in ("top", "all"):
            raise ValueError(f"{p}: unknown expert or router kind")
        if f.groups:
            if f.score != "all" or f.experts % f.groups or \
                    not (0 < f.keep <= f.groups) or \
                    f.top > f.keep * (f.experts // f.groups):
                raise ValueError(f"{p}: expert groups do not fit the router")
        self.f = f
        # clamp_glu's constants: the silu form is the unclamped one with
        # alpha 1 and no shift
        self.glu = ((f.limit, self.alpha, 1.0) if f.act == "clamp"
                    else (float("inf"), 1.0, 0.0))
        dev = dict(device=device, dtype=dtype)
        self.shared = None
        if f.shared_ff:
            sp = (f.shared_ff + 7) // 8 * 8
            sgu = torch.zeros(2 * sp, width, **dev)
            sgu[:f.shared_ff] = t[p + "shared.gate"].to(**dev)
            sgu[sp: sp + f.shared_ff] = t[p + "shared.up"].to(**dev)
            self.shared = (nn.Parameter(sgu.contiguous(),
                                        requires_grad=False),
                           nn.Parameter(t[p + "shared.down"].to(**dev)
                                        .contiguous(), requires_grad=False),
                           sp)
        pad = (f.ff + 7) // 8 * 8
        self.up_col = pad
        gu = torch.zeros(f.experts, 2 * pad, width, **dev)
        for e in range(f.experts):
            gu[e, :f.ff] = t[p + f"e{e}.gate"].to(**dev)
            gu[e, pad: pad + f.ff] = t[p + f"e{e}.up"].to(**dev)
        self.w_gu = nn.Parameter(gu.contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(torch.stack(
            [t[p + f"e{e}.down"] for e in range(f.experts)]).to(**dev)
            .contiguous(), requires_grad=False)
        # in the activation format: products of two bf16 numbers are exact
        # in fp32, so the fp32-output GEMM over bf16 rows IS the fp32 router
        self.w_router = t[p + "router"].to(**dev).contiguous()
        if f.score == "all" and f.experts % 16:
            # the score product is made 16 columns wide at least (zero rows
            # below the experts'); the router reads the first `experts`
            self.w_router = pad_rows(self.w_router, 16)

    @staticmethod
    def tensor_shapes(f: FFCfg, width: int, vocab: int) -> Dict[str, tuple]:
        out = {"router": (f.experts, width)}
        for e in range(f.experts):
            out[f"e{e}.gate"] = (f.ff, width)
            out[f"e{e}.up"] = (f.ff, width)
            out[f"e{e}.down"] = (width, f.ff)
        if f.shared_ff:
            out.update({"shared.gate": (f.shared_ff, width),
                        "shared.up": (f.shared_ff, width),
                        "shared.down": (width, f.shared_ff)})
        return out

    def _route(self, idx, wts, logits, dense_rows: int) -> None:
        """Fill the first `top` columns of idx and wts."""
        f = self.f
        if f.score == "all":
            ops.router_select(idx, wts, logits, f.top, f.groups, f.keep,
                              f.route_scale, dense_rows)
        elif idx.shape[1] == f.top:
            ops.router_topk(idx, wts, logits, f.top, dense_rows)
        else:
            i2 = torch.empty(idx.shape[0], f.top, dtype=idx.dtype,
                             device=idx.device)
            w2 = torch.empty(idx.shape[0], f.top, dtype=wts.dtype,
                             device=idx.device)
            ops.router_topk(i2, w2, logits, f.top, dense_rows)
            idx[:, :f.top] = i2
            wts[:, :f.top] = w2

    def _shared_into(self, dst, h) -> None:
        """dst [T, W] = the shared expert's output."""
        w_gu, w_down, sp = self.shared
        ff = self.f.shared_ff
        z = ops.linear(h, w_gu)
        a = torch.empty(h.shape[0], ff, dtype=h.dtype, device=h.device)
        ops.clamp_glu(a, z[:, :ff], z[:, sp: sp + ff], None, None, *self.glu)
        if h.shape[0] > 64:
            torch.mm(a, w_down.t(), out=dst)
        else:
            dst.copy_(ops.linear(a, w_down))

    def forward(self, h: torch.Tensor, ids: torch.Tensor,
                meta=None) -> torch.Tensor:
        f = self.f
        T, W = h.shape
        logits = ops.linear_f32(h, self.w_router)[:, :f.experts]
        # with a shared expert the fold takes one more row per token
        cols = f.top + (1 if self.shared is not None else 0)
        idx = torch.empty(T, cols, dtype=torch.int32, device=h.device)
        wts = torch.empty(T, cols, dtype=torch.float32, device=h.device)
        out = torch.empty_like(h)
        on_host = getattr(meta, "host_ids", None) is not None
        if on_host and T >= self.sorted_min_rows:
            self._route(idx, wts, logits, 0)
            return self._forward_sorted(out, h, idx, wts)
        # every expert over every row; idx names rows of the [E*T, W] result
        self._route(idx, wts, logits, T)
        E, ff = f.experts, f.ff
        z = torch.bmm(h.unsqueeze(0).expand(E, T, W),
                      self.w_gu.transpose(1, 2)).view(E * T, -1)
        a = torch.empty(E * T, ff, dtype=h.dtype, device=h.device)
        ops.clamp_glu(a, z[:, :ff], z[:, self.up_col: self.up_col + ff],
                      None, None, *self.glu)
        if self.shared is None:
            y = torch.bmm(a.view(E, T, ff), self.w_down.transpose(1, 2))
            ops.combine_rows_weighted(out, y.view(E * T, W), idx, wts)
            return out
        y = torch.empty((E + 1) * T, W, dtype=h.dtype, device=h.device)
        torch.bmm(a.view(E, T, ff), self.w_down.transpose(1, 2),
                  out=y[: E * T].view(E, T, W))
        self._shared_into(y[E * T:], h)
        idx[:, f.top] = self._arange(T, h.device) + E * T
        wts[:, f.top] = 1.0
        ops.combine_rows_weighted(out, y, idx, wts)
        return out

    def _arange(self, n: int, device) -> torch.Tensor:
        """0 .. n-1 as int32, kept so that a captured step allocates and
        fills nothing new."""
        a = getattr(self, "_ar", None)
        if a is None or a.numel() < n or a.device != device:
            a = self._ar = torch.arange(max(n, 64), dtype=torch.int32,
                                        device=device)
        return a[:n]

    def _forward_sorted(self, out, h, idx, wts) -> torch.Tensor:
        f = self.f
        T, W = h.shape
        E, ff, top = f.experts, f.ff, f.top
        flat = idx[:, :top].reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=E).tolist()  # host sync
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=h.device)
        rows = torch.empty(T * top, W, dtype=h.dtype, device=h.device)
        ops.gather_rows(rows, h, (order // top).to(torch.int32))
        shared = self.shared is not None
        done = torch.empty(T * (top + 1) if shared else T * top, W,
                           dtype=h.dtype, device=h.device)
        a = torch.empty(T * top, ff, dtype=h.dtype, device=h.device)
        at = 0
        for e in range(E):
            n = counts[e]
            if n == 0:
                continue
            z = ops.linear(rows[at: at + n], self.w_gu[e])
            ops.clamp_glu(a[at: at + n], z[:, :ff],
                          z[:, self.up_col: self.up_col + ff], None, None,
                          *self.glu)
            if n > 64:      # straight into its rows, no copy
                torch.mm(a[at: at + n], self.w_down[e].t(),
                         out=done[at: at + n])
            else:
                done[at: at + n] = ops.linear(a[at: at + n], self.w_down[e])
            at += n
        if shared:
            self._shared_into(done[T * top:], h)
            idx[:, :top] = inv.view(T, top).to(torch.int32)
            idx[:, top] = self._arange(T, h.device) + T * top
            wts[:, top] = 1.0
            ops.combine_rows_weighted(out, done, idx, wts)
            return out
        ops.combine_rows_weighted(out, done, inv.view(T, top)
                                  .to(torch.int32), wts)
        return out
