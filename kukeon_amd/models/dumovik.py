"""Dumovik: a decoder whose layers pick one of three sequence mixers —
latent attention, chunk-local grouped-query attention, or linear attention
with a fixed decay — and whose sublayers are normed on the OUTPUT side only:

    x <- x + layernorm(mixer(x)) ;  x <- x + layernorm(ff(x))

The sublayers read the fp32 residual stream itself (its rounding to the
activation format in bf16 mode); the layer norm takes the mean off, has a
weight and no bias. The feed-forward is a gelu-gated dense layer or a
mixture of clamped gated experts chosen by a router; a layer may have none.
The logits come from the embedding table after a final layer norm.

Everything a checkpoint's config.json states (sizes, layer order, which
layer reads whose keys, constants) is read from it. Attention layers keep
pages in the paged cache (one latent row per token, or key and value rows
per kv head); linear-attention layers keep a state matrix per head in the
engine's state slots.

Tensor parallelism is not implemented for this family (tp_size must be 1).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kukeon_amd import ops
from kukeon_amd import parallel
from kukeon_amd.models.feedforward import FFCfg, GeluGatedFF, RoutedMoE
from kukeon_amd.models.mixers import (ChunkAttnCfg, ChunkedAttention,
                                      LatentAttention, LatentAttnCfg,
                                      LightningCfg, LightningMixer)
from kukeon_amd.models.rotary import angle_table

_DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
           "fp32": torch.float32, "float32": torch.float32}

MIXERS = {"latent_attention": LatentAttention, "attention": ChunkedAttention,
          "lightning": LightningMixer}
FEED_FORWARDS = {"dense": GeluGatedFF, "moe": RoutedMoE}


@dataclass
class DumovikLayerCfg:
    type: str
    mixer: object
    mlp: Optional[FFCfg]


@dataclass
class DumovikConfig:
    family = "dumovik"
    name: str = "dumovik"
    width: int = 1024
    vocab_size: int = 32000
    norm_eps: float = 1e-5
    layers: List[DumovikLayerCfg] = field(default_factory=list)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    @staticmethod
    def from_json(c: dict, name: str = "dumovik") -> "DumovikConfig":
        layers = []
        for i, L in enumerate(c["layers"]):
            kind = L.get("type")
            m = L["mixer"]
            if kind == "latent_attention":
                r = m["rot"]
                mix = LatentAttnCfg(
                    heads=int(m["heads"]), dim=int(m["dim"]),
                    rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                    q_rank=0, kv_rank=int(m["kv_rank"]),
                    scale=float(m["scale"]), window=0,
                    rot_dims=int(r["dims"]), rot_base=float(r["base"]),
                    rot_layout="half", gate="element")
            elif kind == "attention":
                mix = ChunkAttnCfg(
                    heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                    dim=int(m["dim"]), vdim=int(m["vdim"]),
                    scale=float(m["scale"]),
                    softcap=float(m.get("softcap") or 0.0),
                    chunk=int((m.get("mask") or {}).get("size") or 0),
                    kv_from=(int(m["kv_from"])
                             if m.get("kv_from") is not None else None))
            elif kind == "lightning":
                mix = LightningCfg(
                    heads=int(m["heads"]), dim=int(m["dim"]),
                    vdim=int(m["vdim"]),
                    decay=tuple(float(d) for d in m["decay"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = None
            if L.get("mlp"):
                f = L["mlp"]
                fk = f.get("kind", "dense")
                if fk == "dense":
                    mlp = FFCfg("dense", int(f["ff"]))
                elif fk == "moe":
                    mlp = FFCfg("moe", int(f["expert"]["ff"]),
                                experts=int(f["router"]["experts"]),
                                top=int(f["router"]["top"]),
                                limit=float(f["expert"]["limit"]))
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind "
                                     f"{fk!r}")
            layers.append(DumovikLayerCfg(kind, mix, mlp))
        return DumovikConfig(
            name=name, width=int(c["width"]), vocab_size=int(c["vocab"]),
            norm_eps=float(c["norm"]["eps"]), layers=layers)


def head_decays(heads: int) -> tuple:
    """A spread of decays for random-weight stacks: fast-forgetting heads
    first, the last head close to 1."""
    return tuple(1.0 - 2.0 ** (-1.0 - 8.0 * h / max(1, heads - 1))
                 for h in range(heads))


def dumovik_bench(width=4096, layers=8, heads=32, kv_heads=8, ff=14336,
                  vocab=128256, chunk=2048, experts=16, top=2,
                  name="dumovik-8b-like") -> DumovikConfig:
    """A layer stack at real-model sizes (random weights) for throughput
    runs, in periods of four layers: chunked attention (128-wide heads),
    two linear-attention layers (128-wide heads), latent attention (heads
    of 128 + 64, a 512-wide latent); the second chunked-attention layer of
    every two reads the first one's pages; feed-forwards alternate between
    dense and routed experts of the same total active size."""
    ls = []
    first_attn = None
    for i in range(layers):
        k = i % 4
        if k == 0:
            kind = "attention"
            share = first_attn if (first_attn is not None and
                                   (i // 4) % 2 == 1) else None
            mix = ChunkAttnCfg(heads=heads, kv_heads=kv_heads, dim=128,
                               vdim=128, scale=128 ** -0.5, softcap=30.0,
                               chunk=chunk, kv_from=share)
            if share is None:
                first_attn = i
        elif k == 3:
            kind = "latent_attention"
            mix = LatentAttnCfg(heads=heads, dim=128, rot_dim=64, vdim=128,
                                q_rank=0, kv_rank=512, scale=192 ** -0.5,
                                window=0, rot_dims=64, rot_base=10000.0,
                                rot_layout="half", gate="element")
        else:
            kind = "lightning"
            mix = LightningCfg(heads=heads, dim=128, vdim=128,
                               decay=head_decays(heads))
        if i % 2:
            mlp = FFCfg("moe", max(8, ff // top // 8 * 8), experts=experts,
                        top=top, limit=7.0)
        else:
            mlp = FFCfg("dense", ff)
        ls.append(DumovikLayerCfg(kind, mix, mlp))
    return DumovikConfig(name=name, width=width, vocab_size=vocab,
                         norm_eps=1e-5, layers=ls)


def tensor_shapes(cfg: DumovikConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        out[p + "norm1"] = (W,)
        for n, s in MIXERS[L.type].tensor_shapes(L.mixer, W).items():
            out[p + "mix." + n] = s
        if L.mlp is not None:
            out[p + "norm2"] = (W,)
            shapes = FEED_FORWARDS[L.mlp.kind].tensor_shapes(
                L.mlp, W, cfg.vocab_size)
            for n, s in shapes.items():
                out[p + "mlp." + n] = s
    out["final.norm"] = (W,)
    return out


def random_tensors(cfg: DumovikConfig, seed: int = 0,
                   device="cpu") -> Dict[str, torch.Tensor]:
    """Random bf16 weights at a scale that keeps activations O(1)."""
    on_gpu = torch.device(device).type == "cuda"
    gdev = device if on_gpu else "cpu"
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if len(shp) == 2:
            std = shp[1] ** -0.5 if name != "embed" else 1.0
            if leaf == "router":
                std *= 2.0
            t = torch.randn(shp, generator=g, device=gdev) * std
        elif leaf in ("norm1", "norm2"):
            t = 0.5 + torch.randn(shp, generator=g, device=gdev) * 0.1
        else:
            t = 1.0 + torch.randn(shp, generator=g, device=gdev) * 0.1
        out[name] = t.to(torch.bfloat16).to(device)
    return out


class DumovikLayer(nn.Module):
    def __init__(self, cfg: DumovikConfig, idx: int,
                 t: Dict[str, torch.Tensor], device, dtype):
        super().__init__()
        L = cfg.layers[idx]
        p = f"l{idx}."
        W = cfg.width
        self.idx = idx
        f32 = dict(device=device, dtype=torch.float32)
        self.norm1 = t[p + "norm1"].to(**f32).contiguous()
        self.mixer = MIXERS[L.type](L.mixer, W, cfg.norm_eps, t, p + "mix.",
                                    device, dtype)
        # the layer whose pages this layer's mixer reads
        self.kv_layer = getattr(L.mixer, "kv_from", None)
        if self.kv_layer is None:
            self.kv_layer = idx
        self.ff = None
        if L.mlp is not None:
            self.norm2 = t[p + "norm2"].to(**f32).contiguous()
            self.ff = FEED_FORWARDS[L.mlp.kind](L.mlp, W, t, p + "mlp.",
                                                device, dtype)


class DumovikModel(nn.Module):
    family = "dumovik"
    op_groups = ("hyb",)        # kernel groups the forward pass needs

    def __init__(self, cfg: DumovikConfig, device="cuda", dtype="bf16",
                 tensors: Optional[Dict[str, torch.Tensor]] = None,
                 max_position: int = 4096, seed: int = 0):
        super().__init__()
        if parallel.tp_size() != 1:
            raise NotImplementedError("Dumovik runs with tp_size == 1 only")
        self.cfg = cfg
        self.device_ = torch.device(device)
        self.dtype = _DTYPES[dtype] if isinstance(dtype, str) else dtype
        if tensors is None:
            tensors = random_tensors(cfg, seed, device=self.device_)
        for name, shp in tensor_shapes(cfg).items():
            if name not in tensors:
                raise KeyError(f"checkpoint lacks tensor {name}")
            if tuple(tensors[name].shape) != tuple(shp):
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}"
                                 f", configuration says {tuple(shp)}")
        for i, L in enumerate(cfg.layers):
            j = getattr(L.mixer, "kv_from", None)
            if j is None:
                continue
            ok = 0 <= j < i and cfg.layers[j].type == L.type and \
                cfg.layers[j].mixer.kv_from is None
            if not ok:
                raise ValueError(f"layer {i}: kv_from must name an earlier "
                                 "layer of the same kind with keys of its "
                                 "own")
        dev, dt = self.device_, self.dtype
        self.embed = nn.Parameter(tensors["embed"].to(dev).to(dt),
                                  requires_grad=False)
        self.layers = nn.ModuleList(
            [DumovikLayer(cfg, i, tensors, dev, dt)
             for i in range(cfg.num_layers)])
        self.final_norm = tensors["final.norm"].to(dev).float().contiguous()
        self.set_max_position(max_position)

    @classmethod
    def from_checkpoint(cls, model_dir: str, device="cuda", dtype="bf16",
                        max_position: int = 4096):
        from kukeon_amd.models.weights import read_checkpoint
        config, tensors = read_checkpoint(model_dir)
        cfg = DumovikConfig.from_json(config)
        return cfg, cls(cfg, device=device, dtype=dtype, tensors=tensors,
                        max_position=max_position)

    def set_max_position(self, n: int) -> None:
        """(Re)build the angle tables for positions 0 .. n-1."""
        self.max_position = n
        tables: Dict[tuple, torch.Tensor] = {}
        for L in self.layers:
            mx = L.mixer
            if isinstance(mx, LatentAttention):
                key = (mx.m.rot_dims, mx.m.rot_base)
                if key not in tables:
                    tables[key] = angle_table(n, key[0], key[1]).to(
                        self.device_)
                mx.cs = tables[key]

    # ---- what the engine asks of a model with its own cache layout ----
    def kv_specs(self):
        return [L.mixer.kv_spec() for L in self.layers]

    def state_shapes(self):
        return [L.mixer.state_shape() for L in self.layers]

    def activation_dtype(self) -> torch.dtype:
        return self.dtype

    # ---- forward ----
    def forward(self, input_ids: torch.Tensor, kv_k, kv_v, meta,
                taps: Optional[list] = None) -> torch.Tensor:
        """-> final-normed hidden [T, W]. `taps`, if a list, receives the
        fp32 residual stream after every layer."""
        eps = self.cfg.norm_eps
        h = F.embedding(input_ids.long(), self.embed)
        x = h.float().contiguous()
        if h.dtype == torch.float32:
            h = x
        for i, layer in enumerate(self.layers):
            st = meta.state[i] if meta.state is not None else None
            j = layer.kv_layer
            y = layer.mixer(h, kv_k[j], st, meta, kv_v[j])
            h = torch.empty_like(h)
            ops.layernorm_residual(x, y, layer.norm1, eps, h)
            if layer.ff is not None:
                y = layer.ff(h, input_ids, meta)
                h = torch.empty_like(h)
                ops.layernorm_residual(x, y, layer.norm2, eps, h)
            if taps is not None:
                taps.append(x.clone())
        out = torch.empty_like(h)
        ops.layernorm(out, x, self.final_norm, eps)
        return out

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(hidden, self.embed)
