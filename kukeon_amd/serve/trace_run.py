"""Replay a token trace through the serving engine and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3],
                             "want": [0, 2]}], "end": ["a"]}

Every entry brings a request's next tokens (a prompt portion or a single
token); all entries of a step run as one engine batch on top of the pages
and state slots earlier steps left. The logits at the wanted places go to
DIR/<step>.f32 (little-endian fp32, [wanted, vocab]); `done <step>` is
printed after every step. Requests named in `end` give their pages and
state slot back. Nothing is sampled: this drives LLMEngine.forward_tokens,
the teacher-forced twin of the generation step.

The model class is chosen by config.json's `architecture`. Kernel groups
the model needs are compiled on first use if the built modules are absent.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built(groups) -> None:
    """Compile the kernel groups that are not importable yet."""
    from kukeon_amd.ops import build as kbuild
    missing = [g for g in groups if not kbuild.so_path(g).exists()]
    if missing:
        print(f"building kernel groups {missing}", file=sys.stderr,
              flush=True)
        os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
        kbuild.build(verbose=False, groups=missing)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser("trace_run", description=__doc__,
                                 formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"),
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time")
    ap.add_argument("--device", default=None)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--slots", type=int, default=4,
                    help="requests live at any time (state slots)")
    args = ap.parse_args(argv)

    with open(os.path.join(args.model, "config.json")) as f:
        arch = json.load(f).get("architecture")
    from kukeon_amd.models.registry import ARCHITECTURES, OP_GROUPS
    if arch not in ARCHITECTURES:
        print(f"no model class for architecture {arch!r}", file=sys.stderr)
        return 2

    import torch
    device = args.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    if device.startswith("cuda"):
        _ensure_built(OP_GROUPS[ARCHITECTURES[arch]])
    # exact mode: no reduced-precision matrix products
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")

    from kukeon_amd.engine.config import EngineConfig
    from kukeon_amd.engine.engine import LLMEngine
    from kukeon_amd.engine.kv_cache import SequenceKV
    from kukeon_amd.models.registry import load_checkpoint

    bs = args.block_size
    per_req = -(-64 // bs) * bs            # a request's count rounds up to 64
    nblocks = -(-args.max_tokens // per_req) * (per_req // bs)
    cfg, model = load_checkpoint(
        args.model, device=device,
        dtype="fp32" if args.dtype == "float32" else "bf16")
    max_len = nblocks * bs
    model.set_max_position(max_len)
    # a model with a position table bounds the longest sequence itself
    max_len = min(max_len, getattr(model, "max_position", max_len))
    ecfg = EngineConfig(block_size=bs, max_model_len=max_len,
                        max_sessions=args.slots, state_slots=args.slots,
                        num_kv_blocks=nblocks, use_graphs=False)
    engine = LLMEngine(model, cfg, ecfg, device=device)
    os.makedirs(args.out, exist_ok=True)

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries, want = [], []
        for e in step.get("entries", []):
            kv = live.get(e["id"])
            if kv is None:
                kv = live[e["id"]] = SequenceKV(bs)
            entries.append((kv, e["tokens"]))
            want.append(list(e.get("want", [])))
        if any(want):
            logits = engine.forward_tokens(entries, want)
            data = logits.detach().to("cpu", torch.float32).contiguous()
            path = os.path.join(args.out, "%d.f32" % step["step"])
            with open(path + ".part", "wb") as f:
                f.write(data.numpy().astype("<f4", copy=False).tobytes())
            os.replace(path + ".part", path)
        elif entries:
            engine.forward_tokens(entries, want)
            if device.startswith("cuda"):
                torch.cuda.synchronize()
        for rid in step.get("end", []):
            kv = live.pop(rid, None)
            if kv is not None:
                engine.free_sequence(kv)
        print("done %d" % step["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
