#!/usr/bin/env python3
"""Flagship serving benchmark: agent turns/sec, 64 Sessions on Llama-3-8B.

Driver contract: `python bench.py --gpus N --steps K --warmup W` (for N>1 the
driver launches via torch.distributed.run, one rank per GPU over RCCL).
One *step* = one lockstep round in which EVERY session completes one agent
turn (prompt prefill + decode) against its persistent paged-KV context.
Sessions are sharded across GPUs (data parallel — the production answer for
an 8B backing model on an 8-GPU node); per-GPU work is fixed => weak scaling.

Rank 0 prints one JSON line with the whole-job aggregate turns/sec.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch


# layer sizes for --compare-families: (width, q heads, kv heads, ff, layers)
COMPARE_SIZES = {
    "2k": (2048, 16, 4, 8192, 4),
    "4k": (4096, 32, 8, 14336, 4),
    "8k": (8192, 64, 8, 28672, 2),
}


def compare_families(args) -> None:
    """Prefill and decode tokens/s of Lipedra, Rasesun, Dumovik or Bezizen
    and of Llama (or another family) through the same engine at equal sizes: same
    width, head counts,
    feed-forward size, layer count and vocabulary (Llama head_dim 128;
    Lipedra two score maps of 64 and value rows of 128 — equal cache bytes
    per token; Rasesun three state-space layers to one latent-attention
    layer with a 1024-token window, every second feed-forward a mixture of
    16 table-routed experts, two active; Dumovik periods of chunk-local
    attention over 8192-token chunks, two linear-attention layers and latent
    attention, every second feed-forward a mixture of 16 routed experts, two
    active; Bezizen four residual streams, three wkv layers to one parallel
    layer of windowed attention over 1024 tokens beside a gated linear
    attention, a shared expert everywhere and every second feed-forward a
    mixture of 16 routed experts, two active)."""
    from kukeon_amd.engine.config import (EngineConfig, ModelConfig,
                                          SamplingParams)
    from kukeon_amd.engine.engine import LLMEngine
    from kukeon_amd.engine.kv_cache import SequenceKV
    from kukeon_amd.models import registry
    from kukeon_amd.models.bezizen import bezizen_bench
    from kukeon_amd.models.dumovik import dumovik_bench
    from kukeon_amd.models.lipedra import lipedra_bench
    from kukeon_amd.models.rasesun import rasesun_bench

    device = args.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    on_gpu = device != "cpu"
    nseq, plen, dlen = (32, 1024, 64) if on_gpu else (2, 40, 4)
    vocab = 32000 if on_gpu else 512
    rows = []
    for size in args.compare_sizes.split(","):
        W, hq, hk, ff, nl = COMPARE_SIZES[size]
        if not on_gpu:
            W, hq, hk, ff, nl = 256, 2, 2, 512, 2
        for fam in (args.compare_against, args.compare_family):
            if fam == "llama":
                cfg = ModelConfig(name=f"llama-{size}", hidden_size=W,
                                  num_layers=nl, num_q_heads=hq,
                                  num_kv_heads=hk, head_dim=128,
                                  intermediate_size=ff, vocab_size=vocab,
                                  max_position=4096)
            elif fam == "rasesun":
                cfg = rasesun_bench(width=W, layers=nl, heads=hq, ff=ff,
                                    vocab=vocab, attn_every=min(4, nl),
                                    window=1024 if on_gpu else 16,
                                    experts=16 if on_gpu else 4,
                                    name=f"rasesun-{size}")
            elif fam == "bezizen":
                cfg = bezizen_bench(width=W, layers=nl, heads=hq,
                                    kv_heads=hk, ff=ff, vocab=vocab,
                                    window=1024 if on_gpu else 16,
                                    experts=16 if on_gpu else 4,
                                    max_positions=2048,
                                    name=f"bezizen-{size}")
            elif fam == "dumovik":
                cfg = dumovik_bench(width=W, layers=nl, heads=hq,
                                    kv_heads=hk, ff=ff, vocab=vocab,
                                    chunk=8192 if on_gpu else 16,
                                    experts=16 if on_gpu else 4,
                                    name=f"dumovik-{size}")
            else:
                cfg = lipedra_bench(width=W, layers=nl, heads=hq,
                                    kv_heads=hk, dim=64, vdim=128, ff=ff,
                                    vocab=vocab, share_every=0,
                                    name=f"lipedra-{size}")
            print(f"[compare] {size} {fam}: building", file=sys.stderr,
                  flush=True)
            model = registry.build_model(cfg, device)
            ecfg = EngineConfig(max_model_len=2048, max_sessions=nseq,
                                num_kv_blocks=nseq * 80 + 64,
                                use_graphs=on_gpu and not args.no_graphs,
                                graph_buckets=(nseq,),
                                decode_microbatch=dlen,
                                max_prefill_tokens=16384)
            engine = LLMEngine(model, cfg, ecfg, device=device)
            gen = torch.Generator().manual_seed(7)
            sp = SamplingParams(temperature=0.7, top_k=50, top_p=0.9,
                                max_new_tokens=dlen + 1)

            def sync():
                if on_gpu:
                    torch.cuda.synchronize()

            best = None
            for rnd in range(1 + max(1, args.steps)):
                kvs = [SequenceKV(ecfg.block_size) for _ in range(nseq)]
                for kv in kvs:
                    engine.add_request(kv, torch.randint(
                        0, vocab, (plen,), generator=gen).tolist(), sp)
                print(f"[compare] {size} {fam}: round {rnd}", file=sys.stderr,
                      flush=True)
                sync()
                t0 = time.perf_counter()
                while engine.waiting:
                    engine.step()
                sync()
                t1 = time.perf_counter()
                while engine.has_work():
                    engine.step()
                sync()
                t2 = time.perf_counter()
                for kv in kvs:
                    engine.free_sequence(kv)
                if rnd == 0:
                    continue            # warmup: graph capture, BLAS plans
                cur = (nseq * plen / (t1 - t0), nseq * dlen / (t2 - t1))
                best = cur if best is None else (max(best[0], cur[0]),
                                                 max(best[1], cur[1]))
            rows.append({"size": size, "family": fam, "width": W,
                         "layers": nl, "q_heads": hq, "kv_heads": hk,
                         "ff": ff, "sequences": nseq, "prompt_len": plen,
                         "decode_len": dlen,
                         "prefill_tok_s": round(best[0], 1),
                         "decode_tok_s": round(best[1], 1)})
            del engine, model
            if on_gpu:
                torch.cuda.empty_cache()
    print(json.dumps({"metric": "family_compare_tokens_per_sec",
                      "dtype": "bf16", "data": "synthetic",
                      "rows": rows}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--model", default="llama-3-8b")
    ap.add_argument("--sessions", type=int, default=64)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--followup-len", type=int, default=256)
    ap.add_argument("--decode-len", type=int, default=128)
    ap.add_argument("--ctx-cap", type=int, default=3584)
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--decode-microbatch", type=int, default=64)
    ap.add_argument("--kv-dtype", choices=["bf16", "fp8"], default="bf16")
    ap.add_argument("--moe-ep", action="store_true",
                    help="MoE expert parallelism: experts partitioned "
                         "across ranks, tokens routed over all-to-all "
                         "(RCCL over xGMI); sessions stay rank-local")
    ap.add_argument("--device", default=None)
    ap.add_argument("--compare-families", action="store_true",
                    help="instead of the headline workload: prefill and "
                         "decode throughput of the Lipedra family beside "
                         "Llama at equal layer sizes (random weights)")
    ap.add_argument("--compare-family", default="lipedra",
                    choices=["lipedra", "rasesun", "dumovik", "bezizen"],
                    help="with --compare-families: the family that runs "
                         "beside Llama")
    ap.add_argument("--compare-against", default="llama",
                    choices=["llama", "lipedra", "rasesun", "dumovik"],
                    help="with --compare-families: the family it runs "
                         "beside (default Llama)")
    ap.add_argument("--compare-sizes", default="2k,4k,8k",
                    help="with --compare-families: which of 2k,4k,8k")
    args = ap.parse_args()
    if args.compare_families:
        compare_families(args)
        return

    from kukeon_amd import parallel
    from kukeon_amd.engine.config import (EngineConfig, MODEL_PRESETS,
                                          SamplingParams)
    from kukeon_amd.engine.engine import LLMEngine
    from kukeon_amd.serve.sessions import TurnDriver

    rank, world = parallel.init_distributed()
    n_gpus = max(args.gpus, world)

    if args.device:
        device = args.device
    elif torch.cuda.is_available():
        dev_i = int(os.environ.get("LOCAL_RANK", 0)) % torch.cuda.device_count()
        device = f"cuda:{dev_i}"
        torch.cuda.set_device(device)
    else:
        device = "cpu"

    from kukeon_amd.models import registry
    cfg = registry.preset(args.model)
    tp_size = world if args.model == "llama-3-70b" else 1
    # TP ranks share a sampling seed (identical draws, no collective needed)
    ecfg = EngineConfig(max_model_len=args.max_model_len,
                        max_sessions=max(args.sessions, 8),
                        use_graphs=(not args.no_graphs and device != "cpu"),
                        decode_microbatch=args.decode_microbatch,
                        kv_dtype=args.kv_dtype,
                        seed=1234 + rank // tp_size)
    if device == "cpu":
        ecfg.num_kv_blocks = (args.sessions *
                              (args.ctx_cap // ecfg.block_size + 2) + 64)

    if args.model == "llama-3-70b":
        parallel.init_tensor_parallel(world)
        ecfg.tp_size = world
    use_ep = args.moe_ep and world > 1
    if use_ep:
        parallel.init_expert_parallel(world)
        ecfg.use_graphs = False  # all-to-all splits are data-dependent
    model = registry.build_model(cfg, device)

    engine = LLMEngine(model, cfg, ecfg, device=device)
    tp = ecfg.tp_size
    dp = max(1, world // tp)
    sessions_per_engine = args.sessions
    vocab = cfg.vocab_size
    sampling = SamplingParams(temperature=0.7, top_k=50, top_p=0.9,
                              max_new_tokens=args.decode_len)
    driver = TurnDriver(engine, sessions_per_engine, vocab,
                        first_prompt=args.prompt_len,
                        followup_prompt=args.followup_len,
                        decode_len=args.decode_len, ctx_cap=args.ctx_cap,
                        sampling=sampling, seed=1234 + (rank // tp))

    def sync():
        if device != "cpu":
            torch.cuda.synchronize()
        parallel.barrier()

    engine.capture_all()
    for _ in range(args.warmup):
        driver.run_round()
    driver.turn_latencies.clear()

    sync()
    t0 = time.perf_counter()
    turns = 0
    for _ in range(args.steps):
        turns += driver.run_round()
    sync()
    elapsed = time.perf_counter() - t0

    # max over ranks (slowest rank defines the job)
    if world > 1:
        import torch.distributed as dist
        t = torch.tensor([elapsed], dtype=torch.float64,
                         device=device if device != "cpu" else None)
        dist.all_reduce(t, op=dist.ReduceOp.MAX)
        elapsed = float(t[0])

    total_turns = turns * dp  # TP ranks serve the same sessions once
    value = total_turns / elapsed
    p50 = (statistics.median(driver.turn_latencies) * 1000
           if driver.turn_latencies else None)

    if rank == 0:
        out = {
            "metric": "agent_turns_per_sec",
            "value": round(value, 3),
            "unit": "turns/s",
            "n_gpus": n_gpus,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(elapsed / args.steps * 1000, 2),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            # weights/compute are always bf16; a reduced-precision KV
            # cache is reported so the line never overstates the dtype
            "dtype": ("bf16" if args.kv_dtype == "bf16"
                      else f"bf16+kv_{args.kv_dtype}"),
            "data": "synthetic",
            "p50_turn_latency_ms": round(p50, 1) if p50 else None,
            "config": {
                "model": args.model,
                "global_batch": sessions_per_engine * dp,
                "seq_len": args.ctx_cap,
                "parallelism": (f"ep{world}" if use_ep else
                                f"tp{tp}" if tp > 1 else f"dp{dp}"),
                "sessions_per_gpu_group": sessions_per_engine,
                "prompt_len": args.prompt_len,
                "followup_len": args.followup_len,
                "decode_len": args.decode_len,
                "turns_per_step": sessions_per_engine * dp,
            },
        }
        print(json.dumps(out))


if __name__ == "__main__":
    main()
