"""Scenarios for the Bezizen family, run by the CPU tests (reference ops,
fp32) and the GPU tests (HIP kernels, fp32 and bf16). Every scenario builds
a small configuration with random weights, runs it through the engine and
compares with the plain model in bezizen_oracle.py."""
import torch

import bezizen_oracle as oracle
from kukeon_amd.engine.config import EngineConfig, SamplingParams
from kukeon_amd.engine.engine import LLMEngine
from kukeon_amd.engine.kv_cache import SequenceKV
from kukeon_amd.models.bezizen import BezizenConfig, BezizenModel


def wkv(heads=3, dim=5):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}}


def par(heads=4, kv_heads=2, dim=6, window=7, conv=3, temp=(0.4, 5),
        scale=None, rheads=2, rdim=5, rvdim=7, tau=4.0, ls=0.7, rs=1.2):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
            "scale": scale if scale is not None else 2.0 * dim ** -0.5}
    if window:
        left["mask"] = {"size": window}
    if conv:
        left["conv"] = conv
    if temp:
        left["q_temp"] = {"coef": temp[0], "every": temp[1]}
    right = {"heads": rheads, "dim": rdim, "vdim": rvdim, "tau": tau}
    return {"type": "parallel",
            "mixer": {"left": left, "right": right, "left_scale": ls,
                      "right_scale": rs}}


def moe(experts, top, ff, groups=None, scale=1.5, shared=0):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    f = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def layer(mix, mlp):
    return dict(mix, mlp=mlp)


def config(layers, width=40, vocab=45, eps=1e-5, streams=3, positions=400,
           embed_scale=3.0, logit_scale=0.5):
    c = {"architecture": "Bezizen", "width": width, "vocab": vocab,
         "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
         "logit_scale": logit_scale, "max_positions": positions,
         "layers": layers}
    if streams:
        c["streams"] = streams
    return c


CONFIGS = {
    # both mixers, grouped routing with a shared expert, a layer without a
    # feed-forward, fewer kv heads than heads
    "hybrid": lambda: config([
        layer(wkv(), moe(6, 2, 12, groups=(3, 2), shared=9)),
        layer(par(), moe(4, 3, 9)),
        layer(wkv(heads=2, dim=9), None),
        layer(par(heads=3, kv_heads=3, dim=4, window=5, conv=2, temp=None,
                  rheads=1, rdim=20, rvdim=12, tau=1.0),
              moe(8, 2, 10, groups=(4, 1), scale=1.0, shared=16)),
    ]),
    # rows of whole 16-byte pieces everywhere (the vector forms of the
    # kernels), four query heads on one kv head, state rows spread over
    # lanes, one expert per token, four streams
    "aligned": lambda: config([
        layer(wkv(heads=2, dim=64), moe(4, 1, 64, shared=32)),
        layer(par(heads=4, kv_heads=1, dim=16, window=20, conv=4,
                  temp=(0.5, 16), rheads=2, rdim=64, rvdim=40, tau=16.0),
              moe(8, 2, 64, groups=(2, 1), shared=64)),
        layer(wkv(heads=4, dim=32), None),
    ], width=128, vocab=50, eps=1e-3, streams=4),
    # one plain residual stream; no window, no convolution, no temperature,
    # no groups, no shared expert, every expert chosen, unit scales, a
    # width that is not a multiple of 8, no position table
    "plain": lambda: config([
        layer(par(heads=2, kv_heads=2, dim=6, window=0, conv=0, temp=None,
                  rheads=1, rdim=5, rvdim=7, ls=1.0, rs=1.0),
              moe(3, 3, 10, scale=1.0)),
        layer(wkv(heads=1, dim=7), moe(2, 1, 5)),
        layer(par(heads=3, kv_heads=1, dim=4, window=1, conv=1, temp=(1.0, 1),
                  rheads=2, rdim=3, rvdim=3), None),
    ], width=26, vocab=31, streams=0, positions=0, embed_scale=1.0,
        logit_scale=1.0),
    # a single stream WITH read, write and mix weights
    "one_stream": lambda: config([
        layer(wkv(heads=2, dim=4), moe(4, 2, 8, groups=(2, 2))),
        layer(par(heads=2, kv_heads=1, dim=8, window=9), None),
    ], width=16, vocab=21, streams=1),
    "only_wkv": lambda: config([
        layer(wkv(heads=2, dim=4), moe(3, 2, 8)),
        layer(wkv(heads=1, dim=40), None),
    ], width=16, vocab=21, streams=2),
    "only_parallel": lambda: config([
        layer(par(heads=2, kv_heads=1, dim=8, window=300, conv=5), None),
        layer(par(heads=1, kv_heads=1, dim=8, window=3, conv=2),
              moe(3, 2, 8, shared=4)),
    ], width=16, vocab=21, streams=2),
    # heads of 128 on pages of 16: the sizes of the matrix-core attention
    # kernel that long portions take; a window that ends inside a key tile,
    # three query heads per kv head
    "tiles": lambda: config([
        layer(par(heads=6, kv_heads=2, dim=128, window=40, conv=4,
                  temp=(0.3, 32), scale=0.12, rheads=1, rdim=8, rvdim=8),
              moe(4, 2, 16)),
        layer(wkv(heads=2, dim=8), None),
        layer(par(heads=3, kv_heads=1, dim=128, window=0, conv=2, temp=None,
                  scale=0.1, rheads=1, rdim=8, rvdim=8), None),
    ], width=48, vocab=40, streams=2),
    # a window longer than one pass of the attention kernel over the keys
    "long_window": lambda: config([
        layer(par(heads=2, kv_heads=1, dim=8, window=150, conv=3,
                  temp=(0.5, 64), scale=0.5), None),
        layer(wkv(heads=2, dim=8), moe(4, 2, 8, groups=(2, 1))),
    ], width=16, vocab=19, streams=2),
}


def weights(cfg, seed=0, rank=6):
    """Random checkpoint for a config dictionary, bf16 like a stored one."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    V = cfg["vocab"]
    S = cfg.get("streams") or 0

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(
            torch.bfloat16)

    t = {"embed": r(V, W), "final.norm": r(W, std=0.2, mean=1.0),
         "head": r(V, W, std=W ** -0.5)}
    if cfg.get("max_positions"):
        t["pos"] = r(cfg["max_positions"], W, std=0.5)
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = L["mixer"]
        for q in ("1", "2") if L["mlp"] else ("1",):
            t[p + "norm" + q] = r(W, std=0.2, mean=0.7)
            if S:
                t[p + f"hc{q}.in"] = r(S, std=0.3, mean=1.0 / S)
                t[p + f"hc{q}.out"] = r(S, std=0.3, mean=0.8)
                t[p + f"hc{q}.mix"] = (torch.eye(S) + torch.randn(
                    S, S, generator=g) * 0.2).to(torch.bfloat16)
        q = p + "mix."
        if L["type"] == "wkv":
            C = m["heads"] * m["dim"]
            for n in "rkvgw":
                t[q + "mu." + n] = torch.rand(W, generator=g).to(
                    torch.bfloat16)
            for n in "rkvg":
                t[q + n] = r(C, W, std=1.5 * W ** -0.5)
            t[q + "w1"] = r(rank, W, std=W ** -0.5)
            t[q + "w2"] = r(C, rank, std=rank ** -0.5)
            t[q + "w0"] = r(C, std=0.7, mean=-1.0)
            t[q + "u"] = r(m["heads"], m["dim"], std=0.5)
            t[q + "norm"] = r(C, std=0.2, mean=1.0)
            t[q + "o"] = r(W, C, std=C ** -0.5)
        else:
            a, b = m["left"], m["right"]
            Cq, Ck = a["heads"] * a["dim"], a["kv_heads"] * a["dim"]
            t[q + "left.q"] = r(Cq, W, std=1.5 * W ** -0.5)
            t[q + "left.k"] = r(Ck, W, std=1.5 * W ** -0.5)
            if a.get("conv"):
                t[q + "left.q.conv"] = r(Cq, a["conv"], std=0.4, mean=0.4)
                t[q + "left.k.conv"] = r(Ck, a["conv"], std=0.4, mean=0.4)
            t[q + "left.g"] = r(Cq, W, std=2.0 * W ** -0.5)
            t[q + "left.o"] = r(W, Cq, std=Cq ** -0.5)
            H, d, dv = b["heads"], b["dim"], b["vdim"]
            t[q + "right.q"] = r(H * d, W, std=2.0 * W ** -0.5)
            t[q + "right.k"] = r(H * d, W, std=W ** -0.5)
            t[q + "right.v"] = r(H * dv, W, std=W ** -0.5)
            t[q + "right.g"] = r(H * dv, W, std=2.0 * W ** -0.5)
            t[q + "right.a1"] = r(rank, W, std=W ** -0.5)
            t[q + "right.a2"] = r(H * d, rank, std=2.0 * rank ** -0.5)
            t[q + "right.a2.b"] = r(H * d, std=1.0, mean=1.0)
            t[q + "right.norm"] = r(dv, std=0.2, mean=1.0)
            t[q + "right.o"] = r(W, H * dv, std=(H * dv) ** -0.5)
        f = L["mlp"]
        if not f:
            continue
        q = p + "mlp."
        E, ff = f["router"]["experts"], f["expert"]["ff"]
        t[q + "router"] = r(E, W, std=3.0 * W ** -0.5)
        names = [f"e{e}." for e in range(E)]
        sizes = [ff] * E
        if f.get("shared"):
            names.append("shared.")
            sizes.append(f["shared"]["ff"])
        for n, sz in zip(names, sizes):
            t[q + n + "gate"] = r(sz, W, std=2.0 * W ** -0.5)
            t[q + n + "up"] = r(sz, W, std=2.0 * W ** -0.5)
            t[q + n + "down"] = r(W, sz, std=sz ** -0.5)
    return t


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def _poison(eng):
    # whatever a sequence has not written itself must never be read
    for t in list(eng.kv.k) + list(eng.kv.v):
        if t is not None and t.numel():
            t.fill_(300.0)
    for st in eng.states.layers:
        for piece in (st if isinstance(st, tuple) else (st,)):
            if piece is not None:
                piece.fill_(-700.0)


def make_engine(cfg, tensors, device, dtype, blocks=96, slots=4,
                block_size=4, max_len=384, poison=True, **ekw):
    mcfg = BezizenConfig.from_json(cfg)
    model = BezizenModel(mcfg, device=device, dtype=dtype, tensors=tensors,
                         max_position=max_len)
    kw = dict(block_size=block_size, max_model_len=max_len,
              max_sessions=slots, state_slots=slots, num_kv_blocks=blocks,
              use_graphs=False)
    kw.update(ekw)
    eng = LLMEngine(model, mcfg, EngineConfig(**kw), device=device)
    if poison:
        _poison(eng)
    return eng


def tol(dtype):
    return 2e-4 if dtype == "fp32" else 0.08


def row_errors(got, want):
    """Error of every logits row as the ratio of centred root mean
    squares."""
    got = got.detach().cpu().double()
    want = want.detach().cpu().double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() /
            w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).reshape(-1)


def check(got, want, dtype, what=""):
    """fp32: every row within the tolerance. bf16: rounding can flip a close
    call of a router for a single token, which moves that row (and, through
    the carried state, some after it) by much more than rounding does
    elsewhere, so one row in ten (at least one) may be off. With groups a
    flip can exchange ALL experts of a token, in the last layer nearly the
    whole row, so such a row is only held below the distance of unrelated
    rows; a wrong mechanism shows in every row."""
    e = row_errors(got, want)
    if dtype == "fp32":
        assert float(e.max()) <= tol(dtype), \
            f"{what}: error {float(e.max()):.3g} over {tol(dtype)}"
        return
    allowed = max(1, e.numel() // 10)
    over = int((e > tol(dtype)).sum())
    assert over <= allowed and float(e.max()) <= 1.0, \
        f"{what}: {over} rows over {tol(dtype)}, worst {float(e.max()):.3g}"


def logits_of(cfg, W, toks):
    return oracle.forward(toks, W, cfg)


def run_schedule(eng, prompts, schedule):
    """schedule: list of steps, each a list of (request index, count).
    -> per request the logits at every position [len, vocab]. A request is
    freed when it is through."""
    bs = eng.ecfg.block_size
    kvs, at = {}, {}
    out = {i: [] for i in range(len(prompts))}
    for step in schedule:
        entries, want = [], []
        for i, n in step:
            if i not in kvs:
                kvs[i] = SequenceKV(bs)
                at[i] = 0
            entries.append((kvs[i], prompts[i][at[i]: at[i] + n]))
            want.append(list(range(n)))
        lg = eng.forward_tokens(entries, want)
        row = 0
        for i, n in step:
            out[i].append(lg[row: row + n])
            row += n
            at[i] += n
            if at[i] == len(prompts[i]):
                eng.free_sequence(kvs.pop(i))
    return {i: torch.cat(v) for i, v in out.items() if v}


def portions(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out


# ---------------------------------------------------------------- scenarios
def case_whole(name, device, dtype, n=27):
    cfg = CONFIGS[name]()
    W = weights(cfg, 1)
    toks = tokens(cfg, n, 1)
    eng = make_engine(cfg, W, device, dtype, block_size=16 if name == "tiles"
                      else 4)
    got = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
    check(got, logits_of(cfg, W, toks), dtype, name)


def case_layers(device, dtype):
    """The sum of the streams after every layer."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 2)
    toks = tokens(cfg, 11, 2)
    eng = make_engine(cfg, W, device, dtype)
    want = []
    oracle.forward(toks, W, cfg, want)
    kv = SequenceKV(eng.ecfg.block_size)
    got = []
    fwd = eng.model.forward
    eng.model.forward = lambda *a, **k: fwd(*a, taps=got, **k)
    eng.forward_tokens([(kv, toks)])
    eng.model.forward = fwd
    assert len(got) == len(want) == len(cfg["layers"])
    for i, (g, w) in enumerate(zip(got, want)):
        e = float((g.cpu().double() - w).abs().max() / w.abs().max())
        assert e <= tol(dtype), f"layer {i}: {e:.3g}"


def case_prefill_vs_decode(name, device, dtype):
    cfg = CONFIGS[name]()
    W = weights(cfg, 3)
    toks = tokens(cfg, 25, 3)
    want = logits_of(cfg, W, toks)
    whole = run_schedule(make_engine(cfg, W, device, dtype), [toks],
                         [[(0, len(toks))]])[0]
    one = run_schedule(make_engine(cfg, W, device, dtype), [toks],
                       [[(0, 1)] for _ in toks])[0]
    check(whole, want, dtype, "whole")
    check(one, want, dtype, "token by token")
    check(one, whole, dtype, "token by token against whole")


def case_portions(name, device, dtype, sizes, n=41):
    cfg = CONFIGS[name]()
    W = weights(cfg, 4)
    toks = tokens(cfg, n, 4)
    sched = [[(0, k)] for k in portions(len(toks), sizes)]
    got = run_schedule(make_engine(cfg, W, device, dtype), [toks], sched)[0]
    check(got, logits_of(cfg, W, toks), dtype, f"portions {sizes}")


def case_batch(name, device, dtype):
    """Unequal requests in one batch, portions beside single tokens."""
    cfg = CONFIGS[name]()
    W = weights(cfg, 5)
    prompts = [tokens(cfg, n, 10 + n) for n in (19, 1, 7, 30)]
    sched = [
        [(0, 5), (1, 1), (3, 2)],
        [(0, 1), (2, 7), (3, 9)],
        [(3, 1), (0, 1)],
        [(0, 12), (3, 1)],
        [(3, 17)],
    ]
    got = run_schedule(make_engine(cfg, W, device, dtype), prompts, sched)
    for i, p in enumerate(prompts):
        check(got[i], logits_of(cfg, W, p), dtype, f"request {i}")


def case_reuse(device, dtype):
    """A pool too small for all requests at once: pages and state slots of
    finished requests are handed to the next ones."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 6)
    prompts = [tokens(cfg, n, 20 + n) for n in (14, 11, 16, 3, 13)]
    eng = make_engine(cfg, W, device, dtype, blocks=8, slots=2, block_size=4)
    sched = [
        [(0, 6), (1, 4)],
        [(0, 8), (1, 1)],          # 0 ends: 4 pages and a slot come back
        [(1, 6), (2, 9)],          # 1 ends
        [(2, 7), (3, 2)],          # 2 ends
        [(3, 1), (4, 12)],         # 3 ends
        [(4, 1)],
    ]
    got = run_schedule(eng, prompts, sched)
    for i, p in enumerate(prompts):
        check(got[i], logits_of(cfg, W, p), dtype, f"request {i}")
    assert eng.kv.allocator.num_free == 8 and eng.states.num_free == 2


def case_first_tokens(device, dtype):
    """Short sequences started in used pages and slots, and a start cut
    into single tokens."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 7)
    eng = make_engine(cfg, W, device, dtype, slots=1)
    for n, sched in ((1, [1]), (2, [2]), (3, [1, 2]), (9, [1, 1, 1, 2, 4]),
                     (6, [2, 1, 3])):
        toks = tokens(cfg, n, 30 + n)
        got = run_schedule(eng, [toks], [[(0, k)] for k in sched])[0]
        check(got, logits_of(cfg, W, toks), dtype, f"length {n}")


def case_long_decode(device, dtype):
    """Decoding past the windows and through many pages."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 8)
    toks = tokens(cfg, 75, 8)
    sched = [[(0, 3)]] + [[(0, 1)] for _ in range(72)]
    got = run_schedule(make_engine(cfg, W, device, dtype, block_size=4),
                       [toks], sched)[0]
    check(got, logits_of(cfg, W, toks), dtype, "long decode")


def case_long_window(device, dtype):
    """A window longer than one pass of the attention kernel over the keys,
    a prompt longer than the window, portions that end inside it."""
    cfg = CONFIGS["long_window"]()
    W = weights(cfg, 9)
    toks = tokens(cfg, 330, 9)
    want = logits_of(cfg, W, toks)
    eng = make_engine(cfg, W, device, dtype, blocks=200, max_len=400)
    got = run_schedule(eng, [toks], [[(0, 330)]])[0]
    check(got, want, dtype, "whole")
    sched = [[(0, 149)], [(0, 2)], [(0, 146)]] + [[(0, 1)]] * 33
    got = run_schedule(eng, [toks], sched)[0]
    check(got, want, dtype, "portions and decoding")


def case_long_portions(device, dtype):
    """Portions long enough for the matrix-core attention kernel beside
    single tokens, cut inside a window and inside a key tile."""
    cfg = CONFIGS["tiles"]()
    W = weights(cfg, 13)
    prompts = [tokens(cfg, n, 80 + n) for n in (150, 61, 40)]
    want = [logits_of(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, blocks=40, block_size=16,
                      max_len=256)
    sched = [
        [(0, 70), (1, 20)],
        [(0, 1), (1, 41), (2, 39)],
        [(0, 45), (2, 1)],
        [(0, 34)],
    ]
    got = run_schedule(eng, prompts, sched)
    for i in range(3):
        check(got[i], want[i], dtype, f"request {i}")


def case_sorted_experts(device, dtype):
    """Long portions sort their rows by expert and run each expert over its
    rows at once; short steps run every expert on every row. Both against
    the plain model, two requests in the long step."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 12)
    prompts = [tokens(cfg, n, 70 + n) for n in (90, 71)]
    want = [logits_of(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, blocks=64, max_len=128)
    got = run_schedule(eng, prompts, [[(0, 90), (1, 70)], [(1, 1)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"sorted rows, request {i}")


def case_generate(device, dtype, use_graphs=False):
    """Greedy generation through add_request / step against greedy decoding
    with the plain model (a token whose two best logits nearly tie in the
    plain model may differ: generation is compared up to the first such
    place)."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 10)
    prompts = [tokens(cfg, n, 50 + n) for n in (9, 4, 13)]
    new = 12
    eng = make_engine(cfg, W, device, dtype, use_graphs=use_graphs,
                      graph_buckets=(4,), decode_microbatch=4)
    sp = SamplingParams(temperature=0.0, top_k=1, top_p=1.0,
                        max_new_tokens=new)
    kvs = [SequenceKV(eng.ecfg.block_size) for _ in prompts]
    rids = [eng.add_request(kv, p, sp) for kv, p in zip(kvs, prompts)]
    outs = {r: [] for r in rids}
    for _ in range(200):
        if not eng.has_work():
            break
        for o in eng.step():
            outs[o.req_id].extend(o.new_tokens)
    assert not eng.has_work()
    margin = 0.02 if dtype == "fp32" else 0.6
    for rid, p in zip(rids, prompts):
        got = outs[rid]
        assert len(got) == new
        seq = list(p)
        for k in range(new):
            lg = logits_of(cfg, W, seq)[-1]
            top2 = lg.topk(2).values
            if float(top2[0] - top2[1]) < margin:
                break
            assert got[k] == int(lg.argmax()), f"request {rid}, token {k}"
            seq.append(got[k])
    for kv in kvs:
        eng.free_sequence(kv)
    assert eng.kv.allocator.num_free == eng.kv.num_blocks


def assert_greedy(cfg, W, prompt, got, what=""):
    """Every generated token is the plain model's best one, up to the
    rounding of the logits to bfloat16 that the sampler works on."""
    toks = list(prompt)
    for i, t in enumerate(got):
        lg = logits_of(cfg, W, toks)[-1]
        best = float(lg.max())
        assert float(lg[t]) >= best - abs(best) * 2.0 ** -7, \
            f"{what}: token {i} is {t}, the plain model says " \
            f"{int(lg.argmax())}"
        toks.append(t)


def _generate(eng, kv, prompt, n):
    sp = SamplingParams(temperature=0.0, max_new_tokens=n)
    eng.add_request(kv, prompt, sp)
    out = []
    while eng.has_work():
        for o in eng.step():
            out.extend(o.new_tokens)
    return out


def case_multi_turn(device, dtype):
    """A session's second turn continues from its pages and state slot; an
    idle session whose pages and slot were taken away is rebuilt from its
    history."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 15)
    eng = make_engine(cfg, W, device, dtype, blocks=12, slots=2, max_len=64,
                      poison=False, decode_microbatch=2)
    a, b = SequenceKV(4), SequenceKV(4)
    p1, p2, p3 = tokens(cfg, 9, 60), tokens(cfg, 5, 61), tokens(cfg, 30, 62)
    t1 = _generate(eng, a, p1, 4)
    assert_greedy(cfg, W, p1, t1, "first turn")
    t2 = _generate(eng, a, p2, 3)
    assert_greedy(cfg, W, p1 + t1 + p2, t2, "second turn")
    assert a.num_tokens > 0 and a.state_slot >= 0
    tb = _generate(eng, b, p3, 4)       # needs a's pages
    assert_greedy(cfg, W, p3, tb, "other session")
    assert a.num_tokens == 0 and a.state_slot < 0 and a.history
    eng.free_sequence(b)
    t3 = _generate(eng, a, [7, 3], 3)
    assert_greedy(cfg, W, p1 + t1 + p2 + t2 + [7, 3], t3, "rebuilt session")


# ----------------------------------------------------- mechanisms, one by one
def case_window_edges(device, dtype, decode):
    """The attention side alone, one head pair whose query at position p is
    made to point at ONE key: the oldest key inside the window, the first
    one outside it, a key at a page border, the query's own. Values are the
    keys, so with the key visible the output is that key's row; hidden, it
    is not."""
    window, bs = 9, 4
    cfg = config([layer(par(heads=2, kv_heads=1, dim=8, window=window, conv=0,
                            temp=None, scale=6.0, rheads=1, rdim=4, rvdim=4,
                            ls=1.0, rs=0.0), None)],
                 width=16, vocab=64, streams=0, positions=0, embed_scale=1.0)
    W = weights(cfg, 20)
    # embed row v: a component along axis (v % 8) for the key, and one along
    # 8 + (v // 8) that the query projection reads: token v = 8 a + b asks
    # for keys of kind a and is itself a key of kind b
    V, Wd = cfg["vocab"], cfg["width"]
    emb = torch.zeros(V, Wd)
    for v in range(V):
        emb[v, v % 8] = 1.0
        emb[v, 8 + v // 8] = 1.0
    W["embed"] = emb.to(torch.bfloat16)
    W["l0.norm1"] = torch.ones(Wd).to(torch.bfloat16)
    wq = torch.zeros(16, Wd)
    wk = torch.zeros(8, Wd)
    for a in range(8):
        wq[a, 8 + a] = 1.0          # head 0 asks for kind a
        wq[8 + a, 8 + a] = 1.0      # head 1 the same
        wk[a, a] = 1.0
    W["l0.mix.left.q"] = wq.to(torch.bfloat16)
    W["l0.mix.left.k"] = wk.to(torch.bfloat16)
    n = 3 * window + 5
    for target in (0, 3, bs * 2 - 1, bs * 2, window, 2 * window + 1, n - 1):
        # every token is kind 0 and asks for kind 1; only `target` is kind 1
        toks = [8 * 1 + 0] * n
        toks[target] = 8 * 1 + 1
        want = logits_of(cfg, W, toks)
        eng = make_engine(cfg, W, device, dtype, block_size=bs)
        if decode:
            sched = [[(0, 2)]] + [[(0, 1)]] * (n - 2)
        else:
            sched = [[(0, n - 7)], [(0, 7)]]
        got = run_schedule(eng, [toks], sched)[0]
        check(got, want, dtype, f"key {target}")
        # the construction bites: the last row that sees the target differs
        # from the next row, which does not
        last_seen = target + window - 1
        if last_seen + 1 < n:
            a, b = want[last_seen], want[last_seen + 1]
            assert float((a - b).abs().max()) > 0.05


def case_state_carry(device, dtype):
    """Both recurrences with decays pushed to (nearly) one: what the first
    token wrote must survive every cut and reach the last position."""
    cfg = config([layer(wkv(heads=2, dim=8), None),
                  layer(par(heads=1, kv_heads=1, dim=8, window=2, conv=2,
                            rheads=2, rdim=8, rvdim=8, ls=0.1, rs=2.0),
                        None)],
                 width=16, vocab=32, streams=2)
    W = weights(cfg, 22)
    W["l0.mix.w0"] = torch.full_like(W["l0.mix.w0"], -12.0)
    W["l1.mix.right.a2.b"] = torch.full_like(W["l1.mix.right.a2.b"], 12.0)
    n = 120
    toks = tokens(cfg, n, 22)
    want = logits_of(cfg, W, toks)
    other = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    far = logits_of(cfg, W, other)
    assert float((far[-1] - want[-1]).abs().max()) > 0.05
    eng = make_engine(cfg, W, device, dtype, blocks=64, max_len=128)
    for sched in ([n], [1, 2, 70] + [1] * 47, [50, 33, 2, 35]):
        got = run_schedule(eng, [toks], [[(0, k)] for k in sched])[0]
        check(got, want, dtype, f"cuts {sched[:4]}")


def case_router(device, dtype):
    """Routed experts alone against the plain model: groups, every `top`,
    rows in both forms of the expert pass."""
    from kukeon_amd.models.feedforward import FFCfg, RoutedMoE
    Wd = 24
    for E, top, groups, shared, T in ((6, 2, (3, 2), 8, 5), (8, 3, (2, 1), 0, 70),
                                      (4, 4, None, 6, 66), (5, 1, None, 0, 3)):
        f = moe(E, top, 10, groups=groups, scale=1.3, shared=shared)
        cfg = config([layer(wkv(), f)], width=Wd)
        W = weights(cfg, 30 + E)
        t64 = {k: v.double() for k, v in W.items()}
        g = torch.Generator().manual_seed(E)
        h = torch.randn(T, Wd, generator=g).to(torch.bfloat16)
        want = oracle.moe(h.double(), t64, "l0.mlp.", f)
        fc = BezizenConfig.from_json(cfg).layers[0].mlp
        act = torch.float32 if dtype == "fp32" else torch.bfloat16
        mod = RoutedMoE(fc, Wd, W, "l0.mlp.", device, act)

        class Meta:
            host_ids = list(range(T))
        got = mod(h.to(device=device, dtype=act), None, Meta())
        check(got, want, dtype, f"experts {E} top {top}")


# ------------------------------------------------------- single operations
def _act(dtype):
    return torch.float32 if dtype == "fp32" else torch.bfloat16


def _close(got, want, dtype, what):
    got = got.detach().cpu().double()
    want = want.detach().cpu().double()
    lim = (1e-5 if dtype == "fp32" else 2e-2) * \
        max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= lim, f"{what}: {err:.3g} over {lim:.3g}"


def _maps(cuts, start, device, slots):
    pos, row_seq, cu = [], [], [0]
    for s, (n, p0) in enumerate(zip(cuts, start)):
        pos += list(range(p0, p0 + n)) if p0 >= 0 else [-1] * n
        row_seq += [s] * n
        cu.append(cu[-1] + n)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    return i32(pos), i32(row_seq), i32(cu), i32(slots)


def case_op_streams(device, dtype):
    """Read, and write followed by the next read, for one to five streams
    and widths on and off the vector path."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(5)
    for S, Wd in ((1, 16), (3, 40), (4, 128), (5, 26)):
        T = 7
        xs = torch.randn(T, S, Wd, generator=g)
        y = torch.randn(T, Wd, generator=g).to(_act(dtype))
        mix = torch.randn(S, S, generator=g)
        outc = torch.randn(S, generator=g)
        coef = torch.randn(S, generator=g)
        w = torch.randn(Wd, generator=g)
        rows = [xs[:, s].double() for s in range(S)]
        want_r = oracle.unit_rms(oracle.streams_read(rows, coef.double()),
                                 1e-5) * w.double()
        new = oracle.streams_write(rows, y.double(), mix.double(),
                                   outc.double())
        want_w = oracle.unit_rms(oracle.streams_read(new, coef.double()),
                                 1e-5) * w.double()
        d = lambda t: t.to(device)
        xd = d(xs.clone())
        out = torch.empty(T, Wd, dtype=_act(dtype), device=device)
        ops.stream_read_norm(out, xd, d(coef), d(w), 1e-5)
        _close(out, want_r, dtype, f"read {S}")
        ops.stream_write_read_norm(xd, d(y), d(mix), d(outc), d(coef), d(w),
                                   1e-5, out)
        _close(out, want_w, dtype, f"write {S}")
        _close(xd, torch.stack(new, 1), "fp32", f"streams {S}")


def case_op_shift(device, dtype):
    """Token shift over portions with a dirty slot, a sequence at its start
    and an inactive neighbour; then single rows that move the slot
    themselves."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(6)
    Wd, N = 24, 3
    mu = torch.rand(N, Wd, generator=g)
    seqs = [torch.randn(9, Wd, generator=g).to(_act(dtype)) for _ in range(2)]
    state = torch.full((4, Wd), -700.0, device=device)
    for cuts in ((4, 1, 4), (1, 1, 7)):
        at = 0
        got = [[], []]
        for n in cuts:
            h = torch.cat([seqs[0][at: at + n], torch.zeros(2, Wd).to(
                _act(dtype)), seqs[1][at: at + n]]).to(device)
            pos, row_seq, cu, slots = _maps([n, 2, n], [at, -1, at], device,
                                            [2, 1, 0])
            out = torch.full((N, h.shape[0], Wd), 9.0, dtype=_act(dtype),
                             device=device)
            one = n == 1
            # (an inactive sequence of two rows keeps the step off the
            # single-row form; run the live ones alone for it)
            if one:
                h = torch.cat([seqs[0][at: at + 1], seqs[1][at: at + 1]]).to(
                    device)
                pos, row_seq, cu, slots = _maps([1, 1], [at, at], device,
                                                [2, 0])
                out = torch.empty(N, 2, Wd, dtype=_act(dtype), device=device)
            ops.token_shift(out, h, mu.to(device), state, pos, row_seq, cu,
                            slots, one)
            if not one:
                ops.token_shift_tail(state, h, pos, cu, slots)
            got[0].append(out[:, :n])
            got[1].append(out[:, -n:])
            at += n
        for k in range(2):
            full = seqs[k].double()
            before = torch.cat([torch.zeros(1, Wd, dtype=torch.float64),
                                full[:-1]])
            want = full[None] + (before - full)[None] * mu.double()[:, None]
            _close(torch.cat(got[k], 1), want, dtype, f"sequence {k}")


def case_op_scan(device, dtype, mode=0, H=3, d=5, dv=7, cuts=(4, 1, 9, 1, 1)):
    """The recurrence with a decay per key channel over portions with a
    dirty slot and an inactive neighbour."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(7 + d)
    n = sum(cuts)
    act = _act(dtype)
    q = torch.randn(n, H * d, generator=g).to(act)
    k = (torch.randn(n, H * d, generator=g) * 0.5).to(act)
    v = torch.randn(n, H * dv, generator=g).to(act)
    R = 3
    lo = torch.randn(n, R, generator=g)
    w2 = torch.randn(H * d, R, generator=g) * 0.6
    z = (torch.tanh(lo.double()) if mode == 0 else lo.double()) @ \
        w2.double().T
    zb = torch.randn(H * d, generator=g) - (1.0 if mode == 0 else -1.0)
    bonus = torch.randn(H * d, generator=g)
    tau, qs = 3.0, d ** -0.5 if mode else 1.0
    # plain recurrence
    want = torch.zeros(n, H, dv, dtype=torch.float64)
    zz = (z.double() + zb.double()).view(n, H, d)
    a = torch.exp(-torch.exp(zz)) if mode == 0 else \
        torch.sigmoid(zz) ** (1.0 / tau)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=torch.float64)
        for i in range(n):
            qi = q[i].double().view(H, d)[hd] * qs
            ki = k[i].double().view(H, d)[hd]
            vi = v[i].double().view(H, dv)[hd]
            kv = torch.outer(ki, vi)
            if mode == 0:
                want[i, hd] = (S + bonus.double().view(H, d)[hd][:, None] *
                               kv).T @ qi
                S = a[i, hd][:, None] * S + kv
            else:
                S = a[i, hd][:, None] * S + kv
                want[i, hd] = S.T @ qi
    state = torch.full((3, H, dv, d), -700.0, device=device)
    got, at = [], 0
    dd = lambda t: t.to(device)
    for c in cuts:
        pad = lambda t: torch.cat([t[at: at + c], torch.ones(2, t.shape[1],
                                                           dtype=t.dtype)])
        pos, _, cu, slots = _maps([c, 2], [at, -1], device, [1, 0])
        y = torch.full((c + 2, H * dv), 5.0, device=device)
        ops.decay_scan(y, dd(pad(q)), dd(pad(k)), dd(pad(v)), dd(pad(lo)),
                       dd(w2), dd(zb), dd(bonus) if mode == 0 else None,
                       state, pos,
                       cu, slots, H, d, dv, mode, tau, qs)
        assert float(y[c:].abs().max()) == 0.0
        got.append(y[:c])
        at += c
    assert float(state[0].min()) == -700.0 and float(state[2].min()) == -700.0
    _close(torch.cat(got), want.view(n, H * dv), dtype, "scan")


def case_op_router(device, dtype="fp32"):
    """Group-limited choice and weights, ties and equal logits included."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(8)
    for E, top, groups, keep in ((8, 3, 4, 2), (6, 2, 0, 0), (12, 4, 3, 2),
                                 (4, 4, 2, 2), (16, 1, 16, 1)):
        z = torch.randn(40, E, generator=g)
        z[3] = 0.25                      # all equal: the lowest indices win
        z[5, :] = z[5, 0]
        z[7, E - 1] = z[7].max()         # a tie between two experts
        idx = torch.zeros(40, top + 1, dtype=torch.int32, device=device)
        wts = torch.zeros(40, top + 1, device=device)
        idx[:, top] = -5
        ops.router_select(idx, wts, z.to(device), top, groups, keep, 1.7, 0)
        r = {"experts": E, "top": top, "scale": 1.7}
        if groups:
            r["groups"] = {"count": groups, "keep": keep}
        pick, w = oracle.route(z.double(), {"x.router": torch.eye(
            E, dtype=torch.float64)}, "x.", r)
        assert torch.equal(idx[:, :top].cpu().long(), pick)
        assert int(idx[:, top].max()) == -5
        _close(wts[:, :top], w, "fp32", f"weights {E}")


# ------------------------------------------------- folders, programs, servers
def case_registry(tmp_path, device, dtype):
    """A checkpoint folder is found by its architecture name and read."""
    from dumovik_cases import write_checkpoint
    from kukeon_amd.models.registry import load_checkpoint
    cfg = CONFIGS["one_stream"]()
    W = weights(cfg, 11, rank=3)
    write_checkpoint(tmp_path, cfg, W)
    mcfg, model = load_checkpoint(str(tmp_path), device=device, dtype=dtype)
    assert mcfg.family == "bezizen" and len(model.layers) == 2
    eng = LLMEngine(model, mcfg, EngineConfig(
        block_size=4, max_model_len=64, max_sessions=2, state_slots=2,
        num_kv_blocks=16, use_graphs=False), device=device)
    toks = tokens(cfg, 13, 11)
    got = run_schedule(eng, [toks], [[(0, 6)], [(0, 7)]])[0]
    check(got, logits_of(cfg, W, toks), dtype, "from a folder")


def case_trace_runner(tmp_path, device, dtype):
    """The trace runner as a program: a checkpoint folder, steps on standard
    input, logits files and `done` lines back. Three requests through a pool
    sized for two, portions beside single tokens, a request left out of a
    step."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from dumovik_cases import write_checkpoint
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 14)
    model_dir = tmp_path / "model"
    out_dir = tmp_path / "out"
    model_dir.mkdir()
    write_checkpoint(model_dir, cfg, W)
    prompts = {"a": tokens(cfg, 70, 90), "b": tokens(cfg, 40, 91),
               "c": tokens(cfg, 33, 92)}
    want = {k: logits_of(cfg, W, p) for k, p in prompts.items()}
    steps = [[("a", 30), ("b", 1)], [("a", 1), ("b", 38)], [("a", 39)],
             [("b", 1), ("c", 2)], [("c", 30)], [("c", 1)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
           str(model_dir), "--dtype",
           "float32" if dtype == "fp32" else "bfloat16", "--out",
           str(out_dir), "--max-tokens", "128", "--slots", "2", "--device",
           device]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True, cwd=root)
    at = {k: 0 for k in prompts}
    try:
        for n, step in enumerate(steps):
            entries, end = [], []
            for k, cnt in step:
                toks = prompts[k][at[k]: at[k] + cnt]
                entries.append({"id": k, "tokens": toks,
                                "want": [0, cnt - 1] if cnt > 1 else [0]})
                at[k] += cnt
                if at[k] == len(prompts[k]):
                    end.append(k)
            p.stdin.write(json.dumps({"step": n, "entries": entries,
                                      "end": end}) + "\n")
            p.stdin.flush()
            line = p.stdout.readline()
            while line and line.strip() != "done %d" % n:
                line = p.stdout.readline()
            assert line, "the runner ended early"
            got = np.fromfile(out_dir / ("%d.f32" % n), dtype="<f4").reshape(
                -1, cfg["vocab"])
            row = 0
            for k, cnt in step:
                a = at[k] - cnt
                for w in ([0, cnt - 1] if cnt > 1 else [0]):
                    check(torch.from_numpy(got[row].copy())[None],
                          want[k][a + w][None], dtype, f"step {n} {k}+{w}")
                    row += 1
            assert row == got.shape[0]
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()


def case_modelhub(device):
    """The serving daemon's model server with this family: sessions over the
    unix socket, two turns on one session, greedy tokens as the plain model
    gives them."""
    import uuid
    from kukeon_amd.serve.server import ModelhubClient, ModelhubServer
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 16)
    mcfg = BezizenConfig.from_json(cfg)
    model = BezizenModel(mcfg, device=device, dtype="fp32", tensors=W,
                         max_position=128)
    ecfg = EngineConfig(block_size=4, max_model_len=128, max_sessions=4,
                        state_slots=4, num_kv_blocks=64, use_graphs=False)
    sock = f"/tmp/mh-{uuid.uuid4().hex[:10]}.sock"
    hub = ModelhubServer(model, mcfg, ecfg, sock, device=device)
    hub.start()
    try:
        c = ModelhubClient(sock, timeout=120)
        p1, p2 = tokens(cfg, 6, 70), tokens(cfg, 3, 71)
        r1 = c.generate("s", p1, max_new_tokens=4, temperature=0.0)
        assert len(r1["tokens"]) == 4
        assert_greedy(cfg, W, p1, r1["tokens"], "first turn")
        r2 = c.generate("s", p2, max_new_tokens=3, temperature=0.0)
        assert len(r2["tokens"]) == 3
        assert_greedy(cfg, W, p1 + r1["tokens"] + p2, r2["tokens"],
                      "second turn")
        rb = c.generate("t", p2, max_new_tokens=2, temperature=0.0)
        assert_greedy(cfg, W, p2, rb["tokens"], "other session")
        assert c.call("stats")["sessions"] == 2
        c.close()
    finally:
        hub.stop()


def case_real_sizes(device, say=lambda s: None):
    """A stack at the layer sizes of a served model (heads of 128, pages of
    16, rows of thousands of entries): the bf16 serving kernels against the
    exact fp32 kernels, prompts on the packed path and decoding under
    hipGraphs."""
    from kukeon_amd.models.bezizen import bezizen_bench, random_tensors
    mcfg = bezizen_bench(width=2048, layers=4, heads=16, kv_heads=4, ff=4096,
                         vocab=512, window=96, experts=16, streams=4,
                         max_positions=512, name="bezizen-sizes")
    W = random_tensors(mcfg, 5)
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist()
               for n in (150, 70, 129)]
    outs = {}
    for dtype in ("fp32", "bf16"):
        say(f"model {dtype}")
        model = BezizenModel(mcfg, device=device, dtype=dtype, tensors=W)
        eng = LLMEngine(model, mcfg, EngineConfig(
            block_size=16, max_model_len=512, max_sessions=4, state_slots=4,
            num_kv_blocks=64, use_graphs=False), device=device)
        say("prompts")
        kvs = [SequenceKV(16) for _ in prompts]
        lg = [eng.forward_tokens([(kv, p[:-6]) for kv, p in
                                  zip(kvs, prompts)])]
        say("single tokens")
        for k in range(6, 0, -1):
            lg.append(eng.forward_tokens([(kv, [p[-k]]) for kv, p in
                                          zip(kvs, prompts)]))
        outs[dtype] = torch.cat(lg).float().cpu()
        assert bool(torch.isfinite(outs[dtype]).all())
        for kv in kvs:
            eng.free_sequence(kv)
        if dtype == "bf16":
            say("generation under graphs")
            eng.ecfg.use_graphs = True
            eng.ecfg.graph_buckets = (4,)
            eng.ecfg.decode_microbatch = 8
            sp = SamplingParams(temperature=0.7, top_k=50, top_p=0.9,
                                max_new_tokens=17)
            kvs = [SequenceKV(16) for _ in prompts]
            rids = [eng.add_request(kv, p, sp) for kv, p in
                    zip(kvs, prompts)]
            n = 0
            while eng.has_work():
                for o in eng.step():
                    n += len(o.new_tokens)
                    assert all(0 <= t < 512 for t in o.new_tokens)
            assert n == 17 * len(rids)
        del eng, model
    e = row_errors(outs["bf16"], outs["fp32"])
    over = int((e > 0.15).sum())
    assert over <= max(1, e.numel() // 4), f"{over} rows off, worst " \
        f"{float(e.max()):.3g}"
