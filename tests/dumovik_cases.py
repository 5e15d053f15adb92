"""Scenarios for the Dumovik family, run by the CPU tests (reference ops,
fp32) and the GPU tests (HIP kernels, fp32 and bf16). Every scenario builds
a small configuration with random weights, runs it through the engine and
compares with the plain model in dumovik_oracle.py."""
import torch

import dumovik_oracle as oracle
from kukeon_amd.engine.config import EngineConfig, SamplingParams
from kukeon_amd.engine.engine import LLMEngine
from kukeon_amd.engine.kv_cache import SequenceKV
from kukeon_amd.models.dumovik import DumovikConfig, DumovikModel


def attn(heads=4, kv_heads=2, dim=8, vdim=6, chunk=7, softcap=5.0,
         scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale if scale is not None else 2.0 * dim ** -0.5}
    if chunk:
        m["mask"] = {"size": chunk}
    if softcap:
        m["softcap"] = softcap
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def latent(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=24, base=100.0,
           scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim,
                      "vdim": vdim, "kv_rank": kv_rank,
                      "rot": {"dims": rot_dim, "base": base},
                      "scale": scale if scale is not None
                      else (dim + rot_dim) ** -0.5}}


def lightning(heads=3, dim=8, vdim=6, decay=None):
    decay = decay or [0.5 + 0.45 * h / max(1, heads - 1)
                      for h in range(heads)]
    return {"type": "lightning",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim,
                      "decay": decay}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top}}


def layer(mix, mlp):
    return dict(mix, mlp=mlp)


def config(layers, width=40, vocab=45, eps=1e-5):
    return {"architecture": "Dumovik", "width": width, "vocab": vocab,
            "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    # all three mixers, both feed-forwards, a layer without one, a layer
    # that reads an earlier layer's keys
    "hybrid": lambda: config([
        layer(attn(), dense(56)),
        layer(lightning(), moe(5, 2, 12)),
        layer(latent(), None),
        layer(attn(kv_from=0, chunk=5, softcap=3.0), moe(4, 3, 9)),
        layer(lightning(heads=2, dim=20, vdim=12, decay=[0.9975, 0.3]),
              dense(33)),
    ]),
    # rows of whole 16-byte pieces everywhere (the vector forms of the
    # kernels), five query heads on one kv head, six heads on a latent head
    # group of four, one expert per token, state rows spread over lanes
    "aligned": lambda: config([
        layer(lightning(heads=2, dim=64, vdim=40), moe(4, 1, 64)),
        layer(attn(heads=5, kv_heads=1, dim=16, vdim=48, chunk=20),
              dense(128)),
        layer(latent(heads=6, dim=16, rot_dim=8, vdim=16, kv_rank=32),
              moe(3, 2, 128)),
        layer(attn(heads=5, kv_heads=1, dim=16, vdim=48, chunk=33,
                   softcap=0, kv_from=1), None),
    ], width=128, vocab=50, eps=1e-3),
    # no chunks and no cap (plain causal attention), heads == kv_heads,
    # every expert chosen, a chunk of one, a decay of exactly one, a width
    # that is not a multiple of 8
    "plain": lambda: config([
        layer(attn(heads=2, kv_heads=2, dim=6, vdim=5, chunk=0, softcap=0),
              moe(3, 3, 10)),
        layer(attn(heads=3, kv_heads=1, dim=4, vdim=4, chunk=1), None),
        layer(lightning(heads=1, dim=5, vdim=7, decay=[1.0]), dense(20)),
    ], width=26, vocab=31),
    # no attention at all (no cache pages), and no recurrence (no state)
    "only_lightning": lambda: config([
        layer(lightning(heads=2, dim=4, vdim=4), dense(20)),
        layer(lightning(heads=1, dim=40, vdim=3, decay=[0.9]), None),
    ], width=16, vocab=21),
    "only_attention": lambda: config([
        layer(latent(heads=2, dim=4, rot_dim=4, vdim=4, kv_rank=8),
              moe(3, 2, 8)),
        layer(attn(heads=2, kv_heads=1, dim=8, vdim=8, chunk=300), None),
        layer(latent(heads=1, dim=8, rot_dim=2, vdim=3, kv_rank=16), None),
    ], width=16, vocab=21),
    # heads of 128 on pages of 16: the sizes of the matrix-core attention
    # kernel that long portions take; chunks that end inside a key tile, a
    # sharing layer without chunks or cap, three query heads per kv head
    "tiles": lambda: config([
        layer(attn(heads=6, kv_heads=2, dim=128, vdim=128, chunk=40,
                   softcap=6.0, scale=0.3), dense(48)),
        layer(lightning(heads=2, dim=8, vdim=8), None),
        layer(attn(heads=6, kv_heads=2, dim=128, vdim=128, chunk=0,
                   softcap=0, scale=0.2, kv_from=0), None),
    ], width=48, vocab=40),
    # a chunk longer than one pass of the attention kernel over the keys
    "long_chunk": lambda: config([
        layer(attn(heads=2, kv_heads=1, dim=8, vdim=8, chunk=150,
                   softcap=4.0), None),
        layer(lightning(heads=2, dim=8, vdim=8, decay=[0.99, 0.9]),
              dense(24)),
    ], width=16, vocab=19),
}


def weights(cfg, seed=0):
    """Random checkpoint for a config dictionary, bf16 like a stored one."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    V = cfg["vocab"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(
            torch.bfloat16)

    t = {"embed": r(V, W), "final.norm": r(W, std=0.2, mean=1.0)}
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = L["mixer"]
        t[p + "norm1"] = r(W, std=0.2, mean=0.7)
        q = p + "mix."
        if L["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[q + "q"] = r(H * d, W, std=W ** -0.5)
            t[q + "q.norm"] = r(H * d, std=0.3, mean=1.5)
            t[q + "o"] = r(W, H * dv, std=(H * dv) ** -0.5)
            if m.get("kv_from") is None:
                t[q + "k"] = r(G * d, W, std=W ** -0.5)
                t[q + "k.norm"] = r(G * d, std=0.3, mean=1.5)
                t[q + "v"] = r(G * dv, W, std=W ** -0.5)
        elif L["type"] == "latent_attention":
            H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R = m["kv_rank"]
            t[q + "q"] = r(H * (dn + dr), W, std=2.0 * W ** -0.5)
            t[q + "dkv"] = r(R + dr, W, std=W ** -0.5)
            t[q + "dkv.norm"] = r(R, std=0.2, mean=1.0)
            t[q + "uk"] = r(H * dn, R, std=2.0 * R ** -0.5)
            t[q + "uv"] = r(H * dv, R, std=R ** -0.5)
            t[q + "g"] = r(H * dv, W, std=2.0 * W ** -0.5)
            t[q + "o"] = r(W, H * dv, std=(H * dv) ** -0.5)
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            t[q + "q"] = r(H * d, W, std=W ** -0.5)
            t[q + "k"] = r(H * d, W, std=W ** -0.5)
            t[q + "v"] = r(H * dv, W, std=W ** -0.5)
            t[q + "g"] = r(H * dv, W, std=2.0 * W ** -0.5)
            t[q + "norm"] = r(H * dv, std=0.2, mean=1.0)
            t[q + "o"] = r(W, H * dv, std=(H * dv) ** -0.5)
        f = L["mlp"]
        if not f:
            continue
        t[p + "norm2"] = r(W, std=0.2, mean=0.7)
        q = p + "mlp."
        if f["kind"] == "dense":
            t[q + "gate"] = r(f["ff"], W, std=1.5 * W ** -0.5)
            t[q + "up"] = r(f["ff"], W, std=1.5 * W ** -0.5)
            t[q + "down"] = r(W, f["ff"], std=f["ff"] ** -0.5)
        else:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            t[q + "router"] = r(E, W, std=3.0 * W ** -0.5)
            for e in range(E):
                t[q + f"e{e}.gate"] = r(ff, W, std=2.0 * W ** -0.5)
                t[q + f"e{e}.up"] = r(ff, W, std=2.0 * W ** -0.5)
                t[q + f"e{e}.down"] = r(W, ff, std=ff ** -0.5)
    return t


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def _poison(eng):
    # whatever a sequence has not written itself must never be read
    for t in list(eng.kv.k) + list(eng.kv.v):
        if t is not None:
            t.fill_(300.0)
    for st in eng.states.layers:
        if st is not None:
            st.fill_(-700.0)


def make_engine(cfg, tensors, device, dtype, blocks=96, slots=4,
                block_size=4, max_len=384, poison=True, **ekw):
    mcfg = DumovikConfig.from_json(cfg)
    model = DumovikModel(mcfg, device=device, dtype=dtype, tensors=tensors,
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
    call of a router for a single token, which moves that row by much more
    than rounding does elsewhere, so one row in ten (at least one) may be
    off, though never as far as a wrong mechanism puts it."""
    e = row_errors(got, want)
    if dtype == "fp32":
        assert float(e.max()) <= tol(dtype), \
            f"{what}: error {float(e.max()):.3g} over {tol(dtype)}"
        return
    allowed = max(1, e.numel() // 10)
    over = int((e > tol(dtype)).sum())
    assert over <= allowed and float(e.max()) <= 0.5, \
        f"{what}: {over} rows over {tol(dtype)}, worst {float(e.max()):.3g}"


def logits_of(cfg, W, toks):
    return oracle.forward(cfg, W, toks)[0]


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
    eng = make_engine(cfg, W, device, dtype)
    got = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
    check(got, logits_of(cfg, W, toks), dtype, name)


def case_layers(device, dtype):
    """The residual stream after every layer."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 2)
    toks = tokens(cfg, 11, 2)
    eng = make_engine(cfg, W, device, dtype)
    want = oracle.forward(cfg, W, toks)[1]
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
    """Decoding through many chunks and pages."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 8)
    toks = tokens(cfg, 75, 8)
    sched = [[(0, 3)]] + [[(0, 1)] for _ in range(72)]
    got = run_schedule(make_engine(cfg, W, device, dtype, block_size=4),
                       [toks], sched)[0]
    check(got, logits_of(cfg, W, toks), dtype, "long decode")


def case_long_chunk(device, dtype):
    """A chunk longer than one pass of the attention kernel over the keys,
    a prompt longer than the chunk, portions that end inside it."""
    cfg = CONFIGS["long_chunk"]()
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
    short ones and single tokens that take the other form; cuts inside a
    chunk and inside a key tile."""
    cfg = CONFIGS["tiles"]()
    W = weights(cfg, 13)
    prompts = [tokens(cfg, n, 80 + n) for n in (300, 70)]
    want = [logits_of(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, blocks=30, block_size=16,
                      max_len=400)
    got = run_schedule(eng, prompts, [[(0, 300), (1, 69)], [(1, 1)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"whole, request {i}")
    got = run_schedule(eng, prompts,
                       [[(0, 21)], [(0, 270), (1, 2)], [(0, 1), (1, 68)],
                        [(0, 8)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"portions, request {i}")


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


# ----------------------------------------------------- mechanisms, one by one
def case_chunk_edges(device, dtype, decode):
    """One attention head whose query at position p is made to point at ONE
    key: the first key of p's chunk, the last key of the chunk before (which
    must not be seen), a key at a page border, the query's own. With the
    key visible the output is that key's value row; hidden, it is not."""
    chunk, bs = 12, 4
    cfg = config([layer(attn(heads=2, kv_heads=1, dim=8, vdim=8, chunk=chunk,
                             softcap=30.0, scale=1.0), None)],
                 width=16, vocab=64)
    W = weights(cfg, 20)
    # embed row v: a strong component along axis (v % 8) for the key, and
    # the query projection reads axis 8 + (v // 8): token v = 8 a + b asks
    # for keys of kind a and is itself a key of kind b
    V, Wd = cfg["vocab"], cfg["width"]
    emb = torch.zeros(V, Wd)
    for v in range(V):
        emb[v, v % 8] = 1.0
        emb[v, 8 + v // 8] = 1.0
    W["embed"] = emb.to(torch.bfloat16)
    wq = torch.zeros(16, Wd)
    wk = torch.zeros(8, Wd)
    wv = torch.zeros(8, Wd)
    for a in range(8):
        wq[a, 8 + a] = 1.0          # head 0 asks for kind a
        wq[8 + a, 8 + a] = 1.0      # head 1 the same
        wk[a, a] = 1.0
        wv[a, a] = 1.0
    W["l0.mix.q"] = wq.to(torch.bfloat16)
    W["l0.mix.k"] = wk.to(torch.bfloat16)
    W["l0.mix.v"] = wv.to(torch.bfloat16)
    W["l0.mix.q.norm"] = torch.full((16,), 16.0).to(torch.bfloat16)
    W["l0.mix.k.norm"] = torch.full((8,), 4.0).to(torch.bfloat16)
    n = 3 * chunk + 5
    for target in (chunk, chunk - 1, 2 * chunk, 2 * chunk - 1, bs * 5,
                   bs * 5 - 1, n - 1):
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
        # the construction bites: rows that see the target differ from rows
        # of the next chunk, which do not
        last_seen = min(n - 1, (target // chunk + 1) * chunk - 1)
        if last_seen + 1 < n:
            a, b = want[last_seen], want[last_seen + 1]
            assert float((a - b).abs().max()) > 0.05


def case_far_latent_key(device, dtype, decode):
    """Latent attention: among hundreds of keys one far back carries the
    only large score (its rotated key part is scaled up); prompts and
    decoded tokens must find it."""
    cfg = config([layer(latent(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=16,
                               scale=1.0), None)], width=16, vocab=32)
    W = weights(cfg, 21)
    W["l0.mix.uk"] = (W["l0.mix.uk"].float() * 3.0).to(torch.bfloat16)
    n = 300
    toks = tokens(cfg, n, 21)
    want = logits_of(cfg, W, toks)
    eng = make_engine(cfg, W, device, dtype, blocks=100, max_len=400)
    sched = ([[(0, 260)]] + [[(0, 1)]] * 40) if decode else \
        [[(0, 200)], [(0, 100)]]
    got = run_schedule(eng, [toks], sched)[0]
    check(got, want, dtype, "far key")


def case_state_carry(device, dtype):
    """Linear attention with a decay of one: the first token's key and value
    stay in the state for ever, so every later output depends on a state
    that was carried through every cut, slot and step."""
    cfg = config([layer(lightning(heads=2, dim=8, vdim=8,
                                  decay=[1.0, 0.97]), None)],
                 width=16, vocab=32)
    W = weights(cfg, 22)
    prompts = [tokens(cfg, n, 80 + n) for n in (120, 57)]
    want = [logits_of(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, slots=2)
    sched = [[(0, 50), (1, 2)], [(0, 2), (1, 30)], [(0, 1), (1, 1)]] + \
        [[(0, 1), (1, 1)]] * 24 + [[(0, 67 - 24)]]
    got = run_schedule(eng, prompts, sched)
    for i in range(2):
        check(got[i], want[i], dtype, f"request {i}")


def case_router(device, dtype):
    """Routed experts alone against the plain model: every `top`, rows in
    the dense and in the sorted form."""
    for top in (1, 2, 4):
        cfg = config([layer(lightning(heads=1, dim=4, vdim=4, decay=[0.5]),
                            moe(4, top, 16, limit=0.7))], width=16, vocab=40)
        W = weights(cfg, 23 + top)
        toks = tokens(cfg, 80, 23)
        want = logits_of(cfg, W, toks)
        eng = make_engine(cfg, W, device, dtype)
        got = run_schedule(eng, [toks], [[(0, 70)], [(0, 9)], [(0, 1)]])[0]
        check(got, want, dtype, f"top {top}")


# ------------------------------------------------ the framework's entry points
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


def case_modelhub(device):
    """The serving daemon's model server with this family: sessions over the
    unix socket, two turns on one session, greedy tokens as the plain model
    gives them."""
    import uuid
    from kukeon_amd.serve.server import ModelhubClient, ModelhubServer
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 16)
    mcfg = DumovikConfig.from_json(cfg)
    model = DumovikModel(mcfg, device=device, dtype="fp32", tensors=W,
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


def write_checkpoint(folder, cfg, W):
    """config.json and model.safetensors (8-byte header length, JSON header,
    raw data) of a config dictionary and its tensors."""
    import json
    import os
    import struct
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    head, blobs, at = {}, [], 0
    for name, t in W.items():
        raw = t.view(torch.int16).contiguous().numpy().tobytes()
        head[name] = {"dtype": "BF16", "shape": list(t.shape),
                      "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(head).encode()
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def case_registry(tmp_path, device, dtype):
    """A checkpoint folder is found by its architecture name and read."""
    from kukeon_amd.models.registry import load_checkpoint
    cfg = CONFIGS["plain"]()
    W = weights(cfg, 11)
    write_checkpoint(tmp_path, cfg, W)
    mcfg, model = load_checkpoint(str(tmp_path), device=device, dtype=dtype)
    assert mcfg.family == "dumovik" and len(model.layers) == 3
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


# ------------------------------------------------------- single operations
def _act(dtype):
    return torch.float32 if dtype == "fp32" else torch.bfloat16


def _close(got, want, dtype, what):
    got = got.detach().cpu().double()
    want = want.detach().cpu().double()
    e = float((got - want).abs().max()) / max(float(want.abs().max()), 1e-9)
    lim = 2e-5 if dtype == "fp32" else 2e-2
    assert e <= lim, f"{what}: error {e:.3g} over {lim}"


def case_op_layer_norm(device, dtype):
    """Output-side layer norm with the residual sum, and the plain one, for
    rows on and off the vector path and wider than one pass."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(31)
    for T, Wd, ld in ((5, 40, 40), (3, 37, 50), (4, 2304, 2304),
                      (2, 4104, 4200)):
        x = torch.randn(T, Wd, generator=g)
        y = (torch.randn(T, ld, generator=g) * 3 + 0.7).to(_act(dtype))
        w = torch.randn(Wd, generator=g)
        yd = y[:, :Wd].double()
        want_x = x.double() + oracle.layer_norm(yd, w.double(), 1e-4)
        xd = x.to(device).clone()
        out = torch.empty(T, Wd, dtype=_act(dtype), device=device)
        ops.layernorm_residual(xd, y.to(device)[:, :Wd], w.to(device), 1e-4,
                               out)
        _close(xd, want_x, "fp32", f"stream {Wd}")
        _close(out, want_x, dtype, f"cast {Wd}")
        ops.layernorm(out, xd, w.to(device), 1e-4)
        _close(out, oracle.layer_norm(xd.cpu().double(), w.double(), 1e-4),
               dtype, f"plain {Wd}")


def case_op_gated(device, dtype):
    """The gelu-gated product and the sigmoid-gated norm."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(32)
    for T, F in ((7, 24), (3, 13), (2, 4096 + 8)):
        z = (torch.randn(T, 2 * F + 8, generator=g) * 2).to(_act(dtype))
        zd = z.to(device)
        out = torch.empty(T, F, dtype=_act(dtype), device=device)
        ops.gelu_glu(out, zd[:, :F], zd[:, F + 8: 2 * F + 8])
        want = oracle.gelu_tanh(z[:, :F].double()) * \
            z[:, F + 8: 2 * F + 8].double()
        _close(out, want, dtype, f"gelu {F}")
        y = torch.randn(T, F, generator=g) * 4
        w = torch.randn(F, generator=g)
        ops.gated_rmsnorm(out, y.to(device), zd[:, :F], w.to(device), 1e-3)
        want = oracle.unit_rms(y.double(), 1e-3) * w.double() * \
            torch.sigmoid(z[:, :F].double())
        _close(out, want, dtype, f"gated norm {F}")


def case_op_scan(device, dtype, H=3, d=5, dv=7, cuts=(4, 1, 9, 1, 1)):
    """The decayed recurrence over portions with a dirty slot and an
    inactive neighbour, against the token-by-token sums."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(33)
    n = sum(cuts)
    C = 2 * H * d + H * dv
    proj = torch.randn(n, C + 3, generator=g).to(_act(dtype))
    decay = torch.rand(H, generator=g) * 0.5 + 0.5
    decay[-1] = 1.0
    silu = lambda z: z * torch.sigmoid(z)
    pd = proj.double()
    q = silu(pd[:, 3: 3 + H * d]).view(n, H, d)
    k = silu(pd[:, 3 + H * d: 3 + 2 * H * d]).view(n, H, d)
    v = silu(pd[:, 3 + 2 * H * d:]).view(n, H, dv)
    S = torch.zeros(H, d, dv, dtype=torch.float64)
    want = torch.zeros(n, H * dv, dtype=torch.float64)
    for i in range(n):
        S = decay.double()[:, None, None] * S + \
            k[i][:, :, None] * v[i][:, None, :]
        want[i] = torch.einsum("hde,hd->he", S, q[i]).reshape(-1)
    state = torch.full((3, H, dv, d), 9.0, device=device)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    got = []
    at = 0
    for c in cuts:
        # a second, inactive sequence of one row rides along
        rows = torch.cat([proj[at: at + c], proj[:1]]).to(device)
        y = torch.full((c + 1, H * dv), 5.0, device=device)
        ops.lightning_scan(y, rows, 3, 3 + H * d, 3 + 2 * H * d,
                           decay.to(device), state,
                           i32(list(range(at, at + c)) + [-1]),
                           i32([0, c, c + 1]), i32([2, 0]), H, d, dv)
        assert float(y[c].abs().max()) == 0.0
        got.append(y[:c].cpu())
        at += c
    lim = "fp32" if dtype == "fp32" else "bf16"
    _close(torch.cat(got), want, lim, f"scan {H}x{d}x{dv}")
    assert float((state[0] - 9.0).abs().max()) == 0.0
    _close(state[2].cpu().transpose(1, 2), S, "fp32", "carried state")


def case_op_router(device, dtype):
    """Top experts and their weights, ties and equal logits included."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(34)
    for T, E, top in ((9, 5, 2), (300, 12, 4), (4, 3, 3), (6, 7, 1)):
        z = torch.randn(T, E, generator=g)
        z[0] = 0.25                      # all equal: the lowest indices win
        if E > 2:
            z[1, 2] = z[1, 0]
        idx = torch.empty(T, top, dtype=torch.int32, device=device)
        wts = torch.empty(T, top, dtype=torch.float32, device=device)
        ops.router_topk(idx, wts, z.to(device), top, 0)
        for t in range(T):
            order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
            assert idx[t].tolist() == order, f"row {t}"
            w = torch.softmax(z[t, order].double(), -1)
            _close(wts[t], w, "fp32", f"weights of row {t}")
        ops.router_topk(idx, wts, z.to(device), top, T)
        assert idx[3].tolist() == [
            e * T + 3 for e in sorted(range(E),
                                      key=lambda e: (-float(z[3, e]), e))[:top]]
