"""Device-op dispatch for kukeon_amd.

On a CUDA (ROCm) device every op is the hand-written gfx950 HIP kernel from
``kukeon_amd._C`` — if the extension is missing there we raise instead of
falling back, so a GPU run can never silently use an eager path.  On CPU the
fp32 reference implementations run (tests, GPU-less control-plane hosts).
"""
from __future__ import annotations

import torch

from . import reference

_C = None
_IMPORT_ERROR: Exception | None = None
try:
    from kukeon_amd import _C  # type: ignore
except Exception as e:  # pragma: no cover - exercised only on broken installs
    _IMPORT_ERROR = e


_C_mix = None
_MIX_IMPORT_ERROR: Exception | None = None
try:
    from kukeon_amd import _C_mix  # type: ignore
except Exception as e:  # pragma: no cover
    _MIX_IMPORT_ERROR = e


_C_recur = None
_RECUR_IMPORT_ERROR: Exception | None = None
try:
    from kukeon_amd import _C_recur  # type: ignore
except Exception as e:  # pragma: no cover
    _RECUR_IMPORT_ERROR = e


def native_available() -> bool:
    return _C is not None


def mix_available() -> bool:
    return _C_mix is not None


def _mix(t: torch.Tensor):
    """Kernel group of the sequence mixers: native on a GPU tensor (an
    error if the module is not built), the fp32 references on CPU."""
    global _C_mix, _MIX_IMPORT_ERROR
    if not t.is_cuda:
        return reference
    if _C_mix is None:
        # the module may have been built after this package was imported
        try:
            import importlib
            _C_mix = importlib.import_module("kukeon_amd._C_mix")
        except Exception as e:
            _MIX_IMPORT_ERROR = e
    if _C_mix is None:
        raise RuntimeError(
            "kukeon_amd._C_mix (gfx950 HIP extension) is not built but an op "
            "was called on a CUDA device. Run `python -m kukeon_amd.ops.build "
            f"mix` (import error: {_MIX_IMPORT_ERROR})")
    return _C_mix


def recur_available() -> bool:
    return _C_recur is not None


def _recur(t: torch.Tensor):
    """Kernel group of the recurrent and latent mixers: native on a GPU
    tensor (an error if the module is not built), fp32 references on CPU."""
    global _C_recur, _RECUR_IMPORT_ERROR
    if not t.is_cuda:
        return reference
    if _C_recur is None:
        try:
            import importlib
            _C_recur = importlib.import_module("kukeon_amd._C_recur")
        except Exception as e:
            _RECUR_IMPORT_ERROR = e
    if _C_recur is None:
        raise RuntimeError(
            "kukeon_amd._C_recur (gfx950 HIP extension) is not built but an "
            "op was called on a CUDA device. Run `python -m "
            f"kukeon_amd.ops.build recur` (import error: "
            f"{_RECUR_IMPORT_ERROR})")
    return _C_recur


_C_hyb = None
_HYB_IMPORT_ERROR: Exception | None = None
try:
    from kukeon_amd import _C_hyb  # type: ignore
except Exception as e:  # pragma: no cover
    _HYB_IMPORT_ERROR = e


def hyb_available() -> bool:
    return _C_hyb is not None


def _hyb(t: torch.Tensor):
    """Kernel group of the hybrid stacks (output-side layer norm, chunked
    attention, decayed linear attention, routed experts): native on a GPU
    tensor (an error if the module is not built), fp32 references on CPU."""
    global _C_hyb, _HYB_IMPORT_ERROR
    if not t.is_cuda:
        return reference
    if _C_hyb is None:
        try:
            import importlib
            _C_hyb = importlib.import_module("kukeon_amd._C_hyb")
        except Exception as e:
            _HYB_IMPORT_ERROR = e
    if _C_hyb is None:
        raise RuntimeError(
            "kukeon_amd._C_hyb (gfx950 HIP extension) is not built but an "
            "op was called on a CUDA device. Run `python -m "
            f"kukeon_amd.ops.build hyb` (import error: {_HYB_IMPORT_ERROR})")
    return _C_hyb


_C_strm = None
_STRM_IMPORT_ERROR: Exception | None = None
try:
    from kukeon_amd import _C_strm  # type: ignore
except Exception as e:  # pragma: no cover
    _STRM_IMPORT_ERROR = e


def strm_available() -> bool:
    return _C_strm is not None


def _strm(t: torch.Tensor):
    """Kernel group of the multi-stream stacks (stream read/write with the
    norm, token shift, linear attention with a decay per key channel,
    windowed attention with a distance bias, group-limited routing): native
    on a GPU tensor (an error if the module is not built), fp32 references
    on CPU."""
    global _C_strm, _STRM_IMPORT_ERROR
    if not t.is_cuda:
        return reference
    if _C_strm is None:
        try:
            import importlib
            _C_strm = importlib.import_module("kukeon_amd._C_strm")
        except Exception as e:
            _STRM_IMPORT_ERROR = e
    if _C_strm is None:
        raise RuntimeError(
            "kukeon_amd._C_strm (gfx950 HIP extension) is not built but an "
            "op was called on a CUDA device. Run `python -m "
            f"kukeon_amd.ops.build strm` (import error: "
            f"{_STRM_IMPORT_ERROR})")
    return _C_strm


def _shared(t: torch.Tensor, first, second):
    """A kernel that two groups compile from the same source: whichever of
    the two modules is built serves it (`first` preferred)."""
    if not t.is_cuda:
        return reference
    key = (first, second)
    mod = _SHARED_CHOICE.get(key)
    if mod is None:
        try:
            mod = first(t)
        except RuntimeError:
            mod = second(t)
        _SHARED_CHOICE[key] = mod
    return mod


_SHARED_CHOICE: dict = {}


def _shared3(t: torch.Tensor, first, second, third):
    """As _shared, for a kernel that three groups compile."""
    if not t.is_cuda:
        return reference
    key = (first, second, third)
    mod = _SHARED_CHOICE.get(key)
    if mod is None:
        for get in key:
            try:
                mod = get(t)
                break
            except RuntimeError as e:
                err = e
        if mod is None:
            raise err
        _SHARED_CHOICE[key] = mod
    return mod


def _native():
    if _C is None:
        raise RuntimeError(
            "kukeon_amd._C (gfx950 HIP extension) is not built but an op was "
            "called on a CUDA device. Run `python -m kukeon_amd.ops.build` "
            f"(import error: {_IMPORT_ERROR})")
    return _C


def _impl(t: torch.Tensor):
    return _native() if t.is_cuda else reference


def rmsnorm(out, input, weight, eps: float) -> None:
    _impl(input).rmsnorm(out, input, weight, eps)


def fused_add_rmsnorm(input, residual, weight, eps: float) -> None:
    _impl(input).fused_add_rmsnorm(input, residual, weight, eps)


def silu_mul(out, gate_up) -> None:
    _impl(gate_up).silu_mul(out, gate_up)


def rope_kv_append(qkv, k_cache, v_cache, cos_sin, positions, slot_mapping,
                   num_q_heads: int, num_kv_heads: int, head_dim: int,
                   block_table=None) -> None:
    if block_table is None:
        block_table = torch.empty(0, dtype=torch.int32, device=qkv.device)
    _impl(qkv).rope_kv_append(qkv, k_cache, v_cache, cos_sin, positions,
                              slot_mapping, num_q_heads, num_kv_heads,
                              head_dim, block_table)


def decode_advance(ids, pos, seq_lens, tokens, ring, counter) -> None:
    _impl(ids).decode_advance(ids, pos, seq_lens, tokens, ring, counter)


def paged_attention(out, q, k_cache, v_cache, block_table, seq_lens,
                    q_offset: int, num_splits: int, scale: float,
                    tmp_out, tmp_ml) -> None:
    _impl(q).paged_attention(out, q, k_cache, v_cache, block_table, seq_lens,
                             q_offset, num_splits, scale, tmp_out, tmp_ml)


def prefill_attention(out, q, k_cache, v_cache, block_table, seq_lens,
                      q_starts, qb_seq, qb_start, q_offset: int,
                      scale: float) -> None:
    _impl(q).prefill_attention(out, q, k_cache, v_cache, block_table,
                               seq_lens, q_starts, qb_seq, qb_start, q_offset,
                               scale)


def sample(tokens, logits, temps, top_k, top_p, seed, workspace) -> None:
    _impl(logits).sample(tokens, logits, temps, top_k, top_p, seed, workspace)


_SKINNY_WS = {}
# replaced (outgrown) workspaces are pinned here forever: a hipGraph
# captured earlier may still hold the old tensor's device pointer, and
# letting it free would put a use-after-free inside every later replay
_SKINNY_WS_RETIRED = []
# Per-shape dispatch, from the measured sweep (profiles/r01_progress.md,
# scripts/sweep_splitk.py on MI355X): the glds-staged skinny kernel beats
# hipBLASLt on square o-projection shapes (N==K: 16.6us vs 19.3 at M=64,
# 11.9 vs 19.2 at M=16 on 4096x4096) and trails it on qkv/gate_up/down/
# lm_head, where hipBLASLt is 55-100% of the HBM floor. KUKEON_SKINNY_GEMM=1
# forces the skinny kernel for every eligible shape (benchmarking).
_USE_SKINNY = __import__("os").environ.get("KUKEON_SKINNY_GEMM", "0")
# silu-into-down-staging fusion: measured SLOWER in situ (54.2us fused vs
# 42.9 for silu_mul + gemm cold; bench 51.7 vs 53.6 turns/s same box) —
# the doubled x staging traffic outweighs the saved launch. Off by
# default; kernel + numerics test stay as the documented negative result.
_FUSE_SILU = __import__("os").environ.get("KUKEON_FUSE_SILU", "0") == "1"


def _skinny_wins(rows: int, N: int, K: int) -> bool:
    if _USE_SKINNY == "off":   # A/B: force the library everywhere
        return False
    return N == K == 4096


# v5 (full-line never-drain pipeline, KS=128/2 blocks-per-CU): beats
# hipBLASLt cold on the down-projection (32.2us vs 39.6 on 4096x14336 at
# M=64, floor 18.6 — profiles/r02_progress.md); qkv ties, gate_up and
# lm_head stay on the library. KUKEON_SKINNY_GEMM=5 forces it everywhere
# for benchmarking.
def _skinny5_wins(rows: int, N: int, K: int) -> bool:
    if _USE_SKINNY == "off":   # A/B: force the library everywhere
        return False
    # llama-3-8b down (32.2us vs blas 39.6 cold) and llama-3-70b down
    # (79.3 vs 83.1 at M=16, 92.6 vs 139.3 at M=64) — measured on
    # MI355X, profiles/r02_progress.md
    if (N, K) in ((4096, 14336), (8192, 28672)):
        return True
    # the same regime — few output columns, a long reduction — that the
    # split-K stream was built for: an output projection over a
    # concatenated [attention | feed-forward] input
    return N % 2048 == 0 and N <= 8192 and K % 128 == 0 and K >= 3 * N


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """F.linear with the weight-streaming skinny-GEMM kernel on the decode
    shapes where it measured faster than hipBLASLt; hipBLASLt otherwise."""
    rows = x.shape[0]
    if _C is None:
        # the weight-streaming kernels are an optimisation over the vendor
        # GEMM, not a requirement: without the core module every shape goes
        # to the library
        return torch.nn.functional.linear(x, w)
    if (x.is_cuda and x.dim() == 2 and rows <= 64
            and w.shape[0] % 128 == 0 and w.shape[1] % 128 == 0
            and x.dtype == torch.bfloat16
            and (_USE_SKINNY == "5"
                 or _skinny5_wins(rows, w.shape[0], w.shape[1]))):
        N = w.shape[0]
        K = w.shape[1]
        out = torch.empty(rows, N, dtype=x.dtype, device=x.device)
        key = (x.device.index or 0)
        ws = _SKINNY_WS.get(key)
        ngroups = N // 128
        nslices = -(-K // 128)
        splitk = 1 if ngroups >= 256 else min(nslices, -(-256 // ngroups))
        need = max(1, splitk) * 64 * N
        if ws is None or ws.numel() < need:
            if ws is not None:
                _SKINNY_WS_RETIRED.append(ws)
            ws = torch.empty(need, dtype=torch.float32, device=x.device)
            _SKINNY_WS[key] = ws
        _native().skinny_gemm5(out, x, w, ws)
        return out
    if (x.is_cuda and x.dim() == 2 and rows <= 64
            and w.shape[0] % 64 == 0 and w.shape[1] % 32 == 0
            and x.dtype == torch.bfloat16
            and (_USE_SKINNY == "1"
                 or _skinny_wins(rows, w.shape[0], w.shape[1]))):
        N = w.shape[0]
        K = w.shape[1]
        out = torch.empty(rows, N, dtype=x.dtype, device=x.device)
        key = (x.device.index or 0)
        ws = _SKINNY_WS.get(key)
        ntiles = N // 64
        nslices = -(-K // 256)
        splitk = 1 if ntiles >= 512 else min(nslices, -(-256 // ntiles))
        need = max(1, splitk) * 64 * N
        if ws is None or ws.numel() < need:
            # grown only outside graph capture (engine warmup runs eager)
            if ws is not None:
                _SKINNY_WS_RETIRED.append(ws)
            ws = torch.empty(need, dtype=torch.float32, device=x.device)
            _SKINNY_WS[key] = ws
        _native().skinny_gemm(out, x, w, ws)
        return out
    return torch.nn.functional.linear(x, w)


def linear_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w.T with fp32 OUTPUT: the vendor GEMM accumulates bf16 products
    in fp32 either way, so keeping the sums unrounded costs nothing. For
    results that are compared or ranked (logits, router scores)."""
    if x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return torch.nn.functional.linear(x.float(), w.float())


def linear_add_rmsnorm(x: torch.Tensor, w: torch.Tensor,
                       residual: torch.Tensor, norm_weight: torch.Tensor,
                       eps: float) -> torch.Tensor:
    """out-projection + TP all-reduce + residual add + RMSNorm as one
    fused path. On the skinny decode shapes (TP=1) the split-K reduce,
    residual add and norm run in a single kernel — the separate epilogue
    pair cost two launches at the ~4.5us in-graph dispatch floor for
    <1us of work. Mutates `residual` (+= x@w.T) and returns the normed
    activations, exactly like linear() followed by fused_add_rmsnorm().
    """
    from kukeon_amd import parallel
    rows = x.shape[0]
    N, K = w.shape
    if (x.is_cuda and parallel.tp_size() == 1 and x.dim() == 2
            and rows <= 64 and N % 2048 == 0 and N <= 8192 and K % 128 == 0
            and x.dtype == torch.bfloat16
            and (_USE_SKINNY == "5" or _skinny5_wins(rows, N, K))):
        key = (x.device.index or 0)
        ws = _SKINNY_WS.get(key)
        ngroups = N // 128
        nslices = -(-K // 128)
        splitk = min(nslices, -(-256 // ngroups))
        need = max(1, splitk) * 64 * N
        if ws is None or ws.numel() < need:
            if ws is not None:
                _SKINNY_WS_RETIRED.append(ws)
            ws = torch.empty(need, dtype=torch.float32, device=x.device)
            _SKINNY_WS[key] = ws
        normed = torch.empty(rows, N, dtype=x.dtype, device=x.device)
        _native().skinny_gemm5_fused_norm(normed, x, w, ws, residual,
                                          norm_weight, eps)
        return normed
    if (x.is_cuda and parallel.tp_size() == 1 and x.dim() == 2
            and rows <= 64 and N % 2048 == 0 and N <= 8192 and K % 32 == 0
            and x.dtype == torch.bfloat16
            and (_USE_SKINNY == "1" or _skinny_wins(rows, N, K))):
        key = (x.device.index or 0)
        ws = _SKINNY_WS.get(key)
        ntiles = N // 64
        nslices = -(-K // 256)
        splitk = min(nslices, -(-256 // ntiles))
        need = max(1, splitk) * 64 * N
        if ws is None or ws.numel() < need:
            if ws is not None:
                _SKINNY_WS_RETIRED.append(ws)
            ws = torch.empty(need, dtype=torch.float32, device=x.device)
            _SKINNY_WS[key] = ws
        normed = torch.empty(rows, N, dtype=x.dtype, device=x.device)
        _native().skinny_gemm_fused_norm(normed, x, w, ws, residual,
                                         norm_weight, eps)
        return normed
    h = parallel.tp_all_reduce(linear(x, w))
    fused_add_rmsnorm(h, residual, norm_weight, eps)
    return h



def mlp_down_fused(gu: torch.Tensor, w: torch.Tensor,
                   residual: torch.Tensor, norm_weight: torch.Tensor,
                   eps: float) -> torch.Tensor:
    """The decode MLP tail — silu(gate)*up -> down-projection ->
    TP all-reduce -> residual add -> RMSNorm — with the activation fused
    into the down GEMM's x staging on the skinny decode shapes (the
    standalone silu_mul launch and its act-tensor HBM round trip
    disappear; profiles/r02_progress.md). `gu` is the fused gate_up GEMM
    output [rows, 2K]. Equivalent to silu_mul + linear_add_rmsnorm.
    """
    from kukeon_amd import parallel
    rows = gu.shape[0]
    N, K = w.shape
    if (_FUSE_SILU and gu.is_cuda and parallel.tp_size() == 1
            and gu.dim() == 2
            and rows <= 64 and gu.shape[1] == 2 * K
            and N % 2048 == 0 and N <= 8192 and K % 128 == 0
            and gu.dtype == torch.bfloat16
            and (_USE_SKINNY == "5" or _skinny5_wins(rows, N, K))):
        key = (gu.device.index or 0)
        ws = _SKINNY_WS.get(key)
        ngroups = N // 128
        nslices = -(-K // 128)
        splitk = min(nslices, -(-256 // ngroups))
        need = max(1, splitk) * 64 * N
        if ws is None or ws.numel() < need:
            if ws is not None:
                _SKINNY_WS_RETIRED.append(ws)
            ws = torch.empty(need, dtype=torch.float32, device=gu.device)
            _SKINNY_WS[key] = ws
        normed = torch.empty(rows, N, dtype=gu.dtype, device=gu.device)
        _native().skinny_gemm5_silu_fused_norm(normed, gu, w, ws,
                                               residual, norm_weight, eps)
        return normed
    act = torch.empty(rows, K, dtype=gu.dtype, device=gu.device)
    silu_mul(act, gu)
    return linear_add_rmsnorm(act, w, residual, norm_weight, eps)


def moe_router_weights(wdense, logits, k: int) -> None:
    _impl(logits).moe_router_weights(wdense, logits, k)


def moe_dense_combine(out, y, wdense) -> None:
    _impl(y).moe_dense_combine(out, y, wdense)


def moe_gather_tokens(out, input, row_map) -> None:
    _impl(input).moe_gather_tokens(out, input, row_map)


def moe_scatter_tokens(out, input, inv_map, weights, top_k: int) -> None:
    _impl(input).moe_scatter_tokens(out, input, inv_map, weights, top_k)


# ---- sequence-mixer group -------------------------------------------------
def _e(t: torch.Tensor):
    return torch.empty(0, dtype=t.dtype, device=t.device)


def residual_add_rmsnorm(x, a, bias, w, w_offset: float, eps: float,
                         out) -> None:
    """x (fp32 residual, in place) += a (+ bias); out = rmsnorm(x) scaled by
    (w_offset + w). `a` / `bias` may be None."""
    _mix(x).residual_add_rmsnorm(
        x, a if a is not None else _e(out),
        bias if bias is not None else _e(x), w, w_offset, eps, out)


def clamp_glu(out, gate, up, bg, bu, limit: float, alpha: float = 1.702,
              up_shift: float = 1.0) -> None:
    none = torch.empty(0, dtype=torch.float32, device=out.device)
    _shared3(out, _mix, _hyb, _strm).clamp_glu(
        out, gate, up, bg if bg is not None else none,
        bu if bu is not None else none, limit, alpha, up_shift)


def conv_rope_append(q_out, k_cache, v_cache, proj, bias, cw, state, cs,
                     positions, row_seq, cu_rows, state_slots, block_table,
                     q_col: int, k_col: int, v_col: int, Cq: int, Ck: int,
                     Cv: int, map_dim: int, rot_dims: int,
                     one_row_per_seq: bool = False) -> bool:
    """-> True when the state slots were shifted in the same launch (only
    possible when every sequence brings one row); otherwise the caller
    runs conv_state_update."""
    if k_cache is None:
        k_cache = v_cache = _e(proj)
    return bool(_mix(proj).conv_rope_append(
        q_out, k_cache, v_cache, proj, bias, cw, state, cs, positions,
        row_seq, cu_rows, state_slots, block_table, q_col, k_col, v_col,
        Cq, Ck, Cv, map_dim, rot_dims, one_row_per_seq))


def conv_state_update(state, proj, bias, positions, cu_rows, state_slots,
                      q_col: int, k_col: int, v_col: int, Cq: int, Ck: int,
                      Cv: int) -> None:
    _mix(proj).conv_state_update(state, proj, bias, positions, cu_rows,
                                 state_slots, q_col, k_col, v_col, Cq, Ck, Cv)


def diff_attention(out, q, k_cache, v_cache, gate, positions, row_seq,
                   block_table, H: int, scale: float, lam: float, eps: float,
                   out_scale: float) -> None:
    _mix(q).diff_attention(out, q, k_cache, v_cache,
                           gate if gate is not None else _e(q), positions,
                           row_seq, block_table, H, scale, lam, eps,
                           out_scale)


def diff_tiles_supported(t: torch.Tensor, dim: int, vdim: int) -> bool:
    """Whether the matrix-core kernel for prompt portions serves these
    sizes (bf16 on a GPU only)."""
    return (t.is_cuda and t.dtype == torch.bfloat16
            and _mix(t).diff_attention_tiles_supported(dim, vdim))


def diff_attention_tiles(out, q, k_cache, v_cache, gate, positions, cu_rows,
                         block_table, tile_seq, tile_row0, H: int, hpw: int,
                         scale: float, lam: float, eps: float,
                         out_scale: float) -> None:
    _mix(q).diff_attention_tiles(out, q, k_cache, v_cache,
                                 gate if gate is not None else _e(q),
                                 positions, cu_rows, block_table, tile_seq,
                                 tile_row0, H, hpw, scale, lam, eps,
                                 out_scale)


def diff_decode_supported(t: torch.Tensor, H: int, G: int, dim: int,
                          vdim: int) -> bool:
    return (t.is_cuda and _mix(t).diff_attention_decode_supported(
        H, G, dim, vdim, t.dtype == torch.bfloat16))


_DECODE_SPLITS = {}


def diff_decode_splits(t: torch.Tensor, rows: int, H: int, G: int,
                       dim: int) -> int:
    """Split count that makes one launch exactly one full round of units
    on the device (measured: a partly filled second round costs as much as
    the first)."""
    key = (t.device, t.dtype, H, G, dim)
    cap = _DECODE_SPLITS.get(key)
    if cap is None:
        m = _mix(t)
        cap = (m.diff_attention_decode_capacity(
            H, G, dim, t.dtype == torch.bfloat16),
            m.diff_attention_decode_units_per_row(H, G))
        _DECODE_SPLITS[key] = cap
    return max(1, min(32, cap[0] // max(1, rows * cap[1])))


def diff_attention_decode(out, q, k_cache, v_cache, gate, positions, row_seq,
                          block_table, part_o, part_ml, H: int, scale: float,
                          lam: float, eps: float, out_scale: float) -> None:
    _mix(q).diff_attention_decode(out, q, k_cache, v_cache,
                                  gate if gate is not None else _e(q),
                                  positions, row_seq, block_table, part_o,
                                  part_ml, H, scale, lam, eps, out_scale)


# ---- recurrent / latent group ----------------------------------------------
def norm_only(x, w, eps: float, out) -> None:
    """out = rmsnorm(x) * w over the fp32 residual stream (x unchanged)."""
    _recur(x).residual_add_rmsnorm(x, _e(out), _e(x), w, 0.0, eps, out)


def postnorm_residual_rmsnorm(x, y, post_w, w, eps: float, out) -> None:
    """Sandwich norms in one pass over a row: x (fp32, in place) +=
    rmsnorm(y) * post_w, then out = rmsnorm(x) * w."""
    _recur(x).postnorm_residual_rmsnorm(x, y, post_w, w, eps, out)


def conv_act(out, proj, col0: int, cw, bias, state, positions, row_seq,
             cu_rows, state_slots, act: int = 1,
             shift_state: bool = False) -> None:
    """Short causal convolution per channel over proj[:, col0:col0+C] with
    carried taps, bias after the sum, then the activation (1: silu, 0:
    none). With `shift_state` (every sequence brings exactly one row) the
    same launch shifts the state slots; otherwise conv_tail_update does."""
    _recur(proj).conv_act(out, proj, col0, cw, bias, state, positions,
                          row_seq, cu_rows, state_slots, act, shift_state)


def conv_tail_update(state, proj, col0: int, zero_bias, positions, cu_rows,
                     state_slots) -> None:
    """Shift a portion's last inputs into the convolution state slots."""
    C = state.shape[2]
    _recur(proj).conv_state_update(state, proj, zero_bias, positions,
                                   cu_rows, state_slots, col0, 0, 0, C, 0, 0)


def ssm_scan(y, xbc, dt, dt_bias, rate, skip, state, positions, cu_rows,
             state_slots, H: int, P: int, N: int, G: int) -> None:
    _recur(xbc).ssm_scan(y, xbc, dt, dt_bias, rate, skip, state, positions,
                         cu_rows, state_slots, H, P, N, G)


def gated_group_rmsnorm(out, y, z, w, groups: int, eps: float) -> None:
    _recur(out).gated_group_rmsnorm(out, y, z, w, groups, eps)


def latent_kv_append(cq_out, cache, proj, q_col: int, kv_col: int, wq, wkv,
                     eps: float, cs, positions, row_seq,
                     block_table) -> None:
    _shared(proj, _recur, _hyb).latent_kv_append(
        cq_out, cache, proj, q_col, kv_col, wq, wkv, eps, cs, positions,
        row_seq, block_table)


def latent_attention(out, q_abs, q, cache, cs, positions, row_seq,
                     block_table, H: int, dn: int, dr: int, window: int,
                     scale: float) -> None:
    _shared(q, _recur, _hyb).latent_attention(
        out, q_abs, q, cache, cs, positions, row_seq, block_table, H, dn, dr,
        window, scale)


def head_gate(out, o, gate) -> None:
    _shared(out, _recur, _hyb).head_gate(out, o, gate)


def xielu(out, z, ap: float, aq: float) -> None:
    _recur(out).xielu(out, z, ap, aq)


def table_moe(out, h, ids, table, w_up, w_down) -> None:
    _recur(h).table_moe(out, h, ids, table, w_up, w_down)


def gather_rows(out, inp, row_map) -> None:
    _shared3(out, _recur, _hyb, _strm).gather_rows(out, inp, row_map)


def relu_square_(x) -> None:
    _recur(x).relu_square_(x)


def combine_rows(out, inp, inv) -> None:
    _recur(out).combine_rows(out, inp, inv)


def softcap_(logits, cap: float) -> None:
    _recur(logits).softcap_(logits, cap)


# ---- hybrid group ----------------------------------------------------------
def layernorm_residual(x, y, w, eps: float, out) -> None:
    """x (fp32 residual, in place) += layernorm(y) * w (mean taken off, no
    bias); out = x in the activation format."""
    _hyb(x).layernorm_residual(x, y, w, eps, out)


def layernorm(out, x, w, eps: float) -> None:
    _hyb(x).layernorm(out, x, w, eps)


def gelu_glu(out, gate, up) -> None:
    """out = gelu_tanh(gate) * up; gate and up are views into one fused
    projection."""
    _hyb(out).gelu_glu(out, gate, up)


def qk_norm_append(q_out, k_cache, v_cache, proj, q_col: int, k_col: int,
                   v_col: int, wq, wk, eps: float, positions, row_seq,
                   block_table) -> None:
    """RMS norm over the WHOLE query projection (and the whole key
    projection) of a row, then the key and value rows go to their page. A
    layer that reads another layer's pages passes k_cache = None."""
    if k_cache is None:
        k_cache = v_cache = _e(proj)
        wk = _e(wq)
    _hyb(proj).qk_norm_append(q_out, k_cache, v_cache, proj, q_col, k_col,
                              v_col, wq, wk, eps, positions, row_seq,
                              block_table)


def chunk_attention(out, q, k_cache, v_cache, positions, row_seq,
                    block_table, H: int, scale: float, softcap: float,
                    chunk: int) -> None:
    _hyb(q).chunk_attention(out, q, k_cache, v_cache, positions, row_seq,
                            block_table, H, scale, softcap, chunk)


def chunk_tiles_supported(t: torch.Tensor, d: int, dv: int, BS: int) -> bool:
    """Whether the matrix-core kernel for prompt portions serves these
    sizes (bf16 on a GPU only)."""
    return (t.is_cuda and t.dtype == torch.bfloat16
            and _hyb(t).chunk_attention_tiles_supported(d, dv, BS))


def chunk_attention_tiles(out, q, k_cache, v_cache, block_table, seq_lens,
                          q_starts, qb_seq, qb_start, scale: float,
                          softcap: float, chunk: int) -> None:
    _hyb(q).chunk_attention_tiles(out, q, k_cache, v_cache, block_table,
                                  seq_lens, q_starts, qb_seq, qb_start,
                                  scale, softcap, chunk)


def lightning_scan(y, proj, q_col: int, k_col: int, v_col: int, decay, state,
                   positions, cu_rows, state_slots, H: int, d: int,
                   dv: int) -> None:
    _hyb(proj).lightning_scan(y, proj, q_col, k_col, v_col, decay, state,
                              positions, cu_rows, state_slots, H, d, dv)


def gated_rmsnorm(out, y, gate, w, eps: float) -> None:
    _hyb(out).gated_rmsnorm(out, y, gate, w, eps)


def router_topk(idx, wts, logits, top: int, dense_rows: int = 0) -> None:
    _hyb(logits).router_topk(idx, wts, logits, top, dense_rows)


def combine_rows_weighted(out, inp, inv, wts) -> None:
    _shared(out, _hyb, _strm).combine_rows_weighted(out, inp, inv, wts)


# ---- stream group ----------------------------------------------------------
def embed_streams(xs, ids, positions, table, pos_table, scale: float) -> None:
    """xs [T, S, W] fp32: every stream = table[id] * scale + pos_table[p]."""
    _strm(xs).embed_streams(xs, ids, positions, table,
                            pos_table if pos_table is not None else _e(table),
                            scale)


def stream_read_norm(out, xs, coef, w, eps: float) -> None:
    """out = rmsnorm(sum_s coef[s] xs[:, s]) * w."""
    _strm(xs).stream_read_norm(out, xs, coef, w, eps)


def stream_write_read_norm(xs, y, mix, outc, coef, w, eps: float,
                           out) -> None:
    """xs[:, j] <- sum_s mix[s, j] xs[:, s] + outc[j] y in place, then the
    next sublayer's read: out = rmsnorm(sum_j coef[j] xs[:, j]) * w."""
    _strm(xs).stream_write_read_norm(xs, y, mix, outc, coef, w, eps, out)


def token_shift(out, h, mu, state, positions, row_seq, cu_rows, state_slots,
                shift_state: bool = False) -> None:
    """out[n] = h + (row before - h) * mu[n]; the row before a portion's
    first comes from the state slot."""
    _strm(h).token_shift(out, h, mu, state, positions, row_seq, cu_rows,
                         state_slots, shift_state)


def token_shift_tail(state, h, positions, cu_rows, state_slots) -> None:
    _strm(h).token_shift_tail(state, h, positions, cu_rows, state_slots)


def decay_scan(y, q, k, v, lo, w2, zb, bonus, state, positions, cu_rows,
               state_slots, H: int, d: int, dv: int, mode: int,
               tau: float = 1.0, q_scale: float = 1.0) -> None:
    """Linear attention with a token-dependent decay per key channel whose
    pre-activation is w2 f(lo) + zb (f = tanh in mode 0)."""
    _strm(q).decay_scan(y, q, k, v, lo, w2, zb,
                        bonus if bonus is not None else _e(zb), state,
                        positions, cu_rows, state_slots, H, d, dv, mode, tau,
                        q_scale)


def head_rmsnorm_gate(out, y, gate, w, H: int, eps: float, act: int,
                      scale: float = 1.0) -> None:
    """out (a [T, C] view) = y / rms_per_head(y) * w * act(gate) * scale;
    act 0 = silu, 1 = sigmoid."""
    _strm(out).head_rmsnorm_gate(out, y, gate, w, H, eps, act, scale)


def scaled_gate(out, a, gate, act: int, scale: float = 1.0) -> None:
    """out (a [T, C] view) = a * act(gate) * scale; act 0 = silu,
    1 = sigmoid."""
    _strm(out).scaled_gate(out, a, gate, act, scale)


def conv_scale_append(q_out, k_cache, proj, q_col: int, k_col: int, cw, state,
                      coef: float, every: int, positions, row_seq, cu_rows,
                      state_slots, block_table,
                      shift_state: bool = False) -> None:
    _strm(proj).conv_scale_append(q_out, k_cache, proj, q_col, k_col, cw,
                                  state, coef, every, positions, row_seq,
                                  cu_rows, state_slots, block_table,
                                  shift_state)


def conv_pair_tail_update(state, proj, q_col: int, k_col: int, Cq: int,
                          Ck: int, zero_bias, positions, cu_rows,
                          state_slots) -> None:
    """Shift a portion's last query and key inputs into the slots."""
    _strm(proj).conv_state_update(state, proj, zero_bias, positions, cu_rows,
                                  state_slots, q_col, k_col, 0, Cq, Ck, 0)


def window_attention(out, q, k_cache, v_cache, slopes, positions, row_seq,
                     block_table, H: int, scale: float, window: int) -> None:
    """Values are the keys when v_cache is None or empty."""
    _strm(q).window_attention(out, q, k_cache,
                              v_cache if v_cache is not None else _e(q),
                              slopes if slopes is not None
                              else torch.empty(0, dtype=torch.float32,
                                               device=q.device),
                              positions, row_seq, block_table, H, scale,
                              window)


def window_tiles_supported(t: torch.Tensor, d: int, BS: int) -> bool:
    return (t.is_cuda and t.dtype == torch.bfloat16
            and _strm(t).window_attention_tiles_supported(d, BS))


def window_attention_tiles(out, q, k_cache, slopes, block_table, seq_lens,
                           q_starts, qb_seq, qb_start, scale: float,
                           window: int) -> None:
    _strm(q).window_attention_tiles(out, q, k_cache, slopes, block_table,
                                    seq_lens, q_starts, qb_seq, qb_start,
                                    scale, window)


def router_select(idx, wts, logits, top: int, groups: int, keep: int,
                  scale: float, dense_rows: int = 0) -> None:
    _strm(logits).router_select(idx, wts, logits, top, groups, keep, scale,
                                dense_rows)
