"""Plain-PyTorch fp32 reference implementations of every HIP op.

These are the numerics oracles for the GPU test suite (each HIP kernel is
compared against the fp32 reference of the same op, per the repo test
contract) and the CPU execution path for control-plane / scheduler tests on
GPU-less hosts.  They are never used on a CUDA device — `kukeon_amd.ops`
fails loudly there if the native extension is missing.
"""
from __future__ import annotations

import torch


def rmsnorm(out: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
            eps: float) -> None:
    x = input.float()
    rs = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((x * rs * weight.float()).to(out.dtype))


def fused_add_rmsnorm(input: torch.Tensor, residual: torch.Tensor,
                      weight: torch.Tensor, eps: float) -> None:
    r = (residual.float() + input.float())
    residual.copy_(r.to(residual.dtype))
    # match the kernel: it normalizes the bf16-rounded residual it wrote
    r = residual.float()
    rs = torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps)
    input.copy_((r * rs * weight.float()).to(input.dtype))


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor) -> None:
    I = out.shape[-1]
    g = gate_up[..., :I].float()
    u = gate_up[..., I:].float()
    out.copy_((torch.nn.functional.silu(g) * u).to(out.dtype))


def _rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    # NEOX half-rotation; x [T, H, D], cos/sin [T, D/2]
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c = cos.unsqueeze(1)
    s = sin.unsqueeze(1)
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def rope_kv_append(qkv: torch.Tensor, k_cache: torch.Tensor,
                   v_cache: torch.Tensor, cos_sin: torch.Tensor,
                   positions: torch.Tensor, slot_mapping: torch.Tensor,
                   num_q_heads: int, num_kv_heads: int, head_dim: int,
                   block_table=None) -> None:
    T = qkv.shape[0]
    D = head_dim
    half = D // 2
    q = qkv[:, : num_q_heads * D].view(T, num_q_heads, D).float()
    k = qkv[:, num_q_heads * D: (num_q_heads + num_kv_heads) * D].view(
        T, num_kv_heads, D).float()
    v = qkv[:, (num_q_heads + num_kv_heads) * D:].view(T, num_kv_heads, D)
    cs = cos_sin[positions.long().clamp_min(0)]
    cos, sin = cs[:, :half], cs[:, half:]
    qr = _rotate(q, cos, sin).to(qkv.dtype)
    kr = _rotate(k, cos, sin).to(qkv.dtype)
    # inactive decode rows (pos < 0) are skipped entirely, like the kernel
    act = (positions >= 0).view(T, 1)
    qkv[:, : num_q_heads * D] = torch.where(
        act, qr.reshape(T, -1), qkv[:, : num_q_heads * D])
    qkv[:, num_q_heads * D: (num_q_heads + num_kv_heads) * D] = torch.where(
        act, kr.reshape(T, -1),
        qkv[:, num_q_heads * D: (num_q_heads + num_kv_heads) * D])
    BS = k_cache.shape[2]
    fp8 = k_cache.dtype == torch.uint8
    if fp8:
        kr = kr.float().to(torch.float8_e4m3fn).view(torch.uint8)
        v = v.float().to(torch.float8_e4m3fn).view(torch.uint8)
    table_mode = block_table is not None and block_table.dim() == 2
    for t in range(T):
        if table_mode:
            pos_t = int(positions[t])
            if pos_t < 0:
                continue
            slot = int(block_table[t, pos_t // BS]) * BS + pos_t % BS
        else:
            slot = int(slot_mapping[t])
            if slot < 0:
                continue
        blk, off = slot // BS, slot % BS
        k_cache[blk, :, off] = kr[t]
        v_cache[blk, :, off] = v[t]


def _gather_kv(cache: torch.Tensor, block_table: torch.Tensor, ctx: int,
               b: int) -> torch.Tensor:
    """-> [ctx, Hk, D] from paged cache [NB, Hk, BS, D] (bf16 or fp8)."""
    BS = cache.shape[2]
    nb = (ctx + BS - 1) // BS
    blocks = block_table[b, :nb].long()
    flat = cache[blocks]                      # [nb, Hk, BS, D]
    if flat.dtype == torch.uint8:
        flat = flat.view(torch.float8_e4m3fn).float()
    flat = flat.permute(0, 2, 1, 3).reshape(nb * BS, cache.shape[1], -1)
    return flat[:ctx]


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, block_table: torch.Tensor,
                    seq_lens: torch.Tensor, q_offset: int, num_splits: int,
                    scale: float, tmp_out=None, tmp_ml=None) -> None:
    B = q.shape[0]
    Hk, BS, D = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    Hq = out.shape[1] // D
    G = Hq // Hk
    qv = q.view(B, -1)[:, q_offset: q_offset + Hq * D].view(B, Hq, D).float()
    for b in range(B):
        ctx = int(seq_lens[b])
        if ctx <= 0:
            # inactive decode row: write zeros so downstream logits stay
            # finite (the row's sample is discarded by the advance guard,
            # but NaNs from uninitialized memory would crash the CPU
            # sampler's multinomial)
            out.view(B, -1)[b] = 0
            continue
        k = _gather_kv(k_cache, block_table, ctx, b).float()  # [ctx,Hk,D]
        v = _gather_kv(v_cache, block_table, ctx, b).float()
        for h in range(Hq):
            hk = h // G
            s = (k[:, hk] @ qv[b, h]) * scale                  # [ctx]
            p = torch.softmax(s, dim=-1)
            o = p @ v[:, hk]                                   # [D]
            out.view(B, Hq, D)[b, h] = o.to(out.dtype)


def prefill_attention(out: torch.Tensor, q: torch.Tensor,
                      k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_table: torch.Tensor, seq_lens: torch.Tensor,
                      q_starts: torch.Tensor, qb_seq=None, qb_start=None,
                      q_offset: int = 0, scale: float = 1.0) -> None:
    """Varlen causal attention where queries are the tail of each sequence.

    q: [T_total, q_stride] packed new tokens over all sequences (row i of
    sequence s is absolute position q_starts[s] + i); KV (including the new
    tokens, already appended) lives in the paged cache; seq_lens[s] is the
    total context after append. out: [T_total, Hq*D].
    """
    Hk, BS, D = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    Hq = out.shape[1] // D
    G = Hq // Hk
    nseq = seq_lens.shape[0]
    for s in range(nseq):
        ctx = int(seq_lens[s])
        start = int(q_starts[s, 0])
        row = int(q_starts[s, 1])
        qlen = ctx - start
        if qlen <= 0:
            continue
        k = _gather_kv(k_cache, block_table, ctx, s).float()
        v = _gather_kv(v_cache, block_table, ctx, s).float()
        qs = q[row: row + qlen, q_offset: q_offset + Hq * D].view(
            qlen, Hq, D).float()
        pos = torch.arange(start, ctx)
        kvpos = torch.arange(ctx)
        mask = kvpos[None, :] <= pos[:, None]                  # [qlen, ctx]
        for h in range(Hq):
            hk = h // G
            sc = (qs[:, h] @ k[:, hk].T) * scale               # [qlen, ctx]
            sc = sc.masked_fill(~mask, float("-inf"))
            p = torch.softmax(sc, dim=-1)
            o = p @ v[:, hk]
            out[row: row + qlen].view(qlen, Hq, D)[:, h] = o.to(out.dtype)
        pass


def sample(tokens: torch.Tensor, logits: torch.Tensor, temps: torch.Tensor,
           top_k: torch.Tensor, top_p: torch.Tensor, seed: torch.Tensor,
           workspace=None) -> None:
    """Reference sampler. Greedy rows match the kernel exactly; stochastic
    rows draw from the same masked distribution (the GPU test checks the
    distribution, not the draw)."""
    B, V = logits.shape
    lg = logits.float()
    for b in range(B):
        T = float(temps[b])
        row = lg[b]
        if T <= 0:
            tokens[b] = int(torch.argmax(row))
            continue
        k = int(top_k[b])
        p = float(top_p[b])
        probs = torch.softmax((row - row.max()) / T, dim=-1)
        keep = torch.ones(V, dtype=torch.bool)
        if 0 < k < V:
            th = torch.topk(row, k).values.min()
            keep &= row >= th
        if 0 < p < 1:
            srt, idx = torch.sort(probs, descending=True)
            cum = torch.cumsum(srt, 0)
            cut = int(torch.searchsorted(cum, p).clamp(max=V - 1))
            keep2 = torch.zeros(V, dtype=torch.bool)
            keep2[idx[: cut + 1]] = True
            keep &= keep2
        probs = probs * keep
        probs = probs / probs.sum()
        tokens[b] = int(torch.multinomial(probs, 1))
    seed += 1


def linear_add_rmsnorm(x, w, residual, norm_weight, eps: float):
    h = torch.nn.functional.linear(x, w)
    fused_add_rmsnorm(h, residual, norm_weight, eps)
    return h


def decode_advance(ids, pos, seq_lens, tokens, ring, counter) -> None:
    step = int(counter[0])
    B = ids.shape[0]
    for b in range(B):
        if int(seq_lens[b]) > 0:
            ids[b] = tokens[b]
            pos[b] += 1
            seq_lens[b] += 1
            ring[step * B + b] = tokens[b]
    counter[0] = step + 1


def moe_gather_tokens(out: torch.Tensor, input: torch.Tensor,
                      row_map: torch.Tensor) -> None:
    out.copy_(input[row_map.long()])


def moe_scatter_tokens(out: torch.Tensor, input: torch.Tensor,
                       inv_map: torch.Tensor, weights: torch.Tensor,
                       top_k: int) -> None:
    T = out.shape[0]
    acc = (input[inv_map.long()].float() *
           weights.unsqueeze(-1)).sum(dim=1)  # [T, H]
    out.copy_(acc.to(out.dtype))

def moe_router_weights(wdense: torch.Tensor, logits: torch.Tensor,
                       K: int) -> None:
    # accepts bf16 or fp32 logits, like the HIP kernel
    probs = torch.softmax(logits.float(), dim=-1)
    topv, topi = probs.topk(K, dim=-1)
    topv = topv / topv.sum(dim=-1, keepdim=True)
    wdense.zero_()
    wdense.scatter_(1, topi, topv)


def moe_dense_combine(out: torch.Tensor, y: torch.Tensor,
                      wdense: torch.Tensor) -> None:
    acc = (y.float() * wdense.t().unsqueeze(-1)).sum(dim=0)
    out.copy_(acc.to(out.dtype))


# ---------------------------------------------------------------------------
# sequence-mixer group (fp32 residual stream; activations bf16 or fp32)
# ---------------------------------------------------------------------------

def residual_add_rmsnorm(x: torch.Tensor, a, bias, w: torch.Tensor,
                         w_offset: float, eps: float,
                         out: torch.Tensor) -> None:
    """x (fp32, in place) += a (+ bias); out = x / rms(x) * (w_offset + w)."""
    W = x.shape[1]
    if a is not None and a.numel():
        x += a[:, :W].float()
    if bias is not None and bias.numel():
        x += bias
    rs = 1.0 / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((x * rs * (w_offset + w)).to(out.dtype))


def clamp_glu(out, gate, up, bg, bu, limit: float, alpha: float,
              up_shift: float) -> None:
    g = gate.float()
    u = up.float()
    if bg is not None and bg.numel():
        g = g + bg
        u = u + bu
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    out.copy_((g * torch.sigmoid(alpha * g) * (u + up_shift)).to(out.dtype))


def _conv_cols(q_col, k_col, v_col, Cq, Ck, Cv):
    cols = list(range(q_col, q_col + Cq))
    cols += list(range(k_col, k_col + Ck))
    cols += list(range(v_col, v_col + Cv))
    return torch.tensor(cols, dtype=torch.long)


def conv_rope_append(q_out, k_cache, v_cache, proj, bias, cw, state, cs,
                     positions, row_seq, cu_rows, state_slots, block_table,
                     q_col: int, k_col: int, v_col: int, Cq: int, Ck: int,
                     Cv: int, map_dim: int, rot_dims: int,
                     one_row_per_seq: bool = False) -> bool:
    C = Cq + Ck + Cv
    taps = cw.shape[0]                     # cw: [taps, C]
    back = taps - 1
    cols = _conv_cols(q_col, k_col, v_col, Cq, Ck, Cv)
    nseq = cu_rows.numel() - 1
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        n = r1 - r0
        p0 = int(positions[r0])
        u = proj[r0:r1][:, cols].float() + bias              # [n, C]
        hist = state[int(state_slots[s])].clone() if back else u[:0]
        if back:
            # entries that lie before the sequence start count as zeros
            for k in range(back):
                if p0 - back + k < 0:
                    hist[k] = 0
        full = torch.cat([hist, u], 0)                       # [back+n, C]
        y = torch.zeros(n, C)
        for j in range(taps):
            y = y + cw[j] * full[j: j + n]
        pos = positions[r0:r1].long()
        ang = cs[pos.clamp(max=cs.shape[0] - 1)]             # [n, rot_dims]
        half = rot_dims // 2
        co, si = ang[:, :half], ang[:, half:]

        def rot(seg):                                        # [n, maps*dim]
            m = seg.reshape(n, -1, map_dim).clone()
            a, b = m[..., 0:rot_dims:2], m[..., 1:rot_dims:2]
            ra = a * co[:, None] - b * si[:, None]
            rb = b * co[:, None] + a * si[:, None]
            m[..., 0:rot_dims:2] = ra
            m[..., 1:rot_dims:2] = rb
            return m.reshape(n, -1)

        q_out[r0:r1] = rot(y[:, :Cq]).to(q_out.dtype)
        if Ck or Cv:
            G, BS = k_cache.shape[1], k_cache.shape[2]
            kk = rot(y[:, Cq:Cq + Ck]).reshape(n, G, -1).to(k_cache.dtype)
            vv = y[:, Cq + Ck:].reshape(n, G, -1).to(v_cache.dtype)
            for i in range(n):
                p = p0 + i
                blk = int(block_table[s, p // BS])
                k_cache[blk, :, p % BS] = kk[i]
                v_cache[blk, :, p % BS] = vv[i]
    return False


def conv_state_update(state, proj, bias, positions, cu_rows, state_slots,
                      q_col: int, k_col: int, v_col: int, Cq: int, Ck: int,
                      Cv: int) -> None:
    back = state.shape[1]
    if back == 0:
        return
    cols = _conv_cols(q_col, k_col, v_col, Cq, Ck, Cv)
    nseq = cu_rows.numel() - 1
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        u = proj[r0:r1][:, cols].float() + bias
        slot = int(state_slots[s])
        full = torch.cat([state[slot], u], 0)
        state[slot] = full[-back:]


def diff_attention(out, q, k_cache, v_cache, gate, positions, row_seq,
                   block_table, H: int, scale: float, lam: float, eps: float,
                   out_scale: float) -> None:
    G, BS = k_cache.shape[1], k_cache.shape[2]
    dim = k_cache.shape[3] // 2
    vdim = v_cache.shape[3]
    rows = q.shape[0]
    for r in range(rows):
        p = int(positions[r])
        if p < 0:
            out[r, : H * vdim] = 0
            continue
        s = int(row_seq[r])
        k = _gather_kv(k_cache, block_table, p + 1, s).float()  # [ctx,G,2d]
        v = _gather_kv(v_cache, block_table, p + 1, s).float()
        qr = q[r].float().view(H, 2, dim)
        for h in range(H):
            g = h // (H // G)
            a = []
            for m in range(2):
                sc = (k[:, g, m * dim:(m + 1) * dim] @ qr[h, m]) * scale
                a.append(torch.softmax(sc, -1) @ v[:, g])
            o = a[0] - lam * a[1]
            o = o / torch.sqrt(o.pow(2).mean() + eps) * out_scale
            if gate is not None and gate.numel():
                o = o * torch.sigmoid(gate[r, h].float())
            out[r, h * vdim:(h + 1) * vdim] = o.to(out.dtype)


# ---------------------------------------------------------------------------
# recurrent / latent group (state-space scan, short convolution with an
# activation, latent attention, sandwich norms, table-routed experts)
# ---------------------------------------------------------------------------

def _unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def postnorm_residual_rmsnorm(x, y, post_w, w, eps: float, out) -> None:
    """x (fp32, in place) += rmsnorm(y) * post_w; out = rmsnorm(x) * w."""
    x += _unit_rms(y.float(), eps) * post_w
    out.copy_((_unit_rms(x, eps) * w).to(out.dtype))


def conv_act(out, proj, col0: int, cw, bias, state, positions, row_seq,
             cu_rows, state_slots, act: int = 1,
             shift_state: bool = False) -> None:
    """out = act(causal_conv(proj[:, col0:col0+C]) + bias) per sequence;
    the taps before a portion come from the state slot (zeros before the
    sequence start). cw [taps, C] with the newest tap last. act 1 = silu."""
    taps, C = cw.shape
    back = taps - 1
    nseq = cu_rows.numel() - 1
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        n = r1 - r0
        p0 = int(positions[r0])
        u = proj[r0:r1, col0: col0 + C].float()
        hist = state[int(state_slots[s])].clone() if back else u[:0]
        for k in range(back):
            if p0 - back + k < 0:
                hist[k] = 0
        full = torch.cat([hist, u], 0)
        y = torch.zeros(n, C)
        for j in range(taps):
            y = y + cw[j] * full[j: j + n]
        y = y + bias
        if act == 1:
            y = y * torch.sigmoid(y)
        out[r0:r1] = y.to(out.dtype)
        if shift_state and back:
            assert n == 1
            slot = int(state_slots[s])
            state[slot] = torch.cat([state[slot], u], 0)[-back:]


def ssm_scan(y, xbc, dt, dt_bias, rate, skip, state, positions, cu_rows,
             state_slots, H: int, P: int, N: int, G: int) -> None:
    """Selective scan, one token after the other. xbc [T, H*P + 2*G*N] =
    [x | B | C]; dt [T, H] raw step sizes; state [slots, H, P, N] fp32;
    y [T, H*P] fp32. Per head: S = exp(-rate softplus(dt + dt_bias)) S +
    dt B x^T, y = S^T C + skip x."""
    inner = H * P
    nseq = cu_rows.numel() - 1
    per = H // G
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        slot = int(state_slots[s])
        S = state[slot].transpose(1, 2).clone()              # [H, N, P]
        if int(positions[r0]) == 0:
            S.zero_()
        for r in range(r0, r1):
            x = xbc[r, :inner].float().view(H, P)
            B = xbc[r, inner: inner + G * N].float().view(G, N)
            C = xbc[r, inner + G * N:].float().view(G, N)
            B = B.repeat_interleave(per, 0)                  # [H, N]
            C = C.repeat_interleave(per, 0)
            step = torch.nn.functional.softplus(
                dt[r].float() + dt_bias, threshold=30.0)     # [H]
            decay = torch.exp(-rate * step)
            S = decay[:, None, None] * S + \
                (step[:, None] * B)[:, :, None] * x[:, None, :]
            y[r] = ((S * C[:, :, None]).sum(1) +
                    skip[:, None] * x).reshape(inner)
        state[slot] = S.transpose(1, 2)


def gated_group_rmsnorm(out, y, z, w, groups: int, eps: float) -> None:
    """out = rmsnorm_by_group(y * silu(z)) * w; the row is cut into
    `groups` equal parts, each divided by its own root mean square."""
    T, C = y.shape
    zf = z.float()
    g = y.float() * (zf * torch.sigmoid(zf))
    g = _unit_rms(g.view(T, groups, C // groups), eps).view(T, C)
    out.copy_((g * w).to(out.dtype))


def _rot_pairs(v: torch.Tensor, ang: torch.Tensor, dims: int):
    """v [..., n] one position; ang = [cos | sin] of dims/2 pairs."""
    half = dims // 2
    co, si = ang[:half], ang[half:]
    out = v.clone()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * co - b * si
    out[..., 1:dims:2] = b * co + a * si
    return out


def latent_kv_append(cq_out, cache, proj, q_col: int, kv_col: int, wq, wkv,
                     eps: float, cs, positions, row_seq,
                     block_table) -> None:
    """cq_out = rmsnorm(proj[:, q_col:+Rq]) * wq; the cache row of every
    token = [rmsnorm(proj[:, kv_col:+R]) * wkv | rotary(next dr columns)].
    cache [blocks, 1, BS, R + dr]."""
    Rq, R = wq.numel(), wkv.numel()
    dr = cache.shape[3] - R
    BS = cache.shape[2]
    dims = cs.shape[1]
    for r in range(proj.shape[0]):
        p = int(positions[r])
        if p < 0:
            continue
        row = proj[r].float()
        cq_out[r] = (_unit_rms(row[q_col: q_col + Rq], eps) * wq).to(
            cq_out.dtype)
        c = _unit_rms(row[kv_col: kv_col + R], eps) * wkv
        kr = _rot_pairs(row[kv_col + R: kv_col + R + dr], cs[p], dims)
        blk = int(block_table[int(row_seq[r]), p // BS])
        cache[blk, 0, p % BS] = torch.cat([c, kr]).to(cache.dtype)


def latent_attention(out, q_abs, q, cache, cs, positions, row_seq,
                     block_table, H: int, dn: int, dr: int, window: int,
                     scale: float) -> None:
    """Attention of H heads over ONE shared cache row per token,
    [latent (R) | rotated key part (dr)]. q_abs [H, T, R] is the query
    already multiplied into latent space; q [T, H*(dn+dr)] holds the
    unrotated rotary part of every head behind its first dn entries.
    out [H, T, R] = softmax-weighted sum of the latents over the last
    `window` positions."""
    R = q_abs.shape[2]
    BS = cache.shape[2]
    dims = cs.shape[1]
    T = q.shape[0]
    for r in range(T):
        p = int(positions[r])
        if p < 0:
            out[:, r] = 0
            continue
        s = int(row_seq[r])
        lo = max(0, p - window + 1) if window > 0 else 0
        js = torch.arange(lo, p + 1)
        blk = block_table[s, (js // BS).long()].long()
        rows = cache[blk, 0, (js % BS).long()].float()       # [n, R+dr]
        qr = _rot_pairs(q[r, : H * (dn + dr)].float().view(H, dn + dr)[:, dn:], cs[p], dims)
        sc = (q_abs[:, r].float() @ rows[:, :R].T +
              qr @ rows[:, R:].T) * scale                    # [H, n]
        w = torch.softmax(sc, -1)
        out[:, r] = (w @ rows[:, :R]).to(out.dtype)


def head_gate(out, o, gate) -> None:
    """out[t, h*dv:(h+1)*dv] = o[h, t] * sigmoid(gate[t, h]); a gate with
    H*dv columns acts entry by entry."""
    Hh, T, dv = o.shape
    g = torch.sigmoid(gate.float())                  # [T, H] or [T, H*dv]
    g = g.view(T, Hh, -1)                            # per head or per entry
    out.copy_((o.float().permute(1, 0, 2) * g).reshape(
        T, Hh * dv).to(out.dtype))


def xielu(out, z, ap: float, aq: float) -> None:
    """z > 0: ap z^2 + z/2;  z <= 0: aq (exp(z) - 1 - z) + z/2."""
    zf = z.float()
    pos = ap * zf * zf + 0.5 * zf
    neg = aq * (torch.expm1(zf.clamp(max=0.0)) - zf) + 0.5 * zf
    out.copy_(torch.where(zf > 0, pos, neg).to(out.dtype))


def table_moe(out, h, ids, table, w_up, w_down) -> None:
    """out[t] = mean over the experts table[ids[t]] of
    w_down[e] relu(w_up[e] h[t])^2."""
    top = table.shape[1]
    for r in range(h.shape[0]):
        acc = torch.zeros(h.shape[1])
        for e in table[int(ids[r])].tolist():
            a = torch.relu(torch.nn.functional.linear(h[r], w_up[e]))
            a = (a.float() ** 2).to(h.dtype)
            acc += torch.nn.functional.linear(a, w_down[e]).float()
        out[r] = (acc / top).to(out.dtype)


def softcap_(logits, cap: float) -> None:
    logits.copy_(cap * torch.tanh(logits / cap))


def gather_rows(out, inp, row_map) -> None:
    out.copy_(inp[row_map.long()])


def relu_square_(x) -> None:
    x.copy_((torch.relu(x.float()) ** 2).to(x.dtype))


def combine_rows(out, inp, inv) -> None:
    """out[t] = mean over k of inp[inv[t, k]]."""
    out.copy_(inp[inv.long()].float().mean(1).to(out.dtype))


# ---------------------------------------------------------------------------
# hybrid group (output-side layer norm, chunk-masked attention with a score
# cap, linear attention with a fixed per-head decay, routed experts)
# ---------------------------------------------------------------------------

def _layer_norm(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    d = v - v.mean(-1, keepdim=True)
    return d / torch.sqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w


def layernorm_residual(x, y, w, eps: float, out) -> None:
    """x (fp32, in place) += layernorm(y) * w; out = x in the activation
    format (the next sublayer reads the stream itself)."""
    x += _layer_norm(y.float(), w, eps)
    out.copy_(x.to(out.dtype))


def layernorm(out, x, w, eps: float) -> None:
    out.copy_(_layer_norm(x.float(), w, eps).to(out.dtype))


def gelu_glu(out, gate, up) -> None:
    """out = gelu_tanh(gate) * up."""
    g = gate.float()
    a = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 *
                                    (g + 0.044715 * g * g * g)))
    out.copy_((a * up.float()).to(out.dtype))


def qk_norm_append(q_out, k_cache, v_cache, proj, q_col: int, k_col: int,
                   v_col: int, wq, wk, eps: float, positions, row_seq,
                   block_table) -> None:
    """q_out = rmsnorm(proj[:, q_col:+Cq]) * wq over the whole projection
    row; with caches given, the token's page rows get rmsnorm(k) * wk and
    v. k_cache [blocks, G, BS, d], v_cache [blocks, G, BS, dv]."""
    Cq = wq.numel()
    own = k_cache is not None and k_cache.numel() > 0
    for r in range(proj.shape[0]):
        p = int(positions[r])
        if p < 0:
            continue
        row = proj[r].float()
        q_out[r] = (_unit_rms(row[q_col: q_col + Cq], eps) * wq).to(
            q_out.dtype)
        if not own:
            continue
        G, BS, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
        dv = v_cache.shape[3]
        k = _unit_rms(row[k_col: k_col + G * d], eps) * wk
        v = row[v_col: v_col + G * dv]
        blk = int(block_table[int(row_seq[r]), p // BS])
        k_cache[blk, :, p % BS] = k.view(G, d).to(k_cache.dtype)
        v_cache[blk, :, p % BS] = v.view(G, dv).to(v_cache.dtype)


def chunk_attention(out, q, k_cache, v_cache, positions, row_seq,
                    block_table, H: int, scale: float, softcap: float,
                    chunk: int) -> None:
    """Grouped-query attention of row r (position p) over the keys
    lo .. p with lo = the first position of p's chunk (0 without chunks);
    scores are capped as softcap tanh(score / softcap) when softcap > 0."""
    G, BS = k_cache.shape[1], k_cache.shape[2]
    d, dv = k_cache.shape[3], v_cache.shape[3]
    for r in range(q.shape[0]):
        p = int(positions[r])
        if p < 0:
            out[r] = 0
            continue
        s = int(row_seq[r])
        lo = (p // chunk) * chunk if chunk > 0 else 0
        js = torch.arange(lo, p + 1)
        blk = block_table[s, (js // BS).long()].long()
        k = k_cache[blk, :, (js % BS).long()].float()         # [n, G, d]
        v = v_cache[blk, :, (js % BS).long()].float()
        qr = q[r].float().view(H, d)
        for h in range(H):
            g = h // (H // G)
            sc = (k[:, g] @ qr[h]) * scale
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            out[r, h * dv:(h + 1) * dv] = (torch.softmax(sc, -1) @
                                           v[:, g]).to(out.dtype)


def lightning_scan(y, proj, q_col: int, k_col: int, v_col: int, decay, state,
                   positions, cu_rows, state_slots, H: int, d: int,
                   dv: int) -> None:
    """Linear attention with a fixed decay per head, token after token:
    q, k, v = silu of the projection columns; S = decay_h S + k v^T;
    y = S^T q. state [slots, H, dv, d] fp32 holds S^T (taken as zeros at
    position 0); y [T, H*dv] fp32."""
    nseq = cu_rows.numel() - 1
    silu = lambda z: z * torch.sigmoid(z)
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0:
            continue
        if int(positions[r0]) < 0:
            y[r0:r1] = 0
            continue
        slot = int(state_slots[s])
        S = state[slot].transpose(1, 2).clone()              # [H, d, dv]
        if int(positions[r0]) == 0:
            S.zero_()
        for r in range(r0, r1):
            row = proj[r].float()
            qq = silu(row[q_col: q_col + H * d]).view(H, d)
            kk = silu(row[k_col: k_col + H * d]).view(H, d)
            vv = silu(row[v_col: v_col + H * dv]).view(H, dv)
            S = decay[:, None, None] * S + kk[:, :, None] * vv[:, None, :]
            y[r] = (S * qq[:, :, None]).sum(1).reshape(H * dv)
        state[slot] = S.transpose(1, 2)


def gated_rmsnorm(out, y, gate, w, eps: float) -> None:
    """out = rmsnorm(y) * w * sigmoid(gate), the norm over the whole row."""
    out.copy_((_unit_rms(y.float(), eps) * w *
               torch.sigmoid(gate.float())).to(out.dtype))


def router_topk(idx, wts, logits, top: int, dense_rows: int = 0) -> None:
    """The `top` largest logits of every row (ties: the lower index) and the
    softmax over just those. With dense_rows = T the index written is
    expert * T + row: the row of that pair in an [E, T, W] result."""
    val, ix = torch.sort(logits.float(), dim=-1, descending=True, stable=True)
    val, ix = val[:, :top], ix[:, :top]
    wts.copy_(torch.softmax(val, -1))
    if dense_rows:
        ix = ix * dense_rows + torch.arange(logits.shape[0])[:, None]
    idx.copy_(ix.to(idx.dtype))


def combine_rows_weighted(out, inp, inv, wts) -> None:
    """out[t] = sum over k of wts[t, k] * inp[inv[t, k]]."""
    out.copy_((inp[inv.long()].float() * wts[:, :, None]).sum(1).to(
        out.dtype))


# ---------------------------------------------------------------------------
# stream group (several residual streams with learned read/write weights,
# token shift, linear attention with a decay per key channel, windowed
# attention with a distance bias, group-limited routing)
# ---------------------------------------------------------------------------

def embed_streams(xs, ids, positions, table, pos_table, scale: float) -> None:
    """xs[r, s] = table[ids[r]] * scale + pos_table[positions[r]] for every
    stream s (fp32); an inactive row (position < 0) gets zeros."""
    p = positions.long()
    live = (p >= 0)
    x = table[ids.long()].float() * scale
    if pos_table is not None and pos_table.numel():
        x = x + pos_table[p.clamp_min(0)].float()
    x = x * live[:, None]
    xs.copy_(x[:, None, :].expand_as(xs))


def stream_read_norm(out, xs, coef, w, eps: float) -> None:
    """out = rmsnorm(sum_s coef[s] xs[:, s]) * w."""
    u = (xs * coef[None, :, None]).sum(1)
    out.copy_((_unit_rms(u, eps) * w).to(out.dtype))


def stream_write_read_norm(xs, y, mix, outc, coef, w, eps: float,
                           out) -> None:
    """xs[:, j] <- sum_s mix[s, j] xs[:, s] + outc[j] y (all streams from the
    old ones, in place), then out = rmsnorm(sum_j coef[j] xs[:, j]) * w."""
    new = torch.einsum("sj,tsw->tjw", mix, xs) + \
        outc[None, :, None] * y.float()[:, None, :]
    xs.copy_(new)
    stream_read_norm(out, xs, coef, w, eps)


def token_shift(out, h, mu, state, positions, row_seq, cu_rows, state_slots,
                shift_state: bool = False) -> None:
    """out[n, r] = h[r] + (prev[r] - h[r]) * mu[n], prev being the row before
    in the same sequence: the portion's own, or the state slot's for its
    first row (zeros at position 0). With `shift_state` (one row per
    sequence) the slot takes h[r] in the same call."""
    nseq = cu_rows.numel() - 1
    hf = h.float()
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        slot = int(state_slots[s])
        first = state[slot].clone() if int(positions[r0]) > 0 else \
            torch.zeros_like(state[slot])
        prev = torch.cat([first[None], hf[r0:r1 - 1]], 0)
        cur = hf[r0:r1]
        out[:, r0:r1] = (cur[None] + (prev - cur)[None] * mu[:, None, :]).to(
            out.dtype)
        if shift_state:
            state[slot] = hf[r1 - 1]


def token_shift_tail(state, h, positions, cu_rows, state_slots) -> None:
    """state[slot of s] = the last row of sequence s's portion."""
    nseq = cu_rows.numel() - 1
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        state[int(state_slots[s])] = h[r1 - 1].float()


def decay_scan(y, q, k, v, lo, w2, zb, bonus, state, positions, cu_rows,
               state_slots, H: int, d: int, dv: int, mode: int, tau: float,
               q_scale: float) -> None:
    """Linear attention with a decay per key channel, token after token.
    The decay's pre-activation is z_t = w2 f(lo_t) + zb with lo [T, R] fp32,
    w2 [H*d, R] and f = tanh (mode 0) or the identity (mode 1); the decay is
    a_t = exp(-exp(z_t)) (mode 0) or sigmoid(z_t)^(1/tau) (mode 1), all
    fp32. Mode 0 reads before it writes and gives the current
    token a bonus: y_t = (S + diag(bonus) k_t v_t^T)^T q_t, then
    S = diag(a_t) S + k_t v_t^T. Mode 1: S = diag(a_t) S + k_t v_t^T, then
    y_t = S^T (q_scale q_t). state [slots, H, dv, d] holds S^T (zeros at
    position 0); y [T, H*dv] fp32; q, k [T, H*d], v [T, H*dv] views."""
    nseq = cu_rows.numel() - 1
    lof = lo.float()
    z = (torch.tanh(lof) if mode == 0 else lof) @ w2.float().T + zb
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0:
            continue
        if int(positions[r0]) < 0:
            y[r0:r1] = 0
            continue
        slot = int(state_slots[s])
        S = state[slot].transpose(1, 2).clone()              # [H, d, dv]
        if int(positions[r0]) == 0:
            S.zero_()
        for r in range(r0, r1):
            qq = q[r].float().view(H, d) * q_scale
            kk = k[r].float().view(H, d)
            vv = v[r].float().view(H, dv)
            zz = z[r].view(H, d)
            kv = kk[:, :, None] * vv[:, None, :]
            if mode == 0:
                a = torch.exp(-torch.exp(zz))
                y[r] = ((S + bonus.view(H, d)[:, :, None] * kv) *
                        qq[:, :, None]).sum(1).reshape(H * dv)
                S = a[:, :, None] * S + kv
            else:
                a = torch.exp(torch.nn.functional.logsigmoid(zz) / tau)
                S = a[:, :, None] * S + kv
                y[r] = (S * qq[:, :, None]).sum(1).reshape(H * dv)
        state[slot] = S.transpose(1, 2)


def _gate_act(gate, act: int):
    g = gate.float()
    return g * torch.sigmoid(g) if act == 0 else torch.sigmoid(g)


def head_rmsnorm_gate(out, y, gate, w, H: int, eps: float, act: int,
                      scale: float = 1.0) -> None:
    """out = y / rms_per_head(y) * w * act(gate) * scale: act 0 = silu,
    1 = sigmoid; the row is cut into H heads, each divided by its own root
    mean square."""
    T, C = y.shape
    n = _unit_rms(y.float().view(T, H, C // H), eps).view(T, C) * w
    out.copy_((n * _gate_act(gate, act) * scale).to(out.dtype))


def scaled_gate(out, a, gate, act: int, scale: float = 1.0) -> None:
    """out = a * act(gate) * scale."""
    out.copy_((a.float() * _gate_act(gate, act) * scale).to(out.dtype))


def conv_scale_append(q_out, k_cache, proj, q_col: int, k_col: int, cw, state,
                      coef: float, every: int, positions, row_seq, cu_rows,
                      state_slots, block_table,
                      shift_state: bool = False) -> None:
    """Short causal convolution (no bias, no activation) over the query and
    the key columns of a projection, carried taps in `state`
    [slots, taps-1, Cq+Ck]. The queries are scaled by
    1 + coef ln(floor((p + 1) / every) + 1) and go to q_out [T, Cq]; the
    keys go to the row's page, k_cache [blocks, G, BS, d]."""
    taps, C = cw.shape
    Cq = q_out.shape[1]
    Ck = C - Cq
    back = taps - 1
    G, BS = k_cache.shape[1], k_cache.shape[2]
    cols = _conv_cols(q_col, k_col, 0, Cq, Ck, 0)
    nseq = cu_rows.numel() - 1
    for s in range(nseq):
        r0, r1 = int(cu_rows[s]), int(cu_rows[s + 1])
        if r1 <= r0 or int(positions[r0]) < 0:
            continue
        n = r1 - r0
        p0 = int(positions[r0])
        u = proj[r0:r1][:, cols].float()
        slot = int(state_slots[s])
        hist = state[slot].clone() if back else u[:0]
        for j in range(back):
            if p0 - back + j < 0:
                hist[j] = 0
        full = torch.cat([hist, u], 0)
        yv = torch.zeros(n, C)
        for j in range(taps):
            yv = yv + cw[j] * full[j: j + n]
        pp = torch.arange(p0, p0 + n)
        temp = torch.ones(n)
        if every > 0:
            temp = 1.0 + coef * torch.log(
                torch.div(pp + 1, every, rounding_mode="floor").float() + 1.0)
        q_out[r0:r1] = (yv[:, :Cq] * temp[:, None]).to(q_out.dtype)
        kk = yv[:, Cq:].reshape(n, G, -1).to(k_cache.dtype)
        for i in range(n):
            p = p0 + i
            blk = int(block_table[s, p // BS])
            k_cache[blk, :, p % BS] = kk[i]
        if shift_state and back:
            state[slot] = full[-back:]


def window_attention(out, q, k_cache, v_cache, slopes, positions, row_seq,
                     block_table, H: int, scale: float, window: int) -> None:
    """Grouped-query softmax attention of row r (position p) over the keys
    max(0, p - window + 1) .. p (all of 0 .. p when window is 0), with
    slopes[h] (p - j) taken off head h's scores. Without a value cache
    (None or empty) the values are the keys."""
    G, BS, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    own_v = v_cache is not None and v_cache.numel() > 0
    dv = v_cache.shape[3] if own_v else d
    for r in range(q.shape[0]):
        p = int(positions[r])
        if p < 0:
            out[r] = 0
            continue
        s = int(row_seq[r])
        lo = max(0, p - window + 1) if window > 0 else 0
        js = torch.arange(lo, p + 1)
        blk = block_table[s, (js // BS).long()].long()
        k = k_cache[blk, :, (js % BS).long()].float()         # [n, G, d]
        v = v_cache[blk, :, (js % BS).long()].float() if own_v else k
        qr = q[r].float().view(H, d)
        for h in range(H):
            g = h // (H // G)
            sc = (k[:, g] @ qr[h]) * scale
            if slopes is not None and slopes.numel():
                sc = sc - slopes[h] * (p - js).float()
            out[r, h * dv:(h + 1) * dv] = (torch.softmax(sc, -1) @
                                           v[:, g]).to(out.dtype)


def router_select(idx, wts, logits, top: int, groups: int, keep: int,
                  scale: float, dense_rows: int = 0) -> None:
    """Scores = softmax over all logits. With groups > 0 the experts form
    `groups` equal runs of neighbours, a run's score is its largest, and
    only the `keep` best runs can be chosen (ties: the lower index). The
    `top` best allowed experts get their scores divided by the scores' sum
    (+ 1e-20), times scale. With dense_rows = T the index written is
    expert * T + row. idx and wts may have more than `top` columns; the
    others are left alone."""
    T, E = logits.shape
    s = torch.softmax(logits.float(), -1)
    allowed = s.clone()
    if groups > 0:
        best = s.view(T, groups, E // groups).max(-1).values
        kept = torch.sort(best, dim=-1, descending=True,
                          stable=True).indices[:, :keep]
        mask = torch.zeros(T, groups, dtype=torch.bool)
        mask.scatter_(1, kept, True)
        allowed = torch.where(mask.repeat_interleave(E // groups, 1), s,
                              torch.full_like(s, -1.0))
    ix = torch.sort(allowed, dim=-1, descending=True,
                    stable=True).indices[:, :top]
    w = s.gather(1, ix)
    wts[:, :top] = w / (w.sum(-1, keepdim=True) + 1e-20) * scale
    if dense_rows:
        ix = ix * dense_rows + torch.arange(T)[:, None]
    idx[:, :top] = ix.to(idx.dtype)
