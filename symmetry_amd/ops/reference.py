"""Plain-PyTorch fp32 reference implementations of every symmetry_amd kernel.

They define the semantics the HIP kernels in ``csrc/kernels`` must match
(tests compare the two) and are the execution path for CPU tensors (unit
tests, the tiny CPU models).  Layout conventions are identical to the
kernels':

* ``LinOut``: a projection output is bf16 ``[T, N]`` or fp32 split-K slabs
  ``[S, T, N]`` (summed by the consumer);
* ``k_cache [NB, Hkv, BS, D]`` token-major, ``v_cache [NB, Hkv, D, BS]``
  dim-major;
* RoPE uses the rotate-half convention with a ``[max_pos, D]`` table
  ``[cos | sin]``.
"""
from __future__ import annotations

import math

import torch

MASK32 = 0xFFFFFFFF


def _mm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w.T in fp32.  On the CPU (the numerics oracle) both operands are upcast; on a GPU (only in the
    SYMMETRY_OPS=torch eager baseline) the product runs as a bf16 library GEMM with fp32 output, so the
    baseline never materialises fp32 copies of the weights."""
    if x.device.type == "cpu":
        return x.float() @ w.float().t()
    return (x.to(w.dtype) @ w.t()).float()


def linout_sum(x: torch.Tensor) -> torch.Tensor:
    """Collapse a LinOut to fp32 ``[T, N]``."""
    if x.dtype == torch.float32 and x.dim() == 3:
        return x.sum(0)
    return x.float()


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    xf = linout_sum(x)
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    out.copy_(y.view_as(out).to(out.dtype))


def add_rms_norm(delta, residual, w, eps, out) -> None:
    residual.add_(linout_sum(delta).view_as(residual))
    rms_norm(residual, w, eps, out)


def embed_rms_norm(ids, table, residual, w, eps, out) -> None:
    residual.copy_(table[ids.long()].float())
    rms_norm(residual, w, eps, out)


def _unperm_qk(x: torch.Tensor, nqk: int, D: int) -> torch.Tensor:
    """Undo the decode layout (models/layout.py) of the first ``nqk`` heads of x [T, H, D]."""
    from ..models.layout import _pair_perm

    inv = torch.empty(D, dtype=torch.long)
    inv[_pair_perm(D // 2)] = torch.arange(D)
    x = x.clone()
    x[:, :nqk] = x[:, :nqk].index_select(-1, inv.to(x.device))
    return x


def rope_cache(qkv, positions, slots, cos_sin, q_out, k_cache, v_cache, Hq: int, Hkv: int, perm: bool = False) -> None:
    T = positions.numel()
    D = k_cache.shape[3]
    BS = k_cache.shape[2]
    x = linout_sum(qkv).view(T, Hq + 2 * Hkv, D)
    if perm:
        x = _unperm_qk(x, Hq + Hkv, D)
    cs = cos_sin[positions.long()]  # [T, D]
    half = D // 2
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    qk = x[:, : Hq + Hkv]
    x1, x2 = qk[..., :half], qk[..., half:]
    rot = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
    q_out.copy_(rot[:, :Hq].reshape(q_out.shape).to(q_out.dtype))
    k = rot[:, Hq:].to(k_cache.dtype)
    v = x[:, Hq + Hkv:].to(v_cache.dtype)
    s = slots.long()
    valid = s >= 0
    if valid.any():
        s, k, v = s[valid], k[valid], v[valid]
        blk, off = s // BS, s % BS
        k_cache[blk, :, off, :] = k
        v_cache[blk, :, :, off] = v


def _gather_kv(k_cache, v_cache, block_table, ctx: int):
    """Contiguous K, V [ctx, Hkv, D] of one sequence (fp32)."""
    BS = k_cache.shape[2]
    nb = (ctx + BS - 1) // BS
    blocks = block_table[:nb].long()
    k = k_cache[blocks].permute(0, 2, 1, 3).reshape(nb * BS, k_cache.shape[1], -1)[:ctx]
    v = v_cache[blocks].permute(0, 3, 1, 2).reshape(nb * BS, v_cache.shape[1], -1)[:ctx]
    return k.float(), v.float()


def _attend(q, k, v, scale, causal_offset=None):
    """q [n, Hq, D], k/v [ctx, Hkv, D] -> [n, Hq, D] fp32 (GQA by repeat)."""
    Hq, Hkv = q.shape[1], k.shape[1]
    G = Hq // Hkv
    k = k.repeat_interleave(G, dim=1)
    v = v.repeat_interleave(G, dim=1)
    s = torch.einsum("qhd,khd->hqk", q.float(), k) * scale
    if causal_offset is not None:
        n, ctx = q.shape[0], k.shape[0]
        qpos = torch.arange(n, device=q.device)[:, None] + causal_offset
        kpos = torch.arange(ctx, device=q.device)[None, :]
        s = s.masked_fill(kpos > qpos, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hqk,khd->qhd", p, v)


def attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, out, tmp_o=None, tmp_ml=None, scale=1.0) -> None:
    S = q.shape[0]
    res = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    for i in range(S):
        ctx = int(ctx_lens[i])
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], ctx)
        res[i] = _attend(q[i : i + 1], k, v, scale)[0]
    out.copy_(res.view_as(out).to(out.dtype))


def attn_prefill(q, k_cache, v_cache, block_tables, ctx_lens, cu_q, tiles, out, scale) -> None:
    nseq = ctx_lens.numel()
    res = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    for i in range(nseq):
        a, b = int(cu_q[i]), int(cu_q[i + 1])
        if b == a:
            continue
        ctx = int(ctx_lens[i])
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], ctx)
        res[a:b] = _attend(q[a:b], k, v, scale, causal_offset=ctx - (b - a))
    out.copy_(res.view_as(out).to(out.dtype))


def skinny_gemm(x, w, y) -> None:
    S = y.shape[0]
    K = x.shape[1]
    kc = K // S
    for s in range(S):
        y[s] = _mm(x[:, s * kc : (s + 1) * kc], w[:, s * kc : (s + 1) * kc])


# ----- sampling: same counter-based RNG and packed keys as the kernel ----------------------------
def _u32(x):
    return x & MASK32


def uniform01(seed: torch.Tensor, counter: torch.Tensor) -> torch.Tensor:
    """Bit-exact torch port of ``uniform01`` in csrc/kernels/common.h (int64 tensors)."""
    x0 = _u32(counter)
    x1 = _u32(counter >> 32)
    k0 = _u32(seed).expand_as(x0).clone()
    k1 = _u32(seed >> 32).expand_as(x0).clone()
    for _ in range(7):
        p0h, p0l = _mulhilo(x0, 0xD2511F53)
        p1h, p1l = _mulhilo(x1, 0xCD9E8D57)
        n0 = p1h ^ k0 ^ p0l
        n1 = p0h ^ k1 ^ p1l
        x0, x1 = n0, n1
        k0 = _u32(k0 + 0x9E3779B9)
        k1 = _u32(k1 + 0xBB67AE85)
    return ((x0 >> 8).double() + 0.5) * (1.0 / 16777216.0)


def _mulhilo(a: torch.Tensor, b: int):
    """Unsigned 32x32->64 multiply of int64 tensors holding u32 values."""
    al, ah = a & 0xFFFF, a >> 16
    bl, bh = b & 0xFFFF, b >> 16
    ll = al * bl
    lh = al * bh
    hl = ah * bl
    hh = ah * bh
    mid = (ll >> 16) + (lh & 0xFFFF) + (hl & 0xFFFF)
    lo = _u32((mid << 16) | (ll & 0xFFFF))
    hi = _u32(hh + (lh >> 16) + (hl >> 16) + (mid >> 16))
    return hi, lo


def _ordered_bits(v: torch.Tensor) -> torch.Tensor:
    u = v.float().view(torch.int32).long() & MASK32
    neg = (u & 0x80000000) != 0
    return torch.where(neg, _u32(~u), u | 0x80000000)


def sample_keys(logits: torch.Tensor, temps: torch.Tensor, seeds: torch.Tensor, step: int, n_offset: int = 0):
    """Packed argmax keys (int64 bit pattern of the kernel's u64) and token ids per row."""
    M, N = logits.shape
    gidx = torch.arange(N, device=logits.device, dtype=torch.int64) + n_offset
    vals = logits.float().clone()
    for m in range(M):
        t = float(temps[m])
        if t > 0:
            seed = int(seeds[m]) & 0xFFFFFFFFFFFFFFFF
            mixed = seed ^ ((step << 20) & 0xFFFFFFFFFFFFFFFF)
            if mixed >= 1 << 63:
                mixed -= 1 << 64
            u = uniform01(torch.tensor(mixed, dtype=torch.int64, device=gidx.device), gidx).float()
            vals[m] = vals[m] / t - torch.log(-torch.log(u))
    ob = _ordered_bits(vals)
    low = 0xFFFFFFFF - gidx
    ids = torch.empty(M, dtype=torch.int64, device=logits.device)
    keys = torch.empty(M, dtype=torch.int64, device=logits.device)
    for m in range(M):
        # max over (ob, low) lexicographic == max key
        best = ob[m].max()
        cand = torch.nonzero(ob[m] == best).flatten()
        j = int(cand.min())  # smallest index wins ties (largest ~idx)
        ids[m] = int(gidx[j])
        key = (int(best) << 32) | int(low[j])
        keys[m] = key - (1 << 64) if key >= 1 << 63 else key
    return keys, ids


def lm_head_sample(x, w, temps, seeds, step, tile_keys, out_keys, out_ids, n_offset: int, logits=None) -> None:
    lg = _mm(x, w)
    if logits is not None:
        logits.copy_(lg)
    keys, ids = sample_keys(lg, temps, seeds, int(step.reshape(-1)[0]), n_offset)
    M = x.shape[0]
    out_keys[:M].copy_(keys)
    out_ids[:M].copy_(ids.to(out_ids.dtype))


def logits_argmax(logits, temps, seeds, step, out_keys, out_ids, n_offset: int = 0) -> None:
    keys, ids = sample_keys(logits, temps, seeds, int(step.reshape(-1)[0]), n_offset)
    M = logits.shape[0]
    out_keys[:M].copy_(keys)
    out_ids[:M].copy_(ids.to(out_ids.dtype))


def swiglu(gu, out, interleaved: bool = False) -> None:
    g = linout_sum(gu)
    F = out.shape[1]
    if interleaved:
        from ..models.layout import _inverse, gu_perm

        g = g.index_select(-1, _inverse(gu_perm(F)).to(g.device))
    y = torch.nn.functional.silu(g[:, :F]) * g[:, F:]
    out.copy_(y.to(out.dtype))


# ----- fused decode GEMMs (csrc/kernels/decode_gemm.hip) -----------------------------------------
def unshuffled(W, wshuf: bool):
    """Row-major view of a decode weight stored MFMA-preshuffled (models/layout.py::preshuffle)."""
    if not wshuf:
        return W
    from ..models.layout import unshuffle

    return unshuffle(W)


def _row_scale(ss_in, eps: float, K: int, M: int):
    if ss_in is None:
        return None
    return torch.rsqrt(ss_in[:M].float().sum(-1, keepdim=True) / K + eps)


def _dg(x, W, ss_in, eps):
    y = _mm(x, W)
    rn = _row_scale(ss_in, eps, x.shape[1], x.shape[0])
    return y if rn is None else y * rn


def dg_f32(x, W, ss_in, eps, y) -> None:
    y[: x.shape[0]].copy_(_dg(x, W, ss_in, eps))


def dg_qkv(x, W, ss_in, eps, positions, slots, cos_sin, q_out, k_cache, v_cache, Hq: int, Hkv: int) -> None:
    rope_cache(_dg(x, W, ss_in, eps), positions, slots, cos_sin, q_out, k_cache, v_cache, Hq, Hkv, perm=True)


def dg_resid(x, W, resid, w_next, xw_out, ss_out) -> None:
    M = x.shape[0]
    r = resid[:M]
    r.add_(_mm(x, W))
    xw_out[:M].copy_((r * w_next.float()).to(xw_out.dtype))
    ss_out[:M].copy_(r.pow(2).view(M, -1, 16).sum(-1))


def dg_swiglu(x, W, ss_in, eps, act) -> None:
    swiglu(_dg(x, W, ss_in, eps), act[: x.shape[0]], interleaved=True)


def dg_argmax(x, W, ss_in, eps, temps, seeds, step, tile_keys, out_keys, out_ids, n_offset: int, logits=None) -> None:
    lg = _dg(x, W, ss_in, eps)
    if logits is not None:
        logits[: x.shape[0]].copy_(lg)
    keys, ids = sample_keys(lg, temps, seeds, int(step.reshape(-1)[0]), n_offset)
    M = x.shape[0]
    out_keys[:M].copy_(keys)
    out_ids[:M].copy_(ids.to(out_ids.dtype))


def resolve_ids(ids, src=None, prev=None):
    """Token per row: prev[src] where src >= 0 (previous step's on-device samples), else ids."""
    if src is None:
        return ids.long()
    s = src[: ids.numel()].long()
    return torch.where(s >= 0, prev.long()[s.clamp(min=0)], ids.long())


def embed_prep(ids, table, resid, w, xw, ss, src=None, prev=None) -> None:
    T = ids.numel()
    r = table[resolve_ids(ids, src, prev)].float()
    resid[:T].copy_(r)
    xw[:T].copy_((r * w.float()).to(xw.dtype))
    if ss.dim() == 2 and ss.shape[1] > 1:  # [>=T, P]: partial sums over P column slices of each row
        ss[:T].copy_(r.pow(2).view(T, ss.shape[1], -1).sum(-1))
    else:
        ss.view(-1)[:T].copy_(r.pow(2).sum(-1))  # ss: [>=T] or [>=T, 1] (one tile per row)


def add_prep(delta, resid, w, xw, ss) -> None:
    d = linout_sum(delta)
    T = d.shape[0]
    r = resid[:T]
    r.add_(d)
    xw[:T].copy_((r * w.float()).to(xw.dtype))
    if ss.dim() == 2 and ss.shape[1] > 1:  # [>=T, P]: partial sums over P column slices of each row
        ss[:T].copy_(r.pow(2).view(T, ss.shape[1], -1).sum(-1))
    else:
        ss.view(-1)[:T].copy_(r.pow(2).sum(-1))  # ss: [>=T] or [>=T, 1] (one tile per row)


def rownorm(xw, ss, eps, out) -> None:
    T, d = out.shape
    rn = torch.rsqrt(ss[:T].float().sum(-1, keepdim=True) / d + eps)
    out.copy_((xw[:T].float() * rn).to(out.dtype))


def rope_table(max_pos: int, head_dim: int, theta: float, scaling: dict | None = None,
               device="cpu") -> torch.Tensor:
    """``[max_pos, D]`` fp32 table ``[cos | sin]`` incl. Llama-3.1 NTK-by-parts scaling."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling["factor"]
        lo, hi = scaling.get("low_freq_factor", 1.0), scaling.get("high_freq_factor", 4.0)
        old = scaling.get("original_max_position_embeddings", 8192)
        lo_wl, hi_wl = old / lo, old / hi
        wl = 2 * math.pi / inv
        smooth = (old / wl - lo) / (hi - lo)
        scaled = torch.where(wl > lo_wl, inv / factor, inv)
        mid = (wl <= lo_wl) & (wl >= hi_wl)
        scaled = torch.where(mid, (1 - smooth) * inv / factor + smooth * inv, scaled)
        inv = scaled
    pos = torch.arange(max_pos, dtype=torch.float64)
    ang = pos[:, None] * inv[None, :]
    return torch.cat([ang.cos(), ang.sin()], dim=-1).float().to(device)


# ----- MoE ---------------------------------------------------------------------------------------
def moe_route_permute(logits, x, k: int, E: int, ids, w, counts, offsets, cursor, xs, dst) -> None:
    """Top-k routing (softmax over the selected logits), expert segments in token order."""
    T = x.shape[0]
    lg = linout_sum(logits)[:, :E]
    topv, topi = torch.topk(lg, k, dim=-1)  # ties -> lower index first (same as the kernel)
    wt = torch.softmax(topv, dim=-1)
    ids[: T * k].copy_(topi.reshape(-1).to(ids.dtype))
    w[: T * k].copy_(wt.reshape(-1))
    flat = topi.reshape(-1)
    cnt = torch.bincount(flat, minlength=E)[:E]
    counts[:E].copy_(cnt.to(counts.dtype))
    off = torch.zeros(E + 1, dtype=torch.int64)
    off[1:] = torch.cumsum(cnt, 0)
    offsets[: E + 1].copy_(off.to(offsets.dtype))
    cur = off[:-1].clone()
    rows = torch.empty(T * k, dtype=torch.int64)
    for a in range(T * k):
        e = int(flat[a])
        rows[a] = cur[e]
        cur[e] += 1
    dst[: T * k].copy_(rows.to(dst.dtype))
    xs[rows] = x[torch.arange(T * k) // k].to(xs.dtype)


def moe_route(logits, T: int, k: int, E: int, ids, w) -> None:
    lg = linout_sum(logits)[:T, :E]
    topv, topi = torch.topk(lg, k, dim=-1)  # ties -> lower index first (same as the kernel)
    ids[: T * k].copy_(topi.reshape(-1).to(ids.dtype))
    w[: T * k].copy_(torch.softmax(topv, dim=-1).reshape(-1))


def moe_align(ids, G: int, counts, offsets, cursor) -> None:
    v = ids.long()
    v = v[(v >= 0) & (v < G)]
    cnt = torch.bincount(v, minlength=G)[:G]
    counts[:G].copy_(cnt.to(counts.dtype))
    off = torch.zeros(G + 1, dtype=torch.int64)
    off[1:] = torch.cumsum(cnt, 0)
    offsets[: G + 1].copy_(off.to(offsets.dtype))
    cursor[:G].zero_()


def moe_scatter(x, ids, k: int, G: int, offsets, cursor, xs, dst, src_tok=None) -> None:
    """Rows into group segments in assignment order (the kernel's order within a segment varies; every
    consumer indexes through dst, so results agree)."""
    T = x.shape[0]
    R = xs.shape[0]
    for a in range(T * k):
        g = int(ids[a])
        if g < 0 or g >= G:
            continue
        row = int(offsets[g]) + int(cursor[g])
        cursor[g] += 1
        dst[a] = row
        if 0 <= row < R:
            xs[row] = x[a // k].to(xs.dtype)
            if src_tok is not None:
                src_tok[row] = a // k


def grouped_gemm(xs, W, offsets, e0: int, y, mode: int) -> None:
    """Y[rows of e] = Xs[rows of e] . W[e]^T (mode 0 bf16 / 1 fp32), or SwiGLU of the [gate; up] product;
    mode + 4: W MFMA-preshuffled per expert."""
    if mode & 4:
        from ..models.layout import unshuffle

        W = torch.stack([unshuffle(W[e]) for e in range(W.shape[0])])
        mode &= 3
    for e in range(W.shape[0]):
        a, b = int(offsets[e0 + e]), int(offsets[e0 + e + 1])
        if b <= a:
            continue
        p = _mm(xs[a:b], W[e])
        if mode == 2:
            F = p.shape[1] // 2
            p = torch.nn.functional.silu(p[:, :F]) * p[:, F:]
        y[a:b] = p.to(y.dtype)


def grouped_skinny(xs, W, offsets, e0: int, y) -> None:
    S = y.shape[0]
    y.zero_()
    for e in range(W.shape[0]):
        a, b = int(offsets[e0 + e]), int(offsets[e0 + e + 1])
        if b > a:
            y[0, a:b] = _mm(xs[a:b], W[e])


def moe_combine(y, dst, ids, e_lo: int, e_hi: int, w, k: int, out, accumulate: bool) -> None:
    T, d = out.shape
    yy = linout_sum(y)
    res = torch.zeros(T, d, dtype=torch.float32)
    for t in range(T):
        for j in range(k):
            a = t * k + j
            e = int(ids[a])
            if e_lo <= e < e_hi and int(dst[a]) >= 0:
                res[t] += float(w[a]) * yy[int(dst[a])]
    if accumulate:
        out.add_(res)
    else:
        out.copy_(res)


def moe_owner_pack(y, dst, ids, w, e_lo: int, e_hi: int, k: int, S: int, cursor, send, side) -> None:
    """Weighted partial over each token's local experts ([e_lo, e_hi)), one row per token that has one, pushed
    into its slice owner's block (owner = t // S; token order here, arrival order on the GPU: the owner's
    combine does not depend on it); side = the token's index in the owner's slice."""
    N = cursor.numel()
    cap = send.shape[0] // N
    T = dst.numel() // k
    yy = linout_sum(y)
    cursor.zero_()
    for t in range(T):
        row = None
        for j in range(k):
            a = t * k + j
            e = int(ids[a])
            if e_lo <= e < e_hi and int(dst[a]) >= 0:
                v = float(w[a]) * yy[int(dst[a])]
                row = v if row is None else row + v
        if row is None:
            continue
        o = t // S
        c = int(cursor[o])
        cursor[o] += 1
        send[o * cap + c] = row
        side[o * cap + c] = t - o * S


def moe_owner_combine(recv, side, rcnt, Tr: int, pos, out) -> None:
    """out [S, d] bf16: row t = sum over sources (rank order) of the received partial for slice token t."""
    N = rcnt.numel()
    cap = recv.shape[0] // N
    S, d = out.shape
    acc = torch.zeros(S, d, dtype=torch.float32)
    pos.view(-1)[: N * S] = -1
    for s in range(N):
        for i in range(min(int(rcnt[s]), cap)):
            t = int(side[s * cap + i])
            if 0 <= t < S:
                pos[s * S + t] = i
    for t in range(Tr):
        for s in range(N):
            p = int(pos[s * S + t])
            if p >= 0:
                acc[t] += recv[s * cap + p].float()
    out.copy_(acc.to(out.dtype))


def sample_filtered(logits, temps, top_k, top_p, seeds, step, out_ids) -> None:
    """Temperature + top-k + top-p (nucleus) resampling of full-vocab rows (csrc/kernels/sampling.hip).

    Kept set = {tokens whose logit >= the k-th largest} intersected with the smallest descending prefix
    whose probability mass reaches top_p (ties at the threshold are kept).  Rows with t == 0 or without a
    filter are left untouched.  Same RNG stream as the fused lm_head sampler."""
    st = int(step.reshape(-1)[0])
    B, V = logits.shape
    for r in range(B):
        t, k, p = float(temps[r]), int(top_k[r]), float(top_p[r])
        use_k, use_p = 0 < k < V, p < 1.0
        if t <= 0 or not (use_k or use_p):
            continue
        l = logits[r].float()
        thr = -float("inf")
        srt = torch.sort(l, descending=True).values
        if use_k:
            thr = max(thr, float(srt[k - 1]))
        if use_p:
            w = torch.exp((srt - srt[0]) / t)
            cum = torch.cumsum(w, 0)
            j = int(torch.searchsorted(cum, max(p, 0.0) * float(w.sum())).clamp(max=V - 1))
            thr = max(thr, float(srt[j]))
        seed = int(seeds[r]) & 0xFFFFFFFFFFFFFFFF
        mixed = seed ^ ((st << 20) & 0xFFFFFFFFFFFFFFFF)
        if mixed >= 1 << 63:
            mixed -= 1 << 64
        u = uniform01(torch.tensor(mixed, dtype=torch.int64), torch.arange(V, dtype=torch.int64)).float()
        v = l / t - torch.log(-torch.log(u.to(l.device)))
        v = torch.where(l >= thr, v, torch.full_like(v, -float("inf")))
        out_ids[r] = int(torch.argmax(v))


def moe_decode_route(resid, lnw, eps, Wr, k: int, ids, w, counts, offsets, cursor, xs, dst) -> None:
    """rms_norm + router logits + moe_route_permute (the fused decode routing kernel's contract)."""
    T, d = resid.shape
    xn = torch.empty(T, d, dtype=torch.bfloat16)
    rms_norm(resid, lnw, eps, xn)
    logits = _mm(xn, Wr)
    moe_route_permute(logits, xn, k, Wr.shape[0], ids, w, counts, offsets, cursor, xs, dst)


def moe_combine_prep(y, dst, ids, E: int, w, k: int, resid, w_next, xw, ss) -> None:
    """moe_combine over every expert + add_prep (one sum-of-squares partial per row)."""
    T, d = resid.shape
    out = torch.empty(T, d, dtype=torch.float32)
    moe_combine(y, dst, ids, 0, E, w, k, out, False)
    add_prep(out, resid, w_next, xw, ss)


# ======================================================================================================
# torch references of the latent-attention model family's ops (CPU path of symmetry_amd.ops; same contracts:
# outputs written in place, activations in the tensors' own dtype, statistics / scores / sums in fp32)
# ======================================================================================================
def embed_rows(ids, table, x, hist0) -> None:
    v = table[ids.long()].float()
    x.copy_(v)
    hist0.view_as(x).copy_(v)


def token_shift(x, mu, prev_row, state, h) -> None:
    T = x.shape[0]
    pr = prev_row[:T].long()
    prev = torch.zeros_like(x)
    rows = pr >= 0
    prev[rows] = x[pr[rows]]
    st = pr <= -2
    prev[st] = state[-(pr[st] + 2)]
    h.copy_((x + (prev - x) * mu.float()).to(h.dtype))


def _ln(v, w, eps):
    mean = v.mean(-1, keepdim=True)
    var = ((v - mean) ** 2).mean(-1, keepdim=True)
    return (v - mean) / torch.sqrt(var + eps) * w.float()


def add_layer_norm(delta, w, eps, x, save, state, hist, coef, hist_idx, out_act) -> None:
    T = x.shape[0]
    if save is not None:
        sv = save[:T].long()
        keep = sv >= 0
        state[sv[keep]] = x[keep]
    xn = x + _ln(delta.float().view_as(x), w, eps)
    if hist is not None:
        hist[hist_idx].copy_(xn)
        xn = (coef.float().view(-1, 1, 1) * hist[: hist_idx + 1]).sum(0)
    x.copy_(xn)
    if out_act is not None:
        out_act.copy_(xn.to(out_act.dtype))


def layer_norm(x, rows, w, eps, out) -> None:
    n = out.shape[0]
    v = x[rows[:n].long()] if rows is not None else x[:n]
    out.copy_(_ln(v, w, eps).to(out.dtype))


def rope_pair_table(max_pos: int, dims: int, base: float, device=None) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = (torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)).float()  # angles are fp32 products
    a = torch.arange(max_pos, dtype=torch.float32)[:, None] * freq[None, :]
    a = a.double()
    return torch.stack([torch.cos(a), torch.sin(a)], -1).float().to(device or "cpu")


def _rot_pairs(v, cs):
    """v [..., rot] fp32, cs [..., rot/2, 2] broadcastable."""
    u, w = v[..., 0::2], v[..., 1::2]
    c, s = cs[..., 0], cs[..., 1]
    return torch.stack([u * c - w * s, w * c + u * s], -1).flatten(-2)


def _rot_half(v, cs, dims):
    """Half layout: entry i < dims / 2 pairs with entry i + dims / 2 (table pair i); entries past ``dims`` pass."""
    h = dims // 2
    u, w = v[..., :h], v[..., h:dims]
    c, s = cs[..., :h, 0], cs[..., :h, 1]
    return torch.cat([u * c - w * s, w * c + u * s, v[..., dims:]], -1)


def _rot(v, cs, half_dims):
    return _rot_half(v, cs, half_dims) if half_dims else _rot_pairs(v, cs)


def latent_prep(z, q_rank, kv_rank, rot, wq, wkv, eps, positions, slots, rope, cq, cache, half_dims=0) -> None:
    T = z.shape[0]
    zf = z.float()
    q = zf[:, :q_rank]
    cq.copy_((q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * wq.float()).to(cq.dtype))
    if not kv_rank:
        return
    c = zf[:, q_rank:q_rank + kv_rank]
    c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * wkv.float()
    kr = _rot(zf[:, q_rank + kv_rank:q_rank + kv_rank + rot], rope[positions[:T].long()], half_dims)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    sl = slots[:T].long()
    keep = sl >= 0
    cache.view(-1, kv_rank + rot)[sl[keep]] = row[keep]


def rope_pairs(src, dst, positions, rope, half_dims=0) -> None:
    T = src.shape[0]
    dst.copy_(_rot(src.float(), rope[positions[:T].long()][:, None], half_dims).to(dst.dtype))


def latent_attn(q, cache, block_tables, row_seq, positions, scale, kv_rank, out, window=0) -> None:
    T, H, Dk = q.shape
    BS = cache.shape[1]
    o = out.view(T, H, kv_rank)
    for r in range(T):
        n = int(positions[r]) + 1
        bt = block_tables[int(row_seq[r])].long()
        idx = torch.arange(max(0, n - window) if window > 0 else 0, n)
        rows = cache[bt[idx // BS], idx % BS].float()          # [n, Dk]
        s = (q[r].float() @ rows.t()) * scale                   # [H, n]
        p = torch.softmax(s, -1)
        o[r] = (p @ rows[:, :kv_rank]).to(out.dtype)


def clamped_glu(gu, limit, alpha, out) -> None:
    F = out.shape[1]
    g = gu[:, :F].float().clamp(max=limit)
    u = gu[:, F:].float().clamp(-limit, limit)
    out.copy_((g * torch.sigmoid(alpha * g) * (u + 1)).to(out.dtype))


def sigmoid_topk(x, Wr, k, ids, w) -> None:
    T = x.shape[0]
    s = torch.sigmoid(x.float() @ Wr.float().t())
    top = s.topk(k, dim=-1)
    ids[: T * k].copy_(top.indices.reshape(-1).int())
    w[: T * k].copy_(top.values.reshape(-1))


def expert_offsets(ids, R, E, offsets, cursor) -> None:
    counts = torch.bincount(ids[:R].long(), minlength=E)
    offsets[0] = 0
    offsets[1:E + 1] = counts.cumsum(0).int()
    cursor[:E] = 0


def scatter_scaled(x, ids, w, k, offsets, cursor, xs, dst) -> None:
    R = x.shape[0] * k
    e = ids[:R].long()
    order = torch.sort(e, stable=True).indices       # assignment a lands at the rank of (expert, a)
    pos = torch.empty(R, dtype=torch.long)
    pos[order] = torch.arange(R)
    dst[:R] = pos.int()
    xs.view(R, -1)[pos] = (w[:R, None] * x.float().repeat_interleave(k, 0)).to(xs.dtype)


def grouped_linear(xs, W, offsets, y) -> None:
    offs = offsets.tolist()
    for e in range(W.shape[0]):
        a, b = offs[e], offs[e + 1]
        if b > a:
            y[a:b] = (xs[a:b].float() @ W[e].float().t()).to(y.dtype)


def gather_sum(y, dst, k, extra, out) -> None:
    T = out.shape[0]
    s = y.float()[dst[: T * k].long()].view(T, k, -1).sum(1)
    if extra is not None:
        s = s + extra.float().view_as(s)
    out.copy_(s)


# ======================================================================================================
# torch references of the hybrid family's ops (windowed attention beside decaying linear recurrences, state-space
# layers, parallel feed-forward; csrc/kernels/hybrid_*.hip).  Same contracts as the kernels: outputs in place,
# activations in the tensors' own dtype, everything the recurrences and statistics touch in fp32.
# ======================================================================================================
def _unit_rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def embed_norm(ids, table, w, eps, offset, x) -> None:
    x.copy_(_unit_rms(table[ids.long()].float(), eps) * (offset + w.float()))


def rms_norm_rows(x, rows, w, eps, offset, out) -> None:
    n = out.shape[0]
    v = x[rows[:n].long()] if rows is not None else x[:n]
    out.copy_((_unit_rms(v.float(), eps) * (offset + w.float())).to(out.dtype))


def residual_mix_norm(x, a, sa, bias_a, b, sb, c, sc, w, eps, offset, out) -> None:
    s = a.float().view_as(x)
    if bias_a is not None:
        s = s + bias_a.float()
    s = sa * s
    if b is not None:
        s = s + sb * b.float().view_as(x)
    if c is not None:
        s = s + sc * c.float().view_as(x)
    x.add_(s)
    if out is not None:
        out.copy_((_unit_rms(x, eps) * (offset + w.float())).to(out.dtype))


def rope_scaled_table(max_pos: int, dims: int, base: float, factor: float, original: float, fast: float, slow: float,
                      device=None) -> torch.Tensor:
    """[max_pos, dims / 2, 2] fp32 (cos, sin) * magnitude of the angles p * f_i; with factor > 0 the frequencies are
    blended towards f_i / factor over the pairs between the ones turning ``fast`` and ``slow`` times in ``original``
    positions, and the magnitude is 0.1 ln(factor) + 1.  Angles are fp32 products, cos / sin evaluated in double."""
    import math

    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    mag = 1.0
    if factor > 0:
        def at(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo, hi = max(math.floor(at(fast)), 0), min(math.ceil(at(slow)), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = (torch.arange(max_pos, dtype=torch.float32)[:, None] * f.float()[None, :]).double()
    return (torch.stack([torch.cos(a), torch.sin(a)], -1) * mag).float().to(device or "cpu")


def qkv_rope_cache(z, bias, H, G, dk, dv, positions, slots, rope, q_out, k_cache, v_cache, half_dims=0) -> None:
    T = z.shape[0]
    nq, nk, nv = H * dk, G * dk, G * dv
    zf = z[:, :nq + nk + nv].float()
    if bias is not None:
        zf = zf + bias.float()[:nq + nk + nv]
    if rope is not None:
        cs = rope[positions[:T].long()][:, None]                  # [T, 1, rot / 2, 2]
        rot = 2 * rope.shape[1]

        def turn(v):
            return _rot_half(v, cs, half_dims) if half_dims else torch.cat([_rot_pairs(v[..., :rot], cs), v[..., rot:]], -1)
    else:
        def turn(v):
            return v

    q_out.copy_(turn(zf[:, :nq].view(T, H, dk)).to(q_out.dtype))
    k = turn(zf[:, nq:nq + nk].view(T, G, dk)).to(k_cache.dtype)
    v = zf[:, nq + nk:].view(T, G, dv).to(v_cache.dtype)
    sl = slots[:T].long()
    keep = sl >= 0
    k_cache.view(-1, G, dk)[sl[keep]] = k[keep]
    v_cache.view(-1, G, dv)[sl[keep]] = v[keep]


def window_attn(q, k_cache, v_cache, block_tables, row_seq, positions, window, scale, gate, out, bias=None, keep_first=0,
                sink=None) -> None:
    T, H, dk = q.shape
    BS, G = k_cache.shape[1], k_cache.shape[2]
    rep = H // G
    for r in range(T):
        p = int(positions[r])
        j0 = max(0, p - window + 1)
        bt = block_tables[int(row_seq[r])].long()
        idx = torch.cat([torch.arange(0, min(keep_first, j0)), torch.arange(j0, p + 1)])
        K = k_cache[bt[idx // BS], idx % BS].float()            # [n, G, dk]
        V = v_cache[bt[idx // BS], idx % BS].float()
        qr = q[r].float().view(G, rep, dk)
        s = torch.einsum("grd,ngd->grn", qr, K) * scale
        if bias is not None:     # [2, H]: score -= bias[0, h] * ln(1 + bias[1, h] * distance)
            dist = (p - idx).float()
            s = s - (bias[0].float()[:, None] * torch.log1p(bias[1].float()[:, None] * dist[None, :])).view(G, rep, -1)
        if sink is not None:     # one more logit in the denominator, without a value
            s = torch.cat([s, sink.float().view(G, rep, 1)], -1)
            V = torch.cat([V, torch.zeros_like(V[:1])], 0)
        o = torch.einsum("grn,ngv->grv", torch.softmax(s, -1), V).reshape(H, -1)
        if gate is not None:
            o = o * torch.sigmoid(gate[r].float())[:, None]
        out[r] = o.to(out.dtype)


def _runs(T, cu_q, runs):
    if cu_q is None:
        return [(r, r + 1) for r in range(runs)]
    cu = cu_q.tolist()
    return [(cu[i], cu[i + 1]) for i in range(runs)]


def decay_scan(mode, q, k, v, dz, dbias, dparam, skip, q_scale, H, N, P, hpg, state, cu_q, prev_row, save_slot, runs,
               out, mout=None) -> None:
    """S <- diag(a_t) S + b_t k_t v_t^T, o_t = S^T (q_scale q_t) (+ skip_h v_t) per head over every run of rows.
    mode 0: a = sigmoid(dz + dbias) ** (1 / dparam) per key channel, b = 1;
    mode 1: b = softplus(dz + dbias[h]), a = exp(-exp(dparam[h]) * b) per head.  q / k of head h: group h // hpg.
    mode 2: log gates i = c tanh((dz[:, h] + dbias[h]) / c), f = logsigmoid(c tanh((dz[:, H + h] + dbias[H + h]) / c)),
    c = dparam; running maximum m_t = max(f + m_(t-1), i) (0 at a sequence's start, written to mout); a = exp(f + m_(t-1)
    - m_t), b = exp(i - m_t); the state and the output have one more column, fed by v = 1, and the state one more row
    that carries m (the same value in every column)."""
    T = q.shape[0]
    qf = q.float().reshape(T, -1, N) * q_scale
    kf, vf = k.float().reshape(T, -1, N), v.float().reshape(T, H, P)
    if mode == 0:
        ls = torch.nn.functional.logsigmoid(dz.float().reshape(T, H, N) + dbias.float().view(H, N))
        a = torch.exp(ls / float(dparam))                              # [T, H, N]
        b = torch.ones(T, H)
    elif mode == 1:
        b = torch.nn.functional.softplus(dz.float().reshape(T, H) + dbias.float(), beta=1.0, threshold=1e9)
        a = torch.exp(-torch.exp(dparam.float()) * b)[:, :, None].expand(T, H, N)
    else:
        c = float(dparam)
        g = c * torch.tanh((dz.float().reshape(T, 2 * H) + dbias.float()) / c)
        li, lf = g[:, :H], torch.nn.functional.logsigmoid(g[:, H:])
        vf = torch.cat([vf, torch.ones(T, H, 1)], -1)
        P = P + 1
    grp = torch.arange(H) // hpg
    o = out.view(T, H, P)
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 <= s0:
            continue
        pr = int(prev_row[s0])
        S = state[-(pr + 2)][:, :N].clone() if pr <= -2 else torch.zeros(H, N, P)
        if mode == 2:
            m = state[-(pr + 2)][:, N, 0].clone() if pr <= -2 else torch.zeros(H)
        for t in range(s0, s1):
            if mode == 2:
                mn = torch.maximum(lf[t] + m, li[t])
                at, bt = torch.exp(lf[t] + m - mn)[:, None].expand(H, N), torch.exp(li[t] - mn)
                m = mn
                mout[t] = m
            else:
                at, bt = a[t], b[t]
            S = at[:, :, None] * S + (bt[:, None] * kf[t, grp])[:, :, None] * vf[t][:, None, :]
            y = torch.einsum("hnp,hn->hp", S, qf[t, grp])
            if skip is not None:
                y = y + skip.float()[:, None] * vf[t]
            o[t] = y
        sv = int(save_slot[s1 - 1])
        if sv >= 0:
            state[sv][:, :N] = S
            if mode == 2:
                state[sv][:, N] = m[:, None]


def memory_norm_gate(y, m, gate, w, eps, out) -> None:
    """y [T, H, P + 1] (last column: the normaliser n . q), m [T, H]: o = y[..., :P] / (max(|n . q|, exp(-m)) + 1e-6),
    brought to unit RMS per head, times w, times sigmoid(gate)."""
    T, H, P1 = y.shape
    den = torch.maximum(y[..., -1].abs(), torch.exp(-m)) + 1e-6
    o = _unit_rms(y[..., :-1] / den[..., None], eps).reshape(T, H * (P1 - 1))
    out.copy_((o * w.float() * torch.sigmoid(gate.float())).to(out.dtype))


def gated_group_norm(y, gate, w, eps, group, gate_first, out) -> None:
    T, C = y.shape
    g = gate.float()
    g = g * torch.sigmoid(g)
    v = y * g if gate_first else y
    v = _unit_rms(v.view(T, C // group, group), eps).reshape(T, C)
    v = v * w.float().repeat(C // w.numel())
    out.copy_((v if gate_first else v * g).to(out.dtype))


def causal_conv_silu(xin, w, b, state, cu_q, prev_row, runs, out) -> None:
    T, C = out.shape
    taps = w.shape[1]
    wf, xf = w.float(), xin.float()
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 <= s0:
            continue
        pr = int(prev_row[s0])
        hist = state[-(pr + 2)].float() if pr <= -2 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, xf[s0:s1]], 0)
        y = b.float()[None, :].expand(s1 - s0, -1).clone()
        for j in range(taps):
            y = y + full[j:j + s1 - s0] * wf[:, j]
        out[s0:s1] = (y * torch.sigmoid(y)).to(out.dtype)


def conv_state_update(xin, state, cu_q, prev_row, save_slot, runs) -> None:
    T = xin.shape[0]
    keep = state.shape[1]
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 <= s0:
            continue
        sv = int(save_slot[s1 - 1])
        if sv < 0:
            continue
        pr = int(prev_row[s0])
        hist = state[-(pr + 2)] if pr <= -2 else torch.zeros_like(state[0])
        state[sv] = torch.cat([hist, xin[s0:s1].to(state.dtype)], 0)[-keep:] if keep else hist


def relu_sq(a, out) -> None:
    out.copy_((torch.relu(a.float()) ** 2).to(out.dtype))


def silu_mul(gate, up, out) -> None:
    g = gate.float()
    out.copy_((g * torch.sigmoid(g) * up.float()).to(out.dtype))


def softmax_topk(x, Wr, corr, k, ids, w, groups=1, keep=1, renorm=False) -> None:
    T = x.shape[0]
    s = torch.softmax(x.float() @ Wr.float().t(), -1)
    c = s + corr.float() if corr is not None else s
    if keep < groups:            # only the experts of the ``keep`` groups with the largest best entry stay eligible
        En = c.shape[1]
        gs = c.view(T, groups, En // groups).max(-1).values
        kept = torch.argsort(gs, dim=-1, descending=True, stable=True)[:, :keep]
        ok = torch.zeros(T, groups, dtype=torch.bool)
        ok.scatter_(1, kept, True)
        c = torch.where(ok.repeat_interleave(En // groups, 1), c, torch.full_like(c, -float("inf")))
    pick = torch.argsort(c, dim=-1, descending=True, stable=True)[:, :k]
    wt = torch.gather(s, 1, pick)
    if renorm:
        wt = wt / (wt.sum(-1, keepdim=True) + 1e-20)
    ids[: T * k].copy_(pick.reshape(-1).int())
    w[: T * k].copy_(wt.reshape(-1))


def moe_mix(y, dst, ids, w, k, E, h, shared, sgate, out) -> None:
    T = out.shape[0]
    e = ids[: T * k].long().view(T, k)
    rows = y.float()[dst[: T * k].long()].view(T, k, -1)
    rows = torch.where((e >= E)[:, :, None], h.float()[:, None, :], rows)
    s = (w[: T * k].view(T, k, 1) * rows).sum(1)
    if shared is not None:
        s = s + torch.sigmoid(sgate.float()).view(T, 1) * shared.float().view_as(s)
    out.copy_(s)


# ---- post-norm stream, input convolutions, normed grouped heads (the Komazen layers) ----------------------------
def embed_scale(ids, table, scale, x) -> None:
    x.copy_(table[ids.long()].float() * scale)


def residual_conv(x, w, state, cu_q, prev_row, runs, out) -> None:
    T, C = out.shape
    taps = w.shape[0]                      # w [taps, C]
    wf = w.float().t()
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 <= s0:
            continue
        pr = int(prev_row[s0])
        hist = state[-(pr + 2)].float() if pr <= -2 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, x[s0:s1]], 0)
        y = x[s0:s1].clone()
        for j in range(taps):
            y = y + full[j:j + s1 - s0] * wf[:, j]
        out[s0:s1] = y.to(out.dtype)


def post_rms_norm(x, alpha, delta, w, eps) -> None:
    x.copy_(_unit_rms(alpha * x + delta.float().view_as(x), eps) * w.float())


def qk_norm_cache(z, H, G, dk, dv, wq, wk, q_mult, eps, slots, q_out, k_cache, v_cache) -> None:
    T = z.shape[0]
    nq, nk, nv = H * dk, G * dk, G * dv
    zf = z[:, :nq + nk + nv].float()
    q = _unit_rms(zf[:, :nq].view(T, H, dk), eps) * wq.float()
    if q_mult is not None:
        q = q * q_mult.float()[None, :, None]
    q_out.copy_(q.to(q_out.dtype))
    k = (_unit_rms(zf[:, nq:nq + nk].view(T, G, dk), eps) * wk.float()).to(k_cache.dtype)
    v = zf[:, nq + nk:].view(T, G, dv).to(v_cache.dtype)
    sl = slots[:T].long()
    keep = sl >= 0
    k_cache.view(-1, G, dk)[sl[keep]] = k[keep]
    v_cache.view(-1, G, dv)[sl[keep]] = v[keep]


def gelu_tanh_mul(gate, up, out) -> None:
    g = gate.float()
    act = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
    out.copy_((act * up.float()).to(out.dtype))


def sigmoid_mul(a, gate, out) -> None:
    out.copy_((a.float() * torch.sigmoid(gate.float())).to(out.dtype))


# ---- several residual streams, hashed token pairs, convolved projections (the Dalalix layers) -------------------
def embed_pair_hash(ids, table, pair_table, buckets, mul_prev, mul_cur, prev_row, tok_state, x) -> None:
    """x [T, S, d]: every stream = table[token] + pair_table[(prev * mul_prev + token * mul_cur) mod buckets]; a row
    without a previous token takes pair_table[buckets]."""
    T = x.shape[0]
    tok = ids[:T].long()
    e = table[tok].float()
    if pair_table is not None:
        pr = prev_row[:T].long()
        prev = torch.where(pr >= 0, tok[pr.clamp(min=0)], tok_state[(-(pr + 2)).clamp(min=0)].long())
        rows = torch.where(pr == -1, torch.full_like(tok, buckets), (prev * mul_prev + tok * mul_cur) % buckets)
        e = e + pair_table[rows].float()
    x.copy_(e[:, None, :].expand_as(x))


def token_state_update(ids, tok_state, cu_q, save_slot, runs) -> None:
    T = ids.shape[0]
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 > s0 and int(save_slot[s1 - 1]) >= 0:
            tok_state[int(save_slot[s1 - 1])] = ids[s1 - 1]


def hyper_mix_norm(xs, a, sa, b, sb, mix, outc, inc, w, eps, rows, out) -> None:
    """xs [T, S, d] fp32.  With ``a``: y = sa a + sb b; xs[:, t] <- sum_s mix[s, t] xs[:, s] + outc[t] y.  Then
    out[i] = rms_norm(sum_s inc[s] xs[rows[i], s]) * w (inc None: the plain sum)."""
    if a is not None:
        y = sa * a.float()
        if b is not None:
            y = y + sb * b.float()
        xs.copy_(torch.einsum("st,nsd->ntd", mix.float(), xs)
                 + outc.float()[None, :, None] * y[:, None, :])
    if out is not None:
        src = xs if rows is None else xs[rows.long()]
        n = out.shape[0]
        u = src[:n].sum(1) if inc is None else torch.einsum("s,nsd->nd", inc.float(), src[:n])
        out.copy_((_unit_rms(u, eps) * w.float()).to(out.dtype))


def conv_qkv_cache(z, w, state, cu_q, prev_row, runs, H, G, dk, dv, v_eps, slots, q_out, k_cache, v_cache) -> None:
    """z [T, H dk | G dk | G dv] through a causal per-channel convolution (w [C, taps], no bias, inputs before a run
    from state [slots, taps - 1, C]); q -> q_out, k and the unit-RMS (per head, v_eps) v -> the paged caches."""
    T = z.shape[0]
    C, taps = w.shape
    nq, nk = H * dk, G * dk
    y = torch.zeros(T, C)
    zf, wf = z.float(), w.float()
    for s0, s1 in _runs(T, cu_q, runs):
        if s1 <= s0:
            continue
        pr = int(prev_row[s0])
        hist = state[-(pr + 2)].float() if pr <= -2 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, zf[s0:s1]], 0)
        for j in range(taps):
            y[s0:s1] += full[j:j + s1 - s0] * wf[:, j]
    q_out.copy_(y[:, :nq].view(T, H, dk).to(q_out.dtype))
    k = y[:, nq:nq + nk].view(T, G, dk).to(k_cache.dtype)
    v = _unit_rms(y[:, nq + nk:].view(T, G, dv), v_eps).to(v_cache.dtype)
    sl = slots[:T].long()
    keep = sl >= 0
    k_cache.view(-1, G, dk)[sl[keep]] = k[keep]
    v_cache.view(-1, G, dv)[sl[keep]] = v[keep]


def logit_softcap(logits, cap) -> None:
    logits.copy_(cap * torch.tanh(logits / cap))
