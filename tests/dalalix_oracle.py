"""Plain, slow implementation of the Dalalix design, one function per mechanism, written from the design's equations.
It shares no code with the product path (no symmetry_amd import): whole-sequence recompute in float64, no cache, no
paging, no batching.  The tests compare the engine against it.

Notation: ``W`` maps checkpoint tensor names to tensors; matrices are stored [out, in] and applied as ``x @ M.T``;
``cfg`` is the checkpoint's config.json as a dict; positions count from 0.

    e_t = E[tok_t] + B[(tok_(t-1) a + tok_t b) mod n]        (t = 0: the extra last row of B)
    streams X_1 .. X_S = e;  per sublayer:  u = sum_s c_in[s] X_s;  y = f(n(u, g));  X_t' = sum_s M[s, t] X_s + c_out[t] y
    logits = cap tanh(W_head n(sum_s X_s, g_f) / cap),       n(v, g) = v / sqrt(mean(v^2) + eps) * g
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def embed_tokens(W, cfg, tokens):
    """Token rows plus the hashed pair rows: the pair (previous token, token) picks a row of ``bigram``; the first token
    of a sequence takes the table's extra last row."""
    x = W["embed"][tokens].clone()
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        n = int(bg["buckets"])
        rows = [n] + [(int(tokens[t - 1]) * int(bg["mul_prev"]) + int(tokens[t]) * int(bg["mul_cur"])) % n
                      for t in range(1, len(tokens))]
        x = x + W["bigram"][torch.tensor(rows)]
    return x


def rotate_half(x, positions, base, dims):
    """Entries i and i + dims / 2 (i < dims / 2) of the last axis turn by positions * base^(-2 i / dims); entries past
    ``dims`` pass.  x [T, heads, D]."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    f = base ** (-2.0 * i / dims)
    a = positions.to(x.dtype)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(i, j, window=None, keep_first=0):
    """Does position i see position j?  Causal; with a window only the newest ``window`` positions and the sequence's
    first ``keep_first``."""
    if j > i:
        return False
    return window is None or i - j < window or j < keep_first


def softmax_attention(q, k, v, scale, window=None, keep_first=0, sink=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H, dv].  Query head h reads key / value head h // (H / G).  With
    ``sink`` [H] the denominator of head h also holds exp(sink_h) (no key, no value, not scaled)."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        for i in range(T):
            idx = [j for j in range(T) if visible(i, j, window, keep_first)]
            row = s[i, idx]
            m = row.max() if sink is None else torch.maximum(row.max(), sink[h])
            e = torch.exp(row - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[idx, g]
    return out


def short_conv(u, w):
    """Causal per-channel convolution: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start.  u [T, C]."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def attention_plain(W, p, m, h):
    """Mixer "attention_2": biased projections, grouped heads, causal softmax, no positions."""
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, m["heads"], m["dim"])
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, m["kv_heads"], m["dim"])
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, m["kv_heads"], m["vdim"])
    o = softmax_attention(q, k, v, m["scale"])
    return o.reshape(T, -1) @ W[p + "o"].T


def attention_conv_gated(W, p, m, h, eps):
    """Mixer "attention": projections, a short causal convolution on q, k and v, unit-RMS values per head, causal
    softmax, an element-wise sigmoid gate from the same input, output projection."""
    T = h.shape[0]
    q = short_conv(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, m["heads"], m["dim"])
    k = short_conv(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, m["kv_heads"], m["dim"])
    v = short_conv(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, m["kv_heads"], m["vdim"])
    v = unit_rms(v, eps)
    o = softmax_attention(q, k, v, m["scale"]).reshape(T, -1)
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def attention_window_sink(W, p, m, h, positions):
    """Left half of "parallel": biased projections, rotation of part of each head (half layout), a sliding window that
    keeps the first tokens, a per-head sink in the softmax's denominator."""
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, m["heads"], m["dim"])
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, m["kv_heads"], m["dim"])
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, m["kv_heads"], m["vdim"])
    q = rotate_half(q, positions, m["rot"]["base"], m["rot"]["dims"])
    k = rotate_half(k, positions, m["rot"]["base"], m["rot"]["dims"])
    o = softmax_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"].get("keep_first", 0), W[p + "sink"])
    return o.reshape(T, -1) @ W[p + "o"].T


def matrix_memory(W, p, m, h, eps):
    """Right half of "parallel": a matrix memory per head with exponential input gate and a running maximum.

    i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)); m_t = max(f + m_(t-1), i), m_0 = 0;
    S_t = e^(f + m_(t-1) - m_t) S_(t-1) + e^(i - m_t) k v^T, n_t alike with k; o = S^T q / (max(|n . q|, e^(-m_t)) + 1e-6).
    Heads are brought to unit RMS, weighted, gated by sigmoid(W_g h) and projected."""
    T = h.shape[0]
    H, N, P, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, N) * N ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, N)
    v = (h @ W[p + "v"].T).view(T, H, P)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    out = torch.zeros(T, H, P, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(N, P, dtype=h.dtype)
        n = torch.zeros(N, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for t in range(T):
            mn = torch.maximum(fg[t, hd] + mx, ig[t, hd])
            a, b = torch.exp(fg[t, hd] + mx - mn), torch.exp(ig[t, hd] - mn)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            mx = mn
            den = torch.maximum(torch.abs(n @ q[t, hd]), torch.exp(-mx)) + 1e-6
            out[t, hd] = (S.T @ q[t, hd]) / den
    o = unit_rms(out, eps).reshape(T, -1) * W[p + "norm"]
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def route(z, top, groups, keep):
    """Router: softmax over all experts; experts form ``groups`` equal groups of neighbours, a group scores as its best
    expert, only the ``keep`` best groups stay eligible; the ``top`` best eligible experts, weights = their scores over
    their sum.  z [E] -> (ids, weights, margin).  The margin says how far the choice is from another one, in units of the
    logits: the last chosen expert against the best eligible one left out, and the last kept group against the best one
    dropped; infinite where the expert that a flip would swap carries next to no weight."""
    s = torch.softmax(z, -1)
    E = s.shape[0]
    per = E // groups
    gs = s.view(groups, per).max(-1).values
    kept = torch.topk(gs, keep).indices
    ok = torch.zeros(E, dtype=torch.bool)
    for g in kept.tolist():
        ok[g * per:(g + 1) * per] = True
    masked = torch.where(ok, s, torch.full_like(s, -1.0))
    val, ids = torch.topk(masked, top)
    w = s[ids] / (s[ids].sum() + 1e-20)
    margin = math.inf
    if float(w[-1]) > 0.03:
        rest = torch.where(ok, z, torch.full_like(z, -math.inf))
        rest[ids] = -math.inf
        if top < int(ok.sum()):
            margin = float(z[ids[-1]] - rest.max())
        if keep < groups:
            gz = z.view(groups, per).max(-1).values
            gl = gz.clone()
            gl[kept] = -math.inf
            margin = min(margin, float(gz[kept].min() - gl.max()))
    return ids, w, margin


def expert(W, p, h, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def moe(W, p, f, h, margins=None):
    r = f["router"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ W[p + "router"].T
    out = torch.zeros_like(h)
    ms = []
    for t in range(h.shape[0]):
        ids, w, mg = route(z[t], r["top"], grp["count"], grp["keep"])
        ms.append(mg)
        for e, we in zip(ids.tolist(), w):
            out[t] += we * expert(W, f"{p}e{e}.", h[t], f["expert"]["limit"])
    if margins is not None:
        margins.append(torch.tensor(ms))
    return out


def mixer(W, cfg, L, p, h, positions):
    eps = cfg["norm"]["eps"]
    kind, m = L["type"], L["mixer"]
    if kind == "attention_2":
        return attention_plain(W, p + "mix.", m, h)
    if kind == "attention":
        return attention_conv_gated(W, p + "mix.", m, h, eps)
    if kind == "parallel":
        left = attention_window_sink(W, p + "mix.left.", m["left"], h, positions)
        right = matrix_memory(W, p + "mix.right.", m["right"], h, eps)
        return m["left_scale"] * left + m["right_scale"] * right
    raise ValueError(kind)


def forward(W, cfg, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of one sequence, float64.  ``layers_out`` (a list) receives the sum of the streams after every
    layer; ``margins`` one tensor [T] per routed sublayer: the routers' margins (see ``route``)."""
    W = {k: v.to(F64) for k, v in W.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T)
    eps = cfg["norm"]["eps"]
    e = embed_tokens(W, cfg, tokens)
    S = cfg.get("streams")
    X = [e.clone() for _ in range(S or 1)]
    for i, L in enumerate(cfg["layers"]):
        j = i
        while cfg["layers"][j].get("weights_of") is not None:      # (a borrowed layer may itself borrow)
            j = cfg["layers"][j]["weights_of"]
        p = f"l{j}."
        subs = [(1, lambda h: mixer(W, cfg, L, p, h, positions))]
        if L.get("mlp") is not None:
            subs.append((2, lambda h: moe(W, p + "mlp.", L["mlp"], h, margins)))
        for q, f in subs:
            if S:
                cin, cout, M = W[f"{p}hc{q}.in"], W[f"{p}hc{q}.out"], W[f"{p}hc{q}.mix"]
                u = sum(cin[s] * X[s] for s in range(S))
                y = f(rms_norm(u, W[f"{p}norm{q}"], eps))
                X = [sum(M[s, t] * X[s] for s in range(S)) + cout[t] * y for t in range(S)]
            else:
                X = [X[0] + f(rms_norm(X[0], W[f"{p}norm{q}"], eps))]
        if layers_out is not None:
            layers_out.append(sum(X))
    logits = rms_norm(sum(X), W["final.norm"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
