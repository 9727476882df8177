"""Plain, slow implementation of the Komazen design, one function per mechanism, written from the design's
equations.  It shares no code with the product path (no symmetry_amd import): whole-sequence recompute in float64,
no cache, no paging, no batching.  The tests compare the engine against it.

Notation: ``W`` maps checkpoint tensor names to tensors; matrices are stored [out, in] and applied as ``x @ M.T``;
``cfg`` is the checkpoint's config.json as a dict; positions count from 0.

    x = E[token] * embedding.scale
    per layer:   x = n(alpha x + mixer(x + conv1(x)), g1);   x = n(alpha x + ff(x + conv2(x)), g2)     (norm after the sum)
    logits = W_head n(x, g_f),      n(v, g) = v / sqrt(mean(v^2) + eps) * g
"""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def input_conv(h, w):
    """h [T, d] -> h + conv(h): per channel, conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j), zeros before the start."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_half(x, positions, base, dims):
    """Entries i and i + dims / 2 (i < dims / 2) of the last axis turn by positions * base^(-2 i / dims); entries past
    ``dims`` pass.  x [T, ..., D]."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    f = base ** (-2.0 * i / dims)
    a = positions.to(x.dtype)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def latent_pair(W, pre, m, h, positions, eps):
    """What a layer with a down-projection caches: the normed latent c [T, r] and the rotated shared key part [T, rot]."""
    r, rot = m["kv_rank"], m["rot_dim"]
    z = h @ W[pre + "dkv"].T
    c = rms_norm(z[:, :r], W[pre + "dkv.norm"], eps)
    kr = rotate_half(z[:, r:r + rot], positions, m["rot"]["base"], m["rot"]["dims"])
    return c, kr


def latent_attention(W, pre, m, h, positions, eps, c, kr):
    """Queries through a latent; keys / values from the latents (c, kr) of this or another layer; sliding window;
    elementwise sigmoid output gate."""
    H, dn, rot, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    cq = rms_norm(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].T).view(T, H, dn + rot)
    qn = q[..., :dn]
    qr = rotate_half(q[..., dn:], positions, m["rot"]["base"], m["rot"]["dims"])
    kn = (c @ W[pre + "uk"].T).view(T, H, dn)
    v = (c @ W[pre + "uv"].T).view(T, H, dv)
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * m["scale"]
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    visible = (dist >= 0) & (dist < m["mask"]["size"])
    s = s.masked_fill(~visible, float("-inf"))
    p = torch.softmax(s, -1)
    o = torch.einsum("hts,shd->thd", p, v).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def biased_attention(W, pre, m, h, eps):
    """Grouped heads, per-head RMS norm of queries and keys, no rotation; score = scale * temp_h * q.k - r1_h ln(1 + r2_h
    (i - j)); causal softmax."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_norm((h @ W[pre + "q"].T).view(T, H, dk), W[pre + "q.norm"], eps)
    k = rms_norm((h @ W[pre + "k"].T).view(T, G, dk), W[pre + "k.norm"], eps)
    v = (h @ W[pre + "v"].T).view(T, G, dv)
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).clamp(min=0).to(h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] * W[pre + "temp"][hd]
        s = s - W[pre + "r1"][hd] * torch.log(1.0 + W[pre + "r2"][hd] * dist)
        s = s.masked_fill(i[:, None] < i[None, :], float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, g]
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def gelu_ff(W, pre, h):
    return (gelu_tanh(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def forward(cfg: dict, W: dict, tokens, trace=None):
    """tokens (list of ids) -> logits [T, vocab] in float64.  ``trace``: a list that receives the stream after every
    layer."""
    W = {k: (v.double() if v.is_floating_point() else v) for k, v in W.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = W["embed"][ids] * cfg["embedding"]["scale"]
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        h = input_conv(x, W[pre + "canon1"])
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_pair(W, pre + "mix.", m, h, positions, eps)
                src = i
            a = latent_attention(W, pre + "mix.", m, h, positions, eps, *latents[src])
        elif layer["type"] == "attention":
            a = biased_attention(W, pre + "mix.", m, h, eps)
        else:
            raise ValueError(layer["type"])
        x = rms_norm(alpha * x + a, W[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            h = input_conv(x, W[pre + "canon2"])
            x = rms_norm(alpha * x + gelu_ff(W, pre + "mlp.", h), W[pre + "norm2"], eps)
        if trace is not None:
            trace.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T
