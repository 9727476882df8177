"""Komazen decoder forward on the symmetry_amd ops: one code path for CPU (torch references) and MI355X (HIP).

The design, in this file's notation (x: the fp32 stream, one row per token; W stored [out, in]; n(v, g) =
v / sqrt(mean(v^2) + eps) * g; c(v) = v + a causal per-channel convolution of v over the sequence's rows)::

    x = E[token] * embed_scale
    per layer:   x = n(alpha x + mixer(c1(x)), g1);   x = n(alpha x + ff(c2(x)), g2)      (the norm comes after the sum)
    logits = W_head n(x, g_f)

    mixer "latent_attention" (H heads; per head dn unrotated + rot rotated query/key dims, dv value dims; ranks rq, r):
      c_q = n(W_dq h, g_q)              q = W_uq c_q = [q_n | q_r] per head, q_r rotated (entry i with i + dims / 2)
      [c' | k'] = W_dkv h               c = n(c', g_kv), k_r = rotary(k')                 -- the cache row [c | k_r]
      score_h(t, j) = scale (q_n . W_uk,h c_j + q_r . k_r,j) over t - window < j <= t, softmax,
      out = W_o ((W_uv,h sum_j p_j c_j)_h * sigmoid(W_g h))
      evaluated with the up-projections folded into the query / output (ops.latent_attn: multi-query attention over
      the paged latent cache).  A layer with ``kv_from`` = j has no W_dkv and attends layer j's plane.
    mixer "attention" (H query heads on G key / value heads, no rotation):
      q = n_head(W_q h, g_q) temp_h,  k = n_head(W_k h, g_k),  v = W_v h
      score_h(t, j) = scale q . k - r1_h ln(1 + r2_h (t - j)) over j <= t, softmax, W_o
    ff: W_down (gelu_tanh(W_gate h) * W_up h)

Every projection that reads a sublayer's input is one row block of one fused weight (a single library GEMM); the
kernels take column ranges of its output as views.  Step launches per layer: GEMM (the mixer's projections),
then latent: latent_prep, GEMM W_uq, bmm (absorb W_uk), rope_pairs, latent_attn, bmm (W_uv), sigmoid_mul, GEMM W_o
     plain:  qk_norm_cache, window_attn (distance bias), GEMM W_o
post_rms_norm, residual_conv, conv_state_update; GEMM gate|up, gelu_tanh_mul, GEMM down; post_rms_norm, residual_conv,
conv_state_update (the next layer's input).  In decode steps every row is a run of its own, and one post_rms_norm launch
norms the stream, convolves with the row's carried taps and moves them on.
All intermediates live in the preallocated Workspace, so decode steps are hipGraph-capturable.

fp32 in both serving dtypes: the stream, the convolutions' carried inputs, norm statistics, rotary angles, attention
scores / weights / distance bias.  ``dtype=torch.float32`` runs every product in true 32-bit as well.
"""
from __future__ import annotations

import torch

from .. import ops
from .config import KomazenConfig
from .transformer import MAX_STEP_SEQS, ForwardBatch, Workspace
from .weights import ModelWeights

SEG_ALIGN = 8             # row blocks of a fused projection start at multiples of 8 columns (16-byte bf16 accesses)
NO_WINDOW = 1 << 30       # window of a plainly causal layer for the windowed attention kernels


class KomazenCache:
    """What the model keeps per sequence.

    ``lat``: one plane [NB, BS, r + rot] per latent-attention layer that owns a down-projection (a row = normalised
    latent | rotated shared key part; layers with ``kv_from`` read their source's plane); ``k`` / ``v``: one pair of
    planes [NB, BS, G, dk] / [NB, BS, G, dv] per plain attention layer.  All planes share the engine's BlockManager
    numbering, so one block table serves them.  ``conv`` [2 L, slots, taps - 1, d] fp32: per layer and sublayer the
    newest taps - 1 rows of the stream that the sublayer's input convolution has seen.  Slots are handed out by the
    scheduler's StateSlotManager; a new sequence never reads a slot's old content (its first run starts from zeros).
    Zero-initialised: every byte finite."""

    def __init__(self, cfg: KomazenConfig, num_blocks: int, block_size: int, num_slots: int, device, dtype):
        self.num_layers, self.num_blocks, self.block_size = cfg.num_layers, num_blocks, block_size
        self.lat, self.k, self.v = {}, {}, {}
        for i in cfg.latent_layers():
            m = cfg.layers[i].mixer
            self.lat[i] = torch.zeros(num_blocks, block_size, m.kv_rank + m.rot_dim, device=device, dtype=dtype)
        for i in cfg.attn_layers():
            m = cfg.layers[i].mixer
            self.k[i] = torch.zeros(num_blocks, block_size, m.kv_heads, m.dim, device=device, dtype=dtype)
            self.v[i] = torch.zeros(num_blocks, block_size, m.kv_heads, m.vdim, device=device, dtype=dtype)
        self.conv = torch.zeros(2 * cfg.num_layers, num_slots, cfg.conv_taps - 1, cfg.hidden_size, device=device,
                                dtype=torch.float32)

    def nbytes(self) -> int:
        planes = list(self.lat.values()) + list(self.k.values()) + list(self.v.values()) + [self.conv]
        return sum(t.numel() * t.element_size() for t in planes)


def _fuse(blocks: list) -> tuple:
    """Row blocks [(name, weight)] -> (one weight, name -> (first output column, width)), blocks padded to SEG_ALIGN."""
    parts, cols, n = [], {}, 0
    for name, w in blocks:
        cols[name] = (n, w.shape[0])
        parts.append(w)
        n += w.shape[0]
        pad = -n % SEG_ALIGN
        if pad:
            parts.append(torch.zeros(pad, w.shape[1], dtype=w.dtype, device=w.device))
            n += pad
    return torch.cat(parts, 0).contiguous(), cols


class KomazenLM:
    has_seq_state = True      # the engine allots a state slot per live sequence and sends prev_row / save_slot / row_seq
    fused = False
    single_copy = False
    moe = None
    tp = None

    def __init__(self, weights: ModelWeights, device, tp_comm=None, ep_comm=None, max_decode_ctx: int | None = None,
                 decode_weights: str = "auto", kv_reserve_bytes: int = 0, dtype=torch.bfloat16):
        if weights.shard.tp_size > 1 or weights.shard.ep_size > 1:
            raise NotImplementedError("Komazen runs on one GPU per replica")
        self.cfg: KomazenConfig = weights.cfg
        self.w = weights
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp_size, self.tp_rank = 1, 0
        self.ws = Workspace()
        self.last_ids = torch.zeros(MAX_STEP_SEQS, dtype=torch.int32, device=self.device)
        self.last_logits = None
        cfg = self.cfg
        max_pos = min(cfg.max_position, max_decode_ctx or cfg.max_position)
        self._rope: dict = {}
        self.L = [self._prepare_layer(i, max_pos) for i in range(cfg.num_layers)]
        self.embed = weights["embed"].to(dtype)
        self.final_norm = weights["final.norm"].float()
        self.head = weights["head"].to(dtype)

    # ------------------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, num_slots: int) -> KomazenCache:
        return KomazenCache(self.cfg, num_blocks, block_size, num_slots, self.device, self.dtype)

    def extra_weight_bytes(self) -> int:
        return 0

    def _rope_table(self, m, max_pos: int) -> torch.Tensor:
        """[max_pos, rot_dim / 2, 2] (cos, sin): the first rot.dims / 2 pairs turn, the others are the identity."""
        key = (m.rot_dim, m.rot_dims, m.rot_base, max_pos)
        if key not in self._rope:
            t = torch.zeros(max_pos, m.rot_dim // 2, 2, dtype=torch.float32)
            t[..., 0] = 1.0
            t[:, : m.rot_dims // 2] = ops.rope_pair_table(max_pos, m.rot_dims, m.rot_base)
            self._rope[key] = t.to(self.device)
        return self._rope[key]

    def _prepare_layer(self, i: int, max_pos: int) -> dict:
        """The fused / converted tensors layer i's launches read.  Matrices in the activation dtype; norm weights,
        convolution taps, temperatures and bias parameters in fp32."""
        w, layer, dt = self.w, self.cfg.layers[i], self.dtype
        m = layer.mixer
        p = f"l{i}."

        def t(name):
            return w[p + name].to(dt)

        def f(name):
            return w[p + name].float().contiguous()

        def taps(name):      # [width, taps] in the checkpoint -> tap-major, so that neighbouring channels load together
            return w[p + name].float().t().contiguous()

        P = {"kind": layer.type, "mixer": m, "mlp": layer.mlp, "norm1": f("norm1"), "canon1": taps("canon1"), "o": t("mix.o")}
        if layer.type == "latent_attention":
            if m.kv_rank > 512:
                raise NotImplementedError(f"layer {i}: kv_rank {m.kv_rank} > 512 (latent_attn's accumulator registers)")
            owner = m.kv_from is None
            # (the kv part follows the query latent directly: latent_prep reads them as one column range)
            lat = torch.cat([t("mix.dq"), t("mix.dkv")], 0) if owner else t("mix.dq")
            P["w_in"], P["cols"] = _fuse([("lat", lat), ("g", t("mix.g"))])
            P["owner"], P["plane_of"] = owner, i if owner else m.kv_from
            P["gq"], P["gkv"] = t("mix.dq.norm"), t("mix.dkv.norm") if owner else None
            P["uq"] = t("mix.uq")
            P["uk"] = t("mix.uk").view(m.heads, m.dim, m.kv_rank)                     # [H, dn, r]: q_n @ uk[h]
            P["uvt"] = t("mix.uv").view(m.heads, m.vdim, m.kv_rank).transpose(1, 2)   # [H, r, dv] view
            P["rope"] = self._rope_table(m, max_pos)
        else:
            if m.vdim > 512:
                raise NotImplementedError(f"layer {i}: value heads wider than 512")
            P["w_in"], P["cols"] = _fuse([("qkv", torch.cat([t("mix.q"), t("mix.k"), t("mix.v")], 0))])
            P["gq"], P["gk"] = f("mix.q.norm"), f("mix.k.norm")
            P["temp"] = f("mix.temp")
            P["bias"] = torch.stack([f("mix.r1"), f("mix.r2")]).contiguous()           # [2, H]
        if layer.mlp is not None:
            P["norm2"], P["canon2"] = f("norm2"), taps("canon2")
            P["w_gu"] = torch.cat([t("mlp.gate"), t("mlp.up")], 0).contiguous()
            P["w_down"] = t("mlp.down")
        return P

    # ------------------------------------------------------------------------------------------
    def _buf(self, name, shape, dtype=None):
        return self.ws.get(name, shape, dtype or self.dtype, self.device)

    def _linear(self, name: str, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [R, K] @ w[N, K]^T -> [R, N] in the activation dtype (library GEMM, fp32 accumulation)."""
        return ops.linear(x, w, out=self._buf(name, (x.shape[0], w.shape[0])))

    @staticmethod
    def _cols(z: torch.Tensor, P: dict, name: str) -> torch.Tensor:
        c0, n = P["cols"][name]
        return z[:, c0:c0 + n]

    def _conv(self, b: ForwardBatch, x: torch.Tensor, w: torch.Tensor, state: torch.Tensor, runs: int) -> torch.Tensor:
        """The sublayer input x + conv(x) in the activation dtype; the run's newest rows of x become the carried taps."""
        h = self._buf("h", x.shape)
        if b.kind == "decode":      # every row a run of its own: one launch convolves and moves the carried taps on
            ops.residual_conv(x, w, state, None, b.row_seq, b.prev_row, runs, h, save_slot=b.save_slot)
        else:
            ops.residual_conv(x, w, state, b.cu_q, b.row_seq, b.prev_row, runs, h)
            ops.conv_state_update(x, state, b.cu_q, b.prev_row, b.save_slot, runs)
        return h

    def _norm_conv(self, b: ForwardBatch, x: torch.Tensor, delta: torch.Tensor, w: torch.Tensor, conv, runs: int):
        """x <- n(alpha x + delta, w); then the next sublayer's input from ``conv`` = (taps, carried state), if there is
        one.  In decode steps one launch does both (a row is a run of its own there)."""
        alpha, eps = self.cfg.postln_alpha, self.cfg.norm_eps
        if conv is None:
            ops.post_rms_norm(x, alpha, delta, w, eps)
            return None
        if b.kind == "decode":
            h = self._buf("h", x.shape)
            ops.post_rms_norm(x, alpha, delta, w, eps, conv[0], conv[1], b.prev_row, b.save_slot, h)
            return h
        ops.post_rms_norm(x, alpha, delta, w, eps)
        return self._conv(b, x, conv[0], conv[1], runs)

    def _latent(self, P: dict, b: ForwardBatch, cache: KomazenCache, h: torch.Tensor) -> torch.Tensor:
        m = P["mixer"]
        T, H, r, rot, dn = h.shape[0], m.heads, m.kv_rank, m.rot_dim, m.dim
        plane = cache.lat[P["plane_of"]]
        z = self._linear("z", h, P["w_in"])
        cq = self._buf("cq", (T, m.q_rank))
        half = m.rot_dims if m.rot_half else 0
        ops.latent_prep(self._cols(z, P, "lat"), m.q_rank, r if P["owner"] else 0, rot, P["gq"], P["gkv"], self.cfg.norm_eps,
                        b.positions, b.slot_mapping, P["rope"], cq, plane if P["owner"] else None, half)
        q = self._linear("q", cq, P["uq"]).view(T, H, dn + rot)
        qa = self._buf("qa", (T, H, r + rot))
        torch.bmm(q[:, :, :dn].transpose(0, 1), P["uk"], out=qa[:, :, :r].transpose(0, 1))
        ops.rope_pairs(q[:, :, dn:], qa[:, :, r:], b.positions, P["rope"], half)
        olat = self._buf("olat", (T, H, r))
        part_o = part_ml = None
        if b.kind == "decode" and self.device.type != "cpu":
            span = b.block_tables.shape[1] * cache.block_size
            parts = ops.latent_attn_parts(T, min(span, m.window) if m.window > 0 else span)
            if parts > 1:
                part_o = self._buf("attn.part_o", (T, H, parts, r), torch.float32)
                part_ml = self._buf("attn.part_ml", (T, H, parts, 2), torch.float32)
        tiled = b.kind != "decode" and self.dtype == torch.bfloat16
        ops.latent_attn(qa, plane, b.block_tables, b.row_seq, b.positions, m.scale, r, olat, part_o, part_ml,
                        b.tiles if tiled else None, b.cu_q if tiled else None, window=m.window)
        ov = self._buf("ov", (T, H * m.vdim))
        torch.bmm(olat.transpose(0, 1), P["uvt"], out=ov.view(T, H, m.vdim).transpose(0, 1))
        if m.gate:
            ops.sigmoid_mul(ov, self._cols(z, P, "g"), ov)
        return self._linear("att", ov, P["o"])

    def _attention(self, i: int, P: dict, b: ForwardBatch, cache: KomazenCache, h: torch.Tensor) -> torch.Tensor:
        m = P["mixer"]
        T = h.shape[0]
        prefill = b.kind != "decode"
        z = self._linear("z", h, P["w_in"])
        q = self._buf("att.q", (T, m.heads, m.dim))
        ops.qk_norm_cache(self._cols(z, P, "qkv"), m.heads, m.kv_heads, m.dim, m.vdim, P["gq"], P["gk"], P["temp"],
                          self.cfg.norm_eps, b.slot_mapping, q, cache.k[i], cache.v[i])
        att = self._buf("att.o", (T, m.heads, m.vdim))
        ops.window_attn(q, cache.k[i], cache.v[i], b.block_tables, b.row_seq, b.positions, NO_WINDOW, m.scale, None, att,
                        b.tiles if prefill else None, b.cu_q if prefill else None, bias=P["bias"])
        return self._linear("att", att.view(T, m.heads * m.vdim), P["o"])

    @torch.no_grad()
    def forward(self, b: ForwardBatch, cache: KomazenCache) -> torch.Tensor:
        """Run one step; returns sampled token ids [num_seqs] int32 (device).  ``b.logit_rows`` (prefill-kind steps)
        or ``b.need_logits`` (decode steps: every row) leave fp32 logits in ``self.last_logits``."""
        cfg = self.cfg
        T, d, eps, alpha = b.num_tokens, cfg.hidden_size, cfg.norm_eps, cfg.postln_alpha
        runs = b.num_seqs if b.kind != "decode" else T
        x = self._buf("x", (T, d), torch.float32)
        src = b.src if b.src is not None and b.kind == "decode" else None
        ops.embed_scale(b.input_ids, self.embed, cfg.embed_scale, x, src, self.last_ids if src is not None else None)
        h = self._conv(b, x, self.L[0]["canon1"], cache.conv[0], runs)
        for i, P in enumerate(self.L):
            att = self._latent(P, b, cache, h) if P["kind"] == "latent_attention" else self._attention(i, P, b, cache, h)
            nxt = self.L[i + 1] if i + 1 < len(self.L) else None
            after = (nxt["canon1"], cache.conv[2 * i + 2]) if nxt is not None else None
            if P["mlp"] is None:
                h = self._norm_conv(b, x, att, P["norm1"], after, runs)
                continue
            h = self._norm_conv(b, x, att, P["norm1"], (P["canon2"], cache.conv[2 * i + 1]), runs)
            F = P["mlp"].ff
            gu = self._linear("ff.gu", h, P["w_gu"])
            act = self._buf("ff.act", (T, F))
            ops.gelu_tanh_mul(gu[:, :F], gu[:, F:], act)
            h = self._norm_conv(b, x, self._linear("ff.down", act, P["w_down"]), P["norm2"], after, runs)
        n = b.num_seqs
        ids = self.last_ids[:n]
        self.last_logits = None
        if b.sample or b.need_logits:
            rows = None if b.kind == "decode" else b.last_idx
            logits = self._logits("logits", x, rows, n)
            if b.need_logits:
                self.last_logits = logits
            if b.sample:
                keys = self._buf("keys", (n,), torch.int64)
                ops.logits_argmax(logits, b.temps, b.seeds, b.step, keys, ids, 0)
                if b.filtered:
                    ops.sample_filtered(logits, b.temps, b.top_k, b.top_p, b.seeds, b.step, ids)
        if b.logit_rows is not None and b.logit_rows.numel():
            self.last_logits = self._logits("want_logits", x, b.logit_rows, int(b.logit_rows.numel()))
        return ids

    def _logits(self, name: str, x: torch.Tensor, rows, n: int) -> torch.Tensor:
        """fp32 logits [n, V] = n(x[rows], g_f) . W_head^T (fp32 output from the library GEMM)."""
        cfg = self.cfg
        xn = self._buf(name + ".xn", (n, cfg.hidden_size))
        ops.rms_norm_rows(x, rows, self.final_norm, cfg.norm_eps, 0.0, xn)
        logits = self._buf(name, (n, cfg.vocab_size), torch.float32)
        if self.dtype == torch.float32:
            torch.matmul(xn, self.head.t(), out=logits)
        elif self.device.type == "cpu":
            logits.copy_(xn.float() @ self.head.float().t())
        else:
            torch.bmm(xn[None], self.head.t()[None], out_dtype=torch.float32, out=logits[None])
        return logits
