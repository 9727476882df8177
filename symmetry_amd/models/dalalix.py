"""Dalalix decoder forward on the symmetry_amd ops: one code path for CPU (torch references) and MI355X (HIP).

The design, in this file's notation (X: S fp32 residual streams, one row per token and stream; W stored [out, in];
n(v, g) = v / sqrt(mean(v^2) + eps) * g)::

    e_t = E[tok_t] + B[(tok_(t-1) a + tok_t b) mod n_b]     (a sequence's first token: B's extra last row);  X_s = e
    per sublayer f (mixer, then feed-forward), with its vectors c_in, c_out [S] and matrix M [S, S]:
        u = sum_s c_in[s] X_s;   y = f(n(u, g));   X_t <- sum_s M[s, t] X_s + c_out[t] y     (all streams at once)
    logits = cap tanh(W_head n(sum_s X_s, g_f) / cap)

    mixer "attention_2": q, k, v = W h + b; causal softmax over grouped heads (query head h reads key / value head
         h // (H / G)), no positions; W_o
    mixer "attention":   q, k, v = conv(W h) (causal per-channel taps, carried from step to step); v brought to unit RMS
         per head (cached so); causal softmax; heads times sigmoid(W_g h) element by element; W_o
    mixer "parallel" = c_l * A(h) + c_r * R(h), both reading h:
      A: q, k, v = W h + b; q, k turned on their first rot.dims entries (entry i with i + dims / 2); a position sees the
         newest ``window`` positions and the sequence's first ``keep_first``; the softmax's denominator also holds
         exp(sink_h); W_o
      R: per head i = c tanh(. / c), f = logsigmoid(c tanh(. / c)), m_t = max(f + m_(t-1), i), m_0 = 0,
         S <- e^(f + m_(t-1) - m_t) S + e^(i - m_t) k v^T, n alike with k, o = S^T q / (max(|n . q|, e^(-m_t)) + 1e-6),
         q scaled by dim^(-1/2); heads brought to unit RMS, times the norm weight, times sigmoid(W_g h); W_o
    ff: s = softmax(W_r h); experts in equal groups of neighbours, the best ``keep`` groups (by their best expert) stay
         eligible, the ``top`` best eligible experts with weights s_e / sum; expert = W_down (g' sigmoid(1.702 g') (u' + 1)),
         g' = min(W_gate h, limit), u' = clamp(W_up h, +-limit)

A layer with ``weights_of`` reads another layer's prepared tensors; its cache planes and state slots are its own.
Every projection that reads h is one row block of ONE fused weight per layer (a single library GEMM); the kernels take
column ranges of its output as views.  Step launches per layer: GEMM (all of h's projections), then
attention_2: qkv_rope_cache (bias, no table), window_attn (causal), GEMM W_o
attention:   conv_qkv_cache (+ conv_state_update in prompt steps), window_attn, sigmoid_mul, GEMM W_o
parallel:    qkv_rope_cache (half layout), window_attn (window, kept first tokens, sink), GEMM W_o | GEMM gates (fp32),
             decay_scan (log gates), memory_norm_gate, GEMM W_o
ff:          softmax_topk (groups), expert_offsets, scatter, grouped gate|up, clamped_glu, grouped down, moe_mix
and after every sublayer one hyper_mix_norm that mixes the streams, adds the sublayer's output and emits the next
sublayer's normalised input.  All intermediates live in the preallocated Workspace, so decode steps are
hipGraph-capturable.

fp32 in both serving dtypes: the streams and their mixing, norm statistics, rotary angles, attention scores and weights,
the memory's gates, maxima, states and normaliser, the unit norms, router scores.  ``dtype=torch.float32`` runs every
product in true 32-bit as well.
"""
from __future__ import annotations

import torch

from .. import ops
from .config import DalalixConfig
from .lemunex import _Fused
from .transformer import MAX_STEP_SEQS, ForwardBatch, Workspace
from .weights import ModelWeights

GLU_ALPHA = 1.702     # the experts' sigmoid slope (fixed by the design)
CAUSAL = 1 << 30      # a window that never ends: plain causal attention through the windowed kernel
MAX_STREAMS = 8


class DalalixCache:
    """What a Dalalix model keeps per sequence.

    ``k`` / ``v``: one pair of paged planes per layer, [NB, BS, G, dk] / [NB, BS, G, dv] (token-major), on the engine's
    BlockManager numbering (one block table serves all planes).  Per state slot: ``tok`` the sequence's last token
    (int32), ``conv`` per convolving layer the newest taps - 1 projected rows [slots, taps - 1, C], ``mem`` per matrix
    memory [slots, H, N + 1, P + 1] fp32 (the last column is the normaliser, the last row the running maximum).
    Slots are handed out by the scheduler's StateSlotManager; a slot's old content is never read by a new sequence (its
    first run starts from zero).  Zero-initialised: every byte finite."""

    def __init__(self, cfg: DalalixConfig, num_blocks: int, block_size: int, num_slots: int, device, dtype):
        self.num_layers, self.num_blocks, self.block_size = cfg.num_layers, num_blocks, block_size
        self.k, self.v, self.conv, self.mem = {}, {}, {}, {}
        self.tok = torch.zeros(num_slots, device=device, dtype=torch.int32)
        for i, layer in enumerate(cfg.layers):
            a = cfg.attn_spec(i)
            self.k[i] = torch.zeros(num_blocks, block_size, a.kv_heads, a.dim, device=device, dtype=dtype)
            self.v[i] = torch.zeros(num_blocks, block_size, a.kv_heads, a.vdim, device=device, dtype=dtype)
            if layer.type == "parallel":
                g = layer.mixer.right
                self.mem[i] = torch.zeros(num_slots, g.heads, g.dim + 1, g.vdim + 1, device=device, dtype=torch.float32)
            elif a.conv:
                C = a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)
                self.conv[i] = torch.zeros(num_slots, a.conv - 1, C, device=device, dtype=dtype)

    def nbytes(self) -> int:
        return self.tok.numel() * 4 + sum(t.numel() * t.element_size()
                                          for d in (self.k, self.v, self.conv, self.mem) for t in d.values())


class DalalixLM:
    has_seq_state = True      # the engine allots a state slot per live sequence and sends prev_row / save_slot / row_seq
    fused = False
    single_copy = False
    moe = None
    tp = None

    def __init__(self, weights: ModelWeights, device, tp_comm=None, ep_comm=None, max_decode_ctx: int | None = None,
                 decode_weights: str = "auto", kv_reserve_bytes: int = 0, dtype=torch.bfloat16):
        if weights.shard.tp_size > 1 or weights.shard.ep_size > 1:
            raise NotImplementedError("Dalalix runs on one GPU per replica")
        self.cfg: DalalixConfig = weights.cfg
        self.w = weights
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp_size, self.tp_rank = 1, 0
        self.ws = Workspace()
        self.last_ids = torch.zeros(MAX_STEP_SEQS, dtype=torch.int32, device=self.device)
        self.last_logits = None
        self.layer_sums: list | None = None   # set to a list: every forward appends the streams' sum after each layer
        cfg = self.cfg
        self.S = max(cfg.streams, 1)
        if self.S > MAX_STREAMS:
            raise NotImplementedError(f"{cfg.streams} residual streams: at most {MAX_STREAMS}")
        max_pos = min(cfg.max_position, max_decode_ctx or cfg.max_position)
        self._rope: dict = {}
        self._ones: torch.Tensor | None = None
        own = {i: self._prepare_layer(i, max_pos) for i in range(cfg.num_layers) if cfg.layers[i].weights_of is None}
        self.L = [own[cfg.owner(i)] for i in range(cfg.num_layers)]
        self.embed = weights["embed"].to(dtype)
        self.pair_table = weights["bigram"].to(dtype) if cfg.bigram else None
        self.final_norm = weights["final.norm"].float()
        self.head = weights["head"].to(dtype)
        # the sublayers in execution order: (layer, which, prepared tensors)
        self.subs = [(i, q) for i in range(cfg.num_layers) for q in (1, 2) if q == 1 or cfg.layers[i].mlp is not None]

    # ------------------------------------------------------------------------------------------
    def make_cache(self, num_blocks: int, block_size: int, num_slots: int) -> DalalixCache:
        return DalalixCache(self.cfg, num_blocks, block_size, num_slots, self.device, self.dtype)

    def extra_weight_bytes(self) -> int:
        return 0

    def _rope_table(self, rot, max_pos: int) -> torch.Tensor:
        key = (rot.dims, rot.base, max_pos)
        if key not in self._rope:
            self._rope[key] = ops.rope_pair_table(max_pos, rot.dims, rot.base).to(self.device)
        return self._rope[key]

    def _prepare_layer(self, i: int, max_pos: int) -> dict:
        """The fused / converted tensors layer i's launches read.  Matrices in the activation dtype; norm weights,
        biases, sinks, stream mixing and the gates' biases in fp32."""
        w, layer, dt, S = self.w, self.cfg.layers[i], self.dtype, self.S
        p = f"l{i}."

        def t(name):
            return w[p + name].to(dt)

        def f(name):
            return w[p + name].float().contiguous()

        fz = _Fused()
        P = {"kind": layer.type, "mixer": layer.mixer, "mlp": layer.mlp}
        for q in (1, 2):
            if q == 2 and layer.mlp is None:
                continue
            P[f"norm{q}"] = f(f"norm{q}")
            if self.cfg.streams:
                P[f"in{q}"], P[f"out{q}"], P[f"mix{q}"] = f(f"hc{q}.in"), f(f"hc{q}.out"), f(f"hc{q}.mix")
            else:   # the plain residual sum: one stream, kept, plus the sublayer's output
                one = torch.ones(1, dtype=torch.float32, device=self.device)
                P[f"in{q}"], P[f"out{q}"], P[f"mix{q}"] = one, one, one.view(1, 1)
        m = layer.mixer
        if layer.type == "parallel":
            a = m.left
            fz.add("left", torch.cat([t("mix.left.q"), t("mix.left.k"), t("mix.left.v")], 0))
            for nm in ("q", "k", "v", "g"):
                fz.add("right." + nm, t("mix.right." + nm))
            P["left.b"] = torch.cat([f("mix.left.q.b"), f("mix.left.k.b"), f("mix.left.v.b")]).contiguous()
            P["left.sink"], P["left.o"] = f("mix.left.sink"), t("mix.left.o")
            P["right.gates"] = torch.cat([t("mix.right.i"), t("mix.right.f")], 0).contiguous()
            P["right.gates.b"] = torch.cat([f("mix.right.i.b"), f("mix.right.f.b")]).contiguous()
            P["right.norm"], P["right.o"] = f("mix.right.norm"), t("mix.right.o")
            P["rope"] = self._rope_table(a.rot, max_pos) if a.rot.dims else None
        else:
            fz.add("qkv", torch.cat([t("mix.q"), t("mix.k"), t("mix.v")], 0))
            if m.bias:
                P["qkv.b"] = torch.cat([f("mix.q.b"), f("mix.k.b"), f("mix.v.b")]).contiguous()
            if m.conv:
                P["conv"] = torch.cat([t("mix.q.conv"), t("mix.k.conv"), t("mix.v.conv")], 0).contiguous()
            if m.gate:
                fz.add("g", t("mix.g"))
            P["o"] = t("mix.o")
        mlp = layer.mlp
        if mlp is not None:
            E = mlp.experts
            P["router"] = t("mlp.router").contiguous()
            P["w13"] = torch.stack([torch.cat([t(f"mlp.e{e}.gate"), t(f"mlp.e{e}.up")], 0) for e in range(E)]).contiguous()
            P["w2"] = torch.stack([t(f"mlp.e{e}.down") for e in range(E)]).contiguous()
        P["w_h"], P["cols"] = fz.weight(), fz.cols
        return P

    # ------------------------------------------------------------------------------------------
    def _buf(self, name, shape, dtype=None):
        return self.ws.get(name, shape, dtype or self.dtype, self.device)

    def _linear(self, name: str, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [R, K] @ w[N, K]^T -> [R, N] in the activation dtype (library GEMM, fp32 accumulation)."""
        return ops.linear(x, w, out=self._buf(name, (x.shape[0], w.shape[0])))

    def _linear_f32(self, name: str, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x [R, K] @ w[N, K]^T -> fp32 [R, N] (the library GEMM's fp32 accumulator, unrounded)."""
        out = self._buf(name, (x.shape[0], w.shape[0]), torch.float32)
        if self.dtype == torch.float32:
            torch.matmul(x, w.t(), out=out)
        elif self.device.type == "cpu":
            out.copy_(x.float() @ w.float().t())
        else:
            torch.bmm(x[None], w.t()[None], out_dtype=torch.float32, out=out[None])
        return out

    @staticmethod
    def _cols(z: torch.Tensor, P: dict, name: str) -> torch.Tensor:
        c0, n = P["cols"][name]
        return z[:, c0:c0 + n]

    def _grouped(self, xs: torch.Tensor, W: torch.Tensor, offsets: torch.Tensor, y: torch.Tensor) -> None:
        """y = xs @ W[e]^T over the expert segments: the main kernel library's MFMA grouped GEMM (bf16, shapes that
        tile for it: K % 64, N % 128, at most 64 experts) where that library is built, else the all-shapes kernel."""
        E, N, K = W.shape
        if (self.dtype == torch.bfloat16 and self.device.type != "cpu" and not ops.torch_mode() and E <= 64
                and K % 64 == 0 and N % 128 == 0 and ops.native_available()):
            ops.grouped_gemm(xs, W, offsets, 0, y, ops.GROUPED_BF16)
        else:
            ops.hyb_grouped_linear(xs, W, offsets, y)

    def _routed(self, P: dict, h: torch.Tensor) -> torch.Tensor:
        """Routed feed-forward -> fp32 [T, d].  Segment bounds stay on the device (no host sync: graph-capturable)."""
        spec = P["mlp"]
        T, d = h.shape
        E, k, F = spec.experts, spec.top, spec.expert_ff
        R = T * k
        i32 = torch.int32
        ids, wts = self._buf("moe.ids", (R,), i32), self._buf("moe.w", (R,), torch.float32)
        offsets, cursor = self._buf("moe.offsets", (E + 1,), i32), self._buf("moe.cursor", (E,), i32)
        dst = self._buf("moe.dst", (R,), i32)
        xs = self._buf("moe.xs", (R, d))
        if self._ones is None or self._ones.numel() < R:
            self._ones = torch.ones(max(R, 4096), dtype=torch.float32, device=self.device)
        ops.softmax_topk(h, P["router"], None, k, ids, wts, spec.groups, spec.keep, True)
        ops.hyb_expert_offsets(ids, R, E, offsets, cursor)
        ops.hyb_scatter_scaled(h, ids, self._ones[:R], k, offsets, cursor, xs, dst)
        y1 = self._buf("moe.y1", (R, 2 * F))
        self._grouped(xs, P["w13"], offsets, y1)
        act = self._buf("moe.act", (R, F))
        ops.hyb_clamped_glu(y1, spec.limit, GLU_ALPHA, act)
        y2 = self._buf("moe.y2", (R, d))
        self._grouped(act, P["w2"], offsets, y2)
        out = self._buf("moe.out", (T, d), torch.float32)
        ops.moe_mix(y2, dst, ids, wts, k, E, h, None, None, out)
        return out

    def _attend(self, i: int, a, b: ForwardBatch, cache: DalalixCache, q: torch.Tensor, window: int, keep_first: int,
                sink) -> torch.Tensor:
        T = q.shape[0]
        prefill = b.kind != "decode"
        att = self._buf("att.o", (T, a.heads, a.vdim))
        ops.window_attn(q, cache.k[i], cache.v[i], b.block_tables, b.row_seq, b.positions, window, a.scale, None, att,
                        b.tiles if prefill else None, b.cu_q if prefill else None, keep_first=keep_first, sink=sink)
        return att.view(T, a.heads * a.vdim)

    def _causal(self, i: int, P: dict, b: ForwardBatch, cache: DalalixCache, z: torch.Tensor, runs: int) -> torch.Tensor:
        """Mixers "attention_2" and "attention" -> [T, d]."""
        a = P["mixer"]
        T = z.shape[0]
        prefill = b.kind != "decode"
        qkv = self._cols(z, P, "qkv")
        q = self._buf("att.q", (T, a.heads, a.dim))
        if a.conv:
            cu = b.cu_q if prefill else None
            state = cache.conv[i]
            ops.conv_qkv_cache(qkv, P["conv"], state, cu, b.row_seq, b.prev_row, runs, a.heads, a.kv_heads, a.dim, a.vdim,
                               self.cfg.norm_eps, b.slot_mapping, q, cache.k[i], cache.v[i],
                               save_slot=None if prefill else b.save_slot)
            if prefill and a.conv > 1:
                ops.conv_state_update(qkv, state, cu, b.prev_row, b.save_slot, runs)
        else:
            ops.qkv_rope_cache(qkv, P.get("qkv.b"), a.heads, a.kv_heads, a.dim, a.vdim, b.positions, b.slot_mapping, None,
                               q, cache.k[i], cache.v[i])
        att = self._attend(i, a, b, cache, q, CAUSAL, 0, None)
        if a.gate:
            ops.sigmoid_mul(att, self._cols(z, P, "g"), att)
        return self._linear("att.out", att, P["o"])

    def _pair(self, i: int, P: dict, b: ForwardBatch, cache: DalalixCache, h: torch.Tensor, z: torch.Tensor, runs: int):
        """Both halves of a parallel mixer -> (attention output, memory output), each [T, d] before its scale."""
        m = P["mixer"]
        a, g = m.left, m.right
        T = z.shape[0]
        prefill = b.kind != "decode"
        q = self._buf("att.q", (T, a.heads, a.dim))
        ops.qkv_rope_cache(self._cols(z, P, "left"), P["left.b"], a.heads, a.kv_heads, a.dim, a.vdim, b.positions,
                           b.slot_mapping, P["rope"], q, cache.k[i], cache.v[i], half_dims=a.rot.dims)
        att = self._attend(i, a, b, cache, q, a.window, a.keep_first, P["left.sink"])
        left = self._linear("att.out", att, P["left.o"])
        gates = self._linear_f32("mem.gates", h, P["right.gates"])
        y = self._buf("mem.y", (T, g.heads, g.vdim + 1), torch.float32)
        mx = self._buf("mem.m", (T, g.heads), torch.float32)
        ops.decay_scan(ops.DECAY_LOG_GATES, self._cols(z, P, "right.q"), self._cols(z, P, "right.k"),
                       self._cols(z, P, "right.v"), gates, P["right.gates.b"], g.gate_cap, None, g.dim ** -0.5, g.heads,
                       g.dim, g.vdim, 1, cache.mem[i], b.cu_q if prefill else None, b.prev_row, b.save_slot, runs, y,
                       mout=mx)
        gy = self._buf("mem.gy", (T, g.heads * g.vdim))
        ops.memory_norm_gate(y, mx, self._cols(z, P, "right.g"), P["right.norm"], self.cfg.norm_eps, gy)
        right = self._linear("mem.out", gy, P["right.o"])
        return left, right

    @torch.no_grad()
    def forward(self, b: ForwardBatch, cache: DalalixCache) -> torch.Tensor:
        """Run one step; returns sampled token ids [num_seqs] int32 (device).  ``b.logit_rows`` (prefill-kind steps)
        or ``b.need_logits`` (decode steps: every row) leave fp32 logits in ``self.last_logits``."""
        cfg = self.cfg
        T, d, eps, S = b.num_tokens, cfg.hidden_size, cfg.norm_eps, self.S
        prefill = b.kind != "decode"
        runs = b.num_seqs if prefill else T
        xs = self._buf("xs", (T, S, d), torch.float32)
        h = self._buf("h", (T, d))
        src = b.src if b.src is not None and not prefill else None
        bg = cfg.bigram
        ops.embed_pair_hash(b.input_ids, self.embed, self.pair_table, bg.buckets if bg else 0, bg.mul_prev if bg else 0,
                            bg.mul_cur if bg else 0, b.prev_row, cache.tok, xs, None if prefill else b.save_slot, src,
                            self.last_ids if src is not None else None)
        if prefill and bg:
            ops.token_state_update(b.input_ids, cache.tok, b.cu_q, b.save_slot, runs)
        P0 = self.L[0]
        ops.hyper_mix_norm(xs, inc=P0["in1"], w=P0["norm1"], eps=eps, out=h)
        for n, (i, q) in enumerate(self.subs):
            P = self.L[i]
            nxt = self.subs[n + 1] if n + 1 < len(self.subs) else None
            kw = {}
            if nxt is not None:
                PN = self.L[nxt[0]]
                kw = {"inc": PN[f"in{nxt[1]}"], "w": PN[f"norm{nxt[1]}"], "eps": eps, "out": h}
            if q == 1:
                z = self._linear("z", h, P["w_h"])
                if P["kind"] == "parallel":
                    left, right = self._pair(i, P, b, cache, h, z, runs)
                    m = P["mixer"]
                    ops.hyper_mix_norm(xs, left, m.left_scale, right, m.right_scale, P["mix1"], P["out1"], **kw)
                else:
                    ops.hyper_mix_norm(xs, self._causal(i, P, b, cache, z, runs), 1.0, None, 0.0, P["mix1"], P["out1"], **kw)
            else:
                ops.hyper_mix_norm(xs, self._routed(P, h), 1.0, None, 0.0, P["mix2"], P["out2"], **kw)
            if self.layer_sums is not None and (nxt is None or nxt[0] != i):
                self.layer_sums.append(xs.sum(1))
        n = b.num_seqs
        ids = self.last_ids[:n]
        self.last_logits = None
        if b.sample or b.need_logits:
            rows = None if not prefill else b.last_idx
            logits = self._logits("logits", xs, rows, n)
            if b.need_logits:
                self.last_logits = logits
            if b.sample:
                keys = self._buf("keys", (n,), torch.int64)
                ops.logits_argmax(logits, b.temps, b.seeds, b.step, keys, ids, 0)
                if b.filtered:
                    ops.sample_filtered(logits, b.temps, b.top_k, b.top_p, b.seeds, b.step, ids)
        if b.logit_rows is not None and b.logit_rows.numel():
            self.last_logits = self._logits("want_logits", xs, b.logit_rows, int(b.logit_rows.numel()))
        return ids

    def _logits(self, name: str, xs: torch.Tensor, rows, n: int) -> torch.Tensor:
        """fp32 logits [n, V] = cap tanh(n(sum_s xs[rows, s], g_f) . W_head^T / cap) (fp32 output from the library GEMM)."""
        cfg = self.cfg
        xn = self._buf(name + ".xn", (n, cfg.hidden_size))
        ops.hyper_mix_norm(xs, w=self.final_norm, eps=cfg.norm_eps, rows=rows, out=xn)
        logits = self._linear_f32(name, xn, self.head)
        if cfg.logit_softcap:
            ops.logit_softcap(logits, cfg.logit_softcap)
        return logits
