"""Model weights: random init (the benchmark mode), safetensors loading, TP/EP sharding.

Weights live in the fused layout the kernels consume:

=================  =======================  ========================================
name               shape (per rank)          notes
=================  =======================  ========================================
embed              [V, d]                    replicated (1 GB for Llama-3-8B)
layers.i.ln1/ln2   [d]
layers.i.wqkv      [(Hq+2Hkv)/tp * D, d]    q|k|v rows of this rank's heads
layers.i.wo        [d, Hq/tp * D]           row-parallel (input columns split)
layers.i.w_gu      [2F/tp, d]               gate rows | up rows of this rank
layers.i.w_down    [d, F/tp]                row-parallel
layers.i.router    [E, d]                   MoE only (replicated)
layers.i.w13       [E/ep, 2F, d]            MoE experts of this rank (gate | up)
layers.i.w2        [E/ep, d, F]
norm               [d]
lm_head            [V/tp, d]                vocab-parallel
=================  =======================  ========================================

``mode="full"`` generates every full tensor from a per-name seed and slices
it, so any TP degree sees the same model (used by the TP-equivalence tests);
``mode="shard"`` generates each rank's shard directly (no full copy: the
70B/TP=8 path), seeded by (name, rank).
"""
from __future__ import annotations

import hashlib
import json
import os
from dataclasses import dataclass, field

import torch

from .config import ModelConfig

INIT_STD = 0.02
# matrices are drawn with std = INIT_GAIN / sqrt(fan_in): 0.02 at d = 4096 (the Llama init),
# and the same activation scale for the small test configs
INIT_GAIN = 1.28


def _std(name: str, shape) -> float:
    if name == "embed":
        return INIT_STD
    return INIT_GAIN / (shape[-1] ** 0.5)


@dataclass
class ShardSpec:
    tp_rank: int = 0
    tp_size: int = 1
    ep_rank: int = 0
    ep_size: int = 1

    def validate(self, cfg: ModelConfig) -> None:
        tp = self.tp_size
        if cfg.num_heads % tp or cfg.num_kv_heads % tp:
            raise ValueError(f"tp={tp} must divide num_heads={cfg.num_heads} and num_kv_heads={cfg.num_kv_heads}")
        if cfg.intermediate_size % tp:
            raise ValueError(f"tp={tp} must divide intermediate_size")
        if cfg.vocab_size % (16 * tp):
            raise ValueError(f"vocab {cfg.vocab_size} must be a multiple of 16*tp")
        if cfg.is_moe and cfg.num_experts % self.ep_size:
            raise ValueError(f"ep={self.ep_size} must divide num_experts={cfg.num_experts}")


@dataclass
class ModelWeights:
    cfg: ModelConfig
    shard: ShardSpec
    tensors: dict = field(default_factory=dict)
    layout: str = "natural"  # "decode" after models.layout.apply_decode_layout
    # names of tensors stored MFMA-preshuffled in place (decode_weights="replace": one copy per weight)
    shuffled: frozenset = frozenset()

    def to(self, device) -> "ModelWeights":
        """Copy on ``device`` (keeps the layout tags)."""
        return ModelWeights(self.cfg, self.shard, {k: v.to(device) for k, v in self.tensors.items()}, self.layout,
                            self.shuffled)

    def __getitem__(self, k):
        return self.tensors[k]

    def layer(self, i: int, name: str) -> torch.Tensor:
        return self.tensors[f"layers.{i}.{name}"]

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors.values())


def _seed(base: int, name: str, rank: int = -1) -> int:
    h = hashlib.sha256(f"{base}:{name}:{rank}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def _randn(shape, seed: int, device, dtype, std=INIT_STD) -> torch.Tensor:
    gdev = device if torch.device(device).type != "cpu" else "cpu"
    g = torch.Generator(device=gdev)
    g.manual_seed(seed)
    t = torch.randn(shape, generator=g, device=device, dtype=torch.float32 if gdev == "cpu" else dtype)
    t.mul_(std)
    return t.to(dtype)


def _row_slices(cfg: ModelConfig, shard: ShardSpec):
    tp, r = shard.tp_size, shard.tp_rank
    D = cfg.head_dim
    hq, hkv = cfg.num_heads // tp, cfg.num_kv_heads // tp
    q = slice(r * hq * D, (r + 1) * hq * D)
    k = slice(cfg.q_size + r * hkv * D, cfg.q_size + (r + 1) * hkv * D)
    v = slice(cfg.q_size + cfg.kv_size + r * hkv * D, cfg.q_size + cfg.kv_size + (r + 1) * hkv * D)
    f = cfg.intermediate_size // tp
    return q, k, v, slice(r * f, (r + 1) * f)


def shard_full(cfg: ModelConfig, shard: ShardSpec, full: dict) -> dict:
    """Slice full (unsharded, fused-layout) tensors to one rank's shards."""
    q, k, v, fs = _row_slices(cfg, shard)
    F = cfg.intermediate_size
    out = {}
    vs = cfg.vocab_size // shard.tp_size
    for name, t in full.items():
        if name.endswith(".wqkv"):
            out[name] = torch.cat([t[q], t[k], t[v]], 0).contiguous()
        elif name.endswith(".wo"):
            out[name] = t[:, q].contiguous()
        elif name.endswith(".w_gu"):
            out[name] = torch.cat([t[fs], t[F + fs.start : F + fs.stop]], 0).contiguous()
        elif name.endswith(".w_down"):
            out[name] = t[:, fs].contiguous()
        elif name == "lm_head":
            out[name] = t[shard.tp_rank * vs : (shard.tp_rank + 1) * vs].contiguous()
        elif name.endswith(".w13") or name.endswith(".w2"):
            e = cfg.num_experts // shard.ep_size
            out[name] = t[shard.ep_rank * e : (shard.ep_rank + 1) * e].contiguous()
        else:
            out[name] = t
    return out


def full_shapes(cfg: ModelConfig) -> dict:
    d, F, V, E = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_experts
    shapes = {"embed": (V, d), "norm": (d,), "lm_head": (V, d)}
    for i in range(cfg.num_layers):
        p = f"layers.{i}."
        shapes[p + "ln1"] = (d,)
        shapes[p + "ln2"] = (d,)
        shapes[p + "wqkv"] = (cfg.q_size + 2 * cfg.kv_size, d)
        shapes[p + "wo"] = (d, cfg.q_size)
        if cfg.is_moe:
            shapes[p + "router"] = (E, d)
            shapes[p + "w13"] = (E, 2 * F, d)
            shapes[p + "w2"] = (E, d, F)
        else:
            shapes[p + "w_gu"] = (2 * F, d)
            shapes[p + "w_down"] = (d, F)
    return shapes


def shard_shape(cfg: ModelConfig, shard: ShardSpec, name: str, shape: tuple) -> tuple:
    tp = shard.tp_size
    if name.endswith(".wqkv"):
        return ((cfg.q_size + 2 * cfg.kv_size) // tp, shape[1])
    if name.endswith(".wo"):
        return (shape[0], cfg.q_size // tp)
    if name.endswith(".w_gu"):
        return (2 * cfg.intermediate_size // tp, shape[1])
    if name.endswith(".w_down"):
        return (shape[0], cfg.intermediate_size // tp)
    if name == "lm_head":
        return (cfg.vocab_size // tp, shape[1])
    if name.endswith(".w13") or name.endswith(".w2"):
        return (cfg.num_experts // shard.ep_size,) + tuple(shape[1:])
    return shape


def random_weights(cfg: ModelConfig, shard: ShardSpec | None = None, device="cpu", dtype=torch.bfloat16,
                   seed: int = 0, mode: str = "full") -> ModelWeights:
    shard = shard or ShardSpec()
    if getattr(cfg, "family", "llama") == "bozevik":
        return bozevik_random_weights(cfg, shard, device, dtype, seed)
    if getattr(cfg, "family", "llama") == "lemunex":
        return lemunex_random_weights(cfg, shard, device, dtype, seed)
    if getattr(cfg, "family", "llama") == "komazen":
        return komazen_random_weights(cfg, shard, device, dtype, seed)
    if getattr(cfg, "family", "llama") == "dalalix":
        return dalalix_random_weights(cfg, shard, device, dtype, seed)
    shard.validate(cfg)
    shapes = full_shapes(cfg)
    tensors = {}
    if mode == "full":
        full = {}
        for name, shape in shapes.items():
            if len(shape) == 1:
                full[name] = torch.ones(shape, dtype=dtype)
            else:
                full[name] = _randn(shape, _seed(seed, name), "cpu", dtype, _std(name, shape))
        if cfg.tie_embeddings:
            full["lm_head"] = full["embed"]
        for name, t in shard_full(cfg, shard, full).items():
            tensors[name] = t.to(device)
    elif mode == "shard":
        for name, shape in shapes.items():
            sshape = shard_shape(cfg, shard, name, shape)
            if len(sshape) == 1:
                tensors[name] = torch.ones(sshape, dtype=dtype, device=device)
            else:
                rank = shard.tp_rank if name not in ("embed",) and not name.endswith("router") else -1
                tensors[name] = _randn(sshape, _seed(seed, name, rank), device, dtype, _std(name, shape))
    else:
        raise ValueError(mode)
    return ModelWeights(cfg, shard, tensors)


# --------------------------------------------------------------------------------------------------
# HuggingFace safetensors checkpoints (Llama / Mixtral naming) -> fused, sharded layout
# --------------------------------------------------------------------------------------------------
def _hf_index(path: str) -> dict:
    idx = os.path.join(path, "model.safetensors.index.json")
    if os.path.exists(idx):
        with open(idx) as f:
            return json.load(f)["weight_map"]
    files = [f for f in os.listdir(path) if f.endswith(".safetensors")]
    from safetensors import safe_open

    wmap = {}
    for fn in files:
        with safe_open(os.path.join(path, fn), framework="pt") as f:
            for k in f.keys():
                wmap[k] = fn
    return wmap


def load_hf_weights(path: str, cfg: ModelConfig, shard: ShardSpec | None = None, device="cpu",
                    dtype=torch.bfloat16) -> ModelWeights:
    """Load a HF safetensors checkpoint directory and fuse/shard it (no pickle anywhere)."""
    from safetensors import safe_open

    shard = shard or ShardSpec()
    if getattr(cfg, "family", "llama") == "bozevik":
        return load_bozevik_weights(path, cfg, shard, device, dtype)
    if getattr(cfg, "family", "llama") == "lemunex":
        return load_lemunex_weights(path, cfg, shard, device, dtype)
    if getattr(cfg, "family", "llama") == "komazen":
        return load_komazen_weights(path, cfg, shard, device, dtype)
    if getattr(cfg, "family", "llama") == "dalalix":
        return load_dalalix_weights(path, cfg, shard, device, dtype)
    shard.validate(cfg)
    wmap = _hf_index(path)
    handles = {}

    def get(name: str) -> torch.Tensor:
        fn = wmap[name]
        if fn not in handles:
            handles[fn] = safe_open(os.path.join(path, fn), framework="pt")
        return handles[fn].get_tensor(name).to(dtype)

    full = {"embed": get("model.embed_tokens.weight"), "norm": get("model.norm.weight")}
    full["lm_head"] = get("lm_head.weight") if "lm_head.weight" in wmap else full["embed"]
    for i in range(cfg.num_layers):
        p, h = f"layers.{i}.", f"model.layers.{i}."
        full[p + "ln1"] = get(h + "input_layernorm.weight")
        full[p + "ln2"] = get(h + "post_attention_layernorm.weight")
        full[p + "wqkv"] = torch.cat([get(h + f"self_attn.{n}_proj.weight") for n in "qkv"], 0)
        full[p + "wo"] = get(h + "self_attn.o_proj.weight")
        if cfg.is_moe:
            m = h + "block_sparse_moe."
            full[p + "router"] = get(m + "gate.weight")
            full[p + "w13"] = torch.stack([
                torch.cat([get(m + f"experts.{e}.w1.weight"), get(m + f"experts.{e}.w3.weight")], 0)
                for e in range(cfg.num_experts)])
            full[p + "w2"] = torch.stack([get(m + f"experts.{e}.w2.weight") for e in range(cfg.num_experts)])
        else:
            full[p + "w_gu"] = torch.cat([get(h + "mlp.gate_proj.weight"), get(h + "mlp.up_proj.weight")], 0)
            full[p + "w_down"] = get(h + "mlp.down_proj.weight")
    tensors = {k: v.to(device) for k, v in shard_full(cfg, shard, full).items()}
    return ModelWeights(cfg, shard, tensors)


def save_hf_weights(weights: ModelWeights, path: str) -> None:
    """Write full (tp=1) fused weights back out in HF naming (used to test the loader)."""
    from safetensors.torch import save_file

    from .layout import natural_tensors

    cfg = weights.cfg
    t = natural_tensors(weights)
    out = {"model.embed_tokens.weight": t["embed"], "model.norm.weight": t["norm"], "lm_head.weight": t["lm_head"]}
    q, kv, F = cfg.q_size, cfg.kv_size, cfg.intermediate_size
    for i in range(cfg.num_layers):
        p, h = f"layers.{i}.", f"model.layers.{i}."
        out[h + "input_layernorm.weight"] = t[p + "ln1"]
        out[h + "post_attention_layernorm.weight"] = t[p + "ln2"]
        w = t[p + "wqkv"]
        out[h + "self_attn.q_proj.weight"] = w[:q]
        out[h + "self_attn.k_proj.weight"] = w[q : q + kv]
        out[h + "self_attn.v_proj.weight"] = w[q + kv :]
        out[h + "self_attn.o_proj.weight"] = t[p + "wo"]
        if cfg.is_moe:
            m = h + "block_sparse_moe."
            out[m + "gate.weight"] = t[p + "router"]
            for e in range(cfg.num_experts):
                out[m + f"experts.{e}.w1.weight"] = t[p + "w13"][e, :F]
                out[m + f"experts.{e}.w3.weight"] = t[p + "w13"][e, F:]
                out[m + f"experts.{e}.w2.weight"] = t[p + "w2"][e]
        else:
            out[h + "mlp.gate_proj.weight"] = t[p + "w_gu"][:F]
            out[h + "mlp.up_proj.weight"] = t[p + "w_gu"][F:]
            out[h + "mlp.down_proj.weight"] = t[p + "w_down"]
    os.makedirs(path, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in out.items()}, os.path.join(path, "model.safetensors"))


# --------------------------------------------------------------------------------------------------
# Bozevik checkpoints: tensors keep the checkpoint's names (embed, l<i>.norm1, l<i>.mix.dq, l<i>.mlp.e<j>.gate, ...);
# the model fuses what its GEMMs read (models/bozevik.py).  Linear weights are [out, in].
# --------------------------------------------------------------------------------------------------
def bozevik_shapes(cfg) -> dict:
    from .config import GluSpec, MoeSpec

    d = cfg.hidden_size
    shapes = {"embed": (cfg.vocab_size, d), "final.norm": (d,)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = (d,)
        shapes[p + "norm2"] = (d,)
        shapes[p + "shift"] = (d,)
        shapes[p + "dwa"] = (i + 2,)
        shapes[p + "mix.dq"] = (m.q_rank, d)
        shapes[p + "mix.dq.norm"] = (m.q_rank,)
        shapes[p + "mix.uq"] = (m.heads * (m.dim + m.rot_dim), m.q_rank)
        if m.kv_from is None:
            shapes[p + "mix.dkv"] = (m.kv_rank + m.rot_dim, d)
            shapes[p + "mix.dkv.norm"] = (m.kv_rank,)
        shapes[p + "mix.uk"] = (m.heads * m.dim, m.kv_rank)
        shapes[p + "mix.uv"] = (m.heads * m.vdim, m.kv_rank)
        shapes[p + "mix.o"] = (d, m.heads * m.vdim)

        def glu(prefix, f):
            shapes[prefix + "gate"], shapes[prefix + "up"], shapes[prefix + "down"] = (f, d), (f, d), (d, f)

        if isinstance(layer.mlp, GluSpec):
            glu(p + "mlp.", layer.mlp.ff)
        elif isinstance(layer.mlp, MoeSpec):
            for e in range(layer.mlp.experts):
                glu(f"{p}mlp.e{e}.", layer.mlp.expert.ff)
            shapes[p + "mlp.router"] = (layer.mlp.experts, d)
            if layer.mlp.shared:
                glu(p + "mlp.shared.", layer.mlp.shared.ff)
    return shapes


def bozevik_random_weights(cfg, shard: ShardSpec | None = None, device="cpu", dtype=torch.bfloat16,
                           seed: int = 0) -> ModelWeights:
    """Random init (benchmarks, tests): matrices N(0, (1.28 / sqrt(fan_in))^2), norm weights 1, token-shift weights
    uniform in [0, 1), depth weights uniform with the newest layer's raised (a plain residual stream plus a tail)."""
    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Bozevik runs on one GPU per replica (its tensors are not sharded)")
    tensors = {}
    for name, shape in bozevik_shapes(cfg).items():
        sd = _seed(seed, name)
        if name.endswith("shift") or name.endswith("dwa"):
            g = torch.Generator().manual_seed(sd)
            t = torch.rand(shape, generator=g)
            if name.endswith("dwa"):
                t = t * (0.5 / len(t))
                t[-1] += 1.0
            tensors[name] = t.to(dtype).to(device)
        elif len(shape) == 1:
            tensors[name] = torch.ones(shape, dtype=dtype, device=device)
        else:
            tensors[name] = _randn(shape, sd, device, dtype, 1.0 if name == "embed" else _std(name, shape))
    return ModelWeights(cfg, shard, tensors)


def load_bozevik_weights(path: str, cfg, shard: ShardSpec | None = None, device="cpu",
                         dtype=torch.bfloat16) -> ModelWeights:
    """model.safetensors of a Bozevik checkpoint directory; every tensor the configuration implies must be there
    with the implied shape, and no other."""
    from safetensors import safe_open

    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Bozevik runs on one GPU per replica (its tensors are not sharded)")
    shapes = bozevik_shapes(cfg)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        missing, extra = sorted(set(shapes) - names), sorted(names - set(shapes))
        if missing or extra:
            raise ValueError(f"checkpoint does not fit its config: missing {missing[:4]}, unexpected {extra[:4]}")
        for name, shape in shapes.items():
            t = f.get_tensor(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config implies {tuple(shape)}")
            tensors[name] = t.to(dtype).to(device)
    return ModelWeights(cfg, shard, tensors)


def save_bozevik_checkpoint(weights: ModelWeights, path: str) -> None:
    """config.json + model.safetensors (bf16) of a Bozevik model, in the form the loader reads."""
    from safetensors.torch import save_file

    from .config import bozevik_to_config

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(bozevik_to_config(weights.cfg), f, indent=1)
    save_file({k: v.detach().to(torch.bfloat16).contiguous().cpu() for k, v in weights.tensors.items()},
              os.path.join(path, "model.safetensors"))


# --------------------------------------------------------------------------------------------------
# Lemunex checkpoints: tensors keep the checkpoint's names (embed, embed.norm, l<i>.norm1, l<i>.mix.left.q,
# l<i>.mix.in, l<i>.mlp.e<j>.gate, ..., final.norm, head); models/lemunex.py fuses what its GEMMs read.
# --------------------------------------------------------------------------------------------------
def safetensors_shapes(path: str) -> dict:
    """Tensor name -> shape from the header of ``path``/model.safetensors (8-byte little-endian length + JSON)."""
    import struct

    with open(os.path.join(path, "model.safetensors"), "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in head.items() if k != "__metadata__"}


def lemunex_shapes(cfg) -> dict:
    from .config import ReluSqSpec, RoutedSpec

    d = cfg.hidden_size
    shapes = {"embed": (cfg.vocab_size, d), "embed.norm": (d,), "final.norm": (d,), "head": (cfg.vocab_size, d)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = (d,)
        if layer.type == "parallel":
            a, g, q = m.left, m.right, p + "mix."
            for nm, rows in (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)):
                shapes[f"{q}left.{nm}"], shapes[f"{q}left.{nm}.b"] = (rows, d), (rows,)
            shapes[q + "left.g"] = (a.heads, d)
            shapes[q + "left.o"], shapes[q + "left.o.b"] = (d, a.heads * a.vdim), (d,)
            shapes[q + "right.q"] = shapes[q + "right.k"] = (g.heads * g.dim, d)
            shapes[q + "right.v"] = shapes[q + "right.g"] = (g.heads * g.vdim, d)
            shapes[q + "right.o"] = (d, g.heads * g.vdim)
            shapes[q + "right.norm"] = (g.vdim,)
            shapes[q + "right.a1"] = (g.decay_rank, d)
            shapes[q + "right.a2"], shapes[q + "right.a2.b"] = (g.heads * g.dim, g.decay_rank), (g.heads * g.dim,)
        else:
            q = p + "mix."
            shapes[q + "in"] = (2 * m.inner + 2 * m.groups * m.state + m.heads, d)
            shapes[q + "conv"], shapes[q + "conv.b"] = (m.conv_channels, m.conv), (m.conv_channels,)
            shapes[q + "dt_bias"] = shapes[q + "A_log"] = shapes[q + "D"] = (m.heads,)
            shapes[q + "norm"] = (m.inner,)
            shapes[q + "o"] = (d, m.inner)

        def glu(prefix, f):
            shapes[prefix + "gate"], shapes[prefix + "up"], shapes[prefix + "down"] = (f, d), (f, d), (d, f)

        f = layer.mlp
        if isinstance(f, ReluSqSpec):
            shapes[p + "mlp.up"], shapes[p + "mlp.down"] = (f.ff, d), (d, f.ff)
        elif isinstance(f, RoutedSpec):
            for e in range(f.experts):
                glu(f"{p}mlp.e{e}.", f.expert_ff)
            shapes[p + "mlp.router"] = (f.experts + f.identity, d)
            shapes[p + "mlp.correction"] = (f.experts + f.identity,)
            if f.shared_ff:
                glu(p + "mlp.shared.", f.shared_ff)
                shapes[p + "mlp.shared.sg"] = (1, d)
    return shapes


def lemunex_random_weights(cfg, shard: ShardSpec | None = None, device="cpu", dtype=torch.bfloat16,
                           seed: int = 0) -> ModelWeights:
    """Random init (benchmarks, tests): matrices N(0, (1.28 / sqrt(fan_in))^2); norm offsets, biases and router
    corrections small and nonzero (so a dropped one shows); decay / step-size parameters in the ranges where the
    recurrences remember hundreds of tokens."""
    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Lemunex runs on one GPU per replica (its tensors are not sharded)")
    tensors = {}
    for name, shape in lemunex_shapes(cfg).items():
        g = torch.Generator().manual_seed(_seed(seed, name))
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith("right.norm") or name.endswith("mix.norm"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif leaf in ("norm", "norm1"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif name.endswith("a2.b"):
            t = 3.0 + torch.randn(shape, generator=g)            # sigmoid(z) near one: slow decay
        elif leaf == "b":
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.02 * torch.randn(shape, generator=g)
        elif leaf == "dt_bias":
            t = -2.0 + torch.rand(shape, generator=g)
        elif leaf == "A_log":
            t = torch.log(0.05 + 0.5 * torch.rand(shape, generator=g))
        elif leaf == "D":
            t = 0.5 + torch.rand(shape, generator=g)
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * shape[1] ** -0.5
        else:
            tensors[name] = _randn(shape, _seed(seed, name), device, dtype, 1.0 if name == "embed" else _std(name, shape))
            continue
        tensors[name] = t.to(dtype).to(device)
    return ModelWeights(cfg, shard, tensors)


def load_lemunex_weights(path: str, cfg, shard: ShardSpec | None = None, device="cpu",
                         dtype=torch.bfloat16) -> ModelWeights:
    """model.safetensors of a Lemunex checkpoint directory; every tensor the configuration implies must be there
    with the implied shape, and no other.  Tensors stay in the file's precision (the model converts what it fuses)."""
    from safetensors import safe_open

    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Lemunex runs on one GPU per replica (its tensors are not sharded)")
    shapes = lemunex_shapes(cfg)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        missing, extra = sorted(set(shapes) - names), sorted(names - set(shapes))
        if missing or extra:
            raise ValueError(f"checkpoint does not fit its config: missing {missing[:4]}, unexpected {extra[:4]}")
        for name, shape in shapes.items():
            t = f.get_tensor(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config implies {tuple(shape)}")
            tensors[name] = t.to(device)
    return ModelWeights(cfg, shard, tensors)


def save_lemunex_checkpoint(weights: ModelWeights, path: str) -> None:
    """config.json + model.safetensors (bf16) of a Lemunex model, in the form the loader reads."""
    from safetensors.torch import save_file

    from .config import lemunex_to_config

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(lemunex_to_config(weights.cfg), f, indent=1)
    save_file({k: v.detach().to(torch.bfloat16).contiguous().cpu() for k, v in weights.tensors.items()},
              os.path.join(path, "model.safetensors"))


# --------------------------------------------------------------------------------------------------
# Komazen checkpoints: tensors keep the checkpoint's names (embed, l<i>.norm1, l<i>.canon1, l<i>.mix.dq, l<i>.mix.q,
# l<i>.mix.temp, l<i>.mlp.gate, ..., final.norm, head); models/komazen.py fuses what its GEMMs read.
# --------------------------------------------------------------------------------------------------
def komazen_shapes(cfg, optional: set | None = None) -> dict:
    """Tensor name -> shape.  ``optional`` (a set) receives the names a checkpoint may carry without this code reading
    them: the second norm and convolution of a layer that has no feed-forward."""
    d = cfg.hidden_size
    shapes = {"embed": (cfg.vocab_size, d), "final.norm": (d,), "head": (cfg.vocab_size, d)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        shapes[p + "norm1"] = (d,)
        shapes[p + "canon1"] = (d, cfg.conv_taps)
        if layer.type == "latent_attention":
            shapes[p + "mix.dq"] = (m.q_rank, d)
            shapes[p + "mix.dq.norm"] = (m.q_rank,)
            shapes[p + "mix.uq"] = (m.heads * (m.dim + m.rot_dim), m.q_rank)
            if m.kv_from is None:
                shapes[p + "mix.dkv"] = (m.kv_rank + m.rot_dim, d)
                shapes[p + "mix.dkv.norm"] = (m.kv_rank,)
            shapes[p + "mix.uk"] = (m.heads * m.dim, m.kv_rank)
            shapes[p + "mix.uv"] = (m.heads * m.vdim, m.kv_rank)
            shapes[p + "mix.g"] = (m.heads * m.vdim, d)
            shapes[p + "mix.o"] = (d, m.heads * m.vdim)
        else:
            shapes[p + "mix.q"] = (m.heads * m.dim, d)
            shapes[p + "mix.k"] = (m.kv_heads * m.dim, d)
            shapes[p + "mix.v"] = (m.kv_heads * m.vdim, d)
            shapes[p + "mix.q.norm"] = (m.dim,)
            shapes[p + "mix.k.norm"] = (m.dim,)
            for nm in ("r1", "r2", "temp"):
                shapes[p + "mix." + nm] = (m.heads,)
            shapes[p + "mix.o"] = (d, m.heads * m.vdim)
        if layer.mlp is not None:
            f = layer.mlp.ff
            shapes[p + "norm2"] = (d,)
            shapes[p + "canon2"] = (d, cfg.conv_taps)
            shapes[p + "mlp.gate"], shapes[p + "mlp.up"], shapes[p + "mlp.down"] = (f, d), (f, d), (d, f)
        elif optional is not None:
            optional.update((p + "norm2", p + "canon2"))
    return shapes


def komazen_random_weights(cfg, shard: ShardSpec | None = None, device="cpu", dtype=torch.bfloat16,
                           seed: int = 0) -> ModelWeights:
    """Random init (benchmarks, tests): matrices N(0, (1.28 / sqrt(fan_in))^2); norm weights around one; convolution
    taps small and of both signs; temperatures around one, distance-bias parameters positive -- all away from the
    values at which a dropped parameter would not show (1 for a factor, 0 for a term)."""
    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Komazen runs on one GPU per replica (its tensors are not sharded)")
    tensors = {}
    for name, shape in komazen_shapes(cfg).items():
        g = torch.Generator().manual_seed(_seed(seed, name))
        if "canon" in name:
            t = (torch.rand(shape, generator=g) - 0.5) * 0.6
        elif name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2"):
            t = 0.75 + 0.5 * torch.rand(shape, generator=g)
        elif name.endswith(".temp"):
            t = 0.6 + 0.8 * torch.rand(shape, generator=g)
        elif name.endswith(".r1"):
            t = 0.2 + 0.8 * torch.rand(shape, generator=g)
        elif name.endswith(".r2"):
            t = 0.05 + 0.5 * torch.rand(shape, generator=g)
        else:
            t = None
        if t is not None:
            tensors[name] = t.to(dtype).to(device)
        else:
            tensors[name] = _randn(shape, _seed(seed, name), device, dtype, 1.0 if name == "embed" else _std(name, shape))
    return ModelWeights(cfg, shard, tensors)


def load_komazen_weights(path: str, cfg, shard: ShardSpec | None = None, device="cpu",
                         dtype=torch.bfloat16) -> ModelWeights:
    """model.safetensors of a Komazen checkpoint directory; every tensor the configuration implies must be there with
    the implied shape, and no other.  Tensors stay in the file's precision (the model converts what it fuses)."""
    from safetensors import safe_open

    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Komazen runs on one GPU per replica (its tensors are not sharded)")
    optional: set = set()
    shapes = komazen_shapes(cfg, optional)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        missing, extra = sorted(set(shapes) - names), sorted(names - set(shapes) - optional)
        if missing or extra:
            raise ValueError(f"checkpoint does not fit its config: missing {missing[:4]}, unexpected {extra[:4]}")
        for name, shape in shapes.items():
            t = f.get_tensor(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config implies {tuple(shape)}")
            tensors[name] = t.to(device)
    return ModelWeights(cfg, shard, tensors)


def save_komazen_checkpoint(weights: ModelWeights, path: str) -> None:
    """config.json + model.safetensors (bf16) of a Komazen model, in the form the loader reads."""
    from safetensors.torch import save_file

    from .config import komazen_to_config

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(komazen_to_config(weights.cfg), f, indent=1)
    save_file({k: v.detach().to(torch.bfloat16).contiguous().cpu() for k, v in weights.tensors.items()},
              os.path.join(path, "model.safetensors"))


# --------------------------------------------------------------------------------------------------
# Dalalix checkpoints: tensors keep the checkpoint's names (embed, bigram, l<i>.norm1, l<i>.hc1.in, l<i>.mix.q,
# l<i>.mix.left.sink, l<i>.mix.right.i, l<i>.mlp.e<j>.gate, ..., final.norm, head); a layer that borrows another's
# weights has no tensors.  models/dalalix.py fuses what its GEMMs read.
# --------------------------------------------------------------------------------------------------
def dalalix_shapes(cfg, optional: set | None = None) -> dict:
    """Tensor name -> shape.  ``optional`` (a set) receives the names a checkpoint may carry without this code reading
    them: the second norm and stream mixing of a layer that has no feed-forward."""
    d, S = cfg.hidden_size, cfg.streams
    shapes = {"embed": (cfg.vocab_size, d), "final.norm": (d,), "head": (cfg.vocab_size, d)}
    if cfg.bigram:
        shapes["bigram"] = (cfg.bigram.buckets + 1, d)
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p, m = f"l{i}.", layer.mixer
        subs = {1: True, 2: layer.mlp is not None}
        for q, there in subs.items():
            names = {f"{p}norm{q}": (d,)}
            if S:
                names.update({f"{p}hc{q}.in": (S,), f"{p}hc{q}.out": (S,), f"{p}hc{q}.mix": (S, S)})
            if there:
                shapes.update(names)
            elif optional is not None:
                optional.update(names)
        if layer.type == "parallel":
            a, g, q = m.left, m.right, p + "mix."
            for nm, rows in (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)):
                shapes[f"{q}left.{nm}"], shapes[f"{q}left.{nm}.b"] = (rows, d), (rows,)
            shapes[q + "left.sink"] = (a.heads,)
            shapes[q + "left.o"] = (d, a.heads * a.vdim)
            shapes[q + "right.q"] = shapes[q + "right.k"] = (g.heads * g.dim, d)
            shapes[q + "right.v"] = shapes[q + "right.g"] = (g.heads * g.vdim, d)
            shapes[q + "right.o"] = (d, g.heads * g.vdim)
            shapes[q + "right.norm"] = (g.heads * g.vdim,)
            for nm in ("i", "f"):
                shapes[f"{q}right.{nm}"], shapes[f"{q}right.{nm}.b"] = (g.heads, d), (g.heads,)
        else:
            q = p + "mix."
            for nm, rows in (("q", m.heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim)):
                shapes[q + nm] = (rows, d)
                if m.bias:
                    shapes[f"{q}{nm}.b"] = (rows,)
                if m.conv:
                    shapes[f"{q}{nm}.conv"] = (rows, m.conv)
            if m.gate:
                shapes[q + "g"] = (m.heads * m.vdim, d)
            shapes[q + "o"] = (d, m.heads * m.vdim)
        f = layer.mlp
        if f is not None:
            for e in range(f.experts):
                shapes[f"{p}mlp.e{e}.gate"] = shapes[f"{p}mlp.e{e}.up"] = (f.expert_ff, d)
                shapes[f"{p}mlp.e{e}.down"] = (d, f.expert_ff)
            shapes[p + "mlp.router"] = (f.experts, d)
    return shapes


def dalalix_random_weights(cfg, shard: ShardSpec | None = None, device="cpu", dtype=torch.bfloat16,
                           seed: int = 0) -> ModelWeights:
    """Random init (benchmarks, tests): matrices N(0, (1.28 / sqrt(fan_in))^2); norm weights around one; stream mixing
    near a permutation-free average with every entry nonzero; biases, sinks and convolution taps nonzero; forget-gate
    biases high enough that the memory remembers hundreds of tokens -- all away from the values at which a dropped
    parameter would not show."""
    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Dalalix runs on one GPU per replica (its tensors are not sharded)")
    tensors = {}
    S = max(cfg.streams, 1)
    for name, shape in dalalix_shapes(cfg).items():
        g = torch.Generator().manual_seed(_seed(seed, name))
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1", "norm2"):
            t = 0.75 + 0.5 * torch.rand(shape, generator=g)
        elif name.endswith(".mix") and ".hc" in name:
            t = torch.eye(S) * 0.7 + 0.3 / S + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "in" and ".hc" in name:
            t = 1.0 / S + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "out" and ".hc" in name:
            t = 1.0 / S + 0.3 * torch.rand(shape, generator=g)
        elif name.endswith("right.f.b"):
            t = 3.0 + torch.randn(shape, generator=g)
        elif name.endswith("right.i.b"):
            t = -1.0 + torch.randn(shape, generator=g)
        elif leaf == "sink":
            t = torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.2 * torch.randn(shape, generator=g)
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * shape[1] ** -0.5
        elif name == "bigram":
            t = torch.randn(shape, generator=g)
        else:
            tensors[name] = _randn(shape, _seed(seed, name), device, dtype, 1.0 if name == "embed" else _std(name, shape))
            continue
        tensors[name] = t.to(dtype).to(device)
    return ModelWeights(cfg, shard, tensors)


def load_dalalix_weights(path: str, cfg, shard: ShardSpec | None = None, device="cpu",
                         dtype=torch.bfloat16) -> ModelWeights:
    """model.safetensors of a Dalalix checkpoint directory; every tensor the configuration implies must be there with
    the implied shape, and no other.  Tensors stay in the file's precision (the model converts what it fuses)."""
    from safetensors import safe_open

    shard = shard or ShardSpec()
    if shard.tp_size > 1 or shard.ep_size > 1:
        raise NotImplementedError("Dalalix runs on one GPU per replica (its tensors are not sharded)")
    optional: set = set()
    shapes = dalalix_shapes(cfg, optional)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        missing, extra = sorted(set(shapes) - names), sorted(names - set(shapes) - optional)
        if missing or extra:
            raise ValueError(f"checkpoint does not fit its config: missing {missing[:4]}, unexpected {extra[:4]}")
        for name, shape in shapes.items():
            t = f.get_tensor(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config implies {tuple(shape)}")
            tensors[name] = t.to(device)
    return ModelWeights(cfg, shard, tensors)


def save_dalalix_checkpoint(weights: ModelWeights, path: str) -> None:
    """config.json + model.safetensors (bf16) of a Dalalix model, in the form the loader reads."""
    from safetensors.torch import save_file

    from .config import dalalix_to_config

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(dalalix_to_config(weights.cfg), f, indent=1)
    save_file({k: v.detach().to(torch.bfloat16).contiguous().cpu() for k, v in weights.tensors.items()},
              os.path.join(path, "model.safetensors"))
