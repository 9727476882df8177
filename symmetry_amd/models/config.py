"""Model configurations and the ``modelName`` registry.

``provider.yaml``'s ``modelName`` (REF: read at ``src/provider.ts:313`` and
forwarded to the upstream server) selects the architecture the native engine
runs.  Ollama-style tags (``llama3:8b``) and HF-style ids both resolve here.
Shapes are the public configs of the named models.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field


@dataclass(frozen=True)
class ModelConfig:
    family = "llama"  # which model class runs it (models.model_class); not a field
    name: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_position: int = 8192
    rope_scaling: dict | None = field(default=None, hash=False, compare=False)
    tie_embeddings: bool = False
    # mixture of experts (Mixtral); num_experts == 0 -> dense MLP
    num_experts: int = 0
    top_k: int = 2
    # special tokens of the chat format
    bos_token_id: int = 128000
    eos_token_ids: tuple = (128001, 128009)
    chat_format: str = "llama3"

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        d, f, v = self.hidden_size, self.intermediate_size, self.vocab_size
        attn = d * (self.q_size + 2 * self.kv_size) + self.q_size * d
        mlp = 3 * d * f * (self.num_experts if self.is_moe else 1) + (d * self.num_experts if self.is_moe else 0)
        per_layer = attn + mlp + 2 * d
        head = 0 if self.tie_embeddings else v * d
        return v * d + self.num_layers * per_layer + d + head

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    def replace(self, **kw) -> "ModelConfig":
        return dataclasses.replace(self, **kw)


# --------------------------------------------------------------------------------------------------
# Bozevik: per-layer specs (every layer names its mixer and feed-forward), latent attention, clamped GLU / MoE
# --------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class LatentMixerSpec:
    """Attention through low-rank latents: queries via q_rank, keys / values via a cached kv_rank latent plus one
    rotated key part of rot_dim shared by all heads.  ``kv_from``: the layer whose cache this layer attends
    (it then has no down-projection of its own)."""
    heads: int
    dim: int            # unrotated query / key dims per head
    rot_dim: int        # rotated dims per head (and of the shared key part)
    vdim: int
    kv_rank: int
    q_rank: int
    rot_base: float
    rot_dims: int       # leading dims of the rotated part that turn (pairs 2i, 2i + 1)
    scale: float
    kv_from: int | None = None
    window: int = 0             # > 0: a position sees itself and the window - 1 positions before it; 0: all before it
    rot_half: bool = False      # rotary pairs dimension i with i + rot_dims / 2 instead of 2i with 2i + 1
    gate: bool = False          # head outputs times sigmoid(W_g h), element by element


@dataclass(frozen=True)
class GluSpec:
    ff: int
    limit: float


@dataclass(frozen=True)
class MoeSpec:
    experts: int
    top: int
    expert: GluSpec
    shared: GluSpec | None = None


@dataclass(frozen=True)
class LayerSpec:
    type: str                       # mixer kind: "latent_attention"
    mixer: LatentMixerSpec
    mlp: GluSpec | MoeSpec | None = None


@dataclass(frozen=True)
class BozevikConfig:
    family = "bozevik"
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    max_position: int = 131072
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    chat_format: str = "llama3"
    tie_embeddings = True
    rope_scaling = None

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(layer.mlp, MoeSpec) for layer in self.layers)

    def cache_layers(self) -> list:
        """Layers that own a cache plane (a down-projection of their own), in order."""
        return [i for i, layer in enumerate(self.layers) if layer.mixer.kv_from is None]

    def num_params(self) -> int:
        d, n = self.hidden_size, self.vocab_size * self.hidden_size + self.hidden_size
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            n += 3 * d + i + 2 + m.q_rank * (d + 1) + m.heads * (m.dim + m.rot_dim) * m.q_rank
            n += m.heads * (m.dim + m.vdim) * m.kv_rank + d * m.heads * m.vdim
            if m.kv_from is None:
                n += (m.kv_rank + m.rot_dim) * d + m.kv_rank
            if isinstance(layer.mlp, GluSpec):
                n += 3 * d * layer.mlp.ff
            elif isinstance(layer.mlp, MoeSpec):
                n += layer.mlp.experts * (3 * d * layer.mlp.expert.ff + d)
                n += 3 * d * layer.mlp.shared.ff if layer.mlp.shared else 0
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum((self.layers[i].mixer.kv_rank + self.layers[i].mixer.rot_dim) for i in self.cache_layers()) * dtype_bytes

    def state_bytes_per_seq(self) -> int:
        return self.num_layers * self.hidden_size * 4

    def replace(self, **kw) -> "BozevikConfig":
        return dataclasses.replace(self, **kw)


def _glu(d: dict) -> GluSpec:
    return GluSpec(ff=int(d["ff"]), limit=float(d["limit"]))


def bozevik_from_config(cfg: dict, name: str = "bozevik") -> BozevikConfig:
    """A Bozevik checkpoint's config.json: every size and constant is read here; a key this reader does not
    know means a mechanism this code does not have, so it raises rather than ignore it."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        if L["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        m = dict(L["mixer"])
        rot = dict(m.pop("rot"))
        spec = LatentMixerSpec(heads=int(m.pop("heads")), dim=int(m.pop("dim")), rot_dim=int(m.pop("rot_dim")),
                               vdim=int(m.pop("vdim")), kv_rank=int(m.pop("kv_rank")), q_rank=int(m.pop("q_rank")),
                               rot_base=float(rot.pop("base")), rot_dims=int(rot.pop("dims")), scale=float(m.pop("scale")),
                               kv_from=(lambda v: None if v is None else int(v))(m.pop("kv_from", None)))
        if m or rot:
            raise ValueError(f"layer {i}: unknown mixer keys {sorted(m) + sorted(rot)}")
        if spec.rot_dims > spec.rot_dim or spec.rot_dims % 2:
            raise ValueError(f"layer {i}: rot.dims {spec.rot_dims} must be even and <= rot_dim {spec.rot_dim}")
        if spec.kv_from is not None:
            src = layers[spec.kv_from].mixer if 0 <= spec.kv_from < i else None
            if src is None or src.kv_from is not None or (src.kv_rank, src.rot_dim, src.rot_base, src.rot_dims) != (
                    spec.kv_rank, spec.rot_dim, spec.rot_base, spec.rot_dims):
                raise ValueError(f"layer {i}: kv_from {spec.kv_from} must name an earlier layer that owns a cache of "
                                 "the same latent / rotary sizes")
        mlp = L.get("mlp")
        if mlp is None:
            ff = None
        elif mlp["kind"] == "dense":
            ff = _glu(mlp)
        elif mlp["kind"] == "moe":
            ff = MoeSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]), expert=_glu(mlp["expert"]),
                         shared=_glu(mlp["shared"]) if mlp.get("shared") else None)
        else:
            raise ValueError(f"layer {i}: unknown mlp kind {mlp['kind']!r}")
        layers.append(LayerSpec(type=L["type"], mixer=spec, mlp=ff))
    return BozevikConfig(name=name, vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=tuple(layers),
                         norm_eps=float(cfg["norm"]["eps"]), logit_scale=float(cfg.get("logit_scale", 1.0)),
                         bos_token_id=int(cfg.get("bos_token_id", 1)),
                         eos_token_ids=tuple(cfg.get("eos_token_ids", (2,))))


def bozevik_to_config(c: BozevikConfig) -> dict:
    """The config.json form of a BozevikConfig (exports, tests)."""
    layers = []
    for layer in c.layers:
        m = layer.mixer
        md = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank, "q_rank": m.q_rank,
              "rot": {"base": m.rot_base, "dims": m.rot_dims}, "rot_dim": m.rot_dim, "scale": m.scale, "vdim": m.vdim}
        if m.kv_from is not None:
            md["kv_from"] = m.kv_from
        f = layer.mlp
        if f is None:
            fd = None
        elif isinstance(f, GluSpec):
            fd = {"ff": f.ff, "kind": "dense", "limit": f.limit}
        else:
            fd = {"expert": {"ff": f.expert.ff, "limit": f.expert.limit}, "kind": "moe",
                  "router": {"experts": f.experts, "top": f.top}}
            if f.shared:
                fd["shared"] = {"ff": f.shared.ff, "limit": f.shared.limit}
        layers.append({"mixer": md, "mlp": fd, "type": layer.type})
    return {"architecture": "Bozevik", "layers": layers, "logit_scale": c.logit_scale, "norm": {"eps": c.norm_eps},
            "vocab": c.vocab_size, "width": c.hidden_size}


def _bozevik_stack(name, vocab, width, n_layers, heads, dim, rot_dim, vdim, kv_rank, q_rank, ff, experts=0, top=2,
                   expert_ff=0, shared_ff=0, share_every=2, moe_every=None, **kw) -> BozevikConfig:
    """n_layers latent-attention layers; every ``share_every``-th attends the previous owner's cache; with experts > 0
    every ``moe_every``-th layer routes (default: the sharing layers), the others are dense."""
    layers, owner = [], 0
    for i in range(n_layers):
        shares = share_every > 0 and i % share_every == share_every - 1
        if not shares:
            owner = i
        mix = LatentMixerSpec(heads, dim, rot_dim, vdim, kv_rank, q_rank, 10000.0, rot_dim, (dim + rot_dim) ** -0.5,
                              owner if shares else None)
        routed = shares if moe_every is None else i % moe_every == moe_every - 1
        if experts and routed:
            mlp = MoeSpec(experts, top, GluSpec(expert_ff, 7.0), GluSpec(shared_ff, 7.0) if shared_ff else None)
        else:
            mlp = GluSpec(ff, 7.0)
        layers.append(LayerSpec("latent_attention", mix, mlp))
    return BozevikConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), **kw)


TINY_BOZEVIK = _bozevik_stack("tiny-bozevik", 512, 128, 4, heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=64, q_rank=48,
                              ff=256, experts=4, top=2, expert_ff=64, shared_ff=64, max_position=2048, bos_token_id=500,
                              eos_token_ids=(501, 502))
# layer shapes of a mid-size latent-attention model (benchmarks; random weights)
SMALL_BOZEVIK = _bozevik_stack("small-bozevik", 32768, 2048, 4, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512,
                               q_rank=1536, ff=8192, share_every=0, max_position=8192, bos_token_id=32000,
                               eos_token_ids=(32001, 32002))
SMALL_BOZEVIK_MOE = _bozevik_stack("small-bozevik-moe", 32768, 2048, 4, heads=16, dim=128, rot_dim=64, vdim=128,
                                   kv_rank=512, q_rank=1536, ff=8192, experts=16, top=4, expert_ff=1024, shared_ff=2048,
                                   max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))

# --------------------------------------------------------------------------------------------------
# Lemunex: parallel layers (one norm feeds the mixer and the feed-forward, both added to the stream).  Mixers: windowed
# softmax attention beside gated linear attention ("parallel"), or a state-space layer ("mamba2"); feed-forward:
# squared-ReLU, or routed gated experts with identity experts and a gated shared expert.
# --------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class RotarySpec:
    """Interleaved-pair rotary on the first ``dims`` entries of a head.  ``factor`` > 0 with ``original`` / ``fast`` /
    ``slow`` set: frequencies are blended towards f / factor between the pairs that turn ``fast`` and ``slow`` times
    over ``original`` positions, and cos / sin are scaled by 0.1 ln(factor) + 1."""
    dims: int
    base: float
    factor: float = 0.0          # 0: no frequency scaling
    original: float = 0.0
    fast: float = 0.0
    slow: float = 0.0
    half: bool = False           # True: entry i turns with entry i + dims / 2 (half layout) instead of the pairs (2i, 2i + 1)


@dataclass(frozen=True)
class WindowAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int                  # a position sees itself and the window - 1 positions before it
    scale: float
    rot: RotarySpec
    keep_first: int = 0          # the sequence's first positions stay visible past the window (at their true positions)
    sink: bool = False           # a learned per-head logit in the softmax's denominator (no key, no value)
    gate: bool = True            # per-head sigmoid output gate
    out_bias: bool = True        # bias on the output projection


@dataclass(frozen=True)
class GatedLinearAttnSpec:
    heads: int
    dim: int
    vdim: int
    tau: float                   # decay = sigmoid(z) ** (1 / tau)
    decay_rank: int              # inner size of the low-rank decay projection (from the checkpoint's tensor shapes)


@dataclass(frozen=True)
class PairMixerSpec:
    """Two mixers side by side on the same input: scale_left * attention + scale_right * linear attention."""
    left: WindowAttnSpec
    right: GatedLinearAttnSpec
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class StateSpaceSpec:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int                    # taps of the causal convolution
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class ReluSqSpec:
    ff: int


@dataclass(frozen=True)
class RoutedSpec:
    """Softmax router over experts + identity experts; choice by score + correction, weights = the plain scores."""
    experts: int                 # experts that have tensors
    identity: int                # further router outputs whose "expert" returns its input
    top: int
    expert_ff: int
    shared_ff: int = 0           # 0: no shared expert


@dataclass(frozen=True)
class LemunexLayer:
    type: str                    # "parallel" | "mamba2"
    mixer: PairMixerSpec | StateSpaceSpec
    mlp: ReluSqSpec | RoutedSpec | None = None


@dataclass(frozen=True)
class LemunexConfig:
    family = "lemunex"
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    norm_eps: float = 1e-5
    max_position: int = 131072
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    chat_format: str = "llama3"
    tie_embeddings = False
    rope_scaling = None

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(layer.mlp, RoutedSpec) for layer in self.layers)

    def attn_layers(self) -> list:
        """Layers that own planes of the paged key / value cache, in order."""
        return [i for i, layer in enumerate(self.layers) if layer.type == "parallel"]

    def num_params(self) -> int:
        from .weights import lemunex_shapes

        n = 0
        for shape in lemunex_shapes(self).values():
            k = 1
            for v in shape:
                k *= v
            n += k
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(self.layers[i].mixer.left.kv_heads * (self.layers[i].mixer.left.dim + self.layers[i].mixer.left.vdim)
                   for i in self.attn_layers()) * dtype_bytes

    def state_bytes_per_seq(self, dtype_bytes: int = 2) -> int:
        n = 0
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "parallel":
                n += m.right.heads * m.right.dim * m.right.vdim * 4
            else:
                n += m.heads * m.state * m.vdim * 4 + (m.conv - 1) * m.conv_channels * dtype_bytes
        return n

    def replace(self, **kw) -> "LemunexConfig":
        return dataclasses.replace(self, **kw)


def _take(d: dict, where: str, *keys, optional=()):
    """The values of ``keys`` (+ optional ones, None if absent); any other key in ``d`` is a mechanism this reader
    does not know, so it raises."""
    d = dict(d)
    out = [d.pop(k) for k in keys] + [d.pop(k, None) for k in optional]
    if d:
        raise ValueError(f"{where}: unknown keys {sorted(d)}")
    return out


def lemunex_from_config(cfg: dict, name: str = "lemunex", shapes: dict | None = None) -> LemunexConfig:
    """config.json of a Lemunex checkpoint.  ``shapes`` (tensor name -> shape, the checkpoint's header) supplies the
    sizes the configuration leaves to the tensors (the rank of the decay projection)."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        kind, mixer, mlp = _take(L, f"layer {i}", "type", "mixer", optional=("mlp",))
        if kind == "parallel":
            left, right, ls, rs = _take(mixer, f"layer {i} mixer", "left", "right", "left_scale", "right_scale")
            dim, heads, kvh, mask, rot, scale, vdim = _take(left, f"layer {i} left", "dim", "heads", "kv_heads", "mask",
                                                            "rot", "scale", "vdim")
            (window,) = _take(mask, f"layer {i} mask", "size")
            base, dims, scaling = _take(rot, f"layer {i} rot", "base", "dims", optional=("scaling",))
            if scaling:
                factor, fast, orig, slow = _take(scaling, f"layer {i} rot.scaling", "factor", "fast", "original", "slow")
                rspec = RotarySpec(int(dims), float(base), float(factor), float(orig), float(fast), float(slow))
            else:
                rspec = RotarySpec(int(dims), float(base))
            lspec = WindowAttnSpec(int(heads), int(kvh), int(dim), int(vdim), int(window), float(scale), rspec)
            if lspec.heads % lspec.kv_heads or rspec.dims % 2 or rspec.dims > lspec.dim or lspec.window < 1:
                raise ValueError(f"layer {i}: heads {heads} / kv_heads {kvh} / rot.dims {dims} / dim {dim} do not fit")
            rdim, rheads, tau, rvdim = _take(right, f"layer {i} right", "dim", "heads", "tau", "vdim")
            key = f"l{i}.mix.right.a1"
            if shapes is None or key not in shapes:
                raise ValueError(f"layer {i}: the decay projection's rank comes from the shape of {key}")
            rspec2 = GatedLinearAttnSpec(int(rheads), int(rdim), int(rvdim), float(tau), int(shapes[key][0]))
            mix = PairMixerSpec(lspec, rspec2, float(ls), float(rs))
        elif kind == "mamba2":
            conv, groups, heads, ng, state, vdim = _take(mixer, f"layer {i} mixer", "conv", "groups", "heads",
                                                         "norm_groups", "state", "vdim")
            mix = StateSpaceSpec(int(heads), int(vdim), int(state), int(groups), int(conv), int(ng))
            if mix.heads % mix.groups or mix.inner % mix.norm_groups or mix.conv < 1:
                raise ValueError(f"layer {i}: heads {heads} / groups {groups} / norm_groups {ng} do not fit")
        else:
            raise ValueError(f"layer {i}: unknown layer type {kind!r}")
        if mlp is None:
            ff = None
        elif mlp.get("kind") == "dense":
            (_, f) = _take(mlp, f"layer {i} mlp", "kind", "ff")
            ff = ReluSqSpec(int(f))
        elif mlp.get("kind") == "moe":
            _, expert, router, shared = _take(mlp, f"layer {i} mlp", "kind", "expert", "router", optional=("shared",))
            (eff,) = _take(expert, f"layer {i} mlp.expert", "ff")
            experts, top, ident = _take(router, f"layer {i} mlp.router", "experts", "top", optional=("identity",))
            sff = _take(shared, f"layer {i} mlp.shared", "ff")[0] if shared else 0
            ff = RoutedSpec(int(experts), int(ident or 0), int(top), int(eff), int(sff))
            if not 1 <= ff.top <= ff.experts + ff.identity:
                raise ValueError(f"layer {i}: top {top} of {ff.experts + ff.identity} router outputs")
        else:
            raise ValueError(f"layer {i}: unknown mlp kind {mlp.get('kind')!r}")
        layers.append(LemunexLayer(kind, mix, ff))
    vocab, width, norm, _, _, bos, eos = _take(cfg, "config", "vocab", "width", "norm", "layers",
                                               optional=("architecture", "bos_token_id", "eos_token_ids"))
    (eps,) = _take(norm, "norm", "eps")
    return LemunexConfig(name=name, vocab_size=int(vocab), hidden_size=int(width), layers=tuple(layers),
                         norm_eps=float(eps), bos_token_id=int(bos if bos is not None else 1),
                         eos_token_ids=tuple(eos) if eos is not None else (2,))


def lemunex_to_config(c: LemunexConfig) -> dict:
    """The config.json form of a LemunexConfig (exports, tests)."""
    layers = []
    for layer in c.layers:
        m = layer.mixer
        if layer.type == "parallel":
            a, g = m.left, m.right
            rot = {"base": a.rot.base, "dims": a.rot.dims}
            if a.rot.factor > 0:
                rot["scaling"] = {"factor": a.rot.factor, "fast": a.rot.fast, "original": a.rot.original,
                                  "slow": a.rot.slow}
            md = {"left": {"dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads, "mask": {"size": a.window},
                           "rot": rot, "scale": a.scale, "vdim": a.vdim},
                  "left_scale": m.left_scale,
                  "right": {"dim": g.dim, "heads": g.heads, "tau": g.tau, "vdim": g.vdim},
                  "right_scale": m.right_scale}
        else:
            md = {"conv": m.conv, "groups": m.groups, "heads": m.heads, "norm_groups": m.norm_groups, "state": m.state,
                  "vdim": m.vdim}
        f = layer.mlp
        if f is None:
            fd = None
        elif isinstance(f, ReluSqSpec):
            fd = {"ff": f.ff, "kind": "dense"}
        else:
            fd = {"expert": {"ff": f.expert_ff}, "kind": "moe",
                  "router": {"experts": f.experts, "identity": f.identity, "top": f.top}}
            if f.shared_ff:
                fd["shared"] = {"ff": f.shared_ff}
        layers.append({"mixer": md, "mlp": fd, "type": layer.type})
    return {"architecture": "Lemunex", "layers": layers, "norm": {"eps": c.norm_eps}, "vocab": c.vocab_size,
            "width": c.hidden_size}


def lemunex_stack(name, vocab, width, pattern, heads, kv_heads, dim, window, gla_heads, gla_dim, gla_vdim, ssm_heads,
                  ssm_vdim, ssm_state, ff, experts=0, top=2, identity=0, expert_ff=0, shared_ff=0, decay_rank=16,
                  ssm_groups=1, **kw) -> LemunexConfig:
    """A stack from a pattern string: "P" parallel layer (attention + linear attention), "M" state-space layer;
    lower case = that layer with the dense feed-forward, upper case with the routed one (if ``experts`` > 0)."""
    layers = []
    for ch in pattern:
        if ch in "Pp":
            rot = RotarySpec(dim // 2, 10000.0, 4.0, 4096.0, 32.0, 1.0)
            mix = PairMixerSpec(WindowAttnSpec(heads, kv_heads, dim, dim, window, dim ** -0.5, rot),
                                GatedLinearAttnSpec(gla_heads, gla_dim, gla_vdim, 16.0, decay_rank), 0.5, 0.5)
            kind = "parallel"
        else:
            mix = StateSpaceSpec(ssm_heads, ssm_vdim, ssm_state, ssm_groups, 4, 1)
            kind = "mamba2"
        routed = experts > 0 and ch.isupper()
        mlp = RoutedSpec(experts, identity, top, expert_ff, shared_ff) if routed else ReluSqSpec(ff)
        layers.append(LemunexLayer(kind, mix, mlp))
    return LemunexConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), **kw)


TINY_LEMUNEX = lemunex_stack("tiny-lemunex", 512, 128, "pMMP", heads=4, kv_heads=2, dim=32, window=48, gla_heads=2,
                             gla_dim=16, gla_vdim=32, ssm_heads=4, ssm_vdim=16, ssm_state=16, ff=256, experts=6, top=2,
                             identity=1, expert_ff=64, shared_ff=64, decay_rank=8, max_position=2048, bos_token_id=500,
                             eos_token_ids=(501, 502))
# layer shapes of a mid-size hybrid model (benchmarks; random weights)
SMALL_LEMUNEX = lemunex_stack("small-lemunex", 32768, 2048, "pmmp", heads=16, kv_heads=4, dim=128, window=1024,
                              gla_heads=8, gla_dim=128, gla_vdim=256, ssm_heads=64, ssm_vdim=64, ssm_state=128, ff=8192,
                              max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))
SMALL_LEMUNEX_MOE = lemunex_stack("small-lemunex-moe", 32768, 2048, "PMMP", heads=16, kv_heads=4, dim=128, window=1024,
                                  gla_heads=8, gla_dim=128, gla_vdim=256, ssm_heads=64, ssm_vdim=64, ssm_state=128,
                                  ff=8192, experts=16, top=4, identity=2, expert_ff=1024, shared_ff=2048,
                                  max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))

# --------------------------------------------------------------------------------------------------
# Komazen: norm after the sum (x <- n(alpha x + sublayer(x))), a short causal convolution in front of every sublayer,
# mixers: windowed latent attention (half-layout rotary, output gate, optional shared cache) or grouped-head softmax
# attention with query / key norm, per-head temperature and a logarithmic distance bias; gelu-gated feed-forward.
# --------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class BiasedAttnSpec:
    """Causal softmax attention, no rotation: score = scale * temp_h * n(q) . n(k) - r1_h ln(1 + r2_h (i - j))."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float


@dataclass(frozen=True)
class GeluGluSpec:
    ff: int


@dataclass(frozen=True)
class KomazenLayer:
    type: str                    # "latent_attention" | "attention"
    mixer: LatentMixerSpec | BiasedAttnSpec
    mlp: GeluGluSpec | None = None


@dataclass(frozen=True)
class KomazenConfig:
    family = "komazen"
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    embed_scale: float = 1.0
    postln_alpha: float = 1.0
    conv_taps: int = 4
    norm_eps: float = 1e-5
    max_position: int = 131072
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    chat_format: str = "llama3"
    tie_embeddings = False
    rope_scaling = None

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    def latent_layers(self) -> list:
        """Layers that own a plane of the paged latent cache (a down-projection of their own), in order."""
        return [i for i, layer in enumerate(self.layers) if layer.type == "latent_attention" and layer.mixer.kv_from is None]

    def attn_layers(self) -> list:
        """Layers that own planes of the paged key / value cache, in order."""
        return [i for i, layer in enumerate(self.layers) if layer.type == "attention"]

    def num_params(self) -> int:
        from .weights import komazen_shapes

        n = 0
        for shape in komazen_shapes(self).values():
            k = 1
            for v in shape:
                k *= v
            n += k
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        n = sum(self.layers[i].mixer.kv_rank + self.layers[i].mixer.rot_dim for i in self.latent_layers())
        n += sum(self.layers[i].mixer.kv_heads * (self.layers[i].mixer.dim + self.layers[i].mixer.vdim)
                 for i in self.attn_layers())
        return n * dtype_bytes

    def state_bytes_per_seq(self) -> int:
        """The newest taps - 1 inputs of every sublayer's convolution (fp32)."""
        subs = sum(1 + (layer.mlp is not None) for layer in self.layers)
        return subs * (self.conv_taps - 1) * self.hidden_size * 4

    def replace(self, **kw) -> "KomazenConfig":
        return dataclasses.replace(self, **kw)


def komazen_from_config(cfg: dict, name: str = "komazen") -> KomazenConfig:
    """config.json of a Komazen checkpoint: every size and constant is read here; a key this reader does not know means
    a mechanism this code does not have, so it raises."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        kind, mixer, mlp = _take(L, f"layer {i}", "type", "mixer", optional=("mlp",))
        if kind == "latent_attention":
            dim, heads, r, mask, qr, rot, rd, scale, vdim, src = _take(
                mixer, f"layer {i} mixer", "dim", "heads", "kv_rank", "mask", "q_rank", "rot", "rot_dim", "scale", "vdim",
                optional=("kv_from",))
            (window,) = _take(mask, f"layer {i} mask", "size")
            base, dims = _take(rot, f"layer {i} rot", "base", "dims")
            mix = LatentMixerSpec(heads=int(heads), dim=int(dim), rot_dim=int(rd), vdim=int(vdim), kv_rank=int(r),
                                  q_rank=int(qr), rot_base=float(base), rot_dims=int(dims), scale=float(scale),
                                  kv_from=None if src is None else int(src), window=int(window), rot_half=True, gate=True)
            if mix.rot_dims > mix.rot_dim or mix.rot_dims % 2 or mix.rot_dim % 2 or mix.window < 1:
                raise ValueError(f"layer {i}: rot.dims {dims} / rot_dim {rd} / mask.size {window} do not fit")
            if mix.kv_from is not None:
                s = layers[mix.kv_from] if 0 <= mix.kv_from < i else None
                if s is None or s.type != "latent_attention" or s.mixer.kv_from is not None or (
                        s.mixer.kv_rank, s.mixer.rot_dim, s.mixer.rot_base, s.mixer.rot_dims) != (
                        mix.kv_rank, mix.rot_dim, mix.rot_base, mix.rot_dims):
                    raise ValueError(f"layer {i}: kv_from {mix.kv_from} must name an earlier layer that owns a cache of "
                                     "the same latent / rotary sizes")
        elif kind == "attention":
            dim, heads, kvh, scale, vdim = _take(mixer, f"layer {i} mixer", "dim", "heads", "kv_heads", "scale", "vdim")
            mix = BiasedAttnSpec(int(heads), int(kvh), int(dim), int(vdim), float(scale))
            if mix.heads % mix.kv_heads:
                raise ValueError(f"layer {i}: heads {heads} / kv_heads {kvh} do not fit")
        else:
            raise ValueError(f"layer {i}: unknown layer type {kind!r}")
        if mlp is None:
            ff = None
        elif mlp.get("kind") == "dense":
            (_, f) = _take(mlp, f"layer {i} mlp", "kind", "ff")
            ff = GeluGluSpec(int(f))
        else:
            raise ValueError(f"layer {i}: unknown mlp kind {mlp.get('kind')!r}")
        layers.append(KomazenLayer(kind, mix, ff))
    vocab, width, norm, _, canon, emb, alpha, _, bos, eos = _take(
        cfg, "config", "vocab", "width", "norm", "layers", "canon", "embedding", "postln_alpha",
        optional=("architecture", "bos_token_id", "eos_token_ids"))
    (eps,) = _take(norm, "norm", "eps")
    (taps,) = _take(canon, "canon", "taps")
    (escale,) = _take(emb, "embedding", "scale")
    if not 1 <= int(taps) <= 16:
        raise ValueError(f"canon.taps {taps}: 1..16")
    return KomazenConfig(name=name, vocab_size=int(vocab), hidden_size=int(width), layers=tuple(layers),
                         embed_scale=float(escale), postln_alpha=float(alpha), conv_taps=int(taps), norm_eps=float(eps),
                         bos_token_id=int(bos if bos is not None else 1),
                         eos_token_ids=tuple(eos) if eos is not None else (2,))


def komazen_to_config(c: KomazenConfig) -> dict:
    """The config.json form of a KomazenConfig (exports, tests)."""
    layers = []
    for layer in c.layers:
        m = layer.mixer
        if layer.type == "latent_attention":
            md = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank, "mask": {"size": m.window}, "q_rank": m.q_rank,
                  "rot": {"base": m.rot_base, "dims": m.rot_dims}, "rot_dim": m.rot_dim, "scale": m.scale, "vdim": m.vdim}
            if m.kv_from is not None:
                md["kv_from"] = m.kv_from
        else:
            md = {"dim": m.dim, "heads": m.heads, "kv_heads": m.kv_heads, "scale": m.scale, "vdim": m.vdim}
        fd = None if layer.mlp is None else {"ff": layer.mlp.ff, "kind": "dense"}
        layers.append({"mixer": md, "mlp": fd, "type": layer.type})
    return {"architecture": "Komazen", "canon": {"taps": c.conv_taps}, "embedding": {"scale": c.embed_scale},
            "layers": layers, "norm": {"eps": c.norm_eps}, "postln_alpha": c.postln_alpha, "vocab": c.vocab_size,
            "width": c.hidden_size}


def komazen_stack(name, vocab, width, pattern, heads, kv_heads, dim, ff, window=1024, rot_dim=64, kv_rank=512, q_rank=1536,
                  vdim=None, embed_scale=1.0, postln_alpha=1.0, taps=4, **kw) -> KomazenConfig:
    """A stack from a pattern string: "L" latent-attention layer with a cache of its own, "S" one that attends the
    newest "L" layer's cache, "A" biased grouped-head attention; every layer with the gelu-gated feed-forward."""
    layers, owner = [], None
    vdim = vdim or dim
    for i, ch in enumerate(pattern):
        if ch in "LS":
            if ch == "S" and owner is None:
                raise ValueError("an S layer needs an L layer before it")
            mix = LatentMixerSpec(heads, dim, rot_dim, vdim, kv_rank, q_rank, 10000.0, rot_dim, (dim + rot_dim) ** -0.5,
                                  owner if ch == "S" else None, window, True, True)
            if ch == "L":
                owner = i
            layers.append(KomazenLayer("latent_attention", mix, GeluGluSpec(ff)))
        elif ch == "A":
            layers.append(KomazenLayer("attention", BiasedAttnSpec(heads, kv_heads, dim, vdim, dim ** -0.5), GeluGluSpec(ff)))
        else:
            raise ValueError(f"pattern letter {ch!r}")
    return KomazenConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), embed_scale=embed_scale,
                         postln_alpha=postln_alpha, conv_taps=taps, **kw)


TINY_KOMAZEN = komazen_stack("tiny-komazen", 512, 128, "LASA", heads=4, kv_heads=2, dim=16, ff=192, window=40, rot_dim=16,
                             kv_rank=48, q_rank=40, vdim=24, embed_scale=8.0, postln_alpha=2.0, max_position=2048,
                             bos_token_id=500, eos_token_ids=(501, 502))
# layer shapes of a mid-size model (benchmarks; random weights)
SMALL_KOMAZEN = komazen_stack("small-komazen", 32768, 2048, "LASA", heads=16, kv_heads=4, dim=128, ff=8192, window=1024,
                              max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))

# --------------------------------------------------------------------------------------------------
# Dalalix: several residual streams mixed by learned matrices (hyper-connections) around pre-norm sublayers; the token
# embedding plus a hashed (previous token, token) embedding; layers that borrow another layer's weights; mixers: causal
# grouped-head attention (biased projections, or a short convolution on q / k / v + unit-RMS values + an element-wise
# output gate), or windowed attention with kept first tokens and a sink beside a matrix memory with exponential gating;
# routed clamped-GLU experts with group-limited choice; soft-capped logits.
# --------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class HashPairSpec:
    """Row (prev * mul_prev + tok * mul_cur) mod buckets of a [buckets + 1, width] table; a sequence's first token takes
    the last row."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class CausalAttnSpec:
    """Causal softmax attention with grouped key / value heads and no positions in the scores."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias: bool = False           # q / k / v projections carry biases
    conv: int = 0                # taps of the causal per-channel convolution on q, k and v (0: none)
    v_norm: bool = False         # values are brought to unit RMS per head before they are cached
    gate: bool = False           # element-wise sigmoid(W_g h) on the concatenated heads


@dataclass(frozen=True)
class MatrixMemorySpec:
    """Matrix memory with exponential input gate, sigmoid forget gate (both soft-capped) and a running maximum."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class GroupRoutedSpec:
    """Softmax router; experts in ``groups`` equal groups of neighbours, only the ``keep`` best groups (by their best
    expert) are eligible; weights = chosen scores over their sum; clamped-GLU experts."""
    experts: int
    top: int
    expert_ff: int
    limit: float
    groups: int = 1
    keep: int = 1


@dataclass(frozen=True)
class DalalixLayer:
    type: str                    # "attention" | "attention_2" | "parallel"
    mixer: CausalAttnSpec | PairMixerSpec
    mlp: GroupRoutedSpec | None = None
    weights_of: int | None = None   # the layer whose tensors this one reads (cache and state stay its own)


@dataclass(frozen=True)
class DalalixConfig:
    family = "dalalix"
    name: str
    vocab_size: int
    hidden_size: int
    layers: tuple
    streams: int = 0             # residual streams; 0: the plain residual sum (no mixing tensors)
    bigram: HashPairSpec | None = None
    logit_softcap: float = 0.0   # 0: none
    norm_eps: float = 1e-5
    max_position: int = 131072
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    chat_format: str = "llama3"
    tie_embeddings = False
    rope_scaling = None

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(layer.mlp is not None for layer in self.layers)

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i reads (a borrowed layer may itself borrow: the chain ends at an owner)."""
        while self.layers[i].weights_of is not None:
            i = self.layers[i].weights_of
        return i

    def attn_spec(self, i: int):
        """The softmax-attention part of layer i's mixer (every layer has one)."""
        layer = self.layers[i]
        return layer.mixer.left if layer.type == "parallel" else layer.mixer

    def num_params(self) -> int:
        from .weights import dalalix_shapes

        n = 0
        for shape in dalalix_shapes(self).values():
            k = 1
            for v in shape:
                k *= v
            n += k
        return n

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(a.kv_heads * (a.dim + a.vdim) for a in map(self.attn_spec, range(self.num_layers))) * dtype_bytes

    def state_bytes_per_seq(self, dtype_bytes: int = 2) -> int:
        n = 4 if self.bigram else 0
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "parallel":
                n += m.right.heads * (m.right.dim + 1) * (m.right.vdim + 1) * 4
            elif m.conv > 1:
                n += (m.conv - 1) * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) * dtype_bytes
        return n

    def replace(self, **kw) -> "DalalixConfig":
        return dataclasses.replace(self, **kw)


def dalalix_from_config(cfg: dict, name: str = "dalalix") -> DalalixConfig:
    """config.json of a Dalalix checkpoint: every size and constant is read here; a key this reader does not know means
    a mechanism this code does not have, so it raises."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        kind, mixer, mlp, wof = _take(L, f"layer {i}", "type", "mixer", optional=("mlp", "weights_of"))
        if kind in ("attention", "attention_2"):
            dim, heads, kvh, scale, vdim, conv = _take(mixer, f"layer {i} mixer", "dim", "heads", "kv_heads", "scale",
                                                       "vdim", optional=("conv",))
            if (kind == "attention") != (conv is not None):
                raise ValueError(f"layer {i}: {kind!r} and conv = {conv!r} do not fit")
            plain = kind == "attention_2"
            mix = CausalAttnSpec(int(heads), int(kvh), int(dim), int(vdim), float(scale), bias=plain,
                                 conv=0 if plain else int(conv), v_norm=not plain, gate=not plain)
            if mix.heads % mix.kv_heads or (not plain and not 1 <= mix.conv <= 16):
                raise ValueError(f"layer {i}: heads {heads} / kv_heads {kvh} / conv {conv} do not fit")
        elif kind == "parallel":
            left, right, ls, rs = _take(mixer, f"layer {i} mixer", "left", "right", "left_scale", "right_scale")
            dim, heads, kvh, mask, rot, scale, vdim = _take(left, f"layer {i} left", "dim", "heads", "kv_heads", "mask",
                                                            "rot", "scale", "vdim")
            window, keep = _take(mask, f"layer {i} mask", "size", optional=("keep_first",))
            base, dims = _take(rot, f"layer {i} rot", "base", "dims")
            lspec = WindowAttnSpec(int(heads), int(kvh), int(dim), int(vdim), int(window), float(scale),
                                   RotarySpec(int(dims), float(base), half=True), keep_first=int(keep or 0), sink=True,
                                   gate=False, out_bias=False)
            if lspec.heads % lspec.kv_heads or lspec.rot.dims % 2 or lspec.rot.dims > lspec.dim or lspec.window < 1 \
                    or lspec.keep_first < 0:
                raise ValueError(f"layer {i}: heads {heads} / kv_heads {kvh} / rot.dims {dims} / dim {dim} / mask do not fit")
            rdim, cap, rheads, rvdim = _take(right, f"layer {i} right", "dim", "gate_cap", "heads", "vdim")
            mix = PairMixerSpec(lspec, MatrixMemorySpec(int(rheads), int(rdim), int(rvdim), float(cap)), float(ls), float(rs))
        else:
            raise ValueError(f"layer {i}: unknown layer type {kind!r}")
        if mlp is None:
            ff = None
        elif mlp.get("kind") == "moe":
            _, expert, router = _take(mlp, f"layer {i} mlp", "kind", "expert", "router")
            eff, limit = _take(expert, f"layer {i} mlp.expert", "ff", "limit")
            experts, top, groups = _take(router, f"layer {i} mlp.router", "experts", "top", optional=("groups",))
            count, keep = _take(groups, f"layer {i} mlp.router.groups", "count", "keep") if groups else (1, 1)
            ff = GroupRoutedSpec(int(experts), int(top), int(eff), float(limit), int(count), int(keep))
            if ff.experts % ff.groups or not 1 <= ff.keep <= ff.groups or not 1 <= ff.top <= ff.keep * (ff.experts // ff.groups):
                raise ValueError(f"layer {i}: top {top} of {experts} experts in {count} groups, {keep} kept")
        else:
            raise ValueError(f"layer {i}: unknown mlp kind {mlp.get('kind')!r}")
        layer = DalalixLayer(kind, mix, ff, None if wof is None else int(wof))
        if layer.weights_of is not None:
            src = layers[layer.weights_of] if 0 <= layer.weights_of < i else None
            if src is None or (src.type, src.mixer, src.mlp) != (kind, mix, ff):
                raise ValueError(f"layer {i}: weights_of {wof} must name an earlier layer of the same kind and sizes")
        layers.append(layer)
    vocab, width, norm, _, _, emb, streams, cap, bos, eos = _take(
        cfg, "config", "vocab", "width", "norm", "layers",
        optional=("architecture", "embedding", "streams", "logit_softcap", "bos_token_id", "eos_token_ids"))
    (eps,) = _take(norm, "norm", "eps")
    (bg,) = _take(emb, "embedding", optional=("bigram",)) if emb else (None,)
    if bg:
        buckets, mc, mp = _take(bg, "embedding.bigram", "buckets", "mul_cur", "mul_prev")
        bg = HashPairSpec(int(buckets), int(mp), int(mc))
        if bg.buckets < 1:
            raise ValueError("embedding.bigram.buckets < 1")
    return DalalixConfig(name=name, vocab_size=int(vocab), hidden_size=int(width), layers=tuple(layers),
                         streams=int(streams or 0), bigram=bg or None, logit_softcap=float(cap or 0.0),
                         norm_eps=float(eps), bos_token_id=int(bos if bos is not None else 1),
                         eos_token_ids=tuple(eos) if eos is not None else (2,))


def dalalix_to_config(c: DalalixConfig) -> dict:
    """The config.json form of a DalalixConfig (exports, tests)."""
    layers = []
    for layer in c.layers:
        m = layer.mixer
        if layer.type == "parallel":
            a, g = m.left, m.right
            md = {"left": {"dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads,
                           "mask": {"keep_first": a.keep_first, "size": a.window},
                           "rot": {"base": a.rot.base, "dims": a.rot.dims}, "scale": a.scale, "vdim": a.vdim},
                  "left_scale": m.left_scale,
                  "right": {"dim": g.dim, "gate_cap": g.gate_cap, "heads": g.heads, "vdim": g.vdim},
                  "right_scale": m.right_scale}
        else:
            md = {"dim": m.dim, "heads": m.heads, "kv_heads": m.kv_heads, "scale": m.scale, "vdim": m.vdim}
            if layer.type == "attention":
                md["conv"] = m.conv
        f = layer.mlp
        fd = None if f is None else {"expert": {"ff": f.expert_ff, "limit": f.limit}, "kind": "moe",
                                     "router": {"experts": f.experts, "groups": {"count": f.groups, "keep": f.keep},
                                                "top": f.top}}
        d = {"mixer": md, "mlp": fd, "type": layer.type}
        if layer.weights_of is not None:
            d["weights_of"] = layer.weights_of
        layers.append(d)
    out = {"architecture": "Dalalix", "layers": layers, "norm": {"eps": c.norm_eps}, "vocab": c.vocab_size,
           "width": c.hidden_size}
    if c.bigram:
        out["embedding"] = {"bigram": {"buckets": c.bigram.buckets, "mul_cur": c.bigram.mul_cur,
                                       "mul_prev": c.bigram.mul_prev}}
    if c.streams:
        out["streams"] = c.streams
    if c.logit_softcap:
        out["logit_softcap"] = c.logit_softcap
    return out


def dalalix_stack(name, vocab, width, pattern, heads, kv_heads, dim, experts, top, expert_ff, window=1024, keep_first=4,
                  rot_dims=None, vdim=None, mem_heads=None, mem_dim=None, mem_vdim=None, conv=4, groups=1, keep=1,
                  limit=7.0, streams=4, buckets=0, softcap=30.0, **kw) -> DalalixConfig:
    """A stack from a pattern string: "B" causal attention with biased projections, "C" causal attention with the short
    convolution, unit-RMS values and the output gate, "P" windowed attention beside the matrix memory; a digit repeats
    the layer with that index with its weights (cache and state its own); lower case = no feed-forward."""
    vdim = vdim or dim
    layers = []
    for ch in pattern:
        if ch.isdigit():
            src = layers[int(ch)]
            layers.append(dataclasses.replace(src, weights_of=int(ch)))
            continue
        if ch in "Bb":
            kind, mix = "attention_2", CausalAttnSpec(heads, kv_heads, dim, vdim, dim ** -0.5, bias=True)
        elif ch in "Cc":
            kind, mix = "attention", CausalAttnSpec(heads, kv_heads, dim, vdim, dim ** -0.5, conv=conv, v_norm=True,
                                                    gate=True)
        elif ch in "Pp":
            left = WindowAttnSpec(heads, kv_heads, dim, vdim, window, dim ** -0.5,
                                  RotarySpec(rot_dims or dim // 2, 10000.0, half=True), keep_first=keep_first, sink=True,
                                  gate=False, out_bias=False)
            right = MatrixMemorySpec(mem_heads or heads, mem_dim or dim, mem_vdim or vdim, 15.0)
            kind, mix = "parallel", PairMixerSpec(left, right, 0.5, 0.5)
        else:
            raise ValueError(f"pattern letter {ch!r}")
        mlp = GroupRoutedSpec(experts, top, expert_ff, limit, groups, keep) if ch.isupper() else None
        layers.append(DalalixLayer(kind, mix, mlp))
    bg = HashPairSpec(buckets, 1000003, 31) if buckets else None
    return DalalixConfig(name=name, vocab_size=vocab, hidden_size=width, layers=tuple(layers), streams=streams, bigram=bg,
                         logit_softcap=softcap, **kw)


TINY_DALALIX = dalalix_stack("tiny-dalalix", 512, 128, "BPC1", heads=4, kv_heads=2, dim=32, experts=6, top=2, expert_ff=64,
                             window=48, keep_first=3, rot_dims=16, mem_heads=2, mem_dim=16, mem_vdim=32, conv=3, groups=3,
                             keep=2, limit=3.0, streams=3, buckets=251, max_position=2048, bos_token_id=500,
                             eos_token_ids=(501, 502))
# layer shapes of a mid-size model (benchmarks; random weights)
SMALL_DALALIX = dalalix_stack("small-dalalix", 32768, 2048, "BPCC", heads=16, kv_heads=4, dim=128, experts=16, top=4,
                              expert_ff=1024, window=1024, mem_heads=8, mem_dim=128, mem_vdim=256, groups=4, keep=2,
                              buckets=65521, max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))

LLAMA31_SCALING = {
    "rope_type": "llama3",
    "factor": 8.0,
    "low_freq_factor": 1.0,
    "high_freq_factor": 4.0,
    "original_max_position_embeddings": 8192,
}

LLAMA3_8B = ModelConfig(
    name="llama3:8b", vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_layers=32, num_heads=32,
    num_kv_heads=8, rope_theta=500000.0, max_position=8192,
)
LLAMA31_8B = LLAMA3_8B.replace(name="llama3.1:8b", max_position=131072, rope_scaling=LLAMA31_SCALING)
LLAMA3_70B = ModelConfig(
    name="llama3:70b", vocab_size=128256, hidden_size=8192, intermediate_size=28672, num_layers=80, num_heads=64,
    num_kv_heads=8, rope_theta=500000.0, max_position=8192,
)
LLAMA31_70B = LLAMA3_70B.replace(name="llama3.1:70b", max_position=131072, rope_scaling=LLAMA31_SCALING)
MIXTRAL_8X7B = ModelConfig(
    name="mixtral:8x7b", vocab_size=32000, hidden_size=4096, intermediate_size=14336, num_layers=32, num_heads=32,
    num_kv_heads=8, rope_theta=1e6, max_position=32768, num_experts=8, top_k=2, bos_token_id=1,
    eos_token_ids=(2,), chat_format="mistral",
)
# Small configs with the same structure, for CPU tests and GPU smoke runs.
TINY_LLAMA = ModelConfig(
    name="tiny-llama", vocab_size=512, hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4,
    num_kv_heads=2, rope_theta=10000.0, max_position=2048, bos_token_id=500, eos_token_ids=(501, 502),
)
TINY_MIXTRAL = TINY_LLAMA.replace(name="tiny-mixtral", num_experts=4, top_k=2)
# 8 KV heads like Llama-3-70B / Mixtral: TP=8 leaves one KV head (and two q heads) per rank, the 70B TP=8
# shard geometry; the MoE variant has 8 experts, one per rank at EP=8
TINY_LLAMA_KV8 = TINY_LLAMA.replace(name="tiny-llama-kv8", num_heads=16, num_kv_heads=8, intermediate_size=2048)
TINY_MIXTRAL_E8 = TINY_LLAMA_KV8.replace(name="tiny-mixtral-e8", num_experts=8, top_k=2)
SMALL_LLAMA = ModelConfig(
    name="small-llama", vocab_size=32768, hidden_size=1024, intermediate_size=3584, num_layers=4, num_heads=8,
    num_kv_heads=2, max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002),
)

_REGISTRY = {
    c.name: c
    for c in (LLAMA3_8B, LLAMA31_8B, LLAMA3_70B, LLAMA31_70B, MIXTRAL_8X7B, TINY_LLAMA, TINY_MIXTRAL, SMALL_LLAMA,
              TINY_LLAMA_KV8, TINY_MIXTRAL_E8, TINY_BOZEVIK, SMALL_BOZEVIK, SMALL_BOZEVIK_MOE, TINY_LEMUNEX,
              SMALL_LEMUNEX, SMALL_LEMUNEX_MOE, TINY_KOMAZEN, SMALL_KOMAZEN, TINY_DALALIX, SMALL_DALALIX)
}
_ALIASES = {
    "llama3": "llama3:8b",
    "llama3:latest": "llama3:8b",
    "llama3:8b-instruct": "llama3:8b",
    "llama3.1": "llama3.1:8b",
    "llama3.1:latest": "llama3.1:8b",
    "meta-llama/meta-llama-3-8b": "llama3:8b",
    "meta-llama/meta-llama-3-8b-instruct": "llama3:8b",
    "meta-llama/llama-3.1-8b-instruct": "llama3.1:8b",
    "meta-llama/meta-llama-3-70b-instruct": "llama3:70b",
    "meta-llama/llama-3.1-70b-instruct": "llama3.1:70b",
    "mixtral": "mixtral:8x7b",
    "mixtral:latest": "mixtral:8x7b",
    "mistralai/mixtral-8x7b-instruct-v0.1": "mixtral:8x7b",
}


def resolve(model_name: str) -> ModelConfig:
    key = model_name.strip().lower()
    key = _ALIASES.get(key, key)
    if key not in _REGISTRY:
        raise KeyError(f"unknown modelName {model_name!r}; known: {sorted(_REGISTRY) + sorted(_ALIASES)}")
    return _REGISTRY[key]


def known_models() -> list[str]:
    return sorted(set(_REGISTRY) | set(_ALIASES))


def from_config_json(cfg: dict, name: str = "hf", shapes: dict | None = None):
    """The model configuration of a checkpoint directory's config.json: the design is chosen by its
    ``architecture`` key (Bozevik, Lemunex, Komazen, Dalalix), otherwise the HuggingFace Llama / Mixtral keys.  ``shapes``: the
    checkpoint's tensor shapes, for designs that leave some sizes to them."""
    if cfg.get("architecture") == "Bozevik":
        return bozevik_from_config(cfg, name)
    if cfg.get("architecture") == "Lemunex":
        return lemunex_from_config(cfg, name, shapes)
    if cfg.get("architecture") == "Komazen":
        return komazen_from_config(cfg, name)
    if cfg.get("architecture") == "Dalalix":
        return dalalix_from_config(cfg, name)
    return from_hf_config(cfg, name)


def from_hf_config(cfg: dict, name: str = "hf") -> ModelConfig:
    """Build a ModelConfig from a HuggingFace ``config.json`` dict (Llama / Mixtral)."""
    d = cfg["hidden_size"]
    nh = cfg["num_attention_heads"]
    eos = cfg.get("eos_token_id", 2)
    return ModelConfig(
        name=name,
        vocab_size=cfg["vocab_size"],
        hidden_size=d,
        intermediate_size=cfg["intermediate_size"],
        num_layers=cfg["num_hidden_layers"],
        num_heads=nh,
        num_kv_heads=cfg.get("num_key_value_heads", nh),
        head_dim=cfg.get("head_dim", d // nh),
        rope_theta=float(cfg.get("rope_theta", 10000.0)),
        rms_eps=float(cfg.get("rms_norm_eps", 1e-5)),
        max_position=int(cfg.get("max_position_embeddings", 8192)),
        rope_scaling=cfg.get("rope_scaling"),
        tie_embeddings=bool(cfg.get("tie_word_embeddings", False)),
        num_experts=int(cfg.get("num_local_experts", 0)),
        top_k=int(cfg.get("num_experts_per_tok", 2)),
        bos_token_id=int(cfg.get("bos_token_id", 1)),
        eos_token_ids=tuple(eos) if isinstance(eos, list) else (int(eos),),
        chat_format="mistral" if cfg.get("model_type") == "mixtral" else "llama3",
    )
