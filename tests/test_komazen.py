"""Komazen through the engine and op by op, against the plain oracle in tests/komazen_oracle.py.

Every test builds its own small configuration and random weights (sizes all different from one another and from any
shipped checkpoint), writes them as a checkpoint, loads that through the engine, and compares with the oracle.  The CPU
runs use the torch reference ops, the ``gpu`` ones the HIP kernels; float32 comparisons are tight (rounding only),
bfloat16 ones use the spread that bf16 rounding gives.  A dictated step goes through LLMEngine.replay_step, i.e. the
scheduler, the block / slot managers, the runner's packed metadata (and decode hipGraphs on the GPU) and model.forward.
"""
from __future__ import annotations

import copy
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import komazen_oracle as O  # noqa: E402

from symmetry_amd import ops  # noqa: E402
from symmetry_amd.engine.llm_engine import EngineConfig, LLMEngine  # noqa: E402
from symmetry_amd.engine.sequence import SamplingParams  # noqa: E402
from symmetry_amd.models import config as C  # noqa: E402
from symmetry_amd.models.weights import komazen_random_weights, save_komazen_checkpoint  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def say(*a):
    print(*a, flush=True)


# ---- configurations ---------------------------------------------------------------------------------------------
def lat(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, q_rank=14, window=7, dims=None, base=100.0, scale=0.3, src=None):
    return C.LatentMixerSpec(heads, dim, rot_dim, vdim, kv_rank, q_rank, base, rot_dim if dims is None else dims, scale, src,
                             window, True, True)


def att(heads=6, kv=2, dim=10, vdim=14, scale=0.4):
    return C.BiasedAttnSpec(heads, kv, dim, vdim, scale)


def cfg_mixed(width=40, vocab=67, taps=3, alpha=1.7):
    """Every branch once: latent layers that own a cache and that borrow one, windows shorter and longer than the
    prompts, rotary on part of the rotated dims, plain attention with 3 and 1 query heads per key head, layers with
    and without feed-forward; all head sizes different from one another."""
    layers = (
        C.KomazenLayer("latent_attention", lat(), C.GeluGluSpec(56)),
        C.KomazenLayer("attention", att(), C.GeluGluSpec(24)),
        C.KomazenLayer("latent_attention", lat(heads=2, dim=6, vdim=16, q_rank=9, window=200, src=0), None),
        C.KomazenLayer("latent_attention", lat(heads=5, dim=4, rot_dim=12, vdim=6, kv_rank=9, q_rank=30, window=19, dims=8,
                                               base=31.0), C.GeluGluSpec(32)),
        C.KomazenLayer("attention", att(heads=2, kv=2, dim=7, vdim=3, scale=0.9), None),
        C.KomazenLayer("latent_attention", lat(heads=1, dim=16, rot_dim=12, vdim=8, kv_rank=9, q_rank=5, window=1, dims=8,
                                               base=31.0, src=3), C.GeluGluSpec(16)),
    )
    return C.KomazenConfig(name="t-mixed", vocab_size=vocab, hidden_size=width, layers=layers, embed_scale=3.5,
                           postln_alpha=alpha, conv_taps=taps, norm_eps=1e-5)


def cfg_tiled(width=64, vocab=97, taps=5):
    """Head sizes that the tiled kernels take (cache rows of 64 + 32, plain heads of 32 for keys and values), windows
    that cross blocks."""
    layers = (
        C.KomazenLayer("latent_attention", lat(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, q_rank=48, window=40),
                       C.GeluGluSpec(128)),
        C.KomazenLayer("attention", att(heads=8, kv=2, dim=32, vdim=32, scale=0.25), C.GeluGluSpec(64)),
        C.KomazenLayer("latent_attention", lat(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, q_rank=48, window=23, src=0),
                       C.GeluGluSpec(64)),
    )
    return C.KomazenConfig(name="t-tiled", vocab_size=vocab, hidden_size=width, layers=layers, embed_scale=0.8,
                           postln_alpha=2.5, conv_taps=taps, norm_eps=1e-6)


def cfg_plain(width=24, vocab=50):
    """The values at which parameters vanish: one tap (no carried input), alpha 1, embedding scale 1."""
    layers = (C.KomazenLayer("attention", att(heads=2, kv=1, dim=8, vdim=8), C.GeluGluSpec(32)),
              C.KomazenLayer("latent_attention", lat(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=12, q_rank=12, window=3),
                             C.GeluGluSpec(16)))
    return C.KomazenConfig(name="t-plain", vocab_size=vocab, hidden_size=width, layers=layers, embed_scale=1.0,
                           postln_alpha=1.0, conv_taps=1, norm_eps=1e-5)


def checkpoint(cfg, tmp_path, seed=0, sharpen=None):
    w = komazen_random_weights(cfg, seed=seed)
    if sharpen:
        sharpen(w.tensors)
    path = str(tmp_path / f"{cfg.name}-{seed}")
    save_komazen_checkpoint(w, path)
    return path, C.komazen_to_config(cfg), {k: v.to(torch.bfloat16) for k, v in w.tensors.items()}


def engine(path, device, dtype, blocks=24, seqs=4, block_size=16, graphs=True):
    return LLMEngine(EngineConfig(model="t", weights=path, dtype=dtype, device=device, max_num_seqs=seqs,
                                  block_size=block_size, num_kv_blocks=blocks + 1, max_model_len=blocks * block_size,
                                  max_num_batched_tokens=8192, use_graphs=graphs, enable_prefix_caching=False,
                                  pipeline=False))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run_schedule(eng, prompts: dict, schedule: list) -> dict:
    """schedule: steps of [(request, tokens this step)]; every position's logits are asked for.  -> id -> [n, V]."""
    at = {r: 0 for r in prompts}
    got = {r: [] for r in prompts}
    for step in schedule:
        entries, ends = [], []
        for r, n in step:
            lo = at[r]
            entries.append((r, prompts[r][lo:lo + n], list(range(n))))
            at[r] = lo + n
            if at[r] == len(prompts[r]):
                ends.append(r)
        lg = eng.replay_step(entries, ends)
        o = 0
        for r, n in step:
            got[r].append(lg[o:o + n].clone())
            o += n
    return {r: torch.cat(v) for r, v in got.items() if v}


def err(a, b):
    d = (a.double() - b.double())
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / b.double().std(-1).clamp_min(1e-6)).max())


TOL = {"float32": 2e-4, "bfloat16": 0.15}   # bf16: a lost mechanism gives errors near 1


def oracle_logits(cj, W, toks):
    return O.forward(cj, W, toks).float()


def _sharp(t):
    """Attention that looks hard at single keys: a key one place outside a window, or a lost far key, moves the logits
    by far more than the tolerance."""
    for k in t:
        if k.endswith("mix.uq"):
            t[k] = t[k] * 4.0
        if k.endswith("mix.temp"):
            t[k] = t[k] * 6.0


# ---- the whole model through the engine ------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("make", [cfg_mixed, cfg_tiled, cfg_plain])
def test_prompt_decode_portions(tmp_path, device, dtype, make):
    """Whole prompt, prompt then token-by-token decoding, portions down to two tokens, and token by token from the first
    token all give the oracle's logits."""
    say("prompt/decode/portions", make.__name__, device, dtype)
    cfg = make()
    path, cj, W = checkpoint(cfg, tmp_path)
    toks = tokens(75, cfg.vocab_size, 1)
    want = oracle_logits(cj, W, toks)
    eng = engine(path, device, dtype)
    for name, cuts in (("whole", [75]), ("decode", [30] + [1] * 45), ("portions", [2, 3, 17, 2, 16, 1, 1, 5, 2, 26]),
                       ("tokens", [1] * 24)):
        say("  ", name)
        n = sum(cuts)
        got = run_schedule(eng, {"a": toks[:n]}, [[("a", c)] for c in cuts])["a"]
        assert err(got, want[:n]) < TOL[dtype], (name, err(got, want[:n]))


def test_layer_by_layer_against_the_oracle(tmp_path):
    """The stream after every layer (float32, CPU): the first layer that differs names the mechanism."""
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=2)
    toks = tokens(33, cfg.vocab_size, 4)
    trace = []
    O.forward(cj, W, toks, trace)
    eng = engine(path, "cpu", "float32")
    seen = []
    real = ops.post_rms_norm

    def spy(x, *a):
        real(x, *a)
        seen.append(x.clone())

    ops.post_rms_norm = spy
    try:
        run_schedule(eng, {"a": toks}, [[("a", len(toks))]])
    finally:
        ops.post_rms_norm = real
    ends, k = [], -1
    for layer in cfg.layers:
        k += 2 if layer.mlp is not None else 1
        ends.append(seen[k])
    for i, (a, b) in enumerate(zip(ends, trace)):
        assert float((a.double() - b).abs().max()) < 2e-4 * float(b.abs().max()), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(tmp_path, device, dtype):
    """Unequal requests side by side (portions beside single tokens, a request that pauses), in a pool of three slots
    and few blocks that are freed and used again: every request's logits equal the oracle's for it alone."""
    say("mixed batches", device, dtype)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=3)
    P = {r: tokens(n, cfg.vocab_size, 10 + i) for i, (r, n) in enumerate([("a", 40), ("b", 23), ("c", 9), ("d", 31), ("e", 1),
                                                                           ("f", 18)])}
    sched = [[("a", 7), ("b", 2)], [("a", 1), ("b", 16), ("c", 3)], [("a", 16), ("c", 1)], [("b", 1), ("c", 1), ("a", 1)],
             [("a", 15), ("b", 4), ("c", 4)],                      # a, b, c end; their pages and slots go back
             [("d", 5), ("e", 1), ("f", 2)], [("d", 1), ("f", 1)], [("f", 15), ("d", 24)], [("d", 1)]]
    eng = engine(path, device, dtype, blocks=7, seqs=3)
    got = run_schedule(eng, P, sched)
    assert len(eng.blocks.free) == 7 and eng.slots.num_free == 3
    alone = engine(path, device, dtype) if dtype == "bfloat16" else None
    for r, toks in P.items():
        want = oracle_logits(cj, W, toks)
        assert err(got[r], want) < TOL[dtype], (r, err(got[r], want))
        if alone is not None:   # the same arithmetic without the batch: far closer than the bf16 spread
            ref = run_schedule(alone, {r: toks}, [[(r, len(toks))]])[r]
            assert err(got[r], ref) < 0.05, (r, err(got[r], ref))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("block_size", [16, 64])
def test_window_and_block_edges(tmp_path, device, block_size):
    """Sharp attention, cuts and decoding at and around the windows' and the blocks' edges (float32)."""
    say("edges", device, block_size)
    cfg = cfg_tiled()
    path, cj, W = checkpoint(cfg, tmp_path, seed=5, sharpen=_sharp)
    toks = tokens(90, cfg.vocab_size, 7)
    want = oracle_logits(cj, W, toks)
    # dropping the oldest key of a window or adding the one before it must show: the oracle with a window -+ 1 differs
    for layer in (0, 2):
        for dw in (-1, 1):
            cj2 = copy.deepcopy(cj)
            cj2["layers"][layer]["mixer"]["mask"]["size"] += dw
            assert err(oracle_logits(cj2, W, toks)[45:], want[45:]) > 50 * TOL["float32"], (layer, dw)
    eng = engine(path, device, "float32", block_size=block_size, blocks=12)
    for cuts in ([39, 1, 1, 1, 48], [40, 50], [41, 49], [22, 1, 1, 24, 42], [15, 1, 16, 1, 7] + [1] * 50, [16, 16, 8, 50],
                 [63, 1, 1, 25], [64, 2, 24]):
        assert sum(cuts) == len(toks)
        got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
        assert err(got, want) < TOL["float32"], (cuts, err(got, want))


@pytest.mark.gpu
def test_tiled_kernels_windows_and_bias_bf16(tmp_path):
    """bfloat16 on the GPU with the shapes the MFMA kernels take: prompt tiles that continue cached context, cut inside
    windows and blocks, against the oracle and against the same engine run whole."""
    cfg = cfg_tiled()
    path, cj, W = checkpoint(cfg, tmp_path, seed=6)
    toks = tokens(200, cfg.vocab_size, 9)
    want = oracle_logits(cj, W, toks)
    eng = engine(path, "cuda", "bfloat16", block_size=64, blocks=8)
    whole = run_schedule(eng, {"a": toks}, [[("a", 200)]])["a"]
    assert err(whole, want) < TOL["bfloat16"]
    for cuts in ([70, 130], [33, 64, 65, 38], [100, 1, 1, 1, 97], [17] * 11 + [13]):
        got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
        assert err(got, want) < TOL["bfloat16"], (cuts, err(got, want))
        assert err(got, whole) < 0.05, (cuts, err(got, whole))


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_and_far_keys(tmp_path, device):
    """200 tokens decoded one by one after a short prompt, two sequences of different lengths in the batch; the causal
    layers reach back to the first tokens (the oracle with the first token changed differs at the end)."""
    say("long decode", device)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=8, sharpen=_sharp)
    a, b = tokens(230, cfg.vocab_size, 20), tokens(120, cfg.vocab_size, 21)
    want_a, want_b = oracle_logits(cj, W, a), oracle_logits(cj, W, b)
    other = oracle_logits(cj, W, [(a[0] + 1) % cfg.vocab_size] + a[1:])
    assert err(other[-5:], want_a[-5:]) > 20 * TOL["float32"]
    eng = engine(path, device, "float32", blocks=30)
    sched = [[("a", 30), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 117 + [[("a", 1)]] * 83
    got = run_schedule(eng, {"a": a, "b": b}, sched)
    assert err(got["a"], want_a) < TOL["float32"] and err(got["b"], want_b) < TOL["float32"]
    if device != "cpu":
        assert eng.runner.graph_replays > 0      # decode steps ran as replayed hipGraphs


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """engine.add_request / step(): five requests, three slots, greedy; each output token is the oracle's argmax (tokens
    whose top two logits are closer than the tolerance are skipped)."""
    say("generate", device)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=11)
    eng = engine(path, device, "float32", blocks=12, seqs=3)
    prompts = [tokens(n, cfg.vocab_size, 30 + i) for i, n in enumerate((5, 19, 2, 33, 11))]
    outs = {}
    for i, p in enumerate(prompts):
        eng.add_request(f"r{i}", p, SamplingParams(max_tokens=12, ignore_eos=True))
    while eng.has_unfinished():
        for o in eng.step():
            if o.finished:
                outs[o.request_id] = list(o.seq.output_ids)
    assert len(eng.blocks.free) == 12 and eng.slots.num_free == 3
    for i, p in enumerate(prompts):
        out = outs[f"r{i}"]
        assert len(out) == 12
        lg = oracle_logits(cj, W, p + out[:-1])[len(p) - 1:]
        for j, t in enumerate(out):
            top = lg[j].topk(2).values
            assert float(lg[j].max() - lg[j][t]) <= 1e-3 * float(lg[j].std()) or float(top[0] - top[1]) < 1e-3, (i, j)


def test_config_reader_rejects_unknown_keys_and_roundtrips(tmp_path):
    cfg = cfg_mixed()
    _, cj, _ = checkpoint(cfg, tmp_path)
    assert C.from_config_json(cj, "t-mixed") == cfg
    bad = copy.deepcopy(cj)
    bad["layers"][0]["mixer"]["sink"] = 1
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x")
    bad = copy.deepcopy(cj)
    bad["layers"][2]["mixer"]["kv_from"] = 1      # not a latent layer that owns a cache
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x")
    assert C.resolve("tiny-komazen").family == "komazen"


def test_registered_model_by_name_and_checkpoint_tensors(tmp_path):
    """The registry name runs with random weights as every other modelName does (the command line's path), and equals the
    oracle; a checkpoint may carry the second norm / convolution of a layer without feed-forward, and no other extra."""
    from safetensors.torch import load_file, save_file

    from symmetry_amd.models.weights import random_weights

    c = C.resolve("tiny-komazen")
    eng = LLMEngine(EngineConfig(model="tiny-komazen", weights="random", dtype="float32", device="cpu", max_num_seqs=2,
                                 block_size=16, num_kv_blocks=9, max_model_len=128, use_graphs=False,
                                 enable_prefix_caching=False, pipeline=False, seed=3))
    W = {k: v.to(torch.bfloat16) for k, v in random_weights(c, seed=3).tensors.items()}
    toks = tokens(50, c.vocab_size, 2)
    got = run_schedule(eng, {"a": toks}, [[("a", 31)], [("a", 19)]])["a"]
    assert err(got, oracle_logits(C.komazen_to_config(c), W, toks)) < TOL["float32"]
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=4)
    f = os.path.join(path, "model.safetensors")
    t = load_file(f)
    t["l2.norm2"], t["l2.canon2"] = torch.ones(cfg.hidden_size), torch.zeros(cfg.hidden_size, cfg.conv_taps)
    save_file(t, f)
    toks = tokens(20, cfg.vocab_size, 5)
    got = run_schedule(engine(path, "cpu", "float32"), {"a": toks}, [[("a", 20)]])["a"]
    assert err(got, oracle_logits(cj, W, toks)) < TOL["float32"]
    t["l2.sink"] = torch.zeros(3)
    save_file(t, f)
    with pytest.raises(ValueError):
        engine(path, "cpu", "float32")


# ---- mechanisms alone: op against oracle function ---------------------------------------------------------------
def _dev(device, *ts):
    return [t.to(device) if torch.is_tensor(t) else t for t in ts]


def _paged(n, BS, seed):
    """A block table over shuffled blocks (block 0 stays unused), positions and cache rows of n tokens."""
    NB = n // BS + 3
    bt = (torch.randperm(NB - 1, generator=torch.Generator().manual_seed(seed))[None] + 1).int()
    pos = torch.arange(n, dtype=torch.int32)
    slots = (bt[0][(pos // BS).long()] * BS + pos % BS).int()
    return NB, bt, pos, slots


@pytest.mark.parametrize("device", DEVICES)
def test_embedding_scale_norm_after_sum_and_activations(device):
    say("op rows", device)
    torch.manual_seed(1)
    table, ids = torch.randn(30, 24), torch.randint(0, 30, (9,), dtype=torch.int32)
    x = torch.empty(9, 24)
    table, ids, x = _dev(device, table, ids, x)
    ops.embed_scale(ids, table, 2.5, x)
    assert torch.equal(x.cpu(), table.cpu()[ids.cpu().long()] * 2.5)
    for d in (24, 300, 2500):
        x0, delta, w = torch.randn(5, d), torch.randn(5, d), torch.rand(d) + 0.5
        want = O.rms_norm(1.75 * x0.double() + delta.double(), w.double(), 1e-5)
        x, dl, wd = _dev(device, x0.clone(), delta, w)
        ops.post_rms_norm(x, 1.75, dl, wd, 1e-5)
        assert float((x.cpu().double() - want).abs().max()) < 1e-5
    g, u, a = torch.randn(7, 40) * 3, torch.randn(7, 40), torch.randn(7, 20)
    gu = torch.cat([g, u], 1)
    out, out2 = torch.empty(7, 40), torch.empty(7, 20)
    gu, a, out, out2 = _dev(device, gu, a, out, out2)
    ops.gelu_tanh_mul(gu[:, :40], gu[:, 40:], out)
    assert float((out.cpu().double() - O.gelu_tanh(g.double()) * u.double()).abs().max()) < 1e-5
    ops.sigmoid_mul(a, gu[:, 3:23], out2)
    want = a.cpu().double() * torch.sigmoid(torch.cat([g, u], 1)[:, 3:23].double())
    assert float((out2.cpu().double() - want).abs().max()) < 1e-6
    ops.sigmoid_mul(a, gu[:, 3:23], a)        # in place
    assert float((a.cpu().double() - want).abs().max()) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_input_convolution_with_carried_taps(device, taps):
    """x + conv(x) over runs that continue a sequence through its state slot: whatever the cut, the result is the
    whole-sequence convolution; unused slots hold garbage that must not be read."""
    say("op residual_conv", device, taps)
    torch.manual_seed(taps)
    d, n = 37, 29
    xa, xb, w = torch.randn(n, d), torch.randn(11, d), torch.randn(d, taps) * 0.5
    want_a, want_b = O.input_conv(xa.double(), w.double()), O.input_conv(xb.double(), w.double())
    state = torch.full((3, taps - 1, d), 1e4)
    state, wd = _dev(device, state, w.t().contiguous())      # the op takes the taps tap-major
    i32 = torch.int32

    def step(rows_a, rows_b, first_a, first_b, decode=False):
        """One step: sequence a's rows (slot 2) beside sequence b's (slot 0)."""
        x = torch.cat([xa[rows_a[0]:rows_a[1]], xb[rows_b[0]:rows_b[1]]])
        na, nb = rows_a[1] - rows_a[0], rows_b[1] - rows_b[0]
        prev, save, rs = [], [], []
        r0 = 0
        for s, (cnt, first, slot) in enumerate(((na, first_a, 2), (nb, first_b, 0))):
            if not cnt:
                continue
            prev += [-1 if first else -(slot + 2)] + list(range(r0, r0 + cnt - 1))
            save += [-1] * (cnt - 1) + [slot]
            rs += [len(set(rs))] * cnt
            r0 += cnt
        runs = len(set(rs))
        cu = torch.tensor([0] + [rs.count(i) for i in range(runs)], dtype=i32).cumsum(0).to(i32)
        out = torch.empty(na + nb, d)
        x, cu, rs_t, prev, save, out = _dev(device, x, cu, torch.tensor(rs, dtype=i32), torch.tensor(prev, dtype=i32),
                                            torch.tensor(save, dtype=i32), out)
        if decode:
            cu, runs = None, na + nb
        if decode:      # the launch that convolves also moves the carried taps on
            ops.residual_conv(x, wd, state, None, rs_t, prev, runs, out, save_slot=save)
        else:
            ops.residual_conv(x, wd, state, cu, rs_t, prev, runs, out)
            ops.conv_state_update(x, state, cu, prev, save, runs)
        return out.cpu().double()

    got_a, got_b = [], []
    o = step((0, 2), (0, 5), True, True)
    got_a.append(o[:2]), got_b.append(o[2:])
    o = step((2, 3), (5, 6), False, False, decode=True)
    got_a.append(o[:1]), got_b.append(o[1:])
    o = step((3, 20), (6, 6), False, False)
    got_a.append(o)
    o = step((20, 21), (6, 11), False, False)
    got_a.append(o[:1]), got_b.append(o[1:])
    o = step((21, 29), (0, 0), False, False)
    got_a.append(o)
    assert float((torch.cat(got_a) - want_a).abs().max()) < 1e-5
    assert float((torch.cat(got_b) - want_b).abs().max()) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_prompt_sized_convolution_and_activation(device):
    """Launches of hundreds of rows (several channels / columns per thread on the GPU): two runs, one of which continues
    its slot; the gated activation in bfloat16 on views of a wider matrix."""
    say("op prompt-sized rows", device)
    torch.manual_seed(5)
    d, taps = 72, 4
    xa, xb, w = torch.randn(330, d), torch.randn(150, d), torch.randn(d, taps) * 0.5
    want_a, want_b = O.input_conv(xa.double(), w.double()), O.input_conv(xb.double(), w.double())
    state = torch.full((2, taps - 1, d), 1e4)
    state[1] = xa[27:30]                                  # sequence a's rows 0..29 ran in an earlier step
    x = torch.cat([xb, xa[30:]])
    i32 = torch.int32
    prev = torch.tensor([-1] + list(range(0, 149)) + [-(1 + 2)] + list(range(150, 449)), dtype=i32)
    save = torch.full((450,), -1, dtype=i32)
    save[149], save[449] = 0, 1
    rs = torch.tensor([0] * 150 + [1] * 300, dtype=i32)
    cu = torch.tensor([0, 150, 450], dtype=i32)
    out = torch.empty(450, d)
    x, w, state, prev, save, rs, cu, out = _dev(device, x, w.t().contiguous(), state, prev, save, rs, cu, out)
    ops.residual_conv(x, w, state, cu, rs, prev, 2, out)
    ops.conv_state_update(x, state, cu, prev, save, 2)
    assert float((out.cpu().double()[:150] - want_b).abs().max()) < 1e-5
    assert float((out.cpu().double()[150:] - want_a[30:]).abs().max()) < 1e-5
    assert torch.equal(state.cpu()[0], xb[-3:]) and torch.equal(state.cpu()[1], xa[-3:])
    gu = (torch.randn(300, 144) * 3).bfloat16()
    act = torch.empty(300, 64, dtype=torch.bfloat16)
    gu, act = _dev(device, gu, act)
    ops.gelu_tanh_mul(gu[:, :64], gu[:, 72:136], act)
    want = O.gelu_tanh(gu.cpu().double()[:, :64]) * gu.cpu().double()[:, 72:136]
    assert float((act.cpu().double() - want).abs().max()) < 0.01 * float(want.abs().max())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,d", [(1, 24), (3, 40), (4, 2500)])
def test_norm_and_convolution_in_one_launch(device, taps, d):
    """Decode rows: post_rms_norm with the convolution's arguments equals the norm followed by residual_conv and the
    state update; a row at position 0 reads no state, a row without a slot writes none."""
    say("op post_rms_norm + conv", device, taps, d)
    torch.manual_seed(taps)
    T = 5
    x0, delta, w, cw = torch.randn(T, d), torch.randn(T, d), torch.rand(d) + 0.5, torch.randn(d, taps) * 0.4
    st0 = torch.randn(7, taps - 1, d)
    prev = torch.tensor([-2, -1, -(4 + 2), -(6 + 2), -1], dtype=torch.int32)     # slots 0, -, 4, 6, - (padding row)
    save = torch.tensor([0, 3, 4, 6, -1], dtype=torch.int32)
    xa, xb, delta, w, cw, sa, sb, prev, save = _dev(device, x0.clone(), x0.clone(), delta, w, cw.t().contiguous(),
                                                    st0.clone(), st0.clone(), prev, save)
    ha, hb = torch.empty(T, d, device=device), torch.empty(T, d, device=device)
    ops.post_rms_norm(xa, 2.25, delta, w, 1e-5)
    ops.residual_conv(xa, cw, sa, None, None, prev, T, ha)
    ops.conv_state_update(xa, sa, None, prev, save, T)
    ops.post_rms_norm(xb, 2.25, delta, w, 1e-5, cw, sb, prev, save, hb)
    assert torch.allclose(xa, xb, atol=1e-6) and torch.allclose(ha, hb, atol=1e-5) and torch.allclose(sa, sb, atol=1e-6)
    want = O.rms_norm(2.25 * x0.double() + delta.cpu().double(), w.cpu().double(), 1e-5)
    assert float((xb.cpu().double() - want).abs().max()) < 1e-5
    if taps > 1:      # row 0 continued slot 0: its input one place back is that slot's newest tap
        h0 = want[0] + cw.cpu().double()[-1] * want[0] + (cw.cpu().double()[:-1] * st0[0].double()).sum(0)
        assert float((hb.cpu().double()[0] - h0).abs().max()) < 1e-4
        assert torch.equal(sb.cpu()[1], st0[1]) and torch.equal(sb.cpu()[5], st0[5])        # untouched slots


@pytest.mark.parametrize("device", DEVICES)
def test_half_layout_rotary(device):
    """rope_pairs / latent_prep in the half layout against the oracle's rotation, also with fewer turning dims than the
    vector has."""
    say("op rotary", device)
    torch.manual_seed(2)
    n, H = 21, 3
    pos = torch.arange(n, dtype=torch.int32) * 3
    for rot, dims in ((8, 8), (12, 8), (16, 2), (6, 0)):
        v = torch.randn(n, H, rot + 5)
        want = O.rotate_half(v[..., 5:].double(), pos, 31.0, dims) if dims else v[..., 5:].double()
        table = torch.zeros(64, rot // 2, 2)
        table[..., 0] = 1.0
        if dims:
            table[:, : dims // 2] = ops.rope_pair_table(64, dims, 31.0)
        out = torch.zeros(n, H, rot + 2)
        vd, posd, table, out = _dev(device, v, pos, table, out)
        if dims:
            ops.rope_pairs(vd[:, :, 5:], out[:, :, 2:], posd, table, dims)
            assert float((out.cpu()[..., 2:].double() - want).abs().max()) < 1e-5, (rot, dims)
    # latent_prep: both norms, the rotated shared key part into the paged cache row, input columns of a wider matrix
    q_rank, r, rot, dims = 10, 14, 12, 8
    z = torch.randn(n, q_rank + r + rot + 9)
    wq, wkv = torch.rand(q_rank) + 0.5, torch.rand(r) + 0.5
    table = torch.zeros(64, rot // 2, 2)
    table[..., 0] = 1.0
    table[:, : dims // 2] = ops.rope_pair_table(64, dims, 31.0)
    NB, bt, _, slots = _paged(n, 4, 3)
    cache, cq = torch.zeros(NB, 4, r + rot), torch.empty(n, q_rank)
    zd, wqd, wkvd, posd, slots, table, cache, cq = _dev(device, z, wq, wkv, pos, slots, table, cache, cq)
    ops.latent_prep(zd[:, :q_rank + r + rot], q_rank, r, rot, wqd, wkvd, 1e-5, posd, slots, table, cq, cache, dims)
    zz = z.double()
    assert float((cq.cpu().double() - O.rms_norm(zz[:, :q_rank], wq.double(), 1e-5)).abs().max()) < 1e-5
    rows = cache.cpu().view(-1, r + rot)[slots.cpu().long()].double()
    assert float((rows[:, :r] - O.rms_norm(zz[:, q_rank:q_rank + r], wkv.double(), 1e-5)).abs().max()) < 1e-5
    assert float((rows[:, r:] - O.rotate_half(zz[:, q_rank + r:q_rank + r + rot], pos, 31.0, dims)).abs().max()) < 1e-5


def _latent_case(n, H, Dk, r, BS, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, H, Dk, generator=g)
    rows = torch.randn(n, Dk, generator=g)
    NB, bt, pos, slots = _paged(n, BS, seed)
    cache = torch.zeros(NB, BS, Dk)
    cache.view(-1, Dk)[slots.long()] = rows
    return q, rows, cache, bt, pos


def _latent_want(q, rows, r, window, scale):
    n = q.shape[0]
    i = torch.arange(n)
    dist = i[:, None] - i[None, :]
    s = torch.einsum("thd,sd->hts", q.double(), rows.double()) * scale
    s = s.masked_fill((dist < 0) | (dist >= window), float("-inf"))
    return torch.einsum("hts,sd->thd", torch.softmax(s, -1), rows[:, :r].double())


@pytest.mark.parametrize("device", DEVICES)
def test_latent_attention_window_edges(device):
    """latent_attn with a sliding window on a crafted cache: one key dominates (its score stands out by a scaled query /
    key pair); rows that see it just inside the window's far edge, rows one further that must not, keys at block borders
    and at position 0; prompt rows and single rows (with split-KV partials on the GPU)."""
    say("op latent_attn window", device)
    for (n, H, Dk, r, BS, window, hot) in [(70, 3, 20, 12, 8, 9, 24), (150, 2, 96, 64, 16, 33, 63), (140, 5, 36, 36, 16, 64, 0),
                                           (40, 1, 8, 8, 4, 1, 17), (300, 4, 32, 16, 64, 130, 128)]:
        q, rows, cache, bt, pos = _latent_case(n, H, Dk, r, BS, n)
        rows[hot] *= 3.0
        q[:, :, :] += 2.0 * rows[hot] / rows[hot].norm()     # every query looks at the hot key while it is visible
        cache.view(-1, Dk)[(bt[0][(pos // BS).long()] * BS + pos % BS).long()] = rows
        want = _latent_want(q, rows, r, window, 0.35)
        # the hot key leaves the window between rows hot + window - 1 and hot + window: the outputs there differ widely
        if hot + window < n:
            assert float((want[hot + window - 1] - want[hot + window]).abs().max()) > 0.1
        out = torch.empty(n, H, r)
        rs = torch.zeros(n, dtype=torch.int32)
        qd, cached, btd, posd, rsd, out = _dev(device, q, cache, bt, pos, rs, out)
        ops.latent_attn(qd, cached, btd, rsd, posd, 0.35, r, out, window=window)
        assert float((out.cpu().double() - want).abs().max()) < 1e-4, (n, window)
        if device == "cpu":
            continue
        # single rows as a decode step sees them: every row its own sequence entry, split-KV partitions over the window
        pick = torch.tensor([0, 1, hot + window - 1, hot + window, n - 1, BS - 1, BS], dtype=torch.long).clamp(0, n - 1)
        for parts in (1, 3, 8):
            T = len(pick)
            o2 = torch.empty(T, H, r, device=device)
            po = torch.empty(T, H, parts, r, device=device) if parts > 1 else None
            pm = torch.empty(T, H, parts, 2, device=device) if parts > 1 else None
            ops.latent_attn(qd[pick.to(device)].contiguous(), cached, btd.expand(T, -1).contiguous(),
                            torch.arange(T, dtype=torch.int32, device=device), posd[pick.to(device)].contiguous(), 0.35, r, o2,
                            po, pm, window=window)
            assert float((o2.cpu().double() - want[pick]).abs().max()) < 1e-4, (n, window, parts)


@pytest.mark.gpu
def test_latent_attention_mfma_window_against_wave():
    """The MFMA kernel's prompt and decode forms with a window (bf16) against the one-wave kernel on the same cache:
    runs that continue cached context, tiles cut by the window on both sides."""
    dev = "cuda"
    for (n, H, Dk, r, BS, window) in [(300, 4, 96, 64, 64, 40), (260, 6, 128, 96, 64, 96), (200, 2, 64, 32, 16, 7),
                                      (330, 16, 96, 64, 64, 150)]:
        q, rows, cache, bt, pos = _latent_case(n, H, Dk, r, BS, 7 + n)
        want = _latent_want(q.bfloat16().float(), rows.bfloat16().float(), r, window, 0.2)
        qd, cached, btd, posd = _dev(dev, q.bfloat16(), cache.bfloat16(), bt, pos)
        rs = torch.zeros(n, dtype=torch.int32, device=dev)
        # a run of the last `m` rows that continues n - m cached tokens, as tiles of 64 rows
        for m in (n, 130, 65, 3):
            tiles = torch.tensor([[0, t] for t in range(0, m, 64)], dtype=torch.int32, device=dev)
            cu = torch.tensor([0, m], dtype=torch.int32, device=dev)
            out = torch.empty(m, H, r, device=dev, dtype=torch.bfloat16)
            used = ops.latent_attn(qd[n - m:].contiguous(), cached, btd, rs[:m], posd[n - m:].contiguous(), 0.2, r, out, None,
                                   None, tiles, cu, impl=0, window=window)
            assert used == 0
            assert float((out.float().cpu().double() - want[n - m:]).abs().max()) < 0.03, (n, window, m)
        pick = torch.tensor([0, 5, window - 1, window, n - 1], device=dev)
        T = len(pick)
        for parts in (1, 2, 5):
            o2 = torch.empty(T, H, r, device=dev, dtype=torch.bfloat16)
            po = torch.empty(T, H, parts, r, device=dev) if parts > 1 else None
            pm = torch.empty(T, H, parts, 2, device=dev) if parts > 1 else None
            used = ops.latent_attn(qd[pick].contiguous(), cached, btd.expand(T, -1).contiguous(),
                                   torch.arange(T, dtype=torch.int32, device=dev), posd[pick].contiguous(), 0.2, r, o2, po, pm,
                                   impl=0, window=window)
            assert used == 0
            assert float((o2.float().cpu().double() - want[pick.cpu()]).abs().max()) < 0.03, (n, window, parts)


def _biased_case(n, H, G, dk, dv, d, seed):
    g = torch.Generator().manual_seed(seed)
    W = {"q": torch.randn(H * dk, d, generator=g), "k": torch.randn(G * dk, d, generator=g),
         "v": torch.randn(G * dv, d, generator=g), "q.norm": torch.rand(dk, generator=g) + 0.5,
         "k.norm": torch.rand(dk, generator=g) + 0.5, "temp": torch.rand(H, generator=g) * 4 + 2,
         "r1": torch.rand(H, generator=g) + 0.2, "r2": torch.rand(H, generator=g) * 0.5 + 0.05, "o": torch.eye(H * dv)}
    h = torch.randn(n, d, generator=g)
    return {k: v.double() for k, v in W.items()}, h.double()


def _run_biased(device, W, h, H, G, dk, dv, scale, BS, dtype=torch.float32, tiles=False, rows=None):
    n = h.shape[0]
    z = torch.cat([h @ W["q"].T, h @ W["k"].T, h @ W["v"].T, h[:, :3]], 1).to(dtype)     # (+ columns that are not read)
    NB, bt, pos, slots = _paged(n, BS, n)
    kc, vc = torch.zeros(NB, BS, G, dk, dtype=dtype), torch.zeros(NB, BS, G, dv, dtype=dtype)
    q, out = torch.empty(n, H, dk, dtype=dtype), torch.empty(n, H, dv, dtype=dtype)
    bias = torch.stack([W["r1"], W["r2"]]).float()
    z, bt, pos, slots, kc, vc, q, out, bias = _dev(device, z, bt, pos, slots, kc, vc, q, out, bias)
    wq, wk, temp = _dev(device, W["q.norm"].float(), W["k.norm"].float(), W["temp"].float())
    ops.qk_norm_cache(z[:, :-3], H, G, dk, dv, wq, wk, temp, 1e-5, slots, q, kc, vc)
    rs = torch.zeros(n, dtype=torch.int32, device=device)
    if rows is not None:       # single rows as a decode step sees them
        T = len(rows)
        o2 = torch.empty(T, H, dv, dtype=dtype, device=device)
        sel = rows.to(device)
        ops.window_attn(q[sel].contiguous(), kc, vc, bt.expand(T, -1).contiguous(),
                        torch.arange(T, dtype=torch.int32, device=device), pos[sel].contiguous(), 1 << 30, scale, None, o2,
                        bias=bias)
        return o2.float().cpu().double().reshape(T, H * dv)
    tl = cu = None
    if tiles:
        tl = torch.tensor([[0, t] for t in range(0, n, 64)], dtype=torch.int32, device=device)
        cu = torch.tensor([0, n], dtype=torch.int32, device=device)
    used = ops.window_attn(q, kc, vc, bt, rs, pos, 1 << 30, scale, None, out, tl, cu, bias=bias)
    return out.float().cpu().double().reshape(n, H * dv), used


@pytest.mark.parametrize("device", DEVICES)
def test_biased_attention_far_keys_and_heads(device):
    """qk_norm_cache + window_attn with the distance bias against the oracle's attention: grouped heads (1, 2, 3 query
    heads per key head), different key / value sizes, a far key among hundreds that one head keeps looking at."""
    say("op biased attention", device)
    # (the last case: single rows over more than a thousand keys, where the GPU kernel spreads a row over sixteen waves)
    for (n, H, G, dk, dv, BS) in [(37, 4, 2, 24, 8, 8), (90, 6, 2, 10, 12, 16), (420, 2, 2, 16, 70, 64), (64, 3, 1, 7, 3, 4),
                                  (1100, 4, 2, 16, 24, 64)]:
        W, h = _biased_case(n, H, G, dk, dv, 20, n)
        m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.45}
        if n > 400:
            # head 0 asks for keys like its own input's first half; values read the second half.  The last row repeats the
            # first half of token 3, 400 places back: that key scores like the row's own, less the distance bias
            W["k"][:, 10:] = 0.0
            W["q"][:dk] = W["k"][:dk]
            W["v"][:, :10] = 0.0
            W["temp"][0] = 40.0
            W["r1"][0] = 0.3
            h[-1, :10] = h[3, :10]
        want = O.biased_attention(W, "", m, h, 1e-5)
        got, _ = _run_biased(device, W, h, H, G, dk, dv, 0.45, BS)
        assert float((got - want).abs().max()) < 2e-4 * float(want.abs().max()), (n, float((got - want).abs().max()))
        if n > 400:
            # without the far key the last rows change: it carries weight there
            W2 = dict(W)
            h2 = h.clone()
            h2[3] = -h2[3]
            assert float((O.biased_attention(W2, "", m, h2, 1e-5)[-1] - want[-1]).abs().max()) > 0.05 * float(want.abs().max())
        if device != "cpu":
            rows = torch.tensor([0, 1, BS - 1, BS, n // 2, n - 1])
            got1 = _run_biased(device, W, h, H, G, dk, dv, 0.45, BS, rows=rows)
            assert float((got1 - want[rows]).abs().max()) < 2e-4 * float(want.abs().max())


@pytest.mark.gpu
def test_biased_attention_tiled_bf16():
    """The tiled prompt kernel with the distance bias (bf16, equal key / value head sizes) against the oracle."""
    for (n, H, G, d_head, BS) in [(200, 4, 2, 32, 64), (330, 8, 2, 64, 64), (150, 2, 1, 128, 16)]:
        W, h = _biased_case(n, H, G, d_head, d_head, 24, n + 1)
        m = {"heads": H, "kv_heads": G, "dim": d_head, "vdim": d_head, "scale": 0.3}
        Wb = {k: v.bfloat16().double() for k, v in W.items()}
        want = O.biased_attention(W, "", m, h, 1e-5)
        got, used = _run_biased("cuda", Wb, h, H, G, d_head, d_head, 0.3, BS, dtype=torch.bfloat16, tiles=True)
        assert used == 1
        assert float((got - want).abs().max()) < 0.06 * float(want.abs().max()), (n, float((got - want).abs().max()))
