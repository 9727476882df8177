"""Dalalix through the engine and op by op, against the plain oracle in tests/dalalix_oracle.py.

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
import dalalix_oracle as O  # noqa: E402

from symmetry_amd import ops  # noqa: E402
from symmetry_amd.engine.llm_engine import EngineConfig, LLMEngine  # noqa: E402
from symmetry_amd.engine.sequence import SamplingParams  # noqa: E402
from symmetry_amd.models import config as C  # noqa: E402
from symmetry_amd.models.weights import dalalix_random_weights, save_dalalix_checkpoint  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def say(*a):
    print(*a, flush=True)


# ---- configurations ---------------------------------------------------------------------------------------------
def plain(heads=6, kv=2, dim=10, vdim=14, scale=0.4):
    return C.CausalAttnSpec(heads, kv, dim, vdim, scale, bias=True)


def convd(heads=4, kv=2, dim=6, vdim=9, scale=0.5, taps=3):
    return C.CausalAttnSpec(heads, kv, dim, vdim, scale, conv=taps, v_norm=True, gate=True)


def pair(heads=4, kv=2, dim=12, vdim=10, window=7, keep=2, dims=8, base=100.0, scale=0.3, mh=3, mn=9, mp=5, cap=6.0,
         ls=0.7, rs=1.3):
    left = C.WindowAttnSpec(heads, kv, dim, vdim, window, scale, C.RotarySpec(dims, base, half=True), keep_first=keep,
                            sink=True, gate=False, out_bias=False)
    return C.PairMixerSpec(left, C.MatrixMemorySpec(mh, mn, mp, cap), ls, rs)


def moe(experts=6, top=2, ff=12, limit=1.5, groups=3, keep=2):
    return C.GroupRoutedSpec(experts, top, ff, limit, groups, keep)


def cfg_mixed(width=40, vocab=67):
    """Every branch once: three streams, the pair table, all three mixers, a layer without feed-forward, layers that
    borrow weights (windowed ones and a convolving one, so cache, memory and taps are the borrower's own), windows
    shorter and longer than the prompts, rotation on part of the head; all head sizes different from one another."""
    m1, m2, f1 = pair(), convd(), moe()
    layers = (
        C.DalalixLayer("attention_2", plain(), moe(experts=4, top=1, ff=20, limit=0.8, groups=2, keep=1)),
        C.DalalixLayer("parallel", m1, f1),
        C.DalalixLayer("attention", m2, None),
        C.DalalixLayer("parallel", m1, f1, weights_of=1),
        C.DalalixLayer("parallel", pair(heads=2, kv=1, dim=8, vdim=16, window=200, keep=0, dims=8, mh=1, mn=20, mp=3, cap=3.0),
                       moe(experts=5, top=3, ff=8, groups=1, keep=1)),
        C.DalalixLayer("attention", m2, None, weights_of=2),
        C.DalalixLayer("parallel", m1, f1, weights_of=3),          # borrows from a borrower: layer 1's tensors
    )
    return C.DalalixConfig(name="t-mixed", vocab_size=vocab, hidden_size=width, layers=layers, streams=3,
                           bigram=C.HashPairSpec(29, 7, 3), logit_softcap=4.0, norm_eps=1e-5)


def cfg_tiled(width=64, vocab=97):
    """Head sizes that the tiled attention kernel takes (32 for keys and values), windows and kept tokens that cross
    blocks, four taps, a memory of 16 x 32."""
    f = moe(experts=8, top=2, ff=32, limit=2.0, groups=4, keep=2)
    layers = (
        C.DalalixLayer("parallel", pair(heads=8, kv=2, dim=32, vdim=32, window=40, keep=5, dims=16, scale=0.2, mh=2, mn=16,
                                        mp=32), f),
        C.DalalixLayer("attention", convd(heads=4, kv=2, dim=32, vdim=32, scale=0.2, taps=4), f),
        C.DalalixLayer("attention_2", plain(heads=4, kv=4, dim=32, vdim=32, scale=0.2), None),
        C.DalalixLayer("parallel", pair(heads=4, kv=4, dim=32, vdim=32, window=23, keep=70, dims=32, scale=0.2, mh=4, mn=8,
                                        mp=64), f),
    )
    return C.DalalixConfig(name="t-tiled", vocab_size=vocab, hidden_size=width, layers=layers, streams=4,
                           bigram=C.HashPairSpec(101, 13, 5), logit_softcap=30.0, norm_eps=1e-6)


def cfg_plain(width=24, vocab=50, streams=1):
    """The values at which mechanisms vanish: one stream (or none: the plain residual sum), one tap, no kept tokens, one
    group, one expert per token, as many key heads as query heads, full rotation, mixer scales of one, no pair table, no
    soft cap."""
    layers = (C.DalalixLayer("attention", convd(heads=2, kv=2, dim=8, vdim=8, taps=1), moe(experts=3, top=1, ff=16, groups=1, keep=1)),
              C.DalalixLayer("parallel", pair(heads=2, kv=2, dim=8, vdim=8, window=3, keep=0, dims=8, mh=2, mn=4, mp=4, ls=1.0,
                                              rs=1.0), None),
              C.DalalixLayer("attention_2", plain(heads=1, kv=1, dim=16, vdim=4), moe(experts=2, top=2, ff=8, groups=2, keep=2)))
    return C.DalalixConfig(name=f"t-plain{streams}", vocab_size=vocab, hidden_size=width, layers=layers, streams=streams,
                           bigram=None, logit_softcap=0.0, norm_eps=1e-5)


def cfg_plain0():
    return cfg_plain(streams=0)


def checkpoint(cfg, tmp_path, seed=0, sharpen=None):
    w = dalalix_random_weights(cfg, seed=seed)
    for k in w.tensors:       # decisive routers: few choices that bf16 rounding could flip
        if k.endswith("mlp.router"):
            w.tensors[k] = w.tensors[k] * 4.0
    if sharpen:
        sharpen(w.tensors)
    path = str(tmp_path / f"{cfg.name}-{seed}")
    save_dalalix_checkpoint(w, path)
    return path, C.dalalix_to_config(cfg), {k: v.to(torch.bfloat16) for k, v in w.tensors.items()}


def engine(path, device, dtype, blocks=24, seqs=4, block_size=16, graphs=True, pipeline=False):
    return LLMEngine(EngineConfig(model="t", weights=path, dtype=dtype, device=device, max_num_seqs=seqs,
                                  block_size=block_size, num_kv_blocks=blocks + 1, max_model_len=blocks * block_size,
                                  max_num_batched_tokens=8192, use_graphs=graphs, enable_prefix_caching=False,
                                  pipeline=pipeline))


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
    return O.forward(W, cj, toks).float()


def safe_rows(cj, W, toks, dtype, thresh=0.03):
    """Rows to compare: all of them in float32; in bfloat16 the rows before the first token at which some router's last
    chosen and first rejected experts (or groups) have logits closer than ``thresh`` while the choice carries weight
    (bf16 rounding may flip that choice, and attention and the memory carry the difference to every later token)."""
    if dtype == "float32":
        return len(toks)
    margins = []
    O.forward(W, cj, toks, margins=margins)
    if not margins:
        return len(toks)
    close = (torch.stack(margins).min(0).values < thresh).nonzero()
    return int(close[0]) if len(close) else len(toks)


def _sharp(t):
    """Attention that looks hard at single keys, and a memory that forgets slowly: a key one place outside a window, a
    lost kept token or a lost far token moves the logits by far more than the tolerance."""
    for k in t:
        if k.endswith(".q") and "right" not in k or k.endswith(".q.b"):
            t[k] = t[k] * 4.0
        if k.endswith("right.f.b"):
            t[k] = t[k] + 3.0


# ---- the whole model through the engine ------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("make", [cfg_mixed, cfg_tiled, cfg_plain, cfg_plain0])
def test_prompt_decode_portions(tmp_path, device, dtype, make):
    """Whole prompt, prompt then token-by-token decoding, portions down to two tokens, and token by token from the first
    token all give the oracle's logits."""
    say("prompt/decode/portions", make.__name__, device, dtype)
    cfg = make()
    path, cj, W = checkpoint(cfg, tmp_path, seed=1 if make is cfg_mixed else 0)   # (weights without a close router choice)
    toks = tokens(75, cfg.vocab_size, 1)
    want = oracle_logits(cj, W, toks)
    safe = safe_rows(cj, W, toks, dtype)
    assert safe >= 60, safe
    eng = engine(path, device, dtype)
    for name, cuts in (("whole", [75]), ("decode", [30] + [1] * 45), ("portions", [2, 3, 17, 2, 16, 1, 1, 5, 2, 26]),
                       ("tokens", [1] * 24)):
        say("  ", name)
        n = sum(cuts)
        got = run_schedule(eng, {"a": toks[:n]}, [[("a", c)] for c in cuts])["a"]
        m = min(n, safe)
        assert err(got[:m], want[:m]) < TOL[dtype], (name, err(got[:m], want[:m]))


@pytest.mark.parametrize("device", DEVICES)
def test_layer_by_layer_against_the_oracle(tmp_path, device):
    """The sum of the streams after every layer (float32): the first layer that differs names the mechanism."""
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=2)
    toks = tokens(33, cfg.vocab_size, 4)
    trace = []
    O.forward(W, cj, toks, trace)
    eng = engine(path, device, "float32")
    eng.model.layer_sums = []
    run_schedule(eng, {"a": toks}, [[("a", len(toks))]])
    assert len(eng.model.layer_sums) == len(trace) == cfg.num_layers
    for i, (a, b) in enumerate(zip(eng.model.layer_sums, trace)):
        assert float((a.cpu().double() - b).abs().max()) < 2e-4 * float(b.abs().max()), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(tmp_path, device, dtype):
    """Unequal requests side by side (portions beside single tokens, a request that pauses), in a pool of three slots
    and few blocks that are freed and used again: every request's logits equal the oracle's for it alone."""
    say("mixed batches", device, dtype)
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=1)
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
        m = safe_rows(cj, W, toks, dtype)
        if m:
            assert err(got[r][:m], want[:m]) < TOL[dtype], (r, err(got[r][:m], want[:m]))
        if alone is not None and m:   # the same arithmetic without the batch: far closer than the bf16 spread
            ref = run_schedule(alone, {r: toks}, [[(r, len(toks))]])[r]
            assert err(got[r][:m], ref[:m]) < 0.05, (r, err(got[r][:m], ref[:m]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("block_size", [16, 64])
def test_window_kept_tokens_sink_and_block_edges(tmp_path, device, block_size):
    """Sharp attention, cuts and decoding at and around the windows', the kept tokens' and the blocks' edges (float32)."""
    say("edges", device, block_size)
    cfg = cfg_tiled()
    path, cj, W = checkpoint(cfg, tmp_path, seed=5, sharpen=_sharp)
    toks = tokens(90, cfg.vocab_size, 7)
    want = oracle_logits(cj, W, toks)
    # dropping the oldest key of a window or the last kept token, or adding the next one, must show, and so must the sink
    for key, dw in (("size", -1), ("size", 1), ("keep_first", -1), ("keep_first", 1)):
        cj2 = copy.deepcopy(cj)
        cj2["layers"][0]["mixer"]["left"]["mask"][key] += dw
        assert err(oracle_logits(cj2, W, toks)[50:], want[50:]) > 50 * TOL["float32"], (key, dw)
    W2 = dict(W)
    W2["l0.mix.left.sink"] = W["l0.mix.left.sink"] - 30.0
    assert err(oracle_logits(cj, W2, toks), want) > 50 * TOL["float32"]
    eng = engine(path, device, "float32", block_size=block_size, blocks=12)
    for cuts in ([39, 1, 1, 1, 48], [40, 50], [41, 49], [22, 1, 1, 24, 42], [4, 1, 1, 1, 9, 1, 16, 1, 6] + [1] * 50, [16, 16, 8, 50],
                 [63, 1, 1, 25], [64, 2, 24], [69, 1, 1, 1, 18]):
        assert sum(cuts) == len(toks)
        got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
        assert err(got, want) < TOL["float32"], (cuts, err(got, want))


@pytest.mark.gpu
def test_tiled_kernel_windows_kept_tokens_sink_bf16(tmp_path):
    """bfloat16 on the GPU with the shapes the MFMA kernel takes: prompt tiles that continue cached context, cut inside
    windows, kept tokens and blocks, against the oracle and against the same engine run whole."""
    cfg = cfg_tiled()
    path, cj, W = checkpoint(cfg, tmp_path, seed=6)
    toks = tokens(200, cfg.vocab_size, 17)
    want = oracle_logits(cj, W, toks)
    m = safe_rows(cj, W, toks, "bfloat16")
    assert m >= 80, m
    eng = engine(path, "cuda", "bfloat16", block_size=64, blocks=8)
    whole = run_schedule(eng, {"a": toks}, [[("a", 200)]])["a"]
    assert err(whole[:m], want[:m]) < TOL["bfloat16"]
    for cuts in ([70, 130], [33, 31, 1, 135], [40, 1, 1, 1, 157], [17] * 11 + [13], [3, 2, 67, 128]):
        got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts])["a"]
        assert err(got[:m], want[:m]) < TOL["bfloat16"], (cuts, err(got[:m], want[:m]))
        assert err(got[:m], whole[:m]) < 0.05, (cuts, err(got[:m], whole[:m]))


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_and_far_tokens(tmp_path, device):
    """200 tokens decoded one by one after a short prompt, two sequences of different lengths in the batch; the causal
    layers and the memory reach back to the first tokens (the oracle with the first token changed differs at the end)."""
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


@pytest.mark.gpu
def test_pipelined_decode_takes_the_previous_token_from_the_device(tmp_path):
    """Pipelined decode: a step's input token is the sample the step before left on the device, and so is the token
    the pair table hashes it with; the outputs equal those of the engine that waits for every step."""
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=12)
    prompts = [tokens(n, cfg.vocab_size, 40 + i) for i, n in enumerate((7, 21, 3))]
    outs = {}
    for pipe in (False, True):
        eng = engine(path, "cuda", "float32", blocks=12, seqs=3, pipeline=pipe)
        for i, p in enumerate(prompts):
            eng.add_request(f"r{i}", p, SamplingParams(max_tokens=20, ignore_eos=True))
        res = {}
        while eng.has_unfinished():
            for o in eng.step():
                if o.finished:
                    res[o.request_id] = list(o.seq.output_ids)
        outs[pipe] = res
    assert outs[True] == outs[False] and all(len(v) == 20 for v in outs[True].values())


def test_config_reader_rejects_unknown_keys_and_roundtrips(tmp_path):
    cfg = cfg_mixed()
    _, cj, _ = checkpoint(cfg, tmp_path)
    assert C.from_config_json(cj, "t-mixed").layers == cfg.layers
    assert C.from_config_json(C.dalalix_to_config(cfg_plain0()), "x").streams == 0
    bad = copy.deepcopy(cj)
    bad["layers"][1]["mixer"]["left"]["chunk"] = 8
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x")
    bad = copy.deepcopy(cj)
    bad["layers"][3]["weights_of"] = 2            # not a layer of the same kind and sizes
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x")
    bad = copy.deepcopy(cj)
    bad["layers"][0]["mlp"]["router"]["top"] = 3  # more than the kept groups hold
    with pytest.raises(ValueError):
        C.from_config_json(bad, "x")
    assert C.resolve("tiny-dalalix").family == "dalalix"


def test_registered_model_by_name_and_checkpoint_tensors(tmp_path):
    """The registry name runs with random weights as every other modelName does (the command line's path), and equals the
    oracle; a checkpoint may carry the second norm / stream mixing of a layer without feed-forward, and no other extra;
    a layer that borrows weights has no tensors."""
    from safetensors.torch import load_file, save_file

    from symmetry_amd.models.weights import random_weights

    c = C.resolve("tiny-dalalix")
    eng = LLMEngine(EngineConfig(model="tiny-dalalix", weights="random", dtype="float32", device="cpu", max_num_seqs=2,
                                 block_size=16, num_kv_blocks=9, max_model_len=128, use_graphs=False,
                                 enable_prefix_caching=False, pipeline=False, seed=3))
    W = {k: v.to(torch.bfloat16) for k, v in random_weights(c, seed=3).tensors.items()}
    assert not any(k.startswith("l3.") for k in W)
    toks = tokens(50, c.vocab_size, 2)
    got = run_schedule(eng, {"a": toks}, [[("a", 31)], [("a", 19)]])["a"]
    assert err(got, oracle_logits(C.dalalix_to_config(c), W, toks)) < TOL["float32"]
    cfg = cfg_mixed()
    path, cj, W = checkpoint(cfg, tmp_path, seed=4)
    f = os.path.join(path, "model.safetensors")
    t = load_file(f)
    t["l2.norm2"], t["l2.hc2.in"] = torch.ones(cfg.hidden_size), torch.zeros(cfg.streams)
    save_file(t, f)
    toks = tokens(20, cfg.vocab_size, 5)
    got = run_schedule(engine(path, "cpu", "float32"), {"a": toks}, [[("a", 20)]])["a"]
    assert err(got, oracle_logits(cj, W, toks)) < TOL["float32"]
    t["l3.norm1"] = torch.ones(cfg.hidden_size)
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


def _two_runs(na, nb, first_a, first_b, slot_a=2, slot_b=0):
    """Step metadata of sequence a's rows beside sequence b's: prev_row, save_slot, row_seq, cu_q."""
    prev, save, rs, cu = [], [], [], [0]
    r0 = 0
    for cnt, first, slot in ((na, first_a, slot_a), (nb, first_b, slot_b)):
        if not cnt:
            continue
        prev += [-1 if first else -(slot + 2)] + list(range(r0, r0 + cnt - 1))
        save += [-1] * (cnt - 1) + [slot]
        rs += [len(cu) - 1] * cnt
        r0 += cnt
        cu.append(r0)
    i32 = torch.int32
    return (torch.tensor(prev, dtype=i32), torch.tensor(save, dtype=i32), torch.tensor(rs, dtype=i32),
            torch.tensor(cu, dtype=i32), len(cu) - 1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 3, 8])
def test_stream_mixing_with_the_next_norm(device, S):
    """All streams move at once from the old ones; the next sublayer's input is the normed weighted sum of the new ones;
    the gathered plain sum in front of the head."""
    say("op hyper_mix_norm", device, S)
    torch.manual_seed(S)
    for d in (24, 300, 2500):
        T = 5
        xs0, a, b = torch.randn(T, S, d), torch.randn(T, d), torch.randn(T, d)
        M, co, ci, w = torch.randn(S, S), torch.randn(S), torch.randn(S), torch.rand(d) + 0.5
        y = 0.6 * a.double() + 0.9 * b.double()
        new = torch.einsum("st,nsd->ntd", M.double(), xs0.double()) + co.double()[None, :, None] * y[:, None, :]
        want_h = O.rms_norm(torch.einsum("s,nsd->nd", ci.double(), new), w.double(), 1e-5)
        xs, ad, bd, Md, cod, cid, wd = _dev(device, xs0.clone(), a, b, M, co, ci, w)
        h = torch.empty(T, d, device=device)
        ops.hyper_mix_norm(xs, ad, 0.6, bd, 0.9, Md, cod, cid, wd, 1e-5, None, h)
        assert float((xs.cpu().double() - new).abs().max()) < 1e-4
        assert float((h.cpu().double() - want_h).abs().max()) < 1e-4
        ops.hyper_mix_norm(xs, ad, 1.0, None, 0.0, Md, cod)            # an update alone (the model's last sublayer)
        new2 = torch.einsum("st,nsd->ntd", M.double(), new) + co.double()[None, :, None] * a.double()[:, None, :]
        assert float((xs.cpu().double() - new2).abs().max()) < 1e-3
        rows = torch.tensor([4, 0, 2], device=device)
        out = torch.empty(3, d, device=device)
        ops.hyper_mix_norm(xs, w=wd, eps=1e-5, rows=rows, out=out)
        want = O.rms_norm(xs.cpu().double().sum(1)[rows.cpu()], w.double(), 1e-5)
        assert float((out.cpu().double() - want).abs().max()) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_pair_hash_embedding_carries_the_previous_token(device):
    """Two sequences over several steps, cut anywhere: the pair row of a step's first token comes from the token the
    sequence's slot carries; unused slots hold garbage; a sequence's first token takes the extra row."""
    say("op embed_pair_hash", device)
    torch.manual_seed(3)
    V, d, nb, S = 40, 20, 17, 2
    table, ptab = torch.randn(V, d), torch.randn(nb + 1, d)
    cfg = {"embedding": {"bigram": {"buckets": nb, "mul_prev": 11, "mul_cur": 5}}}
    ta, tb = tokens(14, V, 1), tokens(6, V, 2)
    want_a = O.embed_tokens({"embed": table.double(), "bigram": ptab.double()}, cfg, torch.tensor(ta))
    want_b = O.embed_tokens({"embed": table.double(), "bigram": ptab.double()}, cfg, torch.tensor(tb))
    tok_state = torch.full((3,), 39, dtype=torch.int32)
    table_d, ptab_d, tok_state = _dev(device, table, ptab, tok_state)
    got_a, got_b = [], []
    at_a = at_b = 0
    for na, nb_, decode in ((5, 2, False), (1, 1, True), (6, 0, False), (1, 1, True), (1, 2, False)):
        prev, save, rs, cu, runs = _two_runs(na, nb_, at_a == 0, at_b == 0)
        ids = torch.tensor(ta[at_a:at_a + na] + tb[at_b:at_b + nb_], dtype=torch.int32)
        x = torch.empty(na + nb_, S, d)
        ids, prev, save, cu, x = _dev(device, ids, prev, save, cu, x)
        ops.embed_pair_hash(ids, table_d, ptab_d, nb, 11, 5, prev, tok_state, x, save if decode else None)
        if not decode:
            ops.token_state_update(ids, tok_state, cu, save, runs)
        assert torch.equal(x[:, 0], x[:, 1])
        got_a.append(x[:na, 0].cpu())
        got_b.append(x[na:, 0].cpu())
        at_a, at_b = at_a + na, at_b + nb_
    assert float((torch.cat(got_a).double() - want_a).abs().max()) < 1e-6
    assert float((torch.cat(got_b).double() - want_b).abs().max()) < 1e-6
    assert tok_state.cpu().tolist() == [tb[-1], 39, ta[-1]]
    x = torch.empty(3, 1, d, device=device)
    ops.embed_pair_hash(ids[:3], table_d, None, 0, 0, 0, prev[:3], tok_state, x)      # no pair table: the token rows alone
    assert torch.equal(x[:, 0].cpu(), table[ids[:3].cpu().long()])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_convolved_projections_with_carried_taps(device, taps):
    """q | k | v through the short convolution over runs that continue a sequence through its state slot, values brought
    to unit RMS per head, written through a shuffled block table: whatever the cut, the whole-sequence result."""
    say("op conv_qkv_cache", device, taps)
    torch.manual_seed(taps)
    H, G, dk, dv, BS, n = 3, 1, 5, 7, 4, 23
    C_ = H * dk + G * dk + G * dv
    za, zb, w = torch.randn(n, C_ + 3), torch.randn(9, C_ + 3), torch.randn(C_, taps) * 0.7
    NB, bt, pos, slots_a = _paged(n, BS, 5)

    def whole(z):
        y = O.short_conv(z[:, :C_].double(), w.double())
        return y[:, :H * dk], y[:, H * dk:(H + G) * dk], O.unit_rms(y[:, (H + G) * dk:].view(-1, G, dv), 1e-5).reshape(len(z), -1)

    qa, ka, va = whole(za)
    qb, _, _ = whole(zb)
    state = torch.full((3, taps - 1, C_), 1e4)
    kc, vc = torch.zeros(NB + 3, BS, G, dk), torch.zeros(NB + 3, BS, G, dv)
    state, wd, kc, vc = _dev(device, state, w, kc, vc)
    got_a, got_b = [], []
    at_a = at_b = 0
    for na, nb_, decode in ((3, 2, False), (1, 1, True), (1, 1, True), (taps, 0, False), (1, 1, True), (16 - taps, 3, False),
                            (1, 1, True)):
        prev, save, rs, cu, runs = _two_runs(na, nb_, at_a == 0, at_b == 0)
        z = torch.cat([za[at_a:at_a + na], zb[at_b:at_b + nb_]])
        sl = torch.cat([slots_a[at_a:at_a + na], torch.full((nb_,), -1, dtype=torch.int32)])   # b's rows are not cached
        q = torch.empty(na + nb_, H, dk)
        z, sl, q, prev, save, rs, cu = _dev(device, z, sl, q, prev, save, rs, cu)
        zin = z[:, :C_]
        if decode:
            ops.conv_qkv_cache(zin, wd, state, None, None, prev, na + nb_, H, G, dk, dv, 1e-5, sl, q, kc, vc, save_slot=save)
        else:
            ops.conv_qkv_cache(zin, wd, state, cu, rs, prev, runs, H, G, dk, dv, 1e-5, sl, q, kc, vc)
            if taps > 1:
                ops.conv_state_update(zin, state, cu, prev, save, runs)
        got_a.append(q[:na].cpu().reshape(na, H * dk))
        got_b.append(q[na:].cpu().reshape(nb_, H * dk))
        at_a, at_b = at_a + na, at_b + nb_
    na = at_a
    assert float((torch.cat(got_a).double() - qa[:na]).abs().max()) < 1e-4
    assert float((torch.cat(got_b).double() - qb[:at_b]).abs().max()) < 1e-4
    rows = slots_a[:na].long()
    assert float((kc.cpu().view(-1, G * dk)[rows].double() - ka[:na]).abs().max()) < 1e-4
    assert float((vc.cpu().view(-1, G * dv)[rows].double() - va[:na]).abs().max()) < 1e-4
    if taps > 1:
        assert float(state[1].min()) == 1e4        # the unused slot was never written


@pytest.mark.parametrize("device", DEVICES)
def test_convolved_projections_long_prompt(device):
    """A prompt step of thousands of rows: two runs in one step, the second continuing its sequence from the slot."""
    say("op conv_qkv_cache long", device)
    torch.manual_seed(11)
    H, G, dk, dv, BS, taps = 2, 2, 12, 20, 64, 4
    C_ = H * dk + G * dk + G * dv
    na, nb_ = 1500, 700
    za, zb, w = torch.randn(na, C_), torch.randn(nb_ + 3, C_), torch.randn(C_, taps) * 0.7
    ya, yb = O.short_conv(za.double(), w.double()), O.short_conv(zb.double(), w.double())[3:]
    state = torch.full((3, taps - 1, C_), 1e4)
    state[0] = zb[:3]
    NB, bt, pos, slots = _paged(na + nb_, BS, 4)
    prev, save, rs, cu, runs = _two_runs(na, nb_, True, False)
    kc, vc, q = torch.zeros(NB, BS, G, dk), torch.zeros(NB, BS, G, dv), torch.empty(na + nb_, H, dk)
    z = torch.cat([za, zb[3:]])
    z, wd, state, slots, q, kc, vc, prev, save, rs, cu = _dev(device, z, w, state, slots, q, kc, vc, prev, save, rs, cu)
    ops.conv_qkv_cache(z, wd, state, cu, rs, prev, runs, H, G, dk, dv, 1e-5, slots, q, kc, vc)
    ops.conv_state_update(z, state, cu, prev, save, runs)
    y = torch.cat([ya, yb])
    rows = slots.cpu().long()
    assert float((q.cpu().double().reshape(na + nb_, -1) - y[:, :H * dk]).abs().max()) < 1e-4
    assert float((kc.cpu().view(-1, G * dk)[rows].double() - y[:, H * dk:(H + G) * dk]).abs().max()) < 1e-4
    want_v = O.unit_rms(y[:, (H + G) * dk:].view(-1, G, dv), 1e-5).reshape(na + nb_, -1)
    assert float((vc.cpu().view(-1, G * dv)[rows].double() - want_v).abs().max()) < 1e-4
    assert float((state[0].cpu().double() - zb[-3:].double()).abs().max()) == 0.0
    assert float((state[2].cpu().double() - za[-3:].double()).abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
def test_half_layout_rotation_and_cache_write(device):
    """Bias, rotation of the first dims entries of each head (entry i with i + dims / 2), the rest passing; no rotation
    and no bias where none is given."""
    say("op qkv_rope_cache half", device)
    torch.manual_seed(2)
    H, G, dk, dv, BS, n, dims = 4, 2, 10, 6, 8, 21, 6
    nq, nk, nv = H * dk, G * dk, G * dv
    z, bias = torch.randn(n, nq + nk + nv + 5), torch.randn(nq + nk + nv)
    NB, bt, pos, slots = _paged(n, BS, 3)
    rope = ops.rope_pair_table(64, dims, 50.0)
    zb = z[:, :nq + nk + nv].double() + bias.double()
    want_q = O.rotate_half(zb[:, :nq].view(n, H, dk), pos, 50.0, dims)
    want_k = O.rotate_half(zb[:, nq:nq + nk].view(n, G, dk), pos, 50.0, dims)
    q, kc, vc = torch.empty(n, H, dk), torch.zeros(NB, BS, G, dk), torch.zeros(NB, BS, G, dv)
    z, bias, pos, slots, rope, q, kc, vc = _dev(device, z, bias, pos, slots, rope, q, kc, vc)
    ops.qkv_rope_cache(z, bias, H, G, dk, dv, pos, slots, rope, q, kc, vc, half_dims=dims)
    rows = slots.cpu().long()
    assert float((q.cpu().double() - want_q).abs().max()) < 1e-4
    assert float((kc.cpu().view(-1, G, dk)[rows].double() - want_k).abs().max()) < 1e-4
    assert float((vc.cpu().view(-1, nv)[rows].double() - zb[:, nq + nk:]).abs().max()) < 1e-5
    ops.qkv_rope_cache(z, None, H, G, dk, dv, pos, slots, None, q, kc, vc)
    assert float((q.cpu().reshape(n, -1) - z.cpu()[:, :nq]).abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_windowed_attention_keeps_first_tokens_and_a_sink(device, dtype):
    """One query looks hard at one key: just inside / outside the window, the last kept token / the first that is not
    kept, a far key, keys at block borders; in prompt rows (tiled kernel where it applies) and in single rows."""
    if device == "cpu" and dtype == torch.bfloat16:
        pytest.skip("the reference op is the float32 one")
    say("op window_attn keep_first sink", device, dtype)
    torch.manual_seed(4)
    H, G, dk, dv, BS, n, window, keep = 4, 2, 32, 32, 16, 150, 37, 5
    NB, bt, pos, slots = _paged(n, BS, 9)
    k, v = torch.randn(n, G, dk) * 0.3, torch.randn(n, G, dv)
    sink = torch.tensor([0.5, -1.0, 2.0, 0.0])
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    kc, vc = torch.zeros(NB, BS, G, dk), torch.zeros(NB, BS, G, dv)
    kc.view(-1, G, dk)[slots.long()] = k
    vc.view(-1, G, dv)[slots.long()] = v
    kr, vr = kc.to(dtype).view(-1, G, dk)[slots.long()].double(), vc.to(dtype).view(-1, G, dv)[slots.long()].double()
    for target in (149 - 36, 149 - 37, 4, 5, 0, 16, 15, 127, 128):   # the key that the last query looks at
        q = torch.randn(n, H, dk) * 0.3
        kt = k[target].repeat_interleave(H // G, 0)                  # [H, dk]: each head's copy of the target key
        q[149] = kt * (12.0 / 0.3) / kt.pow(2).sum(-1, keepdim=True)   # score of the target 12, the others around +-2
        qr = q.to(dtype).double()
        want = O.softmax_attention(qr, kr, vr, 0.3, window, keep, sink.double())
        seen = O.visible(149, target, window, keep)
        wide = O.softmax_attention(qr[149:], kr, vr, 0.3, window + 1, keep + 1, sink.double()) if not seen else None
        cu = torch.tensor([0, n], dtype=torch.int32)
        tiles = torch.tensor([[0, r] for r in range(0, n, 64)], dtype=torch.int32)
        rs = torch.zeros(n, dtype=torch.int32)
        out = torch.empty(n, H, dv, dtype=dtype)
        qd, kcd, vcd, btd, rsd, posd, sinkd, out, cud, tilesd = _dev(device, q.to(dtype), kc.to(dtype), vc.to(dtype), bt, rs, pos,
                                                                       sink, out, cu, tiles)
        impl = ops.window_attn(qd, kcd, vcd, btd, rsd, posd, window, 0.3, None, out, tilesd, cud, keep_first=keep, sink=sinkd)
        assert device == "cpu" or impl == (1 if dtype == torch.bfloat16 else 0)
        assert float((out.cpu().double() - want).abs().max()) < tol, target
        one = torch.empty(1, H, dv, dtype=dtype, device=device)
        ops.window_attn(qd[149:], kcd, vcd, btd, rsd[:1], posd[149:], window, 0.3, None, one, keep_first=keep, sink=sinkd)
        assert float((one.cpu().double() - want[149:]).abs().max()) < tol, target
        if not seen:      # with the window and the kept range one longer the answer is another one
            assert float((wide - want[149:]).abs().max()) > 50 * tol, target
    nosink = torch.empty(1, H, dv, dtype=dtype, device=device)
    ops.window_attn(qd[100:101], kcd, vcd, btd, rsd[:1], posd[100:101], window, 0.3, None, nosink, keep_first=keep)
    assert float((nosink.cpu().double() - want[100:101]).abs().max()) > 0.02      # (a row that looks at no key hard)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [(3, 9, 5), (2, 16, 32), (1, 64, 63), (2, 20, 64)])
def test_matrix_memory_handed_over_through_slots(device, shape):
    """The gated memory with its running maximum and normaliser over runs cut anywhere (prompt runs beside single rows),
    states handed over through slots with garbage in the unused one, a forget gate near one so that the first tokens
    still count at the end; then the read-out (division, unit RMS per head, weight, gate)."""
    H, N, P = shape
    say("op decay_scan log gates", device, shape)
    torch.manual_seed(N)
    d, cap = 24, 5.0
    names = ("q", "k", "v", "g", "i", "f")
    rows = {"q": H * N, "k": H * N, "v": H * P, "g": H * P, "i": H, "f": H}
    W = {"m." + nm: torch.randn(rows[nm], d) * d ** -0.5 for nm in names}
    W["m.i.b"], W["m.f.b"] = torch.randn(H) - 1.0, torch.randn(H) + 4.0
    W["m.norm"], W["m.o"] = torch.rand(H * P) + 0.5, torch.eye(H * P)
    spec = {"heads": H, "dim": N, "vdim": P, "gate_cap": cap}
    ha, hb = torch.randn(41, d), torch.randn(12, d)
    Wd = {k_: v_.double() for k_, v_ in W.items()}
    want_a, want_b = O.matrix_memory(Wd, "m.", spec, ha.double(), 1e-5), O.matrix_memory(Wd, "m.", spec, hb.double(), 1e-5)
    ha2 = ha.clone()
    ha2[0] += 1.0
    assert float((O.matrix_memory(Wd, "m.", spec, ha2.double(), 1e-5)[-1] - want_a[-1]).abs().max()) > 1e-3
    state = torch.full((3, H, N + 1, P + 1), 1e4)
    (state,) = _dev(device, state)
    gb = torch.cat([W["m.i.b"], W["m.f.b"]]).to(device)
    nw = W["m.norm"].to(device)
    got_a, got_b = [], []
    at_a = at_b = 0
    for na, nb_, decode in ((7, 3, False), (1, 1, True), (1, 1, True), (17, 0, False), (1, 2, False), (14, 5, False)):
        prev, save, rs, cu, runs = _two_runs(na, nb_, at_a == 0, at_b == 0)
        h = torch.cat([ha[at_a:at_a + na], hb[at_b:at_b + nb_]])
        T = na + nb_
        z = torch.cat([h @ W["m." + nm].t() for nm in ("q", "k", "v", "g")], 1)
        gates = torch.cat([h @ W["m.i"].t(), h @ W["m.f"].t()], 1)
        y, mx, out = torch.empty(T, H, P + 1), torch.empty(T, H), torch.empty(T, H * P)
        z, gates, y, mx, out, prev, save, cu = _dev(device, z, gates, y, mx, out, prev, save, cu)
        c1, c2, c3 = H * N, 2 * H * N, 2 * H * N + H * P
        ops.decay_scan(ops.DECAY_LOG_GATES, z[:, :c1], z[:, c1:c2], z[:, c2:c3], gates, gb, cap, None, N ** -0.5, H, N, P, 1,
                       state, None if decode else cu, prev, save, T if decode else runs, y, mout=mx)
        ops.memory_norm_gate(y, mx, z[:, c3:], nw, 1e-5, out)
        got_a.append(out[:na].cpu())
        got_b.append(out[na:].cpu())
        at_a, at_b = at_a + na, at_b + nb_
    assert float((torch.cat(got_a).double() - want_a).abs().max()) < 2e-4
    assert float((torch.cat(got_b).double() - want_b).abs().max()) < 2e-4
    assert float(state[1].min()) == 1e4            # the unused slot was never written


@pytest.mark.parametrize("device", DEVICES)
def test_router_groups_limit_the_choice(device):
    """The second best expert overall sits in a group that is not kept: the choice stays inside the kept group, and the
    weights are the chosen scores over their sum; without groups the plain top-k."""
    say("op softmax_topk groups", device)
    d, E = 8, 6
    Wr = torch.zeros(E, d)
    for e, s in enumerate((0.1, 2.0, 0.4, 1.5, -1.0, 0.3)):     # groups {0,1} {2,3} {4,5}
        Wr[e, 0] = s
    x = torch.zeros(3, d)
    x[:, 0] = torch.tensor([1.0, 2.0, -1.0])
    ids, w = torch.zeros(6, dtype=torch.int32), torch.zeros(6)
    x, Wr, ids, w = _dev(device, x, Wr, ids, w)
    ops.softmax_topk(x, Wr, None, 2, ids, w, 3, 1, True)
    for t in range(3):
        i2, w2, _ = O.route((x[t].cpu().double() @ Wr.cpu().double().t()), 2, 3, 1)
        assert ids.cpu().view(3, 2)[t].tolist() == i2.tolist(), t
        assert float((w.cpu().view(3, 2)[t].double() - w2).abs().max()) < 1e-6
    assert ids.cpu().view(3, 2)[0].tolist() == [1, 0]            # not expert 3, the second best overall
    ops.softmax_topk(x, Wr, None, 2, ids, w, 3, 2, True)
    assert ids.cpu().view(3, 2)[0].tolist() == [1, 3]
    ops.softmax_topk(x, Wr, None, 2, ids, w)
    s = torch.softmax(x.cpu() @ Wr.cpu().t(), -1)
    assert ids.cpu().view(3, 2)[0].tolist() == [1, 3] and abs(float(w[0]) - float(s[0, 1])) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_clamped_experts_and_soft_cap(device):
    say("op clamped_glu softcap", device)
    torch.manual_seed(6)
    g, u = torch.randn(5, 24) * 3, torch.randn(5, 24) * 3
    gu, out = torch.cat([g, u], 1), torch.empty(5, 24)
    gu, out = _dev(device, gu, out)
    ops.hyb_clamped_glu(gu, 1.5, 1.702, out)
    gc, uc = g.double().clamp(max=1.5), u.double().clamp(-1.5, 1.5)
    assert float((out.cpu().double() - gc * torch.sigmoid(1.702 * gc) * (uc + 1)).abs().max()) < 1e-5
    lg = torch.randn(4, 300) * 20
    (x,) = _dev(device, lg.clone())
    ops.logit_softcap(x, 7.0)
    assert float((x.cpu().double() - 7.0 * torch.tanh(lg.double() / 7.0)).abs().max()) < 1e-5
