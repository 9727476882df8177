#!/usr/bin/env python3
"""Prefill and decode throughput of a Bozevik, Lemunex, Komazen or Dalalix stack beside the closest Llama / Mixtral stack
of equal size.

Random weights, layer shapes of real models, a few layers each (throughput per layer is what is compared; the
vocabulary projection is the same size on both sides).  Per size and family, through the engine's own scheduler:

* prefill: ``--prompts`` prompts of ``--prompt-len`` tokens arriving together, one prefill step -> prompt tokens/s;
* decode: the same sequences decoding together (hipGraph replay, pipelined) for ``--decode-steps`` steps -> tokens/s.

One JSON line per (size, family) and a last line with the ratios.  ``python bench.py --families`` runs this.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _pairs():
    from symmetry_amd.models.config import ModelConfig, _bozevik_stack

    kw = dict(max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))
    lat = dict(dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=1536)
    return {
        # width 2048: 16 heads, GLU 8192
        "w2048": (_bozevik_stack("bozevik-w2048", 32768, 2048, 4, heads=16, ff=8192, share_every=0, **lat, **kw),
                  ModelConfig("llama-w2048", 32768, 2048, 8192, 4, 16, 4, **kw)),
        # width 4096: the Llama-3-8B layer (32 heads, 8 KV heads, GLU 14336)
        "w4096": (_bozevik_stack("bozevik-w4096", 32768, 4096, 4, heads=32, ff=14336, share_every=0, **lat, **kw),
                  ModelConfig("llama-w4096", 32768, 4096, 14336, 4, 32, 8, **kw)),
        # every second layer attends its neighbour's latents (half the cache planes)
        "w4096-shared": (_bozevik_stack("bozevik-w4096s", 32768, 4096, 4, heads=32, ff=14336, share_every=2, **lat, **kw),
                         ModelConfig("llama-w4096", 32768, 4096, 14336, 4, 32, 8, **kw)),
        # routed: 16 experts, 4 per token (+ a shared expert on the Bozevik side; equal active width 6144)
        "moe-w2048": (_bozevik_stack("bozevik-moe", 32768, 2048, 4, heads=16, ff=8192, experts=16, top=4, expert_ff=1024,
                                     shared_ff=2048, share_every=2, moe_every=1, **lat, **kw),
                      ModelConfig("mixtral-w2048", 32768, 2048, 1536, 4, 16, 4, num_experts=16, top_k=4, **kw)),
    }


def _lemunex_pairs():
    """Lemunex stacks (attention + linear attention layers around state-space layers) beside the Llama / Mixtral stack of
    the same width, head count and feed-forward width; the attention window equals the benchmark's prompt length."""
    from symmetry_amd.models.config import ModelConfig, lemunex_stack

    kw = dict(max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))
    return {
        "w2048": (lemunex_stack("lemunex-w2048", 32768, 2048, "pmmp", heads=16, kv_heads=4, dim=128, window=1024,
                                gla_heads=8, gla_dim=128, gla_vdim=256, ssm_heads=64, ssm_vdim=64, ssm_state=128, ff=8192,
                                **kw),
                  ModelConfig("llama-w2048", 32768, 2048, 8192, 4, 16, 4, **kw)),
        "w4096": (lemunex_stack("lemunex-w4096", 32768, 4096, "pmmp", heads=32, kv_heads=8, dim=128, window=1024,
                                gla_heads=16, gla_dim=128, gla_vdim=256, ssm_heads=128, ssm_vdim=64, ssm_state=128,
                                ff=14336, **kw),
                  ModelConfig("llama-w4096", 32768, 4096, 14336, 4, 32, 8, **kw)),
        "moe-w2048": (lemunex_stack("lemunex-moe", 32768, 2048, "PMMP", heads=16, kv_heads=4, dim=128, window=1024,
                                    gla_heads=8, gla_dim=128, gla_vdim=256, ssm_heads=64, ssm_vdim=64, ssm_state=128,
                                    ff=8192, experts=16, top=4, identity=2, expert_ff=1024, shared_ff=2048, **kw),
                      ModelConfig("mixtral-w2048", 32768, 2048, 1536, 4, 16, 4, num_experts=16, top_k=4, **kw)),
    }


def _komazen_pairs():
    """Komazen stacks (latent attention with a sliding window, one layer attending its neighbour's cache, between plain
    grouped-head attention layers with the distance bias) beside the Llama stack of the same width, head count and
    feed-forward width; the window equals the benchmark's prompt length."""
    from symmetry_amd.models.config import ModelConfig, komazen_stack

    kw = dict(max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))
    return {
        "w2048": (komazen_stack("komazen-w2048", 32768, 2048, "LASA", heads=16, kv_heads=4, dim=128, ff=8192, window=1024,
                                embed_scale=8.0, postln_alpha=2.0, **kw),
                  ModelConfig("llama-w2048", 32768, 2048, 8192, 4, 16, 4, **kw)),
        "w4096": (komazen_stack("komazen-w4096", 32768, 4096, "LASA", heads=32, kv_heads=8, dim=128, ff=14336, window=1024,
                                embed_scale=8.0, postln_alpha=2.0, **kw),
                  ModelConfig("llama-w4096", 32768, 4096, 14336, 4, 32, 8, **kw)),
    }


def _dalalix_pairs():
    """Dalalix stacks (causal attention with biased projections, windowed attention with kept first tokens and a sink
    beside a matrix memory, two causal layers with convolved projections; four residual streams; routed clamped experts
    with group-limited choice) beside the Mixtral stack of the same width, head count, expert count and expert width, and
    beside the Lemunex stack with routed layers (the closest model with a recurrence beside windowed attention); the
    window equals the benchmark's prompt length."""
    from symmetry_amd.models.config import ModelConfig, dalalix_stack, lemunex_stack

    kw = dict(max_position=8192, bos_token_id=32000, eos_token_ids=(32001, 32002))
    dk = dict(window=1024, keep_first=4, groups=4, keep=2, streams=4, buckets=65521, conv=4)
    return {
        "w2048": (dalalix_stack("dalalix-w2048", 32768, 2048, "BPCC", heads=16, kv_heads=4, dim=128, experts=16, top=4,
                                expert_ff=1536, mem_heads=8, mem_dim=128, mem_vdim=256, **dk, **kw),
                  ModelConfig("mixtral-w2048", 32768, 2048, 1536, 4, 16, 4, num_experts=16, top_k=4, **kw)),
        "w4096": (dalalix_stack("dalalix-w4096", 32768, 4096, "BPCC", heads=32, kv_heads=8, dim=128, experts=8, top=2,
                                expert_ff=14336, mem_heads=16, mem_dim=128, mem_vdim=256, **{**dk, "groups": 2, "keep": 1},
                                **kw),
                  ModelConfig("mixtral-w4096", 32768, 4096, 14336, 4, 32, 8, num_experts=8, top_k=2, **kw)),
        "moe-w2048": (dalalix_stack("dalalix-w2048", 32768, 2048, "BPCC", heads=16, kv_heads=4, dim=128, experts=16, top=4,
                                    expert_ff=1536, mem_heads=8, mem_dim=128, mem_vdim=256, **dk, **kw),
                      lemunex_stack("lemunex-moe", 32768, 2048, "PMMP", heads=16, kv_heads=4, dim=128, window=1024,
                                    gla_heads=8, gla_dim=128, gla_vdim=256, ssm_heads=64, ssm_vdim=64, ssm_state=128,
                                    ff=8192, experts=16, top=4, identity=2, expert_ff=1024, shared_ff=2048, **kw)),
    }


def measure(mcfg, prompts: int, plen: int, steps: int, reps: int = 3) -> dict:
    import torch

    from symmetry_amd.engine.llm_engine import EngineConfig, LLMEngine
    from symmetry_amd.engine.sequence import SamplingParams

    block = 64
    eng = LLMEngine(EngineConfig(model=mcfg.name, model_config=mcfg, device="auto", max_num_seqs=prompts,
                                 max_model_len=plen + steps + 2 * block, block_size=block,
                                 num_kv_blocks=prompts * (-(-(plen + steps) // block) + 2) + 16,
                                 max_num_batched_tokens=max(8192, prompts * plen), burst_split_tokens=0,
                                 arrival_quiet_us=0, enable_prefix_caching=False))
    gpu = eng.device.type != "cpu"
    sync = torch.cuda.synchronize if gpu else (lambda: None)
    g = torch.Generator().manual_seed(0)
    pre, dec = [], []
    for rep in range(reps + 1):  # the first repetition warms up (library heuristics, graph capture)
        ids = [torch.randint(0, mcfg.vocab_size * 3 // 4, (plen,), generator=g).tolist() for _ in range(prompts)]
        seqs = [eng.add_request(f"b{rep}-{i}", p, SamplingParams(max_tokens=steps + 1, ignore_eos=True))
                for i, p in enumerate(ids)]
        sync()
        t0 = time.perf_counter()
        while any(s.first_token_time is None for s in seqs):
            eng.step()
        sync()
        t1 = time.perf_counter()
        n0 = sum(len(s.output_ids) for s in seqs)
        while eng.has_unfinished():
            eng.step()
        sync()
        t2 = time.perf_counter()
        n1 = sum(len(s.output_ids) for s in seqs)
        if rep:
            pre.append(prompts * plen / (t1 - t0))
            dec.append((n1 - n0) / (t2 - t1))
    med = lambda v: sorted(v)[len(v) // 2]
    out = {"model": mcfg.name, "params_M": round(mcfg.num_params() / 1e6, 1), "prompts": prompts, "prompt_len": plen,
           "decode_steps": steps, "prefill_tok_s": round(med(pre)), "decode_tok_s": round(med(dec)),
           "decode_ms_per_step": round(1e3 * prompts / med(dec), 3)}
    del eng
    if gpu:
        torch.cuda.empty_cache()
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sizes", default="w2048,w4096,moe-w2048")
    ap.add_argument("--prompts", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--decode-steps", type=int, default=64)
    ap.add_argument("--only", default="", help="bozevik | lemunex | komazen | dalalix | baseline: one side only (profiling)")
    ap.add_argument("--design", default="bozevik", choices=("bozevik", "lemunex", "komazen", "dalalix"),
                    help="the family measured")
    a = ap.parse_args(argv)
    pairs = {"bozevik": _pairs, "lemunex": _lemunex_pairs, "komazen": _komazen_pairs, "dalalix": _dalalix_pairs}[a.design]()
    ratios = {}
    for size in a.sizes.split(","):
        if size not in pairs:     # (a design without routed layers has no routed size)
            continue
        boz, base = pairs[size]
        rows = {}
        for side, cfg in ((a.design, boz), ("baseline", base)):
            if a.only and a.only != side:
                continue
            rows[side] = measure(cfg, a.prompts, a.prompt_len, a.decode_steps)
            print(json.dumps({"size": size, "family": side, **rows[side]}), flush=True)
        if len(rows) == 2:
            ratios[size] = {k: round(rows[a.design][k] / rows["baseline"][k], 3) for k in ("prefill_tok_s", "decode_tok_s")}
    if ratios:
        print(json.dumps({a.design + "_over_baseline": ratios}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
