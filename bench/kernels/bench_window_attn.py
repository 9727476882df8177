"""Time the windowed prompt attention kernel (tiled) and the decode form at the family bench's shapes; with --bias the
causal form with the logarithmic distance bias."""
import torch, time, sys
sys.path.insert(0, __import__('os').path.dirname(__import__('os').path.dirname(__import__('os').path.dirname(__import__('os').path.abspath(__file__)))))
from symmetry_amd import ops
dev = 'cuda'
BIAS = "--bias" in sys.argv
def run(H, G, D, win, nseq, n, ctx0=0, BS=64, impl=1):
    bias = torch.stack([torch.rand(H) + 0.2, torch.rand(H) * 0.5 + 0.05]).to(dev) if BIAS else None
    if BIAS:
        win = 1 << 30
    NBs = -(-(ctx0 + n) // BS)
    NB = nseq * NBs + 1
    bt = (torch.arange(nseq * NBs, dtype=torch.int32).view(nseq, NBs) + 1).to(dev)
    kc = torch.randn(NB, BS, G, D, device=dev).bfloat16(); vc = torch.randn(NB, BS, G, D, device=dev).bfloat16()
    pos = torch.arange(ctx0, ctx0 + n, dtype=torch.int32).repeat(nseq).to(dev)
    row_seq = torch.arange(nseq, dtype=torch.int32).repeat_interleave(n).to(dev)
    cu = (torch.arange(nseq + 1, dtype=torch.int32) * n).to(dev)
    tiles = torch.tensor(sorted([(i, r) for i in range(nseq) for r in range(0, n, 64)], key=lambda t: -t[1]), dtype=torch.int32, device=dev)
    T = nseq * n
    q = torch.randn(T, H, D, device=dev).bfloat16(); out = torch.empty_like(q)
    f = lambda: ops.window_attn(q, kc, vc, bt, row_seq, pos, win, D ** -0.5, None, out, tiles if n > 1 else None, cu if n > 1 else None, impl=impl, bias=bias)
    for _ in range(3): f()
    torch.cuda.synchronize(); t0 = time.perf_counter()
    for _ in range(20): f()
    torch.cuda.synchronize(); us = (time.perf_counter() - t0) / 20 * 1e6
    pairs = sum(min(p + 1, win) for p in range(ctx0, ctx0 + n)) * nseq * H
    win = "causal+bias" if BIAS else win
    print(f"H{H} G{G} D{D} win{win} seqs{nseq} rows{n} ctx{ctx0}: {us:8.1f} us  {pairs * 4 * D / us / 1e6:7.1f} TFLOP/s", flush=True)
run(16, 4, 128, 1024, 8, 1024)
run(16, 4, 128, 1024, 8, 1024, impl=2)
run(32, 8, 128, 1024, 8, 1024)
run(32, 8, 128, 1024, 8, 1024, impl=2)
run(16, 4, 128, 4096, 2, 4096)
run(16, 4, 128, 512, 2, 4096)
run(16, 4, 128, 1024, 8, 1, ctx0=1023)
run(32, 8, 128, 1024, 64, 1, ctx0=2047)
