"""Attention with every query head's weights on every value head (``window_bias_attention(..., crossed=True)``)
beside the ordinary form of the same kernel, on synthetic caches: microseconds per launch for a prompt step and for
decoded rows, by the number of value heads that share one computation of the scores."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch  # noqa: E402
from vllm_distributed_amd.ops import hip  # noqa: E402

hip.load()
dev = "cuda"
torch.manual_seed(0)


def timeit(fn, iters=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1e3 / iters


def run(nseq, qlen, ctx, hq, hkv, d=128, bs=64):
    total = ctx + qlen
    nb = (total + bs - 1) // bs
    k = (torch.randn(nseq * nb, hkv, bs, d, device=dev) * 0.5).to(torch.bfloat16)
    v = (torch.randn(nseq * nb, hkv, bs // 8, d, 8, device=dev) * 0.5).to(torch.bfloat16)
    bt = torch.randperm(nseq * nb, device=dev).to(torch.int32).view(nseq, nb)
    sl = torch.full((nseq,), total, device=dev, dtype=torch.int32)
    qsl = (torch.arange(nseq + 1, device=dev) * qlen).to(torch.int32)
    pos = (torch.arange(qlen, device=dev) + ctx).repeat(nseq).to(torch.int32)
    seq = None if qlen == 1 else torch.arange(nseq, device=dev).repeat_interleave(qlen).to(torch.int32)
    q = torch.randn(nseq * qlen, hq, d, device=dev).to(torch.bfloat16)
    r1, r2 = torch.rand(hq, device=dev), torch.rand(hq, device=dev)
    args = (q, k, v, bt, qsl, sl, seq, pos, d ** -0.5, 0.0, 0, 0, r1, r2, None, None, qlen)
    line = f"n={nseq:4d} q={qlen:5d} ctx={ctx:5d} Hq={hq:3d} Hkv={hkv}: ordinary {timeit(lambda: hip.window_bias_attention(*args)):8.1f} us"
    for cg in (1, 2, 4):
        hip.CROSS_GROUP_PROMPT = hip.CROSS_GROUP_DECODE = cg
        line += f"  crossed/{cg} {timeit(lambda: hip.window_bias_attention(*args, crossed=True)):8.1f}"
    print(line, flush=True)


if __name__ == "__main__":
    for hq, hkv in ((16, 4), (8, 2), (32, 8)):
        run(128, 1, 1087, hq, hkv)
        run(64, 1, 4095, hq, hkv)
        run(8, 1024, 0, hq, hkv)
        run(4, 2048, 0, hq, hkv)
