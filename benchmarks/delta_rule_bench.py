"""Time the gated-delta-rule kernel (every tiling) beside the decayed linear attention kernel at equal head sizes:
prompt portions and decode-only launches.  ``python benchmarks/delta_rule_bench.py`` on a GPU box; prints one table."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch  # noqa: E402

from vllm_distributed_amd.ops import hip  # noqa: E402


def timed(fn, reps=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / reps


def main():
    hip.load()
    dev, dt = "cuda", torch.bfloat16
    for heads, dim, vdim in ((8, 128, 128), (16, 128, 128), (32, 64, 64)):
        for seqs, rows in ((4, 2048), (8, 1024), (16, 512), (128, 1), (64, 1)):
            t = seqs * rows
            x = (torch.randn(t, 2 * heads * dim + heads * vdim, device=dev) * 0.5).to(dt)
            beta = torch.randn(t, heads, device=dev).to(dt)
            dtr = torch.randn(t, heads * dim, device=dev).to(dt)
            dt_bias, a_log = torch.zeros(heads * dim, device=dev), torch.zeros(heads, device=dev) - 1.0
            state = torch.zeros(seqs + 1, heads, dim, vdim, device=dev)
            qsl = torch.arange(0, t + 1, rows, dtype=torch.int32, device=dev)
            lens = torch.full((seqs,), rows + 5, dtype=torch.int32, device=dev)
            slots = torch.arange(seqs, dtype=torch.int32, device=dev)
            line = [f"H{heads} d{dim} v{vdim} {seqs:3d} x {rows:4d}:"]
            for parts in (4, 8, 16):
                us = timed(lambda: hip.gated_delta_rule(x, heads, heads, dim, vdim, beta, dtr, dt_bias, a_log, state, slots,
                                                        qsl, lens, 1e-6, rows, parts))
                line.append(f"parts {parts}: {us:8.1f} us")
            decay = torch.full((heads,), 0.97, device=dev)
            us = timed(lambda: hip.decay_linear_attention(x, heads, dim, vdim, decay, state, slots, qsl, lens, True, rows))
            line.append(f"decayed linear attention: {us:8.1f} us")
            print("  ".join(line), flush=True)


if __name__ == "__main__":
    main()
