#!/usr/bin/env python3
"""End-to-end comparison in the format of the reference's README table (README.md:25-36 of the
reference: sequence length, kept ratio, `flash_attention_custom_mask` time including mask
preprocessing, naive matmul+softmax time, speed-up), for this package on an MI355X.

    python kernel_test.py [--seq-len 6400 17536 32000] [--ratio 0.1 1.0] [--heads 8] [--dim 64]

Like the reference's kernel-test.py (:12-19) the inputs are N(0,1) fp16, the block mask is
Bernoulli(ratio), and the naive path expands the mask to N x N; unlike it the runs are seeded,
repeated (median), and the naive path is skipped when its N x N scores would not fit.
"""
import argparse
import math
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from fa2_custom_mask import flash_attention_custom_mask  # noqa: E402
from fa2_custom_mask import utils  # noqa: E402


def timed(fn, reps):
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--seq-len", type=int, nargs="+", default=[6400, 17536, 32000])
    ap.add_argument("--ratio", type=float, nargs="+", default=[0.1, 1.0])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--heads", type=int, default=8)          # kernel-test.py:7
    ap.add_argument("--dim", type=int, default=64)
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--naive-limit-gb", type=float, default=40.0,
                    help="skip the naive path when its fp16 N x N scores exceed this many GB")
    args = ap.parse_args(argv)
    dev = torch.device("cuda:0")
    print("| [seq_len, dim] | ratio | custom mask incl. preprocessing (s) | cached lists (s) | naive matmul+softmax (s) | speed-up | max abs diff |")
    print("|---|---|---|---|---|---|---|")
    for n in args.seq_len:
        for r in args.ratio:
            g = torch.Generator(device="cpu").manual_seed(1234)
            shape = (args.batch, args.heads, n, args.dim)
            q, k, v = [torch.randn(shape, generator=g).to(torch.float16).to(dev) for _ in range(3)]
            nb = n // 64
            mask = (torch.rand(args.batch, args.heads, nb, nb, generator=g) < r).to(dev)
            scale = 1.0 / math.sqrt(args.dim)

            def cold():
                utils.lists_cache.clear()        # every call indexes the mask again
                return flash_attention_custom_mask(q, k, v, mask, scale)

            t_cold = timed(cold, args.reps)
            t_warm = timed(lambda: flash_attention_custom_mask(q, k, v, mask, scale), args.reps)
            out = flash_attention_custom_mask(q, k, v, mask, scale)
            scores_gb = args.batch * args.heads * n * n * 2 / 1e9
            if scores_gb * 2 <= args.naive_limit_gb:
                def naive():
                    big = mask.repeat_interleave(64, 2).repeat_interleave(64, 3)
                    a = torch.matmul(q, k.transpose(-2, -1)) * scale
                    a = a.masked_fill(~big, float("-inf"))
                    return torch.matmul(torch.softmax(a, dim=-1), v)
                t_naive = timed(naive, max(1, args.reps // 2))
                ref = torch.nan_to_num(naive().float(), nan=0.0)     # rows without a kept tile: 0 here
                diff = "%.2e" % float((out.float() - ref).abs().max())
                naive_s, speed = "%.4f" % t_naive, "%.1f" % (t_naive / t_cold)
                del ref
            else:
                naive_s, speed, diff = "skipped", "-", "-"
            print("| [%d, %d] | %.2f | %.6f | %.6f | %s | %s | %s |" % (n, args.dim, r, t_cold, t_warm, naive_s, speed, diff))
            del q, k, v, mask, out
            torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
