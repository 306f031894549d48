#!/usr/bin/env python3
"""Benchmark of the block-sparse attention forward on one MI355X.

Workload (BASELINE.json configs[2]): forward, B=1 H=1 N=17536 D=64 fp16, 274x274 tile grid,
kept-tile ratios {0.05, 0.1, 0.25, 0.5, 1.0} (random tiles + forced diagonal), kernel time
measured separately from mask preprocessing.  One "step" is one forward pass at keep 1.0 with
q/k/v and the kept-tile lists already resident in HBM.  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "customize-block-sparse-attention-with-triton_amd")
sys.path.insert(0, PKG)
sys.path.insert(0, ROOT)

N, D, TILE = 17536, 64, 64
NB = N // TILE
KEEPS = [0.05, 0.1, 0.25, 0.5, 1.0]
PEAK_F16_TFLOPS = 2500.0     # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0
SEED = 1234 + 2
PROFILE = os.path.join(ROOT, "profiles", "fwd_kernel_n17536_d64_fp16.md")


def measured_traffic():
    """HBM-side bytes of one keep-1.0 forward launch as the committed rocprofv3 summary states them (two
    --pmc runs, FETCH_SIZE and WRITE_SIZE, scaled by the readings of a plain device copy): the line
    `traffic_bytes_per_launch = <bytes>` of the summary, or None when the summary does not have it.
    A counter run cannot happen inside this program; the summary names the command and the commit."""
    import re
    try:
        m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", open(PROFILE).read())
    except OSError:
        return None
    return int(m.group(1)) if m else None


def tile_flops(kept):
    return kept * 4.0 * TILE * TILE * D          # QK^T + PV per kept tile


SETTLE_S = 0.1     # untimed run-in before every timed region


def settle(fn, torch, seconds=SETTLE_S):
    """Runs fn back to back, untimed, for about `seconds`: after an idle spell (set-up on the host, a
    synchronisation) the GPU needs some tens of milliseconds of load before its clock is where it stays
    (the dense launch measures 114 us in the first 20 ms, 105 us in the next 20 ms and 103.5 us from 60 ms on)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def event_times(fn, iters, warmup, torch):
    for _ in range(warmup):
        fn()
    settle(fn, torch)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) for a, b in evs)       # ms


def fwd_bwd_c5(torch, dev, fm, steps, warmup, check=True, uniform=0):
    """HIP-event times of one forward call and one backward call at configs[4], in both output modes:
    results typed bf16 like the inputs (what autograd hands back; P and dS rounded to bf16) and results in
    fp32 (P and dS kept in fp16).  With check: relative L2 errors of O, dQ, dK, dV against the oracle
    (numpy fp32 closed-form gradients) on two of the 32 heads.
    uniform = L > 0 replaces the mask of configs[4] by one with exactly L kept tiles in every row and every
    column (row r keeps the columns r + 7 j mod 128, j < L): the time of a launch as a function of the list
    length separates what a launch costs per tile from what it costs per workgroup."""
    import numpy as np
    B, H, Nc, Dc = 2, 16, 8192, 128
    nbc = Nc // TILE
    g = torch.Generator().manual_seed(1238)
    q, k, v, do = [torch.randn(B, H, Nc, Dc, generator=g).to(torch.bfloat16) for _ in range(4)]
    m = (torch.rand(1, 1, nbc, nbc, generator=g) < 0.25) | torch.eye(nbc, dtype=torch.bool)
    m = torch.tril(m.reshape(nbc, nbc)).reshape(1, 1, nbc, nbc)
    if uniform:
        m = torch.zeros(1, 1, nbc, nbc, dtype=torch.bool)
        r = torch.arange(nbc)
        for j in range(uniform):
            m[0, 0, r, (r + 7 * j) % nbc] = True
    qd, kd, vd, dod, md = [x.to(dev) for x in (q, k, v, do, m)]
    lists = fm.block_mask_to_lists(md)
    lists_t = fm.block_mask_to_lists(md, transpose=True)
    tiles = int(lists.counts[1]) * B * H
    sc = 1.0 / Dc ** 0.5
    ff, fb = tiles * 4.0 * TILE * TILE * Dc, tiles * 10.0 * TILE * TILE * Dc
    out = {"workload": "BASELINE configs[4]: fwd+bwd B=2 H=16 N=8192 D=128 bf16, block-causal keep 0.25 shared mask"
                       if not uniform else "shape of BASELINE configs[4] with %d kept tiles in every row and column" % uniform,
           "kept_tiles": tiles,
           "note": "one bsattn_fwd call and one bsattn_bwd call (dq kernel, which also computes delta, and dkdv kernel), buffers allocated beforehand"}
    ref = None
    if check:
        from oracle import bsattn_oracle as orc
        heads = [(0, 0), (1, 15)]
        ref = {}
        for (b, h) in heads:
            sl = (slice(b, b + 1), slice(h, h + 1))
            f = lambda x: x[sl].float().numpy()
            o_r = orc.naive_attention(f(q), f(k), f(v), m.numpy(), sc)
            dq_r, dk_r, dv_r, _ = orc.attention_backward(f(q), f(k), f(v), m.numpy(), sc, f(do))
            ref[(b, h)] = (o_r, dq_r, dk_r, dv_r)
    for mode, odt in (("bf16_results", None), ("fp32_results", torch.float32)):
        fplan = fm.ForwardPlan(qd, kd, vd, lists, sc, out_dtype=odt)
        o, lse = fplan.run()
        o_in = o if o.dtype == qd.dtype else o.to(qd.dtype)
        bplan = fm.BackwardPlan(qd, kd, vd, o_in, dod, lse, lists, lists_t, sc, out_dtype=odt)
        tf = event_times(fplan.run, steps, warmup, torch)
        tb = event_times(bplan.run, steps, warmup, torch)
        mf, mb = tf[len(tf) // 2], tb[len(tb) // 2]
        rec = {"fwd_ms": round(mf, 5), "fwd_tflops": round(ff / mf / 1e9, 1), "bwd_ms": round(mb, 5),
               "bwd_tflops": round(fb / mb / 1e9, 1),
               "frac_mfma_peak": {"fwd": round(ff / mf / 1e9 / PEAK_F16_TFLOPS, 4), "bwd": round(fb / mb / 1e9 / PEAK_F16_TFLOPS, 4)}}
        if ref is not None:
            dq, dk, dv = bplan.run()
            torch.cuda.synchronize()
            worst = {"O": 0.0, "dQ": 0.0, "dK": 0.0, "dV": 0.0}
            for (b, h), rs in ref.items():
                for name, got, r in zip(("O", "dQ", "dK", "dV"), (o, dq, dk, dv), rs):
                    gnp = got[b:b + 1, h:h + 1].float().cpu().numpy()
                    worst[name] = max(worst[name], float(np.linalg.norm(gnp - r) / np.linalg.norm(r)))
            rec["rel_l2_vs_oracle_2_heads"] = {kk: float("%.3e" % vv) for kk, vv in worst.items()}
        out[mode] = rec
        del fplan, bplan, o, lse
    # top level: the mode that meets the stated tolerance (rel-L2 1e-3 needs fp32-typed results with bf16 inputs:
    # rounding an exact result to bf16 alone costs 1.7e-3); the bf16-typed mode, which autograd uses, is beside it
    out.update({kk: out["fp32_results"][kk] for kk in ("fwd_ms", "fwd_tflops", "bwd_ms", "bwd_tflops", "frac_mfma_peak")})
    out["top_level_mode"] = "fp32_results"
    return out


def config_line(torch, dev, fm, name, N_, keeps, causal, seed, dense_mask_paths, reps=20):
    """One BASELINE configuration at B=1 H=1 D=64 fp16: per kept ratio the kernel time (lists ready), the time
    from a block mask on the device (lists built inside the call), optionally the time from a dense N x N
    tile-constant bool mask (reduced to the block mask, or taken as an elementwise mask), and the parity of
    sampled row blocks against the oracle."""
    import numpy as np
    from fa2_custom_mask import utils
    from oracle import c_oracle
    nb_ = N_ // TILE
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(1, 1, N_, D, generator=g).to(torch.float16) for _ in range(3)]
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    sc = 1.0 / D ** 0.5
    out = {"workload": name, "keeps": {}}
    for r in keeps:
        m = (torch.rand(1, 1, nb_, nb_, generator=g) < r) | torch.eye(nb_, dtype=torch.bool)
        if causal:
            m = m & torch.tril(torch.ones(nb_, nb_, dtype=torch.bool))
        md = m.to(dev)
        lists = fm.block_mask_to_lists(md)
        kept = int(lists.counts[1])
        plan = fm.ForwardPlan(qd, kd, vd, lists, sc)
        tk = event_times(plan.run, reps, 3, torch)

        def from_block():
            utils.lists_cache.clear()
            return fm.flash_attention_custom_mask(qd, kd, vd, md, sc)
        tb = event_times(from_block, reps, 3, torch)
        med = tk[len(tk) // 2]
        rec = {"kept_tiles": kept, "kernel_ms": round(med, 5),
               "tflops_on_kept_tiles": round(tile_flops(kept) / med / 1e9, 1),
               "frac_mfma_peak": round(tile_flops(kept) / med / 1e9 / PEAK_F16_TFLOPS, 4),
               "from_block_mask_ms": round(tb[len(tb) // 2], 5)}
        if dense_mask_paths:
            dense = md.repeat_interleave(TILE, 2).repeat_interleave(TILE, 3).contiguous()

            def from_dense_reduced():
                utils.lists_cache.clear()
                return fm.flash_attention_custom_mask(qd, kd, vd, fm.reduce_dense_mask(dense), sc)

            def from_dense_elementwise():
                utils.lists_cache.clear()
                return fm.flash_attention_custom_mask(qd, kd, vd, dense, sc)
            t1 = event_times(from_dense_reduced, reps, 3, torch)
            t2 = event_times(from_dense_elementwise, reps, 3, torch)
            rec["from_dense_mask_reduced_ms"] = round(t1[len(t1) // 2], 5)
            rec["from_dense_mask_elementwise_ms"] = round(t2[len(t2) // 2], 5)
            del dense
        o = plan.run()[0]
        torch.cuda.synchronize()
        worst = 0.0
        for rb in sorted({0, nb_ // 2, nb_ - 1}):
            o_ref, _ = c_oracle.naive_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(), m.numpy(), sc,
                                          rb * TILE, rb * TILE + TILE)
            worst = max(worst, float(np.abs(o[0, 0, rb * TILE:(rb + 1) * TILE].float().cpu().numpy()
                                            - o_ref[0, 0, rb * TILE:(rb + 1) * TILE]).max()))
        rec["max_abs_vs_oracle_sampled_rows"] = worst
        out["keeps"][str(r)] = rec
        del plan, lists
    return out


def elementwise_case(torch, dev, fm, q, k, v, sm_scale):
    """Token-level causal mask [1,1,N,N] at the headline shape: every diagonal tile is partly set.
    Forward time with the packed mask words applied, and the time of the elementwise preprocessing
    (reduce + lists + pack of the 307.5 MB mask), also in the form a call with a backward uses (one pass over
    the mask for the block mask and the packed words of every tile, then row and column lists)."""
    from fa2_custom_mask import utils
    mask = torch.ones(N, N, dtype=torch.bool, device=dev).tril_().reshape(1, 1, N, N)
    lists = utils.mask_to_lists(mask, N)
    tiles = int(lists.counts[1])
    o, _ = fm.fa2_custom_mask._forward(q, k, v, lists, sm_scale, torch.float16, True)
    tf = event_times(lambda: fm.fa2_custom_mask._forward(q, k, v, lists, sm_scale, torch.float16, False), 20, 3, torch)

    def prep():
        utils.lists_cache.clear()
        utils.mask_to_lists(mask, N)
    tp = event_times(prep, 10, 2, torch)

    def prep_both():   # what a call with a backward does: one pass over the mask, then both list orientations
        utils.lists_cache.clear()
        utils.grid_cache.clear()
        utils.mask_to_lists(mask, N, both=True)
        utils.mask_to_lists(mask, N, transpose=True)
    tpb = event_times(prep_both, 10, 2, torch)
    # pack_tiles_kernel alone: the 64 x 64 bytes of every kept tile in, 512 bytes of words and a flag byte out
    tk = event_times(lambda: utils.pack_mask_tiles(mask, lists), 20, 3, torch)
    mk = tk[len(tk) // 2]
    pack_bytes = tiles * (4096 + 513)
    # parity spot check against torch on the first 128 and last 64 queries
    rows = torch.cat([torch.arange(128), torch.arange(N - 64, N)]).to(dev)
    s = (q[0, 0, rows].float() @ k[0, 0].float().T) * sm_scale
    s = s.masked_fill(~mask[0, 0, rows], float("-inf"))
    ref = torch.softmax(s, -1) @ v[0, 0].float()
    err = float((o[0, 0, rows].float() - ref).abs().max())
    mf = tf[len(tf) // 2]
    return {"workload": "token-level causal mask, N=17536 D=64 fp16", "kept_tiles": tiles,
            "fwd_ms": round(mf, 5), "fwd_tflops_on_kept_tiles": round(tile_flops(tiles) / mf / 1e9, 1),
            "preprocess_ms": round(tp[len(tp) // 2], 5),
            "preprocess_for_backward_ms": round(tpb[len(tpb) // 2], 5),
            "pack_tiles": {"ms": round(mk, 5), "bytes": pack_bytes, "GBps": round(pack_bytes / mk / 1e6, 1),
                           "frac_hbm_peak": round(pack_bytes / mk / 1e6 / PEAK_HBM_GBS, 4),
                           "what": "bsattn_pack_mask_tiles over all kept tiles by their row lists, host wrapper included"},
            "max_abs_vs_torch_fp32": err}


def reorder_case(torch, dev, fm):
    """Head-wise token reorder and its inverse (the step either side of attention in the caller) at the
    reference's default video shape, functional.py:22: F, H, W = 13, 30, 45 (17 550 tokens), 48 heads of
    64 fp16 values.  HBM bound: bytes = read + write of the tensor."""
    F, H, W, heads, D = 13, 30, 45, 48, 64
    g = torch.Generator().manual_seed(SEED + 9)
    x = torch.randn(1, heads, F * H * W, D, generator=g).to(torch.float16).to(dev)
    perms = torch.tensor([[0, 1, 2], [0, 2, 1], [1, 2, 0], [1, 0, 2], [2, 1, 0], [2, 0, 1]], dtype=torch.int32)
    invs = torch.tensor([[0, 1, 2], [0, 2, 1], [2, 0, 1], [1, 0, 2], [2, 1, 0], [1, 2, 0]], dtype=torch.int32)
    idx = torch.arange(heads) % 6
    orders, inv_orders = perms[idx].to(dev), invs[idx].to(dev)
    y = fm.apply_head_wise_reorder(x, orders, F, H, W)
    back = fm.apply_inv_reorder(y, orders, inv_orders, F, H, W)
    ok = bool(torch.equal(back, x))
    # closed form of one head: view as (F, H, W), permute, flatten (permute.py:45-58)
    hd = 5
    ref = x[0, hd].view(F, H, W, D).permute(*perms[idx[hd]].tolist(), 3).reshape(F * H * W, D)
    ok = ok and bool(torch.equal(y[0, hd], ref))
    tf = event_times(lambda: fm.apply_head_wise_reorder(x, orders, F, H, W), 20, 3, torch)
    ti = event_times(lambda: fm.apply_inv_reorder(y, orders, inv_orders, F, H, W), 20, 3, torch)
    nbytes = 2.0 * x.numel() * x.element_size()
    mf, mi = tf[len(tf) // 2], ti[len(ti) // 2]
    return {"workload": "reorder + inverse, 1 x 48 heads x 17550 tokens x 64 fp16 (F,H,W = 13,30,45)",
            "bytes": nbytes, "reorder_ms": round(mf, 5), "inverse_ms": round(mi, 5),
            "reorder_GBps": round(nbytes / mf / 1e6, 1), "inverse_GBps": round(nbytes / mi / 1e6, 1),
            "frac_hbm_peak": round(nbytes / mf / 1e6 / PEAK_HBM_GBS, 4), "bit_exact_round_trip_and_closed_form": ok,
            "note": "times include the output allocation of the host wrapper"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-keep", type=float, default=None,
                    help="profiling aid: run only forward passes at this kept-tile ratio and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="profiling aid: run a plain 256 MiB device copy a few times and exit "
                         "(reference reading for the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--fwd-bwd", action="store_true",
                    help="measurement aid: forward and backward at BASELINE configs[4] (B=2 H=16 N=8192 D=128 bf16, "
                         "block-causal mask with keep 0.25 shared by all heads), then exit")
    ap.add_argument("--lists-per-row", type=int, default=0,
                    help="with --fwd-bwd: a mask with exactly this many kept tiles in every row and column "
                         "instead of the block-causal one")
    ap.add_argument("--reorder", action="store_true",
                    help="measurement aid: the head-wise token reorder and its inverse, then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (heads / row blocks shard without "
              "communication; no multi-GPU figure is produced). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import fa2_custom_mask as fm
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": 256 << 20, "copies": 5}))
        return
    if args.reorder:
        print(json.dumps(reorder_case(torch, dev, fm)))
        return
    if args.fwd_bwd:
        print(json.dumps(fwd_bwd_c5(torch, dev, fm, min(args.steps, 50), min(args.warmup, 5),
                                    check=not args.no_cpu and not args.lists_per_row, uniform=args.lists_per_row)))
        return
    g = torch.Generator().manual_seed(SEED)
    q, k, v = [torch.randn(1, 1, N, D, generator=g).to(torch.float16) for _ in range(3)]
    masks = {}
    for r in KEEPS:
        m = torch.rand(1, 1, NB, NB, generator=g) < r
        masks[r] = m | torch.eye(NB, dtype=torch.bool)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    sm_scale = 1.0 / np.sqrt(D)

    lists = {r: fm.block_mask_to_lists(masks[r].to(dev)) for r in KEEPS}
    kept = {r: int(lists[r].counts[1]) for r in KEEPS}

    plans = {r: fm.ForwardPlan(qd, kd, vd, lists[r], sm_scale) for r in KEEPS}

    def fwd(r):
        return plans[r].run()

    if args.only_keep is not None:
        # the protocol of the timed regions below: warm-up, the untimed run-in, then the launches that count; a
        # kernel trace of this command is dominated by launches at the settled clock (the run-in alone is about
        # a thousand launches at keep 1.0), and the last `steps` launches of the trace are the timed ones
        for _ in range(args.warmup):
            fwd(args.only_keep)
        settle(lambda: fwd(args.only_keep), torch)
        ts = event_times(lambda: fwd(args.only_keep), args.steps, 0, torch)
        print(json.dumps({"only_keep": args.only_keep, "kept_tiles": kept[args.only_keep],
                          "timed_launches": args.steps, "ms_avg": round(sum(ts) / len(ts), 5),
                          "ms_median": round(ts[len(ts) // 2], 5)}))
        return

    # ---- headline: K timed steps at keep 1.0 ----
    for _ in range(args.warmup):
        fwd(1.0)
    settle(lambda: fwd(1.0), torch)
    torch.cuda.synchronize()
    region = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    t0 = time.perf_counter()
    region[0].record()          # HIP events on the stream of the launches, around the timed region
    for _ in range(args.steps):
        fwd(1.0)
    region[1].record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    region_ms_per_launch = region[0].elapsed_time(region[1]) / args.steps
    value = tile_flops(kept[1.0]) / (ms_per_step * 1e-3) / 1e12

    # ---- per-launch device time (HIP events on the launch stream), sweep of kept ratios ----
    sweep = {}
    for r in KEEPS:
        ts = event_times(lambda: fwd(r), min(200, max(20, args.steps)), 5, torch)
        avg, med = sum(ts) / len(ts), ts[len(ts) // 2]
        sweep[str(r)] = {"kept_tiles": kept[r], "ms_avg": round(avg, 5), "ms_median": round(med, 5),
                         "tflops": round(tile_flops(kept[r]) / (med * 1e-3) / 1e12, 2),
                         "frac_mfma_peak": round(tile_flops(kept[r]) / (med * 1e-3) / 1e12 / PEAK_F16_TFLOPS, 4)}
    # roofline: the kernel's average duration over the timed region (one launch per step, the launches in stream
    # order, so the region's device time / steps bounds the average dispatch from above; an event pair around a
    # single launch reads 2-3 us more than the dispatch lasts, the sweep above keeps those figures)
    dense_avg_ms = region_ms_per_launch
    achieved = tile_flops(kept[1.0]) / (dense_avg_ms * 1e-3) / 1e12
    ratio = sweep["0.1"]["ms_median"] / sweep["1.0"]["ms_median"]

    # ---- the same sweep with the reference script's 8 heads (kernel-test.py:7: HEADS = 8), as context ----
    g8 = torch.Generator().manual_seed(SEED + 1)
    q8, k8, v8 = [torch.randn(1, 8, N, D, generator=g8).to(torch.float16).to(dev) for _ in range(3)]
    sweep8 = {}
    for r in KEEPS:
        plan8 = fm.ForwardPlan(q8, k8, v8, lists[r], sm_scale)        # the mask is shared by the heads
        ts = event_times(plan8.run, 20, 3, torch)
        med = ts[len(ts) // 2]
        sweep8[str(r)] = {"kept_tiles": 8 * kept[r], "ms_median": round(med, 5),
                          "tflops": round(8 * tile_flops(kept[r]) / (med * 1e-3) / 1e12, 2),
                          "frac_mfma_peak": round(8 * tile_flops(kept[r]) / (med * 1e-3) / 1e12 / PEAK_F16_TFLOPS, 4)}
        del plan8
    sweep8["keep0.1_over_keep1.0_time"] = round(sweep8["0.1"]["ms_median"] / sweep8["1.0"]["ms_median"], 4)
    del q8, k8, v8

    # ---- the same launch on all-zero inputs: same instructions, least switching activity ----
    zq = torch.zeros_like(qd)
    plan_z = fm.ForwardPlan(zq, zq, zq, lists[1.0], sm_scale)
    ts_z = event_times(plan_z.run, 50, 5, torch)
    ts_r = event_times(lambda: fwd(1.0), 50, 5, torch)
    data_dependence = {"dense_ms_median_randn_inputs": round(ts_r[len(ts_r) // 2], 5),
                       "dense_ms_median_zero_inputs": round(ts_z[len(ts_z) // 2], 5),
                       "note": "the sustained clock follows the power drawn, which follows the operand data"}
    del plan_z, zq

    # ---- mask preprocessing: dense N x N bool -> block mask -> lists (HBM bound) ----
    dense_mask = masks[0.1].to(dev).repeat_interleave(TILE, 2).repeat_interleave(TILE, 3)
    ts = event_times(lambda: fm.block_mask_to_lists(fm.reduce_dense_mask(dense_mask)), 20, 3, torch)
    pre_ms = ts[len(ts) // 2]
    pre_bytes = float(N) * N + 4.0 * (kept[0.1] + 5 * NB)
    block_dev = masks[0.1].to(dev)
    ts_b = event_times(lambda: fm.block_mask_to_lists(block_dev), 20, 3, torch)
    del dense_mask

    # ---- parity spot check against the CPU oracle (first 2 row blocks, keep 0.1) ----
    from oracle import c_oracle
    o_gpu, _ = fwd(0.1)
    o_ref, _ = c_oracle.naive_fwd(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                  masks[0.1].numpy(), sm_scale, 0, 128)
    parity = float(np.abs(o_gpu[0, 0, :128].float().cpu().numpy() - o_ref[0, 0, :128]).max())

    out = {
        "metric": "fwd effective TFLOP/s on kept tiles, N=17536 D=64 fp16, keep 1.0 (kernel only)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: fwd B=1 H=1 N=17536 D=64 fp16, 274x274 tiles, keep 1.0",
                   "kept_tiles": kept[1.0], "seed": SEED,
                   "run_in_s": SETTLE_S},     # untimed launches after the warm-up steps, before the timed ones (clock settled)
        "sweep": sweep,
        "keep0.1_over_keep1.0_time": round(ratio, 4),
        "sweep_8_heads": sweep8,
        "mask_preprocess": {"dense_NxN_ms": round(pre_ms, 5), "dense_GBps": round(pre_bytes / (pre_ms * 1e-3) / 1e9, 1),
                            "frac_hbm_peak": round(pre_bytes / (pre_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                            "block_mask_ms": round(ts_b[len(ts_b) // 2], 5)},
        "parity_max_abs_vs_oracle": parity,
        "data_dependence": data_dependence,
        "configs0": config_line(torch, dev, fm, "BASELINE configs[0]: fwd B=1 H=1 N=1024 D=64 fp16, keep 0.5 + diagonal",
                                1024, [0.5], False, 1234, False),
        "configs1": config_line(torch, dev, fm, "BASELINE configs[1]: fwd B=1 H=1 N=6400 D=64 fp16, keep 0.1 / 1.0, "
                                "preprocessing from a dense tile-constant N x N bool mask included",
                                6400, [0.1, 1.0], False, 1235, True),
        "configs3": config_line(torch, dev, fm, "BASELINE configs[3]: fwd B=1 H=1 N=32000 D=64 fp16, block-causal x "
                                "Bernoulli keep 0.1 / 1.0 + diagonal", 32000, [0.1, 1.0], True, 1237, False, reps=10),
        "fwd_bwd_configs4": fwd_bwd_c5(torch, dev, fm, 20, 3, check=not args.no_cpu),
        "elementwise_mask": elementwise_case(torch, dev, fm, qd, kd, vd, sm_scale),
        "token_reorder": reorder_case(torch, dev, fm),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_F16_TFLOPS, 4), "traffic": measured_traffic(),
                     "ms_per_launch": round(dense_avg_ms, 5), "ms_single_launch_between_events": sweep["1.0"]["ms_avg"],
                     "kernel": "fwd_kernel<64, 0, false, false, true> (fp16, contiguous rows, one bsattn_fwd call)",
                     "algorithmic_flops_per_launch": tile_flops(kept[1.0])},
    }
    if not args.no_cpu:
        # CPU baseline: the oracle's C port of the naive path on all host threads, the whole
        # keep-1.0 workload (every query row, every key), median of 3 passes after a short warm-up,
        # reported in the metric's unit.
        qf, kf, vf = q.float().numpy(), k.float().numpy(), v.float().numpy()
        c_oracle.naive_fwd(qf, kf, vf, masks[1.0].numpy(), sm_scale, 0, 256)
        dts = []
        for _ in range(3):
            t0 = time.perf_counter()
            c_oracle.naive_fwd(qf, kf, vf, masks[1.0].numpy(), sm_scale, 0, N)
            dts.append(time.perf_counter() - t0)
        dt = sorted(dts)[1]
        out["cpu_baseline"] = {"value": round(4.0 * N * N * D / dt / 1e12, 5), "unit": "TFLOP/s",
                               "cores": c_oracle.num_threads(), "kind": "port",
                               "sample": "whole workload (%d query rows x %d keys, keep 1.0), fp32 naive masked "
                                         "softmax, oracle C port with OpenMP, median of 3 passes, %.2f s per pass"
                                         % (N, N, dt)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
