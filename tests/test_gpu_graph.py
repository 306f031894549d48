"""The library calls under HIP graph capture: every entry point only enqueues kernels on the
given stream (no allocation, no synchronisation, no memset nodes), so a captured call can be
replayed.  Each graph is replayed several times, with new inputs written in place and eager work
and synchronisations between the replays, and every replay is checked against the eager result
on the same inputs (a replay repeats the launch parameters of the capture, including the number
that marks a launch's partial results in the forward workspace)."""
import numpy as np
import pytest
import torch

from helpers import make_qkv, uniform_block_mask, causal_block_mask, same_up_to_rounding

pytestmark = pytest.mark.gpu


def replay_and_compare(dev, B, H, N, D, dtype, mask, seed, replays=4):
    import fa2_custom_mask as fm
    sc = 1.0 / np.sqrt(D)
    ins = [x.to(dev) for x in make_qkv(B, H, N, D, dtype, seed, n=4)]
    mask = mask.to(dev)
    eager = fm.attention_forward_backward(ins[0], ins[1], ins[2], mask, sc, ins[3])    # also fills the list cache
    torch.cuda.synchronize()
    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        fm.attention_forward_backward(ins[0], ins[1], ins[2], mask, sc, ins[3])          # warm-up on the capture stream
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = fm.attention_forward_backward(ins[0], ins[1], ins[2], mask, sc, ins[3])
    for r in range(replays):
        if r > 0:     # new inputs, written in place into the tensors the graph reads
            fresh = make_qkv(B, H, N, D, dtype, seed + 100 * r, n=4)
            for dst, src in zip(ins, fresh):
                dst.copy_(src.to(dev))
            eager = fm.attention_forward_backward(ins[0], ins[1], ins[2], mask, sc, ins[3])
            torch.cuda.synchronize()
        for t in captured:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("o", "lse", "dq", "dk", "dv"), captured, eager):
            fin = torch.isfinite(ref)
            assert torch.equal(torch.isfinite(got), fin), (r, name)      # lse = -inf for a query without keys
            # (forward nondeterminism: O may round differently, and the gradients see that O)
            assert same_up_to_rounding(got[fin], ref[fin], rel=2.0 ** -7, abs_=4e-3), (r, name)


def test_replay_d64_rows_shared_between_workgroups(dev):
    """One head, 64 row blocks on 512 workgroups: every row block is finished from published parts."""
    replay_and_compare(dev, 1, 1, 4096, 64, torch.float16, uniform_block_mask(1, 1, 64, 0.6, 3001), 3002)


def test_replay_d128_bf16_many_heads(dev):
    """The wavefront-pair forward, the backward without shared lists."""
    replay_and_compare(dev, 2, 8, 2048, 128, torch.bfloat16, causal_block_mask(1, 1, 32, 0.5, 3003), 3004)


def test_replay_d256_lists_shared(dev):
    """Head dimension 256 with few row blocks: forward and backward parts summed by second kernels."""
    replay_and_compare(dev, 1, 2, 2048, 256, torch.float16, uniform_block_mask(1, 2, 32, 0.5, 3005), 3006, replays=3)


def test_replay_elementwise_mask_ragged_length(dev):
    g = torch.Generator().manual_seed(3007)
    N = 1000
    m = (torch.rand(1, 1, N, N, generator=g) < 0.3) & torch.tril(torch.ones(N, N, dtype=torch.bool))
    m[0, 0, 17, :] = False
    replay_and_compare(dev, 1, 3, N, 64, torch.float16, m, 3008, replays=3)


def test_replay_mask_to_lists(dev):
    """The preprocessing kernels in a graph: the mask is rewritten in place between the replays."""
    import fa2_custom_mask as fm
    from oracle import bsattn_oracle as orc
    nb = 96
    mask = uniform_block_mask(2, 3, nb, 0.3, 3009).to(dev)
    fm.block_mask_to_lists(mask, want_groups=True)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        fm.block_mask_to_lists(mask, want_groups=True)
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lists = fm.block_mask_to_lists(mask, want_groups=True)
    for r in range(4):
        new = uniform_block_mask(2, 3, nb, 0.1 + 0.2 * r, 3010 + r)
        if r == 3:
            new[:] = False
        mask.copy_(new.to(dev))
        graph.replay()
        torch.cuda.synchronize()
        g_ref, n_ref = orc.build_groups_from_block_mask(new.numpy())
        G, T = [int(x) for x in lists.counts.cpu()]
        if g_ref is None:
            assert G == 0 and T == 0
            continue
        assert G == len(g_ref) and T == len(n_ref)
        assert np.array_equal(lists.groups[:G].cpu().numpy(), g_ref)
        assert np.array_equal(lists.col_idx[:T].cpu().numpy(), n_ref)
