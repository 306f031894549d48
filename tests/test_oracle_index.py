"""Pins the oracle's index builder (CPU only): hand-worked fixture, the torch.nonzero/cumsum
closed form, structural invariants and special masks."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from oracle import c_oracle

HERE = os.path.dirname(os.path.abspath(__file__))
IMPLS = [orc.build_groups_from_block_mask, c_oracle.build_groups]


def closed_form(mask):
    """torch.nonzero is row-major, i.e. lexicographic in (b,h,m,n)."""
    mask = torch.as_tensor(mask)
    nz = torch.nonzero(mask)
    if nz.numel() == 0:
        return None, None
    cnt = mask.sum(-1).flatten()
    start = torch.cumsum(cnt, 0) - cnt
    B, H, nb, _ = mask.shape
    idx = torch.nonzero(cnt > 0).flatten()
    b, h, m = idx // (H * nb), (idx // nb) % H, idx % nb
    groups = torch.stack([b, h, m, start[idx], cnt[idx]], 1).to(torch.int32)
    return groups.numpy(), nz[:, 3].to(torch.int32).numpy()


@pytest.mark.parametrize("impl", IMPLS)
def test_fixture(impl):
    fx = json.load(open(os.path.join(HERE, "golden", "groups_fixture.json")))
    g, n = impl(np.array(fx["mask"], dtype=bool))
    assert g.dtype == np.int32 and n.dtype == np.int32
    assert g.tolist() == fx["groups"] and n.tolist() == fx["n_list"]


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("seed", range(40))
def test_random_vs_closed_form_and_invariants(impl, seed):
    rng = np.random.default_rng(seed)
    B, H, nb = rng.integers(1, 4), rng.integers(1, 4), rng.integers(1, 20)
    mask = rng.random((B, H, nb, nb)) < rng.choice([0.05, 0.3, 0.7])
    g, n = impl(mask)
    g_ref, n_ref = closed_form(mask)
    if g_ref is None:
        assert g is None and n is None
        return
    assert np.array_equal(g, g_ref) and np.array_equal(n, n_ref)
    assert np.array_equal(g[:, 3], np.cumsum(g[:, 4]) - g[:, 4])          # start = exclusive cumsum
    assert g[:, 4].sum() == len(n) == mask.sum() and (g[:, 4] > 0).all()
    keys = [tuple(r[:3]) for r in g.tolist()]
    assert keys == sorted(set(keys))                                       # strictly lexicographic
    for b, h, m, s, l in g.tolist():
        seg = n[s:s + l]
        assert (np.diff(seg) > 0).all() and mask[b, h, m, seg].all()


@pytest.mark.parametrize("impl", IMPLS)
def test_special_masks(impl):
    nb = 7
    assert impl(np.zeros((2, 2, nb, nb), dtype=bool)) == (None, None)       # fa2_custom_mask.py:34-35
    g, n = impl(np.ones((1, 1, nb, nb), dtype=bool))
    assert np.array_equal(n, np.tile(np.arange(nb), nb)) and (g[:, 4] == nb).all()
    g, n = impl(np.eye(nb, dtype=bool)[None, None])
    assert np.array_equal(n, np.arange(nb)) and np.array_equal(g[:, 2], np.arange(nb))
    g, n = impl(np.tril(np.ones((nb, nb), dtype=bool))[None, None])
    assert np.array_equal(g[:, 4], np.arange(1, nb + 1))


def test_csr_csc_forms():
    rng = np.random.default_rng(3)
    mask = rng.random((2, 3, 9, 9)) < 0.3
    rp, ci = orc.csr_from_block_mask(mask)
    g, n = orc.build_groups_from_block_mask(mask)
    assert np.array_equal(ci, n) and rp[-1] == len(n)
    nonempty = np.nonzero(np.diff(rp))[0]
    assert np.array_equal(rp[nonempty], g[:, 3])
    rpt, cit = orc.csc_from_block_mask(mask)
    for b in range(2):
        for h in range(3):
            for c in range(9):
                r = (b * 3 + h) * 9 + c
                assert np.array_equal(cit[rpt[r]:rpt[r + 1]], np.nonzero(mask[b, h, :, c])[0])


def test_dense_reduce_and_expand_roundtrip():
    rng = np.random.default_rng(5)
    block = rng.random((1, 2, 5, 5)) < 0.4
    dense = orc.expand_block_mask(block)
    ref = torch.as_tensor(block).repeat_interleave(64, 2).repeat_interleave(64, 3).numpy()   # kernel-test.py:18
    assert np.array_equal(dense, ref)
    assert np.array_equal(orc.reduce_dense_mask(dense), block)
    d = np.zeros((1, 1, 128, 128), dtype=bool); d[0, 0, 70, 3] = True
    assert orc.reduce_dense_mask(d).tolist() == [[[[False, False], [True, False]]]]


def test_pack_mask_tiles_format():
    """Packed-tile format: one slot per kept tile in list order; word r bit c = element (r, c);
    the transposed form lists tiles column block by column block with rows and columns swapped.
    Checked by unpacking against the mask itself and against the kept-tile lists."""
    rng = np.random.default_rng(3)
    N, nb = 192, 3
    dense = rng.random((1, 2, N, N)) < 0.4
    dense[0, 0, :64, 64:128] = False                    # empty tile
    dense[0, 0, 64:128, :64] = True                     # full tile
    dense[0, 1, 128:, :] = False                        # empty row block
    block = orc.reduce_dense_mask(dense)
    for transpose in (False, True):
        partial, words = orc.pack_mask_tiles(dense, transpose)
        rp, ci = (orc.csc_from_block_mask(block) if transpose else orc.csr_from_block_mask(block))[:2]
        assert len(partial) == len(ci) == words.shape[0]
        t = 0
        for bh in range(2):
            for a in range(nb):
                for j in range(rp[bh * nb + a], rp[bh * nb + a + 1]):
                    c = ci[j]
                    rb, cb = (c, a) if transpose else (a, c)
                    tile = dense[0, bh, rb * 64:(rb + 1) * 64, cb * 64:(cb + 1) * 64]
                    tile = tile.T if transpose else tile
                    unpacked = (words[t][:, None] >> np.arange(64, dtype=np.uint64)[None, :]) & np.uint64(1)
                    assert np.array_equal(unpacked.astype(bool), tile)
                    assert partial[t] == (0 if tile.all() else 1)
                    t += 1
        assert t == len(partial)
