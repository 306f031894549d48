"""Pins the oracle's token reorder (CPU only) against the torch view/permute closed form."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from oracle import c_oracle


def closed_form(x, orders, F, H, W):
    """Per head: x.view(F,H,W,D).permute(p0,p1,p2,3).reshape(T,D) (== permute.py:45-58)."""
    x = torch.as_tensor(x)
    BS, NH, T, D = x.shape
    out = torch.empty_like(x)
    for hd in range(NH):
        p = [int(v) for v in orders[hd]]
        out[:, hd] = x[:, hd].view(BS, F, H, W, D).permute(0, 1 + p[0], 1 + p[1], 1 + p[2], 4).reshape(BS, T, D)
    return out.numpy()


@pytest.mark.parametrize("F,H,W", [(2, 3, 4), (3, 5, 2), (1, 4, 4), (13, 6, 5)])
def test_reorder_all_permutations(F, H, W):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 6, F * H * W, 8)).astype(np.float32)
    orders = orc.PERMUTATIONS                       # one head per permutation, functional.py:23-26
    ref = closed_form(x, orders, F, H, W)
    for impl in (orc.reorder, c_oracle.reorder):
        assert np.array_equal(impl(x, orders, F, H, W), ref)


@pytest.mark.parametrize("F,H,W", [(2, 3, 4), (3, 5, 2), (13, 6, 5)])
def test_inverse_roundtrip(F, H, W):
    """inv_reorder with the inverse table (functional.py:69-76) undoes reorder exactly."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 6, F * H * W, 4)).astype(np.float16)
    y = orc.reorder(x, orc.PERMUTATIONS, F, H, W)
    for impl in (orc.inv_reorder, c_oracle.inv_reorder):
        assert np.array_equal(impl(y, orc.PERMUTATIONS, orc.PERMUTATIONS_INV, F, H, W), x)


def test_inverse_table_is_inverse():
    for p, pi in zip(orc.PERMUTATIONS.tolist(), orc.PERMUTATIONS_INV.tolist()):
        assert [p[i] for i in pi] == [0, 1, 2]
