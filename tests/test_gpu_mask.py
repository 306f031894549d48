"""GPU parity of the mask preprocessing kernels against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import uniform_block_mask, causal_block_mask

pytestmark = pytest.mark.gpu


def _check_lists(mask_cpu, dev):
    import fa2_custom_mask as fm
    g_ref, n_ref = orc.build_groups_from_block_mask(mask_cpu.numpy())
    g, n = fm.build_groups_from_block_mask(mask_cpu.to(dev))
    if g_ref is None:
        assert g is None and n is None
        return
    assert g.dtype == torch.int32 and n.dtype == torch.int32 and g.is_contiguous() and n.is_contiguous()
    assert g.device.type == "cuda" and tuple(g.shape) == g_ref.shape and tuple(n.shape) == n_ref.shape
    assert np.array_equal(g.cpu().numpy(), g_ref)
    assert np.array_equal(n.cpu().numpy(), n_ref)


@pytest.mark.parametrize("shape,keep", [((1, 1, 16, 16), 0.5), ((1, 2, 3, 3), 0.4), ((2, 3, 37, 37), 0.1),
                                        ((1, 1, 100, 100), 0.1), ((1, 1, 100, 100), 1.0),
                                        ((1, 1, 274, 274), 0.05), ((2, 16, 128, 128), 0.25),
                                        ((1, 1, 500, 500), 0.1), ((1, 1, 65, 65), 0.9), ((3, 5, 1, 1), 0.5),
                                        # either side of the limits of the one-workgroup count and scan
                                        # (1023 rows, 256 KB of block mask)
                                        ((1, 1, 512, 512), 0.5), ((1, 1, 513, 513), 0.5), ((1, 1023, 1, 1), 0.5),
                                        ((1, 1024, 1, 1), 0.5), ((1, 31, 33, 33), 0.3), ((1, 32, 32, 32), 0.3),
                                        ((1, 1, 512, 512), 1.0), ((2, 2, 255, 255), 0.02),
                                        # either side of the size up to which the same workgroup also fills the
                                        # lists (16384 tiles): full, sparse, several heads, an odd row length
                                        ((1, 1, 128, 128), 1.0), ((1, 1, 128, 128), 0.03), ((1, 1, 129, 129), 0.5),
                                        ((2, 2, 64, 64), 0.5), ((1, 4, 64, 64), 1.0), ((1, 3, 73, 73), 0.2),
                                        ((1, 1, 127, 127), 0.97), ((1, 7, 5, 5), 0.5)])
def test_groups_random(dev, shape, keep):
    g = torch.Generator().manual_seed(7)
    _check_lists(torch.rand(*shape, generator=g) < keep, dev)


def test_groups_fixture_and_special(dev):
    m = torch.tensor([[[[1, 0, 1], [0, 0, 0], [0, 1, 1]], [[0, 0, 0], [1, 1, 1], [0, 0, 1]]]], dtype=torch.bool)
    _check_lists(m, dev)
    _check_lists(torch.zeros(2, 2, 5, 5, dtype=torch.bool), dev)            # (None, None)
    _check_lists(torch.ones(1, 2, 70, 70, dtype=torch.bool), dev)           # dense
    _check_lists(torch.eye(130, dtype=torch.bool)[None, None], dev)         # identity
    _check_lists(torch.tril(torch.ones(129, 129, dtype=torch.bool))[None, None], dev)
    _check_lists(causal_block_mask(1, 1, 500, 0.1, 3), dev)


def test_strided_and_broadcast_masks(dev):
    import fa2_custom_mask as fm
    base = uniform_block_mask(2, 4, 40, 0.3, 11)
    view = base.to(dev)[:, ::2, 4:36, 4:36]                                  # non-contiguous view
    g_ref, n_ref = orc.build_groups_from_block_mask(base[:, ::2, 4:36, 4:36].numpy())
    g, n = fm.build_groups_from_block_mask(view)
    assert np.array_equal(g.cpu().numpy(), g_ref) and np.array_equal(n.cpu().numpy(), n_ref)
    exp = base[:1, :1].expand(2, 4, 40, 40)                                  # stride-0 broadcast
    g_ref, n_ref = orc.build_groups_from_block_mask(exp.numpy())
    g, n = fm.build_groups_from_block_mask(base[:1, :1].to(dev).expand(2, 4, 40, 40))
    assert np.array_equal(g.cpu().numpy(), g_ref) and np.array_equal(n.cpu().numpy(), n_ref)


def test_transposed_lists(dev):
    import fa2_custom_mask as fm
    m = uniform_block_mask(2, 2, 33, 0.3, 5)
    rp_ref, ci_ref = orc.csc_from_block_mask(m.numpy())
    lists = fm.block_mask_to_lists(m.to(dev), transpose=True)
    T = int(lists.counts[1])
    assert np.array_equal(lists.row_ptr.cpu().numpy(), rp_ref)
    assert np.array_equal(lists.col_idx[:T].cpu().numpy(), ci_ref)


@pytest.mark.parametrize("N,keep", [(1024, 0.5), (6400, 0.1), (6400, 1.0), (4160, 0.3)])
def test_dense_mask_equals_block_mask(dev, N, keep):
    import fa2_custom_mask as fm
    nb = N // 64
    block = uniform_block_mask(1, 1, nb, keep, 21)
    dense = block.to(dev).repeat_interleave(64, 2).repeat_interleave(64, 3)   # kernel-test.py:18
    red = fm.reduce_dense_mask(dense)
    assert red.dtype == torch.bool and torch.equal(red.cpu(), block)
    g_ref, n_ref = orc.build_groups_from_block_mask(block.numpy())
    g, n = fm.build_groups_from_block_mask(red)
    assert np.array_equal(g.cpu().numpy(), g_ref) and np.array_equal(n.cpu().numpy(), n_ref)


def test_dense_mask_partial_tiles(dev):
    """A tile is kept iff any element in it is set: single set elements at tile corners."""
    import fa2_custom_mask as fm
    N = 640
    dense = torch.zeros(2, 1, N, N, dtype=torch.bool)
    pts = [(0, 0), (63, 63), (64, 127), (639, 0), (320, 325), (100, 639)]
    for r, c in pts:
        dense[0, 0, r, c] = True
    dense[1, 0, 5, 77] = True
    red = fm.reduce_dense_mask(dense.to(dev)).cpu().numpy()
    assert np.array_equal(red, orc.reduce_dense_mask(dense.numpy()))
    assert red.sum() == len(pts)          # (0,0) and (63,63) share a tile


@pytest.mark.parametrize("transpose", [False, True])
def test_pack_mask_tiles_bit_exact(dev, transpose):
    """Packed 64 x 64 tile words and partial flags of elementwise masks: bit-exact against the
    oracle, for both list orientations, a shared (broadcast) mask and a non-contiguous view."""
    import fa2_custom_mask as fm
    from fa2_custom_mask import utils
    g = torch.Generator().manual_seed(17)
    for shape, p in (((1, 1, 256, 256), 0.5), ((2, 3, 192, 192), 0.05), ((1, 2, 320, 320), 0.9)):
        dense = torch.rand(shape, generator=g) < p
        dense[0, 0, :64, :64] = True
        dense[0, -1, 64:128, :] = False
        variants = [dense.to(dev)]
        big = torch.zeros(shape[:3] + (shape[3] + 64,), dtype=torch.bool)
        big[..., :shape[3]] = dense
        variants.append(big.to(dev)[..., :shape[3]])                 # padded rows: not contiguous
        for md in variants:
            block = fm.reduce_dense_mask(md)
            lists = fm.block_mask_to_lists(block, transpose=transpose)
            partial, bits = utils.pack_mask_tiles(md, lists, transpose=transpose)
            T = int(lists.counts[1])
            p_ref, w_ref = orc.pack_mask_tiles(dense.numpy(), transpose)
            assert T == len(p_ref)
            assert np.array_equal(partial[:T].cpu().numpy(), p_ref)
            assert np.array_equal(bits[:T].cpu().numpy().view(np.uint64), w_ref)


@pytest.mark.parametrize("transpose", [False, True])
def test_one_pass_words_bit_exact(dev, transpose):
    """The same words made in one pass over the mask (block mask + grid-ordered words, then gathered into list
    order): bit-exact against the oracle and against the two-pass route, for both list orientations, several
    mask heads, sizes that are not a multiple of 1024 columns, and a non-contiguous view."""
    import fa2_custom_mask as fm
    from fa2_custom_mask import utils
    g = torch.Generator().manual_seed(18)
    for shape, p in (((1, 1, 256, 256), 0.5), ((2, 3, 192, 192), 0.05), ((1, 2, 1344, 1344), 0.9), ((1, 1, 2112, 2112), 0.02)):
        dense = torch.rand(shape, generator=g) < p
        dense[0, 0, :64, :64] = True
        dense[0, -1, 64:128, :] = False
        variants = [dense.to(dev)]
        big = torch.zeros(shape[:3] + (shape[3] + 64,), dtype=torch.bool)
        big[..., :shape[3]] = dense
        variants.append(big.to(dev)[..., :shape[3]])                 # padded rows: not contiguous
        for md in variants:
            block, gp, gb = utils.reduce_pack_dense_mask(md)
            assert np.array_equal(block.cpu().numpy(), orc.reduce_dense_mask(dense.numpy()))
            lists = fm.block_mask_to_lists(block, transpose=transpose)
            partial, bits = utils.gather_mask_tiles(gp, gb, lists, transpose=transpose)
            T = int(lists.counts[1])
            p_ref, w_ref = orc.pack_mask_tiles(dense.numpy(), transpose)
            assert T == len(p_ref)
            assert np.array_equal(partial[:T].cpu().numpy(), p_ref)
            assert np.array_equal(bits[:T].cpu().numpy().view(np.uint64), w_ref)
            p2, b2 = utils.pack_mask_tiles(md, lists, transpose=transpose)
            assert torch.equal(p2[:T], partial[:T]) and torch.equal(b2[:T], bits[:T])
