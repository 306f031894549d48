"""GPU parity of the token reorder kernels against the CPU oracle: pure data movement, bit-exact."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("F,H,W,D", [(2, 3, 4, 64), (13, 6, 5, 128), (3, 5, 7, 6)])
def test_reorder_and_inverse(dev, dtype, F, H, W, D):
    import fa2_custom_mask as fm
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 6, F * H * W, D, generator=g).to(dtype)
    orders = torch.tensor(orc.PERMUTATIONS)
    inv = torch.tensor(orc.PERMUTATIONS_INV)
    xn = x.view(torch.int16 if dtype != torch.float32 else torch.int32).numpy()
    y = fm.apply_head_wise_reorder(x.to(dev), orders.to(dev), F, H, W)
    y_ref = orc.reorder(xn, orc.PERMUTATIONS, F, H, W)
    assert np.array_equal(y.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32).numpy(), y_ref)
    z = fm.apply_inv_reorder(y, orders.to(dev), inv.to(dev), F, H, W)
    assert torch.equal(z.cpu(), x)                                   # exact round trip
    z_ref = orc.inv_reorder(y_ref, orc.PERMUTATIONS, orc.PERMUTATIONS_INV, F, H, W)
    assert np.array_equal(z_ref, xn)


def test_permute_qkv_and_inverse_wrappers(dev):
    """permute_qkv_triton / inv_permute_attn_triton: text tokens untouched, image tokens reordered
    per head, in place (functional.py:22-43, 64-84)."""
    import fa2_custom_mask as fm
    F, H, W, n_text, D, NH = 3, 4, 5, 7, 64, 6
    T = n_text + F * H * W
    g = torch.Generator().manual_seed(2)
    q, k, v = [torch.randn(1, NH, T, D, generator=g).half() for _ in range(3)]
    plan = {"permute": [torch.tensor([5, 0, 3, 2, 1, 4])]}
    orders = orc.PERMUTATIONS[plan["permute"][0].numpy()]
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    plan_d = {"permute": [plan["permute"][0].to(dev)]}
    q2, k2, v2 = fm.permute_qkv_triton(qd, kd, vd, plan_d, 0, F=F, H=H, W=W, n_text_tokens=n_text)
    assert q2.data_ptr() == qd.data_ptr()                              # in place
    for got, src in ((q2, q), (k2, k), (v2, v)):
        ref = src.clone().numpy()
        ref[:, :, n_text:] = orc.reorder(src[:, :, n_text:].numpy(), orders, F, H, W)
        assert np.array_equal(got.cpu().numpy(), ref)
    back = fm.inv_permute_attn_triton(q2, plan_d, 0, F=F, H=H, W=W, n_text_tokens=n_text)
    assert torch.equal(back.cpu(), q)


def test_default_geometry(dev):
    """The reference's defaults F=13, H=30, W=45, n_text_tokens=226 (functional.py:22)."""
    import fa2_custom_mask as fm
    NH, D = 2, 64
    T = 226 + 13 * 30 * 45
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, NH, T, D, generator=g).half()
    plan = {"permute": [torch.tensor([2, 4], device=dev)]}
    xd = x.to(dev)
    a, b_, c = fm.permute_qkv_triton(xd.clone(), xd.clone(), xd.clone(), plan, 0)
    orders = orc.PERMUTATIONS[[2, 4]]
    ref = x.clone().numpy()
    ref[:, :, 226:] = orc.reorder(x[:, :, 226:].numpy(), orders, 13, 30, 45)
    assert np.array_equal(a.cpu().numpy(), ref) and torch.equal(a, b_) and torch.equal(a, c)
    assert torch.equal(fm.inv_permute_attn_triton(a, plan, 0).cpu(), x)
