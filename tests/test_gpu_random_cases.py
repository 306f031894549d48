"""Seeded random cases of the whole operator (forward, LSE, gradients) against the CPU oracle: shapes, head
dimensions, dtypes, mask forms (block / elementwise / none, broadcast or per head), sparsity, score scale and
result type are drawn per case.  The naive masked softmax of kernel-test.py:37-40 and its gradient are the bar.

Tolerances.  Forward: max-abs 2e-2 (fp16) / 3e-2 (bf16), rel-L2 1e-3 (3e-3 for bf16-typed results: the cast of an
exact result alone is 1.7e-3).  Gradients at unit score scale: rel-L2 1e-3 for fp16; 3e-3 for bf16 inputs, because O
enters the backward rounded to bf16 (delta = rowsum(O * dO), as in the reference, fa2_bwd.py:17); 4e-3 when the
gradients are bf16-typed as well.  Cases with q scaled by a gain g > 1 (scores of standard deviation g instead of 1)
get g times these bars: the score scale is folded into the fp16 Q, so the rounding of a score grows with its size.
These cases are there to catch gross errors in the re-centring paths, not to set the precision bar."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import errors, f32

pytestmark = pytest.mark.gpu


def draw_case(seed):
    rs = np.random.RandomState(seed)
    D = int(rs.choice([16, 32, 64, 64, 128, 128, 256]))
    dtype = torch.float16 if rs.rand() < 0.5 else torch.bfloat16
    B, H = int(rs.choice([1, 1, 2, 3])), int(rs.choice([1, 2, 4, 8]))
    if rs.rand() < 0.15:
        B, H = 2, int(rs.choice([32, 64]))                       # many heads: whole row blocks per wavefront / pair
    N = int(rs.choice([64, 128, 192, 320, 512, 768, 1024])) if rs.rand() < 0.75 else int(rs.randint(1, 900))
    if B * H >= 64:
        N = min(N, 512)
    form = rs.choice(["block", "block", "elementwise", "none"])
    keep = float(rs.choice([0.05, 0.2, 0.5, 0.9, 1.0]))
    Bm, Hm = (B if rs.rand() < 0.3 else 1), (H if rs.rand() < 0.3 else 1)
    gain = float(rs.choice([1.0, 1.0, 1.0, 4.0, 8.0]))
    out_fp32 = bool(rs.rand() < 0.6)
    return dict(D=D, dtype=dtype, B=B, H=H, N=N, form=form, keep=keep, Bm=Bm, Hm=Hm, gain=gain, out_fp32=out_fp32,
                seed=seed)


def make_mask(c):
    g = torch.Generator().manual_seed(1000 + c["seed"])
    N, nb = c["N"], -(-c["N"] // 64)
    if c["form"] == "none":
        return None, np.ones((1, 1, N, N), dtype=bool)
    if c["form"] == "block":
        m = torch.rand(c["Bm"], c["Hm"], nb, nb, generator=g) < c["keep"]
        if torch.rand(1, generator=g).item() < 0.5:
            m &= torch.tril(torch.ones(nb, nb, dtype=torch.bool))
        if torch.rand(1, generator=g).item() < 0.7:
            m |= torch.eye(nb, dtype=torch.bool)
        return m, orc.expand_block_mask(m.numpy())[..., :N, :N]
    m = torch.rand(c["Bm"], c["Hm"], N, N, generator=g) < c["keep"]
    if torch.rand(1, generator=g).item() < 0.5:
        m &= torch.tril(torch.ones(N, N, dtype=torch.bool))
    if N > 64 and torch.rand(1, generator=g).item() < 0.5:
        m[..., :, :64] &= (torch.arange(N) % 2 == 1).reshape(N, 1)   # every other query: nothing in the first tile
    return m, m.numpy()


@pytest.mark.parametrize("seed", range(48))
def test_random_case(dev, seed):
    import fa2_custom_mask as fm
    c = draw_case(seed)
    B, H, N, D, dtype = c["B"], c["H"], c["N"], c["D"], c["dtype"]
    g = torch.Generator().manual_seed(2000 + seed)
    q, k, v, do = [torch.randn(B, H, N, D, generator=g).to(dtype) for _ in range(4)]
    q = (q.float() * c["gain"]).to(dtype)
    sc = 1.0 / np.sqrt(D)
    mask, mask_np = make_mask(c)
    print({k_: (str(v_) if k_ == "dtype" else v_) for k_, v_ in c.items()}, flush=True)
    res = fm.attention_forward_backward(q.to(dev), k.to(dev), v.to(dev), None if mask is None else mask.to(dev), sc,
                                        do.to(dev), out_fp32=c["out_fp32"])
    torch.cuda.synchronize()
    # oracle on at most 4 heads (the first two and the last two of the flattened batch x head axis)
    flat = sorted(set([0, 1, B * H - 2, B * H - 1]) & set(range(B * H)))
    gain = max(1.0, c["gain"])
    typed16 = not c["out_fp32"]
    o_rel = (3e-3 if (dtype == torch.bfloat16 and typed16) else 1e-3) * gain
    g_rel = (1e-3 if dtype == torch.float16 else (4e-3 if typed16 else 3e-3)) * gain
    o_abs = 2e-2 if dtype == torch.float16 else 3e-2
    g_abs = o_abs * gain * 1.5
    for i in flat:
        b, h = divmod(i, H)
        mb = mask_np[b if mask_np.shape[0] > 1 else 0, h if mask_np.shape[1] > 1 else 0][None, None]
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_r, lse_r = orc.naive_attention(f32(q[sl]), f32(k[sl]), f32(v[sl]), mb, sc, return_lse=True)
        grads = orc.attention_backward(f32(q[sl]), f32(k[sl]), f32(v[sl]), mb, sc, f32(do[sl]))
        fin = np.isfinite(lse_r)
        lse = res[1][sl].cpu().numpy()
        assert np.array_equal(np.isfinite(lse), fin)
        assert np.abs(lse[fin] - lse_r[fin]).max(initial=0.0) <= 2e-3 * max(1.0, c["gain"])
        for name, got, ref in (("o", res[0], o_r), ("dq", res[2], grads[0]), ("dk", res[3], grads[1]), ("dv", res[4], grads[2])):
            ma, rl = errors(got[sl], ref)
            assert np.isfinite(f32(got[sl])).all(), name
            abs_bar, rel_bar = (o_abs, o_rel) if name == "o" else (g_abs, g_rel)
            assert ma <= abs_bar and (rl <= rel_bar or ma <= 1e-5), (name, i, ma, rl)   # (a zero result has no relative error)
