"""GPU parity of the forward kernel against the CPU oracle's naive fp32 masked softmax
(kernel-test.py:37-40).  Tolerances: max-abs 2e-2 (fp16) / 3e-2 (bf16), rel-L2 1e-3 (for bf16
the rel-L2 bar applies to the fp32-output mode: rounding an exact result to bf16 is 1.7e-3)."""
import numpy as np
import pytest
import torch

from oracle import bsattn_oracle as orc
from helpers import make_qkv, uniform_block_mask, causal_block_mask, errors, f32, same_up_to_rounding

pytestmark = pytest.mark.gpu

MAXABS = {torch.float16: 2e-2, torch.bfloat16: 3e-2}
RELL2 = 1e-3


def run_case(dev, B, H, N, D, dtype, mask, seed, out_fp32=False, check_lse=True):
    import fa2_custom_mask as fm
    q, k, v = make_qkv(B, H, N, D, dtype, seed)
    sm_scale = 1.0 / np.sqrt(D)
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sm_scale, return_lse=True)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sm_scale,
                                                out_fp32=out_fp32)
    torch.cuda.synchronize()
    assert o.dtype == (torch.float32 if out_fp32 else dtype) and tuple(o.shape) == (B, H, N, D)
    ma, rl = errors(o, o_ref)
    print("B%d H%d N%d D%d %s fp32out=%s: max-abs %.3e rel-L2 %.3e" % (B, H, N, D, dtype, out_fp32, ma, rl))
    assert ma <= MAXABS[dtype]
    if dtype == torch.float16 or out_fp32:
        assert rl <= RELL2
    else:
        assert rl <= 3e-3          # bf16-typed output: the cast alone costs 1.7e-3
    if check_lse:
        fin = np.isfinite(lse_ref)
        l = lse.cpu().numpy()
        assert np.array_equal(np.isfinite(l), fin)
        assert np.abs(l[fin] - lse_ref[fin]).max() <= 2e-3
    return o


def test_c1_config(dev):
    """B=1 H=1 N=1024 D=64, 16x16 tiles kept with p=0.5 + diagonal."""
    run_case(dev, 1, 1, 1024, 64, torch.float16, uniform_block_mask(1, 1, 16, 0.5, 1234), 1234)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_small_shapes(dev, D, dtype):
    run_case(dev, 2, 3, 512, D, dtype, uniform_block_mask(2, 3, 8, 0.4, 5), 17)
    run_case(dev, 2, 3, 512, D, dtype, uniform_block_mask(2, 3, 8, 0.4, 5), 17, out_fp32=True)


def test_shared_mask_broadcast(dev):
    m = causal_block_mask(1, 1, 12, 0.5, 9)
    run_case(dev, 2, 4, 768, 64, torch.float16, m, 3)
    run_case(dev, 2, 4, 768, 64, torch.float16, uniform_block_mask(2, 1, 12, 0.3, 4), 3)
    run_case(dev, 2, 4, 768, 64, torch.float16, uniform_block_mask(1, 4, 12, 0.3, 4), 3)


def test_empty_rows_and_all_false(dev):
    import fa2_custom_mask as fm
    m = uniform_block_mask(1, 2, 8, 0.3, 2)
    m[0, 0, 3, :] = False
    m[0, 1, 0, :] = False
    o = run_case(dev, 1, 2, 512, 64, torch.float16, m, 8)
    assert float(o[0, 0, 192:256].abs().max()) == 0.0 and float(o[0, 1, 0:64].abs().max()) == 0.0
    q, k, v = [x.to(dev) for x in make_qkv(1, 2, 512, 64, torch.float16, 8)]
    z = fm.flash_attention_custom_mask(q, k, v, torch.zeros(1, 2, 8, 8, dtype=torch.bool, device=dev), 0.125)
    assert float(z.abs().max()) == 0.0                                       # fa2_custom_mask.py:49-51


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_many_heads_row_block_per_wavefront(dev, D, dtype):
    """Many heads and many row blocks per workgroup: each wavefront runs whole row blocks (no merge,
    no second kernel).  Covers empty row blocks at the start, inside and at the end of a head, a
    head without kept tiles, and a head whose tiles sit in one row block."""
    B, H, nb = 4, 64, 8
    m = uniform_block_mask(B, H, nb, 0.4, 21)
    m[0, 0, 0, :] = False
    m[0, 1, 3:5, :] = False
    m[0, 2, nb - 1, :] = False
    m[1, 5] = False
    m[2, 7] = False
    m[2, 7, 4, :] = True
    o = run_case(dev, B, H, nb * 64, D, dtype, m, 31)
    assert float(o[1, 5].abs().max()) == 0.0 and float(o[0, 0, :64].abs().max()) == 0.0
    run_case(dev, B, H, nb * 64, D, dtype, m, 31, out_fp32=True)


def test_row_block_per_wavefront_several_workgroups_per_head(dev):
    """64 heads x 32 row blocks: four workgroups per head, ranges cut inside row blocks."""
    m = causal_block_mask(1, 1, 32, 0.6, 13)
    run_case(dev, 2, 32, 2048, 64, torch.float16, m, 5)
    m2 = uniform_block_mask(2, 32, 32, 0.15, 14)
    m2[1, 3, 10:20, :] = False
    run_case(dev, 2, 32, 2048, 64, torch.bfloat16, m2, 6, out_fp32=True)


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.bfloat16)])
def test_short_and_long_row_blocks_mixed(dev, D, dtype):
    """Runs of short row blocks inside a workgroup's range go one row block per wavefront, long
    ones are shared by the wavefronts: block-causal masks (lengths 1..nb), alternating short / long /
    empty row blocks, and a mask whose row blocks all hold one or two tiles."""
    nb = 48
    run_case(dev, 1, 2, nb * 64, D, dtype, causal_block_mask(1, 1, nb, 0.6, 3), 41, out_fp32=True)
    g = torch.Generator().manual_seed(9)
    m = torch.zeros(1, 2, nb, nb, dtype=torch.bool)
    for r in range(nb):
        kind = r % 5
        if kind in (0, 1, 3):
            m[0, :, r, torch.randperm(nb, generator=g)[:1 + r % 3]] = True      # 1..3 tiles
        elif kind == 2:
            m[0, 0, r, :] = True                                                   # long
            m[0, 1, r, torch.randperm(nb, generator=g)[:30]] = True
        # kind 4: empty
    run_case(dev, 1, 2, nb * 64, D, dtype, m, 42, out_fp32=True)
    m2 = torch.zeros(2, 3, nb, nb, dtype=torch.bool)
    idx = torch.randint(0, nb, (2, 3, nb, 2), generator=g)
    m2.scatter_(3, idx, True)
    run_case(dev, 2, 3, nb * 64, D, dtype, m2, 43, out_fp32=True)


def test_mask_none_is_dense_attention(dev):
    """mask=None (the default the reference advertises, fa2_custom_mask.py:43) = dense attention:
    against torch's scaled_dot_product_attention in fp32, forward and backward."""
    import fa2_custom_mask as fm
    q, k, v, do = [x.to(dev) for x in make_qkv(2, 2, 512, 64, torch.float16, 91, n=4)]
    qr, kr, vr = [x.float().requires_grad_(True) for x in (q, k, v)]
    ref = torch.nn.functional.scaled_dot_product_attention(qr, kr, vr, scale=0.125)
    ref.backward(do.float())
    qg, kg, vg = [x.clone().requires_grad_(True) for x in (q, k, v)]
    o = fm.flash_attention_custom_mask(qg, kg, vg, None, 0.125)
    o.backward(do)
    assert errors(o, ref.detach().cpu().numpy())[0] <= 2e-2
    for got, want in ((qg.grad, qr.grad), (kg.grad, kr.grad), (vg.grad, vr.grad)):
        assert errors(got, want.cpu().numpy())[0] <= 2e-2


def test_lists_cache_follows_the_mask(dev):
    """The kept-tile lists of a mask tensor are reused while the tensor is unchanged and rebuilt
    after an in-place change or for another tensor."""
    import fa2_custom_mask as fm
    from fa2_custom_mask import utils
    q, k, v = [x.to(dev) for x in make_qkv(1, 1, 512, 64, torch.float16, 92)]
    m = uniform_block_mask(1, 1, 8, 0.5, 93)
    md = m.to(dev)
    utils.lists_cache.clear()
    o1 = fm.flash_attention_custom_mask(q, k, v, md, 0.125)
    first = utils.lists_cache.get(md, 512, False)
    assert first is not None
    o2 = fm.flash_attention_custom_mask(q, k, v, md, 0.125)
    assert utils.lists_cache.get(md, 512, False) is first and same_up_to_rounding(o1, o2)
    m[0, 0, 2, :] = ~m[0, 0, 2, :]
    m[0, 0, 2, 2] = True
    md.copy_(m)                                   # in place: same tensor object, new contents
    assert utils.lists_cache.get(md, 512, False) is None
    o3 = fm.flash_attention_custom_mask(q, k, v, md, 0.125)
    o_ref = orc.naive_attention(f32(q), f32(k), f32(v), m.numpy(), 0.125)
    assert errors(o3, o_ref)[0] <= 2e-2
    md2 = m.to(dev)                               # equal contents, different tensor: not shared
    assert utils.lists_cache.get(md2, 512, False) is None


def test_workspace_contents_do_not_matter(dev):
    """Row blocks shared between workgroups are merged by whichever workgroup arrives last, counted
    in the workspace: stale or random workspace contents, and repeated runs on the same workspace,
    must give the same result."""
    import fa2_custom_mask as fm
    N, D = 4096, 64
    q, k, v = [x.to(dev) for x in make_qkv(1, 2, N, D, torch.float16, 77)]
    m = uniform_block_mask(1, 2, N // 64, 0.5, 78)
    m[0, 1, 5, :] = False
    lists = fm.block_mask_to_lists(m.to(dev))
    o_ref, lse_ref = orc.naive_attention(f32(q.cpu()), f32(k.cpu()), f32(v.cpu()), m.numpy(), 0.125, return_lse=True)
    plan = fm.ForwardPlan(q, k, v, lists, 0.125)
    g = torch.Generator(device="cpu").manual_seed(5)
    for fill in ("ones", "random", None, None, "zeros", None):
        if fill == "ones":
            plan.ws.fill_(255)
        elif fill == "zeros":
            plan.ws.zero_()
        elif fill == "random":
            plan.ws.copy_(torch.randint(0, 256, plan.ws.shape, dtype=torch.uint8, generator=g))
        plan.o.fill_(7.0)
        plan.lse.fill_(7.0)
        o, lse = plan.run()
        torch.cuda.synchronize()
        ma, rl = errors(o, o_ref)
        assert ma <= 2e-2 and rl <= RELL2, (fill, ma, rl)
        fin = np.isfinite(lse_ref)
        assert np.array_equal(np.isfinite(lse.cpu().numpy()), fin)
        assert np.abs(lse.cpu().numpy()[fin] - lse_ref[fin]).max() <= 2e-3


def test_dense_elementwise_mask_c2_small(dev):
    """Tile-constant elementwise mask gives the same result as its block mask."""
    import fa2_custom_mask as fm
    N, D = 1280, 64
    block = uniform_block_mask(1, 1, N // 64, 0.3, 6)
    q, k, v = [x.to(dev) for x in make_qkv(1, 1, N, D, torch.float16, 6)]
    dense = block.to(dev).repeat_interleave(64, 2).repeat_interleave(64, 3)
    o1 = fm.flash_attention_custom_mask(q, k, v, block.to(dev), 0.125)
    o2 = fm.flash_attention_custom_mask(q, k, v, dense, 0.125)
    assert same_up_to_rounding(o1, o2)


def test_strided_inputs(dev):
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 512, 64
    g = torch.Generator().manual_seed(0)
    qkv = torch.randn(B, N, 3, H, D, generator=g).to(torch.float16).to(dev)  # packed layout
    q, k, v = [qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)]
    m = uniform_block_mask(1, 1, 8, 0.5, 1).to(dev)
    o1 = fm.flash_attention_custom_mask(q, k, v, m, 0.125)
    o2 = fm.flash_attention_custom_mask(q.contiguous(), k.contiguous(), v.contiguous(), m, 0.125)
    assert same_up_to_rounding(o1, o2)


@pytest.mark.parametrize("keep", [0.1, 1.0])
def test_c2_config(dev, keep):
    """N=6400 D=64 fp16, 100x100 tiles."""
    run_case(dev, 1, 1, 6400, 64, torch.float16, uniform_block_mask(1, 1, 100, keep, 1235), 1235)


def test_run_to_run_stability(dev):
    """Tiles are handed to wavefronts dynamically, so the fp32 summation order can differ between
    runs: results agree to rounding (one fp16 ulp of the output), not necessarily bit for bit."""
    import fa2_custom_mask as fm
    q, k, v = [x.to(dev) for x in make_qkv(1, 2, 2048, 64, torch.float16, 5)]
    m = uniform_block_mask(1, 2, 32, 0.3, 5).to(dev)
    o1 = fm.flash_attention_custom_mask(q, k, v, m, 0.125)
    o2 = fm.flash_attention_custom_mask(q, k, v, m, 0.125)
    assert float((o1.float() - o2.float()).abs().max()) <= 1e-3


def test_invariants_large(dev):
    """Size-independent properties at the headline size N=17536: v = 1 gives O = 1, and
    k = 0 gives the mean of the kept V rows."""
    import fa2_custom_mask as fm
    N, D, nb = 17536, 64, 274
    q, k, v = [x.to(dev) for x in make_qkv(1, 1, N, D, torch.float16, 77)]
    m = uniform_block_mask(1, 1, nb, 0.1, 77).to(dev)
    o = fm.flash_attention_custom_mask(q, k, torch.ones_like(v), m, 0.125)
    assert float((o.float() - 1).abs().max()) <= 2e-3
    o = fm.flash_attention_custom_mask(q, torch.zeros_like(k), v, m, 0.125)
    mean = torch.zeros(N, D, device=dev)
    vt = v[0, 0].float().view(nb, 64, D).mean(1)                              # per-tile means
    w = m[0, 0].float()
    mean_rows = (w @ vt) / w.sum(1, keepdim=True)
    ref = mean_rows.repeat_interleave(64, 0)
    assert float((o[0, 0].float() - ref).abs().max()) <= 2e-3


def test_inference_mode(dev):
    """Tensors made under torch.inference_mode() keep no write counter (reading it raises): the cache of
    kept-tile lists must not depend on it.  Block mask, elementwise mask and no mask, each called
    twice, with the mask changed in place between the two calls."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 512, 64
    q, k, v = make_qkv(B, H, N, D, torch.float16, 31)
    sm_scale = 0.125
    with torch.inference_mode():
        qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
        block = uniform_block_mask(1, 2, 8, 0.5, 6).to(dev)
        g = torch.Generator().manual_seed(7)
        dense = (torch.rand(1, 1, N, N, generator=g) < 0.3) | torch.eye(N, dtype=torch.bool)
        dense_d = dense.to(dev)
        for _ in range(2):
            o = fm.flash_attention_custom_mask(qd, kd, vd, block, sm_scale)
            o_ref = orc.naive_attention(f32(q), f32(k), f32(v), block.cpu().numpy(), sm_scale)
            assert errors(o, o_ref)[1] <= RELL2
            block[0, 0, 2, :] = False            # a write the cache cannot see on such a tensor
            block[0, 0, 2, 5] = True
        for _ in range(2):
            o = fm.flash_attention_custom_mask(qd, kd, vd, dense_d, sm_scale)
            o_ref = orc.naive_attention(f32(q), f32(k), f32(v), dense_d.cpu().numpy(), sm_scale)
            assert errors(o, o_ref)[1] <= RELL2
            dense_d[0, 0, 100:200, 0:300] = False
            dense_d[0, 0, 100:200, 7] = True
        for _ in range(2):
            o = fm.flash_attention_custom_mask(qd, kd, vd, None, sm_scale)
            o_ref = orc.naive_attention(f32(q), f32(k), f32(v), np.ones((1, 1, 8, 8), dtype=bool), sm_scale)
            assert errors(o, o_ref)[1] <= RELL2


def test_cached_lists_on_another_stream(dev):
    """The lists of a mask are built on the stream of the first call; a call on another stream uses the
    cached lists only after that work (the cache makes the second stream wait)."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 1, 4096, 64
    q, k, v = make_qkv(B, H, N, D, torch.float16, 32)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    mask = uniform_block_mask(1, 1, 64, 0.3, 8)
    o_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), 0.125)
    md = mask.to(dev)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(dev)
    o1 = fm.flash_attention_custom_mask(qd, kd, vd, md, 0.125)          # builds the lists on the current stream
    with torch.cuda.stream(side):
        o2 = fm.flash_attention_custom_mask(qd, kd, vd, md, 0.125)      # cached lists, other stream
    side.synchronize()
    torch.cuda.synchronize()
    assert errors(o1, o_ref)[1] <= RELL2 and errors(o2, o_ref)[1] <= RELL2


@pytest.mark.parametrize("dtype,out_fp32", [(torch.float16, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_large_magnitudes(dev, dtype, out_fp32):
    """Inputs far from N(0,1): scores with a standard deviation of 23 (a nearly one-hot softmax whose reference
    exponent moves by hundreds between tiles) and values of the order of 1e3.  The kernels fold the scale
    into a 16-bit Q, feed exponents through an extra contraction slice and, for bf16 inputs with fp32
    results, convert V to fp16: all of that must hold up, relative to the size of the values."""
    import fa2_custom_mask as fm
    B, H, N, D = 1, 2, 1024, 64
    g = torch.Generator().manual_seed(77)
    q = (torch.randn(B, H, N, D, generator=g) * 4.0).to(dtype)
    k = (torch.randn(B, H, N, D, generator=g) * 4.0).to(dtype)
    v = (torch.randn(B, H, N, D, generator=g) * 1000.0).to(dtype)
    mask = uniform_block_mask(1, 1, 16, 0.5, 12)
    sc = 0.18
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sc, return_lse=True)
    o, lse = fm.flash_attention_custom_mask_lse(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), sc, out_fp32=out_fp32)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o).all())
    ma, rl = errors(o, o_ref)
    scale = float(np.abs(o_ref).max())
    print("%s fp32out=%s: max-abs %.3e of %.3e, rel-L2 %.3e" % (dtype, out_fp32, ma, scale, rl))
    # the bars of the forward tests, relative to the size of the result
    assert ma <= (2e-2 if dtype == torch.float16 else 3e-2) * max(1.0, scale / 4.0)
    assert rl <= (1e-3 if dtype == torch.float16 or out_fp32 else 3e-3) * 1.5
    assert np.abs(lse.cpu().numpy() - lse_ref).max() <= 2e-3 * max(1.0, float(np.abs(lse_ref).max()) / 8.0)


@pytest.mark.parametrize("B,H,Bm,Hm,N,D,dtype", [(1, 1, 1, 1, 1024, 64, torch.float16), (2, 3, 1, 1, 512, 128, torch.bfloat16),
                                                 (2, 2, 2, 2, 768, 64, torch.float16), (1, 2, 1, 2, 4096, 64, torch.float16)])
def test_lists_and_forward_from_one_call(dev, B, H, Bm, Hm, N, D, dtype):
    """bsattn_fwd_block_mask (the reference's whole forward call, fa2_custom_mask.py:43-94: lists of the block mask,
    then the kernel): O and LSE against the oracle, the lists it leaves against the oracle's, bit for bit, and the
    same through flash_attention_custom_mask for a mask that is not in the cache."""
    import ctypes
    import fa2_custom_mask as fm
    from fa2_custom_mask import _ext, utils
    nb = N // 64
    mask = uniform_block_mask(Bm, Hm, nb, 0.4, 300 + N)
    mask[0, 0, 1, :] = False                      # a row block without kept tiles
    q, k, v = make_qkv(B, H, N, D, dtype, 301 + N)
    sc = 1.0 / np.sqrt(D)
    o_ref, lse_ref = orc.naive_attention(f32(q), f32(k), f32(v), mask.numpy(), sc, return_lse=True)
    qd, kd, vd, md = q.to(dev), k.to(dev), v.to(dev), mask.to(dev)
    lib = _ext.lib()
    rows = Bm * Hm * nb
    row_ptr = torch.full((rows + 1,), -1, dtype=torch.int32, device=dev)
    col_idx = torch.full((rows * nb,), -1, dtype=torch.int32, device=dev)
    counts = torch.full((2,), -1, dtype=torch.int32, device=dev)
    o = torch.full((B, H, N, D), float("nan"), dtype=dtype, device=dev)
    lse = torch.full((B, H, N), float("nan"), dtype=torch.float32, device=dev)
    n = ctypes.c_size_t()
    assert lib.bsattn_fwd_block_mask_workspace(Bm, Hm, B, H, N, D, ctypes.byref(n)) == 0
    ws = torch.randint(0, 255, (n.value,), dtype=torch.uint8, device=dev)       # contents must not matter
    args = (qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), lse.data_ptr(), md.data_ptr(), _ext.strides4(md),
            Bm, Hm, row_ptr.data_ptr(), col_idx.data_ptr(), counts.data_ptr(), B, H, N, D, _ext.dtype_code(dtype),
            _ext.dtype_code(dtype), float(sc), _ext.strides4(qd), _ext.strides4(kd), _ext.strides4(vd), _ext.strides4(o))
    assert lib.bsattn_fwd_block_mask(*args, ws.data_ptr(), n.value - 1, _ext.current_stream(dev)) == -6   # workspace too small
    assert lib.bsattn_fwd_block_mask(*args, ws.data_ptr(), n.value, _ext.current_stream(dev)) == 0
    torch.cuda.synchronize()
    rp_ref, ci_ref = orc.csr_from_block_mask(mask.numpy())
    G, T = counts.tolist()
    assert T == len(ci_ref) and G == int((np.diff(rp_ref) > 0).sum())
    assert np.array_equal(row_ptr.cpu().numpy(), rp_ref) and np.array_equal(col_idx[:T].cpu().numpy(), ci_ref)
    tol_abs, tol_rel = (2e-2, 1e-3) if dtype == torch.float16 else (3e-2, 3e-3)
    ma, rl = errors(o, o_ref)
    assert ma <= tol_abs and rl <= tol_rel
    fin = np.isfinite(lse_ref)
    assert np.abs(lse.cpu().numpy()[fin] - lse_ref[fin]).max() <= 2e-3 and bool(torch.isinf(lse[0, 0, 64:128]).all())
    # the Python operator takes the same route for a mask it has not seen
    utils.lists_cache.clear()
    o2 = fm.flash_attention_custom_mask(qd, kd, vd, md, sc)
    cached = utils.lists_cache.get(md, N, False)
    assert cached is not None and np.array_equal(cached.row_ptr.cpu().numpy(), rp_ref)
    ma, rl = errors(o2, o_ref)
    assert ma <= tol_abs and rl <= tol_rel
    o3, lse3 = fm.flash_attention_custom_mask_lse(qd, kd, vd, md, sc)            # second call: cached lists
    assert same_up_to_rounding(o3, o2, rel=2.0 ** -9 if dtype == torch.float16 else 2.0 ** -6, abs_=3e-4 if dtype == torch.float16 else 2e-3)
    assert np.abs(lse3.cpu().numpy()[fin] - lse_ref[fin]).max() <= 2e-3
