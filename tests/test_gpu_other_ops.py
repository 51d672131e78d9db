"""GPU parity of the reference-compatible alternates (both-encoded _sbvr_mm_T and
the trans=True _sbvr_row_deq_mm_T) and of SBVRLinear, against the CPU oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rand_enc(rng, rows, K, S, G, L, oracle):
    sel = rng.integers(0, 1 << S, size=rows * K).astype(np.int32)
    bvr = oracle.C.planes_to_default(oracle.C.sel_to_planes(sel, S, 32), rows, K)
    idx = rng.integers(0, L, size=(K // G, rows)).astype(np.uint8 if L <= 256 else np.uint16)
    cache = (rng.standard_normal((L, S)) * 0.5).astype(np.float16)
    return bvr, idx, cache


def _close(y, yd, ulps=2.0):
    got = y.float().cpu().numpy().astype(np.float64)
    rms = float(np.sqrt(np.mean(yd ** 2))) + 1e-30
    assert (np.abs(got - yd) / np.maximum(np.abs(yd), 1e-2 * rms)).max() <= 1e-2
    assert (np.abs(got - yd) / (np.maximum(np.abs(yd), rms) * 2.0 ** -10)).max() <= ulps


@pytest.mark.parametrize("M,N,K,Sl,Sr,G,Ll,Lr", [(1, 64, 512, 4, 4, 256, 5, 9), (3, 40, 256, 2, 3, 128, 300, 7),
                                                 (2, 33, 512, 8, 6, 256, 4, 400),       # no popcount-kernel instance
                                                 (1, 1000, 160, 4, 4, 32, 16, 256),     # 5 words: a partial chunk
                                                 (1, 130, 4096, 4, 2, 64, 16, 300),     # 16 chunks, uint16 right index
                                                 (2, 200, 14336, 3, 4, 128, 16, 256),   # 7 chunks per wave
                                                 (1, 96, 512, 4, 4, 512, 8, 8),         # group longer than a chunk
                                                 # one left row of up to 4 planes at the decode kernel's shapes: the
                                                 # left planes are that kernel's batch rows
                                                 (1, 256, 1024, 4, 4, 128, 16, 256), (1, 1030, 2048, 3, 4, 128, 300, 300),
                                                 (1, 48, 512, 2, 3, 256, 7, 9), (1, 4096, 4096, 4, 4, 128, 16, 256),
                                                 (1, 14336, 4096, 4, 4, 128, 16, 256), (1, 1000, 1024, 1, 8, 128, 5, 40),
                                                 (1, 4096, 14336, 4, 4, 128, 16, 256),  # K split across workgroups
                                                 (1, 2048, 7168, 4, 2, 256, 16, 300), (1, 512, 4096, 4, 6, 128, 9, 256)])
def test_mm_T(oracle, M, N, K, Sl, Sr, G, Ll, Lr):
    import sbvr
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(M * 100 + N)
    lb, li, lc = _rand_enc(rng, M, K, Sl, G, Ll, oracle)
    rb, ri, rc = _rand_enc(rng, N, K, Sr, G, Lr, oracle)
    t = lambda a: torch.from_numpy(a).to(dev)
    y = sbvr._sbvr_mm_T(t(lb), t(li), t(lc), t(rb), t(ri), t(rc), torch.zeros(0, dtype=torch.float16, device=dev),
                        bvr_len=G)
    _, yd = oracle.C.mm_T(lb, li, lc, rb, ri, rc, G)
    _close(y, yd)
    bias = (rng.standard_normal(N)).astype(np.float16)
    yb = sbvr._sbvr_mm_T(t(lb), t(li), t(lc), t(rb), t(ri), t(rc), t(bias), bvr_len=G)
    want, _ = oracle.C.mm_T(lb, li, lc, rb, ri, rc, G, bias)
    d = np.abs(yb.float().cpu().numpy().astype(np.float64) - want.astype(np.float64))
    assert d.max() <= 2.0 ** -9 * max(np.abs(want.astype(np.float64)).max(), 1.0)


def test_mm_T_without_workspace_and_repeatable(oracle):
    """The reference-shaped entry point (no workspace) at a shape whose decode launch would split K across
    workgroups: it must still answer (through the popcount kernel); and the split form twice, bit for bit."""
    import ctypes
    import sbvr
    from sbvr import hip
    dev = torch.device("cuda:0")
    M, N, K, S, G, L = 1, 4096, 14336, 4, 128, 256
    rng = np.random.default_rng(11)
    lb, li, lc = _rand_enc(rng, M, K, S, G, 16, oracle)
    rb, ri, rc_ = _rand_enc(rng, N, K, S, G, L, oracle)
    t = lambda a: torch.from_numpy(a).to(dev)
    d = [t(a) for a in (lb, li, lc, rb, ri, rc_)]
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    lib = hip._load()
    vp = ctypes.c_void_p
    rc = lib.sbvr_hip_mm_T(vp(d[0].data_ptr()), vp(d[1].data_ptr()), 1, vp(d[2].data_ptr()), vp(d[3].data_ptr()),
                           vp(d[4].data_ptr()), 1, vp(d[5].data_ptr()), None, vp(out.data_ptr()), M, N, K, S, S, G, 16, L,
                           vp(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    _, yd = oracle.C.mm_T(lb, li, lc, rb, ri, rc_, G)
    _close(out, yd)
    none = torch.zeros(0, dtype=torch.float16, device=dev)
    first = sbvr._sbvr_mm_T(*d, none, bvr_len=G)
    _close(first, yd)
    for _ in range(4):
        again = sbvr._sbvr_mm_T(*d, none, bvr_len=G)
        assert torch.equal(first, again)


def test_mm_T_object_api(oracle, golden):
    """sbvr.mm_T(lhs, rhs, bias) on objects built from the reference's encodings."""
    import sbvr
    dev = torch.device("cuda:0")
    g = golden("default_s2")
    mk = lambda: sbvr.sbvr.from_parts(*(torch.from_numpy(g[k]).to(dev) for k in ("bvr", "coeff_idx", "coeff_cache")), 256)
    a, b = mk(), mk()
    y = sbvr.mm_T(a, b, None)
    _, yd = oracle.C.mm_T(g["bvr"], g["coeff_idx"], g["coeff_cache"], g["bvr"], g["coeff_idx"], g["coeff_cache"], 256)
    _close(y, yd)
    w = g["decoded"].astype(np.float64)
    assert np.abs(y.float().cpu().numpy() - w @ w.T).max() <= 1e-2 * np.abs(w @ w.T).max()


@pytest.mark.parametrize("M,N,K,S,G,L", [(1, 256, 64, 4, 256, 9), (2, 512, 40, 2, 128, 300),
                                         (3, 1024, 4096, 4, 128, 256), (1, 96, 1000, 3, 32, 700),
                                         (5, 64, 130, 8, 64, 40), (1, 4096, 2048, 6, 128, 256),
                                         (2, 14336, 512, 4, 128, 256), (1, 32, 1, 4, 32, 2),
                                         # four planes, K a multiple of 128, groups of 64 columns and more: the MFMA form
                                         (1, 64, 128, 4, 64, 5), (4, 256, 640, 4, 64, 300), (2, 192, 256, 4, 192, 9),
                                         (1, 14336, 4096, 4, 128, 256), (1, 4096, 14336, 4, 256, 256)])
def test_row_deq_mm_T(oracle, M, N, K, S, G, L):
    import sbvr
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(N + K)
    # the encoded tensor is W^T: K rows of N columns, groups along N
    bvr, idx, cache = _rand_enc(rng, K, N, S, G, L, oracle)         # (N/32, K, S), (N/G, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    t = lambda a: torch.from_numpy(a).to(dev)
    y = sbvr._sbvr_row_deq_mm_T(t(x), t(bvr), t(idx), t(cache), t(bias), 0, bvr_len=G)
    want = oracle.C.row_deq_mm_T(x, bvr, idx, cache, G, bias).astype(np.float64)
    d = np.abs(y.float().cpu().numpy().astype(np.float64) - want)
    assert d.max() <= 2.0 ** -9 * max(np.abs(want).max(), 1.0)


def test_row_deq_mm_T_without_workspace_and_repeatable(oracle):
    """The reference-shaped entry point (no workspace: K is never split across workgroups) against the oracle at a
    shape the binding would split, and the split form twice: the fixed-point accumulators make it repeatable."""
    import ctypes
    import sbvr
    from sbvr import hip
    dev = torch.device("cuda:0")
    M, N, K, S, G, L = 2, 1024, 2048, 4, 128, 256
    rng = np.random.default_rng(5)
    bvr, idx, cache = _rand_enc(rng, K, N, S, G, L, oracle)
    x = rng.standard_normal((M, K)).astype(np.float16)
    t = lambda a: torch.from_numpy(a).to(dev)
    dx, db, di, dc = t(x), t(bvr), t(idx), t(cache)
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    lib = hip._load()
    vp = ctypes.c_void_p
    rc = lib.sbvr_hip_row_deq_mm_T(vp(dx.data_ptr()), vp(db.data_ptr()), vp(di.data_ptr()), 1, vp(dc.data_ptr()), None,
                                   vp(out.data_ptr()), M, N, K, S, G, L, vp(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    want = oracle.C.row_deq_mm_T(x, bvr, idx, cache, G, None).astype(np.float64)
    assert np.abs(out.float().cpu().numpy() - want).max() <= 2.0 ** -9 * max(np.abs(want).max(), 1.0)
    none = torch.zeros(0, dtype=torch.float16, device=dev)
    first = sbvr._sbvr_row_deq_mm_T(dx, db, di, dc, none, 0, bvr_len=G)
    assert np.abs(first.float().cpu().numpy() - want).max() <= 2.0 ** -9 * max(np.abs(want).max(), 1.0)
    for _ in range(4):
        assert torch.equal(first, sbvr._sbvr_row_deq_mm_T(dx, db, di, dc, none, 0, bvr_len=G))


def test_row_deq_golden(oracle, golden):
    import sbvr
    dev = torch.device("cuda:0")
    g = golden("trans_s2")
    K, N = g["decoded"].shape
    x = torch.randn((2, K), generator=torch.Generator().manual_seed(3)).to(torch.float16)
    t = lambda a: torch.from_numpy(a).to(dev)
    y = sbvr._sbvr_row_deq_mm_T(x.to(dev), t(g["bvr"]), t(g["coeff_idx"]), t(g["coeff_cache"]),
                                torch.zeros(0, dtype=torch.float16, device=dev), 0)
    want = x.numpy().astype(np.float64) @ g["decoded"].astype(np.float64)
    assert np.abs(y.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(want).max()


def test_sbvr_linear_module(oracle, golden):
    """SBVRLinear on a reference encoding: leading dims, padding of K, bias, > 16 rows."""
    import sbvr
    dev = torch.device("cuda:0")
    g = golden("pad_s2")                       # weight (3, 300) padded to 512
    enc = sbvr.sbvr.from_parts(*(torch.from_numpy(g[k]).to(dev) for k in ("bvr", "coeff_idx", "coeff_cache")), 256,
                               original_shape=(3, 300))
    lin = sbvr.SBVRLinear.from_sbvr(enc)
    x = torch.randn((2, 5, 300), generator=torch.Generator().manual_seed(4)).to(torch.float16)
    y = lin(x.to(dev))
    assert y.shape == (2, 5, 3)
    want = x.numpy().astype(np.float64) @ g["decoded"].astype(np.float64).T
    assert np.abs(y.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(want).max()
    from sbvr import synth
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(128, 256, 4, 128, 64, seed=2))
    bias = torch.randn(128, generator=torch.Generator().manual_seed(5)).to(torch.float16)
    lin2 = sbvr.SBVRLinear(256, 128, bvr, idx, cache, 128, bias.to(dev))
    x2 = torch.randn((40, 256), generator=torch.Generator().manual_seed(6)).to(torch.float16)
    y2 = lin2(x2.to(dev))
    yref, _ = oracle.C.linear_f16(x2.numpy(), bvr.cpu().numpy(), idx.cpu().numpy(), cache.cpu().numpy(), 128, bias.numpy())
    d = np.abs(y2.float().cpu().numpy().astype(np.float64) - yref.astype(np.float64))
    assert d.max() <= 1e-2 * np.abs(yref.astype(np.float64)).max()      # 40 rows: the prefill kernel's rounding
    # q | k | v as one layer: the parts' outputs side by side
    encs = []
    for i, rows in enumerate((256, 64, 64)):
        b, ix, c = (t.to(dev) for t in synth.random_encoding(rows, 512, 4, 128, 200, seed=20 + i))
        encs.append(sbvr.sbvr.from_parts(b, ix, c, 128, original_shape=(rows, 512)))
    fused = sbvr.SBVRLinear.fused(encs)
    assert fused.coeff_idx.dtype == torch.uint16 and fused.coeff_cache.shape[0] == 600
    x3 = torch.randn((3, 512), generator=torch.Generator().manual_seed(7)).to(torch.float16)
    y3 = fused(x3.to(dev))
    assert y3.shape == (3, 384)
    at = 0
    for e in encs:
        _, yd = oracle.C.linear_f16(x3.numpy(), e.bvr.cpu().numpy(), e.coeff_idx.cpu().numpy(), e.coeff_cache.cpu().numpy(), 128)
        rows = e.original_data_shape[0]
        _close(y3[:, at:at + rows], yd)
        at += rows


def test_hip_init_and_bad_arguments():
    import sbvr
    dev = torch.device("cuda:0")
    sbvr._sbvr_hip_init(dev)
    from sbvr import synth
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(32, 256, 4, 128, 16))
    x = torch.zeros((1, 256), dtype=torch.float16, device=dev)
    with pytest.raises(TypeError):
        sbvr._sbvr_linear_f16(x.float(), bvr, idx, cache, None, 128)
    with pytest.raises(ValueError):
        sbvr._sbvr_linear_f16(x[:, :128], bvr, idx, cache, None, 128)
    with pytest.raises(ValueError):
        sbvr._sbvr_linear_f16(torch.zeros((2, 512), dtype=torch.float16, device=dev)[:, ::2],
                              bvr, idx, cache, None, 128)                                  # not contiguous
    with pytest.raises(TypeError):
        sbvr._sbvr_linear_f16(x, bvr, idx.to(torch.uint16), cache, None, 128)          # 16 lines want uint8


def test_torch_extension_equals_ctypes_binding(oracle):
    """Both bindings call the same entry points: identical bits, on the caller's stream."""
    import sbvr
    from sbvr import _sbvr_hip_ops as ops, synth
    dev = torch.device("cuda:0")
    ops._sbvr_hip_init()
    none = torch.zeros(0, dtype=torch.float16, device=dev)
    for (M, N, K, S, L) in [(1, 4096, 4096, 4, 256), (3, 1000, 1024, 3, 300), (48, 512, 1024, 4, 64)]:
        bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(N, K, S, 128, L, seed=N))
        x = torch.randn((M, K), generator=torch.Generator().manual_seed(K)).to(torch.float16).to(dev)
        bias = torch.randn((N,), generator=torch.Generator().manual_seed(1)).to(torch.float16).to(dev)
        assert torch.equal(ops._sbvr_linear_f16(x, bvr, idx, cache), sbvr._sbvr_linear_f16(x, bvr, idx, cache))
        assert torch.equal(ops._sbvr_linear_f16(x, bvr, idx, cache, bias, 128),
                           sbvr._sbvr_linear_f16(x, bvr, idx, cache, bias, 128))
    # the reference's two operator forms, reference argument lists
    lb, li, lc = (t.to(dev) for t in synth.random_encoding(2, 1024, 4, 128, 16, seed=3))
    rb, ri, rc = (t.to(dev) for t in synth.random_encoding(640, 1024, 4, 128, 256, seed=4))
    assert torch.equal(ops._sbvr_mm_T(lb, li, lc, rb, ri, rc, none), sbvr._sbvr_mm_T(lb, li, lc, rb, ri, rc, none))
    tb, ti, tc = (t.to(dev) for t in synth.random_encoding(1024, 640, 4, 128, 256, seed=5))      # W^T: (K, N)
    x = torch.randn((2, 1024), generator=torch.Generator().manual_seed(6)).to(torch.float16).to(dev)
    assert torch.equal(ops._sbvr_row_deq_mm_T(x, tb, ti, tc, none, 0), sbvr._sbvr_row_deq_mm_T(x, tb, ti, tc, none, 0))
    # one-row variants
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(512, 1024, 4, 128, 256, seed=7))
    gu = torch.randn((1, 2048), generator=torch.Generator().manual_seed(8)).to(torch.float16).to(dev)
    assert torch.equal(ops._sbvr_linear_f16_swiglu(gu, bvr, idx, cache), sbvr._sbvr_linear_f16_swiglu(gu, bvr, idx, cache))
    x1, d1 = x[:1].contiguous(), x[1:].contiguous()
    w = torch.ones(1024, dtype=torch.float16, device=dev)
    xo1, xo2 = torch.empty_like(x1), torch.empty_like(x1)
    a = ops._sbvr_linear_f16_add_rmsnorm(x1, d1, w, 1e-5, xo1, bvr, idx, cache)
    b = sbvr._sbvr_linear_f16_add_rmsnorm(x1, d1, w, 1e-5, xo2, bvr, idx, cache)
    assert torch.equal(a, b) and torch.equal(xo1, xo2)
    # on a side stream the extension launches there too
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        y = ops._sbvr_linear_f16(x, bvr, idx, cache)
    side.synchronize()
    assert torch.equal(y, sbvr._sbvr_linear_f16(x, bvr, idx, cache))
