"""GPU parity of the SBVR linear operator (through the C ABI of libsbvr_hip.so,
bound by sbvr/hip.py) against the CPU oracle, on seeded inputs.

Tolerance (fp16 outputs, fp32 accumulation): every output must lie within
1e-2 relative of the oracle's unrounded double sum, outputs whose magnitude is
below 1 % of the output RMS being judged against that RMS instead; on top of
that the worst error must stay below 2 fp16 ulps of max(|ref|, RMS), which is
what an fp32-accumulating kernel is expected to reach.  (9 rows and more take
the 32-row kernel by default, which rounds decoded weights to fp16: those runs
are held to that kernel's bound, see check_rounded; flags = 2 keeps the decode
kernel.)  The largest shapes are checked on a seeded sample of columns, the
window edges always among them: the oracle is exact per column."""
import numpy as np
import pytest
import torch

import parity

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch.device("cuda:0")


def check(y_gpu, yd, what=""):
    y = y_gpu.float().cpu().numpy().astype(np.float64)
    rms = float(np.sqrt(np.mean(yd ** 2))) + 1e-30
    scale = np.maximum(np.abs(yd), 1e-2 * rms)
    rel = np.abs(y - yd) / scale
    assert rel.max() <= 1e-2, f"{what}: relative error {rel.max():.3e} > 1e-2"
    ulp = np.abs(y - yd) / (np.maximum(np.abs(yd), rms) * 2.0 ** -10)
    assert ulp.max() <= 2.0, f"{what}: {ulp.max():.2f} fp16 ulps off"
    return rel.max(), ulp.max()


def check_rounded(oracle, y_gpu, yd, operands, rounding, what=""):
    """The 32-row kernel (9..32 rows by default) rounds each decoded weight to fp16: in its table look-up form
    exactly as the reference's decode() does, which the oracle's mode 1 restates (tests/parity.py)."""
    x, bn, inn, cache, G = operands
    _, yd1 = oracle.C.linear_f16(x, bn, inn, cache, G, mode=1)
    return parity.judge(y_gpu.float().cpu().numpy(), yd, yd1, rounding, what)


DECODE, ROWS32 = 2, 3


def run_case(oracle, N, K, S, G, M, L, seed=0, bias=False, flags=0, sigma=0.02, xscale=1.0):
    """flags = 2 keeps the 32-row kernel out: 9..16 rows then take the decode kernel of 5..16 rows, which the
    default dispatch uses up to 8 rows (and for 6 and 8 planes)."""
    import sbvr
    from sbvr import hip, synth
    dev = _dev()
    bvr, idx, cache = synth.random_encoding(N, K, S, G, L, sigma=sigma, seed=seed)
    gen = torch.Generator().manual_seed(seed + 1)
    x = (torch.randn((M, K), generator=gen) * xscale).to(torch.float16)
    b = (torch.randn((N,), generator=gen) * 0.3).to(torch.float16) if bias else None
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev),
                              None if b is None else b.to(dev), bvr_len=G, flags=flags)
    torch.cuda.synchronize()
    ran, rounding = hip.last_kernel(), hip.last_rounding()
    if flags == 2 and M <= 16:
        assert ran != ROWS32 or G % 128 != 0 or N < 16, f"flags=2 ran kernel {ran}"
    bn, inn, bb = bvr.numpy(), idx.numpy(), None if b is None else b.numpy()
    if float(N) * K * M > 2.5e8:
        # Columns are independent: the oracle on a seeded sample of them (the first and last columns and the
        # columns around the window edges of the decode kernel always among them) is exact for those columns.
        rng = np.random.default_rng(seed)
        count = max(256, int(2.5e8 / (float(K) * M)))
        edges = [c for e in (0, 56, 64, 112, 128, N - 128, N - 112, N - 64, N - 56, N) for c in (e - 1, e, e + 1) if 0 <= c < N]
        cols = np.unique(np.concatenate([rng.choice(N, size=min(count, N), replace=False), np.array(edges, dtype=np.int64)]))
        bn, inn = np.ascontiguousarray(bn[:, cols, :]), np.ascontiguousarray(inn[:, cols])
        bb = None if bb is None else np.ascontiguousarray(bb[cols])
        y = y[:, torch.from_numpy(cols).to(y.device)]
    yref, yd = oracle.C.linear_f16(x.numpy(), bn, inn, cache.numpy(), G, bb)
    if b is not None:
        # bias is added after rounding; judge the pre-bias part through the fp16 reference too
        yd = yref.astype(np.float64)
        rms = float(np.sqrt(np.mean(yd ** 2)))
        diff = np.abs(y.float().cpu().numpy().astype(np.float64) - yd)
        assert diff.max() <= 2.0 ** -9 * max(np.abs(yd).max(), rms), f"bias case off by {diff.max()}"
        return
    if ran == ROWS32:
        return check_rounded(oracle, y, yd, (x.numpy(), bn, inn, cache.numpy(), G), rounding,
                             f"N={N} K={K} S={S} G={G} M={M} L={L} flags={flags} (32-row kernel)")
    return check(y, yd, f"N={N} K={K} S={S} G={G} M={M} L={L} flags={flags}")


@pytest.mark.parametrize("S", [2, 3, 4])
@pytest.mark.parametrize("G", [128, 256])
def test_small_m1(oracle, S, G):
    run_case(oracle, 256, 1024, S, G, 1, 200)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 16])
def test_batch(oracle, M):
    run_case(oracle, 512, 1024, 4, 128, M, 256, seed=3)


def test_u16_index(oracle):
    run_case(oracle, 320, 768, 4, 128, 1, 300, seed=4)
    run_case(oracle, 320, 768, 3, 128, 2, 5000, seed=5)


def test_bias(oracle):
    run_case(oracle, 512, 512, 4, 128, 1, 256, seed=6, bias=True)
    run_case(oracle, 512, 512, 2, 128, 4, 256, seed=7, bias=True)


@pytest.mark.parametrize("N", [16, 48, 1000, 1030])
def test_ragged_n(oracle, N):
    run_case(oracle, N, 512, 4, 128, 1, 64, seed=8)
    run_case(oracle, N, 512, 4, 128, 3, 64, seed=9)


def test_config1_4096(oracle):
    run_case(oracle, 4096, 4096, 4, 128, 1, 256, seed=10)


@pytest.mark.parametrize("N,K", [(1024, 4096), (14336, 4096), (4096, 14336)])
def test_llama_shapes(oracle, N, K):
    run_case(oracle, N, K, 4, 128, 1, 256, seed=11)


@pytest.mark.parametrize("N,S,M,L,bias", [(28672, 4, 1, 256, False), (28672, 2, 3, 256, False), (28672, 3, 4, 300, False),
                                          (27000, 4, 2, 256, False), (26000, 4, 1, 300, True), (28672, 8, 1, 256, False)])
def test_one_window_per_cu_up_to_seven_tiles(oracle, N, S, M, L, bias):
    # the fused gate|up width: on 256 CUs one workgroup per CU takes all of K for a window of 104-112 columns
    # (7 column tiles, the last one partly its neighbour's at 104; at 27000 the last window is moved left)
    run_case(oracle, N, 4096, S, 128, M, L, seed=N + S + M, bias=bias)


@pytest.mark.parametrize("S", [2, 3, 4])
@pytest.mark.parametrize("M", [2, 16])
def test_sweep_gate(oracle, S, M):
    run_case(oracle, 14336, 4096, S, 128, M, 256, seed=12)


@pytest.mark.parametrize("S", [2, 3, 4])
@pytest.mark.parametrize("M", [4, 8])
def test_sweep_down(oracle, S, M):
    """The other shape of the batch / plane sweep: 14336 -> 4096, long K (split across workgroups)."""
    run_case(oracle, 4096, 14336, S, 128, M, 256, seed=14)


@pytest.mark.parametrize("flags", [0, 2])
def test_sweep_down_16_rows(oracle, flags):
    """16 rows at the down shape.  Default: the 32-row kernel, K in two parts.  flags = 2: the decode kernel, four
    row tiles, K split 14 ways through the accumulators."""
    run_case(oracle, 4096, 14336, 4, 128, 16, 256, seed=15, flags=flags)


@pytest.mark.parametrize("S", [2, 3, 4])
def test_sweep_gate_16_rows_decode_kernel(oracle, S):
    run_case(oracle, 14336, 4096, S, 128, 16, 256, seed=12, flags=2)


@pytest.mark.parametrize("M,flags", [(5, 0), (6, 0), (7, 0), (8, 0), (9, 0), (9, 2), (12, 0), (12, 2), (13, 0), (13, 2),
                                     (16, 0), (16, 2)])
@pytest.mark.parametrize("N", [32, 48, 64, 100, 1000, 1030])
def test_batch_rows_ragged_n(oracle, M, N, flags):
    """5..16 rows: the waves of a workgroup share the activation operands of a sub-group and split its
    columns.  Windows that end inside a tile, windows moved left at the edge of N, and (N below 64 with more
    than 8 rows) the shapes that fall back to one wave per sub-group."""
    from sbvr import hip
    run_case(oracle, N, 512, 4, 128, M, 64, seed=300 + M + N, flags=flags)
    assert hip.last_kernel() == (DECODE if M <= 8 or flags == 2 else ROWS32)


@pytest.mark.parametrize("flags", [0, 2])
@pytest.mark.parametrize("S", [2, 3, 6, 8])
@pytest.mark.parametrize("M", [7, 11])
def test_batch_rows_planes(oracle, S, M, flags):
    run_case(oracle, 384, 1024, S, 128, M, 200, seed=320 + S + M, flags=flags)


@pytest.mark.parametrize("flags", [0, 2])
@pytest.mark.parametrize("G", [128, 256, 512])
@pytest.mark.parametrize("M", [8, 16])
def test_batch_rows_groups(oracle, G, M, flags):
    run_case(oracle, 512, 2048, 4, G, M, 256, seed=340 + G + M, flags=flags)


@pytest.mark.parametrize("flags", [0, 2])
def test_batch_rows_u16_index_bias_and_scales(oracle, flags):
    run_case(oracle, 320, 768, 4, 128, 6, 3000, seed=350, flags=flags)
    run_case(oracle, 320, 768, 3, 128, 14, 5000, seed=351, bias=True, flags=flags)
    run_case(oracle, 320, 768, 4, 128, 10, 256, seed=352, xscale=100.0, flags=flags)
    run_case(oracle, 320, 768, 4, 128, 5, 256, seed=353, xscale=1e-3, flags=flags)


def test_batch_rows_of_different_magnitude(oracle):
    """Each batch row has its own scale per sub-group: a row 2^12 times larger than its neighbours, and a
    zero row, leave the others exact."""
    import sbvr
    from sbvr import synth
    dev = _dev()
    N, K, S, G, M = 256, 1024, 4, 128, 12
    bvr, idx, cache = synth.random_encoding(N, K, S, G, 256, seed=360)
    x = torch.randn((M, K), generator=torch.Generator().manual_seed(361))
    x[3] *= 4096.0
    x[5] = 0.0
    x[9] *= 1e-3
    x = x.to(torch.float16)
    from sbvr import hip
    _, yd = oracle.C.linear_f16(x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), G)
    _, yd1 = oracle.C.linear_f16(x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), G, mode=1)
    # flags = 2: the decode kernel of 5..16 rows (exact); default: the 32-row kernel (weights rounded to fp16 as
    # decode() rounds them)
    for flags, rounding in ((2, parity.ROUNDING_EXACT), (0, parity.ROUNDING_DECODE)):
        y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None, bvr_len=G, flags=flags)
        assert hip.last_rounding() == rounding
        got = y.float().cpu().numpy()
        for m in range(M):           # row by row: each against its own RMS
            if m == 5:
                assert float(y[m].float().abs().max()) == 0.0
            else:
                parity.judge(got[m:m + 1], yd[m:m + 1], yd1[m:m + 1], rounding, f"row {m}, flags {flags}")


def test_batch_rows_repeatable(oracle):
    """Split K through the accumulators: the same bits on every call, and the workspace left clean."""
    import sbvr
    from sbvr import synth
    dev = _dev()
    N, K, M = 1024, 4096, 16
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(N, K, 4, 128, 256, seed=370))
    x = torch.randn((M, K), generator=torch.Generator().manual_seed(371)).to(torch.float16).to(dev)
    for flags in (2, 0):         # the decode kernel of 5..16 rows; the 32-row kernel, K in two parts
        first = sbvr._sbvr_linear_f16(x, bvr, idx, cache, None, bvr_len=128, flags=flags)
        for _ in range(5):
            again = sbvr._sbvr_linear_f16(x, bvr, idx, cache, None, bvr_len=128, flags=flags)
            assert torch.equal(first, again)


def test_portable_kernel(oracle):
    run_case(oracle, 100, 512, 4, 128, 1, 256, seed=13, flags=1)
    run_case(oracle, 96, 320, 5, 64, 3, 40, seed=14)       # no MFMA kernel for G=64 / S=5
    run_case(oracle, 64, 256, 4, 32, 1, 16, seed=15)


def test_large_and_small_activations(oracle):
    run_case(oracle, 256, 1024, 4, 128, 2, 256, seed=16, xscale=100.0)
    run_case(oracle, 256, 1024, 4, 128, 2, 256, seed=17, xscale=1e-3)


def test_outlier_activation(oracle):
    """One huge activation in a group must not wreck the other groups."""
    import sbvr
    from sbvr import synth
    dev = _dev()
    N, K, S, G = 256, 1024, 4, 128
    bvr, idx, cache = synth.random_encoding(N, K, S, G, 256, seed=18)
    x = torch.randn((1, K), generator=torch.Generator().manual_seed(19)).to(torch.float16)
    x[0, 5] = 2000.0
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None, bvr_len=G)
    _, yd = oracle.C.linear_f16(x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), G)
    check(y, yd, "outlier")


def test_golden_real_encodings(oracle, golden):
    """Encodings produced by the reference's own encoder."""
    import sbvr
    dev = _dev()
    for name in ["default_s2", "default_s3", "default_s4", "weights_s4", "pad_s2"]:
        g = golden(name)
        bvr, idx, cache = (torch.from_numpy(g[k]) for k in ("bvr", "coeff_idx", "coeff_cache"))
        K = bvr.shape[0] * 32
        x = torch.randn((2, K), generator=torch.Generator().manual_seed(1)).to(torch.float16)
        y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None,
                                  bvr_len=int(g["bvr_len"]))
        _, yd = oracle.C.linear_f16(x.numpy(), g["bvr"], g["coeff_idx"], g["coeff_cache"], int(g["bvr_len"]))
        check(y, yd, name)
        # and against x @ decode(W)^T with the reference's own decode() output
        w = g["decoded"].astype(np.float64)
        yd2 = x.numpy().astype(np.float64)[:, :w.shape[1]] @ w.T
        if w.shape[1] == K:
            rms = np.sqrt(np.mean(yd2 ** 2))
            assert np.abs(y.float().cpu().numpy() - yd2).max() <= 1e-2 * max(np.abs(yd2).max(), rms)


def test_closed_form_all_ones(oracle):
    """All planes set: y[n] = sum_g (sum_j c_j) * sum_{k in g} x[k]."""
    import sbvr
    dev = _dev()
    N, K, S, G, L = 64, 512, 4, 128, 7
    bvr = torch.full((K // 32, N, S), -1, dtype=torch.int32).view(torch.uint32)
    gen = torch.Generator().manual_seed(20)
    idx = torch.randint(0, L, (K // G, N), generator=gen).to(torch.uint8)
    cache = (torch.randn((L, S), generator=gen) * 0.05).to(torch.float16)
    x = torch.randn((1, K), generator=gen).to(torch.float16)
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None, bvr_len=G)
    gs = x.double().view(K // G, G).sum(1)                       # (Kg,)
    cs = cache.double().sum(1)[idx.long()]                       # (Kg, N)
    yd = (gs[:, None] * cs).sum(0)[None, :].numpy()
    check(y, yd, "all ones")


def test_repeatable_and_workspace_clean(oracle):
    import sbvr
    from sbvr import synth
    dev = _dev()
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(4096, 4096, 4, 128, 256, seed=21))
    x = torch.randn((1, 4096), generator=torch.Generator().manual_seed(22)).to(torch.float16).to(dev)
    ys = [sbvr._sbvr_linear_f16(x, bvr, idx, cache, None, bvr_len=128).clone() for _ in range(5)]
    torch.cuda.synchronize()
    for y in ys[1:]:
        assert torch.equal(y, ys[0]), "results differ between identical calls"
    # a different shape in between must not disturb the shared workspace
    b2, i2, c2 = (t.to(dev) for t in synth.random_encoding(1024, 2048, 4, 128, 256, seed=23))
    x2 = torch.randn((3, 2048), generator=torch.Generator().manual_seed(24)).to(torch.float16).to(dev)
    y2a = sbvr._sbvr_linear_f16(x2, b2, i2, c2, None, bvr_len=128).clone()
    y1 = sbvr._sbvr_linear_f16(x, bvr, idx, cache, None, bvr_len=128).clone()
    y2b = sbvr._sbvr_linear_f16(x2, b2, i2, c2, None, bvr_len=128).clone()
    assert torch.equal(y1, ys[0]) and torch.equal(y2a, y2b)


def test_linearity_full_size(oracle):
    """f(x1) + f(x2) = f(x1 + x2) at the gate shape, with x1, x2 chosen so that the
    sum is exact in fp16 (a size-independent property; no oracle run needed)."""
    import sbvr
    from sbvr import synth
    dev = _dev()
    N, K = 14336, 4096
    bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(N, K, 4, 128, 256, seed=25))
    gen = torch.Generator().manual_seed(26)
    x1 = (torch.randint(-64, 64, (1, K), generator=gen).float() / 32).to(torch.float16)
    x2 = (torch.randint(-64, 64, (1, K), generator=gen).float() / 32).to(torch.float16)
    f = lambda v: sbvr._sbvr_linear_f16(v.to(dev), bvr, idx, cache, None, bvr_len=128).float()
    y1, y2, y12 = f(x1), f(x2), f(x1 + x2)
    rms = y12.pow(2).mean().sqrt()
    assert ((y1 + y2 - y12).abs().max() <= 3 * 2.0 ** -10 * torch.maximum(y12.abs().max(), rms)).item()
