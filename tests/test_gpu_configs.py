"""The benchmark configurations at their full shapes, on the default dispatch (no flags),
against the oracle.  Output columns are independent of each other, so at shapes where the
oracle over the whole matrix would take minutes it is run on a sample of the columns
(`bvr[:, cols, :]`, `coeff_idx[:, cols]`): exact for those columns, and cheap.

  config 3  gate 4096 -> 14336 and down 14336 -> 4096, batch 1, 2, 4, 8, 16 x 2, 3, 4 planes
  config 5  prefill at 8192 -> 28672 and 28672 -> 8192, 256 .. 2048 rows
  reference-made encodings (tests/golden) through the MFMA kernels, in every layout the
  reference's constructor flags select (default uint32, cpu_kernel_v2 uint8, cpu_kernel 16-lane)
"""
import numpy as np
import pytest
import torch

import parity

pytestmark = pytest.mark.gpu

PORTABLE, DECODE, ROWS32, PREFILL, PREFILL_SPLIT = 1, 2, 3, 4, 5


def _dev():
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch.device("cuda:0")


def sampled_oracle(oracle, x, bvr, idx, cache, G, cols, rows, rounding):
    """Oracle outputs (double, unrounded) for the given rows of x and columns of the weight: over unrounded
    weights, and (for the kernels that round weights) over weights rounded as decode() rounds them."""
    xs, bs, ix = np.ascontiguousarray(x[rows]), np.ascontiguousarray(bvr[:, cols, :]), np.ascontiguousarray(idx[:, cols])
    _, yd0 = oracle.C.linear_f16(xs, bs, ix, cache, G)
    yd1 = None
    if rounding != parity.ROUNDING_EXACT:
        _, yd1 = oracle.C.linear_f16(xs, bs, ix, cache, G, mode=1)
    return yd0, yd1


@pytest.mark.parametrize("S", [2, 3, 4])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("shape", ["gate", "down"])
def test_config3_batch_plane_sweep(oracle, shape, M, S):
    import sbvr
    from sbvr import hip, synth
    dev = _dev()
    N, K = (14336, 4096) if shape == "gate" else (4096, 14336)
    bvr, idx, cache = synth.random_encoding(N, K, S, 128, 256, seed=100 + S)
    x = torch.randn((M, K), generator=torch.Generator().manual_seed(200 + M)).to(torch.float16)
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None, bvr_len=128)
    kernel = hip.last_kernel()
    # up to 8 rows the decode kernels (exact in weights and activations); 16 rows: the 32-row kernel
    want = DECODE if M <= 8 else ROWS32
    assert kernel == want, f"{shape} M={M} S={S}: kernel {kernel} ran, {want} expected"
    rng = np.random.default_rng(M * 10 + S)
    cols = np.sort(rng.choice(N, size=384, replace=False))
    cols[:4] = [0, 1, N // 2, N - 1]           # (edges of the first and the last window always)
    cols = np.unique(cols)
    rounding = hip.last_rounding()
    # (16 rows: the table look-up kernel, whose weights are decode()'s bit for bit)
    assert rounding == (parity.ROUNDING_EXACT if M <= 8 else parity.ROUNDING_DECODE)
    yd0, yd1 = sampled_oracle(oracle, x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), 128, cols, np.arange(M), rounding)
    parity.judge(y.float().cpu().numpy()[:, cols], yd0, yd1, rounding, f"{shape} M={M} S={S}")


@pytest.mark.parametrize("N,K", [(28672, 8192), (8192, 28672)])
def test_config5_prefill_70b_width(oracle, N, K):
    """256, 512, 1024 and 2048 rows at both 70B-width shapes, S = 4, G = 128: 64 sampled columns
    x 8 sampled rows against the oracle, for every M (and whichever of the split / unsplit prefill
    launches the shape takes)."""
    import sbvr
    from sbvr import hip, synth
    dev = _dev()
    bvr, idx, cache = synth.random_encoding(N, K, 4, 128, 256, seed=300)
    dbvr, didx, dcache = bvr.to(dev), idx.to(dev), cache.to(dev)
    rng = np.random.default_rng(N)
    cols = np.unique(np.concatenate([rng.choice(N, size=60, replace=False), [0, 127, 128, N - 1]]))
    lib = hip._load()
    for M in (256, 512, 1024, 2048):
        x = torch.randn((M, K), generator=torch.Generator().manual_seed(400 + M)).to(torch.float16)
        y = sbvr._sbvr_linear_f16(x.to(dev), dbvr, didx, dcache, None, bvr_len=128)
        kernel = hip.last_kernel()
        split = lib.sbvr_hip_linear_f16_workspace(M, N, K, 4, 128) > 0
        assert kernel == (PREFILL_SPLIT if split else PREFILL), f"N={N} K={K} M={M}: kernel {kernel}"
        rows = np.unique(np.concatenate([rng.choice(M, size=6, replace=False), [0, M - 1]]))
        rounding = hip.last_rounding()
        assert rounding == parity.ROUNDING_DECODE, "4 planes, groups of 128: the table look-up prefill kernel"
        yd0, yd1 = sampled_oracle(oracle, x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), 128, cols, rows, rounding)
        got = y[torch.from_numpy(rows).to(dev)][:, torch.from_numpy(cols).to(dev)].float().cpu().numpy()
        # the RMS that the error is judged against is that of the whole output
        rms_all = float(y.float().pow(2).mean().sqrt())
        parity.judge(got, yd0, yd1, rounding, f"N={N} K={K} M={M}", rms=rms_all)
        del x, y
    torch.cuda.empty_cache()


@pytest.mark.parametrize("M,kernel", [(1, DECODE), (4, DECODE), (8, DECODE), (16, ROWS32), (20, ROWS32), (48, PREFILL)])
def test_reference_encoding_through_mfma_kernels(oracle, golden, M, kernel):
    """A 64 x 512 weight encoded by the reference's own encoder (4 planes, its group length of 256):
    enough columns for the MFMA kernels, which the smaller fixtures never reach."""
    import sbvr
    from sbvr import hip
    dev = _dev()
    g = golden("weights_s4_n64")
    G = int(g["bvr_len"])
    bvr, idx, cache = (torch.from_numpy(g[k]).to(dev) for k in ("bvr", "coeff_idx", "coeff_cache"))
    K = bvr.shape[0] * 32
    x = torch.randn((M, K), generator=torch.Generator().manual_seed(500 + M)).to(torch.float16)
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr, idx, cache, None, bvr_len=G)
    assert hip.last_kernel() == kernel
    rounding = hip.last_rounding()
    assert rounding == (parity.ROUNDING_EXACT if kernel == DECODE else parity.ROUNDING_DECODE)
    _, yd0 = oracle.C.linear_f16(x.numpy(), g["bvr"], g["coeff_idx"], g["coeff_cache"], G)
    _, yd1 = oracle.C.linear_f16(x.numpy(), g["bvr"], g["coeff_idx"], g["coeff_cache"], G, mode=1)
    parity.judge(y.float().cpu().numpy(), yd0, yd1, rounding, f"reference encoding, M={M}")
    # and against x @ decode(W)^T with the reference's own decode() output
    w = g["decoded"].astype(np.float64)
    yd2 = x.numpy().astype(np.float64) @ w.T
    rms = np.sqrt(np.mean(yd2 ** 2))
    assert np.abs(y.float().cpu().numpy() - yd2).max() <= 1e-2 * max(np.abs(yd2).max(), rms)
    if rounding == parity.ROUNDING_DECODE:
        # the table look-up kernels use exactly these weights: only the order of the fp32 sums is left
        parity.tight(y.float().cpu().numpy(), yd2, f"reference encoding, M={M}, against x @ decode()^T")


@pytest.mark.parametrize("fixture,flag", [("v1_s2", "cpu_kernel"), ("v2_s2", "cpu_kernel_v2"), ("default_s4", None)])
@pytest.mark.parametrize("M", [1, 4, 16, 48])
def test_uint8_layout_objects_through_sbvrlinear(oracle, golden, fixture, flag, M):
    """Objects in the layouts the reference's `cpu_kernel` (16-lane uint8) and `cpu_kernel_v2`
    (uint8 words) flags select, with the arrays its encoder made, through SBVRLinear.from_sbvr:
    the layer re-words them to the uint32 layout the kernels read."""
    import sbvr
    from sbvr import hip
    dev = _dev()
    g = golden(fixture)
    G = int(g["bvr_len"])
    enc = sbvr.sbvr.from_parts(*(torch.from_numpy(g[k]).to(dev) for k in ("bvr", "coeff_idx", "coeff_cache")), G,
                               original_shape=g["data"].shape)
    assert enc.is_v1_layout() == (flag == "cpu_kernel")
    assert enc.bvr.dtype == (torch.uint8 if flag else torch.uint32)
    layer = sbvr.SBVRLinear.from_sbvr(enc)
    N, K = g["data"].shape
    x = torch.randn((M, K), generator=torch.Generator().manual_seed(600 + M)).to(torch.float16)
    y = layer(x.to(dev))
    kernel = hip.last_kernel()
    # 32 columns reach the decode kernel; the 4- and 8-column fixtures are below its 16 columns
    # (up to 4 rows then take the portable kernel, 5..32 the 32-row kernel, which has no such limit)
    if N >= 16:
        # (16 rows: the 32-row kernel; its table look-up form wants groups of a multiple of 64 elements, which these have)
        assert kernel == {1: DECODE, 4: DECODE, 16: ROWS32, 48: PREFILL}[M]
    else:
        assert kernel == {1: PORTABLE, 4: PORTABLE, 16: ROWS32, 48: PREFILL}[M]
    # The oracle reads the default uint32 layout; the fixture is re-worded for it here, in numpy, from
    # the layouts as the reference defines them (sbvr/core.py:753-780), not by this package's layout code:
    # 16-lane: bvr[row // 16, byte of K, plane, row % 16]; uint8 words: bvr[byte of K, row, plane];
    # a uint32 word is four consecutive bytes of K, the first one lowest.
    raw = g["bvr"]
    if flag == "cpu_kernel":
        raw = raw.transpose(1, 0, 3, 2).reshape(raw.shape[1], raw.shape[0] * 16, raw.shape[2])    # -> (K/8, N, S)
    if flag:
        kb, n_rows, planes = raw.shape
        quad = raw.reshape(kb // 4, 4, n_rows, planes).astype(np.uint32)
        raw = quad[:, 0] | (quad[:, 1] << 8) | (quad[:, 2] << 16) | (quad[:, 3] << 24)
    dflt = np.ascontiguousarray(raw)
    assert np.array_equal(dflt, enc.default_layout(torch.uint32).cpu().numpy()), "re-wording disagrees with the layout's definition"
    rounding = hip.last_rounding()
    _, yd0 = oracle.C.linear_f16(x.numpy(), dflt, g["coeff_idx"], g["coeff_cache"], G)
    _, yd1 = oracle.C.linear_f16(x.numpy(), dflt, g["coeff_idx"], g["coeff_cache"], G, mode=1)
    parity.judge(y.float().cpu().numpy(), yd0, yd1, rounding, f"{fixture} M={M}")
    # independent of this package's re-wording: x @ data^T is close to the encoded product (S = 2: coarse),
    # and for the 3-D layouts the reference's decode() output gives the exact target
    if g["decoded"].size:
        yd2 = x.numpy().astype(np.float64) @ g["decoded"].astype(np.float64).T
        rms = np.sqrt(np.mean(yd2 ** 2))
        assert np.abs(y.float().cpu().numpy() - yd2).max() <= 1e-2 * max(np.abs(yd2).max(), rms)
    else:
        dense = x.numpy().astype(np.float64) @ g["data"].astype(np.float64).T
        got = y.float().cpu().numpy().astype(np.float64)
        # two planes reproduce the data to about a quarter of its variance (the reference's own log): the
        # products correlate strongly with the dense ones; a wrong lane order would give no correlation at all
        corr = np.corrcoef(dense.ravel(), got.ravel())[0, 1]
        assert corr > 0.8, f"encoded and dense products correlate only {corr:.2f}"
