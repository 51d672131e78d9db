"""Seeded random shapes through the default dispatch of the linear and of the trans=True operator, against the
oracle: batch rows 1..32, ragged N, K from one sub-group up, 2..8 planes, groups of 32..512, both index widths,
with and without bias.  Each case names the kernel that ran, so a failure says which path it was."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

KERNELS = {1: "portable", 2: "decode", 3: "rows32", 4: "prefill", 5: "prefill, K split"}


def _cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        G = int(rng.choice([32, 64, 128, 128, 128, 256, 512]))
        K = G * int(rng.integers(1, max(2, 2048 // G) + 1))
        N = int(rng.choice([16, 24, 40, 64, 72, 100, 128, 200, 256, 520, 1000, 1030, 2048]))
        S = int(rng.choice([2, 3, 4, 4, 4, 6, 8]))
        M = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 11, 12, 13, 16, 17, 24, 32]))
        L = int(rng.choice([3, 16, 256, 300, 5000]))
        out.append((N, K, S, G, M, L, bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("N,K,S,G,M,L,bias", _cases(2024, 48))
def test_linear_random_shape(oracle, N, K, S, G, M, L, bias):
    import sbvr
    from sbvr import hip, synth
    dev = torch.device("cuda:0")
    seed = N * 7 + K * 3 + S + G + M + L
    bvr, idx, cache = synth.random_encoding(N, K, S, G, L, seed=seed)
    gen = torch.Generator().manual_seed(seed + 1)
    x = torch.randn((M, K), generator=gen).to(torch.float16)
    b = (torch.randn((N,), generator=gen) * 0.3).to(torch.float16) if bias else None
    y = sbvr._sbvr_linear_f16(x.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), None if b is None else b.to(dev), bvr_len=G)
    ran = KERNELS[hip.last_kernel()]
    yref, yd = oracle.C.linear_f16(x.numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), G, None if b is None else b.numpy())
    got = y.float().cpu().numpy().astype(np.float64)
    if b is not None:
        want = yref.astype(np.float64)
        rms = float(np.sqrt(np.mean(want ** 2)))
        tol = 2.0 ** -9 if ran in ("portable", "decode") else 4e-3
        assert np.abs(got - want).max() <= tol * max(np.abs(want).max(), rms), ran
        return
    rms = float(np.sqrt(np.mean(yd ** 2))) + 1e-30
    err = np.abs(got - yd)
    if ran in ("portable", "decode"):
        assert (err / (np.maximum(np.abs(yd), rms) * 2.0 ** -10)).max() <= 2.0, ran
    else:       # weights decoded to fp16 first
        assert err.max() <= 3e-3 * rms + 2.0 ** -11 * np.abs(yd).max(), ran


def _trans_cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        G = int(rng.choice([32, 64, 64, 128, 128, 256]))
        N = G * int(rng.integers(1, max(2, 1024 // G) + 1))
        K = int(rng.choice([1, 64, 128, 128, 256, 384, 640, 1000, 1024, 2048]))
        S = int(rng.choice([2, 3, 4, 4, 4, 4, 6]))
        M = int(rng.choice([1, 1, 2, 3, 5]))
        L = int(rng.choice([2, 16, 256, 700]))
        out.append((M, N, K, S, G, L, bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("M,N,K,S,G,L,bias", _trans_cases(77, 24))
def test_row_deq_random_shape(oracle, M, N, K, S, G, L, bias):
    import sbvr
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(N * 5 + K + S + G + L)
    sel = rng.integers(0, 1 << S, size=K * N).astype(np.int32)
    bvr = oracle.C.planes_to_default(oracle.C.sel_to_planes(sel, S, 32), K, N)      # W^T: K rows of N columns
    idx = rng.integers(0, L, size=(N // G, K)).astype(np.uint8 if L <= 256 else np.uint16)
    cache = (rng.standard_normal((L, S)) * 0.5).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16) if bias else None
    t = lambda a: torch.from_numpy(a).to(dev)
    y = sbvr._sbvr_row_deq_mm_T(t(x), t(bvr), t(idx), t(cache), t(b) if bias else torch.zeros(0, dtype=torch.float16, device=dev), 0, bvr_len=G)
    want = oracle.C.row_deq_mm_T(x, bvr, idx, cache, G, b).astype(np.float64)
    d = np.abs(y.float().cpu().numpy().astype(np.float64) - want)
    assert d.max() <= 2.0 ** -9 * max(np.abs(want).max(), 1.0)
