"""The linear's one-row entry points that fold SiLU(gate) * up, or the residual
add and RMSNorm, into the activation load (sbvr_hip_linear_f16_swiglu,
sbvr_hip_linear_f16_add_rmsnorm), through the C ABI against the CPU oracle.

The activation row is restated here in numpy with the kernel's roundings
(each intermediate is an fp16 value); the oracle's linear of that row is the
reference for the output, with the tolerance of test_gpu_linear_parity.py
(1e-2 relative, small outputs judged against the RMS).  The norm's sum of
squares is added up in another order on the GPU, so the kernel's row may
differ from numpy's in the last fp16 bit of a few elements: that stays far
inside the tolerance.  x_out of the add + norm entry point is one rounded
addition per element and must match bit for bit."""
import numpy as np
import pytest
import torch

from test_gpu_linear_parity import _dev, check

pytestmark = pytest.mark.gpu

f16, f32 = np.float16, np.float32


def swiglu_row(gate_up):
    k = gate_up.shape[1] // 2
    g = gate_up[:, :k].astype(f32)
    u = gate_up[:, k:].astype(f32)
    act = (g / (f32(1) + np.exp(-g))).astype(f16)
    return (act.astype(f32) * u).astype(f16)


def add_norm_row(x, delta, w, eps):
    r = (x.astype(f32) + delta.astype(f32)).astype(f16)
    var = np.mean(r.astype(np.float64) ** 2)
    inv = f32(1.0 / np.sqrt(var + eps))
    n = (r.astype(f32) * inv).astype(f16)
    return r, (w.astype(f32) * n.astype(f32)).astype(f16)


def encoding(N, K, S, G, L, seed):
    from sbvr import synth
    return synth.random_encoding(N, K, S, G, L, seed=seed)


@pytest.mark.parametrize("N,K,S,L", [
    (4096, 14336, 4, 256),      # the 8B down projection
    (256, 512, 2, 64), (1000, 1024, 3, 300), (48, 128, 4, 16), (8192, 3584, 4, 256),
])
def test_swiglu(oracle, N, K, S, L):
    import sbvr
    dev = _dev()
    bvr, idx, cache = encoding(N, K, S, 128, L, seed=N + K)
    gen = torch.Generator().manual_seed(K)
    gate_up = (torch.randn((1, 2 * K), generator=gen) * 1.5).to(torch.float16)
    y = sbvr._sbvr_linear_f16_swiglu(gate_up.to(dev), bvr.to(dev), idx.to(dev), cache.to(dev), bvr_len=128)
    torch.cuda.synchronize()
    row = swiglu_row(gate_up.numpy())
    _, yd = oracle.C.linear_f16(row, bvr.numpy(), idx.numpy(), cache.numpy(), 128, None)
    check(y, yd, f"swiglu N={N} K={K} S={S}")
    # and the two-launch form gives the same row to the same kernel: identical bits
    act = torch.empty((1, K), dtype=torch.float16, device=dev)
    from sbvr import hip
    hip.dec_silu_mul(gate_up.to(dev), act)
    y2 = sbvr._sbvr_linear_f16(act, bvr.to(dev), idx.to(dev), cache.to(dev), bvr_len=128)
    assert torch.equal(y, y2), "fused and two-launch SwiGLU disagree"


@pytest.mark.parametrize("N,K,S,L", [
    (6144, 4096, 4, 768),       # the 8B fused q|k|v (three tables, uint16 indices)
    (28672, 4096, 4, 512),      # the 8B fused gate|up
    (256, 128, 4, 32), (1000, 1024, 3, 300), (512, 8192, 2, 256), (320, 2304, 4, 100), (64, 16384, 4, 256),
])
def test_add_rmsnorm(oracle, N, K, S, L):
    import sbvr
    dev = _dev()
    bvr, idx, cache = encoding(N, K, S, 128, L, seed=N + K + 1)
    gen = torch.Generator().manual_seed(N)
    x = (torch.randn((1, K), generator=gen) * 2.0).to(torch.float16)
    delta = (torch.randn((1, K), generator=gen) * 0.7).to(torch.float16)
    w = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(torch.float16)
    eps = 1e-5
    x_out = torch.full((1, K), float("nan"), dtype=torch.float16, device=dev)
    y = sbvr._sbvr_linear_f16_add_rmsnorm(x.to(dev), delta.to(dev), w.to(dev), eps, x_out, bvr.to(dev), idx.to(dev),
                                          cache.to(dev), bvr_len=128)
    torch.cuda.synchronize()
    r, row = add_norm_row(x.numpy(), delta.numpy(), w.numpy(), eps)
    assert np.array_equal(x_out.cpu().numpy().view(np.uint16), r.view(np.uint16)), "x_out is not fp16(x + delta)"
    _, yd = oracle.C.linear_f16(row, bvr.numpy(), idx.numpy(), cache.numpy(), 128, None)
    check(y, yd, f"add_rmsnorm N={N} K={K} S={S}")


def test_add_rmsnorm_repeats_and_leaves_inputs(oracle):
    """Two calls in a row (the split-K accumulators are shared) give the same bits; x and delta are untouched."""
    import sbvr
    dev = _dev()
    N, K = 6144, 4096
    bvr, idx, cache = (t.to(dev) for t in encoding(N, K, 4, 128, 768, seed=1))
    gen = torch.Generator().manual_seed(3)
    x = torch.randn((1, K), generator=gen).to(torch.float16).to(dev)
    delta = torch.randn((1, K), generator=gen).to(torch.float16).to(dev)
    w = torch.ones((K,), dtype=torch.float16, device=dev)
    x0, d0 = x.clone(), delta.clone()
    x_out = torch.empty_like(x)
    a = sbvr._sbvr_linear_f16_add_rmsnorm(x, delta, w, 1e-5, x_out, bvr, idx, cache, bvr_len=128).clone()
    b = sbvr._sbvr_linear_f16_add_rmsnorm(x, delta, w, 1e-5, x_out, bvr, idx, cache, bvr_len=128)
    assert torch.equal(a, b)
    assert torch.equal(x, x0) and torch.equal(delta, d0)


def test_rejections():
    import sbvr
    from sbvr.hip import SbvrHipError
    dev = _dev()
    bvr, idx, cache = (t.to(dev) for t in encoding(256, 512, 4, 128, 64, seed=2))
    x = torch.zeros((1, 512), dtype=torch.float16, device=dev)
    w = torch.ones((512,), dtype=torch.float16, device=dev)
    with pytest.raises(SbvrHipError):       # x_out aliases x
        sbvr._sbvr_linear_f16_add_rmsnorm(x, x.clone(), w, 1e-5, x, bvr, idx, cache, bvr_len=128)
    with pytest.raises(SbvrHipError):       # two rows
        sbvr._sbvr_linear_f16_swiglu(torch.zeros((2, 1024), dtype=torch.float16, device=dev), bvr, idx, cache,
                                     bvr_len=128)
    b96, i96, c96 = (t.to(dev) for t in encoding(256, 96 * 4, 4, 96, 64, seed=2))
    with pytest.raises(SbvrHipError):       # a group length the decode kernel does not take
        sbvr._sbvr_linear_f16_swiglu(torch.zeros((1, 768), dtype=torch.float16, device=dev), b96, i96, c96,
                                     bvr_len=96)
