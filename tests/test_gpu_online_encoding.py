"""Activations encoded on the fly (profile_input / _online_tranfrom / online_mm_T): the reference names
these methods and leaves the two run-time ones empty (sbvr/core.py:971-1027), so there is no reference
output to compare with.  What pins them here: the selector rule is the encoder's (core.py:492-494:
nearest subset sum, first on ties, fp16 difference and square), restated in numpy below; the encoded
activations decode (oracle) to the points chosen; and the product is the both-encoded operator's
(oracle.C.mm_T) on those arrays, which in turn approximates x @ W^T."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def nearest_selectors(x, points, G):
    """x (M, K) fp16, points (K/G, P) fp16 -> selector per element (first minimum of the fp16 squares)."""
    M, K = x.shape
    sel = np.zeros((M, K), dtype=np.int64)
    for g in range(K // G):
        seg = x[:, g * G:(g + 1) * G]
        diff = (seg[:, :, None] - points[g][None, None, :]).astype(np.float16)
        sq = (diff * diff).astype(np.float16)
        sel[:, g * G:(g + 1) * G] = sq.argmin(axis=-1)
    return sel


def pack(sel, S):
    """(M, K) selectors -> (K/32, M, S) uint32 planes, bit k%32 of word k/32; plane j is bit S-1-j of the
    selector (the subset sums count their coefficients most significant first, core.py:345-351)."""
    M, K = sel.shape
    out = np.zeros((K // 32, M, S), dtype=np.uint32)
    for j in range(S):
        bits = ((sel >> (S - 1 - j)) & 1).astype(np.uint32).reshape(M, K // 32, 32)
        out[:, :, j] = (bits << np.arange(32, dtype=np.uint32)).sum(axis=-1, dtype=np.uint64).astype(np.uint32).T
    return out


@pytest.mark.parametrize("S,G,M,K", [(2, 128, 3, 512), (4, 32, 1, 96), (4, 128, 5, 4096), (8, 256, 2, 512), (3, 64, 4, 192)])
def test_online_encode_kernel(S, G, M, K):
    from sbvr import hip
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(S * 1000 + K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    x[0, :4] = [0.0, 100.0, -100.0, 1e-4]
    points = (rng.standard_normal((K // G, 1 << S)) * 1.5).astype(np.float16)
    points[0, 1] = points[0, 0]                      # a tie: the first of two equal points wins
    bvr = hip.online_encode(torch.from_numpy(x).to(dev), torch.from_numpy(points).to(dev), G).cpu().numpy()
    assert bvr.shape == (K // 32, M, S) and bvr.dtype == np.uint32
    assert np.array_equal(bvr, pack(nearest_selectors(x, points, G), S))


@pytest.mark.parametrize("S_in", [4, None])
def test_profile_input_and_online_mm_T(oracle, S_in):
    """None: the reference's default of 8 input planes (core.py:982-983)."""
    import sbvr
    dev = torch.device("cuda:0")
    N, K, G = 64, 512, 128
    gen = torch.Generator().manual_seed(31)
    w = (torch.randn((N, K), generator=gen) * 0.02).to(torch.float16)
    obj = sbvr.sbvr(w.to(dev), encoder_config={"num_sums": 4, "bvr_len": G}, device=dev, verbose_level=0)
    samples = torch.randn((24, K), generator=gen).to(torch.float16)
    with pytest.raises(RuntimeError):
        obj.online_mm_T(samples[:1].to(dev))
    obj.profile_input(samples.to(dev), None if S_in is None else {"num_sums": S_in})
    S = 8 if S_in is None else S_in
    assert obj.input_num_sums == S and tuple(obj.input_coeff.shape) == (K // G, S)

    x = torch.randn((2, K), generator=gen).to(torch.float16)
    l_bvr, l_idx, l_cache = obj._online_tranfrom(x.to(dev))
    assert tuple(l_bvr.shape) == (K // 32, 2, S) and tuple(l_idx.shape) == (K // G, 2)
    lb, li, lc = l_bvr.cpu().numpy(), l_idx.cpu().numpy(), l_cache.cpu().numpy()
    assert np.array_equal(li, np.repeat(np.arange(K // G, dtype=li.dtype)[:, None], 2, axis=1))
    # every element carries the nearest subset sum of its group's line
    combs = ((np.arange(1 << S)[:, None] >> np.arange(S - 1, -1, -1)[None, :]) & 1).astype(np.float64)
    points = (l_cache.float().cpu().numpy().astype(np.float64) @ combs.T).astype(np.float16)
    assert np.array_equal(lb, pack(nearest_selectors(x.numpy(), points, G), S))
    x_hat = oracle.C.decode(lb, li, lc, G).astype(np.float64)
    err = ((x_hat - x.numpy().astype(np.float64)) ** 2).mean() / x.numpy().astype(np.float64).var()
    assert err < (0.03 if S == 4 else 0.003), err          # 16 / 256 levels fitted to the samples

    y = obj.online_mm_T(x.to(dev)).float().cpu().numpy().astype(np.float64)
    rb, ri, rc = (t.cpu().numpy() for t in (obj.bvr.data, obj.coeff_idx.data, obj.coeff_cache.data))
    _, yd = oracle.C.mm_T(lb, li, lc, rb, ri, rc, G)
    rms = float(np.sqrt(np.mean(yd ** 2)))
    assert (np.abs(y - yd) / np.maximum(np.abs(yd), 1e-2 * rms)).max() <= 1e-2
    # and stands for x @ W^T up to the two quantisations
    dense = x.numpy().astype(np.float64) @ w.numpy().astype(np.float64).T
    assert np.mean((y - dense) ** 2) < (0.06 if S == 4 else 0.03) * np.mean(dense ** 2)


def test_input_coefficients_survive_save_and_load(tmp_path):
    import sbvr
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(41)
    w = (torch.randn((16, 256), generator=gen) * 0.02).to(torch.float16)
    obj = sbvr.sbvr(w.to(dev), encoder_config={"num_sums": 2, "bvr_len": 128}, device=dev, verbose_level=0)
    obj.profile_input(torch.randn((8, 256), generator=gen).to(torch.float16).to(dev), {"num_sums": 3})
    path = str(tmp_path / "with_input.pt")
    obj.save(path)
    back = sbvr.load(path, device=dev, verbose_level=0)
    assert back.input_num_sums == 3 and torch.equal(back.input_coeff.data, obj.input_coeff.data)
    x = torch.randn((1, 256), generator=gen).to(torch.float16).to(dev)
    assert torch.equal(back.online_mm_T(x), obj.online_mm_T(x))
