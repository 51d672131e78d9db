"""The encoder run on the GPU, as the reference runs it (sbvr(data, device=cuda),
core.py:205-215, 655-813): the arrays it leaves on the device decode to the
nearest points of their lines, meet the error band the reference logs, and
drive the HIP operator directly."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _nearest_point_invariant(w, dec, idx, cache, G, oracle_decode_all):
    """Every element carries the point of its group's line that is nearest to it
    (core.py:492-494).  `oracle_decode_all(line)` -> the 2^S sums of a line."""
    N, K = w.shape
    for g in range(K // G):
        for n in range(N):
            pts = oracle_decode_all(cache[int(idx[g, n])])
            seg_w = w[n, g * G:(g + 1) * G].astype(np.float64)
            seg_d = dec[n, g * G:(g + 1) * G].astype(np.float64)
            best = np.abs(seg_w[:, None] - pts[None, :]).min(axis=1)
            # the search runs in fp16: allow one fp16 step of the data's magnitude
            assert np.all(np.abs(seg_w - seg_d) <= best + 2.0 ** -10 * np.maximum(np.abs(seg_w), 2.0 ** -6))


@pytest.mark.parametrize("S,G,band", [(4, 256, 0.03), (4, 128, 0.03), (2, 256, 0.30), (3, 256, 0.09)])
def test_encode_on_gpu_and_use(oracle, S, G, band):
    import sbvr
    dev = torch.device("cuda:0")
    N, K = 48, 512
    w = (torch.randn((N, K), generator=torch.Generator().manual_seed(S * 1000 + G)) * 0.02).to(torch.float16)
    enc = sbvr.sbvr(w.to(dev), encoder_config={"num_sums": S, "bvr_len": G}, device=dev, verbose_level=0)
    assert enc.bvr.data.device.type == "cuda" and enc.bvr.shape == (K // 32, N, S) and enc.bvr.dtype == torch.uint32
    assert enc.coeff_idx.shape == (K // G, N) and enc.coeff_cache.shape[1] == S

    bvr, idx, cache = (t.cpu().numpy() for t in (enc.bvr.data, enc.coeff_idx.data, enc.coeff_cache.data))
    dec = enc.decode().cpu().numpy()
    # decode() on the device agrees bit for bit with the CPU restatement of the reference's decode
    assert np.array_equal(dec.view(np.uint16), oracle.C.decode(bvr, idx, cache, G).view(np.uint16))
    # error band of the reference's own log (test.txt:30-69: S=2 0.24, S=3 6.5e-2, S=4 1.7e-2 of the variance)
    wf = w.numpy().astype(np.float64)
    rel = ((dec.astype(np.float64) - wf) ** 2).mean() / wf.var()
    assert rel < band, rel

    def all_sums(line):            # the 2^S points of a line: exact sums rounded once to fp16 (core.py:365-366)
        c = line.astype(np.float64)
        pts = [sum(c[j] for j in range(S) if (sel >> j) & 1) for sel in range(1 << S)]
        return np.array(pts, dtype=np.float64).astype(np.float16).astype(np.float64)
    _nearest_point_invariant(w.numpy(), dec, idx, cache, G, all_sums)

    # and the arrays, where they lie, are operands of the HIP operator
    lin = sbvr.SBVRLinear.from_sbvr(enc)
    x = torch.randn((3, K), generator=torch.Generator().manual_seed(9)).to(torch.float16)
    y = lin(x.to(dev)).float().cpu().numpy().astype(np.float64)
    want = x.numpy().astype(np.float64) @ dec.astype(np.float64).T
    assert np.abs(y - want).max() <= 1e-2 * np.abs(want).max()


def test_gpu_and_cpu_encodings_are_of_equal_quality():
    """The search makes the same torch calls on either device; the results may differ in
    the last bit of a reduction, so the comparison is of the error, not of the arrays."""
    import sbvr
    dev = torch.device("cuda:0")
    w = (torch.randn((16, 512), generator=torch.Generator().manual_seed(77)) * 0.02).to(torch.float16)
    conf = {"num_sums": 4, "bvr_len": 128}
    on_gpu = sbvr.sbvr(w.to(dev), encoder_config=conf, device=dev, verbose_level=0).decode().float().cpu()
    on_cpu = sbvr.sbvr(w, encoder_config=conf, device=torch.device("cpu"), verbose_level=0).decode().float()
    e_gpu = (on_gpu - w.float()).pow(2).mean().item()
    e_cpu = (on_cpu - w.float()).pow(2).mean().item()
    assert abs(e_gpu - e_cpu) <= 0.05 * e_cpu


@pytest.mark.parametrize("S,G", [(2, 256), (4, 128), (4, 256), (6, 128)])
def test_search_kernel_is_the_search_expression(S, G):
    """The HIP search kernel against the reference's expression (core.py:485-495) step by step in numpy:
    fp16 difference, fp16 square, minimum over the 2^S points, fp32 sum over the group in element order,
    divided by G -- bit for bit; and against the same expression in torch on the device to 2e-5."""
    from sbvr import hip
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(S * 100 + G)
    B, n, P = 7, 333, 1 << S
    data = (rng.standard_normal((B, G)) * 0.02).astype(np.float16)
    data[2, 5] = 3.0                                   # an outlier, and a group of zeros
    data[4] = 0
    pts = (rng.standard_normal((n, P)) * 0.03).astype(np.float16)
    got = hip.encoder_group_mse(torch.from_numpy(data).to(dev), torch.from_numpy(pts).to(dev)).cpu().numpy()
    diff = (data[:, None, :, None] - pts[None, :, None, :]).astype(np.float16)
    best = (diff * diff).astype(np.float16).min(-1).astype(np.float32)
    want = np.cumsum(best, axis=-1, dtype=np.float32)[..., -1] / np.float32(G)
    assert np.array_equal(got, want)
    d, p = torch.from_numpy(data).to(dev), torch.from_numpy(pts).to(dev)
    t = ((d.view(B, 1, G, 1) - p.view(1, n, 1, P)) ** 2).min(-1)[0].float().mean(-1).cpu().numpy()
    assert np.allclose(got, t, rtol=2e-5, atol=0)          # (torch sums the group in another order)


@pytest.mark.parametrize("case", ["random", "v1_s2", "weights_s4_n64"])
def test_block_lookup_equals_one_group_loop(golden, case):
    """Table look-ups for 512 (or 7) groups at a time give the arrays of the one-group loop: the policy's
    order (hits, the error history, the hit rate that widens the search) is kept."""
    import sbvr
    dev = torch.device("cuda:0")
    if case == "random":
        w = (torch.randn((256, 1024), generator=torch.Generator().manual_seed(1)) * 0.02).to(torch.float16)
        conf = {"num_sums": 4, "bvr_len": 128}
    else:
        g = golden(case)
        w = torch.from_numpy(g["data"])
        conf = {"num_sums": int(g["num_sums"]), "bvr_len": int(g["bvr_len"])}
    made = {}
    for block in (1, 7, 512):
        made[block] = sbvr.sbvr(w.to(dev), encoder_config=dict(conf, group_block=block), device=dev, verbose_level=0)
    for block in (7, 512):
        for part in ("bvr", "coeff_idx", "coeff_cache"):
            assert torch.equal(getattr(made[1], part).data, getattr(made[block], part).data), (block, part)
        assert made[1].encoder_stats == made[block].encoder_stats
    assert made[1].encoder_stats["cache_hits"] > 0


def test_real_4096_encoding_and_config1(oracle, golden):
    """A real (searched, not synthetic) encoding of a 4096 x 4096 weight, 4 planes, groups of 128, made on
    the GPU in seconds: the same arrays as tests/golden/make_encoded_4096.py stored (slice and SHA-256 of
    each array), and the single-row linear of the first benchmark configuration on it against the oracle
    and against the dense product."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import make_encoded_4096 as made
    import sbvr
    from sbvr import hip
    dev = torch.device("cuda:0")
    g = golden("encoded_4096_s4_g128")
    enc, seconds = made.encode(dev)
    assert seconds < 60.0, f"encoding took {seconds:.1f} s"
    bvr, idx, cache = (t.cpu().numpy() for t in (enc.bvr.data, enc.coeff_idx.data, enc.coeff_cache.data))
    assert bvr.shape == (made.K // 32, made.N, made.S) and idx.shape == (made.K // made.G, made.N)
    assert np.array_equal(cache, g["coeff_cache"])
    assert np.array_equal(bvr[:, :made.ROWS, :], g["bvr_rows"]) and np.array_equal(idx[:, :made.ROWS], g["coeff_idx_rows"])
    assert made.digest(bvr) == str(g["sha256_bvr"]) and made.digest(idx) == str(g["sha256_coeff_idx"])
    assert enc.encoder_stats["lines"] == int(g["lines"]) and enc.encoder_stats["cache_hits"] == int(g["cache_hits"])
    # config 1: one row through the decode kernel on the real encoding
    x = torch.randn((1, made.K), generator=torch.Generator().manual_seed(5)).to(torch.float16)
    y = sbvr._sbvr_linear_f16(x.to(dev), enc.bvr.data, enc.coeff_idx.data, enc.coeff_cache.data, None, bvr_len=made.G)
    assert hip.last_kernel() == 2
    _, yd = oracle.C.linear_f16(x.numpy(), bvr, idx, cache, made.G)
    got = y.float().cpu().numpy().astype(np.float64)
    rms = float(np.sqrt(np.mean(yd ** 2)))
    assert (np.abs(got - yd) / np.maximum(np.abs(yd), 1e-2 * rms)).max() <= 1e-2
    assert (np.abs(got - yd) / (np.maximum(np.abs(yd), rms) * 2.0 ** -10)).max() <= 2.0
    # the encoding stands for the weight: 4 planes leave under 1 % of the variance (the reference's log: 1.7e-2)
    w = made.weight().numpy().astype(np.float64)
    dense = x.numpy().astype(np.float64) @ w.T
    assert np.mean((got - dense) ** 2) < 0.02 * np.mean(dense ** 2)
