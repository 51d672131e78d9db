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
