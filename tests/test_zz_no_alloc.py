"""sbvr_hip_linear_f16_noalloc, the entry point that allocates nothing (its split-K
accumulators live in an array inside the library), against sbvr_hip_linear_f16 on the
same inputs: both run the same kernels, so the outputs must be identical bit for bit.
Called through the C ABI directly (ctypes), two calls in a row, the second on a smaller
input, and the library's scratch memory must be left as it was found (all zero), which
a third call on the first input shows."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(lib, entry, x, bvr, idx, cache, bias, G, ws=None):
    M, K = x.shape
    Kw, N, S = bvr.shape
    L = cache.shape[0]
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device=x.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = (x.data_ptr(), bvr.data_ptr(), idx.data_ptr(), idx.element_size(), cache.data_ptr(),
              bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K, S, G, L)
    if entry == "noalloc":
        rc = lib.sbvr_hip_linear_f16_noalloc(*common, 0, stream)
    else:
        rc = lib.sbvr_hip_linear_f16(*common, ws.data_ptr(), ws.numel(), 0, stream)
    assert rc == 0, lib.sbvr_hip_last_error().decode()
    torch.cuda.synchronize()
    return out


def test_noalloc_equals_workspace_entry_point(oracle):
    from sbvr import hip, synth
    assert torch.cuda.is_available(), "this test needs the GPU"
    dev = torch.device("cuda:0")
    lib = hip._load()
    assert lib.sbvr_hip_init(0) == 0, lib.sbvr_hip_last_error().decode()
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)

    def case(N, K, S, M, L, seed, bias):
        bvr, idx, cache = (t.to(dev) for t in synth.random_encoding(N, K, S, 128, L, seed=seed))
        gen = torch.Generator().manual_seed(seed + 100)
        x = torch.randn((M, K), generator=gen).to(torch.float16).to(dev)
        b = (torch.randn((N,), generator=gen) * 0.3).to(torch.float16).to(dev) if bias else None
        return x, bvr, idx, cache, b

    # K split across workgroups in both (few columns, long K): the scratch array is in use
    first = case(1024, 4096, 4, 3, 256, 31, True)
    second = case(512, 2048, 3, 1, 300, 32, False)       # smaller, other plane count, uint16 indices
    free_before = torch.cuda.mem_get_info()[0]
    got = []
    for inputs in (first, second, first):
        got.append(_call(lib, "noalloc", *inputs, 128))
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
    want = [_call(lib, "workspace", *inputs, 128, ws=ws) for inputs in (first, second, first)]
    for g, w in zip(got, want):
        assert not torch.isnan(g.float()).any()
        assert torch.equal(g, w), "noalloc and workspace entry points disagree"
    assert int(ws.max()) == 0
    # and the result is right (oracle), not merely equal
    x, bvr, idx, cache, b = second
    _, yd = oracle.C.linear_f16(x.cpu().numpy(), bvr.cpu().numpy(), idx.cpu().numpy(), cache.cpu().numpy(), 128)
    rms = float(np.sqrt(np.mean(yd ** 2)))
    err = np.abs(got[1].float().cpu().numpy().astype(np.float64) - yd) / np.maximum(np.abs(yd), rms)
    assert err.max() <= 2.0 ** -9

    # more rows than the decode kernel takes: prefill kernel, no scratch needed
    big = case(256, 1024, 4, 48, 256, 33, False)
    assert torch.equal(_call(lib, "noalloc", *big, 128), _call(lib, "workspace", *big, 128, ws=ws))

    # Beyond the array (M * N > 524288).  Every buffer below has its real size: whichever way the call goes, no
    # kernel reads or writes out of bounds.
    def device_case(N, K, S, M, seed):
        gen = torch.Generator(device=dev).manual_seed(seed)
        bvr = torch.randint(-2 ** 31, 2 ** 31, (K // 32, N, S), dtype=torch.int32, generator=gen, device=dev).view(torch.uint32)
        idx = torch.randint(0, 16, (K // 128, N), dtype=torch.int32, generator=gen, device=dev).to(torch.uint8)
        cache = synth.make_lines(16, S, 0.02, seed).to(dev)
        x = torch.randn((M, K), generator=gen, device=dev).to(torch.float16)
        return x, bvr, idx, cache

    plan = (ctypes.c_int * 8)()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (a) a decode launch that cannot do without the split of K (8 rows, K = 14336: a workgroup covers at most
    #     a seventh of K): refused with a clear error, nothing launched
    M, N, K, S = 8, 70016, 14336, 2
    assert lib.sbvr_hip_decode_plan(M, N, K, S, 128, cus, plan) == 0
    assert plan[0] != 0 and plan[6] > 1, f"this shape is expected to split K across workgroups: {list(plan)}"
    x, bvr, idx, cache = device_case(N, K, S, M, 34)
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
    rc = lib.sbvr_hip_linear_f16_noalloc(x.data_ptr(), bvr.data_ptr(), idx.data_ptr(), 1, cache.data_ptr(), None,
                                         out.data_ptr(), M, N, K, S, 128, 16, 0, stream)
    assert rc == -4 and b"noalloc" in lib.sbvr_hip_last_error(), (rc, lib.sbvr_hip_last_error())
    torch.cuda.synchronize()
    assert bool(torch.isnan(out.float()).all()), "a refused call wrote to its output"
    del x, bvr, idx, cache, out
    # (b) 16 rows of 40000 columns: the table look-up kernel, which runs unsplit without accumulators: not refused,
    #     and equal to the workspace entry point up to the order of the fp32 additions (that one may split K)
    M, N, K, S = 16, 40000, 1024, 2
    x, bvr, idx, cache = device_case(N, K, S, M, 35)
    big_ws = torch.zeros(M * N * 8, dtype=torch.uint8, device=dev)
    got = _call(lib, "noalloc", x, bvr, idx, cache, None, 128)
    want = _call(lib, "workspace", x, bvr, idx, cache, None, 128, ws=big_ws)
    assert not torch.isnan(got.float()).any()
    rms = float(want.float().pow(2).mean().sqrt())
    assert float((got.float() - want.float()).abs().max()) <= 2.0 ** -9 * max(rms, float(want.float().abs().max()))
    assert int(big_ws.max()) == 0
