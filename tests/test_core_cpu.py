"""Host-side package tests (no GPU): the sbvr objects, their layouts, decode(),
save/load and the encoder, against the golden vectors the reference wrote."""
import os
import re

import numpy as np
import pytest
import torch

from conftest import GOLDEN, ROOT

CASES = {
    "default_s2": {}, "default_s3": {}, "pad_s2": {}, "v2_s2": {"cpu_kernel_v2": True},
    "trans_s2": {"trans": True}, "v1_s2": {"cpu_kernel": True}, "v1_row_s2": {"cpu_kernel": True},
}


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def _same_bits(a, b):
    return a.shape == b.shape and torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("name", list(CASES))
def test_encoder_reproduces_reference(golden, name):
    """Same input, same configuration, CPU: identical bvr, coeff_idx and coeff_cache."""
    import sbvr
    g = golden(name)
    obj = sbvr.sbvr(_t(g["data"]), encoder_config={"num_sums": int(g["num_sums"])},
                    device=torch.device("cpu"), verbose_level=0, **CASES[name])
    assert _same_bits(obj.bvr.data, _t(g["bvr"]))
    assert _same_bits(obj.coeff_idx.data, _t(g["coeff_idx"]))
    assert _same_bits(obj.coeff_cache.data, _t(g["coeff_cache"]))
    if g["decoded"].size:
        assert _same_bits(obj.decode(), _t(g["decoded"]))


@pytest.mark.parametrize("name,block", [(n, 64) for n in CASES] + [("v1_s2", 3), ("default_s3", 5)])
def test_block_lookup_encoder_reproduces_reference(golden, name, block):
    """Table look-ups for a block of groups at a time (the GPU's default) keep the order-dependent policy:
    the same arrays as the reference's one-group loop, for a short and a long block."""
    import sbvr
    g = golden(name)
    obj = sbvr.sbvr(_t(g["data"]), encoder_config={"num_sums": int(g["num_sums"]), "group_block": block},
                    device=torch.device("cpu"), verbose_level=0, **CASES[name])
    assert _same_bits(obj.bvr.data, _t(g["bvr"]))
    assert _same_bits(obj.coeff_idx.data, _t(g["coeff_idx"]))
    assert _same_bits(obj.coeff_cache.data, _t(g["coeff_cache"]))
    assert obj.encoder_stats["groups"] == obj.coeff_idx.numel()


@pytest.mark.parametrize("name", ["default_s2", "default_s3", "default_s4", "pad_s2", "v2_s2", "v1_row_s2",
                                  "trans_s2", "weights_s4"])
def test_decode_of_reference_arrays(golden, name):
    import sbvr
    g = golden(name)
    obj = sbvr.sbvr.from_parts(_t(g["bvr"]), _t(g["coeff_idx"]), _t(g["coeff_cache"]), int(g["bvr_len"]),
                               original_shape=g["decoded"].shape)
    assert _same_bits(obj.decode(), _t(g["decoded"]))


def test_load_file_written_by_reference(golden):
    """default_s2_saved.pt was written by the reference's save(); the class path in
    the pickle is sbvr.core._sbvr_serialized."""
    import sbvr
    obj = sbvr.load(os.path.join(GOLDEN, "default_s2_saved.pt"), device="cpu", verbose_level=0)
    g = golden("default_s2")
    assert _same_bits(obj.bvr.data, _t(g["bvr"])) and _same_bits(obj.decode(), _t(g["decoded"]))
    assert obj.num_sums == 2 and obj.bvr_len == 256


def test_save_load_round_trip(tmp_path, golden):
    import sbvr
    g = golden("weights_s4")
    obj = sbvr.sbvr.from_parts(_t(g["bvr"]), _t(g["coeff_idx"]), _t(g["coeff_cache"]), 256)
    path = str(tmp_path / "w.pt")
    obj.save(path)
    back = sbvr.load(path, device="cpu", verbose_level=0)
    assert _same_bits(back.bvr.data, obj.bvr.data) and _same_bits(back.coeff_idx.data, obj.coeff_idx.data)
    assert _same_bits(back.coeff_cache.data, obj.coeff_cache.data)
    assert _same_bits(back.decode(), obj.decode())
    with pytest.raises(ValueError):
        sbvr.load(path, device="cpu", verbose_level=0, cpu_kernel_v2=True)     # uint32 file, uint8 requested


def test_layout_conversions(golden):
    """uint32 <-> uint8 re-wording and the 16-lane layout are pure permutations."""
    from sbvr import layout
    g = golden("default_s4")
    bvr = _t(g["bvr"])
    sel = layout.default_to_sel(bvr)
    b8 = layout.rewidth(bvr, torch.uint8)
    assert b8.shape == (bvr.shape[0] * 4, bvr.shape[1], bvr.shape[2])
    assert torch.equal(layout.default_to_sel(b8), sel)
    assert _same_bits(layout.rewidth(b8, torch.uint32), bvr)
    g1 = golden("v1_s2")
    v1 = _t(g1["bvr"])
    planes = layout.v1_to_planes(v1)
    assert _same_bits(layout.planes_to_v1(planes.reshape(planes.shape[0], -1), planes.shape[1]), v1)
    v2 = _t(golden("v2_s2")["bvr"])
    assert _same_bits(layout.planes_to_default(layout.default_to_planes(v2).reshape(v2.shape[2], -1), v2.shape[1]), v2)


def test_group_length_128_extension():
    """bvr_len is a parameter here (the reference fixes 256): encode, decode, error band."""
    import sbvr
    torch.manual_seed(0)
    w = (torch.randn(4, 256) * 0.02).to(torch.float16)
    obj = sbvr.sbvr(w, encoder_config={"num_sums": 4, "bvr_len": 128}, device=torch.device("cpu"), verbose_level=0)
    assert obj.bvr.shape == (8, 4, 4) and obj.coeff_idx.shape == (2, 4) and obj.bvr.dtype == torch.uint32
    rel = ((obj.decode().float() - w.float()) ** 2).mean() / w.float().var()
    assert rel < 0.03          # the reference logs about 1.7e-2 of the variance for 4 planes (test.txt:55-59)


def test_constructor_errors():
    import sbvr
    with pytest.raises(ValueError):
        sbvr.sbvr()
    with pytest.raises(ValueError):
        sbvr.sbvr(torch.zeros(2, 256), sbvr_serialized=object())
    with pytest.raises(ValueError):
        sbvr.sbvr(sbvr_serialized=object())
    with pytest.raises(ValueError):
        sbvr.sbvr(torch.zeros(2, 256), encoder_config={"bvr_len": 48}, device="cpu", verbose_level=0)


def test_synthetic_encoding_shapes():
    from sbvr import synth
    bvr, idx, cache = synth.random_encoding(64, 512, 3, 128, 300, seed=1)
    assert bvr.shape == (16, 64, 3) and bvr.dtype == torch.uint32
    assert idx.shape == (4, 64) and idx.dtype == torch.uint16 and int(idx.to(torch.int32).max()) < 300
    assert cache.shape == (300, 3) and cache.dtype == torch.float16
    assert torch.all(cache.float().abs()[:, :-1] <= cache.float().abs()[:, 1:])     # sorted by magnitude


def test_ops_refuse_cpu_tensors():
    """No CPU fallback: the operators raise on host tensors."""
    import sbvr
    from sbvr import synth
    bvr, idx, cache = synth.random_encoding(32, 256, 4, 128, 16)
    x = torch.zeros((1, 256), dtype=torch.float16)
    with pytest.raises(sbvr.SbvrHipError):
        sbvr._sbvr_linear_f16(x, bvr, idx, cache, None, 128)


# ------------------------------------------------------------------ C ABI

def _declared_symbols():
    text = "".join(open(os.path.join(ROOT, "include", name)).read()
                   for name in sorted(os.listdir(os.path.join(ROOT, "include"))) if name.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sbvr_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    """libsbvr_hip.so loads without a GPU and exports what include/sbvr_hip.h declares."""
    import ctypes
    from sbvr import hip
    path = hip.library_path()
    assert os.path.exists(path), f"{path} missing: run __graft_entry__.build()"
    lib = ctypes.CDLL(path)
    names = _declared_symbols()
    assert len(names) >= 7
    for n in names:
        assert hasattr(lib, n), f"{n} declared in sbvr_hip.h but not exported"
    lib.sbvr_hip_version.restype = ctypes.c_int
    assert lib.sbvr_hip_version() == 104
    lib.sbvr_hip_linear_f16_workspace.restype = ctypes.c_size_t
    assert lib.sbvr_hip_linear_f16_workspace(1, 14336, 4096, 4, 128) == 14336 * 8
    assert lib.sbvr_hip_linear_f16_workspace(1, 64, 96, 4, 32) == 0        # portable kernel: no workspace


def test_workspace_sizes_follow_the_split_predicates():
    """The alternates' workspace queries ask for accumulators only where their launch may split K."""
    import ctypes
    from sbvr import hip
    lib = hip._load()
    assert lib.sbvr_hip_mm_T_workspace(1, 4096) == 4096 * 8           # one left row: the decode kernel, may split
    assert lib.sbvr_hip_mm_T_workspace(2048, 14336) == 0              # more left rows never split
    assert lib.sbvr_hip_row_deq_mm_T_workspace(1, 4096) == 4096 * 8   # 64 column workgroups on 256 CUs: split
    assert lib.sbvr_hip_row_deq_mm_T_workspace(2048, 14336) == 0      # prefill-sized: the columns fill the device


def test_decode_plans_respect_the_launch_bounds():
    """Every launch shape the planners pick for up to 16 rows stays within the waves its kernel
    instance is compiled for (a launch beyond them fails), over a grid of shapes and device sizes."""
    import ctypes
    from sbvr import hip
    lib = hip._load()
    plan = (ctypes.c_int * 8)()
    seen = 0
    for cus in (64, 228, 256, 304):
        for M in (1, 2, 4, 5, 8, 9, 12, 16):
            for N in (16, 48, 512, 1024, 4096, 6144, 14336, 28672, 128256):
                for K in (128, 512, 2048, 4096, 8192, 14336):
                    for S in (2, 3, 4, 6, 8):
                        assert lib.sbvr_hip_decode_plan(M, N, K, S, 128, cus, plan) == 0
                        kind, ct, sp, mt, waves, wgs, ksplit, bound = list(plan)
                        if kind == 0:
                            continue
                        seen += 1
                        assert 1 <= waves <= bound, (cus, M, N, K, S, list(plan))
                        assert mt == (1 if M <= 4 else 2 if M <= 8 else 4), (M, list(plan))
                        assert wgs >= 1 and 1 <= ksplit <= 255 and ct >= 1 and sp >= 1
    assert seen > 4000


def test_argument_validation_without_gpu():
    """Bad arguments are rejected before anything touches a device."""
    import ctypes
    from sbvr import hip
    lib = hip._load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = lib.sbvr_hip_linear_f16(None, p, p, 1, p, None, p, 1, 16, 128, 4, 128, 4, None, 0, 0, None)
    assert rc == -1 and b"null" in lib.sbvr_hip_last_error()
    rc = lib.sbvr_hip_linear_f16(p, p, p, 1, p, None, p, 1, 16, 100, 4, 128, 4, None, 0, 0, None)
    assert rc == -1 and b"multiple" in lib.sbvr_hip_last_error()
    rc = lib.sbvr_hip_linear_f16(p, p, p, 3, p, None, p, 1, 16, 128, 4, 128, 4, None, 0, 0, None)
    assert rc == -1 and b"idx_bytes" in lib.sbvr_hip_last_error()
    rc = lib.sbvr_hip_linear_f16(p, p, p, 1, p, None, p, 1, 16, 128, 4, 128, 300, None, 0, 0, None)
    assert rc == -1 and b"uint8" in lib.sbvr_hip_last_error()
    rc = lib.sbvr_hip_mm_T(p, p, 1, p, p, p, 1, p, None, p, 1, 16, 100, 4, 4, 128, 4, 4, None)
    assert rc == -1
    rc = lib.sbvr_hip_row_deq_mm_T(p, p, p, 1, p, None, p, 1, 48, 64, 4, 32, 4, None)
    assert rc == -1        # N must be a multiple of 32 and of G


def test_torch_extension_mirrors_the_reference_operators():
    """The compiled PyTorch extension (csrc/sbvr_ops_hip.cpp) offers the reference's operator
    names (sbvr_ops.cpp:152-172) and refuses CPU tensors, like the ctypes binding."""
    import torch
    from sbvr import _sbvr_hip_ops as ops, hip
    for name in ("_sbvr_mm_T", "_sbvr_row_deq_mm_T", "_sbvr_cuda_init", "_sbvr_hip_init", "_sbvr_linear_f16",
                 "_sbvr_linear_f16_swiglu", "_sbvr_linear_f16_add_rmsnorm"):
        assert callable(getattr(ops, name)), name
    assert ops.version() == hip._load().sbvr_hip_version()
    x = torch.zeros((1, 128), dtype=torch.float16)
    bvr = torch.zeros((4, 16, 4), dtype=torch.uint32)
    idx = torch.zeros((1, 16), dtype=torch.uint8)
    cache = torch.zeros((4, 4), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        ops._sbvr_linear_f16(x, bvr, idx, cache)
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        ops._sbvr_mm_T(bvr, idx, cache, bvr, idx, cache, torch.zeros(0, dtype=torch.float16))


def test_fuse_rows_decodes_to_the_stacked_weights(oracle):
    """layout.fuse_rows: tables concatenated, indices shifted; index width follows the total line count."""
    from sbvr import layout, synth
    parts = [synth.random_encoding(rows, 256, 3, 128, lines, seed=rows) for rows, lines in ((32, 100), (16, 100), (48, 60))]
    bvr, idx, cache = layout.fuse_rows(parts)
    assert bvr.shape == (8, 96, 3) and idx.shape == (2, 96) and cache.shape == (260, 3) and idx.dtype == torch.uint16
    whole = oracle.C.decode(bvr.numpy(), idx.numpy(), cache.numpy(), 128)
    stacked = np.concatenate([oracle.C.decode(b.numpy(), i.numpy(), c.numpy(), 128) for b, i, c in parts], axis=0)
    assert np.array_equal(whole, stacked)
    small = layout.fuse_rows(parts[:2])
    assert small[1].dtype == torch.uint8 and small[2].shape[0] == 200
    with pytest.raises(ValueError):
        layout.fuse_rows([parts[0], synth.random_encoding(16, 512, 3, 128, 10, seed=1)])


def test_attention_o_cache_layout_round_trip():
    """The blocked element order of the one-launch attention + projection's caches (host-side helper): a
    permutation, its inverse, and the offsets the kernel computes for one element."""
    import torch
    from sbvr import hip
    x = torch.arange(2 * 96 * 128, dtype=torch.float32).view(2, 96, 128)
    for values in (False, True):
        y = hip.attention_o_cache_layout(x, values=values)
        assert y.shape == x.shape and torch.equal(hip.attention_o_cache_layout(y, inverse=True, values=values), x)
        for t, d in ((0, 0), (37, 77), (95, 127), (16, 32), (31, 8)):
            if values:
                off = (t // 32) * 4096 + (d // 16) * 512 + ((t % 32) // 8) * 128 + (d % 16) * 8 + t % 8
            else:
                off = (t // 16) * 2048 + (d // 32) * 512 + ((d % 32) // 8) * 128 + (t % 16) * 8 + d % 8
            assert y[1].flatten()[off] == x[1, t, d]
