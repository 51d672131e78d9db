"""Pins the CPU oracle (oracle/sbvr_oracle.c and the numpy restatements):

* against the golden vectors written by the reference's own sbvr/core.py
  (tests/golden/*.npz: bvr, coeff_idx, coeff_cache, decode() of tiny tensors in
  every layout) -- these fix the conventions mathematics cannot: plane order,
  bit order, array layouts, padding;
* against brute force from the definition on tiny inputs (pure Python loops);
* against closed forms and identities (all-ones planes, single bits, linearity,
  sum popcount(L&R) a b == decode(A) decode(B)^T);
* the C file against the independently written numpy code.
"""
import itertools

import numpy as np
import pytest

DEFAULT_CASES = ["default_s2", "default_s3", "default_s4", "pad_s2", "v2_s2", "v1_row_s2", "trans_s2", "weights_s4"]


def _f16(a):
    return np.asarray(a, dtype=np.float16)


# ------------------------------------------------------------------ fp16 helpers

def test_fp16_conversions_all_values(oracle):
    """h2d is exact and d2h(h2d(h)) == h for every finite fp16; d2h rounds like numpy."""
    bits = np.arange(0, 1 << 16, dtype=np.uint32)
    vals = bits.astype(np.uint16).view(np.float16)
    for b in range(0, 1 << 16, 7):
        v = vals[b]
        if np.isnan(v):
            continue
        assert oracle.C.h2d(b) == float(v)
        assert oracle.C.d2h(float(v)) == b or (v == 0)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(2000) * 10.0 ** rng.integers(-8, 5, 2000),
                        [65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -26, 0.0, -0.0]])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([oracle.C.d2h(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ golden vectors

@pytest.mark.parametrize("name", DEFAULT_CASES)
def test_decode_matches_reference(oracle, golden, name):
    g = golden(name)
    G = int(g["bvr_len"])
    want = g["decoded"]
    for dec in (oracle.C.decode, oracle.np_decode):
        got = dec(g["bvr"], g["coeff_idx"], g["coeff_cache"], G, out_cols=want.shape[1])
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), name


@pytest.mark.parametrize("name", DEFAULT_CASES)
def test_pack_unpack_round_trip_on_reference_arrays(oracle, golden, name):
    """bvr -> selectors -> planes -> bvr reproduces the reference's array bit for bit."""
    g = golden(name)
    bvr = g["bvr"]
    Kw, R, S = bvr.shape
    wb = bvr.dtype.itemsize * 8
    sel = oracle.C.default_to_sel(bvr)
    assert np.array_equal(sel, oracle.np_default_to_sel(bvr))
    assert sel.min() >= 0 and sel.max() < (1 << S)
    planes = oracle.C.sel_to_planes(sel, S, wb)
    assert np.array_equal(planes, oracle.np_sel_to_planes(sel, S, wb))
    back = oracle.C.planes_to_default(planes, R, Kw * wb)
    assert np.array_equal(back, bvr)
    assert np.array_equal(oracle.np_planes_to_default(planes, R), bvr)


def test_selectors_are_nearest_points(oracle, golden):
    """The reference assigns every element the nearest of its line's 2^S points
    (core.py:492-494); with the plane<->coefficient pairing restated here the
    selectors recovered from its bvr must have that property."""
    for name in ["default_s2", "default_s3", "default_s4", "weights_s4"]:
        g = golden(name)
        S, G = int(g["num_sums"]), int(g["bvr_len"])
        sel = oracle.C.default_to_sel(g["bvr"])
        combs = oracle.np_bin_combs(S).astype(np.float16)
        cache = g["coeff_cache"]
        data = g["data"]
        R, K = data.shape
        for r in range(R):
            for grp in range(K // G):
                line = int(g["coeff_idx"][grp, r])
                points = (combs @ cache[line].astype(np.float16)).astype(np.float16)
                d = data[r, grp * G:(grp + 1) * G]
                err = (d[:, None] - points[None, :]) ** 2
                chosen = sel[r, grp * G:(grp + 1) * G]
                assert np.all(err[np.arange(G), chosen] <= err.min(1))


def test_v1_layout_matches_reference(oracle, golden):
    """The 16-lane array of cpu_kernel=True equals planes_to_v1 of the planes, and
    a v2 (uint8) encoding of the same planes re-layouts to it."""
    g = golden("v1_s2")
    bvr = g["bvr"]                       # (R/16, K/8, S, 16)
    r16, Kb, S, lanes = bvr.shape
    R = r16 * lanes
    planes = np.ascontiguousarray(bvr.transpose(2, 0, 3, 1).reshape(S, R * Kb))
    assert np.array_equal(oracle.C.planes_to_v1(planes, R, Kb * 8), bvr)
    assert np.array_equal(oracle.np_planes_to_v1(planes, R), bvr)
    assert g["coeff_idx"].shape == (Kb * 8 // int(g["bvr_len"]), R)
    # decode through the default layout agrees with the data to encoder accuracy
    dflt = oracle.C.planes_to_default(planes, R, Kb * 8)
    dec = oracle.C.decode(dflt, g["coeff_idx"], g["coeff_cache"], int(g["bvr_len"]))
    mse = np.mean((dec.astype(np.float64) - g["data"].astype(np.float64)) ** 2)
    assert mse < 0.25 * np.var(g["data"].astype(np.float64))      # S=2: about 0.13 of the variance


def test_idx_layout(oracle):
    flat = np.arange(12, dtype=np.uint8)                           # 3 rows x 4 groups, row major
    out = oracle.C.idx_to_default(flat, 3, 4)
    assert np.array_equal(out, flat.reshape(3, 4).T)


# ------------------------------------------------------------------ brute force

def _brute_linear(x, bvr, idx, cache, G):
    """Straight from the definition, one element at a time."""
    Kw, N, S = bvr.shape
    M, K = x.shape
    y = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            for k in range(K):
                w = 0.0
                for j in range(S):
                    if (int(bvr[k // 32, n, j]) >> (k % 32)) & 1:
                        w += float(cache[int(idx[k // G, n]), j])
                y[m, n] += float(x[m, k]) * w
    return y


def test_linear_brute_force(oracle):
    rng = np.random.default_rng(1)
    N, K, S, G, L, M = 5, 64, 3, 32, 4, 2
    bvr = rng.integers(0, 1 << 32, size=(K // 32, N, S), dtype=np.uint64).astype(np.uint32)
    idx = rng.integers(0, L, size=(K // G, N)).astype(np.uint8)
    cache = _f16(rng.standard_normal((L, S)))
    x = _f16(rng.standard_normal((M, K)))
    want = _brute_linear(x, bvr, idx, cache, G)
    for fn in (oracle.C.linear_f16, oracle.np_linear_f16):
        y, yd = fn(x, bvr, idx, cache, G)
        assert np.allclose(yd, want, rtol=1e-12, atol=1e-12)
        assert np.array_equal(y.view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_linear_equals_x_times_decode(oracle, golden):
    """y == x @ decode(W)^T with the reference's own decode() output, up to the
    fp16 rounding decode applies to every element."""
    g = golden("weights_s4")
    G = int(g["bvr_len"])
    rng = np.random.default_rng(2)
    K = g["bvr"].shape[0] * 32
    x = _f16(rng.standard_normal((3, K)))
    _, yd = oracle.C.linear_f16(x, g["bvr"], g["coeff_idx"], g["coeff_cache"], G)
    _, yd1 = oracle.C.linear_f16(x, g["bvr"], g["coeff_idx"], g["coeff_cache"], G, mode=1)
    want = x.astype(np.float64) @ g["decoded"].astype(np.float64).T
    assert np.allclose(yd1, want, rtol=1e-12, atol=1e-12)          # mode 1 rounds like decode()
    scale = np.sqrt(np.mean(want ** 2))
    assert np.abs(yd - want).max() < 2e-3 * scale                  # mode 0 skips that rounding


def test_linear_closed_forms(oracle):
    rng = np.random.default_rng(3)
    N, K, S, G, L = 4, 256, 4, 128, 3
    idx = rng.integers(0, L, size=(K // G, N)).astype(np.uint8)
    cache = _f16(rng.standard_normal((L, S)))
    x = _f16(rng.standard_normal((1, K)))
    # all planes set: y[n] = sum_g (sum_j c_j) * sum_{k in g} x[k]
    ones = np.full((K // 32, N, S), 0xFFFFFFFF, dtype=np.uint32)
    _, yd = oracle.C.linear_f16(x, ones, idx, cache, G)
    gs = x.astype(np.float64).reshape(K // G, G).sum(1)
    want = (gs[:, None] * cache.astype(np.float64).sum(1)[idx.astype(int)]).sum(0)
    assert np.allclose(yd[0], want, rtol=1e-12)
    # a single bit: plane j of element (n, k)
    for (n, k, j) in [(0, 0, 0), (3, 255, 3), (2, 129, 1), (1, 31, 2), (1, 32, 2)]:
        one = np.zeros((K // 32, N, S), dtype=np.uint32)
        one[k // 32, n, j] = np.uint32(1) << np.uint32(k % 32)
        _, yd = oracle.C.linear_f16(x, one, idx, cache, G)
        want = np.zeros(N)
        want[n] = float(x[0, k]) * float(cache[int(idx[k // G, n]), j])
        assert np.allclose(yd[0], want, rtol=1e-12, atol=0)
    # no planes set: zero; bias is then the whole answer, added in fp16
    zero = np.zeros((K // 32, N, S), dtype=np.uint32)
    bias = _f16(rng.standard_normal(N))
    y, _ = oracle.C.linear_f16(x, zero, idx, cache, G, bias=bias)
    assert np.array_equal(y[0].view(np.uint16), bias.view(np.uint16))


def test_linear_is_linear_in_x(oracle):
    rng = np.random.default_rng(4)
    N, K, S, G, L = 6, 256, 2, 128, 5
    bvr = rng.integers(0, 1 << 32, size=(K // 32, N, S), dtype=np.uint64).astype(np.uint32)
    idx = rng.integers(0, L, size=(K // G, N)).astype(np.uint8)
    cache = _f16(rng.standard_normal((L, S)))
    x1 = _f16(rng.integers(-32, 32, size=(1, K)) / 16.0)
    x2 = _f16(rng.integers(-32, 32, size=(1, K)) / 16.0)
    f = lambda v: oracle.C.linear_f16(v, bvr, idx, cache, G)[1]
    assert np.allclose(f(x1) + f(x2), f(_f16(x1.astype(np.float64) + x2.astype(np.float64))), rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ both operands encoded

def _rand_enc(rng, rows, K, S, G, L, word_bits, oracle):
    sel = rng.integers(0, 1 << S, size=rows * K).astype(np.int32)
    planes = oracle.C.sel_to_planes(sel, S, word_bits)
    idx = rng.integers(0, L, size=(K // G, rows)).astype(np.uint8 if L <= 256 else np.uint16)
    cache = _f16(rng.standard_normal((L, S)) * 0.5)
    return planes, idx, cache


@pytest.mark.parametrize("word_bits", [32, 8])
def test_mm_T_is_decode_times_decode(oracle, word_bits):
    """sum_g sum_{l,r} popcount_g(L_l & R_r) a_l b_r == decode(A) @ decode(B)^T in
    exact arithmetic (decode taken unrounded)."""
    rng = np.random.default_rng(5)
    M, N, K, Sl, Sr, G = 2, 7, 512, 3, 4, 256
    lp, li, lc = _rand_enc(rng, M, K, Sl, G, 6, word_bits, oracle)
    rp, ri, rc = _rand_enc(rng, N, K, Sr, G, 300, word_bits, oracle)
    lb, rb = oracle.C.planes_to_default(lp, M, K), oracle.C.planes_to_default(rp, N, K)
    y, yd = oracle.C.mm_T(lb, li, lc, rb, ri, rc, G)
    yn, ydn = oracle.np_mm_T(lb, li, lc, rb, ri, rc, G)
    assert np.allclose(yd, ydn, rtol=1e-12, atol=1e-12) and np.array_equal(y.view(np.uint16), yn.view(np.uint16))

    def dense(bvr, idx, cache, S):
        bits = oracle.np_default_to_bits(bvr).astype(np.float64)              # (S, R, K)
        c = cache.astype(np.float64)[idx.astype(int).T]                        # (R, Kg, S)
        c = np.repeat(c, G, axis=1)                                            # (R, K, S)
        return np.einsum("srk,rks->rk", bits, c)
    want = dense(lb, li, lc, Sl) @ dense(rb, ri, rc, Sr).T
    assert np.allclose(yd, want, rtol=1e-10, atol=1e-10)


def test_mm_T_v1_layout_and_wrap(oracle):
    rng = np.random.default_rng(6)
    N, K, Sl, Sr, G = 32, 512, 2, 2, 256
    lp, li, lc = _rand_enc(rng, 1, K, Sl, G, 3, 8, oracle)
    rp, ri, rc = _rand_enc(rng, N, K, Sr, G, 9, 8, oracle)
    lb = oracle.C.planes_to_default(lp, 1, K)
    bias = _f16(rng.standard_normal(N))
    y1 = oracle.C.mm_T_v1(lb, li, lc, oracle.C.planes_to_v1(rp, N, K), ri, rc, G, bias)
    y2, _ = oracle.C.mm_T(lb, li, lc, oracle.C.planes_to_default(rp, N, K), ri, rc, G, bias)
    assert np.array_equal(y1.view(np.uint16), y2.view(np.uint16))
    # a group in which every bit of both operands is set counts 256 == 0 in 8 bits
    ones_l = np.full((K // 8, 1, 1), 255, dtype=np.uint8)
    ones_r = np.full((N // 16, K // 8, 1, 16), 255, dtype=np.uint8)
    one_line = _f16([[1.0]])
    zi_l, zi_r = np.zeros((K // G, 1), np.uint8), np.zeros((K // G, N), np.uint8)
    exact = oracle.C.mm_T_v1(ones_l, zi_l, one_line, ones_r, zi_r, one_line, G)
    wrapped = oracle.C.mm_T_v1(ones_l, zi_l, one_line, ones_r, zi_r, one_line, G, wrap8=True)
    assert np.all(exact == K) and np.all(wrapped == 0)


def test_row_deq_is_transposed_linear(oracle, golden):
    """The trans=True product equals x @ decode(W^T)^T ... i.e. x @ W_dec with W_dec
    the (K, N) tensor the reference decoded (core.py:244-245)."""
    g = golden("trans_s2")
    G = int(g["bvr_len"])
    bvr, idx, cache = g["bvr"], g["coeff_idx"], g["coeff_cache"]          # (N/32, K, S), (N/G, K)
    wt = g["decoded"].astype(np.float64)                                    # (K, N) == decode of W^T
    K, N = wt.shape
    rng = np.random.default_rng(7)
    x = _f16(rng.standard_normal((2, K)))
    bias = _f16(rng.standard_normal(N))
    y = oracle.C.row_deq_mm_T(x, bvr, idx, cache, G, bias)
    want = x.astype(np.float64) @ wt + bias.astype(np.float64)
    assert np.abs(y.astype(np.float64) - want).max() <= 2e-3 * np.abs(want).max()


# ------------------------------------------------------------------ the timed CPU port

def test_cpu_port_matches_oracle(oracle):
    rng = np.random.default_rng(8)
    for (N, K, Sl, Sr, G, Lr) in [(64, 512, 4, 4, 256, 9), (48, 256, 2, 4, 128, 300), (32, 256, 3, 5, 128, 17)]:
        lp, li, lc = _rand_enc(rng, 1, K, Sl, G, 5, 8, oracle)
        rp, ri, rc = _rand_enc(rng, N, K, Sr, G, Lr, 8, oracle)
        lb, rv1 = oracle.C.planes_to_default(lp, 1, K), oracle.C.planes_to_v1(rp, N, K)
        bias = _f16(rng.standard_normal(N))
        want = oracle.C.mm_T_v1(lb, li, lc, rv1, ri, rc, G, bias).astype(np.float64)
        for threads in (1, 3):
            oracle.PORT.init_pool(threads)
            got = oracle.PORT.mm_T_v1(lb, li, lc, rv1, ri, rc, G, bias).astype(np.float64)
            oracle.PORT.finalize_pool()
            # the port rounds every coefficient product to fp16, as the reference does, and adds in another
            # order than the oracle: the two fp16 results are at most one fp16 step of the largest output apart
            assert np.abs(got - want).max() <= 2.0 ** -10 * max(np.abs(want).max(), 1.0)
