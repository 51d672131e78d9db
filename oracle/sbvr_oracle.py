"""TEST INFRASTRUCTURE, not product code.

Two CPU checkers for the SBVR linear path:

* ``numpy`` restatements (functions named ``np_*``) of the reference's packing,
  ``decode()`` and matrix products, vectorised, written independently of the C
  file so that the two can be checked against each other;
* ``C`` -- a ctypes view of ``libsbvr_oracle.so`` (built from ``sbvr_oracle.c`` by
  ``oracle/Makefile``), the element-by-element restatement that the GPU parity
  tests compare with.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  Reference lines are cited per function.
"""
import ctypes
import itertools
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


# --------------------------------------------------------------------------- numpy

def np_bin_combs(S):
    """(2^S, S) table of 0/1, row i = i written MSB first (core.py:345-351)."""
    return np.array(list(itertools.product([0, 1], repeat=S)), dtype=np.int64)


def np_sel_to_planes(sel, S, word_bits):
    """Selectors (numel,) -> planes (S, numel/word_bits).

    core.py:815-818: plane j of an element is bit S-1-j of its selector;
    core.py:842-876: element w*word_bits+i lands in bit i of word w."""
    sel = np.asarray(sel, dtype=np.int64).reshape(-1)
    shifts = np.arange(S - 1, -1, -1, dtype=np.int64)
    bits = (sel[None, :] >> shifts[:, None]) & 1                      # (S, numel)
    bits = bits.reshape(S, -1, word_bits)
    weights = (np.int64(1) << np.arange(word_bits, dtype=np.int64))
    words = (bits * weights).sum(-1)
    return words.astype(np.uint32 if word_bits == 32 else np.uint8)


def np_planes_to_default(planes, R):
    """(S, R*Kw) -> (Kw, R, S), core.py:726-731 and :783."""
    S = planes.shape[0]
    return np.ascontiguousarray(planes.reshape(S, R, -1).transpose(2, 1, 0))


def np_planes_to_v1(planes, R):
    """(S, R*Kw) uint8 -> (R/16, Kw, S, 16), core.py:754-768."""
    S = planes.shape[0]
    return np.ascontiguousarray(planes.reshape(S, R // 16, 16, -1).transpose(1, 3, 0, 2))


def np_default_to_bits(bvr):
    """default bvr (Kw, R, S) -> bits (S, R, Kw*word_bits) of 0/1 (core.py:879-895)."""
    word_bits = bvr.dtype.itemsize * 8
    Kw, R, S = bvr.shape
    b = (bvr.astype(np.uint64)[..., None] >> np.arange(word_bits, dtype=np.uint64)) & 1   # (Kw,R,S,wb)
    return np.ascontiguousarray(b.transpose(2, 1, 0, 3).reshape(S, R, Kw * word_bits)).astype(np.uint8)


def np_default_to_sel(bvr):
    """default bvr -> selectors (R, Kp), core.py:879-901, 820-822."""
    bits = np_default_to_bits(bvr).astype(np.int64)
    S = bits.shape[0]
    w = (np.int64(1) << np.arange(S - 1, -1, -1, dtype=np.int64))
    return (bits * w[:, None, None]).sum(0).astype(np.int32)


def np_decode(bvr, coeff_idx, coeff_cache, G, out_cols=None):
    """decode() of the default layout, core.py:927-949: points of a group are
    fp16(bin_combs @ coeff) (core.py:365-366), every element picks one."""
    sel = np_default_to_sel(bvr)                                       # (R, Kp)
    R, Kp = sel.shape
    S = bvr.shape[2]
    combs = np_bin_combs(S).astype(np.float64)
    points = (combs[None] * coeff_cache.astype(np.float64)[:, None, :]).sum(-1).astype(np.float16)  # (L, 2^S)
    lines = coeff_idx.astype(np.int64).T                               # (R, Kg)
    lines = np.repeat(lines, G, axis=1)                                # (R, Kp)
    w = points[lines, sel]
    return w if out_cols is None else w[:, :out_cols]


def np_linear_f16(x, bvr, coeff_idx, coeff_cache, G, bias=None):
    """x (M,K) fp16 against an encoded (N,K) weight: f16(sum_g sum_j c_j * masked
    sum of x) then + bias in fp16 (sbvr_kernel.cu:479, 555-559)."""
    bits = np_default_to_bits(bvr).astype(np.float64)                  # (S, N, K)
    S, N, K = bits.shape
    xg = x.astype(np.float64).reshape(x.shape[0], K // G, G)           # (M, Kg, G)
    bg = bits.reshape(S, N, K // G, G)
    ps = np.einsum("mgk,sngk->mngs", xg, bg)                           # (M, N, Kg, S)
    c = coeff_cache.astype(np.float64)[coeff_idx.astype(np.int64).T]   # (N, Kg, S)
    yd = (ps * c[None]).sum((-1, -2))
    y = yd.astype(np.float16)
    if bias is not None and bias.size == N:
        y = (y.astype(np.float64) + bias.astype(np.float64)[None]).astype(np.float16)
    return y, yd


def np_mm_T(l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias=None):
    """Both operands encoded: sum_g sum_{l,r} popcount_g(L_l & R_r) a_l b_r
    (sbvr_kernel_v2.cpp:135-194, sbvr_kernel.cu:464-562)."""
    lb = np_default_to_bits(l_bvr).astype(np.float64)                  # (Sl, M, K)
    rb = np_default_to_bits(r_bvr).astype(np.float64)                  # (Sr, N, K)
    Sl, M, K = lb.shape
    Sr, N, _ = rb.shape
    pc = np.einsum("lmgk,rngk->mnglr", lb.reshape(Sl, M, K // G, G), rb.reshape(Sr, N, K // G, G))
    a = l_cache.astype(np.float64)[l_idx.astype(np.int64).T]           # (M, Kg, Sl)
    b = r_cache.astype(np.float64)[r_idx.astype(np.int64).T]           # (N, Kg, Sr)
    yd = np.einsum("mnglr,mgl,ngr->mn", pc, a, b)
    y = yd.astype(np.float16)
    if bias is not None and bias.size == N:
        y = (y.astype(np.float64) + bias.astype(np.float64)[None]).astype(np.float16)
    return y, yd


# ------------------------------------------------------------------------------- C

def build(force=False, targets=("libsbvr_oracle.so", "libsbvr_cpu_port.so")):
    """Compile the C checker and the timed CPU port in place (only what is
    missing, unless ``force``)."""
    for t in targets:
        if force or not os.path.exists(os.path.join(_HERE, t)):
            subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []) + [t])


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class _C:
    """ctypes calls into libsbvr_oracle.so; arrays are contiguous numpy arrays."""

    def __init__(self):
        self._lib = None

    @property
    def lib(self):
        if self._lib is None:
            path = os.path.join(_HERE, "libsbvr_oracle.so")
            if not os.path.exists(path):
                build(targets=("libsbvr_oracle.so",))
            self._lib = ctypes.CDLL(path)
            self._lib.sbvr_oracle_h2d.restype = ctypes.c_double
            self._lib.sbvr_oracle_h2d.argtypes = [ctypes.c_uint16]
            self._lib.sbvr_oracle_d2h.restype = ctypes.c_uint16
            self._lib.sbvr_oracle_d2h.argtypes = [ctypes.c_double]
        return self._lib

    @staticmethod
    def _c(a, dtype=None):
        a = np.ascontiguousarray(a)
        if dtype is not None and a.dtype != dtype:
            a = a.astype(dtype)
        return a

    def h2d(self, bits):
        return self.lib.sbvr_oracle_h2d(int(bits))

    def d2h(self, v):
        return self.lib.sbvr_oracle_d2h(float(v))

    def sel_to_planes(self, sel, S, word_bits):
        sel = self._c(sel, np.int32).reshape(-1)
        out = np.empty((S, sel.size // word_bits), dtype=np.uint32 if word_bits == 32 else np.uint8)
        self.lib.sbvr_oracle_sel_to_planes(_ptr(sel), ctypes.c_int64(sel.size), S, word_bits, _ptr(out))
        return out

    def planes_to_default(self, planes, R, Kp):
        planes = self._c(planes)
        S = planes.shape[0]
        wb = planes.dtype.itemsize * 8
        out = np.empty((Kp // wb, R, S), dtype=planes.dtype)
        self.lib.sbvr_oracle_planes_to_default(_ptr(planes), ctypes.c_int64(R), ctypes.c_int64(Kp), S, wb, _ptr(out))
        return out

    def planes_to_v1(self, planes, R, Kp):
        planes = self._c(planes, np.uint8)
        S = planes.shape[0]
        out = np.empty((R // 16, Kp // 8, S, 16), dtype=np.uint8)
        self.lib.sbvr_oracle_planes_to_v1(_ptr(planes), ctypes.c_int64(R), ctypes.c_int64(Kp), S, _ptr(out))
        return out

    def idx_to_default(self, flat, R, Kg):
        flat = self._c(flat)
        out = np.empty((Kg, R), dtype=flat.dtype)
        self.lib.sbvr_oracle_idx_to_default(_ptr(flat), ctypes.c_int64(R), ctypes.c_int64(Kg), flat.dtype.itemsize, _ptr(out))
        return out

    def default_to_sel(self, bvr):
        bvr = self._c(bvr)
        Kw, R, S = bvr.shape
        wb = bvr.dtype.itemsize * 8
        out = np.empty((R, Kw * wb), dtype=np.int32)
        self.lib.sbvr_oracle_default_to_sel(_ptr(bvr), ctypes.c_int64(R), ctypes.c_int64(Kw * wb), S, wb, _ptr(out))
        return out

    def decode(self, bvr, coeff_idx, coeff_cache, G, out_cols=None):
        bvr, coeff_idx = self._c(bvr), self._c(coeff_idx)
        cache = self._c(coeff_cache, np.float16)
        Kw, R, S = bvr.shape
        wb = bvr.dtype.itemsize * 8
        Kp = Kw * wb
        Kout = Kp if out_cols is None else out_cols
        out = np.empty((R, Kout), dtype=np.float16)
        self.lib.sbvr_oracle_decode(_ptr(bvr), wb, _ptr(coeff_idx), coeff_idx.dtype.itemsize, _ptr(cache),
                                    ctypes.c_int64(R), ctypes.c_int64(Kp), ctypes.c_int64(Kout), S, G, _ptr(out))
        return out

    def linear_f16(self, x, bvr, coeff_idx, coeff_cache, G, bias=None, mode=0):
        x = self._c(x, np.float16)
        bvr, coeff_idx = self._c(bvr), self._c(coeff_idx)
        cache = self._c(coeff_cache, np.float16)
        Kw, N, S = bvr.shape
        wb = bvr.dtype.itemsize * 8
        M, K = x.shape
        assert K == Kw * wb, (K, Kw, wb)
        b = None
        if bias is not None and bias.size == N:
            b = self._c(bias, np.float16)
        y = np.empty((M, N), dtype=np.float16)
        yd = np.empty((M, N), dtype=np.float64)
        self.lib.sbvr_oracle_linear_f16(_ptr(x), _ptr(bvr), wb, _ptr(coeff_idx), coeff_idx.dtype.itemsize,
                                        _ptr(cache), _ptr(b), ctypes.c_int64(M), ctypes.c_int64(N),
                                        ctypes.c_int64(K), S, G, mode, _ptr(y), _ptr(yd))
        return y, yd

    def mm_T(self, l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias=None):
        l_bvr, l_idx, r_bvr, r_idx = map(self._c, (l_bvr, l_idx, r_bvr, r_idx))
        l_cache, r_cache = self._c(l_cache, np.float16), self._c(r_cache, np.float16)
        Kw, M, Sl = l_bvr.shape
        _, N, Sr = r_bvr.shape
        wb = l_bvr.dtype.itemsize * 8
        assert r_bvr.dtype == l_bvr.dtype and r_bvr.shape[0] == Kw
        b = None
        if bias is not None and bias.size == N:
            b = self._c(bias, np.float16)
        y = np.empty((M, N), dtype=np.float16)
        yd = np.empty((M, N), dtype=np.float64)
        self.lib.sbvr_oracle_mm_T(_ptr(l_bvr), _ptr(l_idx), l_idx.dtype.itemsize, _ptr(l_cache),
                                  _ptr(r_bvr), _ptr(r_idx), r_idx.dtype.itemsize, _ptr(r_cache), _ptr(b),
                                  wb, ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(Kw * wb),
                                  Sl, Sr, G, _ptr(y), _ptr(yd))
        return y, yd

    def mm_T_v1(self, l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias=None, wrap8=False):
        l_bvr, l_idx, r_bvr, r_idx = map(self._c, (l_bvr, l_idx, r_bvr, r_idx))
        l_cache, r_cache = self._c(l_cache, np.float16), self._c(r_cache, np.float16)
        Kb, one, Sl = l_bvr.shape
        assert one == 1 and l_bvr.dtype == np.uint8 and r_bvr.dtype == np.uint8
        N = r_bvr.shape[0] * 16
        Sr = r_bvr.shape[2]
        b = None
        if bias is not None and bias.size == N:
            b = self._c(bias, np.float16)
        y = np.empty((1, N), dtype=np.float16)
        self.lib.sbvr_oracle_mm_T_v1(_ptr(l_bvr), _ptr(l_idx), l_idx.dtype.itemsize, _ptr(l_cache),
                                     _ptr(r_bvr), _ptr(r_idx), r_idx.dtype.itemsize, _ptr(r_cache), _ptr(b),
                                     ctypes.c_int64(N), ctypes.c_int64(Kb * 8), Sl, Sr, G, int(wrap8), _ptr(y))
        return y

    def row_deq_mm_T(self, x, r_bvr, r_idx, r_cache, G, bias=None):
        x = self._c(x, np.float16)
        r_bvr, r_idx = self._c(r_bvr, np.uint32), self._c(r_idx)
        cache = self._c(r_cache, np.float16)
        Nw, K, S = r_bvr.shape
        N = Nw * 32
        M = x.shape[0]
        b = None
        if bias is not None and bias.size == N:
            b = self._c(bias, np.float16)
        y = np.empty((M, N), dtype=np.float16)
        self.lib.sbvr_oracle_row_deq_mm_T(_ptr(x), _ptr(r_bvr), _ptr(r_idx), r_idx.dtype.itemsize, _ptr(cache),
                                          _ptr(b), ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K),
                                          S, G, _ptr(y))
        return y


C = _C()


# ------------------------------------------------------------------ timed CPU port

class _Port:
    """ctypes view of libsbvr_cpu_port.so: the x86 port of the reference's timed
    NEON kernel (sbvr_kernel.cpp:251-399, 471-539) with its pinned thread pool.
    Used as the CPU baseline that bench.py reports beside the GPU figure."""

    def __init__(self):
        self._lib = None

    @property
    def lib(self):
        if self._lib is None:
            path = os.path.join(_HERE, "libsbvr_cpu_port.so")
            if not os.path.exists(path):
                build(targets=("libsbvr_cpu_port.so",))
            lib = ctypes.CDLL(path)
            lib.sbvr_port_isa.restype = ctypes.c_char_p
            lib.sbvr_port_time_mm_T_v1.restype = ctypes.c_double
            self._lib = lib
        return self._lib

    def init_pool(self, threads=-1):
        """-1: one worker per hardware thread, as the reference's import does."""
        return self.lib.sbvr_port_init_pool(int(threads))

    def finalize_pool(self):
        self.lib.sbvr_port_finalize_pool()

    def num_threads(self):
        return self.lib.sbvr_port_num_threads()

    def isa(self):
        return self.lib.sbvr_port_isa().decode()

    def _args(self, l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias):
        c = _C._c
        l_bvr, l_idx, r_bvr, r_idx = c(l_bvr, np.uint8), c(l_idx), c(r_bvr, np.uint8), c(r_idx)
        l_cache, r_cache = c(l_cache, np.float16), c(r_cache, np.float16)
        Kb, one, Sl = l_bvr.shape
        assert one == 1 and r_bvr.ndim == 4 and r_bvr.shape[3] == 16
        N, Sr = r_bvr.shape[0] * 16, r_bvr.shape[2]
        b = c(bias, np.float16) if bias is not None and bias.size == N else None
        out = np.empty((1, N), dtype=np.float16)
        keep = (l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, b, out)
        args = [_ptr(l_bvr), _ptr(l_idx), l_idx.dtype.itemsize, _ptr(l_cache), _ptr(r_bvr), _ptr(r_idx),
                r_idx.dtype.itemsize, _ptr(r_cache), _ptr(b), _ptr(out), N, Kb * 8, Sl, Sr, G]
        return args, out, keep

    def mm_T_v1(self, l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias=None):
        args, out, _keep = self._args(l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias)
        rc = self.lib.sbvr_port_mm_T_v1(*args)
        if rc != 0:
            raise RuntimeError(f"sbvr_port_mm_T_v1 failed: {rc}")
        return out

    def time_mm_T_v1(self, l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias=None, warmup=10, iters=100):
        """Mean seconds per call, timed inside the library."""
        args, _out, _keep = self._args(l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, G, bias)
        t = self.lib.sbvr_port_time_mm_T_v1(*args, int(warmup), int(iters))
        if t < 0:
            raise RuntimeError("sbvr_port_time_mm_T_v1 failed")
        return t


PORT = _Port()
