"""Python binding of libsbvr_hip.so (ctypes over the C ABI of include/sbvr_hip.h).

The functions keep the names, argument order and conventions of the reference's
pybind operators (sbvr/kernels/sbvr_ops.cpp:152-172): sizes are taken from the
tensor shapes, the output is allocated here, "no bias" is a 0-length tensor.
Unlike the reference they check dtype, device and contiguity, and launch on
torch's current HIP stream.  There is no CPU fallback: a missing library or a
tensor that is not on a GPU raises.
"""
import ctypes
import os

import torch

_LIB_NAME = "libsbvr_hip.so"
_lib = None
_workspaces = {}
_outgrown = []        # workspaces that were replaced by larger ones (HIP graphs captured earlier still point at them)


class SbvrHipError(RuntimeError):
    pass


def library_path():
    """The in-tree build, unless SBVR_HIP_LIBRARY names another copy."""
    override = os.environ.get("SBVR_HIP_LIBRARY")
    if override:
        return override
    here = os.path.dirname(os.path.abspath(__file__))
    return os.path.join(os.path.dirname(here), "csrc", _LIB_NAME)


def _load():
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise SbvrHipError(f"{path} is missing: build it with `make -C {os.path.dirname(path)}` "
                           "(or __graft_entry__.build()); there is no fallback path")
    lib = ctypes.CDLL(path)
    vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    lib.sbvr_hip_version.restype = i
    lib.sbvr_hip_last_error.restype = ctypes.c_char_p
    lib.sbvr_hip_last_kernel.restype = i
    lib.sbvr_hip_last_rounding.restype = i
    lib.sbvr_hip_init.argtypes = [i]
    lib.sbvr_hip_linear_f16_workspace.restype = sz
    lib.sbvr_hip_linear_f16_workspace.argtypes = [i, i, i, i, i]
    lib.sbvr_hip_linear_f16.argtypes = [vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, vp, sz, i, vp]
    lib.sbvr_hip_linear_f16_swiglu.argtypes = [vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_linear_f16_add_rmsnorm.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, vp, i, vp, vp, vp,
                                                    i, i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_linear_f16_noalloc.argtypes = [vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, i, vp]
    lib.sbvr_hip_linear_f16_stream_floor.argtypes = [vp, vp, i, vp, vp, i, i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_row_deq_mm_T.argtypes = [vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, vp]
    lib.sbvr_hip_row_deq_mm_T_ws.argtypes = [vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_read_floor.argtypes = [vp, sz, sz, i, i, i, i, i, i, vp, vp]
    lib.sbvr_hip_row_deq_mm_T_workspace.restype = sz
    lib.sbvr_hip_row_deq_mm_T_workspace.argtypes = [i, i]
    lib.sbvr_hip_mm_T.argtypes = [vp, vp, i, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, i, i, vp]
    lib.sbvr_hip_mm_T_ws.argtypes = [vp, vp, i, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_mm_T_workspace.restype = sz
    lib.sbvr_hip_mm_T_workspace.argtypes = [i, i]
    fp = ctypes.POINTER(ctypes.c_float)
    lib.sbvr_hip_dec_add_rmsnorm_f16.argtypes = [vp, vp, vp, vp, i, ctypes.c_float, vp]
    lib.sbvr_hip_dec_attention_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp]
    lib.sbvr_hip_dec_attention_o_supported.argtypes = [i, i, i, i, i, i, i]
    lib.sbvr_hip_dec_attention_o_workspace.restype = sz
    lib.sbvr_hip_dec_attention_o_workspace.argtypes = [i, i]
    lib.sbvr_hip_dec_attention_o_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp, vp, i, vp, vp, vp,
                                                 i, i, i, i, vp, sz, vp]
    lib.sbvr_hip_dec_silu_mul_f16.argtypes = [vp, vp, i, vp]
    lib.sbvr_hip_dec_argmax_advance_f16.argtypes = [vp, i, vp, vp, vp, i, vp, vp, i, vp, vp]
    lib.sbvr_hip_dec_head_argmax_f16.argtypes = [vp, vp, vp, ctypes.c_float, vp, i, i, vp, vp, vp, vp, i, vp, vp, i,
                                                 vp, vp, vp]
    lib.sbvr_hip_dec_head_argmax_embed_f16.argtypes = [vp, vp, vp, ctypes.c_float, vp, i, i, vp, vp, vp, vp, i, vp, vp, i,
                                                       vp, vp, vp, vp, vp]
    lib.sbvr_hip_encoder_group_mse_f16.argtypes = [vp, vp, vp, i, i, i, i, vp]
    lib.sbvr_hip_online_encode_f16.argtypes = [vp, vp, vp, i, i, i, i, vp]
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise SbvrHipError(f"libsbvr_hip: error {rc}: {_load().sbvr_hip_last_error().decode()}")


KERNEL_PORTABLE, KERNEL_DECODE, KERNEL_ROWS32, KERNEL_PREFILL, KERNEL_PREFILL_SPLIT = 1, 2, 3, 4, 5


def last_kernel():
    """Which kernel the last linear call of this thread launched (one of the KERNEL_* codes)."""
    return _load().sbvr_hip_last_kernel()


ROUNDING_EXACT, ROUNDING_DECODE, ROUNDING_PLANEWISE = 1, 2, 3


def last_rounding():
    """How the last linear call of this thread treated the weights: ROUNDING_EXACT (no per-weight rounding),
    ROUNDING_DECODE (each weight rounded to fp16 once, as the reference's decode() does) or ROUNDING_PLANEWISE
    (an fp16 sum built plane by plane)."""
    return _load().sbvr_hip_last_rounding()


def _sbvr_hip_init(device=None):
    """Counterpart of ``_sbvr_cuda_init`` (sbvr_ops.cpp:122-150): verifies the
    device is a gfx950 part."""
    dev = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    _check(_load().sbvr_hip_init(int(dev)))


_sbvr_cuda_init = _sbvr_hip_init


def _want(t, name, dtype=None, dim=None, device=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise SbvrHipError(f"{name} must be on a GPU (got {t.device}); this package has no CPU path")
    if device is not None and t.device != device:
        raise SbvrHipError(f"{name} is on {t.device}, expected {device}")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise TypeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if dim is not None and t.dim() != dim:
        raise ValueError(f"{name} must have {dim} dimensions, got shape {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


def _idx_bytes(idx, lines, name):
    want = torch.uint8 if lines <= 256 else torch.uint16      # sbvr_kernel.cu:931-932
    if idx.dtype != want:
        raise TypeError(f"{name} must be {want} for {lines} coefficient lines, got {idx.dtype}")
    return idx.element_size()


def _bias_ptr(bias, n, device):
    """Bias is used only when its length is N (sbvr_ops.cpp:56-58)."""
    if bias is None or bias.numel() == 0 or bias.size(0) != n:
        return None
    _want(bias, "bias", torch.float16, 1, device)
    return bias.data_ptr()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _workspace(nbytes, device):
    """Zero-initialised scratch per (device, stream); grown on demand.  The
    kernels leave the part that must be zero zeroed.  A buffer that is outgrown
    stays allocated: a HIP graph recorded earlier on the stream keeps its address."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _outgrown.append(ws)
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _linear_operands(K, bvr, coeff_idx, coeff_cache, bvr_len, out, M, dev):
    """Shape and dtype checks shared by the linear's entry points; returns
    (N, S, G, L, idx_bytes, out, workspace)."""
    lib = _load()
    _want(bvr, "bvr", torch.uint32, 3, dev)
    _want(coeff_idx, "coeff_idx", (torch.uint8, torch.uint16), 2, dev)
    _want(coeff_cache, "coeff_cache", torch.float16, 2, dev)
    Kw, N, S = bvr.shape
    L = coeff_cache.shape[0]
    if Kw * 32 != K:
        raise ValueError(f"x has K={K} but bvr holds {Kw * 32} columns")
    if coeff_idx.shape[1] != N or coeff_cache.shape[1] != S:
        raise ValueError("coeff_idx / coeff_cache shapes do not match bvr")
    G = bvr_len if bvr_len is not None else K // coeff_idx.shape[0]
    if G * coeff_idx.shape[0] != K:
        raise ValueError(f"coeff_idx has {coeff_idx.shape[0]} groups, K={K}, bvr_len={G}")
    ib = _idx_bytes(coeff_idx, L, "coeff_idx")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
    else:
        _want(out, "out", torch.float16, 2, dev)
        if tuple(out.shape) != (M, N):
            raise ValueError("out has the wrong shape")
    need = lib.sbvr_hip_linear_f16_workspace(M, N, K, S, G)
    ws = _workspace(need, dev) if need else None
    return N, S, G, L, ib, out, ws


def _sbvr_linear_f16(x, bvr, coeff_idx, coeff_cache, bias=None, bvr_len=None, out=None, flags=0):
    """y = x @ decode(W)^T (+ bias) for fp16 ``x`` (M, K) and a weight in the
    default uint32 layout: ``bvr`` (K/32, N, S), ``coeff_idx`` (K/G, N),
    ``coeff_cache`` (L, S).  Returns fp16 (M, N)."""
    lib = _load()
    dev = x.device
    _want(x, "x", torch.float16, 2)
    M, K = x.shape
    N, S, G, L, ib, out, ws = _linear_operands(K, bvr, coeff_idx, coeff_cache, bvr_len, out, M, dev)
    with torch.cuda.device(dev):
        _check(lib.sbvr_hip_linear_f16(
            x.data_ptr(), bvr.data_ptr(), coeff_idx.data_ptr(), ib, coeff_cache.data_ptr(),
            _bias_ptr(bias, N, dev), out.data_ptr(), M, N, K, S, G, L,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            int(flags), _stream()))
    return out


def _sbvr_linear_f16_swiglu(gate_up, bvr, coeff_idx, coeff_cache, bias=None, bvr_len=None, out=None):
    """``_sbvr_linear_f16`` of the row fp16(fp16(silu(gate)) * up) for ``gate_up``
    (1, 2K) = gate | up, without materialising that row (one launch)."""
    lib = _load()
    dev = gate_up.device
    _want(gate_up, "gate_up", torch.float16, 2)
    M, K2 = gate_up.shape
    if K2 % 2:
        raise ValueError("gate_up must have an even number of columns")
    K = K2 // 2
    N, S, G, L, ib, out, ws = _linear_operands(K, bvr, coeff_idx, coeff_cache, bvr_len, out, M, dev)
    with torch.cuda.device(dev):
        _check(lib.sbvr_hip_linear_f16_swiglu(
            gate_up.data_ptr(), bvr.data_ptr(), coeff_idx.data_ptr(), ib, coeff_cache.data_ptr(),
            _bias_ptr(bias, N, dev), out.data_ptr(), M, N, K, S, G, L,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream()))
    return out


def _sbvr_linear_f16_add_rmsnorm(x, delta, norm_weight, eps, x_out, bvr, coeff_idx, coeff_cache, bias=None,
                                 bvr_len=None, out=None):
    """``x_out`` <- r = fp16(x + delta); returns ``_sbvr_linear_f16`` of the row
    norm_weight * fp16(r * rsqrt(mean(r^2) + eps)), in one launch.  ``x``,
    ``delta``, ``x_out``: (1, K) fp16, three different buffers."""
    lib = _load()
    dev = x.device
    _want(x, "x", torch.float16, 2)
    _want(delta, "delta", torch.float16, 2, dev)
    _want(x_out, "x_out", torch.float16, 2, dev)
    _want(norm_weight, "norm_weight", torch.float16, 1, dev)
    M, K = x.shape
    if M != 1 or tuple(delta.shape) != (1, K) or tuple(x_out.shape) != (1, K) or norm_weight.shape[0] != K:
        raise ValueError("x, delta and x_out must be (1, K) and norm_weight (K)")
    N, S, G, L, ib, out, ws = _linear_operands(K, bvr, coeff_idx, coeff_cache, bvr_len, out, 1, dev)
    with torch.cuda.device(dev):
        _check(lib.sbvr_hip_linear_f16_add_rmsnorm(
            x.data_ptr(), delta.data_ptr(), norm_weight.data_ptr(), float(eps), x_out.data_ptr(),
            bvr.data_ptr(), coeff_idx.data_ptr(), ib, coeff_cache.data_ptr(),
            _bias_ptr(bias, N, dev), out.data_ptr(), N, K, S, G, L,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream()))
    return out


def _sbvr_linear_f16_stream_floor(bvr, coeff_idx, coeff_cache, bvr_len=None, out=None):
    """Measurement aid: the one-row launch of ``_sbvr_linear_f16`` for this weight with only
    its plane-word and index requests left in (no arithmetic, ``out`` is not written)."""
    lib = _load()
    dev = bvr.device
    K = bvr.shape[0] * 32
    N, S, G, L, ib, out, ws = _linear_operands(K, bvr, coeff_idx, coeff_cache, bvr_len, out, 1, dev)
    with torch.cuda.device(dev):
        _check(lib.sbvr_hip_linear_f16_stream_floor(
            bvr.data_ptr(), coeff_idx.data_ptr(), ib, coeff_cache.data_ptr(), out.data_ptr(), N, K, S, G, L,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream()))
    return out


_read_sinks = {}


def read_floor(buf, nbytes, workgroups, waves, ahead, pattern=0, row_bytes=0, win_bytes=0):
    """Measurement aid (``sbvr_hip_read_floor``): a launch of ``workgroups`` x ``waves`` waves that only reads
    ``nbytes`` of the tensor ``buf``, 1 KiB per wave request, ``ahead`` requests of a wave in flight."""
    lib = _load()
    dev = buf.device
    sink = _read_sinks.get(dev)
    if sink is None:
        sink = _read_sinks[dev] = torch.zeros(64, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _check(lib.sbvr_hip_read_floor(buf.data_ptr(), buf.numel() * buf.element_size(), nbytes, workgroups, waves,
                                       ahead, pattern, row_bytes, win_bytes, sink.data_ptr(), _stream()))


def _sbvr_row_deq_mm_T(l_w, r_bvr, r_coeff_idx, r_coeff_cache, bias, use_shfl=0, bvr_len=None):
    """fp16 ``l_w`` (M, K) against a ``trans=True`` weight: ``r_bvr`` (N/32, K, S),
    ``r_coeff_idx`` (N/G, K) (sbvr_ops.cpp:79-120).  ``use_shfl`` selected between
    equivalent CUDA kernels in the reference and is ignored."""
    lib = _load()
    dev = l_w.device
    _want(l_w, "l_w", torch.float16, 2)
    _want(r_bvr, "r_bvr", torch.uint32, 3, dev)
    _want(r_coeff_idx, "r_coeff_idx", (torch.uint8, torch.uint16), 2, dev)
    _want(r_coeff_cache, "r_coeff_cache", torch.float16, 2, dev)
    M, K = l_w.shape
    Nw, K2, S = r_bvr.shape
    N = Nw * 32
    L = r_coeff_cache.shape[0]
    if K2 != K or r_coeff_idx.shape[1] != K or r_coeff_cache.shape[1] != S:
        raise ValueError("operand shapes do not match")
    G = bvr_len if bvr_len is not None else N // r_coeff_idx.shape[0]
    ib = _idx_bytes(r_coeff_idx, L, "r_coeff_idx")
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        need = lib.sbvr_hip_row_deq_mm_T_workspace(M, N)
        ws = _workspace(need, dev) if need else None          # (0: the call does not split K)
        _check(lib.sbvr_hip_row_deq_mm_T_ws(l_w.data_ptr(), r_bvr.data_ptr(), r_coeff_idx.data_ptr(), ib,
                                            r_coeff_cache.data_ptr(), _bias_ptr(bias, N, dev), out.data_ptr(),
                                            M, N, K, S, G, L, ws.data_ptr() if need else None, need, _stream()))
    return out


def _sbvr_mm_T(l_bvr, l_coeff_idx, l_coeff_cache, r_bvr, r_coeff_idx, r_coeff_cache, bias, bvr_len=None):
    """Both operands encoded, default uint32 layout: ``l_bvr`` (K/32, M, Sl),
    ``r_bvr`` (K/32, N, Sr) (sbvr_ops.cpp:35-76).  Returns fp16 (M, N)."""
    lib = _load()
    dev = l_bvr.device
    _want(l_bvr, "l_bvr", torch.uint32, 3)
    _want(r_bvr, "r_bvr", torch.uint32, 3, dev)
    _want(l_coeff_idx, "l_coeff_idx", (torch.uint8, torch.uint16), 2, dev)
    _want(r_coeff_idx, "r_coeff_idx", (torch.uint8, torch.uint16), 2, dev)
    _want(l_coeff_cache, "l_coeff_cache", torch.float16, 2, dev)
    _want(r_coeff_cache, "r_coeff_cache", torch.float16, 2, dev)
    Kw, M, Sl = l_bvr.shape
    Kw2, N, Sr = r_bvr.shape
    if Kw != Kw2:
        raise ValueError(f"operands disagree on K: {Kw * 32} vs {Kw2 * 32}")
    K = Kw * 32
    G = bvr_len if bvr_len is not None else K // l_coeff_idx.shape[0]
    if l_coeff_idx.shape != (K // G, M) or r_coeff_idx.shape != (K // G, N):
        raise ValueError("coeff_idx shapes do not match the operands")
    Ll, Lr = l_coeff_cache.shape[0], r_coeff_cache.shape[0]
    out = torch.empty((M, N), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        need = lib.sbvr_hip_mm_T_workspace(M, N)
        ws = _workspace(need, dev) if need else None          # (0: the call does not split K)
        _check(lib.sbvr_hip_mm_T_ws(l_bvr.data_ptr(), l_coeff_idx.data_ptr(), _idx_bytes(l_coeff_idx, Ll, "l_coeff_idx"),
                                    l_coeff_cache.data_ptr(), r_bvr.data_ptr(), r_coeff_idx.data_ptr(),
                                    _idx_bytes(r_coeff_idx, Lr, "r_coeff_idx"), r_coeff_cache.data_ptr(),
                                    _bias_ptr(bias, N, dev), out.data_ptr(), M, N, K, Sl, Sr, G, Ll, Lr,
                                    ws.data_ptr() if need else None, need, _stream()))
    return out


# -- single-token helpers of the decoder (include/sbvr_hip_decoder.h) ------------

def _dec_check(rc, what):
    if rc != 0:
        raise SbvrHipError(f"libsbvr_hip: {what} failed with {rc}")


def dec_add_rmsnorm(x, delta, weight, h, eps):
    """x (n,) fp16 updated in place with `delta` (or None); h <- weight * norm(x)."""
    for t, name in ((x, "x"), (weight, "weight"), (h, "h")) + (((delta, "delta"),) if delta is not None else ()):
        _want(t, name, torch.float16)
    _dec_check(_load().sbvr_hip_dec_add_rmsnorm_f16(x.data_ptr(), delta.data_ptr() if delta is not None else None,
                                                     weight.data_ptr(), h.data_ptr(), x.numel(), float(eps),
                                                     _stream()), "add_rmsnorm")
    return h


def dec_attention(qkv, cos, sin, pos, kcache, vcache, ctx, heads, kv_heads, head_dim, rot_now=None):
    """Rotary embedding, cache append at *pos and attention of the new token.
    ``rot_now``: row *pos of cos | sin (head_dim floats) when the caller keeps it
    up to date (dec_argmax_advance does), which saves the kernel a round trip."""
    for t, name in ((qkv, "qkv"), (kcache, "kcache"), (vcache, "vcache"), (ctx, "ctx")):
        _want(t, name, torch.float16)
    _want(cos, "cos", torch.float32)
    _want(sin, "sin", torch.float32)
    _want(pos, "pos", torch.int64)
    max_seq = kcache.shape[1]
    if kcache.shape != (kv_heads, max_seq, head_dim) or vcache.shape != kcache.shape or \
            cos.shape != (max_seq, head_dim // 2) or sin.shape != cos.shape or \
            qkv.numel() != (heads + 2 * kv_heads) * head_dim or ctx.numel() != heads * head_dim:
        raise SbvrHipError("dec_attention: tensor shapes do not match heads/kv_heads/head_dim/max_seq")
    if rot_now is not None:
        _want(rot_now, "rot_now", torch.float32)
        if rot_now.numel() != head_dim:
            raise SbvrHipError("dec_attention: rot_now must hold head_dim floats")
    _dec_check(_load().sbvr_hip_dec_attention_f16(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                                                   rot_now.data_ptr() if rot_now is not None else None,
                                                   pos.data_ptr(), kcache.data_ptr(), vcache.data_ptr(),
                                                   ctx.data_ptr(), heads, kv_heads, head_dim, max_seq, _stream()),
               "attention")
    return ctx


def dec_attention_o_supported(heads, kv_heads, head_dim, max_seq, N, S, G):
    """Whether ``dec_attention_o`` takes this shape (else: ``dec_attention``, then the linear)."""
    return bool(_load().sbvr_hip_dec_attention_o_supported(heads, kv_heads, head_dim, max_seq, N, S, G))


def attention_o_cache_layout(cache, inverse=False, values=False):
    """(kv_heads, max_seq, 128) fp16 in the natural order -> the blocked order ``dec_attention_o`` keeps its caches
    in (same shape, other element order), or back with ``inverse``.  Keys: blocks of 16 positions, each as four
    runs (dimensions 32 j .. 32 j + 31) of [dimension % 32 // 8][position % 16][dimension % 8].  Values: blocks of
    32 positions, each as eight runs (dimensions 16 b .. 16 b + 15) of [position % 32 // 8][dimension % 16][position % 8]."""
    kv, T, D = cache.shape
    if D != 128 or T % 32:
        raise ValueError("attention_o_cache_layout: head_dim 128 and max_seq a multiple of 32")
    if not values:
        if not inverse:       # (tb, col, j, blk, i) -> (tb, j, blk, col, i)
            return cache.view(kv, T // 16, 16, 4, 4, 8).permute(0, 1, 3, 4, 2, 5).contiguous().view(kv, T, D)
        return cache.view(kv, T // 16, 4, 4, 16, 8).permute(0, 1, 4, 2, 3, 5).contiguous().view(kv, T, D)
    if not inverse:           # (pb, blk, i, db, col) -> (pb, db, blk, col, i)
        return cache.view(kv, T // 32, 4, 8, 8, 16).permute(0, 1, 4, 2, 5, 3).contiguous().view(kv, T, D)
    return cache.view(kv, T // 32, 8, 4, 16, 8).permute(0, 1, 3, 5, 2, 4).contiguous().view(kv, T, D)


def dec_attention_o(qkv, cos, sin, pos, kcache, vcache, heads, kv_heads, head_dim, bvr, coeff_idx, coeff_cache,
                    bias=None, bvr_len=None, out=None, rot_now=None, ctx=None):
    """``dec_attention`` and the encoded output projection of its context row in one launch.  Both caches are
    (kv_heads, max_seq, head_dim) fp16 in the blocked element order of ``attention_o_cache_layout``.  ``ctx``
    (heads * head_dim fp16), when given, receives the context row.  Returns ``out`` (1, N)."""
    lib = _load()
    dev = qkv.device
    for t, name in ((qkv, "qkv"), (kcache, "kcache"), (vcache, "vcache")) + (((ctx, "ctx"),) if ctx is not None else ()):
        _want(t, name, torch.float16, None, dev)
    _want(cos, "cos", torch.float32, None, dev)
    _want(sin, "sin", torch.float32, None, dev)
    _want(pos, "pos", torch.int64, None, dev)
    max_seq = kcache.shape[1]
    if kcache.shape != (kv_heads, max_seq, head_dim) or vcache.shape != kcache.shape or \
            cos.shape != (max_seq, head_dim // 2) or sin.shape != cos.shape or \
            qkv.numel() != (heads + 2 * kv_heads) * head_dim or (ctx is not None and ctx.numel() != heads * head_dim):
        raise SbvrHipError("dec_attention_o: tensor shapes do not match heads/kv_heads/head_dim/max_seq")
    if rot_now is not None:
        _want(rot_now, "rot_now", torch.float32, None, dev)
        if rot_now.numel() != head_dim:
            raise SbvrHipError("dec_attention_o: rot_now must hold head_dim floats")
    K = heads * head_dim
    _want(bvr, "bvr", torch.uint32, 3, dev)
    _want(coeff_idx, "coeff_idx", (torch.uint8, torch.uint16), 2, dev)
    _want(coeff_cache, "coeff_cache", torch.float16, 2, dev)
    Kw, N, S = bvr.shape
    L = coeff_cache.shape[0]
    if Kw * 32 != K or coeff_idx.shape[1] != N or coeff_cache.shape[1] != S:
        raise ValueError("the projection's bvr / coeff_idx / coeff_cache do not match heads * head_dim")
    G = bvr_len if bvr_len is not None else K // coeff_idx.shape[0]
    if G * coeff_idx.shape[0] != K:
        raise ValueError(f"coeff_idx has {coeff_idx.shape[0]} groups, K={K}, bvr_len={G}")
    ib = _idx_bytes(coeff_idx, L, "coeff_idx")
    if out is None:
        out = torch.empty((1, N), dtype=torch.float16, device=dev)
    else:
        _want(out, "out", torch.float16, 2, dev)
        if tuple(out.shape) != (1, N):
            raise ValueError("out has the wrong shape")
    with torch.cuda.device(dev):
        need = lib.sbvr_hip_dec_attention_o_workspace(kv_heads, N)
        ws = _workspace(need, dev) if need else None
        _check(lib.sbvr_hip_dec_attention_o_f16(
            qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), rot_now.data_ptr() if rot_now is not None else None,
            pos.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), ctx.data_ptr() if ctx is not None else None,
            heads, kv_heads, head_dim, max_seq, bvr.data_ptr(), coeff_idx.data_ptr(), ib, coeff_cache.data_ptr(),
            _bias_ptr(bias, N, dev), out.data_ptr(), N, S, G, L,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream()))
    return out


def dec_silu_mul(gate_up, out):
    _want(gate_up, "gate_up", torch.float16)
    _want(out, "out", torch.float16)
    if gate_up.numel() != 2 * out.numel():
        raise SbvrHipError("dec_silu_mul: gate_up must hold 2 * out.numel() elements")
    _dec_check(_load().sbvr_hip_dec_silu_mul_f16(gate_up.data_ptr(), out.data_ptr(), out.numel(), _stream()),
               "silu_mul")
    return out


def dec_argmax_advance(logits, token, generated, pos, cos=None, sin=None, rot_now=None):
    """token <- argmax(logits); generated[pos] <- token; pos <- pos + 1 (all on the device).
    With ``rot_now`` (head_dim floats) and the rotary tables, also rot_now <- cos | sin of the new position."""
    _want(logits, "logits", torch.float16)
    for t, name in ((token, "token"), (generated, "generated"), (pos, "pos")):
        _want(t, name, torch.int64)
    head_dim = 0
    if rot_now is not None:
        for t, name in ((cos, "cos"), (sin, "sin"), (rot_now, "rot_now")):
            _want(t, name, torch.float32)
        head_dim = rot_now.numel()
        if cos.shape != (generated.numel(), head_dim // 2) or sin.shape != cos.shape:
            raise SbvrHipError("dec_argmax_advance: rotary tables must be (max_seq, head_dim / 2)")
    _dec_check(_load().sbvr_hip_dec_argmax_advance_f16(logits.data_ptr(), logits.numel(), token.data_ptr(),
                                                        generated.data_ptr(), pos.data_ptr(), generated.numel(),
                                                        cos.data_ptr() if rot_now is not None else None,
                                                        sin.data_ptr() if rot_now is not None else None, head_dim,
                                                        rot_now.data_ptr() if rot_now is not None else None,
                                                        _stream()), "argmax_advance")


def dec_head_argmax_supported(hidden):
    """Whether dec_head_argmax has a kernel for this hidden size."""
    return hidden in (512, 1024, 2048, 4096, 8192)


def dec_head_argmax(x, delta, weight, eps, head, logits, token, generated, pos, workspace, cos=None, sin=None,
                    rot_now=None, embed=None, x_next=None):
    """Final residual add + RMSNorm, fp16 output head, argmax and position advance in one launch.
    ``head`` (vocab, hidden) fp16; ``logits`` (vocab,) fp16 or None; ``workspace``: two int64 zeros.
    ``embed`` (vocab, hidden) fp16 and ``x_next`` (hidden): the chosen token's embedding row is left in ``x_next``
    (which may be ``x``) for the next step."""
    for t, name in ((x, "x"), (weight, "weight"), (head, "head")) + (((delta, "delta"),) if delta is not None else ()) \
            + (((logits, "logits"),) if logits is not None else ()):
        _want(t, name, torch.float16)
    for t, name in ((token, "token"), (generated, "generated"), (pos, "pos"), (workspace, "workspace")):
        _want(t, name, torch.int64)
    vocab, hidden = head.shape
    if x.numel() != hidden or weight.numel() != hidden or workspace.numel() < 2 or \
            (logits is not None and logits.numel() != vocab):
        raise SbvrHipError("dec_head_argmax: tensor shapes do not match the head")
    head_dim = 0
    if rot_now is not None:
        for t, name in ((cos, "cos"), (sin, "sin"), (rot_now, "rot_now")):
            _want(t, name, torch.float32)
        head_dim = rot_now.numel()
        if cos.shape != (generated.numel(), head_dim // 2) or sin.shape != cos.shape:
            raise SbvrHipError("dec_head_argmax: rotary tables must be (max_seq, head_dim / 2)")
    if (embed is None) != (x_next is None):
        raise SbvrHipError("dec_head_argmax: embed and x_next go together")
    if embed is not None:
        _want(embed, "embed", torch.float16, 2)
        _want(x_next, "x_next", torch.float16)
        if tuple(embed.shape) != (vocab, hidden) or x_next.numel() != hidden:
            raise SbvrHipError("dec_head_argmax: embed must be (vocab, hidden) and x_next hold hidden elements")
    _dec_check(_load().sbvr_hip_dec_head_argmax_embed_f16(
        x.data_ptr(), delta.data_ptr() if delta is not None else None, weight.data_ptr(), float(eps), head.data_ptr(),
        vocab, hidden, logits.data_ptr() if logits is not None else None, token.data_ptr(), generated.data_ptr(),
        pos.data_ptr(), generated.numel(), cos.data_ptr() if rot_now is not None else None,
        sin.data_ptr() if rot_now is not None else None, head_dim,
        rot_now.data_ptr() if rot_now is not None else None, workspace.data_ptr(),
        embed.data_ptr() if embed is not None else None, x_next.data_ptr() if embed is not None else None, _stream()),
        "head_argmax")
    return logits


def encoder_group_mse(data, points):
    """mse[b, l] = mean_g min_p (data[b, g] - points[l, p])^2 in the encoder's arithmetic (fp16 difference
    and square, fp32 sum in element order): data (groups, G) fp16, points (n, P) fp16 -> (groups, n) fp32.
    The error evaluation of the reference's search (sbvr/core.py:485-495) for many groups at once."""
    _want(data, "data", torch.float16, 2)
    _want(points, "points", torch.float16, 2, data.device)
    groups, G = data.shape
    n, P = points.shape
    out = torch.empty((groups, n), dtype=torch.float32, device=data.device)
    with torch.cuda.device(data.device):
        done = 0
        while done < groups:          # (a launch takes at most 65535 groups)
            take = min(groups - done, 65535)
            rc = _load().sbvr_hip_encoder_group_mse_f16(data[done:done + take].data_ptr(), points.data_ptr(),
                                                        out[done:done + take].data_ptr(), take, G, n, P, _stream())
            if rc != 0:
                raise SbvrHipError(f"sbvr_hip_encoder_group_mse_f16: error {rc} (groups={take} G={G} n={n} P={P})")
            done += take
    return out


def encoder_group_mse_supported(dtype, G, P):
    return dtype == torch.float16 and P in (2, 4, 8, 16, 32, 64, 128, 256)


def online_encode(x, points, bvr_len):
    """Activations to bit planes on the fly: x (M, K) fp16 and the 2^S subset sums of every K-group's input
    coefficients, points (K / bvr_len, 2^S) fp16 -> bvr (K/32, M, S) uint32 in the default layout."""
    _want(x, "x", torch.float16, 2)
    _want(points, "points", torch.float16, 2, x.device)
    M, K = x.shape
    S = points.shape[1].bit_length() - 1
    if points.shape[1] != 1 << S or K % bvr_len != 0 or points.shape[0] != K // bvr_len:
        raise ValueError(f"points must be (K / bvr_len, 2^S), got {tuple(points.shape)} for K={K}, bvr_len={bvr_len}")
    bvr = torch.empty((K // 32, M, S), dtype=torch.uint32, device=x.device)
    with torch.cuda.device(x.device):
        rc = _load().sbvr_hip_online_encode_f16(x.data_ptr(), points.data_ptr(), bvr.data_ptr(), M, K, bvr_len, S, _stream())
    if rc != 0:
        raise SbvrHipError(f"sbvr_hip_online_encode_f16: error {rc} (M={M} K={K} bvr_len={bvr_len} S={S})")
    return bvr
