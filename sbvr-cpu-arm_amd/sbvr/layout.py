"""Bit packing and array layouts of SBVR tensors (torch, any device).

An encoded tensor of R rows and Kp (padded) columns with S planes is described
by one selector per element, ``sel`` in ``[0, 2^S)``: plane ``j`` of an element is
bit ``S-1-j`` of its selector and pairs with coefficient ``j`` of the group's line
(reference sbvr/core.py:345-351, 815-822).  Words hold consecutive elements,
element ``w*bits + i`` in bit ``i`` (core.py:852-869).  Three array layouts exist:

* default  ``bvr (Kp/bits, R, S)``, ``bits`` = 32 (uint32) or 8 (uint8, the
  ``cpu_kernel_v2`` flavour); core.py:726-731, 783
* v1       ``bvr (R/16, Kp/8, S, 16)`` uint8; core.py:754-768
* both with ``coeff_idx (Kp/G, R)``; core.py:774, 794-800
"""
import itertools

import torch

_WORD = {torch.uint32: 32, torch.uint8: 8}


def word_bits(dtype):
    try:
        return _WORD[dtype]
    except KeyError:
        raise ValueError(f"bvr dtype must be uint32 or uint8, got {dtype}") from None


def bin_combs(num_sums, dtype=torch.float16, device="cpu"):
    """(2^S, S) matrix of 0/1; row i is i written MSB first (core.py:345-351)."""
    return torch.tensor(list(itertools.product([0, 1], repeat=num_sums)), dtype=dtype, device=device)


def sel_to_planes(sel, num_sums, dtype):
    """Selectors (numel,) -> planes (S, numel/bits) of ``dtype`` (core.py:842-876)."""
    bits = word_bits(dtype)
    sel = sel.reshape(-1).to(torch.int64)
    shifts = torch.arange(num_sums - 1, -1, -1, device=sel.device, dtype=torch.int64)
    weights = torch.ones(bits, dtype=torch.int64, device=sel.device) << torch.arange(bits, device=sel.device)
    out = torch.empty((num_sums, sel.numel() // bits), dtype=torch.int64, device=sel.device)
    step = 1 << 20
    for lo in range(0, sel.numel(), step):          # bounded temporaries
        part = sel[lo:lo + step]
        b = (part.unsqueeze(0) >> shifts.unsqueeze(1)) & 1                      # (S, n)
        out[:, lo // bits:(lo + part.numel()) // bits] = (b.view(num_sums, -1, bits) * weights).sum(-1)
    if dtype == torch.uint32:
        return _to_u32(out)
    return out.to(torch.uint8)


def _to_u32(x64):
    # values are in [0, 2^32): go through int32 two's complement, then reinterpret
    wrapped = torch.where(x64 >= (1 << 31), x64 - (1 << 32), x64).to(torch.int32)
    return wrapped.view(torch.uint32)


def _as_i64(words):
    """uint32 / uint8 words as non-negative int64."""
    if words.dtype == torch.uint32:
        return words.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    return words.to(torch.int64)


def planes_to_default(planes, rows):
    """(S, rows*Kw) -> (Kw, rows, S) (core.py:726-731, 783)."""
    S = planes.shape[0]
    return planes.view(S, rows, -1).permute(2, 1, 0).contiguous()


def default_to_planes(bvr):
    """(Kw, rows, S) -> (S, rows, Kw) (core.py:881)."""
    return bvr.permute(2, 1, 0).contiguous()


def planes_to_v1(planes, rows):
    """(S, rows*Kw) uint8 -> (rows/16, Kw, S, 16) (core.py:762-764)."""
    S = planes.shape[0]
    if rows % 16:
        raise ValueError("the 16-lane layout needs a multiple of 16 rows")
    return planes.view(S, rows // 16, 16, -1).permute(1, 3, 0, 2).contiguous()


def v1_to_planes(bvr):
    """(rows/16, Kw, S, 16) -> (S, rows, Kw)."""
    r16, Kw, S, lanes = bvr.shape
    return bvr.permute(2, 0, 3, 1).contiguous().view(S, r16 * lanes, Kw)


def planes_to_bits(planes):
    """(S, rows, Kw) words -> (S, rows, Kw*bits) of 0/1 uint8 (core.py:884-895)."""
    bits = word_bits(planes.dtype)
    w = _as_i64(planes)
    sh = torch.arange(bits, device=planes.device, dtype=torch.int64)
    return ((w.unsqueeze(-1) >> sh) & 1).to(torch.uint8).flatten(-2)


def bits_to_sel(bitplanes):
    """(S, ...) of 0/1 -> selectors (...) int32 (core.py:820-822)."""
    S = bitplanes.shape[0]
    w = (1 << torch.arange(S - 1, -1, -1, device=bitplanes.device, dtype=torch.int32))
    return (bitplanes.to(torch.int32) * w.view(-1, *([1] * (bitplanes.dim() - 1)))).sum(0).to(torch.int32)


def default_to_sel(bvr):
    """default bvr -> selectors (rows, Kp) int32 (core.py:879-901)."""
    return bits_to_sel(planes_to_bits(default_to_planes(bvr)))


def rewidth(bvr, dtype):
    """Default layout uint32 <-> uint8: the bit stream of every (row, plane) is the
    same, only the word size changes (core.py:227-230, 753-754)."""
    if bvr.dtype == dtype:
        return bvr
    Kw, R, S = bvr.shape
    if dtype == torch.uint8:      # little endian split of every word
        b = bvr.contiguous().view(torch.uint8).view(Kw, R, S, 4)
        return b.permute(0, 3, 1, 2).reshape(Kw * 4, R, S).contiguous()
    if Kw % 4:
        raise ValueError("byte count per row must be a multiple of 4")
    b = bvr.view(Kw // 4, 4, R, S).permute(0, 2, 3, 1).contiguous()
    return b.view(torch.uint32).view(Kw // 4, R, S)


def fuse_rows(parts):
    """One encoding of the row-wise concatenation of several encoded matrices.

    ``parts``: (bvr (Kw, N_i, S), coeff_idx (Kg, N_i), coeff_cache (L_i, S)) in the
    default layout, all with the same K, group length and plane count.  The
    tables are concatenated and every part's indices are shifted by the lines in
    front of it, so the result decodes to the parts' weights stacked on top of
    each other: q|k|v or gate|up of models/sbvr_llama.py:239, 319-321 as one
    operand (one launch instead of three or two).  Returns (bvr, coeff_idx, coeff_cache)."""
    if not parts:
        raise ValueError("nothing to fuse")
    bvr0, idx0, cache0 = parts[0]
    for bvr, idx, cache in parts:
        if bvr.dim() != 3 or bvr.shape[0] != bvr0.shape[0] or bvr.shape[2] != bvr0.shape[2] or bvr.dtype != bvr0.dtype:
            raise ValueError("parts must share K, the plane count and the word type")
        if idx.shape[0] != idx0.shape[0] or idx.shape[1] != bvr.shape[1] or cache.shape[1] != bvr.shape[2]:
            raise ValueError("parts must share the group length, and their arrays must fit together")
    lines = sum(int(c.shape[0]) for _, _, c in parts)
    if lines > 65536:
        raise ValueError(f"{lines} coefficient lines do not fit 16-bit indices")
    idx_dtype = torch.uint8 if lines <= 256 else torch.uint16
    shifted, base = [], 0
    for _, idx, cache in parts:
        shifted.append((idx.to(torch.int32) + base).to(idx_dtype))
        base += int(cache.shape[0])
    return (torch.cat([b for b, _, _ in parts], dim=1).contiguous(),
            torch.cat(shifted, dim=1).contiguous(),
            torch.cat([c for _, _, c in parts], dim=0).contiguous())
