"""SBVR tensor objects: the API of the reference's sbvr/core.py (class ``sbvr``,
``_sbvr_serialized``, ``load``, ``mm_T``) over this package's own layout and
encoder modules, with the matrix products running on the HIP library.

A tensor W (rows, cols) is held as
  bvr          bit planes, layout chosen by the constructor flags (see layout.py)
  coeff_idx    (cols_padded / bvr_len, rows) uint8 if <= 256 lines else uint16
  coeff_cache  (lines, num_sums) fp16
and W[r, k] ~= sum_j bit_j(r, k) * coeff_cache[coeff_idx[k // bvr_len, r], j]
(reference sbvr/core.py:345-366, 926-949).

Differences from the reference, all additive: ``encoder_config`` accepts
``bvr_len`` (the reference fixes 256, core.py:222); ``from_parts`` builds an object
from existing arrays; ``decode`` is vectorised and understands all three
layouts; nothing is printed unless ``verbose_level`` > 0.
"""
import numpy as np
import torch

from . import layout
from .encoder import EncoderConfig, GroupEncoder, default_batch_size

_NP_DTYPES = {
    "torch.uint8": np.uint8, "torch.uint16": np.uint16, "torch.uint32": np.uint32,
    "torch.int32": np.int32, "torch.float16": np.float16, "torch.float32": np.float32,
}


def _padded(n, multiple):
    return (n + multiple - 1) // multiple * multiple


class _sbvr_serialized():
    """On-disk form written by ``sbvr.save`` (torch.save of this object).  The
    attribute names and the byte-tensor encoding are those of the reference
    (core.py:62-201), so files move between the two implementations."""

    def __init__(self, num_sums, bvr_len, compute_dtype, bvr_dtype, original_dtype,
                 original_data_shape, bvr, coeff_idx, coeff_cache, input_num_sums, input_coeff):
        self.num_sums = num_sums
        self.bvr_len = bvr_len
        self.compute_dtype = compute_dtype
        self.bvr_dtype = bvr_dtype
        if bvr_len % layout.word_bits(bvr_dtype) != 0:
            raise ValueError(f"BVR length must be a multiple of {layout.word_bits(bvr_dtype)}")
        self.original_dtype = original_dtype
        self.original_data_shape = original_data_shape
        self.padded_data_shape = list(original_data_shape)
        self.padded_data_shape[-1] = _padded(original_data_shape[-1], bvr_len)
        if bvr.dtype != bvr_dtype:
            raise ValueError(f"The BVR data type does not match - expected type {bvr_dtype} but got {bvr.dtype}")
        lines = coeff_cache.shape[0]
        if lines > 65536:
            raise ValueError(f"Unsupported number of cache lines, {lines}")
        want = torch.uint8 if lines <= 256 else torch.uint16
        if coeff_idx.dtype != want:
            raise ValueError(f"The coefficient index data type must be {want} but got {coeff_idx.dtype}, "
                             f"number of cache lines: {lines}")
        if coeff_cache.dtype != compute_dtype:
            raise ValueError(f"The coefficient cache data type does not match - expected type "
                             f"{compute_dtype} but got {coeff_cache.dtype}")
        self.bvr = self._serialize_tensor(bvr)
        self.bvr_shape = bvr.shape
        self.coeff_idx = self._serialize_tensor(coeff_idx)
        self.coeff_idx_shape = coeff_idx.shape
        self.coeff_idx_dtype = coeff_idx.dtype
        self.coeff_cache = self._serialize_tensor(coeff_cache)
        self.coeff_cache_shape = coeff_cache.shape
        self.coeff_cache_dtype = coeff_cache.dtype
        self.input_num_sums = input_num_sums
        if input_coeff is not None:
            if input_coeff.dtype != compute_dtype:
                raise ValueError("The input coefficient data type does not match the compute dtype")
            self.input_coeff = self._serialize_tensor(input_coeff)
            self.input_coeff_shape = input_coeff.shape
            self.input_coeff_dtype = input_coeff.dtype
        else:
            self.input_coeff = self.input_coeff_shape = self.input_coeff_dtype = None

    @staticmethod
    def _serialize_tensor(tensor):
        raw = tensor.detach().cpu().contiguous().numpy().tobytes()
        return torch.from_numpy(np.frombuffer(raw, dtype=np.int8).copy())

    @staticmethod
    def _deserialize_tensor(data, shape, dtype):
        np_dtype = _NP_DTYPES.get(str(dtype))
        if np_dtype is None:
            raise ValueError(f"Unsupported dtype: {dtype}")
        arr = np.frombuffer(data.detach().cpu().numpy(), dtype=np_dtype).reshape(tuple(shape)).copy()
        return torch.from_numpy(arr).to(dtype=dtype).contiguous()

    def deserialize_sbvr(self):
        d = self._deserialize_tensor
        input_coeff = None
        if self.input_coeff is not None:
            input_coeff = d(self.input_coeff, self.input_coeff_shape, self.input_coeff_dtype)
        return (self.num_sums, self.bvr_len, self.compute_dtype, self.bvr_dtype, self.original_dtype,
                self.original_data_shape,
                d(self.bvr, self.bvr_shape, self.bvr_dtype),
                d(self.coeff_idx, self.coeff_idx_shape, self.coeff_idx_dtype),
                d(self.coeff_cache, self.coeff_cache_shape, self.coeff_cache_dtype),
                self.input_num_sums, input_coeff)


class sbvr(torch.nn.Module):
    """An SBVR-encoded tensor.  Constructor arguments as core.py:205-215:
    ``data`` to encode or ``sbvr_serialized`` to restore; ``trans`` encodes the
    transpose (groups then run along the original rows); ``cpu_kernel`` /
    ``cpu_kernel_v2`` select the uint8 layouts; with neither, words are uint32."""

    def __init__(self, data=None, encoder_config=None, device=None, sbvr_serialized=None,
                 verbose_level=1, trans=False, cpu_kernel=False, cpu_kernel_v2=False,
                 gpu_tensor_gen=False):
        super().__init__()
        dev = device if device is not None else \
            torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")
        dev = torch.device(dev)
        self.verbose_level = verbose_level
        compute_dtype = torch.float16
        if not cpu_kernel and not cpu_kernel_v2:
            bvr_dtype = torch.uint32
        else:
            bvr_dtype = torch.uint8
            dev = torch.device("cuda:0") if gpu_tensor_gen else torch.device("cpu")
        if data is not None and sbvr_serialized is not None:
            raise ValueError("Cannot provide both data and serialized SBVR")
        if data is None and sbvr_serialized is None:
            raise ValueError("Must provide either data or serialized SBVR")
        self.input_coeff = None
        if data is not None:
            if not isinstance(data, torch.Tensor):
                raise ValueError("Data must be a torch tensor")
            if trans:
                data = data.transpose(0, 1).contiguous()
            conf = EncoderConfig(**(encoder_config or {}))
            self.num_sums = conf.num_sums
            self.bvr_len = conf.bvr_len
            self.compute_dtype = compute_dtype
            self.bvr_dtype = bvr_dtype
            if self.num_sums > 11:
                raise UserWarning("compute_dtype float16 does not have sufficient precision for num_sums > 11.")
            if self.bvr_len % layout.word_bits(bvr_dtype) != 0:
                raise ValueError(f"BVR length must be a multiple of {layout.word_bits(bvr_dtype)}")
            self.original_dtype = data.dtype
            self.original_data_shape = data.shape
            self.input_num_sums = -1
            self._encode(data.to(dev).to(compute_dtype), conf, v1=cpu_kernel and not cpu_kernel_v2)
        else:
            if not isinstance(sbvr_serialized, _sbvr_serialized):
                raise ValueError("Serialized SBVR object is not valid")
            (self.num_sums, self.bvr_len, self.compute_dtype, self.bvr_dtype, self.original_dtype,
             self.original_data_shape, bvr, coeff_idx, coeff_cache, self.input_num_sums,
             input_coeff) = sbvr_serialized.deserialize_sbvr()
            if self.compute_dtype != compute_dtype:
                raise ValueError(f"Compute data type does not match the enforced value, expected "
                                 f"{compute_dtype} but got {self.compute_dtype}")
            if self.bvr_dtype != bvr_dtype:
                raise ValueError(f"BVR data type does not match the enforced value, expected "
                                 f"{bvr_dtype} but got {self.bvr_dtype}")
            self._adopt(bvr.to(dev), coeff_idx.to(dev), coeff_cache.to(dev))
            if input_coeff is not None:
                self.input_coeff = torch.nn.Parameter(input_coeff.to(dev), requires_grad=False)

    # -- construction -----------------------------------------------------------

    @classmethod
    def from_parts(cls, bvr, coeff_idx, coeff_cache, bvr_len, original_shape=None,
                   original_dtype=torch.float16):
        """An object around existing arrays (default or v1 layout), no encoding."""
        self = cls.__new__(cls)
        torch.nn.Module.__init__(self)
        self.verbose_level = 0
        self.num_sums = bvr.shape[2]
        self.bvr_len = bvr_len
        self.compute_dtype = torch.float16
        self.bvr_dtype = bvr.dtype
        self.original_dtype = original_dtype
        self.input_num_sums = -1
        self.input_coeff = None
        rows = bvr.shape[1] if bvr.dim() == 3 else bvr.shape[0] * bvr.shape[3]
        kw = bvr.shape[0] if bvr.dim() == 3 else bvr.shape[1]
        cols = kw * layout.word_bits(bvr.dtype)
        self.original_data_shape = torch.Size(original_shape) if original_shape is not None \
            else torch.Size((rows, cols))
        self._adopt(bvr, coeff_idx, coeff_cache)
        return self

    def _adopt(self, bvr, coeff_idx, coeff_cache):
        self.bvr = torch.nn.Parameter(bvr, requires_grad=False)
        self.coeff_idx = torch.nn.Parameter(coeff_idx, requires_grad=False)
        self.coeff_cache = torch.nn.Parameter(coeff_cache, requires_grad=False)

    def _get_bvr_num_bits(self):
        return layout.word_bits(self.bvr_dtype)

    def _get_padded_data_shape(self):
        shape = list(self.original_data_shape)
        shape[-1] = _padded(shape[-1], self.bvr_len)
        return torch.Size(shape)

    def _get_bin_combs(self):
        return layout.bin_combs(self.num_sums, self.compute_dtype, self.coeff_cache.device)

    def _get_dummy_bias(self):
        """The "no bias" argument of the operators: a 0-length fp16 tensor
        (core.py:353-358)."""
        return torch.zeros([0], dtype=self.compute_dtype, device=self.coeff_cache.device)

    @torch.inference_mode()
    def _encode(self, data, conf, v1):
        """Group-by-group search, then packing into the chosen layout
        (core.py:655-805)."""
        if conf.search_batch_size <= 0:
            conf.search_batch_size = default_batch_size(conf, self.compute_dtype, data.device)
        padded_shape = self._get_padded_data_shape()
        if tuple(padded_shape) != tuple(data.shape):
            padded = torch.zeros(padded_shape, dtype=data.dtype, device=data.device)
            padded[tuple(slice(0, s) for s in data.shape)] = data
        else:
            padded = data
        flat = padded.reshape(-1)
        G = self.bvr_len
        n_groups = flat.numel() // G
        enc = GroupEncoder(conf, self.compute_dtype, data.device, verbose=self.verbose_level)
        line_of = torch.empty(n_groups, dtype=torch.uint16, device=data.device)
        sel = torch.empty(flat.numel(), dtype=torch.int32, device=data.device)
        if self.verbose_level > 0:
            print(conf.describe())
        bar = None
        if self.verbose_level > 0:
            from tqdm import tqdm
            bar = tqdm(total=n_groups, ncols=80, desc="Encoding SBVR groups", unit="g")
        # table look-ups for a block of groups at a time on a GPU; the reference's one-group loop on the CPU
        block = getattr(conf, "group_block", None)
        if block is None:
            block = 512 if data.is_cuda else 1
        line_tmp = torch.empty(n_groups, dtype=torch.int32, device=data.device)
        enc.encode_all(flat, line_tmp, sel, block=block, progress=bar.update if bar is not None else None)
        line_of.copy_(line_tmp.to(torch.uint16) if line_of.dtype == torch.uint16 else line_tmp)
        if bar is not None:
            bar.close()
        rows = flat.numel() // padded_shape[-1]
        planes = layout.sel_to_planes(sel, self.num_sums, self.bvr_dtype)
        if v1 and rows > 1:
            bvr = layout.planes_to_v1(planes, rows)
        else:
            bvr = layout.planes_to_default(planes, rows)
        n_lines = conf.num_coeff_cache_lines
        cache = enc.table[:n_lines].contiguous()
        if n_lines <= 256:
            line_of = line_of.to(torch.uint8)
        coeff_idx = line_of.view(rows, -1).transpose(0, 1).contiguous()
        self._adopt(bvr, coeff_idx, cache)
        self.encoder_stats = {"cache_hits": conf.cache_hits, "lines": n_lines, "groups": n_groups}
        if self.verbose_level > 0:
            print("Encoding complete: %d cache hits, %d lines" % (conf.cache_hits, n_lines))
            print(self.get_sbvr_info())

    # -- views ------------------------------------------------------------------

    def is_v1_layout(self):
        return self.bvr.dim() == 4

    def default_layout(self, dtype=None):
        """``bvr`` in the default (Kw, rows, S) layout, optionally re-worded to
        ``dtype`` (uint32 or uint8)."""
        bvr = self.bvr.data
        if bvr.dim() == 4:
            bvr = layout.planes_to_default(layout.v1_to_planes(bvr).reshape(bvr.shape[2], -1),
                                           bvr.shape[0] * bvr.shape[3])
        return layout.rewidth(bvr, dtype) if dtype is not None else bvr

    def _change_bvr_to_coeff_sel(self):
        """Flat selectors of the padded tensor (core.py:879-901)."""
        return layout.default_to_sel(self.default_layout()).reshape(-1)

    @torch.inference_mode()
    def decode(self):
        """The dense tensor this object stands for, in ``original_dtype``: every
        element is one of its group's 2^S points ``bin_combs @ line``
        (core.py:926-949)."""
        sel = layout.default_to_sel(self.default_layout()).to(torch.int64)          # (rows, Kp)
        rows, kp = sel.shape
        points = (self._get_bin_combs().float() @ self.coeff_cache.data.float().T).T   # (lines, 2^S)
        points = points.to(self.compute_dtype)
        lines = self.coeff_idx.data.to(torch.int64).transpose(0, 1)                  # (rows, Kp/G)
        lines = lines.repeat_interleave(self.bvr_len, dim=1)
        out = points[lines, sel].to(self.original_dtype)
        out = out.view(self._get_padded_data_shape())
        if tuple(self.original_data_shape) != tuple(out.shape):
            out = out[tuple(slice(0, s) for s in self.original_data_shape)]
        return out.contiguous()

    # -- persistence --------------------------------------------------------------

    def _serialize(self):
        return _sbvr_serialized(self.num_sums, self.bvr_len, self.compute_dtype, self.bvr_dtype,
                                self.original_dtype, self.original_data_shape, self.bvr.data,
                                self.coeff_idx.data, self.coeff_cache.data, self.input_num_sums,
                                None if self.input_coeff is None else self.input_coeff.data)

    @torch.inference_mode()
    def save(self, filename):
        if self.verbose_level > 0:
            print("Saving SBVR object to: " + filename)
        torch.save(self._serialize(), filename)

    def get_sbvr_info(self):
        return ("SBVR Info: num_sums=%d bvr_len=%d compute=%s bvr=%s %s original=%s %s idx=%s cache=%s" % (
            self.num_sums, self.bvr_len, self.compute_dtype, self.bvr_dtype, tuple(self.bvr.shape),
            self.original_dtype, tuple(self.original_data_shape), tuple(self.coeff_idx.shape),
            tuple(self.coeff_cache.shape)))

    # -- activations encoded on the fly ------------------------------------------
    # The reference declares this path and leaves its two run-time methods empty (core.py:1021-1027 return
    # None): profile_input finds one line of input coefficients per group of K from sample activations
    # (core.py:971-1019); at run time an activation row is encoded against those lines (every element takes
    # the nearest subset sum of its group's line, the selector rule of the encoder, core.py:492-494) and
    # multiplied with the encoded weight by the both-encoded operator (core.py:1029-1039).

    def _get_padded_input_shape(self, input):
        shape = list(input.shape)
        shape[-1] = _padded(shape[-1], self.bvr_len)
        return torch.Size(shape)

    @torch.inference_mode()
    def profile_input(self, input, encoder_config=None):
        """One line of ``num_sums`` (default 8) input coefficients per group of K, searched over all sample
        rows of ``input`` (..., K) at once; kept in ``input_coeff`` (K / bvr_len, num_sums)."""
        if input.shape[-1] != self.original_data_shape[-1]:
            raise ValueError("Inner dimension shape of the input does not match the original data shape, expected "
                             f"{self.original_data_shape[-1]} but got {input.size(-1)}")
        conf = EncoderConfig(**dict(encoder_config if encoder_config is not None else {"num_sums": 8}))
        dev = self.bvr.device
        padded_shape = self._get_padded_input_shape(input)
        padded = torch.zeros(padded_shape, dtype=self.compute_dtype, device=dev)
        padded[tuple(slice(0, s) for s in input.shape)] = input.to(dev).to(self.compute_dtype)
        groups = padded_shape[-1] // self.bvr_len
        # (all rows' values of one group of K side by side: one search per group of K)
        per_group = padded.view(-1, groups, self.bvr_len).permute(1, 0, 2).contiguous().view(groups, -1)
        conf.bvr_len = per_group.shape[1]
        conf.cache_warmup_num = groups                 # every group gets a line of its own
        if conf.search_batch_size <= 0:
            conf.search_batch_size = default_batch_size(conf, self.compute_dtype, dev)
        enc = GroupEncoder(conf, self.compute_dtype, dev, max_lines=groups, verbose=self.verbose_level)
        for g in range(groups):
            before = conf.num_coeff_cache_lines
            line, _ = enc.encode_group(per_group[g])
            if conf.num_coeff_cache_lines == before:   # (a line equal to an earlier group's: keep one per group)
                enc.table[before] = enc.table[int(line)]
                conf.num_coeff_cache_lines = before + 1
        self.input_num_sums = conf.num_sums
        self.input_coeff = torch.nn.Parameter(enc.table[:groups].clone(), requires_grad=False)

    @torch.inference_mode()
    def _online_tranfrom(self, input):
        """(the reference's spelling) ``input`` (M, K) -> the arrays of an encoded left operand: bvr
        (K/32, M, S_in) uint32, coeff_idx (K / bvr_len, M), coeff_cache = the input coefficients."""
        from . import hip
        if self.input_coeff is None:
            raise RuntimeError("profile_input() has not been run: no input coefficients")
        x = input.reshape(-1, input.shape[-1]).to(self.bvr.device).to(self.compute_dtype)
        k_pad = _padded(x.shape[1], self.bvr_len)
        if x.shape[1] != k_pad:
            x = torch.nn.functional.pad(x, (0, k_pad - x.shape[1]))
        coeff = self.input_coeff.data
        points = coeff @ layout.bin_combs(coeff.shape[1], self.compute_dtype, coeff.device).T
        bvr = hip.online_encode(x.contiguous(), points.contiguous(), self.bvr_len)
        groups = coeff.shape[0]
        idx = torch.arange(groups, device=coeff.device).view(-1, 1).expand(groups, x.shape[0])
        idx = idx.to(torch.uint8 if groups <= 256 else torch.uint16).contiguous()
        return bvr, idx, coeff

    _online_transform = _online_tranfrom

    @torch.inference_mode()
    def online_mm_T(self, rhs, bias=None):
        """``rhs`` (M, K) activations, encoded on the fly against the profiled input coefficients, times this
        encoded weight transposed: (M, N) fp16 through the both-encoded operator."""
        from . import hip
        if bias is None:
            bias = self._get_dummy_bias()
        l_bvr, l_idx, l_cache = self._online_tranfrom(rhs)
        return hip._sbvr_mm_T(l_bvr, l_idx, l_cache, self.default_layout(torch.uint32), self.coeff_idx.data,
                              self.coeff_cache.data, bias)


def mm_T(lhs, rhs, bias):
    """lhs @ rhs^T for two encoded operands in the default uint32 layout
    (core.py:1029-1039)."""
    from . import hip
    if bias is None:
        bias = lhs._get_dummy_bias()
    return hip._sbvr_mm_T(lhs.bvr, lhs.coeff_idx, lhs.coeff_cache,
                          rhs.bvr, rhs.coeff_idx, rhs.coeff_cache, bias)


def load(filename, device=None, verbose_level=1, cpu_kernel=False, cpu_kernel_v2=False) -> sbvr:
    """Restores an object written by ``save`` (core.py:1041-1050).  The file is
    read with the weights-only unpickler; ``_sbvr_serialized`` is registered as a
    safe global by the package."""
    serialized = torch.load(filename, weights_only=True)
    obj = sbvr(sbvr_serialized=serialized, verbose_level=verbose_level, device=device,
               cpu_kernel=cpu_kernel, cpu_kernel_v2=cpu_kernel_v2)
    if verbose_level > 0:
        print("Loaded SBVR object from: " + filename)
        print(obj.get_sbvr_info())
    return obj
