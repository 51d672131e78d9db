"""SBVRLinear: the linear layer of models/sbvr_llama.py:66-106 of the reference,
computed in the compressed domain.  The reference's class is a stub whose
intended forward is ``x @ restored_weight.T`` (:86-87); this one holds the three
arrays of an ``sbvr`` object and calls the HIP operator."""
import torch

from . import layout


def _ops():
    """The PyTorch-ROCm extension over the library's C ABI (csrc/sbvr_ops_hip.cpp); there is no fallback."""
    try:
        from . import _sbvr_hip_ops
    except ImportError as exc:
        raise RuntimeError("sbvr._sbvr_hip_ops is not built: run `make -C sbvr-cpu-arm_amd/csrc all` "
                           "(or __graft_entry__.build()); SBVRLinear has no other path") from exc
    return _sbvr_hip_ops


class SBVRLinear(torch.nn.Module):
    def __init__(self, in_features, out_features, bvr, coeff_idx, coeff_cache, bvr_len, bias=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.bvr_len = bvr_len
        self.num_sums = bvr.shape[2]
        self.k_padded = bvr.shape[0] * 32
        self.register_buffer("bvr", bvr)
        self.register_buffer("coeff_idx", coeff_idx)
        self.register_buffer("coeff_cache", coeff_cache)
        self.register_buffer("bias", bias if bias is not None else torch.zeros(0, dtype=torch.float16,
                                                                                 device=bvr.device))

    @classmethod
    def from_sbvr(cls, enc, bias=None):
        """From an ``sbvr`` object that encodes a weight of shape (out, in) in the
        default uint32 layout."""
        out_features, in_features = enc.original_data_shape
        return cls(in_features, out_features, enc.default_layout(torch.uint32), enc.coeff_idx.data,
                   enc.coeff_cache.data, enc.bvr_len, bias)

    @classmethod
    def fused(cls, encs, biases=None):
        """One layer for several ``sbvr`` objects that share their input (q, k, v or
        gate, up): the weights stacked row-wise, see layout.fuse_rows.  The output
        holds the parts' outputs side by side."""
        if any(e.original_data_shape[1] != encs[0].original_data_shape[1] or e.bvr_len != encs[0].bvr_len for e in encs):
            raise ValueError("fused layers must share in_features and the group length")
        bvr, idx, cache = layout.fuse_rows([(e.default_layout(torch.uint32), e.coeff_idx.data, e.coeff_cache.data)
                                            for e in encs])
        bias = None
        if biases is not None:
            bias = torch.cat([b.to(torch.float16) for b in biases])
        return cls(encs[0].original_data_shape[1], sum(e.original_data_shape[0] for e in encs), bvr, idx, cache,
                   encs[0].bvr_len, bias)

    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype != torch.float16:
            x2 = x2.to(torch.float16)
        if x2.shape[1] != self.k_padded:      # the encoder pads K to a multiple of bvr_len
            x2 = torch.nn.functional.pad(x2, (0, self.k_padded - x2.shape[1]))
        x2 = x2.contiguous()
        # any number of rows: the operator picks the decode, 32-row or prefill kernel
        y = _ops()._sbvr_linear_f16(x2, self.bvr, self.coeff_idx, self.coeff_cache, self.bias, self.bvr_len)
        y = y[:, :self.out_features]
        return y.reshape(*lead, self.out_features)
