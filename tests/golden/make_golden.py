"""Writes the golden vectors under tests/golden/ by running the reference's own
`sbvr/core.py` (pure torch; CPU) on tiny seeded tensors, in the container where
/root/reference is mounted.

Only data leaves this script: inputs, the packed tensors the reference produced
(`bvr`, `coeff_idx`, `coeff_cache`), its `decode()` output and one file written by
its `save()`.  They pin the conventions that mathematics cannot fix (plane order,
bit order inside a word, the array layouts selected by `cpu_kernel`,
`cpu_kernel_v2`, `trans`, the padding rule, the on-disk format) and give the
encoder restatement an exact target.

Usage:  python tests/golden/make_golden.py [case ...]
The GPU box has no /root/reference: nothing at test time runs this script.
"""
import importlib.util
import io
import os
import sys
import time
import types
import contextlib

import numpy as np
import torch

REF = "/root/reference/sbvr/core.py"
OUT = os.path.dirname(os.path.abspath(__file__))


def load_reference_core():
    pkg = types.ModuleType("sbvr")
    pkg.__path__ = []
    sys.modules["sbvr"] = pkg
    spec = importlib.util.spec_from_file_location("sbvr.core", REF)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["sbvr.core"] = mod
    spec.loader.exec_module(mod)
    pkg.core = mod
    return mod


# name -> (shape, num_sums, ctor flags, scale)
CASES = {
    "default_s4": ((8, 512), 4, {}, 0.3),
    "default_s2": ((4, 512), 2, {}, 0.3),
    "default_s3": ((4, 512), 3, {}, 0.3),
    "pad_s2": ((3, 300), 2, {}, 0.3),
    "v1_s2": ((32, 512), 2, {"cpu_kernel": True}, 0.3),
    "v1_row_s2": ((1, 512), 2, {"cpu_kernel": True}, 0.3),
    "v2_s2": ((4, 512), 2, {"cpu_kernel_v2": True}, 0.3),
    "trans_s2": ((256, 6), 2, {"trans": True}, 0.3),
    "weights_s4": ((6, 768), 4, {}, 0.02),
    # enough rows for the MFMA kernels (they take 16 columns and more): weights ~ N(0, 0.02)
    "weights_s4_n64": ((64, 512), 4, {}, 0.02),
}


def run_case(core, name):
    shape, num_sums, flags, scale = CASES[name]
    gen = torch.Generator().manual_seed(sum(ord(c) for c in name) * 7919)
    data = (torch.randn(shape, generator=gen, dtype=torch.float32) * scale).to(torch.float16)
    t0 = time.time()
    with contextlib.redirect_stdout(io.StringIO()):
        obj = core.sbvr(data, encoder_config={"num_sums": num_sums},
                        device=torch.device("cpu"), verbose_level=-1, **flags)
        # decode() only understands the 3-D layouts; for the 16-lane v1 array it
        # raises, and the fixture then carries an empty `decoded`.
        dec = obj.decode() if obj.bvr.dim() == 3 else torch.zeros(0, dtype=data.dtype)
    arrs = {
        "data": data.numpy(),
        "bvr": obj.bvr.detach().numpy(),
        "coeff_idx": obj.coeff_idx.detach().numpy(),
        "coeff_cache": obj.coeff_cache.detach().numpy(),
        "decoded": dec.numpy(),
        "num_sums": np.int64(num_sums),
        "bvr_len": np.int64(obj.bvr_len),
        "flags": np.array([int(flags.get("cpu_kernel", False)),
                           int(flags.get("cpu_kernel_v2", False)),
                           int(flags.get("trans", False))], dtype=np.int64),
    }
    np.savez_compressed(os.path.join(OUT, name + ".npz"), **arrs)
    print(f"{name}: bvr{tuple(arrs['bvr'].shape)} {arrs['bvr'].dtype} idx{tuple(arrs['coeff_idx'].shape)} "
          f"{arrs['coeff_idx'].dtype} cache{tuple(arrs['coeff_cache'].shape)} dec{tuple(dec.shape)} "
          f"[{time.time()-t0:.1f}s]", flush=True)
    if name == "default_s2":
        with contextlib.redirect_stdout(io.StringIO()):
            obj.verbose_level = 0
            obj.save(os.path.join(OUT, "default_s2_saved.pt"))


if __name__ == "__main__":
    core = load_reference_core()
    names = sys.argv[1:] or list(CASES)
    for n in names:
        run_case(core, n)
