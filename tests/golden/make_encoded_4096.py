"""Writes tests/golden/encoded_4096_s4_g128.npz: a slice and the checksums of the encoding that this
package's encoder makes ON THE GPU (table look-ups for blocks of groups, errors from the HIP search
kernel) of a seeded 4096 x 4096 fp16 weight, 4 planes, groups of 128.  Run on an MI355X from the
repository root:

    python3 tests/golden/make_encoded_4096.py [output.npz]

The GPU test that reads the file (tests/test_gpu_encoder.py) encodes the same weight again and compares."""
import hashlib
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "sbvr-cpu-arm_amd"))

SEED, N, K, S, G, ROWS = 4096, 4096, 4096, 4, 128, 32


def weight():
    return (torch.randn((N, K), generator=torch.Generator().manual_seed(SEED)) * 0.02).to(torch.float16)


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def encode(device):
    import sbvr
    w = weight().to(device)
    torch.cuda.synchronize()
    t0 = time.time()
    enc = sbvr.sbvr(w, encoder_config={"num_sums": S, "bvr_len": G}, device=device, verbose_level=0)
    torch.cuda.synchronize()
    return enc, time.time() - t0


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "encoded_4096_s4_g128.npz")
    enc, seconds = encode(torch.device("cuda:0"))
    bvr, idx, cache = (t.cpu().numpy() for t in (enc.bvr.data, enc.coeff_idx.data, enc.coeff_cache.data))
    np.savez_compressed(out, bvr_rows=bvr[:, :ROWS, :], coeff_idx_rows=idx[:, :ROWS], coeff_cache=cache,
                        sha256_bvr=digest(bvr), sha256_coeff_idx=digest(idx), sha256_coeff_cache=digest(cache),
                        lines=enc.encoder_stats["lines"], cache_hits=enc.encoder_stats["cache_hits"],
                        groups=enc.encoder_stats["groups"], seconds=seconds,
                        shape=np.array([N, K, S, G, SEED]))
    print(f"{out}: {N}x{K} S={S} G={G} encoded in {seconds:.1f} s, {enc.encoder_stats}, "
          f"bvr {digest(bvr)[:16]} idx {digest(idx)[:16]} cache {digest(cache)[:16]}")


if __name__ == "__main__":
    main()
