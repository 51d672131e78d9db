"""Synthetic SBVR encodings with the layout and value ranges of real ones.

The encoder needs about 30 ms per group (hours for one 4096x4096 layer), so
shapes beyond a few hundred groups are filled directly: Bernoulli(1/2) planes,
uniformly drawn line indices and a table of lines shaped like the ones the
encoder finds for N(0, sigma) weights (alternating-sign geometric families,
sorted by magnitude as sbvr/core.py:480-481 of the reference sorts them)."""
import numpy as np
import torch


def make_lines(num_lines, num_sums, sigma=0.02, seed=0):
    """(num_lines, num_sums) fp16 table: c_j = s * (r^j - mean_j r^j) / spread + b / num_sums,
    r in (-2.1, -0.52), sorted by |c_j|."""
    rng = np.random.default_rng(seed)
    r = -rng.uniform(0.52, 2.09, size=(num_lines, 1))
    base = r ** np.arange(num_sums)[None, :]
    combos = ((np.arange(1 << num_sums)[:, None] >> np.arange(num_sums)[None, :]) & 1).astype(np.float64)
    sums = base @ combos.T
    spread = sums.max(1, keepdims=True) - sums.min(1, keepdims=True)
    s = rng.uniform(4.0, 7.0, size=(num_lines, 1)) * sigma
    b = rng.uniform(-0.3, 0.3, size=(num_lines, 1)) * sigma
    lines = s * base / spread
    # the encoder fits zero-mean weights, so the 2^S points of a line straddle zero; with
    # Bernoulli(1/2) planes that takes coefficients summing to (almost) nothing, or every
    # row of the decoded matrix would share one large offset
    lines = lines - lines.mean(1, keepdims=True) + b / num_sums
    order = np.argsort(np.abs(lines), axis=1)
    lines = np.take_along_axis(lines, order, axis=1)
    return torch.from_numpy(lines.astype(np.float16))


def random_encoding(rows, cols, num_sums=4, bvr_len=128, num_lines=256, sigma=0.02, seed=0,
                    device="cpu"):
    """Default-layout arrays of a random (rows, cols) encoded weight:
    bvr (cols/32, rows, S) uint32, coeff_idx (cols/bvr_len, rows), coeff_cache."""
    if cols % bvr_len or bvr_len % 32:
        raise ValueError("cols must be a multiple of bvr_len, bvr_len of 32")
    gen = torch.Generator(device="cpu").manual_seed(seed)
    bvr = torch.randint(-2 ** 31, 2 ** 31, (cols // 32, rows, num_sums), dtype=torch.int32,
                        generator=gen).view(torch.uint32)
    idx = torch.randint(0, num_lines, (cols // bvr_len, rows), dtype=torch.int32, generator=gen)
    idx = idx.to(torch.uint8 if num_lines <= 256 else torch.uint16)
    cache = make_lines(num_lines, num_sums, sigma, seed)
    return bvr.to(device), idx.to(device), cache.to(device)
