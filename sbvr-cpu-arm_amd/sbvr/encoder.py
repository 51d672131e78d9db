"""SBVR encoder: per group of ``bvr_len`` values, search a line of ``num_sums``
fp16 coefficients whose 2^S subset sums approximate the group best (MSE), and
reuse earlier lines through a table (the "coefficient cache").

This is the reference's CPU/torch algorithm (sbvr/core.py:19-60 configuration,
:368-483 search spaces, :485-553 search, :555-653 per-group policy) restated;
run on the same device with the same configuration it makes the same torch
calls in the same order, so it yields the same lines and selectors.  It is not
a GPU kernel and is not on the hot path.
"""
import math

import torch

from . import layout


class EncoderConfig:
    """Search parameters; keyword names and defaults of core.py:19-38."""

    DEFAULTS = dict(
        num_sums=4, r_search_num=64, b_search_num=40, s_search_num=40,
        error_function="data_diff_mse", mse_window_size=20, search_extend_ratio=1.2,
        coeff_cache=None, cache_warmup_num=10, acceptable_mse=10 ** -12, mse_history=None,
        search_batch_size=0, group_idx=0, cache_hits=0, num_coeff_cache_lines=0,
        extend_ratio=1.2, input_tensor=None, input_vectors=None,
    )

    def __init__(self, **kwargs):
        unknown = set(kwargs) - set(self.DEFAULTS) - {"bvr_len"}
        if unknown:
            raise TypeError(f"unknown encoder option(s): {sorted(unknown)}")
        for k, v in self.DEFAULTS.items():
            setattr(self, k, kwargs.get(k, v))
        if self.mse_history is None:
            self.mse_history = []
        # extension: the reference fixes the group length at 256 (core.py:222)
        self.bvr_len = kwargs.get("bvr_len", 256)

    def describe(self):
        return ("SBVR encoder: num_sums=%d bvr_len=%d r/b/s search=%d/%d/%d window=%d extend=%.2f/%.2f "
                "warmup=%d acceptable_mse=%g batch=%d" % (
                    self.num_sums, self.bvr_len, self.r_search_num, self.b_search_num, self.s_search_num,
                    self.mse_window_size, self.search_extend_ratio, self.extend_ratio,
                    self.cache_warmup_num, self.acceptable_mse, self.search_batch_size))


class GroupEncoder:
    """State of one encoding run: the line table and the hit statistics."""

    def __init__(self, conf, dtype, device, max_lines=1 << 16, verbose=0):
        self.conf = conf
        self.S = conf.num_sums
        self.dtype = dtype
        self.device = device
        self.verbose = verbose
        self.combs = layout.bin_combs(self.S, dtype, device)                 # (2^S, S)
        self.table = torch.zeros((max_lines, self.S), dtype=dtype, device=device)
        conf.coeff_cache = self.table

    # -- candidate lines ------------------------------------------------------

    def _family_space(self, r_list, b_list, s_list):
        """Geometric families c_j = b + s * r^j / spread (core.py:392-403)."""
        expo = torch.arange(self.S, device=r_list.device)
        base = r_list.unsqueeze(1) ** expo.unsqueeze(0)
        sums = base @ self.combs.T
        spread = sums.max(dim=1)[0] - sums.min(dim=1)[0]
        base = base / spread.unsqueeze(1)
        scaled = s_list.view(-1, 1, 1) * base.unsqueeze(0)
        shifted = b_list.view(-1, 1, 1, 1) + scaled.unsqueeze(0)
        return shifted.view(-1, self.S)

    def _grid_space(self, data, extended):
        """Cartesian grid around equal slices of the data range (core.py:368-390)."""
        c = self.conf
        budget = c.r_search_num * c.b_search_num * c.s_search_num * 1.4
        if extended:
            budget *= c.search_extend_ratio ** 3
        per_dim = int(budget ** (1 / self.S))
        lo, hi = torch.min(data), torch.max(data)
        edges = torch.linspace(lo, hi, self.S + 1, device=data.device, dtype=data.dtype)
        axes = []
        for i in range(self.S):
            margin = abs(edges[i]) * 0.8
            axes.append(torch.linspace(edges[i] - margin, edges[i + 1] + margin, per_dim + 1,
                                       device=data.device, dtype=data.dtype))
        return torch.cartesian_prod(*axes)

    def candidate_lines(self, data, extended):
        """All candidate lines for one group, coefficients ordered by magnitude
        (core.py:405-483).  Returns (lines, r_list, b_list, s_list, n_family)."""
        c = self.conf
        hi, lo, avg = torch.max(data), torch.min(data), torch.mean(data)
        q95 = torch.quantile(data.to(torch.float), 0.95)

        r0_lo, r0_hi = math.pi / 6, 0.94
        r1_lo, r1_hi = 1.06, math.pi * 2 / 3
        r0_step = (r0_hi - r0_lo) / (c.r_search_num / 2)
        r1_step = (r1_hi - r1_lo) / (c.r_search_num / 2)
        b_hi = abs(avg) * 2.0 / self.S
        if b_hi < 0.3:
            b_hi = 0.3
        b_lo = -b_hi
        b_step = (b_hi - b_lo) / c.b_search_num
        s_hi = (hi - lo) * 1.1
        s_lo = 2 * q95
        s_step = (s_hi - s_lo) / c.s_search_num
        if extended:
            r0_step /= c.extend_ratio
            r1_step /= c.extend_ratio
            b_step /= c.extend_ratio
            s_step /= c.extend_ratio

        kw = dict(device=data.device, dtype=data.dtype)
        r_list = torch.cat((-torch.arange(r0_lo + r0_step, r0_hi + r0_step, r0_step, **kw),
                            -torch.arange(r1_lo + r1_step, r1_hi + r1_step, r1_step, **kw)))
        if s_step != 0:
            s_list = torch.arange(s_lo + s_step, s_hi + s_step, s_step, **kw)
        else:
            s_list = torch.tensor([s_lo], **kw)
        if b_step != 0:
            b_list = torch.arange(b_lo, b_hi, b_step, **kw)
        else:
            b_list = torch.tensor([b_lo], **kw)

        lines = self._family_space(r_list, b_list, s_list)
        n_family = lines.shape[0]
        if self.S <= 6:
            lines = torch.cat((lines, self._grid_space(data, extended)), dim=0)
        order = torch.sort(lines.abs(), dim=1)[1]
        return torch.gather(lines, dim=1, index=order), r_list, b_list, s_list, n_family

    # -- search ---------------------------------------------------------------

    def _best_in_batch(self, data, lines):
        """MSE of every line's nearest-point quantisation of ``data``; the best
        line and its selectors (core.py:485-501, 521-528)."""
        points = lines @ self.combs.T                                        # (n, 2^S)
        err = (data.view(1, -1, 1) - points.view(points.shape[0], 1, points.shape[1])) ** 2
        best_err, best_point = err.min(dim=-1)
        mse = best_err.to(torch.float32).mean(dim=-1)
        at = mse.argmin()
        return mse[at].item(), at, best_point[at]

    def search(self, lines, data, stop_below):
        """Scan ``lines`` in batches, first strictly better batch winner wins, stop
        as soon as the best MSE is below ``stop_below`` (core.py:530-553)."""
        best = float("inf")
        best_line, best_sel = -1, -1
        step = self.conf.search_batch_size
        for lo in range(0, lines.shape[0], step):
            mse, at, sel = self._best_in_batch(data, lines[lo:lo + step])
            if mse < best:
                best, best_line, best_sel = mse, lo + at, sel
                if best < stop_below:
                    break
        return best, best_line, best_sel

    # -- per-group policy -----------------------------------------------------

    def encode_group(self, data):
        """Returns (line index, selectors) for one group (core.py:555-653)."""
        c = self.conf
        best = float("inf")
        line_idx = sel = None
        c.group_idx += 1
        warming = c.num_coeff_cache_lines < c.cache_warmup_num
        if not warming:
            known = self.table[:c.num_coeff_cache_lines]
            window = c.mse_history[-min(len(c.mse_history), c.mse_window_size):]
            cutoff = (sum(window) / len(window)) * 0.99
            if cutoff < c.acceptable_mse:
                cutoff = c.acceptable_mse
            best, line_idx, sel = self.search(known, data, cutoff)
            if best < cutoff:
                c.cache_hits += 1
                return line_idx, sel
        if c.num_coeff_cache_lines < self.table.shape[0]:
            hit_rate = c.cache_hits / c.group_idx
            lines, _, _, _, _ = self.candidate_lines(data, hit_rate > 0.6 or warming)
            new_mse, new_at, new_sel = self.search(lines, data, c.acceptable_mse)
            if new_mse < best:
                cand = lines[new_at]
                same = (self.table - cand.unsqueeze(0)).abs().sum(-1) < cand.abs().sum(-1) * 0.0001
                if same.any():
                    line_idx = same.nonzero(as_tuple=True)[0][0]
                else:
                    self.table[c.num_coeff_cache_lines] = cand
                    line_idx = c.num_coeff_cache_lines
                    c.num_coeff_cache_lines += 1
                sel = new_sel
                c.mse_history.append(new_mse)
        return line_idx, sel


def default_batch_size(conf, dtype, device):
    """Candidates per search batch: 1024 on the CPU, 80 % of free memory on a GPU
    (core.py:657-664)."""
    if device.type == "cuda":
        elem = torch.tensor(0, dtype=dtype).element_size()
        per_line = 3 * conf.extend_ratio * (2 ** conf.num_sums) * conf.bvr_len * elem
        return int(torch.cuda.mem_get_info(device)[0] * 0.8 / per_line)
    return 1024
