"""SBVR encoder: per group of ``bvr_len`` values, search a line of ``num_sums``
fp16 coefficients whose 2^S subset sums approximate the group best (MSE), and
reuse earlier lines through a table (the "coefficient cache").

This is the reference's CPU/torch algorithm (sbvr/core.py:19-60 configuration,
:368-483 search spaces, :485-553 search, :555-653 per-group policy) restated.
On the CPU it makes the same torch calls in the same order, so it yields the
same lines and selectors.  On a GPU two things differ from the reference's loop
(core.py:711-722, one group at a time):
  * the error of a (group, line) pair comes from a HIP kernel that keeps the
    (lines, G, 2^S) tensor of squared differences in registers (hip.encoder_group_mse;
    fp16 compute type and up to 8 planes, otherwise the torch expression).  The kernel
    sums a group's minima in fp32 in element order where torch's .mean() reduces in
    another order, so on near-ties a GPU run can pick another line than a CPU run
    (parity of GPU encodings with the reference's own GPU runs is unpinned; they are
    compared by their error);
  * table look-ups run for a block of groups at once (``encode_all``): the
    groups of a block are looked up against the table as it stands, the leading
    hits are taken, the first miss goes through the one-group path (which may add
    a line and move the cut-off), and the look-up restarts behind it.  The policy
    is order-dependent and this keeps its order: block size 1 and block size 512
    give the same table, indices and selectors.
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
        unknown = set(kwargs) - set(self.DEFAULTS) - {"bvr_len", "group_block"}
        if unknown:
            raise TypeError(f"unknown encoder option(s): {sorted(unknown)}")
        for k, v in self.DEFAULTS.items():
            setattr(self, k, kwargs.get(k, v))
        if self.mse_history is None:
            self.mse_history = []
        # extension: the reference fixes the group length at 256 (core.py:222)
        self.bvr_len = kwargs.get("bvr_len", 256)
        # extension: groups looked up in the table at a time (None: 512 on a GPU, 1 on the CPU; see encode_all)
        self.group_block = kwargs.get("group_block", None)

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

    def _use_kernel(self, data):
        if not data.is_cuda:
            return False
        from . import hip
        return hip.encoder_group_mse_supported(data.dtype, data.shape[-1], 1 << self.S)

    def _mse_matrix(self, datas, points):
        """(groups, lines) errors: mean over the group of the squared distance to the nearest point, the
        differences and squares in the compute type (core.py:485-495)."""
        if self._use_kernel(datas):
            from . import hip
            return hip.encoder_group_mse(datas.contiguous(), points.contiguous())
        out = torch.empty((datas.shape[0], points.shape[0]), dtype=torch.float32, device=datas.device)
        # (bounded intermediate: about 2^24 squared differences at a time)
        step = max(1, (1 << 24) // max(1, points.shape[0] * datas.shape[1] * points.shape[1]))
        for lo in range(0, datas.shape[0], step):
            d = datas[lo:lo + step]
            err = (d.view(d.shape[0], 1, -1, 1) - points.view(1, points.shape[0], 1, points.shape[1])) ** 2
            out[lo:lo + step] = err.min(dim=-1)[0].to(torch.float32).mean(dim=-1)
        return out

    def _selectors(self, datas, points):
        """Nearest point of its own line for every value: datas (groups, G), points (groups, 2^S)."""
        err = (datas.unsqueeze(-1) - points.unsqueeze(1)) ** 2
        return err.min(dim=-1)[1]

    def _best_in_batch(self, data, lines):
        """MSE of every line's nearest-point quantisation of ``data``; the best
        line and its selectors (core.py:485-501, 521-528)."""
        points = lines @ self.combs.T                                        # (n, 2^S)
        if self._use_kernel(data):
            mse = self._mse_matrix(data.view(1, -1), points)[0]
            at = mse.argmin()
            return mse[at].item(), at, self._selectors(data.view(1, -1), points[at].view(1, -1))[0]
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
            cutoff = self._cutoff()
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


    # -- many groups ----------------------------------------------------------

    def _cutoff(self):
        c = self.conf
        window = c.mse_history[-min(len(c.mse_history), c.mse_window_size):]
        cutoff = (sum(window) / len(window)) * 0.99
        return c.acceptable_mse if cutoff < c.acceptable_mse else cutoff

    def _lookup_block(self, datas, cutoff):
        """``search(table, data, cutoff)`` for every row of ``datas`` at once: the same scan over batches
        of ``search_batch_size`` lines (first strictly better batch winner, stop below the cut-off).
        Returns python lists (best error, line) per group and the points of every table line (from the
        same products the scan used)."""
        c = self.conf
        n = c.num_coeff_cache_lines
        known = self.table[:n]
        step = c.search_batch_size
        B = datas.shape[0]
        best = [float("inf")] * B
        line = [-1] * B
        live = list(range(B))
        all_points = []
        for lo in range(0, n, step):
            points = known[lo:lo + step] @ self.combs.T
            all_points.append(points)
            if not live:
                continue
            rows = datas if len(live) == B else datas[torch.tensor(live, device=datas.device)]
            mse = self._mse_matrix(rows, points)
            at = mse.argmin(dim=1)
            val = mse.gather(1, at.view(-1, 1)).view(-1).tolist()
            at = at.tolist()
            still = []
            for j, b in enumerate(live):
                if val[j] < best[b]:
                    best[b], line[b] = val[j], lo + at[j]
                if not best[b] < cutoff:
                    still.append(b)
            live = still
        return best, line, torch.cat(all_points, dim=0)

    def encode_all(self, flat, line_of, sel, block=512, progress=None):
        """Encodes the groups of ``flat`` (a multiple of bvr_len values) in order into ``line_of`` (one
        line index per group) and ``sel`` (one selector per value).  ``block`` groups are looked up in the
        table at a time; 1 is the reference's loop (core.py:711-722)."""
        c = self.conf
        G = c.bvr_len
        n_groups = flat.numel() // G
        i = 0
        span = block
        while i < n_groups:
            warming = c.num_coeff_cache_lines < c.cache_warmup_num
            if block <= 1 or warming:
                line, s = self.encode_group(flat[i * G:(i + 1) * G])
                line_of[i] = line
                sel[i * G:(i + 1) * G] = s
                i += 1
                if progress is not None:
                    progress(1)
                continue
            B = min(span, n_groups - i)
            datas = flat[i * G:(i + B) * G].view(B, G)
            cutoff = self._cutoff()
            best, line, points = self._lookup_block(datas, cutoff)
            j = 0
            restart = False
            while j < B and not restart:
                if best[j] < cutoff:
                    run = j
                    while run < B and best[run] < cutoff:
                        run += 1
                    lines_t = torch.tensor(line[j:run], device=flat.device)
                    s = self._selectors(datas[j:run], points[lines_t])
                    line_of[i + j:i + run] = lines_t.to(line_of.dtype)
                    sel[(i + j) * G:(i + run) * G] = s.reshape(-1)
                    c.cache_hits += run - j
                    c.group_idx += run - j
                    if progress is not None:
                        progress(run - j)
                    j = run
                else:
                    before = (c.num_coeff_cache_lines, len(c.mse_history))
                    ln, s = self.encode_group(datas[j])
                    line_of[i + j] = ln
                    sel[(i + j) * G:(i + j + 1) * G] = s
                    if progress is not None:
                        progress(1)
                    j += 1
                    # a new line or a new entry of the error history changes what the later groups see
                    restart = (c.num_coeff_cache_lines, len(c.mse_history)) != before
            i += j
            # (short blocks while the table still grows, long ones once it has settled)
            span = block if not restart else max(16, min(block, 2 * j))


def default_batch_size(conf, dtype, device):
    """Candidates per search batch: 1024 on the CPU, 80 % of free memory on a GPU
    (core.py:657-664)."""
    if device.type == "cuda":
        elem = torch.tensor(0, dtype=dtype).element_size()
        per_line = 3 * conf.extend_ratio * (2 ** conf.num_sums) * conf.bvr_len * elem
        return int(torch.cuda.mem_get_info(device)[0] * 0.8 / per_line)
    return 1024
