"""DynamiQ's per-superchunk bit-width allocation -- the host-side mirror of
testbed_evaluation/new_comm_hooks/comm_hooks.py:48-139.

Every superchunk (256 elements) gets q in {2, 4, 8} bits from its reduced
squared norm F and a scalar offset u:
    z = clamp(floor(log2(max(NORM_SCALE * log2(max(F, 1e-20)) + u, 1e-20))), 1, 3),  q = 2^z
and u is steered so that the average q meets a target (nominal bits - 0.625 for
the scale overhead).  ``dynamic_bitrate_qbits`` keeps the reference's torch op
order exactly (each op rounds in the dtype of the norms, which is what makes the
widths reproducible); the two searches are written around one evaluation helper.
"""
import torch

DYNAMIC_BITRATE_HEADROOM = 0.625
DYNAMIC_BITRATE_U_MIN = -10.0
DYNAMIC_BITRATE_U_MAX = 60.0
DYNAMIC_BITRATE_TOL = 0.1
DYNAMIC_BITRATE_MAX_ITERS = 32
DYNAMIC_BITRATE_NORM_SCALE = 4.0 / (512.0 / 17.0)
_EPS = 1e-20


def dynamic_bitrate_target_bitrate(aggregation_method):
    """comm_hooks.py:56-61: the "<n>bit" token of the method name (n = 8 .. 2), 5 when there is none"""
    name = aggregation_method.lower()
    found = [b for b in range(8, 1, -1) if "%dbit" % b in name]
    return float(found[0]) if found else 5.0


def dynamic_bitrate_qbits(norms, u):
    """comm_hooks.py:64-70, op for op: clamp, log2, mul, add, clamp, log2, floor, int64, clamp, shift"""
    score = torch.log2(torch.clamp(norms, min=_EPS)).mul(DYNAMIC_BITRATE_NORM_SCALE).add(float(u))
    z = torch.floor(torch.log2(torch.clamp(score, min=_EPS))).to(torch.int64).clamp_(1, 3)
    return torch.bitwise_left_shift(torch.ones_like(z), z)


def dynamic_bitrate_average_bits(norms_list, u):
    """comm_hooks.py:73-86: mean width over all superchunks of all tensors (0.0 for no superchunks)"""
    tensors = [t for t in norms_list if t.numel() > 0]
    if not tensors:
        return 0.0
    bits = sum(dynamic_bitrate_qbits(t, u).sum() for t in tensors)
    return float(bits.item()) / sum(t.numel() for t in tensors)


def dynamic_bitrate_avg_delta(norms_list, u, target_avg_bits):
    """(average width at u, target - average)"""
    avg = dynamic_bitrate_average_bits(norms_list, u)
    return avg, target_avg_bits - avg


def _clip_u(u):
    return min(DYNAMIC_BITRATE_U_MAX, max(DYNAMIC_BITRATE_U_MIN, float(u)))


class _Best(object):
    """the candidate with the smallest |delta| seen so far (the first one wins ties)"""

    def __init__(self, u, avg, delta):
        self.u, self.avg, self.delta = u, avg, delta

    def offer(self, u, avg, delta):
        if abs(delta) < abs(self.delta):
            self.u, self.avg, self.delta = u, avg, delta

    def triple(self):
        return self.u, self.avg, self.delta


def dynamic_bitrate_binary_search_u(norms_list, target_avg_bits):
    """comm_hooks.py:94-114: bisection of u over [-10, 60]; stops at |delta| <= 0.1 bit or after 32 midpoints, then
    returns the best point seen (the upper end of the interval is the starting candidate)"""
    lo, hi = DYNAMIC_BITRATE_U_MIN, DYNAMIC_BITRATE_U_MAX
    best = _Best(hi, *dynamic_bitrate_avg_delta(norms_list, hi, target_avg_bits))
    for _ in range(DYNAMIC_BITRATE_MAX_ITERS):
        mid = 0.5 * (lo + hi)
        avg, delta = dynamic_bitrate_avg_delta(norms_list, mid, target_avg_bits)
        best.offer(mid, avg, delta)
        if abs(delta) <= DYNAMIC_BITRATE_TOL:
            return mid, avg, delta
        if delta > 0:       # too few bits: raise u
            lo = mid
        else:
            hi = mid
    return best.triple()


def dynamic_bitrate_adjust_u(norms_list, prev_u, target_avg_bits):
    """comm_hooks.py:117-139: the correction used after the first compressed round.  Steps from the previous u by the
    current deficit, halving the step each time, until the tolerance is met or the deficit no longer changes sign."""
    start = _clip_u(prev_u)
    avg0, delta0 = dynamic_bitrate_avg_delta(norms_list, start, target_avg_bits)
    if abs(delta0) <= DYNAMIC_BITRATE_TOL:
        return start, avg0, delta0
    best = _Best(start, avg0, delta0)
    step = delta0
    for _ in range(DYNAMIC_BITRATE_MAX_ITERS):
        u = _clip_u(start + step)
        avg, delta = dynamic_bitrate_avg_delta(norms_list, u, target_avg_bits)
        best.offer(u, avg, delta)
        if abs(delta) <= DYNAMIC_BITRATE_TOL or delta0 * delta >= 0:
            return u, avg, delta
        step *= 0.5
    return best.triple()


# ---- fixed-proportion allocation (the non-dynamic P2P_dynamiQ hook) -------------------------------------

def fixed_proportion_thresholds(aggregation_method):
    """comm_hooks.py:842-856: the fractions of a bucket's superchunks that get 8, 4 and 2 bits, chosen by the
    "<n>bit" token of the method name ("4bit" + "fixed": every superchunk 4 bits; no token: the 5-bit mix)"""
    name = aggregation_method
    if "4bit" in name:
        return {4: 1, 8: 0, 2: 0} if "fixed" in name else {8: 0.05, 4: 0.6, 2: 0.35}
    if "3bit" in name:
        return {8: 1 / 40, 4: 13 / 40, 2: 26 / 40}
    if "6bit" in name:
        return {8: 0.55, 4: 0.35, 2: 0.1}
    if "7bit" in name:
        return {8: 0.75, 4: 0.22, 2: 0.03}
    return {8: 0.35, 4: 0.45, 2: 0.2}


def fixed_proportion_counts(num_superchunks, thresholds):
    """comm_hooks.py:713-716: (superchunks at 8 bits, at 4 bits, at 2 bits); the products are truncated, and the
    2-bit share gives way when the two together exceed the bucket"""
    top = int(num_superchunks * thresholds[8])
    bottom = int(num_superchunks * thresholds[2])
    if top + bottom > num_superchunks:
        bottom = max(0, num_superchunks - top)
    return top, num_superchunks - top - bottom, bottom


def fixed_proportion_groups(norms, thresholds):
    """comm_hooks.py:710-721 as the reference's torch ops: the superchunks in descending order of their reduced
    squared norm (stable: equal norms keep index order; NaN sorts above every number), the first `top` at 8 bits, the
    last `bottom` at 2, the rest at 4.  Returns three int64 index tensors **in sorted order** -- the order in which the
    hook gathers the group tensor, hence the order of the records and of the rounding-randomness rows."""
    norms = norms.float()
    top, _, bottom = fixed_proportion_counts(norms.numel(), thresholds)
    order = torch.argsort(norms, descending=True, stable=True)
    n = norms.numel()
    return order[:top], order[top:n - bottom], order[n - bottom:] if bottom > 0 else order[:0]


def fixed_proportion_plan(stats, thresholds, order=None, work=None, stream=None):
    """The same three lists from the interleaved bf16 (mean, norm) statistics without a read-back (one launch, no sort
    passes, up to 65535 superchunks; a radix sort inside ``work`` for longer buckets): ``order`` int32 [3 * nsc] (the 8-bit list at 0, the 4-bit list at nsc, the 2-bit list at
    2 * nsc, each in sorted order) and ``work[0..2]`` = the three counts, i.e. what the row-list and mixed codec
    kernels take.  Returns (order, work, (n8, n4, n2))."""
    from . import capi
    nsc = stats.numel() // 2
    n8, n4, n2 = fixed_proportion_counts(nsc, thresholds)
    if order is None:
        order = torch.empty(3 * nsc, dtype=torch.int32, device=stats.device)
    if work is None:
        work = torch.empty(max(capi.group_plan_work_ints(nsc), capi.group_plan_sorted_work_ints(nsc)), dtype=torch.int32,
                           device=stats.device)
    capi.group_plan_sorted(stats, n8, n2, order, work, stream)
    return order, work, (n8, n4, n2)


class NormHistogram(object):
    """The two searches above without a pass over the norms per probe: the norm patterns of every bucket are counted
    into a device histogram (``add``, one small launch per bucket, after the statistics all-reduce), and one launch runs
    the whole search on the counts.  Same (u, average, delta) as the functions above on the same norms; one read-back
    per search instead of one per probe."""

    def __init__(self, device):
        from . import capi
        self._capi = capi
        self.hist = torch.zeros(capi.bitrate_hist_ints(), dtype=torch.int32, device=device)
        self.result = torch.zeros(4, dtype=torch.float64, device=device)
        self.count = 0

    def add(self, stats, stream=None):
        """stats: bf16 [nsc, 2] as written by superchunk_mean_center / superchunk_stats"""
        self._capi.norm_histogram(stats, self.hist, stream)
        self.count += stats.numel() // 2

    def launch_search(self, mode, prev_u, target_avg_bits, stream=None):
        """the search as one launch, nothing read back: returns the device tensor float64 [4] = u, average width,
        target - average, probes (also ``self.result``).  mode 0: bisection; 1: correction from prev_u, a number or a
        float64 device tensor -- ``self.result[0:1]`` chains the steps of a training run on the device."""
        self._capi.bitrate_search(self.hist, mode, prev_u, target_avg_bits, self.result, stream)
        self.count = 0                      # the kernel leaves the histogram zeroed
        return self.result

    def _search(self, mode, prev_u, target_avg_bits, stream):
        self.launch_search(mode, prev_u, target_avg_bits, stream)
        # tolist() only waits for torch's current stream: wait for the one the search ran on
        self._capi.torch_stream(stream, self.result.device).synchronize()
        u, avg, delta, _ = self.result.tolist()
        return u, avg, delta

    def binary_search_u(self, target_avg_bits, stream=None):
        """comm_hooks.py:94-114 on the norms added since the last search"""
        return self._search(0, DYNAMIC_BITRATE_U_MAX, target_avg_bits, stream)

    def adjust_u(self, prev_u, target_avg_bits, stream=None):
        """comm_hooks.py:117-139 on the norms added since the last search"""
        return self._search(1, prev_u, target_avg_bits, stream)
