"""DynamiQ's per-superchunk bit-width allocation -- the host-side mirror of
testbed_evaluation/new_comm_hooks/comm_hooks.py:48-139.

Every superchunk (256 elements) gets q in {2, 4, 8} bits from its reduced
squared norm F and a scalar offset u:
    z = clamp(floor(log2(max(NORM_SCALE * log2(max(F, 1e-20)) + u, 1e-20))), 1, 3),  q = 2^z
and u is steered so that the average q meets a target (nominal bits - 0.625 for
the scale overhead).  The functions are the reference's torch-op sequences, so
they run on whatever device and dtype the norms live in (the testbed feeds bf16
norms, the simulation casts to fp32 first).
"""
import torch

DYNAMIC_BITRATE_HEADROOM = 0.625
DYNAMIC_BITRATE_U_MIN = -10.0
DYNAMIC_BITRATE_U_MAX = 60.0
DYNAMIC_BITRATE_TOL = 0.1
DYNAMIC_BITRATE_MAX_ITERS = 32
DYNAMIC_BITRATE_NORM_SCALE = 4.0 / (512.0 / 17.0)


def dynamic_bitrate_target_bitrate(aggregation_method):
    """comm_hooks.py:56-61: "<n>bit" in the method name, default 5"""
    method = aggregation_method.lower()
    for nbits in (8, 7, 6, 5, 4, 3, 2):
        if f"{nbits}bit" in method:
            return float(nbits)
    return 5.0


def dynamic_bitrate_qbits(norms, u):
    """comm_hooks.py:64-70"""
    eps = 1e-20
    log_norms = torch.log2(torch.clamp(norms, min=eps))
    score = log_norms.mul(DYNAMIC_BITRATE_NORM_SCALE).add(float(u))
    z = torch.floor(torch.log2(torch.clamp(score, min=eps))).to(torch.int64)
    z.clamp_(1, 3)
    return torch.bitwise_left_shift(torch.ones_like(z), z)


def dynamic_bitrate_average_bits(norms_list, u):
    """comm_hooks.py:73-86"""
    total_chunks = 0
    total_bits = None
    for norms in norms_list:
        if norms.numel() == 0:
            continue
        qbits = dynamic_bitrate_qbits(norms, u)
        qbits_sum = qbits.sum()
        total_bits = qbits_sum if total_bits is None else total_bits + qbits_sum
        total_chunks += qbits.numel()
    if total_bits is None or total_chunks == 0:
        return 0.0
    return float(total_bits.item()) / total_chunks


def dynamic_bitrate_avg_delta(norms_list, u, target_avg_bits):
    avg_bits = dynamic_bitrate_average_bits(norms_list, u)
    return avg_bits, target_avg_bits - avg_bits


def dynamic_bitrate_binary_search_u(norms_list, target_avg_bits):
    """comm_hooks.py:94-114: bisection on u in [-10, 60], at most 32 steps, tolerance 0.1 bit"""
    low = DYNAMIC_BITRATE_U_MIN
    high = DYNAMIC_BITRATE_U_MAX
    best_u = high
    best_avg, best_delta = dynamic_bitrate_avg_delta(norms_list, best_u, target_avg_bits)
    for _ in range(DYNAMIC_BITRATE_MAX_ITERS):
        mid = (low + high) * 0.5
        avg_bits, delta = dynamic_bitrate_avg_delta(norms_list, mid, target_avg_bits)
        if abs(delta) < abs(best_delta):
            best_u = mid
            best_avg = avg_bits
            best_delta = delta
        if abs(delta) <= DYNAMIC_BITRATE_TOL:
            return mid, avg_bits, delta
        if delta > 0:
            low = mid
        else:
            high = mid
    return best_u, best_avg, best_delta


def dynamic_bitrate_adjust_u(norms_list, prev_u, target_avg_bits):
    """comm_hooks.py:117-139: incremental correction used after the first compressed round"""
    prev_u = max(DYNAMIC_BITRATE_U_MIN, min(DYNAMIC_BITRATE_U_MAX, float(prev_u)))
    old_avg, old_delta = dynamic_bitrate_avg_delta(norms_list, prev_u, target_avg_bits)
    if abs(old_delta) <= DYNAMIC_BITRATE_TOL:
        return prev_u, old_avg, old_delta
    step = old_delta
    best_u = prev_u
    best_avg = old_avg
    best_delta = old_delta
    for _ in range(DYNAMIC_BITRATE_MAX_ITERS):
        candidate_u = max(DYNAMIC_BITRATE_U_MIN, min(DYNAMIC_BITRATE_U_MAX, prev_u + step))
        avg_bits, delta = dynamic_bitrate_avg_delta(norms_list, candidate_u, target_avg_bits)
        if abs(delta) < abs(best_delta):
            best_u = candidate_u
            best_avg = avg_bits
            best_delta = delta
        if abs(delta) <= DYNAMIC_BITRATE_TOL or old_delta * delta >= 0:
            return candidate_u, avg_bits, delta
        step *= 0.5
    return best_u, best_avg, best_delta
