"""Small host-side helpers: layer partitioning, redundancy bookkeeping.

``partition_uniform`` / ``partition_balanced`` answer the same questions as the reference's
``deepspeed/runtime/utils.py:470-547`` (known answers: tests/unit/test_partition.py:103-190);
``get_redundant_stage_ids`` / ``get_redundant_user_stage_ids`` mirror
``deepspeed/runtime/pipe/redundancy.py:7-31``.
"""
from itertools import accumulate


def partition_uniform(num_items, num_parts):
    """Boundaries ``parts[0..num_parts]`` giving every part ``num_items // num_parts`` items and
    the remainder to the last part (one item per part when there are fewer items than parts)."""
    if num_items <= num_parts:
        return [min(p, num_items) for p in range(num_parts + 1)]
    chunk = num_items // num_parts
    return [chunk * p for p in range(num_parts)] + [num_items]


def _pack(weights, num_parts, limit):
    """Greedy left-to-right packing under a per-part weight limit; returns boundaries or None."""
    parts, load, used = [0], 0.0, 1
    for i, w in enumerate(weights):
        if w > limit:
            return None
        if load + w > limit:
            used += 1
            if used > num_parts:
                return None
            parts.append(i)
            load = 0.0
        load += w
    parts += [len(weights)] * (num_parts + 1 - len(parts))
    return parts


def partition_balanced(weights, num_parts, eps=1e-3):
    """Contiguous partition of ``weights`` into ``num_parts`` parts minimising the heaviest part
    (bisection on the bottleneck, greedy packing for a given bottleneck)."""
    n = len(weights)
    if n <= num_parts:
        return partition_uniform(n, num_parts)
    total = list(accumulate(weights))[-1]
    lo, hi = total / num_parts, float(total)
    while hi > lo + eps:
        mid = lo + (hi - lo) / 2
        if _pack(weights, num_parts, mid) is not None:
            hi = mid
        else:
            lo = mid + eps
    parts = _pack(weights, num_parts, hi)
    assert parts is not None
    return parts


def get_redundant_stage_ids(redundant_level, stage_id, num_stages):
    """Stages whose layers ``stage_id`` keeps a shadow copy of: the next ``level`` stages."""
    return [(stage_id + i) % num_stages for i in range(1, redundant_level + 1)]


def get_redundant_user_stage_ids(redundant_level, stage_id, num_stages):
    """Stages that keep a shadow copy of ``stage_id``."""
    return [s for s in range(num_stages)
            if stage_id in get_redundant_stage_ids(redundant_level, s, num_stages)]
