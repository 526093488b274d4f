"""Scale schedules and the block-causal next-scale mask, as host-side tables.

VAR: VAR/models/var.py:27 (patch_nums) and :110-114 (mask).  Infinity ratio
1.0 / '1M': Infinity/infinity/utils/dynamic_resolution.py:7.
"""
from typing import Optional, Sequence

import torch

VAR_PATCH_NUMS = (1, 2, 3, 4, 5, 6, 8, 10, 13, 16)                    # sum of squares = 680
INFINITY_PATCH_NUMS = (1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64)   # sum of squares = 10521


def tokens_per_scale(patch_nums: Sequence[int]):
    return [pn * pn for pn in patch_nums]


def total_tokens(patch_nums: Sequence[int]) -> int:
    return sum(tokens_per_scale(patch_nums))


def kv_limit(patch_nums: Sequence[int], q_start: int = 0, q_len: Optional[int] = None,
             device=None) -> torch.Tensor:
    """int32 [q_len]: number of keys visible to each query under
    mask[q,k] = 0 if level(q) >= level(k) else -inf (VAR/models/var.py:110-114).
    Token levels are non-decreasing, so the visible set is the prefix ending
    where the query's own scale ends."""
    counts = tokens_per_scale(patch_nums)
    ends, acc = [], 0
    for n in counts:
        acc += n
        ends.extend([acc] * n)
    q_len = len(ends) - q_start if q_len is None else q_len
    return torch.tensor(ends[q_start:q_start + q_len], dtype=torch.int32, device=device)
