"""Range statistics and L2-normalised quantization error, written to CSV.

The reference's README promises "on-demand min/max range stats and L2-normalized
error comparison, saved to CSV" (README.md:11) without shipping code for it;
this module provides it for the quantizers of this package.  The quantities
are by-products of the quantize kernel (its scales and zero-points carry the
group ranges); the error is measured by dequantizing the packed result.
"""
import csv
import os
from typing import Any, Dict, Iterable, Optional

import torch

from . import ops

FIELDS = ['tag', 'shape', 'dtype', 'bits', 'group_size', 'symmetric', 'n_groups', 'x_min', 'x_max', 'x_abs_mean',
          'group_range_min', 'group_range_mean', 'group_range_max', 'scale_min', 'scale_max',
          'l2_norm_error', 'max_abs_error', 'max_abs_error_in_steps', 'saturated_fraction', 'packed_bytes', 'ratio_vs_input']


def quant_error_stats(x: torch.Tensor, group_size: int, bits: int, symmetric: bool = False, tag: str = '',
                      eps: float = 1e-12) -> Dict[str, Any]:
    """Quantize+pack x ([..., D], D a multiple of group_size, GPU tensor) with the
    group-wise quantizer and report range and error figures.

    l2_norm_error = ||x - dequant(quant(x))||_2 / ||x||_2 over the whole tensor;
    max_abs_error_in_steps is relative to each element's own group scale (<= 0.5
    unless the element saturates); saturated_fraction counts codes at qmin/qmax
    whose reconstruction error exceeds half a step."""
    shape = tuple(x.shape)
    D = shape[-1]
    x4 = x.reshape(1, 1, -1, D)
    words, scale, zp = ops.quant_pack_rows(x4, group_size, bits, not symmetric, eps)
    deq = ops.dequant(words, scale, zp, D, bits)
    xf = x4.float()
    err = (xf - deq).abs()
    ns = D // group_size
    step = scale.reshape(1, 1, -1, ns, 1).expand(-1, -1, -1, -1, group_size).reshape(1, 1, -1, D)
    err_steps = err / step
    if symmetric:
        rng = scale * float(2 ** (bits - 1) - 1) * 2.0      # 2 * max|x| of the group
    else:
        rng = scale * float(2 ** bits - 1)                   # max - min of the group
    nx = torch.linalg.vector_norm(xf.double())
    packed_bytes = words.numel() * 4 + scale.numel() * 4 + (0 if zp is None else zp.numel() * 4)
    return {
        'tag': tag, 'shape': 'x'.join(str(d) for d in shape), 'dtype': str(x.dtype).replace('torch.', ''), 'bits': bits,
        'group_size': group_size, 'symmetric': symmetric, 'n_groups': scale.numel(),
        'x_min': xf.min().item(), 'x_max': xf.max().item(), 'x_abs_mean': xf.abs().mean().item(),
        'group_range_min': rng.min().item(), 'group_range_mean': rng.mean().item(), 'group_range_max': rng.max().item(),
        'scale_min': scale.min().item(), 'scale_max': scale.max().item(),
        'l2_norm_error': (torch.linalg.vector_norm((xf - deq).double()) / nx.clamp_min(1e-300)).item(),
        'max_abs_error': err.max().item(), 'max_abs_error_in_steps': err_steps.max().item(),
        'saturated_fraction': (err_steps > 0.5 + 1e-3).float().mean().item(),
        'packed_bytes': packed_bytes, 'ratio_vs_input': packed_bytes / (x.numel() * x.element_size()),
    }


class CsvReport:
    """Appends rows of quant_error_stats (or any dict over FIELDS) to a CSV file."""

    def __init__(self, path: str, fields: Optional[Iterable[str]] = None):
        self.path, self.fields = path, list(fields or FIELDS)
        if not os.path.exists(path) or os.path.getsize(path) == 0:
            with open(path, 'w', newline='') as f:
                csv.writer(f).writerow(self.fields)

    def add(self, row: Dict[str, Any]):
        with open(self.path, 'a', newline='') as f:
            csv.writer(f).writerow([row.get(k, '') for k in self.fields])

    def rows(self):
        with open(self.path, newline='') as f:
            return list(csv.DictReader(f))
