"""Shared helpers of the GPU parity tests."""
import sys

import torch


def note(*a):
    """Name the case before the GPU step runs, flushed, so a fault is attributable."""
    print('[case]', *a, flush=True)
    sys.stdout.flush()


def adversarial_rows(c, dtype=torch.float32, seed=0):
    """Rows built to break approximate quantizers: exact .5 ties, all-zero and
    constant rows, denormals, huge magnitudes, big offsets, +-1 ulp around ties."""
    g = torch.Generator().manual_seed(seed)
    rows = []
    rows.append(torch.zeros(c))
    rows.append(torch.full((c,), 3.0))
    rows.append(torch.full((c,), -0.0))
    # scale == 1 exactly for 8-bit symmetric, values on .5 ties
    t = (torch.arange(c, dtype=torch.float32) % 250) - 125 + 0.5
    t[0] = 127.0
    rows.append(t)
    # 4-bit asymmetric ties: range 15 -> scale 1
    t = (torch.arange(c, dtype=torch.float32) % 15) + 0.5
    t[0], t[1] = 0.0, 15.0
    rows.append(t)
    rows.append(torch.randn(c, generator=g) * 1e-41)       # denormals
    rows.append(torch.randn(c, generator=g) * 1e30)
    rows.append(torch.randn(c, generator=g) * 1e-30)
    rows.append(torch.randn(c, generator=g) + 1000.0)      # large zero-point
    rows.append(torch.randn(c, generator=g) * 0.01 - 77.0)
    big = torch.randn(c, generator=g)
    big[c // 2] = 3.0e38
    rows.append(big)
    # values +-1 ulp around ties for an awkward scale
    sc = torch.tensor(0.3137)
    k = (torch.arange(c, dtype=torch.float32) % 14) - 7 + 0.5
    near = k * sc
    rows.append(near)
    rows.append(torch.nextafter(near, torch.tensor(float('inf'))))
    rows.append(torch.nextafter(near, torch.tensor(float('-inf'))))
    for _ in range(18):
        rows.append(torch.randn(c, generator=g) * float(torch.rand(1, generator=g) * 10))
    return torch.stack(rows).to(dtype)
