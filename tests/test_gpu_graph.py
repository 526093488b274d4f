"""A whole schedule -- append and attend per scale on the pre-allocated packed cache --
recorded once into a HIP graph (torch.cuda.CUDAGraph) and replayed on new inputs in the same
buffers: every replay equals the eager run on those inputs.  The library launches kernels
only (no memset nodes, no allocation of its own), which is what makes the recording valid;
replays are separated by the program's eager work, as a caller would interleave them."""
import math

import pytest
import torch

from gpu_util import note
from var_q_amd import PackedKVCache

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('bits', [4, [2, 4, 8, 8, 4, 2]])
def test_schedule_replayed_from_a_graph(dev, bits):
    B, H, D = 2, 6, 128
    ns = [1, 4, 16, 36, 64, 144, 256]
    gen = torch.Generator(device=dev).manual_seed(31)
    steps = [tuple(torch.randn(B, H, n, D, device=dev, generator=gen).bfloat16() for _ in range(3)) for n in ns]
    outs = [torch.empty_like(s[0]) for s in steps]
    cache = PackedKVCache(B, H, sum(ns), D, bits, 64, dev)
    scale = 1 / math.sqrt(D)

    def one_pass():
        cache.reset()
        for (q, k, v), o in zip(steps, outs):
            cache.append(k, v)
            cache.attend(q, scale, out=o)

    note('graph: warm-up on a side stream', bits)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_pass()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    note('graph: capture', bits)
    with torch.cuda.graph(graph):
        one_pass()
    torch.cuda.synchronize()
    for rep in range(4):
        for q, k, v in steps:                      # new values, same memory
            q.normal_(generator=gen)
            k.normal_(generator=gen)
            v.normal_(generator=gen)
        note('graph: eager reference', bits, rep)
        one_pass()
        torch.cuda.synchronize()
        want = [o.clone() for o in outs]
        for o in outs:
            o.fill_(7.0)
        note('graph: replay', bits, rep)
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(want, outs)):
            assert torch.equal(a, b), f'replay {rep}, scale {i}: the graph and the eager run differ'


@pytest.mark.parametrize('fmt,B,H,D', [('BHLc', 2, 4, 128), ('BLHc', 8, 6, 64)])
def test_shipped_rule_pass_replayed_from_a_graph(dev, fmt, B, H, D):
    """The drop-in quantizers' fused step (quantize + cache + attend per scale, the shipped rule
    G_SCALE_HEAD_DIM at 8 bits) recorded once and replayed on new inputs in the same buffers: the
    Python state machine runs at capture time only, the kernels it launched are what a replay
    repeats.  Every replay equals the eager pass on the same inputs."""
    from var_q_amd import VAR_Q
    from var_q_amd.quant import fused_step
    ns = [1, 4, 9, 16, 36, 64, 100]
    gen = torch.Generator(device=dev).manual_seed(41)
    shape = (lambda n: (B, H, n, D)) if fmt == 'BHLc' else (lambda n: (B, n, H, D))
    steps = [tuple(torch.randn(*shape(n), device=dev, generator=gen).bfloat16() for _ in range(3)) for n in ns]
    outs = [torch.empty_like(s[0]) for s in steps]
    scale = 1 / math.sqrt(D)

    def one_pass():
        kq, vq = VAR_Q(8, fmt, 'G_SCALE_HEAD_DIM'), VAR_Q(8, fmt, 'G_SCALE_HEAD_DIM')
        for quantizer in (kq, vq):
            quantizer.reserve_tokens(sum(ns))
        for (q, k, v), o in zip(steps, outs):
            fused_step(q, k, v, kq, vq, scale, out=o)

    note('graph, shipped rule: warm-up on a side stream', fmt)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_pass()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    note('graph, shipped rule: capture', fmt)
    with torch.cuda.graph(graph):
        one_pass()
    torch.cuda.synchronize()
    for rep in range(4):
        for q, k, v in steps:                      # new values, same memory
            q.normal_(generator=gen)
            k.normal_(generator=gen)
            v.normal_(generator=gen)
        note('graph, shipped rule: eager reference', fmt, rep)
        one_pass()
        torch.cuda.synchronize()
        want = [o.clone() for o in outs]
        for o in outs:
            o.fill_(7.0)
        note('graph, shipped rule: replay', fmt, rep)
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(want, outs)):
            assert torch.equal(a, b), f'replay {rep}, scale {i}: the graph and the eager pass differ'
