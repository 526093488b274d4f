"""The HIP kernels against the hand-derived vectors of tests/golden/known_answers.json."""
import json
import os

import pytest
import torch

from gpu_util import note
from var_q_amd import ops

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'known_answers.json')))


def test_pack_and_unpack(dev):
    for k in GOLDEN['pack']:
        note('golden pack', k['bits'], len(k['codes']))
        q = torch.tensor([k['codes']], dtype=torch.int8, device=dev)
        w = ops.pack(q, k['bits'])
        assert w.cpu().tolist() == [k['words']], k
        assert torch.equal(ops.unpack(w, len(k['codes']), k['bits']), q)


def test_symmetric_quantizer(dev):
    for k in GOLDEN['quant_sym']:
        note('golden sym', k['bits'])
        x = torch.tensor(k['x'], dtype=torch.float32, device=dev).view(1, 1, -1, 1)
        q, s, _ = ops.quant_pack(x, (0, 1, 2, 3), k['bits'], asym=False, pack=False)
        want = torch.tensor(k['scale_num'], dtype=torch.float32) / torch.tensor(k['scale_den'], dtype=torch.float32)
        assert float(s) == float(want), k
        assert q.flatten().cpu().tolist() == k['codes'], k


def test_affine_quantizer(dev):
    for k in GOLDEN['quant_asym']:
        note('golden asym', k['bits'])
        x = torch.tensor(k['x'], dtype=torch.float32, device=dev).view(1, 1, -1, 1)
        q, s, z = ops.quant_pack(x, (0, 1, 2, 3), k['bits'], asym=True, pack=False)
        assert float(s) == k['scale'] and float(z) == k['zp'], (k, float(s), float(z))
        assert q.flatten().cpu().tolist() == k['codes'], k
