"""The oracle against the hand-derived vectors of tests/golden/known_answers.json (written
by tests/golden/make_known_answers.py from literals; no code of the reference, the oracle or
this package is involved in producing them)."""
import json
import os

import torch

import varq_oracle as O

GOLDEN = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'known_answers.json')))


def test_pack_and_unpack():
    for k in GOLDEN['pack']:
        q = torch.tensor([k['codes']], dtype=torch.int8)
        w, meta = O.pack_last_dim(q, k['bits'])
        assert w.tolist() == [k['words']], k
        assert meta['pad_len'] == k['pad_len'] and meta['orig_c'] == len(k['codes'])
        assert torch.equal(O.unpack_last_dim(torch.tensor([k['words']], dtype=torch.int32), meta), q)


def test_symmetric_quantizer():
    for k in GOLDEN['quant_sym']:
        x = torch.tensor(k['x'], dtype=torch.float32).view(1, 1, -1, 1)        # one group: reduce everything
        s = O.scale_sym(x, (0, 1, 2, 3), k['bits'])
        want = torch.tensor(k['scale_num'], dtype=torch.float32) / torch.tensor(k['scale_den'], dtype=torch.float32)
        assert float(s) == float(want), k
        assert O.codes_sym(x, s, k['bits']).flatten().tolist() == k['codes'], k


def test_affine_quantizer():
    for k in GOLDEN['quant_asym']:
        x = torch.tensor(k['x'], dtype=torch.float32).view(1, 1, -1, 1)
        q, s, z = O.quant_reduce(x, (0, 1, 2, 3), k['bits'], True)
        assert float(s) == k['scale'] and float(z) == k['zp'], (k, float(s), float(z))
        assert q.flatten().tolist() == k['codes'], k
        # and through the row-local group-wise form: one row holding the same values
        xr = torch.tensor(k['x'], dtype=torch.float32).view(1, 1, 1, -1)
        if xr.shape[3] % 8 == 0:
            q2, s2, z2 = O.quant_groupwise(xr, xr.shape[3], k['bits'], True)
            assert q2.flatten().tolist() == k['codes']
