"""Seeded random cases of both attention entry points against the oracle: head dim, bit
width, grouping, batch, query and key counts (ragged ones included), per-query key limits,
key sharing over workgroups, both layouts and -- for the per-(head, channel) tables --
segment ends at arbitrary keys, so that key tiles straddle one or several changes of tables.
The codes, scales and zero-points are the oracle's; tolerances as in test_gpu_attention.py."""
import math
import random

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _compare
from var_q_amd import ops

pytestmark = pytest.mark.gpu


def _case(rng):
    D = rng.choice([64, 128])
    bits = rng.choice([2, 4, 8])
    mode = rng.choice(['token', 'channel', 'channel'])
    B = rng.choice([1, 2, 3])
    H = rng.choice([1, 2, 5])
    Lq = rng.choice([1, 3, 17, 32, 33, 64, 65, 100, 129, 200, 256, 300])
    Lk = rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 333, 500])
    return dict(D=D, bits=bits, mode=mode, B=B, H=H, Lq=Lq, Lk=Lk, asym=rng.random() < 0.5, splits=rng.choice([0, 1, 2, 3, 8]),
                layout=rng.choice(['BHLc', 'BLHc']), limit=rng.random() < 0.4,
                group=rng.choice([g for g in (32, 64, 128) if g <= D]), nseg=rng.choice([1, 2, 3, 7, 16]))


@pytest.mark.parametrize('seed', range(60))
def test_random_case(dev, seed):
    rng = random.Random(9000 + seed)
    c = _case(rng)
    D, bits, B, H, Lq, Lk, asym, layout = c['D'], c['bits'], c['B'], c['H'], c['Lq'], c['Lk'], c['asym'], c['layout']
    note('random attention case', seed, c)
    g = torch.Generator().manual_seed(seed)
    k = (torch.randn(B, H, Lk, D, generator=g) * rng.choice([0.5, 1.0, 3.0])).bfloat16()
    v = (torch.randn(B, H, Lk, D, generator=g) + rng.choice([0.0, 2.0])).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=g).bfloat16()
    # every query sees at least one key (a query without keys has no softmax to compare)
    lim = torch.randint(1, Lk + 1, (Lq,), generator=g).int() if c['limit'] else None
    bias = None
    if lim is not None:
        bias = torch.zeros(Lq, Lk)
        bias[torch.arange(Lk)[None, :] >= lim[:, None].long()] = float('-inf')
    scale = 1.0 / math.sqrt(D)
    tr = (lambda t: t) if layout == 'BHLc' else (lambda t: None if t is None else t.transpose(1, 2).contiguous())
    put = lambda t: None if t is None else t.to(dev)
    if c['mode'] == 'token':
        grp = c['group']
        packs = []
        for x in (k, v):
            cq, s, z = O.quant_groupwise(x, grp, bits, asym)
            packs.append((O.pack_last_dim(cq, bits)[0], s, z, O.dequant_groupwise(cq, s, z, grp)))
        (kw, ks, kz, kd), (vw, vs, vz, vd) = packs
        out = ops.fused_attn(put(tr(q)), put(tr(kw)), put(tr(ks)), put(tr(kz)), put(tr(vw)), put(tr(vs)), put(tr(vz)), bits, bits, Lk,
                             scale, kv_limit=put(lim), splits=c['splits'], layout=layout)
    else:
        nseg = min(c['nseg'], Lk)
        cuts = sorted(rng.sample(range(1, Lk), nseg - 1)) + [Lk] if nseg > 1 else [Lk]
        per = []
        for x in (k, v):
            ws, ds, ss, zs, a = [], [], [], [], 0
            for e in cuts:
                cq, s, z = O.quant_reduce(x[:, :, a:e], (0, 2), bits, asym)
                ws.append(O.pack_last_dim(cq, bits)[0])
                ds.append(O.dequant_asym(cq, s, z) if asym else O.dequant_sym(cq, s))
                ss.append(s.reshape(H, D))
                zs.append(z.reshape(H, D) if asym else None)
                a = e
            per.append((torch.cat(ws, 2).contiguous(), torch.stack(ss).contiguous(),
                        torch.stack(zs).contiguous() if asym else None, torch.cat(ds, 2)))
        (kw, ks, kz, kd), (vw, vs, vz, vd) = per
        out = ops.fused_attn_channel(put(tr(q)), put(tr(kw)), put(ks), put(kz), put(tr(vw)), put(vs), put(vz), bits, Lk, scale,
                                     kv_limit=put(lim), seg_ends=cuts, splits=c['splits'], layout=layout)
    torch.cuda.synchronize()
    out = tr(out.cpu()) if layout == 'BLHc' else out.cpu()
    _compare(out, O.attention_ref(q, kd, vd, scale, bias), O.attention_exact(q.float(), kd, vd, scale, bias), f'random case {seed}')
