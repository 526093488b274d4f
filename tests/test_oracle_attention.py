"""Oracle checks for the attention leg: schedules, the block-causal mask in its
two forms, and the bf16 SDPA oracle against an fp64 softmax."""
import pytest
import torch

import varq_oracle as O


def test_schedules():
    assert sum(p * p for p in O.VAR_PATCH_NUMS) == 680
    assert sum(p * p for p in O.INFINITY_PATCH_NUMS) == 10521
    lvl = O.level_of_token(O.VAR_PATCH_NUMS)
    assert lvl.numel() == 680 and int(lvl[0]) == 0 and int(lvl[-1]) == 9 and int(lvl[1]) == 1 and int(lvl[5]) == 2


def test_mask_forms_agree():
    pn = (1, 2, 3, 4)
    bias = O.block_causal_bias(pn)
    L = 30
    assert bias.shape == (L, L)
    lim = O.kv_limit_from_schedule(pn)
    for q in range(L):
        vis = (bias[q] == 0).nonzero().flatten()
        assert vis.tolist() == list(range(int(lim[q])))       # a prefix, ending with the query's own scale
    assert lim.tolist()[:6] == [1, 5, 5, 5, 5, 14]
    # the last scale sees everything: the KV-cache inference case is all-visible
    assert bool((bias[-16:] == 0).all())
    sub = O.block_causal_bias(pn, q_start=5, q_len=9)
    assert torch.equal(sub, bias[5:14])


@pytest.mark.parametrize('masked', [False, True])
def test_sdpa_oracle_close_to_exact(masked):
    g = torch.Generator().manual_seed(5)
    pn = (1, 2, 3, 4, 5)
    L = sum(p * p for p in pn)
    q = torch.randn(2, 3, L, 64, generator=g)
    k = torch.randn(2, 3, L, 64, generator=g)
    v = torch.randn(2, 3, L, 64, generator=g)
    bias = O.block_causal_bias(pn) if masked else None
    q16, k16, v16 = (t.bfloat16() for t in (q, k, v))
    ref = O.attention_ref(q16, k16, v16, 0.125, bias)
    exact = O.attention_exact(q16.float(), k16.float(), v16.float(), 0.125, bias)
    assert ref.dtype == torch.bfloat16
    assert float((ref.double() - exact).abs().max()) < 2e-2
    cos = torch.nn.functional.cosine_similarity(ref.double().flatten(), exact.flatten(), dim=0)
    assert float(cos) > 0.9995


def test_synth_kv_is_seeded_and_has_outliers():
    a = O.synth_kv((2, 4, 50, 64), seed=1000)
    b = O.synth_kv((2, 4, 50, 64), seed=1000)
    assert torch.equal(a, b)
    ch_std = a.std(dim=(0, 1, 2))
    assert int((ch_std > 8).sum()) == 1                      # max(1, round(0.02*64)) = 1 channel x15
    t = O.synth_kv((1, 2, 2000, 128), seed=7, dist='student4', outlier_frac=0.01, outlier_mul=20.0)
    assert int((t.std(dim=(0, 1, 2)) > 10).sum()) == 1
