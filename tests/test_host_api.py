"""Host-side mirror of the reference's Python surface: constructor contract,
derived fields, config loader, schedules -- and that CPU tensors are refused
rather than silently computed somewhere else."""
import json
import os

import pytest
import torch

import var_q_amd
from var_q_amd import VAR_Q, VarqError, load_varq_config, schedules
from var_q_amd import pack_unpack as PU

PKG = os.path.dirname(var_q_amd.__file__)


def test_constructor_contract_matches_reference():
    q = VAR_Q()
    assert (q.quant_bits, q.qkv_format, q.quant_method, q.cur_blk_idx, q.pack_to_int32, q.eps) == \
        (8, 'BLHc', 'G_SCALE_HEAD_DIM', 0, True, 1e-12)
    assert q.dim_cat == 1 and q.dim_map['G_TOKEN'] == (0, 2, 3) and q.dim_map['G_SCALE_HEAD_DIM'] == (0, 1)
    assert (q.bound_min, q.bound_max) == (-128, 127)
    assert q.cached_item is None and q.cached_scale is None and q.quantized_item is None and q.scale is None
    assert q._pack_meta is None
    q = VAR_Q(4, 'BHLc', 'G_TOKEN_HEAD', blk_idx=7)
    assert q.dim_cat == 2 and q.dim_map['G_SCALE_HEAD_DIM'] == (0, 2) and q.dim_map['G_TOKEN'] == (0, 1, 3)
    assert (q.bound_min, q.bound_max, q.cur_blk_idx) == (-8, 7, 7)
    for bad in (dict(qkv_format='LBHc'), dict(quant_method='PER_DIM'), dict(quant_bits=1), dict(quant_bits=9)):
        with pytest.raises(AssertionError):
            VAR_Q(**bad)
    with pytest.raises(AssertionError):
        VAR_Q(quant_method='G_GROUP')          # needs group_size


def test_qkv_format_assignment_rederives_layout():
    q = VAR_Q(8, 'BLHc')
    q.qkv_format = 'BHLc'                      # what Infinity's attention does every forward
    assert q.dim_cat == 2 and q.dim_map == VAR_Q(8, 'BHLc').dim_map


def test_cpu_tensors_are_refused():
    q = VAR_Q(8, 'BLHc')
    with pytest.raises(VarqError):
        q.use_var_q(torch.randn(1, 2, 2, 8))
    with pytest.raises(AssertionError):
        PU.pack_last_dim_to_int32_triton(torch.zeros(2, 8, dtype=torch.int8), 4)
    with pytest.raises(AssertionError):
        PU.unpack_last_dim_from_int32_triton(torch.zeros(2, 1, dtype=torch.int32),
                                             {'orig_c': 8, 'vals_per_word': 8, 'pad_len': 0, 'bits': 4})
    # the reference's _python pair takes CPU tensors; this drop-in says why it does not
    with pytest.raises(VarqError, match='no CPU fallback'):
        PU.pack_last_dim_to_int32_python(torch.zeros(2, 8, dtype=torch.int8), 4)
    with pytest.raises(VarqError, match='no CPU fallback'):
        PU.unpack_last_dim_from_int32_python(torch.zeros(2, 1, dtype=torch.int32),
                                             {'orig_c': 8, 'vals_per_word': 8, 'pad_len': 0, 'bits': 4})


def test_reference_import_names_resolve():
    from VAR_Q.quant import VAR_Q as A
    from VAR_Q.pack_unpack import (pack_last_dim_to_int32_triton, unpack_last_dim_from_int32_triton,  # noqa: F401
                                   pack_last_dim_to_int32_python, unpack_last_dim_from_int32_python)  # noqa: F401
    from VAR_Q.config_loader import VARQConfig, load_varq_config as L  # noqa: F401
    assert A is VAR_Q and L is load_varq_config


@pytest.mark.parametrize('name,infinity', [('VAR-VAR_Q-8.json', False), ('Infinity-VAR_Q-8.json', True),
                                           ('VAR-raw.json', False), ('Infinity-VAR_Q-4-g128.json', True),
                                           ('Infinity-VAR_Q-mixed-g64.json', True)])
def test_config_loader(name, infinity, tmp_path):
    cfg = load_varq_config(os.path.join(PKG, name))
    assert cfg.is_infinity_model() == infinity and cfg.is_var_model() != infinity
    qc = cfg.get_quantization_config()
    qc['enable'] = 'changed'
    assert cfg.config['quantization']['enable'] != 'changed'       # getters return copies
    assert cfg.get_device() in ('cuda', 'cpu')
    assert cfg.get_batch_processing_config()['batch_size'] == 50
    if infinity:
        assert cfg.get_checkpoint_paths()[1].endswith('infinity_2b_reg.pth')
    else:
        assert cfg.get_checkpoint_paths(16)[1].endswith('var_d16.pth')
        with pytest.raises(ValueError):
            cfg.get_checkpoint_paths()
    cfg.update_config({'quantization': {'q_bits': 4}, 'extra': {'a': 1}})
    assert cfg.config['quantization']['q_bits'] == 4 and cfg.config['extra'] == {'a': 1}
    if name != 'VAR-raw.json':
        assert cfg.config['quantization']['quant_method'] in ('G_SCALE_HEAD_DIM', 'G_GROUP')
        kw = cfg.quantizer_kwargs()
        VAR_Q(**kw)
    out = tmp_path / 'saved.json'
    cfg.save_config(str(out))
    assert json.load(open(out)) == cfg.config


def test_extended_quantization_schema_is_validated(tmp_path):
    cfg = load_varq_config(os.path.join(PKG, 'Infinity-VAR_Q-mixed-g64.json'))
    kw = cfg.packed_cache_kwargs(B=2, H=16, Lmax=100, D=128)
    assert kw['bits'] == cfg.config['quantization']['per_head_bits'] and kw['group_size'] == 64 and kw['symmetric'] is False
    with pytest.raises(ValueError, match='16 entries for 8 heads'):
        cfg.packed_cache_kwargs(B=2, H=8, Lmax=100, D=128)
    for bad, pat in (({'q_bits': 9}, 'q_bits'), ({'qkv_format': 'LBHc'}, 'qkv_format'), ({'symmetric': 'no'}, 'symmetric'),
                     ({'group_size': 0}, 'group_size'), ({'per_head_bits': [4, 3]}, 'per_head_bits'),
                     ({'quant_method': 'G_TOKEN_HEAD'}, 'per_head_bits')):
        c = load_varq_config(os.path.join(PKG, 'Infinity-VAR_Q-mixed-g64.json'))
        c.update_config({'quantization': bad})
        with pytest.raises(ValueError, match=pat):
            c.validate_quantization()
    # the reference's rule files stay valid and do not describe a packed cache
    ref = load_varq_config(os.path.join(PKG, 'Infinity-VAR_Q-8.json'))
    ref.validate_quantization()
    with pytest.raises(ValueError, match='G_GROUP'):
        ref.packed_cache_kwargs(2, 16, 100, 128)


def test_schedules_and_kv_limit():
    assert schedules.total_tokens(schedules.VAR_PATCH_NUMS) == 680
    assert schedules.total_tokens(schedules.INFINITY_PATCH_NUMS) == 10521
    lim = schedules.kv_limit((1, 2, 3))
    assert lim.dtype == torch.int32 and lim.tolist() == [1] + [5] * 4 + [14] * 9
    assert schedules.kv_limit((1, 2, 3), q_start=5).tolist() == [14] * 9
    import varq_oracle as O
    assert torch.equal(schedules.kv_limit(O.VAR_PATCH_NUMS), O.kv_limit_from_schedule(O.VAR_PATCH_NUMS))


def test_csv_report_appends_rows(tmp_path):
    from var_q_amd.stats import CsvReport, FIELDS
    path = str(tmp_path / 'q.csv')
    rep = CsvReport(path)
    rep.add({'tag': 'k', 'bits': 4, 'l2_norm_error': 0.125})
    CsvReport(path).add({'tag': 'v', 'bits': 2})          # reopening keeps the header and the rows
    rows = rep.rows()
    assert [r['tag'] for r in rows] == ['k', 'v'] and rows[0]['l2_norm_error'] == '0.125' and rows[1]['bits'] == '2'
    assert list(rows[0].keys()) == FIELDS


def test_cache_buffer_validation_of_the_row_map_calls():
    """The quantize-into-cache calls refuse buffers whose row lengths do not match
    (c, bits, group) or that the row map would overrun, before anything is launched."""
    import torch
    from var_q_amd import ops
    from var_q_amd._lib import VarqError
    B, H, L, D, bits, g = 2, 3, 5, 64, 4, 32
    W = D * bits // 32
    words = torch.zeros(B, H, L, W, dtype=torch.int32)
    dense = [B, H, L, H * L, L, 1, 0, -1]
    one = torch.zeros(B, H, L, 1)
    with pytest.raises(VarqError, match='expected 8 / 2'):
        ops._check_cache_buffers(D, g, bits, True, words, one, one.clone(), dense, 't')
    two = torch.zeros(B, H, L, 2)
    ops._check_cache_buffers(D, g, bits, True, words, two, two.clone(), dense, 't')
    ops._check_cache_buffers(D, g, bits, False, words, two, None, dense, 't')
    with pytest.raises(VarqError, match='zp buffer'):
        ops._check_cache_buffers(D, g, bits, True, words, two, None, dense, 't')
    with pytest.raises(VarqError, match='reaches row 30'):
        ops._check_cache_buffers(D, g, bits, True, words, two, two.clone(), [B, H, L, H * L, L, 1, 1, -1], 't')
    # a slot table over the heads: that dim counts from its first slot
    ops._check_cache_buffers(D, g, bits, True, words[:, :1].contiguous(), two[:, :1].contiguous(), two[:, :1].contiguous(),
                             [B, H, L, 1 * L, L, 1, 0, 1], 't')


def test_rows_read_as_channels_for_per_row_tables():
    """The host-side rewrite of a [n0,n1,n2,c] dequantization with one scale per (i2, channel)
    into long rows applies only where the bytes allow it."""
    from var_q_amd import ops
    f = ops._rows_as_channels
    # [B,L,H,c] = [2,100,16,128], table [1,1,H,c]: long rows of 2048 channels = 256 octets
    assert f(True, [2, 100, 16, 128], [0, 0, 128, 1], 1, 4, None) == ([1, 2, 100, 2048], [0, 0, 0, 1], None)
    # a window of a cache with room for 160 tokens per batch entry
    window = f(True, [2, 100, 16, 128], [0, 0, 128, 1], 1, 8, [2, 100, 16, 160 * 16, 16, 1, 32, -1])
    assert window == ([1, 2, 100, 2048], [0, 0, 0, 1], [1, 2, 100, 0, 160, 1, 2, -1])
    same = lambda *a: f(*a) == (a[1], a[2], a[5])
    assert same(True, [2, 100, 30, 64], [0, 0, 64, 1], 1, 8, None)          # 240 octets: not a power of two
    assert same(True, [2, 100, 32, 128], [0, 0, 128, 1], 1, 8, None)        # 512 octets: too long
    assert same(True, [2, 100, 3, 30], [0, 0, 30, 1], 1, 8, None)           # rows that are not whole octets
    assert same(True, [2, 100, 2, 8], [0, 0, 8, 1], 1, 2, None)             # 2-bit rows that are not whole words
    assert same(False, [2, 100, 16, 128], [0, 0, 128, 1], 1, 8, None)       # int8 codes, not packed words
    assert same(True, [2, 100, 16, 128], [0, 128 * 16, 128, 1], 1, 8, None) # the scale depends on i1 too
    assert same(True, [2, 100, 16, 128], [0, 0, 4, 1], 32, 4, None)         # group-wise scales
    assert same(True, [2, 100, 16, 128], [0, 0, 128, 1], 1, 8, [2, 100, 16, 100 * 16, 1, 100, 0, -1])   # rows of a pair apart
    assert same(True, [2, 100, 16, 128], [0, 0, 128, 1], 1, 8, [2, 100, 16, 160 * 16, 16, 1, 8, -1])    # window starts mid-row
