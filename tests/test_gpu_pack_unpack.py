"""Parity of the stand-alone pack / unpack / dequant kernels with the oracle,
through the reference's function names."""
import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import ops
from var_q_amd import pack_unpack as PU

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('shape', [(100, 680, 2, 64), (3, 7, 5, 128), (4, 10), (9, 33), (2, 3, 1), (1, 16), (0, 64)])
def test_pack_unpack_roundtrip_and_layout(dev, bits, shape):
    note('pack/unpack', bits, shape)
    lo, hi = O.qrange(bits)
    g = torch.Generator().manual_seed(bits)
    q = torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8)
    want, meta = O.pack_last_dim(q, bits) if q.numel() else (torch.empty((*shape[:-1], -(-shape[-1] // (32 // bits))), dtype=torch.int32), None)
    w, gmeta = PU.pack_last_dim_to_int32_triton(q.to(dev), bits)
    assert w.dtype == torch.int32 and w.shape == want.shape
    assert torch.equal(w.cpu(), want)
    if meta is not None:
        assert gmeta == meta
    back = PU.unpack_last_dim_from_int32_triton(w, gmeta)
    assert back.dtype == torch.int8 and torch.equal(back.cpu(), q)
    # the _python names are the same kernels
    w2, _ = PU.pack_last_dim_to_int32_python(q.to(dev), bits)
    assert torch.equal(w2, w)
    assert torch.equal(PU.unpack_last_dim_from_int32_python(w, gmeta), back)


def test_known_answer_words_on_gpu(dev):
    note('pack KAT')
    w, _ = PU.pack_last_dim_to_int32_triton(torch.tensor([[-1, -128, 127, 5]], dtype=torch.int8, device=dev), 8)
    assert w.tolist() == [[0x057F80FF]]
    w, _ = PU.pack_last_dim_to_int32_triton(torch.tensor([[-2, -1, 0, 1] * 4], dtype=torch.int8, device=dev), 2)
    assert w.tolist() == [[0x4E4E4E4E]]
    w, _ = PU.pack_last_dim_to_int32_triton(torch.arange(8, dtype=torch.int8, device=dev).view(1, 8), 4)
    assert w.tolist() == [[0x76543210]]


def test_asserts_like_reference(dev):
    with pytest.raises(AssertionError):
        PU.pack_last_dim_to_int32_triton(torch.zeros(2, 8, dtype=torch.int32, device=dev), 4)
    with pytest.raises(AssertionError):
        PU.pack_last_dim_to_int32_triton(torch.zeros(2, 8, dtype=torch.int8, device=dev), 3)
    with pytest.raises(AssertionError):
        PU.unpack_last_dim_from_int32_triton(torch.zeros(2, 1, dtype=torch.int8, device=dev),
                                             {'orig_c': 8, 'vals_per_word': 8, 'pad_len': 0, 'bits': 4})


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_dequant_matches_oracle(dev, bits, out_dtype):
    g = torch.Generator().manual_seed(bits + 40)
    lo, hi = O.qrange(bits)
    B, H, L, c = 2, 3, 11, 64
    q = torch.randint(lo, hi + 1, (B, H, L, c), generator=g, dtype=torch.int8)
    words, _ = O.pack_last_dim(q, bits)
    cases = {
        'per-tensor': (1, 1, 1, 1), 'per-head-dim': (1, H, 1, c), 'token-head': (1, H, L, 1),
        'token': (1, 1, L, 1), 'group32': (B, H, L, 2), 'group64': (B, H, L, 1), 'per-head': (1, H, 1, 1),
    }
    for name, sshape in cases.items():
        for asym in (False, True):
            note('dequant', bits, out_dtype, name, asym)
            s = torch.rand(sshape, generator=g) + 0.01
            z = torch.randint(-9, 9, sshape, generator=g).float() if asym else None
            if sshape[3] in (1, c):
                want = O.dequant_asym(q, s, z) if asym else O.dequant_sym(q, s)
            else:
                want = O.dequant_groupwise(q, s, z, c // sshape[3])
            got = ops.dequant(words.to(dev), s.to(dev), None if z is None else z.to(dev), c, bits, out_dtype)
            assert got.dtype == out_dtype
            assert torch.equal(got.cpu(), want.to(out_dtype)), name
            got8 = ops.dequant(q.to(dev), s.to(dev), None if z is None else z.to(dev), c, bits, out_dtype)
            assert torch.equal(got8.cpu(), want.to(out_dtype)), name + ' (int8 codes)'


@pytest.mark.parametrize('L,c,group', [(680, 64, 32), (680, 64, 64), (300, 128, 64), (257, 64, 8), (40, 64, 16),
                                       (700, 96, 24), (700, 96, 48), (513, 128, 128), (90, 192, 32)])
@pytest.mark.parametrize('bits', [4, 8, 2])
def test_dequant_items_per_lane_and_group_sizes(dev, L, c, group, bits):
    """The launch gives a lane four, two or one octets depending on how many octets a (batch,
    head) pair has and how full its last block would be, and finds an octet's group by a shift
    when the group is 8 times a power of two, by a division otherwise."""
    if c % (32 // bits):
        pytest.skip('rows of whole words only')
    note('dequant items per lane', L, c, group, bits)
    g = torch.Generator().manual_seed(L + c + group + bits)
    lo, hi = O.qrange(bits)
    q = torch.randint(lo, hi + 1, (2, 3, L, c), generator=g, dtype=torch.int8)
    words, _ = O.pack_last_dim(q, bits)
    s = torch.rand(2, 3, L, c // group, generator=g) + 0.01
    z = torch.randint(-9, 9, (2, 3, L, c // group), generator=g).float()
    want = O.dequant_groupwise(q, s, z, group)
    got = ops.dequant(words.to(dev), s.to(dev), z.to(dev), c, bits, torch.bfloat16)
    assert torch.equal(got.cpu(), want.to(torch.bfloat16))
    got = ops.dequant(words.to(dev), s.to(dev), None, c, bits, torch.float32)
    assert torch.equal(got.cpu(), O.dequant_groupwise(q, s, None, group))


def test_dequant_ragged_channels_and_expanded_scale(dev):
    note('dequant ragged')
    g = torch.Generator().manual_seed(9)
    q = torch.randint(-8, 8, (2, 5, 3, 10), generator=g, dtype=torch.int8)
    words, _ = O.pack_last_dim(q, 4)
    s = (torch.rand(1, 1, 3, 10, generator=g) + 0.1).expand(1, 5, 3, 10)     # stride-0 expand along L
    got = ops.dequant(words.to(dev), s.to(dev).expand(1, 5, 3, 10), None, 10, 4)
    assert torch.equal(got.cpu(), O.dequant_sym(q, s))


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('rows,c,word_offset', [(5, 64, 0), (5, 64, 1), (7, 16, 0), (3, 48, 2), (1, 16, 0), (1021, 128, 0), (1021, 128, 3)])
def test_pack_unpack_word_tails_and_unaligned_words(dev, bits, rows, c, word_offset):
    """The fast kernels move 16 bytes per thread; word counts that are not a multiple of four and
    word buffers that start off a 16-byte boundary take the per-word kernel for the rest (or for
    everything).  Through the C ABI, against the oracle's words."""
    from var_q_amd import _lib
    if c % (32 // bits):
        pytest.skip('whole words only')
    note('pack/unpack tails', bits, rows, c, word_offset)
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    lo, hi = O.qrange(bits)
    g = torch.Generator().manual_seed(100 * bits + rows + word_offset)
    q = torch.randint(lo, hi + 1, (rows, c), generator=g, dtype=torch.int8)
    want, _ = O.pack_last_dim(q, bits)
    wpr = c * bits // 32
    qd = q.to(dev)
    buf = torch.full((rows * wpr + 8,), 0x5a5a5a5a, dtype=torch.int32, device=dev)
    words = buf[word_offset:word_offset + rows * wpr]
    _lib.check(lib.varq_pack(qd.data_ptr(), rows, c, bits, words.data_ptr(), st), 'varq_pack')
    torch.cuda.synchronize()
    assert torch.equal(words.cpu().reshape(rows, wpr), want)
    assert int(buf[word_offset + rows * wpr]) == 0x5a5a5a5a and (word_offset == 0 or int(buf[word_offset - 1]) == 0x5a5a5a5a), 'wrote past its words'
    back = torch.full((rows * c + 16,), 99, dtype=torch.int8, device=dev)
    _lib.check(lib.varq_unpack(words.data_ptr(), rows, c, bits, back.data_ptr(), st), 'varq_unpack')
    torch.cuda.synchronize()
    assert torch.equal(back[:rows * c].cpu().reshape(rows, c), q) and int(back[rows * c]) == 99


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('H,c', [(16, 128), (8, 64), (4, 32), (2, 16), (16, 64)])
def test_dequant_table_over_the_inner_rows(dev, bits, H, c):
    """One scale per (head, channel) of a token-major tensor [B,L,H,c] (the reference's default
    method in layout BLHc, VAR_Q/quant.py:84-88): the call reads the H rows of a token as one
    long row of H*c channels where that is a power-of-two number of octets up to 256.  Dense
    tensor and a window of a longer cache, symmetric and affine, fp32 and bf16 out."""
    g = torch.Generator().manual_seed(bits * 100 + H + c)
    lo, hi = O.qrange(bits)
    B, L, Lcap, first = 2, 301, 340, 17
    q = torch.randint(lo, hi + 1, (B, Lcap, H, c), generator=g, dtype=torch.int8)
    words, _ = O.pack_last_dim(q, bits)
    s = torch.rand(1, 1, H, c, generator=g) + 0.01
    z = torch.randint(-9, 9, (1, 1, H, c), generator=g).float()
    W = words.shape[-1]
    for asym in (False, True):
        for out_dtype in (torch.float32, torch.bfloat16):
            note('dequant table over the inner rows', bits, H, c, asym, out_dtype)
            zz = z if asym else None
            want = (O.dequant_asym(q, s, z) if asym else O.dequant_sym(q, s)).to(out_dtype)
            got = ops.dequant(words.to(dev), s.to(dev), None if zz is None else zz.to(dev), c, bits, out_dtype)
            assert torch.equal(got.cpu(), want)
            win = ops.dequant_window(words.to(dev), s.to(dev), None if zz is None else zz.to(dev), (B, L, H, c), [0, 0, c, 1],
                                     1, bits, [B, L, H, Lcap * H, H, 1, first * H, -1], out_dtype)
            assert torch.equal(win.cpu(), want[:, first:first + L])
