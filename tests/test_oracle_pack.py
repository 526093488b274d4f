"""Pins the oracle's bit layout (VAR_Q/pack_unpack.py:167-211) without the
reference: hand-computed words, an independent numpy loop, and invariants."""
import numpy as np
import pytest
import torch

import varq_oracle as O


def test_known_answer_words():
    # 8-bit: bytes little-endian, two's complement.  [-1,-128,127,5] -> 0x057F80FF
    w, meta = O.pack_last_dim(torch.tensor([[-1, -128, 127, 5]], dtype=torch.int8), 8)
    assert w.tolist() == [[0x057F80FF]] and w.dtype == torch.int32
    assert meta == {'orig_c': 4, 'vals_per_word': 4, 'pad_len': 0, 'bits': 8}
    # 4-bit: eight -1 -> all ones -> int32 -1
    w, _ = O.pack_last_dim(torch.full((1, 8), -1, dtype=torch.int8), 4)
    assert w.tolist() == [[-1]]
    # 4-bit: codes 0..7 -> nibble j = j -> 0x76543210
    w, _ = O.pack_last_dim(torch.arange(8, dtype=torch.int8).view(1, 8), 4)
    assert w.tolist() == [[0x76543210]]
    # 4-bit: -8 in field 7 only -> 0x80000000 -> int32 min
    q = torch.zeros(1, 8, dtype=torch.int8); q[0, 7] = -8
    assert O.pack_last_dim(q, 4)[0].tolist() == [[-2 ** 31]]
    # 2-bit: [-2,-1,0,1] x4 -> fields 10,11,00,01 -> byte 0b01001110 = 0x4E per 4 codes
    w, _ = O.pack_last_dim(torch.tensor([[-2, -1, 0, 1] * 4], dtype=torch.int8), 2)
    assert w.tolist() == [[0x4E4E4E4E]]


def test_padding_is_zero_and_meta():
    q = torch.tensor([[1, -1, 2, -2, 3, -3, 4, -4, 5, -5]], dtype=torch.int8)  # C=10, 4-bit -> 2 words
    w, meta = O.pack_last_dim(q, 4)
    assert meta == {'orig_c': 10, 'vals_per_word': 8, 'pad_len': 6, 'bits': 4}
    assert w.shape == (1, 2)
    assert (int(w[0, 1]) & 0xFFFFFFFF) >> 8 == 0            # fields 2..7 of the last word are padding
    assert (int(w[0, 1]) & 0xFF) == (5 & 0xF) | ((-5 & 0xF) << 4)
    assert torch.equal(O.unpack_last_dim(w, meta), q)


def _numpy_pack(q, bits):
    vals = 32 // bits
    rows, c = q.shape
    nw = -(-c // vals)
    out = np.zeros((rows, nw), dtype=np.uint32)
    for r in range(rows):
        for ch in range(c):
            out[r, ch // vals] |= np.uint32((int(q[r, ch]) & ((1 << bits) - 1)) << ((ch % vals) * bits))
    return out.view(np.int32)


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('c', [1, 7, 8, 10, 16, 33, 64])
def test_matches_independent_loop_and_roundtrips(bits, c):
    g = torch.Generator().manual_seed(bits * 100 + c)
    lo, hi = O.qrange(bits)
    q = torch.randint(lo, hi + 1, (5, c), generator=g, dtype=torch.int8)
    w, meta = O.pack_last_dim(q, bits)
    assert np.array_equal(w.numpy(), _numpy_pack(q.numpy(), bits))
    assert torch.equal(O.unpack_last_dim(w, meta), q)


@pytest.mark.parametrize('bits', [2, 4, 8])
def test_bijection_on_full_words(bits):
    """Every code pattern of one word maps to a distinct word (exhaustive for 2
    fields, sampled otherwise) and every field is independent of the others."""
    vals = 32 // bits
    lo, hi = O.qrange(bits)
    base = torch.zeros(1, vals, dtype=torch.int8)
    seen = set()
    for j in range(vals):
        for code in range(lo, hi + 1):
            q = base.clone(); q[0, j] = code
            w = int(O.pack_last_dim(q, bits)[0][0, 0]) & 0xFFFFFFFF
            assert w == ((code & ((1 << bits) - 1)) << (j * bits))
            seen.add((j, code, w))
    assert len({s[2] for s in seen if s[1] != 0}) == vals * (hi - lo)


def test_leading_dims_preserved():
    q = torch.randint(-8, 8, (2, 3, 5, 16), dtype=torch.int8)
    w, meta = O.pack_last_dim(q, 4)
    assert w.shape == (2, 3, 5, 2)
    assert torch.equal(O.unpack_last_dim(w, meta), q)
