"""Writes tests/golden/known_answers.json: small input/output vectors worked out by hand
from the reference's formulas, for the oracle (CPU tests) and the HIP kernels (GPU tests).

Nothing is imported from the reference, the oracle or this package: every expected value
below is a literal with its derivation next to it, and the script only lays the literals
out as JSON.  Sources of the formulas: bit layout VAR_Q/pack_unpack.py:167-211 (field j of
a word = code (c mod vals) in two's complement at bit j*bits, zero padding, little-endian
fields); symmetric quantizer VAR_Q/quant.py:112-121 (scale = max|x| / qmax clamped at eps,
code = clamp(round_half_even(x / scale), qmin, qmax)); the affine variant used by this
build (scale = (max - min) / (2^bits - 1), zp = qmin - round(min / scale),
code = clamp(round(x / scale) + zp)).  Inputs are chosen so that every intermediate is
exactly representable in fp32 (scales are 1 or 8/7 applied to small dyadic numbers)."""
import json
import os


def u32_to_i32(v):
    return v - (1 << 32) if v >= (1 << 31) else v


PACK = [
    # 8 bits, 4 codes per word: bytes little-endian -> 0x05 7F 80 FF
    {'bits': 8, 'codes': [-1, -128, 127, 5], 'words': [u32_to_i32(0x057F80FF)], 'pad_len': 0},
    # 4 bits: eight times -1 = all ones
    {'bits': 4, 'codes': [-1] * 8, 'words': [-1], 'pad_len': 0},
    # 4 bits: code j in field j
    {'bits': 4, 'codes': [0, 1, 2, 3, 4, 5, 6, 7], 'words': [0x76543210], 'pad_len': 0},
    # 4 bits: -8 = 0b1000 in the top field only
    {'bits': 4, 'codes': [0, 0, 0, 0, 0, 0, 0, -8], 'words': [-(1 << 31)], 'pad_len': 0},
    # 2 bits: fields 10 11 00 01 -> byte 0b01001110 = 0x4E, four times
    {'bits': 2, 'codes': [-2, -1, 0, 1] * 4, 'words': [0x4E4E4E4E], 'pad_len': 0},
    # 4 bits, 10 codes: second word holds 5 (0x5) and -5 (0xB) and six zero fields
    {'bits': 4, 'codes': [1, -1, 2, -2, 3, -3, 4, -4, 5, -5],
     'words': [u32_to_i32(0xC4D3E2F1), 0x000000B5], 'pad_len': 6},
    # 8 bits, 5 codes: one padded word
    {'bits': 8, 'codes': [1, 2, 3, 4, -2], 'words': [0x04030201, 0x000000FE], 'pad_len': 3},
]

QUANT_SYM = [
    # max|x| = 127 -> scale 1; ties go to even: -63.5 -> -64, 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -2.5 -> -2
    {'bits': 8, 'x': [127.0, -63.5, 0.5, 1.5, 2.5, -2.5], 'scale_num': 127.0, 'scale_den': 127.0,
     'codes': [127, -64, 0, 2, 2, -2]},
    # max|x| = 8 -> scale 8/7; x * 7/8 = 6.125, 3.0625, 2.1875, -1.3125, -7
    {'bits': 4, 'x': [7.0, 3.5, 2.5, -1.5, -8.0], 'scale_num': 8.0, 'scale_den': 7.0, 'codes': [6, 3, 2, -1, -7]},
    # 2 bits: qmax = 1, scale = 1; 0.5 -> 0 and -0.5 -> 0 (ties to even), -2 is never produced
    {'bits': 2, 'x': [1.0, 0.5, -0.5, -1.0, 0.25], 'scale_num': 1.0, 'scale_den': 1.0, 'codes': [1, 0, 0, -1, 0]},
    # all zeros: scale clamps at eps = 1e-12, codes 0
    {'bits': 8, 'x': [0.0, 0.0, 0.0, 0.0], 'scale_num': 1e-12, 'scale_den': 1.0, 'codes': [0, 0, 0, 0]},
]

QUANT_ASYM = [
    # min 0, max 3, 2 bits: scale 3/3 = 1, zp = -2 - 0 = -2
    {'bits': 2, 'x': [0.0, 1.0, 2.0, 3.0], 'scale': 1.0, 'zp': -2.0, 'codes': [-2, -1, 0, 1]},
    # min -7.5, max 7.5, 4 bits: scale 15/15 = 1, zp = -8 - round(-7.5) = -8 + 8 = 0; 7.5 -> 8 clamps to 7
    {'bits': 4, 'x': [-7.5, 0.0, 7.5], 'scale': 1.0, 'zp': 0.0, 'codes': [-8, 0, 7]},
    # min 10, max 265, 8 bits: scale 255/255 = 1, zp = -128 - 10 = -138; 137.5 -> 138 (even) - 138 = 0
    {'bits': 8, 'x': [10.0, 265.0, 137.5, 11.0], 'scale': 1.0, 'zp': -138.0, 'codes': [-128, 127, 0, -127]},
]

if __name__ == '__main__':
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'known_answers.json')
    with open(out, 'w') as f:
        json.dump({'pack': PACK, 'quant_sym': QUANT_SYM, 'quant_asym': QUANT_ASYM}, f, indent=1)
    print('wrote', out)
