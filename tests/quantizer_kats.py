"""Hand-worked known answers for the groupwise affine quantizer.

The reference calls `MLX.quantized(_, groupSize:, bits:)` (KVCache.swift:506, :508, :975,
:1069, :1070); on `Device.cpu` that is the scalar loop `quantize<T, U>` of MLX core
(mlx/backend/cpu/quantized.cpp), which per group does, all in float32:

    w_max, w_min                     over the group
    mask  = |w_min| > |w_max|        (strict)
    scale = max((w_max - w_min) / n_bins, 1e-7);   scale = mask ? scale : -scale
    edge  = mask ? w_min : w_max
    q0    = rint(edge / scale)       (std::rint: half to even)
    if q0 != 0: scale = edge / q0, bias = edge      else bias = 0
    code  = min(max(rint((w - bias) / scale), 0), n_bins)    with the float32 scale / bias
    scales[i] = T(scale), biases[i] = T(bias)

Every expected value below was worked out by hand from those lines with exact fractions
(the arithmetic is written out beside each case); none was produced by running a
restatement.  Each case is built so that one plausible misreading of the algorithm gives a
different, stated answer.  The same table is run against the numpy oracle, the scalar-C
oracle (tests/test_oracle_kat.py) and the device quantizers (tests/test_gpu_cache.py).

A case is one group of 32 values: `head` followed by `fill` up to 32 elements.
`codes` are the expected codes of `head`, `fill_code` that of every filler element.
"""

U = 2.0 ** -24  # the smallest float16 subnormal

CASES = [
    dict(
        # Codes come from the float32 scale, not from the stored float16 one.
        #   w_max = 1, w_min = 0: mask false, scale = -(1/15), edge = 1, q0 = rint(-15) = -15,
        #   scale = 1 / -15 (float32: -0.066666670), bias = 1.
        #   x = 1639/16384 (a float16 value): (x - 1) / scale = 15 * 14745/16384 = 13.49945
        #   -> 13 (the float32 rounding of 1/15 moves the quotient by 1e-6, not across .5).
        #   Stored scale: float16(-1/15) = -1092/16384 = -0.06665039 (0xAC44).  Dividing by
        #   that instead gives 14745/1092 = 13.50275 -> 14.
        #   0.25 -> 15 * 0.75 = 11.25 -> 11;  0.75 -> 3.75 -> 4;  0 -> 15;  1 -> 0.
        name="float32 scale, not the stored float16 one",
        dtype="float16", bits=4,
        head=[1.0, 0.0, 1639 / 16384, 0.25, 0.75], fill=0.25,
        codes=[0, 15, 13, 11, 4], fill_code=11,
        scale_bits=0xAC44, bias_bits=0x3C00,
        wrong="code 14 for element 2 if the quotient uses the float16 scale",
    ),
    dict(
        # Ties go to even, for q0 and for the codes.
        #   w_min = -17, w_max = 13: mask true, scale = 30/15 = 2, edge = -17,
        #   q0 = rint(-8.5) = -8 (half away from zero: -9), scale = -17 / -8 = 2.125 exactly,
        #   bias = -17.  Codes rint((w + 17) / 2.125), all quotients exact:
        #   -15.9375 -> 0.5 -> 0;  -13.8125 -> 1.5 -> 2;  -11.6875 -> 2.5 -> 2;
        #   -9.5625 -> 3.5 -> 4;   -7.4375 -> 4.5 -> 4;   0 -> 8;  13 -> 14.12 -> 14;  -17 -> 0.
        #   float16(2.125) = 0x4040, float16(-17) = 0xCC40.
        name="round half to even",
        dtype="float16", bits=4,
        head=[-17.0, 13.0, -15.9375, -13.8125, -11.6875, -9.5625, -7.4375], fill=0.0,
        codes=[0, 14, 0, 2, 2, 4, 4], fill_code=8,
        scale_bits=0x4040, bias_bits=0xCC40,
        wrong="q0 = -9 (scale 1.8889) and codes 1, 2, 3, 4, 5 under round-half-away",
    ),
    dict(
        # The 1e-7 floor acts on a group that is not constant.
        #   values 0, 8u, 2u, 6u with u = 2^-24: range / 15 = 3.2e-8 < 1e-7, so scale = -1e-7
        #   (mask false), edge = 8u = 4.768e-7, q0 = rint(-4.768) = -5, scale = 8u / -5 =
        #   -9.537e-8, bias = 8u.  Codes (w - 8u) * -5 / 8u: 0 -> 5; 8u -> 0; 2u -> 3.75 -> 4;
        #   6u -> 1.25 -> 1.  Stored: float16(-1.6u) = -2u (0x8002), float16(8u) = 0x0008.
        #   Without the floor: scale = -8u/15, q0 = -15 and the zeros would get code 15.
        name="1e-7 floor on a non-constant group",
        dtype="float16", bits=4,
        head=[0.0, 8 * U, 2 * U, 6 * U], fill=0.0,
        codes=[5, 0, 4, 1], fill_code=5,
        scale_bits=0x8002, bias_bits=0x0008,
        wrong="code 15 for the zeros, scale bits 0x8001, if the floor is skipped",
    ),
    dict(
        # w_min == -w_max: the comparison is strict, so the edge is w_max and the scale negative.
        #   2 bits: scale = -(6/3) = -2, edge = 3, q0 = rint(-1.5) = -2, scale = 3 / -2 = -1.5,
        #   bias = 3.  Codes (w - 3) / -1.5: 3 -> 0; -3 -> 4 -> clamped to 3; 0 -> 2; 1.5 -> 1.
        #   float16(-1.5) = 0xBE00, float16(3) = 0x4200.  With >= the edge would be -3:
        #   scale +1.5, bias -3, codes 3, 0, 2, 3.
        name="equal magnitudes, 2 bits",
        dtype="float16", bits=2,
        head=[3.0, -3.0, 0.0, 1.5], fill=0.0,
        codes=[0, 3, 2, 1], fill_code=2,
        scale_bits=0xBE00, bias_bits=0x4200,
        wrong="scale +1.5 / bias -3 / codes 3, 0, 2, 3 if the comparison is not strict",
    ),
    dict(
        #   4 bits: w_max = 7.5, w_min = -7.5: scale = -(15/15) = -1, edge = 7.5,
        #   q0 = rint(-7.5) = -8, scale = 7.5 / -8 = -0.9375, bias = 7.5.
        #   Codes (w - 7.5) / -0.9375: 7.5 -> 0; -7.5 -> 16 -> clamped to 15; 0 -> 8;
        #   3.75 -> 4; -3.75 -> 12.  float16(-0.9375) = 0xBB80, float16(7.5) = 0x4780.
        name="equal magnitudes, 4 bits, upper clamp",
        dtype="float16", bits=4,
        head=[7.5, -7.5, 0.0, 3.75, -3.75], fill=0.0,
        codes=[0, 15, 8, 4, 12], fill_code=8,
        scale_bits=0xBB80, bias_bits=0x4780,
        wrong="scale +0.9375 / bias -7.5 / codes 15, 0, 8, 12, 4 if the comparison is not strict",
    ),
    dict(
        # bfloat16 storage of the parameters; 8-bit codes.
        #   w_max = 255, w_min = 0 (both bfloat16 values): scale = -1, edge = 255, q0 = -255,
        #   scale = 255 / -255 = -1, bias = 255.  Codes 255 - w: 0 -> 255; 255 -> 0; 100 -> 155;
        #   1.5 -> 253.5 -> 254 (even); 2.5 -> 252.5 -> 252 (even).
        #   bfloat16(-1) = 0xBF80, bfloat16(255) = 0x437F.
        name="bfloat16, 8 bits, ties at 253.5 and 252.5",
        dtype="bfloat16", bits=8,
        head=[0.0, 255.0, 100.0, 1.5, 2.5], fill=100.0,
        codes=[255, 0, 155, 254, 252], fill_code=155,
        scale_bits=0xBF80, bias_bits=0x437F,
        wrong="codes 254, 253 for the last two under round-half-away",
    ),
    dict(
        # Exact ties at the top of the 8-bit code range with a scale that is not a power of two (the
        # whole-tile device quantizer forms quotients with the hardware reciprocal and must redo these
        # with the exact division: its guard band around half-integers has to hold up to 254.5).
        #   s = 3/256: w_max = 255 s = 765/256, w_min = 0: scale = -(765/256)/255 = -3/256 exactly,
        #   edge = w_max, q0 = -255, scale = edge / q0 = -3/256, bias = 765/256.  Codes (w_max - w) / s:
        #   3/512 = 0.5 s -> 254.5 -> 254;  9/512 = 1.5 s -> 253.5 -> 254;  15/512 = 2.5 s -> 252.5 -> 252;
        #   765/512 = 127.5 s -> 127.5 -> 128;  0 -> 255;  w_max -> 0.
        #   float16(-3/256) = -1.5 * 2^-7 = 0xA200, float16(765/256) = 1.494140625 * 2 = 0x41FA.
        name="8-bit ties at 254.5 with scale 3/256",
        dtype="float16", bits=8,
        head=[765 / 256, 0.0, 3 / 512, 9 / 512, 15 / 512], fill=765 / 512,
        codes=[0, 255, 254, 254, 252], fill_code=128,
        scale_bits=0xA200, bias_bits=0x41FA,
        wrong="255 / 253 / 253 / 127 where a quotient a few 1e-5 off the tie is rounded as it stands",
    ),
]


def group_values(case):
    g = list(case["head"]) + [case["fill"]] * (32 - len(case["head"]))
    assert len(g) == 32
    return g


def group_codes(case):
    return list(case["codes"]) + [case["fill_code"]] * (32 - len(case["codes"]))


def packed_words(case):
    """The uint32 words of the group: element k of a word at bits [k*bits, (k+1)*bits)."""
    bits = case["bits"]
    per = 32 // bits
    codes = group_codes(case)
    words = []
    for i in range(0, 32, per):
        w = 0
        for k in range(per):
            w |= codes[i + k] << (k * bits)
        words.append(w)
    return words
