"""Known-answer vectors that can be checked with pencil and paper against the reference's source text.

Each case below states its inputs, the expected output as literals, and the derivation in the comment
above it; nothing here is computed by the code under test, by the CPU oracle or by any build of the
reference.  tests/test_oracle_kat.py holds the CPU oracle to them, tests/test_gpu_kat.py the HIP kernels.

Generator (naive_random.hpp:15-33): x <- 1103515245 * x + 12345 (mod 2^32); srand(s) sets x = s and
discards one draw.  From x = 0 the sequence is the textbook one of the ANSI-C rand() example:
12345, 3554416254, 2802067423, 3596950572, 229283573.
naive_real_random<float>(0,1) (naive_random.hpp:54-69) returns float(double(x) / 4294967295.0).
"""
import numpy as np

LCG_A, LCG_C, M32 = 1103515245, 12345, 1 << 32


def lcg_draws(seed, count):
    """`count` successive rand() values after `x = seed` (Python integers: independent of every build)."""
    x, out = seed % M32, []
    for _ in range(count):
        x = (LCG_A * x + LCG_C) % M32
        out.append(x)
    return out


def f32(values):
    return np.array(values, dtype=np.float32)


def header(bits, tail, mn, mx):
    """[bitwidth][tail][min f32 LE][max f32 LE], terngrad_body.h:219-224."""
    return bytes([bits, tail]) + np.float32(mn).tobytes() + np.float32(mx).tobytes()


# ---------------------------------------------------------------------------------------------------
# TernGrad, stochastic rounding (compress_with_random, terngrad_body.h:88-96).
#
# All cases use b = 2 and tensors whose minimum is 0 and maximum is 3, so that
#   gap = (3 - 0) / (4 - 1.0f) = 1.0f,  gap_inverse = float(1.0 / (1.0 + 1e-8)) = float(0.99999999) = 1.0f
#   (the next float below 1 is 1 - 2^-24 = 0.99999994: 0.99999999 is nearer to 1),
# and thetimes = (x - 0) * 1.0f = x exactly.  Byte i draws from srand(seed + i): one discarded value,
# then one value per slot; code = uint8(x + u) (truncation), OR-ed into the byte at bit 2 * slot.
#
# Case A, seed 0.
#   byte 0, srand(0): discard 12345; slots draw 3554416254, 2802067423, 3596950572, 229283573, i.e.
#     u = 0.82758, 0.65241, 0.83748, 0.05338 (each value / 4294967295).
#     x = 0.5, 1.4, 2.1, 2.96 -> x + u = 1.328, 2.052, 2.937, 3.013 -> codes 1, 2, 2, 3
#     byte = 1 | 2<<2 | 2<<4 | 3<<6 = 1 + 8 + 32 + 192 = 233 = 0xE9
#   byte 1, srand(1): x1 = 1103515245 + 12345 = 1103527590 (discarded); with the two-step jump
#     x -> 3265436265 x + 3554416254 and its successors the slots draw
#     2524885223, 662824084, 3295386429, 4182499122, i.e. u = 0.58787, 0.15433, 0.76727, 0.97381.
#     x = 0, 3, 1.5, 0.02 -> x + u = 0.588, 3.154, 2.267, 0.994 -> codes 0, 3, 2, 0
#     byte = 0 | 3<<2 | 2<<4 | 0<<6 = 12 + 32 = 44 = 0x2C
#   (byte 1 shows that the seed of byte i is seed + i, and holds the tensor's minimum and maximum.)
TG_A = dict(
    x=f32([0.5, 1.4, 2.1, 2.96, 0.0, 3.0, 1.5, 0.02]), bits=2, random=1, seed=0,
    draws_byte0=[12345, 3554416254, 2802067423, 3596950572, 229283573],
    draws_byte1=[1103527590, 2524885223, 662824084, 3295386429, 4182499122],
    message=header(2, 0, 0.0, 3.0) + bytes([0xE9, 0x2C]),
)

# Case B, the partial last byte (terngrad_body.h:275-298): N = 6, so byte 0 is drawn as above and the last
# two elements go into a tail byte that is ALWAYS rounded to nearest (nearbyint, ties to even) and stored at
# out[size - 1]; header byte 1 = number of unused slots = 2.
#   byte 0, seed 0: x = 0, 3, 2.1, 2.96 -> x + u = 0.828, 3.652, 2.937, 3.013 -> codes 0, 3, 2, 3
#     byte = 0 | 3<<2 | 2<<4 | 3<<6 = 12 + 32 + 192 = 236 = 0xEC
#   tail: nearbyint(1.5) = 2, nearbyint(0.5) = 0 -> 2 | 0<<2 = 2
TG_B = dict(
    x=f32([0.0, 3.0, 2.1, 2.96, 1.5, 0.5]), bits=2, random=1, seed=0,
    message=header(2, 2, 0.0, 3.0) + bytes([0xEC, 0x02]),
)

# Cases C1, C2: a draw that becomes u = 1.0f on the maximum element, so that the code reaches 4 and its
# bit 2 lands in the NEXT slot of the byte, because codes are OR-ed without a mask (terngrad_body.h:94-95).
# Seed 2948924249 is 3265436265^-1 * (0xFFFFFFFF - 3554416254) mod 2^32, i.e. the seed whose first slot draws
# 4294967295: srand gives 230538014 (discarded), then 4294967295, 3191464396, 288979989, 646343466, i.e.
# u = 1.0 (4294967295 / 4294967295), 0.74307, 0.06728, 0.15049.
#   C1: x = 3, 1.1, 0.5, 2.9 -> x + u = 4.0, 1.843, 0.567, 3.050 -> codes 4, 1, 0, 3
#       byte = 4 | 1<<2 | 0 | 3<<6 = 0b100 | 0b100 | 192 = 196 = 0xC4     (adding the fields would give 200)
#   C2: x = 3, 1.5, 0.5, 2.9 -> codes 4, 2, 0, 3
#       byte = 4 | 2<<2 | 0 | 3<<6 = 4 | 8 | 192 = 204 = 0xCC             (masking code 4 to 2 bits would give 200)
#   byte 1 (seed + 1) holds zeros only: 0 + u < 1 for every u < 1 -> 0x00 (its draws are checked to be < 2^32 - 128).
TG_C1 = dict(
    x=f32([3.0, 1.1, 0.5, 2.9, 0.0, 0.0, 0.0, 0.0]), bits=2, random=1, seed=2948924249,
    draws_byte0=[230538014, 4294967295, 3191464396, 288979989, 646343466],
    message=header(2, 0, 0.0, 3.0) + bytes([0xC4, 0x00]),
)
TG_C2 = dict(
    x=f32([3.0, 1.5, 0.5, 2.9, 0.0, 0.0, 0.0, 0.0]), bits=2, random=1, seed=2948924249,
    message=header(2, 0, 0.0, 3.0) + bytes([0xCC, 0x00]),
)

# Case D: the same overflow through the one draw whose quotient is rounded twice.  Seed 2038044377 makes the
# first slot draw 0xFFFFFF7F = 4294967167.  Exactly, 4294967167 / 4294967295 = 1 - 128 / (2^32 - 1), a hair
# BELOW 1 - 2^-25, the midpoint between the floats 1 - 2^-24 and 1; rounded once it would be 1 - 2^-24.  The
# reference first rounds the quotient to double: the hair (2^-57) is far below a double's half-ulp there
# (2^-54), so the double is exactly 1 - 2^-25, and that midpoint then rounds to even: u = 1.0f.
#   srand gives 2965899422 (discarded), then 4294967167, 3675433804, 3219933077, 3886551210:
#   u = 1.0, 0.85575, 0.74970, 0.90491;  x = 3, 0.1, 1.2, 0.05 -> x + u = 4.0, 0.956, 1.950, 0.955
#   codes 4, 0, 1, 0 -> byte = 4 | 0 | 1<<4 | 0 = 20 = 0x14   (with u = 0.99999994 slot 0 would be 3: 0x13)
TG_D = dict(
    x=f32([3.0, 0.1, 1.2, 0.05, 0.0, 0.0, 0.0, 0.0]), bits=2, random=1, seed=2038044377,
    draws_byte0=[2965899422, 4294967167, 3675433804, 3219933077, 3886551210],
    message=header(2, 0, 0.0, 3.0) + bytes([0x14, 0x00]),
)

# Case E, round to nearest (compress_without_random, terngrad_body.h:24-57: nearbyint, ties to even).
#   x = 0.5, 1.5, 2.5, 3 -> 0, 2, 2, 3 -> 0 | 2<<2 | 2<<4 | 3<<6 = 8 + 32 + 192 = 232 = 0xE8
#   x = 0, 0.49, 0.51, 2.5 -> 0, 0, 1, 2 -> 1<<4 | 2<<6 = 16 + 128 = 144 = 0x90
TG_E = dict(
    x=f32([0.5, 1.5, 2.5, 3.0, 0.0, 0.49, 0.51, 2.5]), bits=2, random=0, seed=0,
    message=header(2, 0, 0.0, 3.0) + bytes([0xE8, 0x90]),
)

# Decode (decompress_write_to, terngrad_body.h:101-127): out[i] = code * gap + min with gap = (3 - 0) / 3 = 1.
TG_A_DECODED = f32([1, 2, 2, 3, 0, 3, 2, 0])

TERNGRAD_CASES = {"A": TG_A, "B": TG_B, "C1": TG_C1, "C2": TG_C2, "D": TG_D, "E": TG_E}

# u = float(double(x) / 4294967295.0) for single draws (the last is the double rounding of case D).
U01_KNOWN = [(0, 0.0), (4294967295, 1.0), (0xFFFFFF80, 1.0), (0xFFFFFF7F, 1.0), (0xFFFFFE80, 1.0 - 2.0 ** -24),
             (1, 2.0 ** -32), (0x80000000, 0.5), (0x80000080, 0.5 + 2.0 ** -24)]
#   0x80000000 / (2^32 - 1) = 0.5 * (1 + 2^-32 + ...): above 0.5 by 2^-33, far less than half an ulp (2^-25) -> 0.5
#   0x80000080 = 2^31 + 128: x * 2^-32 = 0.5 + 2^-25, exactly the midpoint between 0.5 and 0.5 + 2^-24; the
#   quotient's excess (x * 2^-64) lifts it above the midpoint -> rounds UP to 0.5 + 2^-24 (ties-to-even on x itself
#   would give 0.5)
#   0xFFFFFE80: x * 2^-32 = 1 - 2^-24 - 2^-25 = midpoint between 1 - 2^-23 and 1 - 2^-24; lifted above -> 1 - 2^-24

# ---------------------------------------------------------------------------------------------------
# GradDrop (gd_body.h:102-232).  N = 16; the k-th sample is |R[(second draw after srand(seed + k)) mod 16]|
# (generate_sample_G, gd_body.h:36-41).  The second draw is 3265436265 * (seed + k) + 3554416254; modulo 16 only
# the low hex digits matter: 3265436265 = 0xC2A2AE69 -> 9, 3554416254 = 0xD3DC167E -> 14, so with seed 0
#   sample index k -> (9 k + 14) mod 16 = 14, 7, 0, 9, 2, 11, 4, 13, 6, 15, 8, 1, 10, 3, 12, 5.
GD_SAMPLE_INDEX_SEED0 = [14, 7, 0, 9, 2, 11, 4, 13, 6, 15, 8, 1, 10, 3, 12, 5]

_E = 0.125  # every value is a small multiple of 1/8: all sums are exact in fp32

# Case A: sample_rate 1 (all 16 indices, each once), drop_ratio 0.75: s = 0.25, expected = ceil(4.0) = 4,
# threshold index = int(16 * 0.25) = 4.  G[i] = (i + 1)/8 with a minus sign at odd i, R = 0, so R + G = G.
# |values| descending: 16/8, 15/8, 14/8, 13/8, 12/8 -> threshold = sample[4] = 1.5.
# Selected (strictly beyond the threshold, gd_body.h:59-67), ascending: i = 12, 13, 14, 15 -> 4 <= expected: no cut.
# Message: int32 4 + 8*4 = 36 | idx 12 13 14 15 | val 13/8, -14/8, 15/8, -16/8; those residual entries become 0.
_ga = f32([(i + 1) * _E * (-1 if i % 2 else 1) for i in range(16)])
GD_A = dict(
    g=_ga, r0=np.zeros(16, np.float32), sample_rate=1.0, drop_ratio=0.75, seed=0,
    threshold=1.5, idx=[12, 13, 14, 15], val=f32([1.625, -1.75, 1.875, -2.0]),
    r1=f32([(i + 1) * _E * (-1 if i % 2 else 1) if i < 12 else 0.0 for i in range(16)]),
)

# Case B: sample_rate 0.5 -> 8 samples at indices 14, 7, 0, 9, 2, 11, 4, 13; threshold index = int(8 * 0.25) = 2;
# expected = 4.  Magnitudes (in eighths): the sampled positions hold 8, 7, 6, 5, 4, 3, 2, 1 in that order, the
# others (i = 1, 3, 5, 6, 8, 10, 12, 15) hold 9, 10, 11, 12, 13, 14, 15, 16; sign minus at odd i.  Here the
# accumulation matters too: G carries half of each value and R the other half (R + G is exact).
# Sample descending: 8, 7, 6 -> threshold 6/8.  Beyond it: 7 (i=7), 8 (i=14) and all of 9..16 -> 10 candidates
# > expected: order by |R| descending and keep 4 (gd_body.h:176-187): 16 (i=15), 15 (i=12), 14 (i=10), 13 (i=8).
# Message: 36 | idx 15 12 10 8 | val -16/8, 15/8, 14/8, 13/8.
_mag_b = {14: 8, 7: 7, 0: 6, 9: 5, 2: 4, 11: 3, 4: 2, 13: 1, 1: 9, 3: 10, 5: 11, 6: 12, 8: 13, 10: 14, 12: 15, 15: 16}
_tb = f32([_mag_b[i] * _E * (-1 if i % 2 else 1) for i in range(16)])
_r1b = _tb.copy()
_r1b[[15, 12, 10, 8]] = 0.0
GD_B = dict(
    g=(_tb / 2).astype(np.float32), r0=(_tb / 2).astype(np.float32), sample_rate=0.5, drop_ratio=0.75, seed=0,
    threshold=0.75, idx=[15, 12, 10, 8], val=f32([-2.0, 1.875, 1.75, 1.625]), r1=_r1b,
)

# Case C: as B, but the three largest magnitudes sit ON sampled positions, so the threshold is high and the
# outcome depends on exactly which positions the index stream visits: i=14 -> 16, i=7 -> 15, i=0 -> 14, the
# other sampled positions 9, 2, 11, 4, 13 -> 5, 4, 3, 2, 1, the unsampled 1, 3, 5, 6, 8, 10, 12, 15 -> 6..13.
# Sample descending: 16, 15, 14 -> threshold 14/8.  Beyond it: 15 (i=7), 16 (i=14) -> 2 <= expected, ascending.
# Message: 4 + 16 = 20 | idx 7 14 | val -15/8, 16/8.
# (Were the FIRST draw used, the stream would be (13 k + 9) mod 16 = 9, 6, 3, 0, 13, 10, 7, 4: threshold 11/8,
#  and i = 0, 7, 12, 14, 15 would be beyond it - five candidates, cut to four.)
_mag_c = {14: 16, 7: 15, 0: 14, 9: 5, 2: 4, 11: 3, 4: 2, 13: 1, 1: 6, 3: 7, 5: 8, 6: 9, 8: 10, 10: 11, 12: 12, 15: 13}
_tc = f32([_mag_c[i] * _E * (-1 if i % 2 else 1) for i in range(16)])
_r1c = _tc.copy()
_r1c[[7, 14]] = 0.0
GD_C = dict(
    g=_tc.copy(), r0=np.zeros(16, np.float32), sample_rate=0.5, drop_ratio=0.75, seed=0,
    threshold=1.75, idx=[7, 14], val=f32([-1.875, 2.0]), r1=_r1c,
)

GRADDROP_CASES = {"A": GD_A, "B": GD_B, "C": GD_C}


def gd_message(case):
    k = len(case["idx"])
    return np.concatenate([np.array([4 + 8 * k], np.int32).view(np.uint8), np.array(case["idx"], np.int32).view(np.uint8),
                           case["val"].view(np.uint8)])


# ---------------------------------------------------------------------------------------------------
# TBQ (compress functor, tbq_body.h:57-88): r += g; r >= thr -> field ^= 3 (01 -> 10), r -= thr;
# r <= -thr -> field ^= 1 (01 -> 00), r += thr; a byte starts as 0b01010101 = 85; the last, partial group
# leaves its unused fields at 01.  thr = 0.25, r = 0, ten elements (all arithmetic exact):
#   g = .5, -.5, .125, -.125 -> codes 2, 0, 1, 1 -> 2 | 0<<2 | 1<<4 | 1<<6 = 2 + 16 + 64 = 82;  r = .25, -.25, .125, -.125
#   g = .25, -.25, 0, 1     -> codes 2, 0, 1, 2 -> 2 + 16 + 128 = 146;                     r = 0, 0, 0, .75
#   g = -1, .375 (+ two unused fields) -> codes 0, 2, 1, 1 -> 0 | 2<<2 | 1<<4 | 1<<6 = 8 + 16 + 64 = 88;  r = -.75, .125
# Decode (tbq_body.h:22-36): (code - 1) * thr.
TBQ_A = dict(
    g=f32([.5, -.5, .125, -.125, .25, -.25, 0, 1, -1, .375]), thr=0.25,
    packed=bytes([82, 146, 88]),
    r1=f32([.25, -.25, .125, -.125, 0, 0, 0, .75, -.75, .125]),
    decoded=f32([.25, -.25, 0, 0, .25, -.25, 0, .25, -.25, .25]),
)
