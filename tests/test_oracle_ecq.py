"""The ECQ oracle (oracle/hpx_oracle.c: orc_ecq_encode / orc_ecq_decode) against a hand-derived message and against
an independent model of the reference's serial execution.

The reference's ecq_body cannot be built here (CHECK_EQ needs glog; the body has neither driver nor caller), so
parity with a build of it is unpinned.  What pins the oracle to the reference's TEXT (ecq_body.h:157-286, :342-423):
a message derived by hand, and a pure-Python model that executes the body's statements one by one on a real byte
buffer, so that the scratch-under-the-payload aliasing happens by itself instead of being reasoned about."""
import warnings

import numpy as np
import pytest

import kat_vectors as kat

f32 = np.float32


def _u8_x86(v):
    """static_cast<uint8_t>(float) as an x86-64 build does it: truncate to int32 (NaN / out of range -> 0x80000000),
    keep the low byte.  Inside [0, 256) this is the C++ conversion; outside it C++ says nothing, and the body gets
    there when scratch elements 2 and 3 are read back with payload bytes in them (4- and 8-bit codes)."""
    v = float(v)
    if not (-2147483648.0 <= v < 2147483648.0):
        return 0
    return int(v) & 0xFF


def _same_floats(a, b):
    """bit-equal, except that any NaN matches any NaN (their payloads differ between machines)."""
    a, b = np.asarray(a), np.asarray(b)
    both_nan = np.isnan(a) & np.isnan(b)
    return bool(np.all((a.view(np.uint32) == b.view(np.uint32)) | both_nan))


def _model_encode(G, H, alpha, beta, bitwidth, seed):
    """ecq_body.h:157-286 statement by statement, serial order, on one byte buffer (out_uint8_t)."""
    N = G.size
    H = H.copy()
    s = (1 << (bitwidth - 1)) - 1
    dpb = 8 // bitwidth
    M = int(np.ceil(N * 1.0 / dpb))
    out = np.full(max(4 * N, 10 + M) + 8, 0xEE, np.uint8)           # out_uint8_t; 0xEE = what the caller left there
    GH = out[:4 * N].view(np.float32)                               # float* GH = reinterpret_cast<float*>(out_uint8_t)
    Q = out[10:]
    warnings.simplefilter("ignore", RuntimeWarning)                  # a corrupted scratch element may overflow; IEEE handles it
    for x in range(N):                                              # generate_GH
        GH[x] = f32(abs(float(G[x]) + alpha * float(H[x])))
    max_GH = f32(GH.max())
    out_true_size = 4 + 4 + 1 + 1 + M
    if float(max_GH) < 1e-6:
        for x in range(M - 1):
            Q[x] = 0
        for x in range(N):
            H[x] = f32(float(H[x]) * beta)
    else:
        gap = f32(max_GH / f32(s))
        gap_inverse = f32(1.0 / float(gap))
        for x in range(M - 1):                                      # generate_Q_update_H over M - 1 bytes
            q = 0
            draws = kat.lcg_draws((seed + x) % (1 << 32), 1 + dpb)[1:]      # srand discards one
            for k, j in enumerate(range(x * dpb, x * dpb + dpb)):
                f = f32(f32(GH[j] + max_GH) * gap_inverse)
                u = f32(float(draws[k]) / 4294967295.0)
                t = _u8_x86(f32(f + u))
                q |= (t << (bitwidth * k)) & 0xFF
                H[j] = f32(beta * float(H[j]) + float(f32(f32(f - f32(t)) * gap)))
            Q[x] = q
    header = np.zeros(10, np.uint8)
    header[0:4] = np.array([out_true_size], np.int32).view(np.uint8)
    header[4:8] = np.array([max_GH], np.float32).view(np.uint8)
    header[8] = bitwidth
    header[9] = M * dpb - N
    out[:10] = header
    return out[:10 + M].copy(), H, bool(9 + M < 4 * N)


# Hand-derived (ecq_body.h:105-131, :262-272).  b = 2: s = 1; alpha = 1, H = 0: GH = |G|; max = 1 -> gap = 1,
# gap_inverse = 1; N = 8 -> M = 2, and the loop covers M - 1 = 1 byte: elements 0..3 with the draws of seed 0
# (u = 0.82758, 0.65241, 0.83748, 0.05338):
#   f = GH + 1 = 1.5, 1.25, 1.75, 2.0 -> f + u = 2.328, 1.902, 2.587, 2.053 -> codes 2, 1, 2, 2
#   byte 0 = 2 | 1<<2 | 2<<4 | 2<<6 = 2 + 4 + 32 + 128 = 166 = 0xA6
#   H[j] = 0.5 * 0 + (f - code) * 1 = -0.5, 0.25, -0.25, 0.0; H[4..7] untouched
#   byte 1 is never written: it keeps scratch byte 9 + M = 11, the top byte of GH[2] = 0.75f = 0x3F400000 -> 0x3F
#   header: int32 12 | 1.0f | 2 | 0
# Decode: code * gap - max = 1, 0, 1, 1 (the signs of G[1], G[3] are gone), and 0x3F = codes 3, 3, 3, 0 -> 2, 2, 2, -1.
ECQ_G = np.array([0.5, -0.25, 0.75, -1.0, 0.1, 0.2, 0.3, 0.4], np.float32)
ECQ_MSG = bytes([12, 0, 0, 0]) + np.float32(1.0).tobytes() + bytes([2, 0, 0xA6, 0x3F])
ECQ_H1 = np.array([-0.5, 0.25, -0.25, 0.0, 0, 0, 0, 0], np.float32)
ECQ_DECODED = np.array([1, 0, 1, 1, 2, 2, 2, -1], np.float32)


# Two longer messages, derived by hand in the same way, that reach the places where the body reads its scratch back
# with payload bytes in it (ecq_body.h:171,180: the scratch GH starts at out[0], the payload Q at out[10]).  In both,
# max |G| = s, so gap = gap_inverse = 1 and f = |G| + s; alpha = 1, beta = 0.5, H = 0, seed 0; slot j of byte x draws
# u = float(X / 4294967295.0) with X = A_{j+2} (x) + C_{j+2} mod 2^32, (A_2, C_2) = (3265436265, 3554416254),
# (A_3, C_3) = (2155723957, 2802067423)  (naive_random.hpp:15-69, one discarded draw after srand(t + x)).
#
# 8 bits (s = 127, one element per byte), N = 20, M = 20, the loop covers bytes 0..18:
#   byte 0: f = 254,    u = 3554416254/(2^32-1) = 0.82758 -> code 254 = FE  -> out[10], byte 2 of GH[2]
#   byte 1: f = 128.5,  u = 2524885223/(2^32-1) = 0.58787 -> 129.09 -> 81   -> out[11], byte 3 of GH[2];  H[1] = 128.5 - 129 = -0.5
#   byte 2: GH[2] was 0.5 = 3F000000 and now reads 81FE0000 = -9.3e-38: f = 127 - 9.3e-38 = 127, u = 0.34816 -> 7F -> out[12],
#           byte 0 of GH[3];  H[2] = 0
#   byte 3: GH[3] was 2.25 = 40100000 and now reads 4010007F = 2.25 + 127 * 2^-22: f = 129.2500303 rounds to 129.25 + 2 * 2^-16,
#           u = 0.10846 -> 81;  H[3] = f - 129 = 0.250030517578125
#   bytes 4..18: untouched scratch, e.g. byte 8: f = 127.25, u = 3908102598/(2^32-1) = 0.90993 -> 128.16 -> 80, H[8] = -0.75
#   byte 19 is never written: it keeps out[29], byte 1 of GH[7] = 1 + 2^-15 = 3F800100 -> 01;  H[19] stays
#   header: int32 30 | 127.0f | 8 | 0
ECQ8_G = np.array([127.0, -1.5, 0.5, -2.25, 3.0, 10.75, -100.0, 1 + 2.0 ** -15, 0.25, 7.0, -31.5, 63.0, -0.125, 90.0, 5.5, -12.0,
                   126.0, 1.0, -2.0, 33.0], np.float32)
ECQ8_MSG = bytes([30, 0, 0, 0]) + np.float32(127.0).tobytes() + bytes([8, 0]) + bytes.fromhex("fe817f81828ae38080869ebe80d9848bfd808101")
ECQ8_H1 = np.array([0.0, -0.5, 0.0, 0.250030517578125, 0.0, -0.25, 0.0, 2.0 ** -15, -0.75, 0.0, 0.5, 0.0, -0.875, 0.0, 0.5, 0.0,
                    0.0, 0.0, 0.0, 0.0], np.float32)
# 4 bits (s = 7, two elements per byte), N = 36, M = 18, the loop covers bytes 0..16:
#   byte 0: elements 0, 1: f = 14, 7.5; u = 0.82758, 2802067423/(2^32-1) = 0.65241 -> codes 14, 8 -> 8E -> out[10], byte 2 of GH[2]
#   byte 1: element 2 was 1.0 = 3F800000 and now reads 3F8E0000 = 1.109375: f = 8.109375, u = 0.58787 -> 8, H[2] = 0.109375;
#           element 3: f = 9.25, u = 662824084/(2^32-1) = 0.15433 -> 9, H[3] = 0.25 -> 98
#   byte 2 onwards: untouched scratch (byte x reads out[8x .. 8x+7] and writes out[10 + x])
#   byte 17 is never written: it keeps out[27], byte 3 of GH[6] = 1.5 + 2^-10 = 3FC02000 -> 3F;  H[34], H[35] stay
#   header: int32 28 | 7.0f | 4 | 0
ECQ4_G = np.array([7.0, -0.5, 1.0, 2.25, -3.0, 4.75, 1.5 + 2.0 ** -10, 0.25, 6.0, -6.5, 0.0, 3.5, -1.25, 5.0, 2.0, -2.75, 0.75, 4.0,
                   -5.25, 1.0, 3.0, 0.5, -6.0, 2.5, 1.75, -0.25, 5.5, 4.25, -3.75, 0.125, 6.75, 2.0, -1.0, 3.25, 0.5, -4.5], np.float32)
ECQ4_MSG = bytes([28, 0, 0, 0]) + np.float32(7.0).tobytes() + bytes([4, 0]) + bytes.fromhex("8e98ca78eda7c899b88c8a9d79bd7b9da83f")
ECQ4_H1 = np.array([0.0, -0.5, 0.109375, 0.25, 0.0, -0.25, 0.5009765625, 0.25, 0.0, -0.5, 0.0, 0.5, 0.25, 0.0, 0.0, 0.75, -0.25, 0.0,
                    0.25, 0.0, 0.0, -0.5, 0.0, 0.5, -0.25, 0.25, -0.5, 0.25, -0.25, 0.125, 0.75, 0.0, 0.0, 0.25, 0.0, 0.0], np.float32)
ECQ_LONG = ((8, ECQ8_G, ECQ8_MSG, ECQ8_H1), (4, ECQ4_G, ECQ4_MSG, ECQ4_H1))


@pytest.mark.parametrize("bitwidth,G,want,h_want", ECQ_LONG, ids=["8bit", "4bit"])
def test_hand_derived_messages_that_reread_the_scratch(oracle_cpu, bitwidth, G, want, h_want):
    h = np.zeros(G.size, np.float32)
    rc, msg, defined = oracle_cpu.ecq_encode(G.copy(), h, 1.0, 0.5, bitwidth, 0)
    assert rc == 0 and defined and msg.tobytes() == want, msg.tobytes().hex()
    assert np.array_equal(h, h_want), h
    m, h2, d = _model_encode(G, np.zeros(G.size, np.float32), 1.0, 0.5, bitwidth, 0)
    assert m.tobytes() == want and np.array_equal(h2, h_want) and d


def test_hand_derived_message(oracle_cpu):
    h = np.zeros(8, np.float32)
    rc, msg, defined = oracle_cpu.ecq_encode(ECQ_G.copy(), h, 1.0, 0.5, 2, 0)
    assert rc == 0 and defined and msg.tobytes() == ECQ_MSG, msg.tobytes().hex()
    assert np.array_equal(h, ECQ_H1)
    out = np.full(8, 9.0, np.float32)
    assert oracle_cpu.ecq_decode(msg, out, 0) == 0 and np.array_equal(out, ECQ_DECODED)
    out = np.full(8, 0.5, np.float32)
    assert oracle_cpu.ecq_decode(msg, out, 1) == 0 and np.array_equal(out, ECQ_DECODED + f32(0.5))
    # the model agrees with the hand derivation too
    m, h2, d = _model_encode(ECQ_G, np.zeros(8, np.float32), 1.0, 0.5, 2, 0)
    assert m.tobytes() == ECQ_MSG and np.array_equal(h2, ECQ_H1) and d


@pytest.mark.parametrize("bitwidth", [2, 4, 8])
def test_against_the_serial_model(oracle_cpu, bitwidth):
    rng = np.random.default_rng(100 + bitwidth)
    for n in [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 64, 100, 257]:
        for seed in (0, 12345, 2**32 - 1, 2**40 + 7):
            G = rng.normal(0, 1e-2, n).astype(np.float32)
            H0 = rng.normal(0, 5e-3, n).astype(np.float32)
            alpha, beta = float(rng.choice([0.0, 0.5, 1.0])), float(rng.choice([0.0, 0.9, 1.0]))
            want, h_want, defined = _model_encode(G, H0, alpha, beta, bitwidth, seed)
            h = H0.copy()
            rc, msg, d = oracle_cpu.ecq_encode(G.copy(), h, alpha, beta, bitwidth, seed)
            assert rc == 0 and d == defined, (n, seed)
            upto = msg.size if defined else msg.size - 1           # the last byte is the caller's when 9 + M >= 4 N
            assert np.array_equal(msg[:upto], want[:upto]), (n, bitwidth, seed, msg.tobytes().hex(), want.tobytes().hex())
            assert _same_floats(h, h_want), (n, bitwidth, seed)
            # decode: code * gap - max for every element the header announces, the junk of the last byte included
            out = np.zeros(n, np.float32)
            assert oracle_cpu.ecq_decode(want, out, 0) == 0
            mx = want[4:8].view(np.float32)[0]
            gap = f32(mx / f32((1 << (bitwidth - 1)) - 1))
            dpb = 8 // bitwidth
            codes = np.array([(int(want[10 + x // dpb]) >> ((x % dpb) * bitwidth)) & ((1 << bitwidth) - 1) for x in range(n)])
            assert np.array_equal(out, (codes.astype(np.float32) * gap - mx).astype(np.float32))


def test_zero_input_and_bad_arguments(oracle_cpu):
    # max |G + alpha H| < 1e-6: payload bytes 0 .. M-2 are zero, H *= beta for ALL elements (ecq_body.h:206-226)
    n = 40
    G = np.full(n, 1e-8, np.float32)
    H0 = np.full(n, 2e-8, np.float32)
    h = H0.copy()
    rc, msg, defined = oracle_cpu.ecq_encode(G, h, 1.0, 0.5, 2, 3)
    assert rc == 0 and not msg[10:-1].any() and np.array_equal(h, (H0.astype(np.float64) * 0.5).astype(np.float32))
    want, h_want, _ = _model_encode(G, H0, 1.0, 0.5, 2, 3)
    assert np.array_equal(msg, want) and np.array_equal(h, h_want)
    # widths other than 2, 4, 8 are refused (the reference aborts there, ecq_body.h:172-175)
    assert oracle_cpu.ecq_encode(G, h, 1.0, 0.5, 1, 0)[0] == -1
    assert oracle_cpu.ecq_encode(G, h, 1.0, 0.5, 3, 0)[0] == -1
    # an output smaller than the message's element count is refused (ecq_body.h:386-390)
    assert oracle_cpu.ecq_decode(want, np.zeros(n - 1, np.float32), 0) == -1


def test_codes_span_the_upper_half_and_history_compensates(oracle_cpu):
    # what the codec does, independent of its quirks: codes s .. 2s+1 (the sign is lost), and the history carries
    # the rounding error, so that with alpha = 1 the next round quantises |G + H|
    rng = np.random.default_rng(5)
    n, b = 4096, 4
    G = rng.normal(0, 1, n).astype(np.float32)
    h = np.zeros(n, np.float32)
    rc, msg, _ = oracle_cpu.ecq_encode(G, h, 1.0, 0.0, b, 1)
    out = np.zeros(n, np.float32)
    assert oracle_cpu.ecq_decode(msg, out, 0) == 0
    body = slice(4, n - 8 // b)                                  # all but the last byte's elements and the scratch elements that may be read back with a payload byte in them
    mx = msg[4:8].view(np.float32)[0]
    gap = mx / 7
    assert (out[body] >= 0).all() and np.abs(out[body] - np.abs(G[body])).max() <= gap * 1.001
    assert np.allclose(h[body], np.abs(G[body]) - out[body], atol=1e-5)     # beta = 0: H = unrounded - rounded
