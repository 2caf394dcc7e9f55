"""Pins the oracle's restatement of the in-tree CompLL operator (min/max b-bit
stochastic quantiser with a 10-byte header) and of the reference's LCG.
Sources: /root/reference/src/CompLL/GCGen/pse/TernGradEncode.pse:22-33,
output/TernGradEncode/TernGradEncode_body.h:114,120-123,
output/TernGradDecode/TernGradDecode_body.h:44,65-72, output/naive_random.hpp:40-68."""
import struct

import numpy as np
import pytest

import oracle

F = np.float32


def codes_of(pay, n, b):
    """Codes read the way the reference decoder reads them."""
    Q = pay[10:]
    return np.array([(Q[i * b // 8] >> ((i % (8 // b)) * b)) & ((1 << b) - 1) for i in range(n)], dtype=np.uint32)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
def test_header_layout_and_sizes(b):
    g = np.array([-2.5, 0.0, 1.0, 3.5, 0.25], dtype=F)
    pay = oracle.compll_encode(g, np.zeros(5, F), b)
    assert pay.size == 10 + (5 * b + 7) // 8 == oracle.compll_payload_bytes(5, b)
    assert pay[0] == b
    assert pay[1] == 5 % (1 << b)  # the DSL's `gradient.size % (1<<bitwidth)`
    assert struct.unpack("<f", pay[2:6].tobytes())[0] == -2.5  # min at byte 2
    assert struct.unpack("<f", pay[6:10].tobytes())[0] == 3.5  # max at byte 6


def test_reduce_initial_values_bound_min_and_max():
    # reduce(gradient, -99999, greater) / reduce(gradient, 99999, smaller)
    pay = oracle.compll_encode(np.array([-2e5, -1e5 - 1], dtype=F), np.zeros(2, F), 2)
    assert struct.unpack("<f", pay[6:10].tobytes())[0] == F(-99999.0)
    pay = oracle.compll_encode(np.array([2e5, 3e5], dtype=F), np.zeros(2, F), 2)
    assert struct.unpack("<f", pay[2:6].tobytes())[0] == F(99999.0)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
def test_grid_points_round_trip_through_reference_decode(b):
    # values on the quantisation grid with noise 0.5 (round to nearest: float32 rounding of
    # (g - min) / gap may land a hair under the integer) decode to themselves
    levels = (1 << b) - 1
    n = 8 * 16  # a multiple of 2^b for b <= 4 keeps tail = 0; for b = 8, 128 % 256 = 128
    rng = np.random.default_rng(b)
    k = rng.integers(0, levels + 1, n)
    k[0], k[1] = 0, levels
    mn, mx = F(-3.0), F(3.0 + 6.0 * 0)  # range 6
    g = (mn + k.astype(F) * (F(mx - mn) / F(levels))).astype(F)
    g[0], g[1] = mn, mx
    u = np.full(n, 0.5, F)
    u[1] = 0.0  # the maximum sits on the top level exactly
    pay = oracle.compll_encode(g, u, b)
    np.testing.assert_array_equal(codes_of(pay, n, b), k)
    out = oracle.compll_decode(pay, 4 * n)
    count = (8 * pay.size - 80) // b - int(pay[1])
    assert out.size == count
    m = min(n, count)
    np.testing.assert_allclose(out[:m], g[:m], rtol=0, atol=float(mx - mn) * 2e-7 * levels)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 63, 1000])
def test_codes_against_float64_closed_form(b, n):
    rng = np.random.default_rng(100 * b + n)
    g = rng.normal(0, 1, n).astype(F)
    u = rng.random(n, dtype=F)
    pay = oracle.compll_encode(g, u, b)
    mn, mx = g.min(), g.max()
    levels = (1 << b) - 1
    codes = codes_of(pay, n, b)
    if mx == mn:
        assert not codes.any()
        return
    gap = F(mx - mn) / F(levels)
    exact = (g.astype(np.float64) - float(mn)) / float(gap) + u.astype(np.float64)
    lo, hi = np.floor(exact - 1e-4), np.floor(exact + 1e-4)  # float32 rounding may move r across an integer
    assert ((codes >= np.clip(lo, 0, levels)) & (codes <= np.clip(hi, 0, levels))).all()
    assert codes.max() <= levels
    # unused bits of the last byte are zero
    used = n * b
    if used % 8:
        assert pay[-1] >> (used % 8) == 0


def test_constant_tensor_has_zero_gap_and_zero_codes():
    pay = oracle.compll_encode(np.full(9, 0.5, F), np.full(9, 0.9, F), 2)
    assert not pay[10:].any()
    np.testing.assert_array_equal(oracle.compll_decode(pay, 64)[:9], np.full(9, 0.5, F))


def test_stochastic_rounding_is_unbiased():
    rng = np.random.default_rng(4)
    g = np.array([-1.0, -0.3, 0.1, 0.77, 1.0], dtype=F)
    acc = np.zeros(5)
    T = 20000
    for _ in range(T):
        pay = oracle.compll_encode(g, rng.random(5, dtype=F), 2)
        acc += codes_of(pay, 5, 2) * (2.0 / 3.0) - 1.0
    assert np.abs(acc / T - g).max() < 4 * (2.0 / 3.0) / np.sqrt(T)


def test_lcg_matches_reference_recurrence():
    # x <- 1103515245*x + 12345 (mod 2^32); value = float(x / (4294967295.0/(hi-lo))) + lo
    seed = 12345
    x = seed
    want = []
    for _ in range(6):
        x = (1103515245 * x + 12345) % (1 << 32)
        want.append(np.float32(x / (4294967295.0 / 1.0)) + np.float32(0.0))
    got = oracle.lcg_uniform(seed, 6)
    np.testing.assert_array_equal(got, np.array(want, dtype=F))
    # first step worked by hand: 1103515245*12345 + 12345 = 13622895711870 -> mod 2^32 = 3554416254
    assert (1103515245 * 12345 + 12345) % (1 << 32) == 3554416254
    assert got[0] == np.float32(3554416254 / 4294967295.0)
    assert got.min() >= 0.0 and got.max() <= 1.0
    lo_hi = oracle.lcg_uniform(7, 1000, -2.0, 3.0)
    assert lo_hi.min() >= -2.0 and lo_hi.max() <= 3.0
