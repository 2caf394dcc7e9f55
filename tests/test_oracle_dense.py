"""Pins the oracle's TBQ, onebit and TernGrad functions with hand-worked known
answers, closed forms in an independent (vectorised numpy / float64)
formulation, invariants and special cases.  The reference holds no source or
fixture for these operators, so nothing here compares with reference output."""
import math

import numpy as np
import pytest

import oracle

F = np.float32


def unpack(words, n, b):
    """Independent unpacker: little-endian bit stream, b bits per code."""
    bits = np.unpackbits(np.ascontiguousarray(words).view(np.uint8), bitorder="little")
    bits = bits[: n * b].reshape(n, b)
    return (bits * (1 << np.arange(b))).sum(axis=1).astype(np.uint32)


# ---------------------------------------------------------------- TBQ
def test_tbq_hand_kat():
    g = np.array([0.06, -0.07, 0.01, 0.05, -0.05, 0.0499], dtype=F)
    pay, r = oracle.tbq_encode(g, np.zeros(6, F), 0.05)
    assert pay.size == 16 + 4
    assert pay[:4].view(F)[0] == F(0.05)
    assert pay[4:8].view(np.uint32)[0] == 6
    assert not pay[8:16].any()
    # codes + - 0 + - 0 -> 1 | 2<<2 | 0<<4 | 1<<6 | 2<<8 | 0<<10 = 0x249
    assert pay[16:20].view(np.uint32)[0] == 0x249
    tau = F(0.05)
    want_r = np.array([F(0.06) - tau, F(-0.07) + tau, F(0.01), F(0.0), F(0.0), F(0.0499)], dtype=F)
    np.testing.assert_array_equal(r, want_r)
    np.testing.assert_array_equal(
        oracle.tbq_decode(pay, 6), np.array([tau, -tau, 0, tau, -tau, 0], dtype=F)
    )


def test_tbq_residual_carries_to_next_step():
    g = np.array([0.03, -0.03, 0.02], dtype=F)
    p1, r1 = oracle.tbq_encode(g, np.zeros(3, F), 0.05)
    assert p1[16:20].view(np.uint32)[0] == 0  # nothing reaches 0.05 yet
    np.testing.assert_array_equal(r1, g)
    p2, r2 = oracle.tbq_encode(g, r1, 0.05)
    # 0.06 >= 0.05 -> +, -0.06 -> -, 0.04 -> 0
    assert p2[16:20].view(np.uint32)[0] == (1 | 2 << 2)
    v = g + g
    np.testing.assert_array_equal(r2, np.array([v[0] - F(0.05), v[1] + F(0.05), v[2]], dtype=F))


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 31, 33, 1000, 4099])
def test_tbq_closed_form_and_invariants(n):
    rng = np.random.default_rng(n)
    g = rng.normal(0, 0.02, n).astype(F)
    r0 = rng.normal(0, 0.03, n).astype(F)
    tau = F(0.05)
    pay, r = oracle.tbq_encode(g, r0, tau)
    assert pay.size == 16 + 4 * ((n + 15) // 16)
    words = pay[16:].view(np.uint32)
    codes = unpack(words, n, 2)
    v = r0 + g
    want = np.where(v >= tau, 1, np.where(v <= -tau, 2, 0))
    np.testing.assert_array_equal(codes, want)
    assert not (codes == 3).any()
    # pad codes are zero
    allc = unpack(words, words.size * 16, 2)
    assert not allc[n:].any()
    d = oracle.tbq_decode(pay, n)
    assert set(np.unique(d)).issubset({F(0), tau, -tau})
    np.testing.assert_array_equal(r, (v - d).astype(F))  # r' = v - d, one rounding
    # error feedback keeps what was not sent: small |v| leaves |r'| < tau
    small = np.abs(v) < 2 * tau
    assert (np.abs(r[small]) < tau).all()


def test_tbq_nan_and_code3():
    g = np.array([np.nan, 1.0], dtype=F)
    pay, r = oracle.tbq_encode(g, np.zeros(2, F), 0.5)
    assert pay[16:20].view(np.uint32)[0] == (0 | 1 << 2)
    assert np.isnan(r[0]) and r[1] == F(0.5)
    pay[16] = 0b1111  # codes 3,3 decode to zero
    np.testing.assert_array_equal(oracle.tbq_decode(pay, 2), np.zeros(2, F))


# ---------------------------------------------------------------- onebit
def test_onebit_hand_kat():
    g = np.array([1.0, -2.0, 3.0, -4.0], dtype=F)
    pay, r = oracle.onebit_encode(g, np.zeros(4, F))
    assert pay[:4].view(F)[0] == F(2.5)
    assert pay[4:8].view(np.uint32)[0] == 4
    assert pay[16:20].view(np.uint32)[0] == 0b0101
    np.testing.assert_array_equal(r, np.array([-1.5, 0.5, 0.5, -1.5], dtype=F))
    np.testing.assert_array_equal(oracle.onebit_decode(pay, 4), np.array([2.5, -2.5, 2.5, -2.5], dtype=F))


@pytest.mark.parametrize("n", [1, 31, 32, 33, 64, 1000, 100003])
def test_onebit_scale_bits_residual(n):
    rng = np.random.default_rng(n)
    g = rng.normal(0, 1e-3, n).astype(F)
    r0 = rng.normal(0, 1e-3, n).astype(F)
    v = r0 + g
    s_ref = math.fsum(np.abs(v).astype(np.float64)) / n
    s = oracle.onebit_scale(g, r0)
    assert abs(float(s) - s_ref) <= 1e-6 * s_ref
    pay, r = oracle.onebit_encode(g, r0)
    assert pay[:4].view(F)[0] == s
    assert pay.size == 16 + 4 * ((n + 31) // 32)
    words = pay[16:].view(np.uint32)
    bits = unpack(words, n, 1)
    np.testing.assert_array_equal(bits, (v >= 0).astype(np.uint32))
    assert not unpack(words, words.size * 32, 1)[n:].any()
    d = np.where(bits == 1, s, -s).astype(F)
    np.testing.assert_array_equal(r, (v - d).astype(F))
    np.testing.assert_array_equal(oracle.onebit_decode(pay, n), d)


def test_onebit_zero_tensor_and_empty():
    pay, r = oracle.onebit_encode(np.zeros(40, F), np.zeros(40, F))
    assert pay[:4].view(F)[0] == 0
    np.testing.assert_array_equal(pay[16:24].view(np.uint32), [0xFFFFFFFF, 0xFF])  # 0 >= 0
    assert not r.any()
    pay, r = oracle.onebit_encode(np.zeros(0, F), np.zeros(0, F))
    assert pay.size == 16 and pay[:4].view(F)[0] == 0


def test_onebit_given_scale_is_used_verbatim():
    g = np.array([0.5, -0.25], dtype=F)
    pay, r = oracle.onebit_encode(g, np.zeros(2, F), scale=0.125)
    assert pay[:4].view(F)[0] == F(0.125)
    np.testing.assert_array_equal(r, np.array([0.375, -0.125], dtype=F))


# ---------------------------------------------------------------- TernGrad
def test_terngrad_hand_kat():
    # bucket 4: scales 4 and 0.5
    g = np.array([1.0, -4.0, 2.0, 0.0, 0.5, -0.25, 0.1], dtype=F)
    u = np.array([0.2, 0.999, 0.5, 0.0, 0.5, 0.5, 0.25], dtype=F)
    # keep iff u*s < |g|: .8<1 y, 3.996<4 y, 2<2 n, 0<0 n | .25<.5 y, .25<.25 n, .125<.1 n
    pay = oracle.terngrad_encode(g, u, bucket=4)
    hdr = pay[:16].view(np.uint32)
    assert list(hdr) == [7, 4, 0, 0]
    np.testing.assert_array_equal(pay[16:32].view(F), np.array([4.0, 0.5, 0, 0], dtype=F))
    assert pay[32:36].view(np.uint32)[0] == (1 | 2 << 2 | 0 << 4 | 0 << 6 | 1 << 8)
    np.testing.assert_array_equal(
        oracle.terngrad_decode(pay, 7), np.array([4.0, -4.0, 0, 0, 0.5, 0, 0], dtype=F)
    )


@pytest.mark.parametrize("n,bucket", [(1, 512), (511, 512), (512, 512), (513, 512), (5000, 512), (777, 16), (4096, 256)])
def test_terngrad_invariants(n, bucket):
    rng = np.random.default_rng(n + bucket)
    g = rng.normal(0, 1e-3, n).astype(F)
    g[rng.random(n) < 0.01] *= 30
    u = rng.random(n, dtype=F)
    pay = oracle.terngrad_encode(g, u, bucket)
    nb = (n + bucket - 1) // bucket
    sb = (4 * nb + 15) // 16 * 16
    assert pay.size == 16 + sb + 4 * ((n + 15) // 16)
    scales = pay[16 : 16 + 4 * nb].view(F)
    pad = np.zeros(nb * bucket, F)
    pad[:n] = np.abs(g)
    np.testing.assert_array_equal(scales, pad.reshape(nb, bucket).max(axis=1))
    codes = unpack(pay[16 + sb :].view(np.uint32), n, 2)
    assert not (codes == 3).any()
    s = np.repeat(scales, bucket)[:n]
    keep = codes != 0
    assert ((u * s)[keep] < np.abs(g)[keep]).all()
    assert ((u * s)[~keep] >= np.abs(g)[~keep]).all()
    np.testing.assert_array_equal(codes[keep] == 2, g[keep] < 0)
    # the bucket maximum is always kept because u < 1
    for k in range(nb):
        seg = slice(k * bucket, min(n, (k + 1) * bucket))
        j = np.argmax(np.abs(g[seg]))
        if scales[k] > 0 and u[seg][j] * scales[k] < scales[k]:
            assert codes[seg][j] != 0
    d = oracle.terngrad_decode(pay, n)
    np.testing.assert_array_equal(d, np.where(codes == 1, s, np.where(codes == 2, -s, 0)).astype(F))


def test_terngrad_zero_bucket_and_unbiasedness():
    g = np.zeros(600, F)
    g[512:] = 0.25
    pay = oracle.terngrad_encode(g, np.zeros(600, F), 512)
    d = oracle.terngrad_decode(pay, 600)
    assert not d[:512].any()  # zero scale: u*0 < 0 is false
    np.testing.assert_array_equal(d[512:], g[512:])
    # E[decode] = g over many uniform draws
    rng = np.random.default_rng(7)
    g = rng.normal(0, 1, 64).astype(F)
    acc = np.zeros(64, np.float64)
    trials = 4000
    for _ in range(trials):
        acc += oracle.terngrad_decode(oracle.terngrad_encode(g, rng.random(64, dtype=F), 64), 64)
    s = np.abs(g).max()
    sigma = s / math.sqrt(trials)  # per-element std of the mean is at most s/sqrt(T)/2
    assert np.abs(acc / trials - g).max() < 4 * sigma
