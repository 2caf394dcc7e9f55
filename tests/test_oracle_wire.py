"""Pins the oracle's bit-placement helpers and the CompLL 10-byte-header decode
against what the reference's generated decode states
(/root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode_body.h:44,65-72)."""
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def ref_byte_rule(codes, b):
    """Byte image built straight from the reference's consumer-side rule:
    code i lives in byte floor(i*b/8) at shift (i mod 8/b)*b."""
    nbytes = (len(codes) * b + 7) // 8
    img = bytearray(nbytes)
    for i, c in enumerate(codes):
        img[i * b // 8] |= (c & ((1 << b) - 1)) << ((i % (8 // b)) * b)
    return bytes(img)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n", list(range(0, 70)) + [127, 128, 129, 130])
def test_put_code_matches_reference_byte_rule(b, n):
    rng = np.random.default_rng(1000 * b + n)
    codes = rng.integers(0, 1 << b, size=n)
    per = 32 // b
    words = np.zeros((n + per - 1) // per + 1, dtype=np.uint32)
    for i, c in enumerate(codes):
        oracle.put_code(words, i, b, int(c))
    img = words.view(np.uint8).tobytes()  # little-endian host
    want = ref_byte_rule(codes, b)
    assert img[: len(want)] == want
    assert all(x == 0 for x in img[len(want) :])
    for i, c in enumerate(codes):
        assert oracle.get_code(words, i, b) == c


def test_put_code_overwrites_only_its_field():
    words = np.full(2, 0xFFFFFFFF, dtype=np.uint32)
    oracle.put_code(words, 17, 2, 0)  # word 1, bits 2..3
    assert words[0] == 0xFFFFFFFF and words[1] == 0xFFFFFFF3


def test_compll_decode_reference_probe_vector():
    """Payload and the first decoded values are what the reference's generated
    decode produced for it (16-element ramp, bitwidth 2)."""
    with open(os.path.join(GOLDEN, "compll_decode_probe.json")) as f:
        fx = json.load(f)
    payload = np.array(fx["payload_bytes"], dtype=np.uint8)
    out = oracle.compll_decode(payload, 64)
    assert out.size == fx["count"]
    np.testing.assert_allclose(out[:4], fx["observed_first_values"], atol=5e-4)
    # the full vector from the stated formula q*gap+min, worked by hand per code
    want = np.array(fx["expected"], dtype=np.float32)
    np.testing.assert_array_equal(out, want)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
def test_compll_decode_formula(b):
    rng = np.random.default_rng(b)
    n = 64
    codes = rng.integers(0, 1 << b, size=n)
    mn, mx = np.float32(-0.75), np.float32(1.5)
    body = ref_byte_rule(codes, b)
    hdr = bytes([b, 0]) + mn.tobytes() + mx.tobytes()
    payload = np.frombuffer(hdr + body, dtype=np.uint8)
    out = oracle.compll_decode(payload, 1024)
    gap = np.float32(mx - mn) / np.float32((1 << b) - 1)
    want = codes.astype(np.float32) * gap + mn
    assert out.size == n
    np.testing.assert_array_equal(out, want.astype(np.float32))


def test_compll_decode_tail_shortens_output():
    codes = [1, 2, 3, 0, 1, 2, 3, 0]
    body = ref_byte_rule(codes, 2)
    hdr = bytes([2, 2]) + np.float32(0).tobytes() + np.float32(3).tobytes()
    out = oracle.compll_decode(np.frombuffer(hdr + body, dtype=np.uint8), 64)
    np.testing.assert_array_equal(out, np.array(codes[:6], dtype=np.float32))
