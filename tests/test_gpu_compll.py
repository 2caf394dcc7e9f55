"""GPU parity of the in-tree CompLL operator (10-byte-header min/max quantiser)
against the oracle, and of its decoder against the payload the reference's own
generated decode was observed on (tests/golden/compll_decode_probe.json)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
F = np.float32
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    hipress_amd._lib.lib()
    return hipress_amd


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 7, 8, 9, 255, 4096, 4097, 70001, 1000003])
def test_encode_decode_match_oracle(hp, n, b):
    rng = np.random.default_rng(31 * n + b)
    g = rng.normal(0, 1e-2, n).astype(F)
    u = rng.random(n, dtype=F)
    nb = hp.compll_payload_bytes(n, b)
    assert nb == oracle.compll_payload_bytes(n, b)
    pay = torch.full((nb,), 0xAB, dtype=torch.uint8, device="cuda")
    hp.compll_terngrad_encode(dev(g), dev(u), pay, b)
    want = oracle.compll_encode(g, u, b)
    np.testing.assert_array_equal(host(pay), want)
    cap = n + 300
    out = torch.full((cap,), 7.0, device="cuda")
    hp.compll_terngrad_decode(pay, out)
    ref = oracle.compll_decode(want, cap)
    got = host(out)
    np.testing.assert_array_equal(got[: ref.size], ref)
    assert (got[ref.size :] == 7.0).all()  # nothing past the reference's element count is touched


def test_payload_needs_no_alignment(hp):
    n, b = 5001, 2
    rng = np.random.default_rng(3)
    g, u = rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F)
    buf = torch.zeros(hp.compll_payload_bytes(n, b) + 3, dtype=torch.uint8, device="cuda")
    pay = buf[3:]
    hp.compll_terngrad_encode(dev(g), dev(u), pay, b)
    want = oracle.compll_encode(g, u, b)
    np.testing.assert_array_equal(host(pay), want)
    out = torch.zeros(n + 64, device="cuda")
    hp.compll_terngrad_decode(pay, out)
    ref = oracle.compll_decode(want, n + 64)
    np.testing.assert_array_equal(host(out)[: ref.size], ref)


def test_decode_never_writes_past_the_callers_buffer(hp):
    # n mod 4 == 1 at bitwidth 2: the reference would write n + 2 elements into an n-element gradient
    n, b = 4097, 2
    rng = np.random.default_rng(5)
    want = oracle.compll_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), b)
    assert (8 * want.size - 80) // b - int(want[1]) == n + 2
    buf = torch.full((n + 8,), 7.0, device="cuda")
    hp.compll_terngrad_decode(dev(want), buf[:n])
    got = host(buf)
    np.testing.assert_array_equal(got[:n], oracle.compll_decode(want, n))
    assert (got[n:] == 7.0).all()


def test_decode_reference_probe_vector(hp):
    with open(os.path.join(GOLDEN, "compll_decode_probe.json")) as f:
        fx = json.load(f)
    pay = dev(np.array(fx["payload_bytes"], dtype=np.uint8))
    out = torch.full((64,), 7.0, device="cuda")
    hp.compll_terngrad_decode(pay, out)
    got = host(out)
    np.testing.assert_array_equal(got[: fx["count"]], np.array(fx["expected"], dtype=F))
    np.testing.assert_allclose(got[:4], fx["observed_first_values"], atol=5e-4)
    assert (got[fx["count"] :] == 7.0).all()


def test_constant_tensor_and_bad_bitwidth(hp):
    n = 1000
    pay = torch.full((hp.compll_payload_bytes(n, 4),), 0xAB, dtype=torch.uint8, device="cuda")
    g = np.full(n, 0.25, F)
    hp.compll_terngrad_encode(dev(g), torch.rand(n, device="cuda"), pay, 4)
    np.testing.assert_array_equal(host(pay), oracle.compll_encode(g, np.zeros(n, F), 4))
    with pytest.raises(hp._lib.HipressError):
        hp.compll_terngrad_encode(dev(g), torch.rand(n, device="cuda"), pay, 3)
    bad = pay.clone()
    bad[0] = 3  # a header with a bit width the format cannot carry decodes to nothing
    out = torch.full((n,), 7.0, device="cuda")
    hp.compll_terngrad_decode(bad, out)
    assert (host(out) == 7.0).all()


@pytest.mark.parametrize("b", [2, 4])
def test_reference_operator_name_is_the_in_tree_operator(hp, b):
    """TernGradEncode(gradient, compressed, bitwidth) under the reference's own name and
    argument order produces the in-tree format, byte for byte the oracle's payload."""
    n = 70001
    rng = np.random.default_rng(41 + b)
    g, u = rng.normal(0, 1e-2, n).astype(F), rng.random(n, dtype=F)
    want = oracle.compll_encode(g, u, b)
    pay = torch.zeros(want.size, dtype=torch.uint8, device="cuda")
    hp.TernGradEncode(dev(g), pay, b, uniform=dev(u))
    np.testing.assert_array_equal(host(pay), want)
    pay.zero_()
    torch.ops.hipress.TernGradEncode(dev(g), pay, b, dev(u))
    np.testing.assert_array_equal(host(pay), want)
    out = torch.zeros(n, device="cuda")
    torch.ops.hipress.TernGradDecode(pay, out)
    ref = oracle.compll_decode(want, n)
    np.testing.assert_array_equal(host(out)[: ref.size], ref)
    # without `uniform` the noise is drawn inside the operator, as in the reference: the header
    # (bit width, tail, min, max) is still the oracle's, the codes stay within one level of it
    pay2 = torch.zeros(want.size, dtype=torch.uint8, device="cuda")
    hp.TernGradEncode(dev(g), pay2, b)
    got = host(pay2)
    np.testing.assert_array_equal(got[:10], want[:10])
    lo, hi = oracle.compll_encode(g, np.zeros(n, F), b), oracle.compll_encode(g, np.full(n, np.nextafter(F(1), F(0)), F), b)
    per = 8 // b
    codes = lambda p: np.stack([(p[10:] >> (b * k)) & ((1 << b) - 1) for k in range(per)], 1).reshape(-1)[:n]
    assert (codes(got) >= codes(lo)).all() and (codes(got) <= codes(hi)).all()


@pytest.mark.parametrize("n,b", [(1000, 8), (4097 + 250, 8), (70015, 4), (4099, 2)])
def test_decode_leaves_the_remainder_as_the_caller_passed_it(hp, n, b):
    """The reference's count (8 * code bytes / b - tail) falls short of n when n mod 2^b != 0:
    out[count, n) keeps the caller's values and hipress_compll_decoded_count names the count."""
    rng = np.random.default_rng(n + b)
    want = oracle.compll_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), b)
    count = hp.compll_decoded_count(n, b)
    ref = oracle.compll_decode(want, n)
    assert count == ref.size and count < n
    out = torch.full((n,), 7.0, device="cuda")
    hp.compll_terngrad_decode(dev(want), out)
    got = host(out)
    np.testing.assert_array_equal(got[:count], ref)
    assert (got[count:] == 7.0).all()
