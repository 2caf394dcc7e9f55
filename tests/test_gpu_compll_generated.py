"""Operators generated from the shipped CompLL programs, on the GPU, against the CPU oracle
and the hand-written kernels.  MinMaxQuant is the in-tree operator of the reference
restated in the language, so its payload must equal the oracle's byte for byte given
the same uniform tensor; ThresholdTernary produces the code words of the TBQ operator
with a zero residual."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32
SIZES = [1, 3, 4, 5, 31, 1000, 4095, 4096, 4097, 12289, 262144, 1000003]


@pytest.fixture(scope="module")
def ops():
    from hipress_amd.compll import runtime

    assert torch.cuda.is_available()
    return runtime.load()  # fails loudly if the generated library is missing


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n", SIZES)
def test_minmax_quant_matches_the_oracle(ops, n, b):
    import hipress_amd as hp

    rng = np.random.default_rng(1000 * b + n)
    g = rng.normal(0, 1e-2, n).astype(F)
    u = rng.random(n, dtype=F)
    want = oracle.compll_encode(g, u, b)
    pay = torch.full((want.size + 5,), 0xAB, dtype=torch.uint8, device="cuda")
    ops.MinMaxQuantEncode(dev(g), pay[: want.size], b, uniform=dev(u))
    got = host(pay)
    np.testing.assert_array_equal(got[: want.size], want)
    assert (got[want.size:] == 0xAB).all(), "wrote past the payload"
    # the hand-written operator produces the same bytes
    pay2 = torch.zeros(hp.compll_payload_bytes(n, b), dtype=torch.uint8, device="cuda")
    hp.compll_terngrad_encode(dev(g), dev(u), pay2, b)
    np.testing.assert_array_equal(host(pay2), want)
    # without a noise tensor both draw the same values from the same seed
    seed = 31 * n + b
    ops.MinMaxQuantEncode(dev(g), pay2, b, seed=seed)
    np.testing.assert_array_equal(host(pay2), oracle.compll_encode(g, oracle.uniform_draws(seed, n), b))
    pay3 = torch.zeros_like(pay2)
    hp.compll_terngrad_encode_seeded(dev(g), pay3, b, seed)
    np.testing.assert_array_equal(host(pay3), host(pay2))
    # decode: as many elements as the payload says, bounded by the output
    ref = oracle.compll_decode(want, n + 8)
    out = torch.full((n + 8,), 7.0, device="cuda")
    ops.MinMaxQuantDecode(pay[: want.size], out)
    o = host(out)
    np.testing.assert_array_equal(o[: ref.size], ref)
    assert (o[ref.size:] == 7.0).all()
    short = torch.full((max(n - 2, 0),), 7.0, device="cuda")
    ops.MinMaxQuantDecode(pay[: want.size], short)
    k = min(short.numel(), ref.size)
    np.testing.assert_array_equal(host(short)[:k], ref[:k])
    assert (host(short)[k:] == 7.0).all()


def test_minmax_quant_constant_and_extreme_inputs(ops):
    n = 5000
    u = np.random.default_rng(3).random(n, dtype=F)
    for g in (np.full(n, 0.25, F), np.zeros(n, F), np.linspace(-2e5, 2e5, n).astype(F)):
        want = oracle.compll_encode(g, u, 2)
        pay = torch.zeros(want.size, dtype=torch.uint8, device="cuda")
        ops.MinMaxQuantEncode(dev(g), pay, 2, uniform=dev(u))
        np.testing.assert_array_equal(host(pay), want)


@pytest.mark.parametrize("n", SIZES)
def test_threshold_ternary_matches_tbq_codes(ops, n):
    rng = np.random.default_rng(n)
    t = F(0.05)
    g = rng.normal(0, 0.04, n).astype(F)
    g[:: 7] = t  # exactly on the threshold: taken
    g[3:: 11] = -t
    nbytes = 4 + (2 * n + 7) // 8
    pay = torch.full((nbytes + 3,), 0xAB, dtype=torch.uint8, device="cuda")
    ops.ThresholdTernaryEncode(dev(g), pay[:nbytes], float(t))
    got = host(pay)
    assert got[:4].view(F)[0] == t and (got[nbytes:] == 0xAB).all()
    tbq, _ = oracle.tbq_encode(g, np.zeros(n, F), t)  # 16-byte header, then the same code words
    np.testing.assert_array_equal(got[4:nbytes], tbq[16 : 16 + nbytes - 4])
    out = torch.full((n,), 7.0, device="cuda")
    ops.ThresholdTernaryDecode(pay[:nbytes], out)
    np.testing.assert_array_equal(host(out), oracle.tbq_decode(tbq, n))


@pytest.mark.parametrize("n", SIZES)
def test_threshold_feedback_matches_tbq_over_steps(ops, n):
    """Codes and the new residual come out of one fused sweep that updates the residual in
    place; three steps against the TBQ oracle, residual carried."""
    rng = np.random.default_rng(n + 99)
    t = F(0.05)
    r_ref = rng.normal(0, 0.02, n).astype(F)
    r_gpu = dev(r_ref)
    nbytes = 4 + (2 * n + 7) // 8
    for step in range(3):
        g = rng.normal(0, 0.03, n).astype(F)
        pay = torch.full((nbytes + 3,), 0xAB, dtype=torch.uint8, device="cuda")
        ops.ThresholdFeedbackEncode(dev(g), r_gpu, pay[:nbytes], float(t))
        tbq, r_ref = oracle.tbq_encode(g, r_ref, t)
        got = host(pay)
        assert got[:4].view(F)[0] == t and (got[nbytes:] == 0xAB).all()
        np.testing.assert_array_equal(got[4:nbytes], tbq[16 : 16 + nbytes - 4], err_msg=f"codes, step {step}")
        np.testing.assert_array_equal(host(r_gpu), r_ref, err_msg=f"residual, step {step}")


def test_threshold_feedback_rejects_a_short_residual(ops):
    from hipress_amd.compll.runtime import GeneratedOpError

    g = torch.zeros(1000, device="cuda")
    with pytest.raises(GeneratedOpError, match="too small"):
        ops.ThresholdFeedbackEncode(g, torch.zeros(999, device="cuda"), torch.zeros(400, dtype=torch.uint8, device="cuda"), 0.05)


@pytest.mark.parametrize("n", [1, 100, 4096, 4097, 1000003])
def test_mean_and_spread(ops, n):
    g = np.random.default_rng(n).normal(0.5, 1.0, n).astype(F)
    pay = torch.zeros(8, dtype=torch.uint8, device="cuda")
    ops.MeanAndSpread(dev(g), pay)
    mean, spread = host(pay).view(F)
    assert abs(float(mean) - float(g.astype(np.float64).mean())) <= 1e-5 * max(1.0, abs(float(g.mean())))  # a sum: order differs
    assert spread == F(g.max()) - F(g.min())  # max and min are exact


@pytest.mark.parametrize("n", SIZES)
def test_sign_mean_matches_onebit_without_residual(ops, n):
    """The magnitudes are a mapped vector that is only folded (never stored); the sign bits
    are the onebit operator's with a zero residual, the scale its mean magnitude."""
    g = np.random.default_rng(n + 7).normal(0, 1e-2, n).astype(F)
    g[:: 13] = 0.0  # zero counts as not negative
    nbytes = 4 + (n + 7) // 8
    pay = torch.full((nbytes + 3,), 0xAB, dtype=torch.uint8, device="cuda")
    ops.SignMeanEncode(dev(g), pay[:nbytes])
    got = host(pay)
    assert (got[nbytes:] == 0xAB).all()
    scale = got[:4].view(F)[0]
    want_scale = oracle.onebit_scale(g, np.zeros(n, F))
    assert abs(float(scale) - float(want_scale)) <= 1e-5 * float(want_scale)
    onebit, _ = oracle.onebit_encode(g, np.zeros(n, F), scale=scale)
    np.testing.assert_array_equal(got[4:nbytes], onebit[16 : 16 + nbytes - 4])
    out = torch.full((n,), 7.0, device="cuda")
    ops.SignMeanDecode(pay[:nbytes], out)
    np.testing.assert_array_equal(host(out), oracle.onebit_decode(onebit, n))


def test_generated_ops_on_empty_and_truncated_inputs(ops):
    empty = torch.zeros(0, device="cuda")
    # no element: the header is still written, nothing else
    pay = torch.full((12,), 0xAB, dtype=torch.uint8, device="cuda")
    ops.MinMaxQuantEncode(empty, pay[:10], 2, uniform=empty)
    got = host(pay)
    want = oracle.compll_encode(np.zeros(0, F), np.zeros(0, F), 2)
    np.testing.assert_array_equal(got[:10], want)
    assert (got[10:] == 0xAB).all()
    pay = torch.full((8,), 0xAB, dtype=torch.uint8, device="cuda")
    ops.ThresholdTernaryEncode(empty, pay[:4], 0.25)
    assert host(pay)[:4].view(F)[0] == F(0.25) and (host(pay)[4:] == 0xAB).all()
    ops.SignMeanEncode(empty, pay[:4])  # the mean of nothing: 0 / 0
    assert np.isnan(host(pay)[:4].view(F)[0])
    # a payload cut off inside its header decodes to nothing
    out = torch.full((16,), 7.0, device="cuda")
    ops.MinMaxQuantDecode(torch.tensor([2, 0, 0, 0, 0], dtype=torch.uint8, device="cuda"), out)
    assert (host(out) == 7.0).all()
    ops.MinMaxQuantDecode(pay[:0], out)
    assert (host(out) == 7.0).all()


def test_generated_ops_report_errors(ops):
    from hipress_amd.compll.runtime import GeneratedOpError

    g = torch.zeros(100, device="cuda")
    u = torch.zeros(100, device="cuda")
    with pytest.raises(GeneratedOpError, match="too small"):
        ops.MinMaxQuantEncode(g, torch.zeros(20, dtype=torch.uint8, device="cuda"), 2, uniform=u)
    with pytest.raises(GeneratedOpError, match="bad parameter"):
        ops.MinMaxQuantEncode(g, torch.zeros(200, dtype=torch.uint8, device="cuda"), 3, uniform=u)
    with pytest.raises(TypeError):
        ops.MinMaxQuantEncode(g, torch.zeros(200, dtype=torch.uint8, device="cuda"), 2, uniform=u.cpu())  # noise not on the GPU
    ops.MinMaxQuantEncode(g, torch.zeros(200, dtype=torch.uint8, device="cuda"), 2)  # no noise tensor: drawn in the kernel
    with pytest.raises(TypeError):
        ops.MinMaxQuantEncode(g.double(), torch.zeros(200, dtype=torch.uint8, device="cuda"), 2, uniform=u)
    # a payload whose header names an impossible width decodes to nothing
    bad = torch.zeros(64, dtype=torch.uint8, device="cuda")
    bad[0] = 3
    out = torch.full((50,), 7.0, device="cuda")
    ops.MinMaxQuantDecode(bad, out)
    assert (host(out) == 7.0).all()


# ---------------------------------------------------------------- the reference's own programs
@pytest.fixture(scope="module")
def reference_ops():
    """The operators compiled from the reference checkout's own two programs, unmodified
    (built on the machine that holds the checkout; the library travels, the checkout does not)."""
    import os

    from hipress_amd.compll import runtime
    from hipress_amd.compll.build import REFERENCE_LIB

    if not os.path.exists(REFERENCE_LIB):
        pytest.skip("the reference checkout's programs were not built on this tree")
    return runtime.Operators(REFERENCE_LIB)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n", [1, 5, 4097, 262144, 1000003])
def test_the_reference_s_own_programs_match_the_oracle(reference_ops, n, b):
    """TernGradEncode(gradient, compressed, bitwidth) / TernGradDecode(compressed, gradient) as
    the reference's generator registers them, generated here from its own program text: payload
    byte for byte against the oracle (which follows the same program), decode value for value."""
    import hipress_amd as hp

    rng = np.random.default_rng(77 * b + n)
    g = rng.normal(0, 1e-3, n).astype(F)
    u = rng.random(n, dtype=F)
    want = oracle.compll_encode(g, u, b)
    pay = torch.full((want.size,), 0xAB, dtype=torch.uint8, device="cuda")
    reference_ops.TernGradEncode(dev(g), pay, b, uniform=dev(u))
    np.testing.assert_array_equal(host(pay), want)
    out = torch.full((n,), 7.0, device="cuda")
    reference_ops.TernGradDecode(pay, out)
    dec = oracle.compll_decode(want, n)
    k = hp.compll_decoded_count(n, b)
    assert dec.size == k
    np.testing.assert_array_equal(host(out)[:k], dec)
    assert (host(out)[k:] == 7.0).all()
    # with the reference's own argument list - no noise tensor - the kernels draw from the seed
    seed = 1000 * n + b
    pay.fill_(0xAB)
    reference_ops.TernGradEncode(dev(g), pay, b, seed=seed)
    np.testing.assert_array_equal(host(pay), oracle.compll_encode(g, oracle.uniform_draws(seed, n), b))
