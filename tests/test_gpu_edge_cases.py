"""GPU parity on the inputs a gradient set does not normally hold: NaN, +-Inf, +-0,
denormals and FLT_MAX mixed into ordinary data, buckets whose elements are all equal,
pointers that are only 4-byte aligned (16-byte vector accesses at dword addresses), and empty tensors -
each compressor and both merges against the CPU oracle, through the C ABI.

Floats are compared value for value with NaN equal to NaN (the bits of a NaN that an
addition produces are the processor's choice); packed codes, indices and counts are
compared bit for bit."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32
FLT_MAX = np.finfo(F).max
FLT_MIN = np.finfo(F).tiny
SPECIALS = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, -3e-42, 1.4e-45, FLT_MAX, -FLT_MAX, FLT_MIN, -FLT_MIN], F)
FINITE_SPECIALS = SPECIALS[3:]


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def payload(nbytes):
    return torch.full((nbytes,), 0xAB, dtype=torch.uint8, device="cuda")


def feq(got, want, msg=""):
    """Equal as floats, NaN matching NaN, and the sign of zero respected."""
    got, want = np.asarray(got), np.asarray(want)
    np.testing.assert_array_equal(got, want, err_msg=msg)
    z = (want == 0)
    np.testing.assert_array_equal(np.signbit(got[z]), np.signbit(want[z]), err_msg=msg + " (sign of zero)")


def sprinkle(rng, n, sigma, specials, every=97):
    """Ordinary N(0, sigma) data with the special values at scattered places, among them
    the first and last element, tile borders and the 64-element group borders."""
    g = rng.normal(0, sigma, n).astype(F)
    places = list(range(5, n, every)) + [0, n - 1, 63, 64, 4095, 4096, 4097]
    for k, p in enumerate(p for p in places if 0 <= p < n):
        g[p] = specials[k % len(specials)]
    return g


def check_sparse(got_pay, want_pay, msg=""):
    g, w = oracle.sparse_unpack(got_pay), oracle.sparse_unpack(want_pay)
    assert g[:3] == w[:3], (msg, g[:3], w[:3])
    assert g[3].view(np.uint32) == w[3].view(np.uint32), (msg, g[3], w[3])
    np.testing.assert_array_equal(g[4], w[4], err_msg=msg + " indices")
    feq(g[5], w[5], msg + " values")


# ================================================================ special values
@pytest.mark.parametrize("n", [4099, 70001])
def test_tbq_special_values(hp, n):
    rng = np.random.default_rng(n)
    r_ref = sprinkle(rng, n, 0.02, SPECIALS, every=89)
    r = dev(r_ref)
    for step in range(3):
        g = sprinkle(rng, n, 0.02, np.roll(SPECIALS, step), every=97)
        pay = payload(hp.tbq_payload_bytes(n))
        hp.tbq_encode(dev(g), r, pay, 0.05)
        want, r_ref = oracle.tbq_encode(g, r_ref, 0.05)
        np.testing.assert_array_equal(host(pay), want, err_msg=f"step {step}")
        feq(host(r), r_ref, f"residual step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.tbq_decode(pay, out)
        feq(host(out), oracle.tbq_decode(want, n))


@pytest.mark.parametrize("kind", ["finite", "inf", "nan"])
def test_onebit_special_values(hp, kind):
    """finite specials leave a finite scale (within 1e-5 of the oracle's); an infinity makes it
    +Inf and a NaN makes it NaN on both sides; with the GPU's scale handed to the oracle the
    bits and the residual agree everywhere."""
    n = 70001
    rng = np.random.default_rng(7)
    specials = {"finite": FINITE_SPECIALS[FINITE_SPECIALS != -FLT_MAX], "inf": SPECIALS[1:], "nan": SPECIALS}[kind]
    g = sprinkle(rng, n, 1e-3, specials, every=4001 if kind == "finite" else 97)
    if kind == "finite":
        g[np.abs(g) == FLT_MAX] = 0.0
        g[12345] = FLT_MAX  # a single one: the sum stays finite in any order
    r_ref = rng.normal(0, 1e-3, n).astype(F)
    r = dev(r_ref)
    pay = payload(hp.onebit_payload_bytes(n))
    hp.onebit_encode(dev(g), r, pay)
    got = host(pay)
    s = got[:4].view(F)[0]
    s_ref = oracle.onebit_scale(g, r_ref)
    if kind == "finite":
        assert np.isfinite(s) and abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref)
    elif kind == "inf":
        assert s == np.inf and s_ref == np.inf
    else:
        assert np.isnan(s) and np.isnan(s_ref)
    want, r_next = oracle.onebit_encode(g, r_ref, scale=s)
    np.testing.assert_array_equal(got[4:], want[4:])  # n, the zero words, every sign bit
    feq(host(r), r_next, "residual")
    out = torch.full((n,), 7.0, device="cuda")
    hp.onebit_decode(pay, out)
    feq(host(out), oracle.onebit_decode(got, n))


@pytest.mark.parametrize("bucket", [512, 100])
def test_terngrad_special_values_and_all_equal_buckets(hp, bucket):
    n = 70001
    rng = np.random.default_rng(bucket)
    g = sprinkle(rng, n, 1e-3, SPECIALS, every=211)
    g[2048:2048 + 512] = 0.25            # a bucket whose elements are all equal: every one is kept (u < 1)
    g[4096:4096 + 1024] = -0.0           # two buckets of negative zeros: scale 0, all codes 0
    g[8192:8192 + 512] = -1e-40          # equal denormals
    u = rng.random(n, dtype=F)
    u[::5] = 0.0
    u[1::7] = np.nextafter(F(1), F(0))
    pay = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode(dev(g), dev(u), pay, bucket)
    want = oracle.terngrad_encode(g, u, bucket)
    got = host(pay)
    nb = (n + bucket - 1) // bucket
    feq(got[16:16 + 4 * nb].view(F), want[16:16 + 4 * nb].view(F), "scales")
    np.testing.assert_array_equal(got[:16], want[:16])
    off = oracle.terngrad_scale_bytes(n, bucket) + 16
    np.testing.assert_array_equal(got[off:], want[off:], err_msg="codes")
    out = torch.full((n,), 7.0, device="cuda")
    hp.terngrad_decode(pay, out)
    feq(host(out), oracle.terngrad_decode(want, n), "decode")
    if bucket == 512:
        assert (host(out)[2048:2048 + 512] == F(0.25)).all()


@pytest.mark.parametrize("alg", ["dgc", "graddrop"])
@pytest.mark.parametrize("n", [4099, 300007])
def test_sparse_special_values(hp, alg, n):
    """NaN orders above infinity in the |x| keys, so NaN and +-Inf are always selected (and
    zeroed in the state); denormals and zeros of either sign ride along in the state."""
    rng = np.random.default_rng(n)
    ratio, m = 0.01, 0.9
    mom_ref, acc_ref = np.zeros(n, F), np.zeros(n, F)
    mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    for step in range(3):
        g = sprinkle(rng, n, 1e-3, np.roll(SPECIALS, 2 * step), every=1009 if n > 100000 else 401)
        pay = payload(hp.sparse_payload_bytes(n, ratio))
        if alg == "dgc":
            hp.dgc_encode(dev(g), mom, acc, pay, m, ratio)
            want, mom_ref, acc_ref = oracle.dgc_encode(g, mom_ref, acc_ref, m, ratio)
            feq(host(mom), mom_ref, f"momentum step {step}")
        else:
            hp.graddrop_encode(dev(g), acc, pay, ratio)
            want, acc_ref = oracle.graddrop_encode(g, acc_ref, ratio)
        check_sparse(host(pay), want, f"step {step}")
        feq(host(acc), acc_ref, f"accumulator step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.dgc_decode(pay, out)
        feq(host(out), oracle.sparse_decode(want, n), "decode")


def _special_tbq_payloads(rng, n, taus):
    """TBQ payloads with chosen header scales and random codes, the unused code 3 among them."""
    pays = []
    for tau in taus:
        codes = rng.integers(0, 4, n).astype(np.uint32)
        words = np.zeros((n + 15) // 16, np.uint32)
        for k in range(16):
            part = codes[k::16]
            words[: part.size] |= part << (2 * k)
        hdr = np.zeros(4, np.uint32)
        hdr[0] = np.array([tau], F).view(np.uint32)[0]
        hdr[1] = n
        pays.append(np.concatenate([hdr, words]).view(np.uint8).copy())
    return pays


def test_tbq_decode_merge_special_scales(hp):
    n = 12289
    rng = np.random.default_rng(3)
    taus = [0.05, np.inf, 1e-40, FLT_MAX, FLT_MAX, -0.0, np.nan, 0.05]
    for P in (5, 8):  # without and with the NaN peer
        pays = _special_tbq_payloads(rng, n, taus[:P])
        r0 = sprinkle(rng, n, 0.02, SPECIALS, every=301)
        agg, res = torch.full((n,), 7.0, device="cuda"), dev(r0)
        outp = payload(hp.tbq_payload_bytes(n))
        hp.tbq_decode_merge([dev(p) for p in pays], agg, res, outp, 0.05)
        want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, r0, 0.05)
        feq(host(agg), want_agg, f"aggregate P={P}")
        np.testing.assert_array_equal(host(outp), want_out)
        feq(host(res), want_r, f"residual P={P}")


def test_onebit_and_terngrad_decode_merge_special_scales(hp):
    n = 12289
    rng = np.random.default_rng(4)
    ob = []
    for s in (1e-3, np.inf, 1e-40, FLT_MAX, np.nan):
        g = rng.normal(0, 1, n).astype(F)
        p, _ = oracle.onebit_encode(g, np.zeros(n, F), scale=F(s))
        ob.append(p)
    for P in (4, 5):
        agg = torch.full((n,), 7.0, device="cuda")
        hp.onebit_decode_merge([dev(p) for p in ob[:P]], agg)
        feq(host(agg), oracle.onebit_decode_merge(ob[:P], n), f"onebit P={P}")
    tg = [oracle.terngrad_encode(sprinkle(rng, n, 1e-3, SPECIALS, every=97 + 10 * k), rng.random(n, dtype=F), 512)
          for k in range(4)]
    agg = torch.full((n,), 7.0, device="cuda")
    hp.terngrad_decode_merge([dev(p) for p in tg], agg)
    feq(host(agg), oracle.terngrad_decode_merge(tg, n), "terngrad")


@pytest.mark.parametrize("n", [4099, 300007])
def test_sparse_decode_merge_special_values(hp, n):
    """Peers whose pairs carry NaN, infinities of both signs at the same index (their sum is
    NaN), FLT_MAX twice (the sum overflows), denormals and signed zeros; merged in peer order
    and re-encoded."""
    rng = np.random.default_rng(n + 1)
    ratio, P = 0.01, 4
    pays = []
    for p in range(P):
        g = sprinkle(rng, n, 1e-3, np.roll(SPECIALS, p), every=257)
        g[100] = [np.inf, -np.inf, 1.0, np.nan][p]
        g[200] = [FLT_MAX, FLT_MAX, -1.0, 0.5][p]
        g[300] = [1e-40, 2e-40, -3e-40, 1e-3][p]
        pay, _ = oracle.graddrop_encode(g, np.zeros(n, F), ratio)
        pays.append(pay)
    acc0 = rng.normal(0, 1e-3, n).astype(F)
    agg, acc = torch.full((n,), 7.0, device="cuda"), dev(acc0)
    outp = payload(hp.sparse_payload_bytes(n, ratio))
    hp.dgc_decode_merge([dev(p) for p in pays], agg, acc, outp, ratio)
    want_agg, want_out, want_acc = oracle.sparse_decode_merge(pays, n, acc0, ratio)
    feq(host(agg), want_agg, "aggregate")
    check_sparse(host(outp), want_out, "re-encoded payload")
    feq(host(acc), want_acc, "accumulator")
    # without the re-encode
    agg2 = torch.full((n,), 7.0, device="cuda")
    hp.dgc_decode_merge([dev(p) for p in pays], agg2)
    feq(host(agg2), oracle.sparse_decode_merge(pays, n), "aggregate alone")


@pytest.mark.parametrize("b", [1, 2, 4, 8])
def test_compll_special_values(hp, b):
    """NaN never wins the min/max folds; an infinity makes the gap infinite and every code 0;
    whatever does not convert (NaN) is code 0."""
    n = 70001
    rng = np.random.default_rng(b)
    for specials in (FINITE_SPECIALS[np.abs(FINITE_SPECIALS) < 1], SPECIALS[:1], SPECIALS):
        g = sprinkle(rng, n, 1e-2, specials, every=503)
        u = rng.random(n, dtype=F)
        pay = payload(hp.compll_payload_bytes(n, b))
        hp.compll_terngrad_encode(dev(g), dev(u), pay, b)
        want = oracle.compll_encode(g, u, b)
        got = host(pay)
        np.testing.assert_array_equal(got[:2], want[:2])
        feq(got[2:10].view(F), want[2:10].view(F), "min / max")
        np.testing.assert_array_equal(got[10:], want[10:], err_msg="codes")
        out = torch.full((n,), 7.0, device="cuda")
        hp.compll_terngrad_decode(pay, out)
        ref = oracle.compll_decode(want, n)
        feq(host(out)[: ref.size], ref, "decode")


# ================================================================ 4-byte-aligned pointers
def views(n, *arrays, offsets=(1, 3, 2, 1, 3)):
    """Device copies of `arrays` that start `offsets[k]` floats into their allocations, so
    that no base address is 16-byte aligned; returns (views, backing buffers)."""
    vs, bufs = [], []
    for k, a in enumerate(arrays):
        off = offsets[k % len(offsets)]
        buf = torch.full((n + 8,), -99.0, device="cuda")
        v = buf[off: off + n]
        assert v.data_ptr() % 16 != 0 and v.data_ptr() % 4 == 0
        if a is not None:
            v.copy_(dev(a))
        vs.append(v)
        bufs.append((buf, off))
    return vs, bufs


def untouched_outside(bufs, n):
    for buf, off in bufs:
        b = host(buf)
        assert (b[:off] == -99.0).all() and (b[off + n:] == -99.0).all(), "wrote outside the view"


def _deferred_steps_against_two_pass_oracle(hp, n, grads, r0, state, sstate, res, check_scale):
    """Runs the deferred-residual onebit pair (hipress_onebit_encode_deferred +
    hipress_onebit_residual, per-tensor entry points) over consecutive steps and holds every
    payload and every materialised residual against the two-pass oracle, which is given the
    GPU's scale of that step."""
    r_ref = r0
    for step, g in enumerate(grads):
        pay = payload(hp.onebit_payload_bytes(n))
        hp.onebit_encode_deferred(g[0], state, sstate, pay)
        got = host(pay)
        s = got[:4].view(F)[0]
        check_scale(step, s, oracle.onebit_scale(g[1], r_ref))
        want, r_ref = oracle.onebit_encode(g[1], r_ref, scale=s)
        np.testing.assert_array_equal(got[4:], want[4:], err_msg=f"payload step {step}")
        assert host(sstate).view(np.uint32)[0] == got[:4].view(np.uint32)[0]
        hp.onebit_residual(state, sstate, res)
        feq(host(res), r_ref, f"residual step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.onebit_decode(pay, out)
        feq(host(out), oracle.onebit_decode(got, n), f"decode step {step}")


@pytest.mark.parametrize("kind", ["finite", "inf", "nan"])
def test_onebit_deferred_special_values_three_steps(hp, kind):
    """The one-pass variant on NaN, infinities, signed zeros, denormals and FLT_MAX: what it
    defers (r = v - d of the step before, formed on the fly) must come out as the two-pass
    operator stores it, also once the scale is infinite or no number."""
    n = 70001
    rng = np.random.default_rng(11)
    specials = {"finite": FINITE_SPECIALS[FINITE_SPECIALS != -FLT_MAX], "inf": SPECIALS[1:], "nan": SPECIALS}[kind]
    grads = []
    for step in range(3):
        g = sprinkle(rng, n, 1e-3, np.roll(specials, step), every=4001 if kind == "finite" else 97)
        if kind == "finite":
            g[np.abs(g) == FLT_MAX] = 0.0
            if step == 2:
                # a single one, in the last step: the sum stays finite in any order.  (Earlier, the
                # scale of FLT_MAX / n it causes would put every residual near 5e33 and the next
                # step's per-tile fp32 sums beyond FLT_MAX, where the oracle's float64 sum is finite.)
                g[12345] = FLT_MAX
        grads.append((dev(g), g))
    r0 = rng.normal(0, 1e-3, n).astype(F)

    def check_scale(step, s, s_ref):
        if kind == "finite":
            assert np.isfinite(s) and abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref), (step, s, s_ref)
        elif kind == "inf" and step == 0:
            assert s == np.inf and s_ref == np.inf
        else:  # a NaN input, or inf - inf from the step before: no number on both sides
            assert np.isnan(s) == np.isnan(s_ref) and (np.isnan(s) or s == s_ref), (step, s, s_ref)

    _deferred_steps_against_two_pass_oracle(hp, n, grads, r0, dev(r0), torch.zeros(1, device="cuda"),
                                            torch.empty(n, device="cuda"), check_scale)


@pytest.mark.parametrize("n", [9001, 70003])
def test_onebit_deferred_unaligned_views_three_steps(hp, n):
    """Gradient, state and residual output only 4-byte aligned (16-byte accesses at dword
    addresses in the one-pass kernel and in hipress_onebit_residual), three steps with the
    state carried."""
    rng = np.random.default_rng(n + 1)
    r0 = rng.normal(0, 1e-3, n).astype(F)
    gs = [rng.normal(0, 1e-3, n).astype(F) for _ in range(3)]
    (g0, g1, g2, sv, resv), bufs = views(n, gs[0], gs[1], gs[2], r0, None)

    def check_scale(step, s, s_ref):
        assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref), (step, s, s_ref)

    _deferred_steps_against_two_pass_oracle(hp, n, list(zip((g0, g1, g2), gs)), r0, sv, torch.zeros(1, device="cuda"), resv,
                                            check_scale)
    untouched_outside(bufs, n)


@pytest.mark.parametrize("n", [9001, 70003])
def test_onebit_unaligned_views(hp, n):
    rng = np.random.default_rng(n)
    g, r0 = rng.normal(0, 1e-3, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
    (gv, rv, ov), bufs = views(n, g, r0, None)
    pay = payload(hp.onebit_payload_bytes(n))
    hp.onebit_encode(gv, rv, pay)
    got = host(pay)
    s = got[:4].view(F)[0]
    assert abs(float(s) - float(oracle.onebit_scale(g, r0))) <= 1e-5 * float(s)
    want, want_r = oracle.onebit_encode(g, r0, scale=s)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(host(rv), want_r)
    hp.onebit_decode(pay, ov)
    np.testing.assert_array_equal(host(ov), oracle.onebit_decode(want, n))
    untouched_outside(bufs, n)
    # the deferred variant on the same views
    (gv, sv, resv), bufs = views(n, g, r0, None)
    sstate = torch.zeros(1, device="cuda")
    pay2 = payload(hp.onebit_payload_bytes(n))
    hp.onebit_encode_deferred(gv, sv, sstate, pay2)
    np.testing.assert_array_equal(host(pay2), got)
    hp.onebit_residual(sv, sstate, resv)
    np.testing.assert_array_equal(host(resv), want_r)
    untouched_outside(bufs, n)


@pytest.mark.parametrize("bucket", [512, 100])
def test_terngrad_unaligned_views(hp, bucket):
    n = 70003
    rng = np.random.default_rng(bucket)
    g, u = rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F)
    (gv, uv, ov), bufs = views(n, g, u, None)
    pay = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode(gv, uv, pay, bucket)
    want = oracle.terngrad_encode(g, u, bucket)
    np.testing.assert_array_equal(host(pay), want)
    hp.terngrad_decode(pay, ov)
    np.testing.assert_array_equal(host(ov), oracle.terngrad_decode(want, n))
    untouched_outside(bufs, n)


@pytest.mark.parametrize("alg,ratio", [("dgc", 0.001), ("graddrop", 0.01)])
@pytest.mark.parametrize("n", [9001, 300007])
def test_sparse_unaligned_views(hp, alg, ratio, n):
    rng = np.random.default_rng(n)
    (gv, mv, av, ov), bufs = views(n, None, np.zeros(n, F), np.zeros(n, F), None)
    mom_ref, acc_ref = np.zeros(n, F), np.zeros(n, F)
    for step in range(3):
        g = rng.normal(0, 1e-3, n).astype(F)
        gv.copy_(dev(g))
        pay = payload(hp.sparse_payload_bytes(n, ratio))
        if alg == "dgc":
            hp.dgc_encode(gv, mv, av, pay, 0.9, ratio)
            want, mom_ref, acc_ref = oracle.dgc_encode(g, mom_ref, acc_ref, 0.9, ratio)
            np.testing.assert_array_equal(host(mv), mom_ref, err_msg=f"momentum step {step}")
        else:
            hp.graddrop_encode(gv, av, pay, ratio)
            want, acc_ref = oracle.graddrop_encode(g, acc_ref, ratio)
        check_sparse(host(pay), want, f"step {step}")
        np.testing.assert_array_equal(host(av), acc_ref, err_msg=f"accumulator step {step}")
        hp.dgc_decode(pay, ov)
        np.testing.assert_array_equal(host(ov), oracle.sparse_decode(want, n))
    untouched_outside(bufs, n)


@pytest.mark.parametrize("n", [9001, 300007])
def test_sparse_overflow_path_unaligned(hp, n):
    """More candidates than slots on views that are only 4-byte aligned: the exact
    re-threshold and the rationed ties run through the element-wise loads."""
    g = np.full(n, 0.5, F)
    g[::3] = -0.5
    (gv, av), bufs = views(n, g, np.zeros(n, F))
    pay = payload(hp.graddrop_payload_bytes(n, 0.001))
    hp.graddrop_encode(gv, av, pay, 0.001)
    want, want_acc = oracle.graddrop_encode(g, np.zeros(n, F), 0.001)
    check_sparse(host(pay), want)
    np.testing.assert_array_equal(host(av), want_acc)
    untouched_outside(bufs, n)


@pytest.mark.parametrize("n", [9001, 1048576 + 5])
def test_dense_merges_unaligned_views(hp, n):
    rng = np.random.default_rng(n)
    P, tau = 8, 0.05
    z = np.zeros(n, F)
    pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), z, tau)[0] for _ in range(P)]
    r0 = rng.normal(0, 0.02, n).astype(F)
    (aggv, resv), bufs = views(n, None, r0)
    outp = payload(hp.tbq_payload_bytes(n))
    hp.tbq_decode_merge([dev(p) for p in pays], aggv, resv, outp, tau)
    want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, r0, tau)
    np.testing.assert_array_equal(host(aggv), want_agg)
    np.testing.assert_array_equal(host(outp), want_out)
    np.testing.assert_array_equal(host(resv), want_r)
    untouched_outside(bufs, n)
    # payload only: no aggregate buffer
    (resv2,), bufs = views(n, r0)
    outp2 = payload(hp.tbq_payload_bytes(n))
    hp.tbq_decode_merge([dev(p) for p in pays], None, resv2, outp2, tau)
    np.testing.assert_array_equal(host(outp2), want_out)
    np.testing.assert_array_equal(host(resv2), want_r)
    untouched_outside(bufs, n)
    ob = [oracle.onebit_encode(rng.normal(0, 0.04, n).astype(F), z)[0] for _ in range(3)]
    (aggv,), bufs = views(n, None)
    hp.onebit_decode_merge([dev(p) for p in ob], aggv)
    np.testing.assert_array_equal(host(aggv), oracle.onebit_decode_merge(ob, n))
    untouched_outside(bufs, n)
    tg = [oracle.terngrad_encode(rng.normal(0, 0.04, n).astype(F), rng.random(n, dtype=F), 512) for _ in range(3)]
    (aggv,), bufs = views(n, None)
    hp.terngrad_decode_merge([dev(p) for p in tg], aggv)
    np.testing.assert_array_equal(host(aggv), oracle.terngrad_decode_merge(tg, n))
    untouched_outside(bufs, n)


@pytest.mark.parametrize("n", [9001, 1048576 + 5])
def test_sparse_merge_unaligned_views(hp, n):
    rng = np.random.default_rng(n + 2)
    P, ratio = 8, 0.001
    z = np.zeros(n, F)
    pays = [oracle.dgc_encode(rng.normal(0, 1e-3, n).astype(F), z, z, 0.9, ratio)[0] for _ in range(P)]
    acc0 = rng.normal(0, 1e-4, n).astype(F)
    (aggv, accv), bufs = views(n, None, acc0)
    outp = payload(hp.sparse_payload_bytes(n, ratio))
    hp.dgc_decode_merge([dev(p) for p in pays], aggv, accv, outp, ratio)
    want_agg, want_out, want_acc = oracle.sparse_decode_merge(pays, n, acc0, ratio)
    np.testing.assert_array_equal(host(aggv), want_agg)
    check_sparse(host(outp), want_out)
    np.testing.assert_array_equal(host(accv), want_acc)
    untouched_outside(bufs, n)
    (aggv,), bufs = views(n, None)
    hp.dgc_decode_merge([dev(p) for p in pays], aggv)
    np.testing.assert_array_equal(host(aggv), oracle.sparse_decode_merge(pays, n))
    untouched_outside(bufs, n)


@pytest.mark.parametrize("alg", ["onebit", "tbq", "terngrad", "dgc", "graddrop"])
def test_batches_on_unaligned_views(hp, alg):
    """Tables of tensors whose every fp32 pointer is only 4-byte aligned, through the batched
    encode and the batched decoders (tile-pointer decode for the sparse formats)."""
    sizes = [9001, 4096, 300007, 1, 70003]
    rng = np.random.default_rng(len(alg))
    ratio = 0.01 if alg == "graddrop" else 0.001
    ts, keep, data = [], [], []
    for n in sizes:
        g, u = rng.normal(0, 0.02 if alg == "tbq" else 1e-3, n).astype(F), rng.random(n, dtype=F)
        (gv, s0, s1, uv, ov), bufs = views(n, g, np.zeros(n, F), np.zeros(n, F), u, None)
        nbytes = {"onebit": hp.onebit_payload_bytes(n), "tbq": hp.tbq_payload_bytes(n),
                  "terngrad": hp.terngrad_payload_bytes(n, 512), "dgc": hp.sparse_payload_bytes(n, ratio),
                  "graddrop": hp.sparse_payload_bytes(n, ratio)}[alg]
        t = {"gradient": gv, "out": ov, "compressed": payload(nbytes)}
        if alg in ("onebit", "tbq"):
            t["residual"] = s0
        elif alg == "dgc":
            t["momentum"], t["accumulator"] = s0, s1
        elif alg == "graddrop":
            t["accumulator"] = s1
        else:
            t["uniform"] = uv
        ts.append(t)
        keep.append(bufs)
        data.append((g, u))
    b = hp.Batch(alg, ts, threshold=0.05, bucket=512, momentum_factor=0.9, ratio=ratio)
    b.encode()
    b.decode()
    for t, n, (g, u), bufs in zip(ts, sizes, data, keep):
        z = np.zeros(n, F)
        got = host(t["compressed"])
        if alg == "onebit":
            want, _ = oracle.onebit_encode(g, z, scale=got[:4].view(F)[0])
            np.testing.assert_array_equal(got, want)
            ref = oracle.onebit_decode(want, n)
        elif alg == "tbq":
            want, want_r = oracle.tbq_encode(g, z, 0.05)
            np.testing.assert_array_equal(got, want)
            np.testing.assert_array_equal(host(t["residual"]), want_r)
            ref = oracle.tbq_decode(want, n)
        elif alg == "terngrad":
            want = oracle.terngrad_encode(g, u, 512)
            np.testing.assert_array_equal(got, want)
            ref = oracle.terngrad_decode(want, n)
        elif alg == "dgc":
            want, want_m, want_a = oracle.dgc_encode(g, z, z, 0.9, ratio)
            check_sparse(got, want)
            np.testing.assert_array_equal(host(t["momentum"]), want_m)
            np.testing.assert_array_equal(host(t["accumulator"]), want_a)
            ref = oracle.sparse_decode(want, n)
        else:
            want, want_a = oracle.graddrop_encode(g, z, ratio)
            check_sparse(got, want)
            np.testing.assert_array_equal(host(t["accumulator"]), want_a)
            ref = oracle.sparse_decode(want, n)
        np.testing.assert_array_equal(host(t["out"]), ref, err_msg=f"decode n={n}")
        untouched_outside(bufs, n)
    b.close()


# ================================================================ empty tensors
def test_every_per_tensor_entry_point_accepts_n_zero(hp):
    """n = 0: nothing but the payload header is written, and it equals the oracle's."""
    e = torch.empty(0, device="cuda")
    z = np.zeros(0, F)
    pay = payload(hp.tbq_payload_bytes(0))
    hp.tbq_encode(e, e, pay, 0.05)
    np.testing.assert_array_equal(host(pay), oracle.tbq_encode(z, z, 0.05)[0])
    hp.tbq_decode(pay, e)
    pay = payload(hp.onebit_payload_bytes(0))
    hp.onebit_encode(e, e, pay)
    np.testing.assert_array_equal(host(pay), oracle.onebit_encode(z, z)[0])
    hp.onebit_decode(pay, e)
    sstate = torch.full((1,), 3.0, device="cuda")
    pay2 = payload(hp.onebit_payload_bytes(0))
    hp.onebit_encode_deferred(e, e, sstate, pay2)
    np.testing.assert_array_equal(host(pay2), host(pay))
    assert host(sstate)[0] == 0.0
    hp.onebit_residual(e, sstate, e)
    pay = payload(hp.terngrad_payload_bytes(0, 512))
    hp.terngrad_encode(e, e, pay, 512)
    np.testing.assert_array_equal(host(pay), oracle.terngrad_encode(z, z, 512))
    hp.terngrad_decode(pay, e)
    for ratio in (0.001, 0.01):
        pay = payload(hp.sparse_payload_bytes(0, ratio))
        hp.dgc_encode(e, e, e, pay, 0.9, ratio)
        want = oracle.dgc_encode(z, z, z, 0.9, ratio)[0]
        np.testing.assert_array_equal(host(pay)[:16], want[:16])
        pay = payload(hp.sparse_payload_bytes(0, ratio))
        hp.graddrop_encode(e, e, pay, ratio)
        np.testing.assert_array_equal(host(pay)[:16], oracle.graddrop_encode(z, z, ratio)[0][:16])
        hp.dgc_decode(pay, e)
    for b in (1, 2, 4, 8):
        pay = payload(hp.compll_payload_bytes(0, b))
        hp.compll_terngrad_encode(e, e, pay, b)
        np.testing.assert_array_equal(host(pay), oracle.compll_encode(z, z, b))
        hp.compll_terngrad_decode(pay, e)
    # merges of empty chunks
    tp = [dev(oracle.tbq_encode(z, z, 0.05)[0]) for _ in range(3)]
    outp = payload(hp.tbq_payload_bytes(0))
    hp.tbq_decode_merge(tp, e)
    hp.tbq_decode_merge(tp, e, e, outp, 0.05)
    np.testing.assert_array_equal(host(outp), oracle.tbq_encode(z, z, 0.05)[0])
    hp.onebit_decode_merge([dev(oracle.onebit_encode(z, z)[0])], e)
    hp.terngrad_decode_merge([dev(oracle.terngrad_encode(z, z, 512))], e)
    sp = [dev(oracle.graddrop_encode(z, z, 0.01)[0]) for _ in range(3)]
    hp.dgc_decode_merge(sp, e)
    outp = payload(hp.sparse_payload_bytes(0, 0.01))
    hp.dgc_decode_merge(sp, e, e, outp, 0.01)
    np.testing.assert_array_equal(host(outp)[:16], oracle.graddrop_encode(z, z, 0.01)[0][:16])
    torch.cuda.synchronize()


def test_batches_accept_empty_tensors_among_others(hp):
    for alg in ("tbq", "onebit", "graddrop"):
        sizes = [0, 5000, 0]
        rng = np.random.default_rng(1)
        ts = []
        for n in sizes:
            g = dev(rng.normal(0, 0.02, n).astype(F))
            nbytes = {"tbq": hp.tbq_payload_bytes(n), "onebit": hp.onebit_payload_bytes(n),
                      "graddrop": hp.sparse_payload_bytes(n, 0.01)}[alg]
            t = {"gradient": g, "out": torch.full((n,), 7.0, device="cuda"), "compressed": payload(nbytes)}
            t["accumulator" if alg == "graddrop" else "residual"] = torch.zeros(n, device="cuda")
            ts.append(t)
        b = hp.Batch(alg, ts, threshold=0.05, ratio=0.01)
        b.encode()
        b.decode()
        g = host(ts[1]["gradient"])
        z = np.zeros(5000, F)
        if alg == "tbq":
            want = oracle.tbq_encode(g, z, 0.05)[0]
            np.testing.assert_array_equal(host(ts[1]["compressed"]), want)
            np.testing.assert_array_equal(host(ts[1]["out"]), oracle.tbq_decode(want, 5000))
            np.testing.assert_array_equal(host(ts[0]["compressed"]), oracle.tbq_encode(z[:0], z[:0], 0.05)[0])
        elif alg == "onebit":
            got = host(ts[1]["compressed"])
            want = oracle.onebit_encode(g, z, scale=got[:4].view(F)[0])[0]
            np.testing.assert_array_equal(got, want)
        else:
            check_sparse(host(ts[1]["compressed"]), oracle.graddrop_encode(g, z, 0.01)[0])
            assert oracle.sparse_unpack(host(ts[2]["compressed"]))[0] == 0
        b.close()


# ================================================================ large single chunks
def test_sparse_merge_of_one_large_chunk(hp):
    """One chunk of 20 M elements at one per cent: 4883 tiles and ~200 K pairs per peer, so the
    index launch spreads every peer's payload over some 200 workgroups and the two ends of a
    run record often come from different ones.  Then the same call with one peer's pairs out of
    order (the slow path), and once more with the sorted payloads on the same workspace."""
    n, P, ratio = 20_000_003, 4, 0.01
    rng = np.random.default_rng(9)
    z = np.zeros(n, F)
    pays = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), z, ratio)[0] for _ in range(P)]
    acc0 = rng.normal(0, 1e-4, n).astype(F)
    want_agg, want_out, want_acc = oracle.sparse_decode_merge(pays, n, acc0, ratio)

    def run(payloads):
        agg, acc = torch.full((n,), 7.0, device="cuda"), dev(acc0)
        outp = payload(hp.sparse_payload_bytes(n, ratio))
        hp.dgc_decode_merge([dev(p) for p in payloads], agg, acc, outp, ratio)
        np.testing.assert_array_equal(host(agg), want_agg)
        check_sparse(host(outp), want_out)
        np.testing.assert_array_equal(host(acc), want_acc)

    run(pays)
    # peer 2 with two far-apart pairs swapped: same content, not in order
    nnz, _, cap, _, idx, val = oracle.sparse_unpack(pays[2])
    shuffled = pays[2].copy()
    i32, f32 = shuffled[16:16 + 4 * cap].view(np.int32), shuffled[16 + 4 * cap:16 + 8 * cap].view(F)
    a, b = 1000, nnz - 2000
    i32[a], i32[b] = idx[b], idx[a]
    f32[a], f32[b] = val[b], val[a]
    run([pays[0], pays[1], shuffled, pays[3]])
    run(pays)


def test_sparse_merge_with_few_pairs_in_many_tiles(hp):
    """Long stretches of tiles without a pair (the index launch fills them workgroup-wide), a
    peer with no pair at all, and pairs in the first and the last tile only."""
    n, ratio = 4096 * 3000 + 17, 0.001
    cap = hp.sparse_capacity(n, ratio)

    def handmade(idx, val):
        p = np.zeros(16 + 8 * cap, np.uint8)
        p[:16].view(np.uint32)[:3] = [len(idx), n, cap]
        p[16:16 + 4 * len(idx)].view(np.int32)[:] = idx
        p[16 + 4 * cap:16 + 4 * cap + 4 * len(val)].view(F)[:] = val
        return p

    pays = [handmade([0, 5, n - 1], [1.0, 2.0, 3.0]), handmade([], []), handmade([4096 * 1500 + 7], [4.0]),
            handmade([5, 4096 * 1500 + 7, n - 1], [0.5, 0.25, 0.125])]
    agg = torch.full((n,), 7.0, device="cuda")
    hp.dgc_decode_merge([dev(p) for p in pays], agg)
    np.testing.assert_array_equal(host(agg), oracle.sparse_decode_merge(pays, n))


# ================================================================ streams and graphs
def test_two_streams_run_different_batches_at_once(hp):
    """Distinct batches are independent: a DGC set on one stream and a TBQ set on another,
    enqueued alternately for several steps without waiting in between, give what each gives
    alone."""
    rng = np.random.default_rng(77)
    sizes = [300007, 70001, 1048576]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    gd = [rng.normal(0, 1e-3, n).astype(F) for n in sizes]
    gt = [rng.normal(0, 0.02, n).astype(F) for n in sizes]
    with torch.cuda.stream(s1):
        td = [{"gradient": dev(g), "momentum": torch.zeros(g.size, device="cuda"), "accumulator": torch.zeros(g.size, device="cuda"),
               "out": torch.empty(g.size, device="cuda"), "compressed": payload(hp.sparse_payload_bytes(g.size, 0.001))} for g in gd]
        bd = hp.Batch("dgc", td, momentum_factor=0.9, ratio=0.001)
    with torch.cuda.stream(s2):
        tt = [{"gradient": dev(g), "residual": torch.zeros(g.size, device="cuda"), "out": torch.empty(g.size, device="cuda"),
               "compressed": payload(hp.tbq_payload_bytes(g.size))} for g in gt]
        bt = hp.Batch("tbq", tt, threshold=0.05)
    torch.cuda.synchronize()
    steps = 4
    for _ in range(steps):
        with torch.cuda.stream(s1):
            bd.encode()
            bd.decode()
        with torch.cuda.stream(s2):
            bt.encode()
            bt.decode()
    torch.cuda.synchronize()
    for g, t in zip(gd, td):
        mom, acc = np.zeros(g.size, F), np.zeros(g.size, F)
        for _ in range(steps):
            want, mom, acc = oracle.dgc_encode(g, mom, acc, 0.9, 0.001)
        check_sparse(host(t["compressed"]), want)
        np.testing.assert_array_equal(host(t["accumulator"]), acc)
        np.testing.assert_array_equal(host(t["out"]), oracle.sparse_decode(want, g.size))
    for g, t in zip(gt, tt):
        r = np.zeros(g.size, F)
        for _ in range(steps):
            want, r = oracle.tbq_encode(g, r, 0.05)
        np.testing.assert_array_equal(host(t["compressed"]), want)
        np.testing.assert_array_equal(host(t["residual"]), r)
    bd.close()
    bt.close()


def test_hip_graph_replay_of_a_sparse_merge_batch(hp):
    """MergeBatch.run (index, merge + accumulate, three select passes, count, scan, emit)
    captured once and replayed with new peer payloads before every replay: each replay equals
    the oracle run from the same state, with the program's own eager work in between."""
    sizes, P, ratio = [1048576, 300007, 4097], 4, 0.001
    rng = np.random.default_rng(5)
    chunks = [{"compressed": [torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda") for _ in range(P)],
               "aggregate": torch.empty(n, device="cuda"), "state": torch.zeros(n, device="cuda"),
               "out_compressed": torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")} for n in sizes]
    mb = hp.MergeBatch("dgc", chunks, ratio=ratio)

    def new_payloads():
        host_pays = []
        for c, n in zip(chunks, sizes):
            ps = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), ratio)[0] for _ in range(P)]
            for dst, p in zip(c["compressed"], ps):
                dst.copy_(dev(p))
            host_pays.append(ps)
        return host_pays

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    new_payloads()
    with torch.cuda.stream(stream):
        mb.run()  # warm-up on the capture stream, then back to the initial state
        stream.synchronize()
        for c in chunks:
            c["state"].zero_()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            mb.run()
    ref = [np.zeros(n, F) for n in sizes]
    for rep in range(3):
        pays = new_payloads()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _ = (chunks[0]["aggregate"] * 2).sum().item()  # unrelated eager work between replays
        for i, (c, n) in enumerate(zip(chunks, sizes)):
            agg, out, ref[i] = oracle.sparse_decode_merge(pays[i], n, ref[i], ratio)
            np.testing.assert_array_equal(host(c["aggregate"]), agg, err_msg=f"aggregate, replay {rep} chunk {i}")
            check_sparse(host(c["out_compressed"]), out, f"replay {rep} chunk {i}")
            np.testing.assert_array_equal(host(c["state"]), ref[i], err_msg=f"state, replay {rep} chunk {i}")
    mb.close()


@pytest.mark.parametrize("bucket", [512, 100])
def test_hip_graph_replay_of_a_terngrad_merge_batch(hp, bucket):
    """The TernGrad merge batch is three launches (headers -> flags, the lean sum, the general sum
    over flagged chunks).  Captured once, replayed with new peer payloads in the same buffers before
    every replay; which chunks hold a peer of another bucket size changes from replay to replay,
    so the flags a replay writes differ from the ones the capture saw."""
    sizes, P = [1048576, 300007, 4097, 70001], 5
    rng = np.random.default_rng(bucket)
    room = {n: max(hp.terngrad_payload_bytes(n, b) for b in (bucket, 64, 300)) for n in sizes}
    chunks = [{"compressed": [torch.zeros(room[n], dtype=torch.uint8, device="cuda") for _ in range(P)],
               "aggregate": torch.empty(n, device="cuda")} for n in sizes]
    mb = hp.MergeBatch("terngrad", chunks, bucket=bucket)

    def new_payloads(odd):
        want = []
        for k, (c, n) in enumerate(zip(chunks, sizes)):
            ps = []
            for p in range(P):
                b = (64 if p == 1 else 300) if k % 2 == odd and p in (1, 4) else bucket
                ps.append(oracle.terngrad_encode(rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F), b))
                c["compressed"][p].zero_()
                c["compressed"][p][: ps[-1].size] = dev(ps[-1])
            want.append(oracle.terngrad_decode_merge(ps, n))
        return want

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    new_payloads(0)
    with torch.cuda.stream(stream):
        mb.run()  # warm-up on the capture stream
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            mb.run()
    for rep in range(4):
        want = new_payloads(rep % 2 if rep < 3 else 2)  # the last replay: no chunk is flagged
        for c in chunks:
            c["aggregate"].fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _ = (chunks[0]["aggregate"] * 2).sum().item()  # unrelated eager work between replays
        for i, (c, w) in enumerate(zip(chunks, want)):
            np.testing.assert_array_equal(host(c["aggregate"]), w, err_msg=f"replay {rep} chunk {i}")
    mb.close()

