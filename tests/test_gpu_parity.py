"""GPU parity: the HIP operators, called through the C ABI (hipress_amd.ops ->
ctypes -> libhipress_amd.so), against the CPU oracle on the same seeded inputs.

Bars: packed words, sparse indices / counts, thresholds and residuals are
bit-exact; the onebit scale (a sum whose order differs) is within 1e-5 relative
and everything derived from it is bit-exact once the oracle is given the GPU's
scale."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32
SIZES = [1, 15, 16, 17, 31, 33, 1000, 4095, 4096, 4097, 12289, 262144, 1000003]


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()  # fails loudly if the HIP library is missing
    return hipress_amd


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def payload(nbytes):
    # poison so that bytes the kernels must write (pad codes, header zeros) are checked
    return torch.full((nbytes,), 0xAB, dtype=torch.uint8, device="cuda")


# ---------------------------------------------------------------- TBQ
@pytest.mark.parametrize("n", SIZES)
def test_tbq_encode_decode(hp, n):
    rng = np.random.default_rng(n)
    tau = 0.05
    r_ref = rng.normal(0, 0.02, n).astype(F)
    r_gpu = dev(r_ref)
    for step in range(3):
        g = rng.normal(0, 0.02, n).astype(F)
        pay = payload(hp.tbq_payload_bytes(n))
        hp.tbq_encode(dev(g), r_gpu, pay, tau)
        want_pay, r_ref = oracle.tbq_encode(g, r_ref, tau)
        np.testing.assert_array_equal(host(pay), want_pay, err_msg=f"payload step {step}")
        np.testing.assert_array_equal(host(r_gpu), r_ref, err_msg=f"residual step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.tbq_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.tbq_decode(want_pay, n))


def test_tbq_unaligned_views(hp):
    n = 9001
    rng = np.random.default_rng(1)
    g, r = rng.normal(0, 0.05, n).astype(F), rng.normal(0, 0.05, n).astype(F)
    gbuf, rbuf, obuf = torch.zeros(n + 3, device="cuda"), torch.zeros(n + 3, device="cuda"), torch.zeros(n + 3, device="cuda")
    gv, rv, ov = gbuf[1 : n + 1], rbuf[3 : n + 3], obuf[2 : n + 2]
    gv.copy_(dev(g)); rv.copy_(dev(r))
    pay = payload(hp.tbq_payload_bytes(n))
    hp.tbq_encode(gv, rv, pay, 0.05)
    want_pay, want_r = oracle.tbq_encode(g, r, 0.05)
    np.testing.assert_array_equal(host(pay), want_pay)
    np.testing.assert_array_equal(host(rv), want_r)
    assert host(rbuf)[:3].tolist() == [0, 0, 0]
    hp.tbq_decode(pay, ov)
    np.testing.assert_array_equal(host(ov), oracle.tbq_decode(want_pay, n))
    assert host(obuf)[:2].tolist() == [0, 0] and host(obuf)[-1] == 0


def test_tbq_config1_full_size(hp):
    """262,144 elements, N(0, 0.02), threshold 0.05, residual zeros, seed 0."""
    n = 262144
    g = np.random.default_rng(0).normal(0, 0.02, n).astype(F)
    r = torch.zeros(n, device="cuda")
    pay = payload(hp.tbq_payload_bytes(n))
    hp.tbq_encode(dev(g), r, pay, 0.05)
    want_pay, want_r = oracle.tbq_encode(g, np.zeros(n, F), 0.05)
    np.testing.assert_array_equal(host(pay), want_pay)
    np.testing.assert_array_equal(host(r), want_r)
    out = torch.empty(n, device="cuda")
    hp.tbq_decode(pay, out)
    np.testing.assert_array_equal(host(out), oracle.tbq_decode(want_pay, n))


def test_tbq_config1_three_steps_on_the_generated_tensor(hp):
    """The first configuration as it is measured: one gradient of 262,144 elements, N(0, 0.02),
    from the library's own counter-based generator with seed 0 (the tensor bench.py times),
    threshold 0.05, residual zeros, three consecutive steps with the residual carried: payload,
    residual and decoded tensor bit for bit against the oracle at every step."""
    from hipress_amd import workloads

    n = 262144
    g_dev = workloads.normal_set([n], torch.device("cuda:0"), 0, sigma=0.02)[0]
    g = host(g_dev)
    assert g.dtype == F and abs(float(g.std()) - 0.02) < 5e-4 and abs(float(g.mean())) < 2e-4
    r_gpu, r_ref = torch.zeros(n, device="cuda"), np.zeros(n, F)
    seen = []
    for step in range(3):
        pay = payload(hp.tbq_payload_bytes(n))
        hp.tbq_encode(g_dev, r_gpu, pay, 0.05)
        want_pay, r_ref = oracle.tbq_encode(g, r_ref, 0.05)
        np.testing.assert_array_equal(host(pay), want_pay, err_msg=f"payload step {step}")
        np.testing.assert_array_equal(host(r_gpu).view(np.uint32), r_ref.view(np.uint32), err_msg=f"residual step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.tbq_decode(pay, out)
        want_out = oracle.tbq_decode(want_pay, n)
        np.testing.assert_array_equal(host(out).view(np.uint32), want_out.view(np.uint32), err_msg=f"decode step {step}")
        seen.append(int(np.count_nonzero(want_out)))
    # the carried residual matters: with sigma = 0.02 and tau = 0.05 later steps send more than the first
    assert seen[0] > 0 and seen[1] > seen[0] and seen[2] > seen[0], seen


# ---------------------------------------------------------------- onebit
@pytest.mark.parametrize("n", SIZES)
def test_onebit_encode_decode(hp, n):
    rng = np.random.default_rng(100 + n)
    r_ref = rng.normal(0, 1e-3, n).astype(F)
    r_gpu = dev(r_ref)
    for step in range(2):
        g = rng.normal(0, 1e-3, n).astype(F)
        pay = payload(hp.onebit_payload_bytes(n))
        hp.onebit_encode(dev(g), r_gpu, pay)
        got = host(pay)
        s_gpu = got[:4].view(F)[0]
        s_ref = oracle.onebit_scale(g, r_ref)
        assert abs(float(s_gpu) - float(s_ref)) <= 1e-5 * float(s_ref), (s_gpu, s_ref)
        # with the GPU's scale the oracle must reproduce every byte and every residual bit
        want_pay, r_next = oracle.onebit_encode(g, r_ref, scale=s_gpu)
        np.testing.assert_array_equal(got, want_pay, err_msg=f"payload step {step}")
        np.testing.assert_array_equal(host(r_gpu), r_next, err_msg=f"residual step {step}")
        # and against the oracle's own scale the residual is within 1e-5 * max(s, |r|)
        _, r_own = oracle.onebit_encode(g, r_ref)
        assert np.all(np.abs(r_next - r_own) <= 1e-5 * np.maximum(s_ref, np.abs(r_own)))
        out = torch.full((n,), 7.0, device="cuda")
        hp.onebit_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.onebit_decode(want_pay, n))
        r_ref = r_next


def test_onebit_scale_is_deterministic(hp):
    n = 3_000_000
    g = dev(np.random.default_rng(2).normal(0, 1e-3, n).astype(F))
    scales = []
    for _ in range(3):
        pay = payload(hp.onebit_payload_bytes(n))
        hp.onebit_encode(g, torch.zeros(n, device="cuda"), pay)
        scales.append(host(pay)[:4].view(np.uint32)[0])
    assert len(set(scales)) == 1


@pytest.mark.parametrize("n", [1, 33, 4097, 1000003])
def test_onebit_deferred_matches_two_pass(hp, n):
    """The one-pass variant must produce the payloads of onebit_encode and, on
    request, the residual it would hold - bit for bit, over several steps."""
    rng = np.random.default_rng(500 + n)
    r0 = rng.normal(0, 1e-3, n).astype(F)
    state, sstate = dev(r0), torch.zeros(1, device="cuda")
    r_two = dev(r0)
    r_ref = r0
    for step in range(4):
        g = rng.normal(0, 1e-3, n).astype(F)
        pay_d = payload(hp.onebit_payload_bytes(n))
        pay_t = payload(hp.onebit_payload_bytes(n))
        hp.onebit_encode_deferred(dev(g), state, sstate, pay_d)
        hp.onebit_encode(dev(g), r_two, pay_t)
        got = host(pay_d)
        np.testing.assert_array_equal(got, host(pay_t), err_msg=f"payload step {step}")
        res = torch.empty(n, device="cuda")
        hp.onebit_residual(state, sstate, res)
        np.testing.assert_array_equal(host(res), host(r_two), err_msg=f"residual step {step}")
        # and against the oracle, given the GPU's scale
        s_gpu = got[:4].view(F)[0]
        assert host(sstate)[0] == s_gpu
        want_pay, r_ref = oracle.onebit_encode(g, r_ref, scale=s_gpu)
        np.testing.assert_array_equal(got, want_pay)
        np.testing.assert_array_equal(host(res), r_ref)


def test_onebit_zero_tensor(hp):
    n = 5000
    pay = payload(hp.onebit_payload_bytes(n))
    r = torch.zeros(n, device="cuda")
    hp.onebit_encode(torch.zeros(n, device="cuda"), r, pay)
    want_pay, want_r = oracle.onebit_encode(np.zeros(n, F), np.zeros(n, F))
    np.testing.assert_array_equal(host(pay), want_pay)
    np.testing.assert_array_equal(host(r), want_r)


# ---------------------------------------------------------------- TernGrad
# 256 / 512 / 1024: the bucket maximum is a wavefront reduction; every other size up to a tile
# (1, 3, 16, 100, 2048, 4095, 4096) goes through the single-pass encoder whose maxima meet in
# LDS, buckets hanging over into the neighbouring tiles included; beyond a tile (4097, 5000,
# 8192: buckets that begin with a tile, 70000: a bucket longer than most of these tensors,
# 2000000: one bucket for all of them) per-tile maxima are folded per bucket by a launch of its own.
@pytest.mark.parametrize("bucket", [512, 256, 1024, 100, 16, 2048, 1, 3, 4095, 4096, 4097, 5000, 8192, 70000, 2000000])
@pytest.mark.parametrize("n", [1, 17, 511, 512, 513, 4097, 70001, 1000003])
def test_terngrad_encode_decode(hp, n, bucket):
    rng = np.random.default_rng(n * 7 + bucket)
    g = rng.normal(0, 1e-3, n).astype(F)
    out_l = rng.random(n) < 0.01
    g[out_l] = rng.laplace(0, 1e-2, out_l.sum()).astype(F)
    u = rng.random(n, dtype=F)
    pay = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode(dev(g), dev(u), pay, bucket)
    want = oracle.terngrad_encode(g, u, bucket)
    np.testing.assert_array_equal(host(pay), want)
    out = torch.full((n,), 7.0, device="cuda")
    hp.terngrad_decode(pay, out)
    np.testing.assert_array_equal(host(out), oracle.terngrad_decode(want, n))


@pytest.mark.parametrize("bucket", [100, 3000, 4096, 6000, 8192, 50000])
def test_terngrad_any_bucket_with_special_values_and_batches(hp, bucket):
    """The LDS maxima of the single-pass encoder on values fmaxf treats specially (NaN is
    passed over, infinities and signed zeros are not), through a batch whose tensors begin at
    odd tile counts, against the oracle."""
    rng = np.random.default_rng(bucket)
    sizes = [4096 * 3 + 17, 1, 4096, 12345, 4095, 70001]
    tensors, want = [], []
    for k, n in enumerate(sizes):
        g = rng.normal(0, 1e-3, n).astype(F)
        if n > 100:
            idx = rng.choice(n, size=min(n // 50, 40), replace=False)
            g[idx] = rng.choice(np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, 3e38, -3e38], F), size=idx.size)
            g[bucket - 1 if bucket - 1 < n else 0] = np.nan        # last element of the first bucket
            g[min(n - 1, 4096)] = -np.inf                          # first element behind a tile border
        u = rng.random(n, dtype=F)
        tensors.append({"gradient": dev(g), "uniform": dev(u), "out": torch.full((n,), 7.0, device="cuda"),
                        "compressed": payload(hp.terngrad_payload_bytes(n, bucket))})
        want.append(oracle.terngrad_encode(g, u, bucket))
    b = hp.Batch("terngrad", tensors, bucket=bucket)
    b.encode()
    b.decode()
    for t, w, n in zip(tensors, want, sizes):
        np.testing.assert_array_equal(host(t["compressed"]), w, err_msg=f"payload n={n}")
        got, ref = host(t["out"]), oracle.terngrad_decode(w, n)
        np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
        np.testing.assert_array_equal(got[~np.isnan(ref)], ref[~np.isnan(ref)], err_msg=f"decode n={n}")
    b.close()


@pytest.mark.parametrize("bucket", [1_000_000, 4096 * 1000, 20_000_003, 2**31 - 1])
def test_terngrad_buckets_over_thousands_of_tiles(hp, bucket):
    """Buckets that cover hundreds to thousands of tiles, up to one bucket for the whole tensor
    (the per-layer scale of the original TernGrad), on a tensor that starts 4 bytes into its
    allocation; the largest magnitudes sit where a fold over tiles could lose them: in the
    first and the last element and either side of a bucket border."""
    n = 20_000_003
    rng = np.random.default_rng(bucket % 1000)
    g = rng.normal(0, 1e-3, n).astype(F)
    g[0], g[n - 1] = 0.5, -0.75
    if bucket < n:
        g[bucket - 1], g[bucket] = 0.25, -0.375
    u = rng.random(n, dtype=F)
    gd = torch.empty(n + 1, device="cuda")[1:]
    gd.copy_(torch.from_numpy(g))
    pay = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode(gd, dev(u), pay, bucket)
    want = oracle.terngrad_encode(g, u, bucket)
    np.testing.assert_array_equal(host(pay), want)
    out = torch.full((n,), 7.0, device="cuda")
    hp.terngrad_decode(pay, out)
    np.testing.assert_array_equal(host(out), oracle.terngrad_decode(want, n))


def test_terngrad_decode_rejects_header_that_overruns_buffer(hp):
    n = 5000
    pay = torch.zeros(hp.terngrad_payload_bytes(n, 512), dtype=torch.uint8, device="cuda")
    hdr = np.zeros(4, np.uint32)
    hdr[:2] = [n, 1]  # bucket 1 would need a 20 KB scale array: does not fit
    pay[:16] = dev(hdr.view(np.uint8))
    out = torch.full((n,), 7.0, device="cuda")
    hp.terngrad_decode(pay, out)
    assert not host(out).any()


# ---------------------------------------------------------------- DGC / GradDrop
def check_sparse(got_pay, want_pay):
    g = oracle.sparse_unpack(got_pay)
    w = oracle.sparse_unpack(want_pay)
    assert g[:3] == w[:3], (g[:3], w[:3])
    assert g[3].view(np.uint32) == w[3].view(np.uint32), (g[3], w[3])
    np.testing.assert_array_equal(g[4], w[4])
    np.testing.assert_array_equal(g[5], w[5])


@pytest.mark.parametrize("n", [1, 63, 1000, 4097, 70001, 262143, 262144, 1000003])
def test_dgc_encode_decode(hp, n):
    rng = np.random.default_rng(200 + n)
    m, ratio = 0.9, 0.001
    mom_ref, acc_ref = np.zeros(n, F), np.zeros(n, F)
    mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    for step in range(3):
        g = rng.normal(0, 1e-3, n).astype(F)
        pay = payload(hp.dgc_payload_bytes(n, ratio))
        hp.dgc_encode(dev(g), mom, acc, pay, m, ratio)
        want_pay, mom_ref, acc_ref = oracle.dgc_encode(g, mom_ref, acc_ref, m, ratio)
        check_sparse(host(pay), want_pay)
        np.testing.assert_array_equal(host(mom), mom_ref, err_msg=f"momentum step {step}")
        np.testing.assert_array_equal(host(acc), acc_ref, err_msg=f"accumulator step {step}")
        out = torch.full((n,), 7.0, device="cuda")
        hp.dgc_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.sparse_decode(want_pay, n))


@pytest.mark.parametrize("n", [1, 1000, 4097, 70001, 262144, 1000003])
def test_graddrop_encode_decode(hp, n):
    rng = np.random.default_rng(300 + n)
    ratio = 0.01
    acc_ref = np.zeros(n, F)
    acc = torch.zeros(n, device="cuda")
    for step in range(2):
        g = rng.normal(0, 1e-3, n).astype(F)
        pay = payload(hp.graddrop_payload_bytes(n, ratio))
        hp.graddrop_encode(dev(g), acc, pay, ratio)
        want_pay, acc_ref = oracle.graddrop_encode(g, acc_ref, ratio)
        check_sparse(host(pay), want_pay)
        np.testing.assert_array_equal(host(acc), acc_ref)
        out = torch.full((n,), 7.0, device="cuda")
        hp.graddrop_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.sparse_decode(want_pay, n))


def test_sparse_threshold_many_sample_tiles(hp):
    """24M elements: 240,000 sample keys = 59 sample tiles, so the per-tensor
    histogram is merged from workgroups on every XCD."""
    n = 24_000_000
    g = np.random.default_rng(12).normal(0, 1e-3, n).astype(F)
    for ratio, enc in ((0.001, "dgc"), (0.01, "graddrop")):
        pay = payload(hp.sparse_payload_bytes(n, ratio))
        acc = torch.zeros(n, device="cuda")
        if enc == "dgc":
            mom = torch.zeros(n, device="cuda")
            hp.dgc_encode(dev(g), mom, acc, pay, 0.9, ratio)
            want_pay, _, want_acc = oracle.dgc_encode(g, np.zeros(n, F), np.zeros(n, F), 0.9, ratio)
        else:
            hp.graddrop_encode(dev(g), acc, pay, ratio)
            want_pay, want_acc = oracle.graddrop_encode(g, np.zeros(n, F), ratio)
        check_sparse(host(pay), want_pay)
        np.testing.assert_array_equal(host(acc), want_acc)


def test_sparse_overflow_ties(hp):
    n = 10000
    g = np.full(n, 0.5, F)
    acc = torch.zeros(n, device="cuda")
    pay = payload(hp.graddrop_payload_bytes(n, 0.001))
    hp.graddrop_encode(dev(g), acc, pay, 0.001)
    want_pay, want_acc = oracle.graddrop_encode(g, np.zeros(n, F), 0.001)
    check_sparse(host(pay), want_pay)
    np.testing.assert_array_equal(host(acc), want_acc)
    assert oracle.sparse_unpack(want_pay)[0] == 64


@pytest.mark.parametrize("alg", ["dgc", "graddrop"])
def test_sparse_overflow_by_clipped_gradients(hp, alg):
    """Gradients clipped by value: 5 % of a 3 M-element tensor sit at exactly +-0.01, far more
    than the slots hold, and nothing lies above them.  The threshold stays at the clip value
    and the ties go out in index order, step after step as the accumulator releases them; the
    second step mixes released ties with accumulated values."""
    n, ratio = 3_000_001, 0.001
    rng = np.random.default_rng(17)
    mom_ref, acc_ref = np.zeros(n, F), np.zeros(n, F)
    mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    for step in range(3):
        g = np.clip(rng.normal(0, 5e-3, n), -0.01, 0.01).astype(F)
        pay = payload(hp.sparse_payload_bytes(n, ratio))
        if alg == "dgc":
            hp.dgc_encode(dev(g), mom, acc, pay, 0.9, ratio)
            want, mom_ref, acc_ref = oracle.dgc_encode(g, mom_ref, acc_ref, 0.9, ratio)
            np.testing.assert_array_equal(host(mom), mom_ref, err_msg=f"momentum, step {step}")
        else:
            hp.graddrop_encode(dev(g), acc, pay, ratio)
            want, acc_ref = oracle.graddrop_encode(g, acc_ref, ratio)
        check_sparse(host(pay), want)
        np.testing.assert_array_equal(host(acc), acc_ref, err_msg=f"accumulator, step {step}")
        nnz, _, cap, *_ = oracle.sparse_unpack(want)
        if step == 0:
            assert nnz == cap  # the case meant: every slot used


def test_sparse_overflow_rethreshold(hp):
    n = 262144
    rng = np.random.default_rng(11)
    a = rng.uniform(1.0, 2.0, n).astype(F) * rng.choice([-1, 1], n).astype(F)
    a[50::100] = rng.uniform(0.001, 0.002, a[50::100].size).astype(F)
    a[1000:1010] = a[2000]  # some exact ties near the top
    mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    pay = payload(hp.dgc_payload_bytes(n, 0.001))
    hp.dgc_encode(dev(a), mom, acc, pay, 0.9, 0.001)
    want_pay, want_mom, want_acc = oracle.dgc_encode(a, np.zeros(n, F), np.zeros(n, F), 0.9, 0.001)
    check_sparse(host(pay), want_pay)
    np.testing.assert_array_equal(host(mom), want_mom)
    np.testing.assert_array_equal(host(acc), want_acc)


def test_sparse_all_zero(hp):
    n = 5000
    acc = torch.zeros(n, device="cuda")
    pay = payload(hp.graddrop_payload_bytes(n, 0.01))
    hp.graddrop_encode(torch.zeros(n, device="cuda"), acc, pay, 0.01)
    nnz, n_, cap, thr, idx, val = oracle.sparse_unpack(host(pay))
    assert (nnz, n_, thr) == (0, n, 0)
    out = torch.full((n,), 7.0, device="cuda")
    hp.graddrop_decode(pay, out)
    assert not host(out).any()


# ---------------------------------------------------------------- decode-and-merge
@pytest.mark.parametrize("n", [1, 4097, 1048576])
@pytest.mark.parametrize("npeers", [1, 8, 9, 16])
def test_tbq_decode_merge(hp, n, npeers):
    rng = np.random.default_rng(n + npeers)
    tau = 0.05
    pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(npeers)]
    dpays = [dev(p) for p in pays]
    agg = torch.full((n,), 7.0, device="cuda")
    hp.tbq_decode_merge(dpays, agg)
    np.testing.assert_array_equal(host(agg), oracle.tbq_decode_merge(pays, n))
    # fused re-encode with the aggregator's residual
    r0 = rng.normal(0, 0.01, n).astype(F)
    r = dev(r0)
    out = payload(hp.tbq_payload_bytes(n))
    agg.fill_(7.0)
    hp.tbq_decode_merge(dpays, agg, r, out, tau)
    want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, r0, tau)
    np.testing.assert_array_equal(host(agg), want_agg)
    np.testing.assert_array_equal(host(out), want_out)
    np.testing.assert_array_equal(host(r), want_r)


@pytest.mark.parametrize("P", [5, 13])
def test_onebit_and_terngrad_decode_merge(hp, P):
    n = 70001
    rng = np.random.default_rng(9 + P)
    ob = [oracle.onebit_encode(rng.normal(0, 1, n).astype(F), np.zeros(n, F))[0] for _ in range(P)]
    agg = torch.empty(n, device="cuda")
    hp.onebit_decode_merge([dev(p) for p in ob], agg)
    np.testing.assert_array_equal(host(agg), oracle.onebit_decode_merge(ob, n))
    for bucket in (512, 100):
        tg = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), bucket) for _ in range(P)]
        hp.terngrad_decode_merge([dev(p) for p in tg], agg)
        np.testing.assert_array_equal(host(agg), oracle.terngrad_decode_merge(tg, n))


def test_terngrad_decode_merge_skips_a_peer_whose_header_does_not_fit(hp):
    """A peer whose header names a bucket size of zero, or one whose scales and words
    would not fit its buffer, adds nothing; the other peers are summed as usual."""
    n, bucket = 20000, 512
    rng = np.random.default_rng(31)
    tg = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), bucket) for _ in range(3)]
    zero_bucket = tg[1].copy()
    zero_bucket[4:8] = 0          # header word 1 = bucket size
    tiny_bucket = tg[1].copy()
    tiny_bucket[4:8] = np.frombuffer(np.uint32(1).tobytes(), np.uint8)  # n scales would not fit the buffer
    agg = torch.empty(n, device="cuda")
    for bad in (zero_bucket, tiny_bucket):
        hp.terngrad_decode_merge([dev(tg[0]), dev(bad), dev(tg[2])], agg)
        np.testing.assert_array_equal(host(agg), oracle.terngrad_decode_merge([tg[0], tg[2]], n))


@pytest.mark.parametrize("roomy", [True, False])
@pytest.mark.parametrize("expected", [512, 100, 4096, 3])
def test_terngrad_merge_batch_with_peers_of_other_bucket_sizes(hp, expected, roomy):
    """A merge batch names the bucket size its peers are expected to have used and asks for
    their words from that before it has seen their headers; a header that names another size
    still decides.  Nine peers per chunk (two rounds of the kernel's eight): most with the
    expected size, the others with sizes of every kind (a multiple of 256, a power of two below
    it, neither, longer than a tile, 1), and one whose header is unusable.  Against the oracle,
    which reads every header."""
    rng = np.random.default_rng(expected)
    others = [256, 64, 100, 6000, 1, expected, expected, expected, expected]
    sizes = [4096 * 2 + 17, 100003, 5, 4096]
    chunks, want = [], []
    for n in sizes:
        pays = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), b) for b in others]
        broken = pays[6].copy()
        broken[4:8] = 0  # bucket size 0: this peer adds nothing
        pays[6] = broken
        # roomy: every buffer as large as the largest layout, so that the expected layout fits all
        # of them and is read before the header corrects it; otherwise every buffer exactly as large
        # as its own layout, so that for some peers the expected layout does not fit and nothing
        # may be read from it
        room = max(p.size for p in pays)
        bufs = []
        for p in pays:
            t = torch.zeros(room if roomy else p.size, dtype=torch.uint8, device="cuda")
            t[: p.size] = dev(p)
            bufs.append(t)
        chunks.append({"compressed": bufs, "aggregate": torch.full((n,), 7.0, device="cuda")})
        want.append(oracle.terngrad_decode_merge([p for k, p in enumerate(pays) if k != 6], n))
    mb = hp.MergeBatch("terngrad", chunks, bucket=expected)
    mb.run()
    for c, w, n in zip(chunks, want, sizes):
        np.testing.assert_array_equal(host(c["aggregate"]), w, err_msg=f"n={n}")
    # and peer by peer through the per-tensor call, which has no expectation to start from
    for c, w, n in zip(chunks, want, sizes):
        agg = torch.full((n,), 7.0, device="cuda")
        hp.terngrad_decode_merge(c["compressed"], agg)
        np.testing.assert_array_equal(host(agg), w, err_msg=f"per-tensor n={n}")
    mb.close()


@pytest.mark.parametrize("bucket", [512, 4096])
def test_terngrad_merge_batch_where_only_some_chunks_hold_another_bucket_size(hp, bucket):
    """With a bucket size that is a multiple of 256 the batch runs a kernel that knows nothing of
    other sizes; chunks in which some header disagrees are flagged by a launch before it and written
    by a launch after it.  Six chunks (one of them starting from a local gradient, 16 peers in two
    rounds), the odd ones with one peer of another size; then the payloads change places in the same
    buffers, so that the flags of the second run are the opposite of the first's."""
    rng = np.random.default_rng(bucket)
    P, sizes = 16, [4096 * 3 + 5, 100003, 4096, 70001, 300007, 17]
    room = {n: max(hp.terngrad_payload_bytes(n, b) for b in (bucket, 100, 64)) for n in sizes}
    grads = {n: [(rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F)) for _ in range(P)] for n in sizes}
    local = rng.normal(0, 1e-3, sizes[1]).astype(F)
    chunks = []
    for k, n in enumerate(sizes):
        c = {"compressed": [torch.zeros(room[n], dtype=torch.uint8, device="cuda") for _ in range(P)],
             "aggregate": torch.full((n,), 7.0, device="cuda")}
        if k == 1:
            c["local"] = dev(local)
        chunks.append(c)
    mb = hp.MergeBatch("terngrad", chunks, bucket=bucket)
    for rnd in range(3):
        for k, (c, n) in enumerate(zip(chunks, sizes)):
            odd_one = (k + rnd) % 2 == 1
            pays = []
            for p, (g, u) in enumerate(grads[n]):
                b = (100 if p == 11 else 64) if odd_one and p in (3, 11) and (p == 3 or rnd == 2) else bucket
                pays.append(oracle.terngrad_encode(g, u, b))
                c["compressed"][p].zero_()
                c["compressed"][p][: pays[-1].size] = dev(pays[-1])
            c["want"] = oracle.terngrad_decode_merge(pays, n, local=local if k == 1 else None)
            c["aggregate"].fill_(7.0)
        mb.run()
        for k, (c, n) in enumerate(zip(chunks, sizes)):
            np.testing.assert_array_equal(host(c["aggregate"]), c["want"], err_msg=f"round {rnd} chunk {k} n={n}")
    mb.close()


@pytest.mark.parametrize("n", [1000, 1048576])
def test_sparse_decode_merge(hp, n):
    P, ratio = 8, 0.001
    rng = np.random.default_rng(n)
    pays = []
    for p in range(P):
        g = rng.normal(0, 1e-3, n).astype(F)
        g[:20] += 1.0  # duplicates across peers
        pays.append(oracle.dgc_encode(g, np.zeros(n, F), np.zeros(n, F), 0.9, ratio)[0])
    dpays = [dev(p) for p in pays]
    agg = torch.full((n,), 7.0, device="cuda")
    hp.dgc_decode_merge(dpays, agg)
    want = oracle.sparse_decode_merge(pays, n)
    np.testing.assert_allclose(host(agg), want, rtol=1e-5, atol=0)
    # re-sparsify for the next hop; compare against the oracle run on the GPU's aggregate
    acc0 = rng.normal(0, 1e-3, n).astype(F)
    acc = dev(acc0)
    out = payload(hp.dgc_payload_bytes(n, ratio))
    hp.dgc_decode_merge(dpays, agg, acc, out, ratio)
    got_agg = host(agg)
    np.testing.assert_allclose(got_agg, want, rtol=1e-5, atol=0)
    want_out, want_acc = oracle.graddrop_encode(got_agg, acc0, ratio)
    check_sparse(host(out), want_out)
    np.testing.assert_array_equal(host(acc), want_acc)


def test_sparse_decode_merge_is_exact_in_peer_order_and_accepts_unsorted(hp):
    n, P, ratio = 300000, 8, 0.001
    rng = np.random.default_rng(17)
    pays = []
    for p in range(P):
        g = rng.normal(0, 1e-3, n).astype(F)
        g[:30] += 1.0 + p * 0.37  # the same leading entries in every peer: sums depend on order
        pays.append(oracle.dgc_encode(g, np.zeros(n, F), np.zeros(n, F), 0.9, ratio)[0])
    agg = torch.full((n,), 7.0, device="cuda")
    hp.dgc_decode_merge([dev(p) for p in pays], agg)
    np.testing.assert_array_equal(host(agg), oracle.sparse_decode_merge(pays, n))  # peer order => bit-exact
    # shuffle the pairs of two peers: still the same aggregate
    shuffled = [p.copy() for p in pays]
    for q in (1, 5):
        nnz, _, cap, _, idx, val = oracle.sparse_unpack(shuffled[q])
        perm = rng.permutation(nnz)
        shuffled[q][16 : 16 + 4 * nnz].view(np.int32)[:] = idx[perm]
        shuffled[q][16 + 4 * cap : 16 + 4 * cap + 4 * nnz].view(F)[:] = val[perm]
    agg.fill_(7.0)
    hp.dgc_decode_merge([dev(p) for p in shuffled], agg)
    np.testing.assert_array_equal(host(agg), oracle.sparse_decode_merge(pays, n))


# ---------------------------------------------------------------- batched launches
def mixed_sizes():
    return [1728, 64, 36864, 64, 73728, 128, 4097, 1, 262144, 512, 1000003, 1000]


def test_batch_onebit_deferred(hp):
    rng = np.random.default_rng(43)
    tensors, refs = [], []
    for n in mixed_sizes():
        r0 = rng.normal(0, 1e-3, n).astype(F)
        tensors.append({"gradient": torch.zeros(n, device="cuda"), "state": dev(r0), "scale_state": torch.zeros(1, device="cuda"),
                        "compressed": payload(hp.onebit_payload_bytes(n)), "out": torch.empty(n, device="cuda")})
        refs.append(r0)
    b = hp.Batch("onebit_deferred", tensors)
    for step in range(3):
        gs = [rng.normal(0, 1e-3, t["gradient"].numel()).astype(F) for t in tensors]
        for t, g in zip(tensors, gs):
            t["gradient"].copy_(dev(g))
        b.encode()
        b.decode()
        for i, (t, g) in enumerate(zip(tensors, gs)):
            n = g.size
            got = host(t["compressed"])
            s = got[:4].view(F)[0]
            want, refs[i] = oracle.onebit_encode(g, refs[i], scale=s)
            np.testing.assert_array_equal(got, want)
            res = torch.empty(n, device="cuda")
            hp.onebit_residual(t["state"], t["scale_state"], res)
            np.testing.assert_array_equal(host(res), refs[i])
            np.testing.assert_array_equal(host(t["out"]), oracle.onebit_decode(want, n))
    b.close()


@pytest.mark.parametrize("alg", ["tbq", "onebit", "terngrad", "dgc", "graddrop"])
def test_batch_matches_oracle(hp, alg):
    rng = np.random.default_rng(42)
    tensors, refs = [], []
    for n in mixed_sizes():
        g = rng.normal(0, 10 ** rng.uniform(-4, -2), n).astype(F)
        t = {"gradient": dev(g), "out": torch.full((n,), 7.0, device="cuda")}
        ref = {"g": g, "n": n}
        if alg in ("tbq", "onebit"):
            ref["r"] = rng.normal(0, 1e-3, n).astype(F)
            t["residual"] = dev(ref["r"])
            nb = hp.tbq_payload_bytes(n) if alg == "tbq" else hp.onebit_payload_bytes(n)
        elif alg == "terngrad":
            ref["u"] = rng.random(n, dtype=F)
            t["uniform"] = dev(ref["u"])
            nb = hp.terngrad_payload_bytes(n, 512)
        elif alg == "dgc":
            ref["mom"], ref["acc"] = rng.normal(0, 1e-3, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
            t["momentum"], t["accumulator"] = dev(ref["mom"]), dev(ref["acc"])
            nb = hp.dgc_payload_bytes(n, 0.001)
        else:
            ref["acc"] = rng.normal(0, 1e-3, n).astype(F)
            t["accumulator"] = dev(ref["acc"])
            nb = hp.graddrop_payload_bytes(n, 0.01)
        t["compressed"] = payload(nb)
        tensors.append(t)
        refs.append(ref)
    ratio = 0.001 if alg == "dgc" else 0.01
    b = hp.Batch(alg, tensors, threshold=0.001, bucket=512, momentum_factor=0.9, ratio=ratio)
    b.encode()
    b.decode()
    for t, ref in zip(tensors, refs):
        n, g = ref["n"], ref["g"]
        got = host(t["compressed"])
        if alg == "tbq":
            want, r = oracle.tbq_encode(g, ref["r"], 0.001)
            np.testing.assert_array_equal(got, want)
            np.testing.assert_array_equal(host(t["residual"]), r)
            dec = oracle.tbq_decode(want, n)
        elif alg == "onebit":
            s = got[:4].view(F)[0]
            s_ref = oracle.onebit_scale(g, ref["r"])
            assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref)
            want, r = oracle.onebit_encode(g, ref["r"], scale=s)
            np.testing.assert_array_equal(got, want)
            np.testing.assert_array_equal(host(t["residual"]), r)
            dec = oracle.onebit_decode(want, n)
        elif alg == "terngrad":
            want = oracle.terngrad_encode(g, ref["u"], 512)
            np.testing.assert_array_equal(got, want)
            dec = oracle.terngrad_decode(want, n)
        elif alg == "dgc":
            want, mom, acc = oracle.dgc_encode(g, ref["mom"], ref["acc"], 0.9, ratio)
            check_sparse(got, want)
            np.testing.assert_array_equal(host(t["momentum"]), mom)
            np.testing.assert_array_equal(host(t["accumulator"]), acc)
            dec = oracle.sparse_decode(want, n)
        else:
            want, acc = oracle.graddrop_encode(g, ref["acc"], ratio)
            check_sparse(got, want)
            np.testing.assert_array_equal(host(t["accumulator"]), acc)
            dec = oracle.sparse_decode(want, n)
        np.testing.assert_array_equal(host(t["out"]), dec)
    b.close()


@pytest.mark.parametrize("alg,ratio", [("dgc", 0.001), ("graddrop", 0.01)])
def test_sparse_batch_many_steps(hp, alg, ratio):
    """A batch object is reused step after step and its workspace keeps the previous
    step's contents.  The steps below change the threshold abruptly, put a burst of
    large neighbours into one place and overflow the payload capacity (many equal large
    values); every step must still match the oracle bit for bit."""
    rng = np.random.default_rng(91)
    sizes = [1000003, 262144, 4097, 70001, 300000, 64]
    tensors, refs = [], []
    for n in sizes:
        t = {"gradient": torch.zeros(n, device="cuda"), "accumulator": torch.zeros(n, device="cuda"),
             "compressed": payload(hp.sparse_payload_bytes(n, ratio)), "out": torch.empty(n, device="cuda")}
        ref = {"acc": np.zeros(n, F)}
        if alg == "dgc":
            t["momentum"] = torch.zeros(n, device="cuda")
            ref["mom"] = np.zeros(n, F)
        tensors.append(t)
        refs.append(ref)
    b = hp.Batch(alg, tensors, momentum_factor=0.9, ratio=ratio)
    plan = ["plain", "plain", "plain", "tiny", "plain", "burst", "big", "ties", "plain", "plain"]
    for step, kind in enumerate(plan):
        for t, ref in zip(tensors, refs):
            n = t["gradient"].numel()
            scale = {"tiny": 1e-5, "big": 5e-3}.get(kind, 1e-3)
            g = rng.normal(0, scale, n).astype(F)
            if kind == "burst" and n > 5000:
                g[3000:5000] += 0.05  # 2000 neighbours far above the threshold
            if kind == "ties" and n > 5000:
                g[::7] = 0.25  # far more equal values than the payload has slots
            t["gradient"].copy_(dev(g))
            ref["g"] = g
        b.encode()
        b.decode()
        for t, ref in zip(tensors, refs):
            n = ref["g"].size
            if alg == "dgc":
                want, ref["mom"], ref["acc"] = oracle.dgc_encode(ref["g"], ref["mom"], ref["acc"], 0.9, ratio)
                np.testing.assert_array_equal(host(t["momentum"]), ref["mom"], err_msg=f"step {step} {kind} n={n}")
            else:
                want, ref["acc"] = oracle.graddrop_encode(ref["g"], ref["acc"], ratio)
            check_sparse(host(t["compressed"]), want)
            np.testing.assert_array_equal(host(t["accumulator"]), ref["acc"], err_msg=f"step {step} {kind} n={n}")
            np.testing.assert_array_equal(host(t["out"]), oracle.sparse_decode(want, n))
    b.close()


def test_terngrad_batch_decode_follows_the_header_bucket(hp):
    """A batch is created with one bucket size, and its decoder starts from it; a payload
    whose header names another bucket size must still be decoded by its header."""
    rng = np.random.default_rng(5)
    sizes = [100000, 4097, 70000]
    tensors, pays = [], []
    for k, n in enumerate(sizes):
        g = rng.normal(0, 1e-2, n).astype(F)
        u = rng.random(n, dtype=F)
        bucket = 256 if k == 1 else 512  # the middle payload disagrees with the batch
        pays.append(oracle.terngrad_encode(g, u, bucket))
        room = max(hp.terngrad_payload_bytes(n, 256), hp.terngrad_payload_bytes(n, 512))
        buf = torch.zeros(room, dtype=torch.uint8, device="cuda")
        buf[: pays[-1].size].copy_(dev(pays[-1]))
        tensors.append({"compressed": buf, "out": torch.full((n,), 7.0, device="cuda")})
    b = hp.Batch("terngrad", tensors, bucket=512)
    b.decode()
    for t, pay, n in zip(tensors, pays, sizes):
        np.testing.assert_array_equal(host(t["out"]), oracle.terngrad_decode(pay, n), err_msg=f"n={n}")
    b.close()


def make_sparse_payload(n, cap, idx, val, nnz=None):
    """A hand-made dgc/graddrop payload: header {nnz, n, cap, thr}, idx[cap], val[cap]."""
    pay = np.zeros(16 + 8 * cap, np.uint8)
    hdr = pay[:16].view(np.uint32)
    hdr[0], hdr[1], hdr[2] = (len(idx) if nnz is None else nnz), n, cap
    pay[16 : 16 + 4 * len(idx)].view(np.int32)[:] = idx
    pay[16 + 4 * cap : 16 + 4 * cap + 4 * len(val)].view(F)[:] = val
    return pay


def test_sparse_batch_decode_handmade_payloads(hp):
    """The batched sparse decode places every tile's run of pairs through tile pointers.
    Payloads made by hand: empty, one pair in a large tensor (long stretches of empty
    tiles), all slots used with the capacity a multiple of 1024, indices outside the
    tensor at both ends, a tensor shorter than a tile, and two payloads out of order
    (every tile then looks through the whole payload) between ordered ones.  Two rounds with the payloads
    exchanged between the rounds, since the batch keeps its pointers and flags."""
    rng = np.random.default_rng(123)

    def ordered(n, k):
        return np.sort(rng.choice(n, size=k, replace=False)).astype(np.int32)

    cases = []  # (n, cap, idx, nnz)
    cases.append((1000003, 4096, np.zeros(0, np.int32), None))                       # empty
    cases.append((3000000, 1024, np.array([2999999], np.int32), None))              # one pair, last element
    cases.append((3000000, 1024, np.array([0], np.int32), None))                    # one pair, first element
    cases.append((500000, 2048, ordered(500000, 2048), None))                       # every slot used
    cases.append((262144, 512, np.concatenate([[-7, -1], ordered(262144, 300), [262144, 2**31 - 1]]).astype(np.int32), None))
    cases.append((1000, 64, ordered(1000, 40), None))                               # shorter than a tile
    cases.append((700001, 8192, rng.permutation(ordered(700001, 5000)).astype(np.int32), None))  # out of order
    cases.append((700001, 8192, ordered(700001, 5000), None))
    cases.append((4097, 64, np.array([4096, 0], np.int32), None))                   # out of order, two tiles
    cases.append((900000, 1024, ordered(900000, 1024), 5000))                       # nnz in the header beyond the capacity
    tensors, pays = [], []
    for n, cap, idx, nnz in cases:
        val = rng.normal(0, 1, idx.size).astype(F)
        val[val == 0] = 1
        pays.append(make_sparse_payload(n, cap, idx, val, nnz))
        tensors.append({"compressed": dev(pays[-1]), "out": torch.full((n,), 7.0, device="cuda")})
    b = hp.Batch("dgc", tensors, ratio=0.001)
    for rnd in range(3):
        b.decode()
        for t, pay, (n, *_rest) in zip(tensors, pays, cases):
            np.testing.assert_array_equal(host(t["out"]), oracle.sparse_decode(pay, n), err_msg=f"round {rnd} n={n}")
        # same buffers, new contents: an ordered payload where a disordered one was and the other way round
        if rnd == 0:
            for k in (6, 7):
                n, cap, idx, _ = cases[k]
                idx2 = np.sort(idx) if k == 6 else rng.permutation(idx).astype(np.int32)
                val = rng.normal(0, 1, idx2.size).astype(F)
                pays[k] = make_sparse_payload(n, cap, idx2, val)
                tensors[k]["compressed"].copy_(dev(pays[k]))
        for t in tensors:
            t["out"].fill_(-3.0)
    b.close()


@pytest.mark.parametrize("alg", ["tbq", "dgc"])
def test_merge_that_only_re_encodes_leaves_the_same_payload_and_state(hp, alg):
    """A re-encoding merge may be called without an aggregate buffer (only the
    re-encoded payload is wanted): payload and state equal those of the call that also
    writes the aggregate, per tensor and through a batch; without the re-encode a
    missing aggregate is refused."""
    rng = np.random.default_rng(5)
    P, tau, ratio = 8, 0.05, 0.001
    sizes = [300001, 4097, 1048576]
    chunks_a, chunks_b = [], []
    for n in sizes:
        if alg == "tbq":
            pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(P)]
            nb = hp.tbq_payload_bytes(n)
        else:
            pays = [oracle.dgc_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), np.zeros(n, F), 0.9, ratio)[0] for _ in range(P)]
            nb = hp.dgc_payload_bytes(n, ratio)
        st = rng.normal(0, 1e-3, n).astype(F)
        dp = [dev(p) for p in pays]
        chunks_a.append({"compressed": dp, "aggregate": torch.empty(n, device="cuda"), "state": dev(st), "out_compressed": payload(nb)})
        chunks_b.append({"compressed": dp, "aggregate": None, "state": dev(st), "out_compressed": payload(nb)})
        # per tensor
        sa, sb, oa, ob = dev(st), dev(st), payload(nb), payload(nb)
        if alg == "tbq":
            hp.tbq_decode_merge(dp, torch.empty(n, device="cuda"), sa, oa, tau)
            hp.tbq_decode_merge(dp, None, sb, ob, tau)
        else:
            hp.dgc_decode_merge(dp, torch.empty(n, device="cuda"), sa, oa, ratio)
            hp.dgc_decode_merge(dp, None, sb, ob, ratio)
        if alg == "tbq":
            np.testing.assert_array_equal(host(ob), host(oa))
        else:
            check_sparse(host(ob), host(oa))
        np.testing.assert_array_equal(host(sb), host(sa))
    ba = hp.MergeBatch(alg, chunks_a, threshold=tau, ratio=ratio)
    bb = hp.MergeBatch(alg, chunks_b, threshold=tau, ratio=ratio)
    ba.run()
    bb.run()
    for ca, cb in zip(chunks_a, chunks_b):
        if alg == "tbq":
            np.testing.assert_array_equal(host(cb["out_compressed"]), host(ca["out_compressed"]))
        else:
            check_sparse(host(cb["out_compressed"]), host(ca["out_compressed"]))
        np.testing.assert_array_equal(host(cb["state"]), host(ca["state"]))
    ba.close()
    bb.close()
    with pytest.raises(TypeError):
        (hp.tbq_decode_merge if alg == "tbq" else hp.dgc_decode_merge)(chunks_a[0]["compressed"], None)


@pytest.mark.parametrize("alg", ["tbq", "dgc"])
def test_merge_batch_matches_oracle(hp, alg):
    rng = np.random.default_rng(77)
    P, tau, ratio = 8, 0.05, 0.001
    chunks, refs = [], []
    for n in [1048576, 4097, 300000]:
        if alg == "tbq":
            pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(P)]
            nb = hp.tbq_payload_bytes(n)
        else:
            pays = [oracle.dgc_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), np.zeros(n, F), 0.9, ratio)[0] for _ in range(P)]
            nb = hp.dgc_payload_bytes(n, ratio)
        st = rng.normal(0, 1e-3, n).astype(F)
        chunks.append({"compressed": [dev(p) for p in pays], "aggregate": torch.full((n,), 7.0, device="cuda"),
                       "state": dev(st), "out_compressed": payload(nb)})
        refs.append((pays, st, n))
    mb = hp.MergeBatch(alg, chunks, threshold=tau, ratio=ratio)
    mb.run()
    for c, (pays, st, n) in zip(chunks, refs):
        if alg == "tbq":
            agg, out, r = oracle.tbq_decode_merge(pays, n, st, tau)
            np.testing.assert_array_equal(host(c["aggregate"]), agg)
            np.testing.assert_array_equal(host(c["out_compressed"]), out)
            np.testing.assert_array_equal(host(c["state"]), r)
        else:
            got_agg = host(c["aggregate"])
            np.testing.assert_array_equal(got_agg, oracle.sparse_decode_merge(pays, n))  # summed in peer order
            want_out, want_acc = oracle.graddrop_encode(got_agg, st, ratio)
            check_sparse(host(c["out_compressed"]), want_out)
            np.testing.assert_array_equal(host(c["state"]), want_acc)
    mb.close()


# ---------------------------------------------------------------- error behaviour
def test_errors_are_raised_not_faulted(hp):
    g = torch.zeros(100, device="cuda")
    r = torch.zeros(100, device="cuda")
    small = torch.zeros(16, dtype=torch.uint8, device="cuda")
    with pytest.raises(hp._lib.HipressError):
        hp.tbq_encode(g, r, small, 0.05)  # payload too small
    with pytest.raises(TypeError):
        hp.tbq_encode(g.double(), r, small, 0.05)
    with pytest.raises(TypeError):
        hp.tbq_encode(g, r, torch.zeros(64, device="cuda"), 0.05)  # compressed must be uint8
    with pytest.raises(ValueError):
        hp.tbq_encode(g, r[:50], torch.zeros(64, dtype=torch.uint8, device="cuda"), 0.05)
    with pytest.raises(hp._lib.HipressError):
        hp.tbq_encode(g, r, torch.zeros(64, dtype=torch.uint8, device="cuda"), -1.0)
    with pytest.raises(hp._lib.HipressError):
        hp.terngrad_encode(g, r, torch.zeros(4096, dtype=torch.uint8, device="cuda"), 0)
    with pytest.raises(hp._lib.HipressError):
        hp.graddrop_encode(g, r, torch.zeros(4096, dtype=torch.uint8, device="cuda"), 0.0)
    ok = torch.zeros(hp.tbq_payload_bytes(100) + 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(hp._lib.HipressError):
        hp.tbq_encode(g, r, ok[1:], 0.05)  # payload not 16-byte aligned
    torch.cuda.synchronize()


def test_torch_ops_namespace(hp):
    n = 1000
    g = np.random.default_rng(5).normal(0, 0.05, n).astype(F)
    r = torch.zeros(n, device="cuda")
    pay = payload(hp.tbq_payload_bytes(n))
    torch.ops.hipress.tbq_encode(dev(g), r, pay, 0.05)
    want, want_r = oracle.tbq_encode(g, np.zeros(n, F), 0.05)
    np.testing.assert_array_equal(host(pay), want)
    out = torch.empty(n, device="cuda")
    torch.ops.hipress.TBQDecode(pay, out)
    np.testing.assert_array_equal(host(out), oracle.tbq_decode(want, n))
