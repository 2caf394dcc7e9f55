"""Seeded random configurations of every operator against the oracle: sizes that fall
anywhere relative to word, bucket, group, tile and sample boundaries, parameters over their
whole range, state carried over two steps.  The cases are fixed by the seed, so a failure
names its case and repeats.  HIPRESS_TEST_SEED=k in the environment shifts every seed by
7919*k for a sweep over other cases (the suite itself runs k = 0)."""
import os

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
F = np.float32
SHIFT = 7919 * int(os.environ.get("HIPRESS_TEST_SEED", "0"))


def seeded(seed):
    return np.random.default_rng(seed + SHIFT)


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


def payload(nbytes):
    return torch.full((nbytes,), 0xAB, dtype=torch.uint8, device="cuda")


def sizes(rng, count, top=400_000):
    """Sizes spread over the orders of magnitude, some of them right at a boundary."""
    out = []
    for _ in range(count):
        n = int(10 ** rng.uniform(0, np.log10(top)))
        if rng.random() < 0.4:
            base = int(rng.choice([16, 32, 64, 512, 1024, 4096, 65536, 262144]))
            n = max(1, base * int(rng.integers(1, 4)) + int(rng.integers(-2, 3)))
        out.append(n)
    return out


def check_sparse(got_pay, want_pay, where):
    g, w = oracle.sparse_unpack(got_pay), oracle.sparse_unpack(want_pay)
    assert g[:3] == w[:3] and g[3].view(np.uint32) == w[3].view(np.uint32), (where, g[:4], w[:4])
    np.testing.assert_array_equal(g[4], w[4], err_msg=where)
    np.testing.assert_array_equal(g[5], w[5], err_msg=where)


def test_dense_quantisers_random_cases(hp):
    rng = seeded(2024)
    for case, n in enumerate(sizes(rng, 150)):
        sigma = 10 ** rng.uniform(-4, 0)
        tau = float(F(sigma * rng.uniform(0.2, 4.0)))
        bucket = int(rng.choice([256, 512, 1024, 16, 100, 777, 4096]))
        where = f"case {case}: n={n} sigma={sigma:.3g} tau={tau:.3g} bucket={bucket}"
        r_t, r_o = rng.normal(0, sigma, n).astype(F), None
        r_o = r_t.copy()
        rt_gpu, ro_gpu = dev(r_t), dev(r_o)
        for step in range(2):
            g, u = rng.normal(0, sigma, n).astype(F), rng.random(n, dtype=F)
            pay = payload(hp.tbq_payload_bytes(n))
            hp.tbq_encode(dev(g), rt_gpu, pay, tau)
            want, r_t = oracle.tbq_encode(g, r_t, tau)
            np.testing.assert_array_equal(host(pay), want, err_msg="tbq " + where)
            np.testing.assert_array_equal(host(rt_gpu), r_t, err_msg="tbq residual " + where)
            out = torch.full((n,), 7.0, device="cuda")
            hp.tbq_decode(pay, out)
            np.testing.assert_array_equal(host(out), oracle.tbq_decode(want, n), err_msg="tbq decode " + where)
            pay = payload(hp.onebit_payload_bytes(n))
            hp.onebit_encode(dev(g), ro_gpu, pay)
            got = host(pay)
            s = got[:4].view(F)[0]
            s_ref = oracle.onebit_scale(g, r_o)
            assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref), "onebit scale " + where
            want, r_o = oracle.onebit_encode(g, r_o, scale=s)
            np.testing.assert_array_equal(got, want, err_msg="onebit " + where)
            np.testing.assert_array_equal(host(ro_gpu), r_o, err_msg="onebit residual " + where)
            pay = payload(hp.terngrad_payload_bytes(n, bucket))
            hp.terngrad_encode(dev(g), dev(u), pay, bucket)
            want = oracle.terngrad_encode(g, u, bucket)
            np.testing.assert_array_equal(host(pay), want, err_msg="terngrad " + where)
            hp.terngrad_decode(pay, out)
            np.testing.assert_array_equal(host(out), oracle.terngrad_decode(want, n), err_msg="terngrad decode " + where)


def test_sparsifiers_random_cases(hp):
    rng = seeded(2025)
    for case, n in enumerate(sizes(rng, 150, top=1_500_000)):
        ratio = float(10 ** rng.uniform(-3.3, -0.5))
        m = float(F(rng.uniform(0.0, 0.99)))
        heavy = rng.random() < 0.3  # many equal magnitudes: ties at the threshold, overflow of the slots
        where = f"case {case}: n={n} ratio={ratio:.4g} m={m:.3g} heavy={heavy}"
        mom_ref, acc_ref, gacc_ref = np.zeros(n, F), np.zeros(n, F), np.zeros(n, F)
        mom, acc, gacc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
        for step in range(2):
            g = rng.normal(0, 1e-3, n).astype(F)
            if heavy:
                g = (np.round(g * 2000) / 2000).astype(F)
            pay = payload(hp.sparse_payload_bytes(n, ratio))
            hp.dgc_encode(dev(g), mom, acc, pay, m, ratio)
            want, mom_ref, acc_ref = oracle.dgc_encode(g, mom_ref, acc_ref, m, ratio)
            check_sparse(host(pay), want, "dgc " + where)
            np.testing.assert_array_equal(host(mom), mom_ref, err_msg="dgc momentum " + where)
            np.testing.assert_array_equal(host(acc), acc_ref, err_msg="dgc accumulator " + where)
            out = torch.full((n,), 7.0, device="cuda")
            hp.dgc_decode(pay, out)
            np.testing.assert_array_equal(host(out), oracle.sparse_decode(want, n), err_msg="decode " + where)
            pay = payload(hp.sparse_payload_bytes(n, ratio))
            hp.graddrop_encode(dev(g), gacc, pay, ratio)
            want, gacc_ref = oracle.graddrop_encode(g, gacc_ref, ratio)
            check_sparse(host(pay), want, "graddrop " + where)
            np.testing.assert_array_equal(host(gacc), gacc_ref, err_msg="graddrop accumulator " + where)


def test_merges_random_cases(hp):
    rng = seeded(2026)
    for case, n in enumerate(sizes(rng, 80, top=1_200_000)):
        P = int(rng.integers(1, 17))
        tau = float(F(rng.uniform(0.01, 0.1)))
        ratio = float(10 ** rng.uniform(-3, -1.3))
        where = f"case {case}: n={n} peers={P} tau={tau:.3g} ratio={ratio:.3g}"
        z = np.zeros(n, F)
        tp = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), z, tau)[0] for _ in range(P)]
        r0 = rng.normal(0, 0.02, n).astype(F)
        agg, res, outp = torch.full((n,), 7.0, device="cuda"), dev(r0), payload(hp.tbq_payload_bytes(n))
        hp.tbq_decode_merge([dev(p) for p in tp], agg, res, outp, tau)
        want_agg, want_out, want_r = oracle.tbq_decode_merge(tp, n, r0, tau)
        np.testing.assert_array_equal(host(agg), want_agg, err_msg="tbq merge " + where)
        np.testing.assert_array_equal(host(outp), want_out, err_msg="tbq merge payload " + where)
        np.testing.assert_array_equal(host(res), want_r, err_msg="tbq merge residual " + where)
        sp = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), z, ratio)[0] for _ in range(P)]
        a0 = rng.normal(0, 1e-4, n).astype(F)
        agg, acc, outp = torch.full((n,), 7.0, device="cuda"), dev(a0), payload(hp.sparse_payload_bytes(n, ratio))
        hp.dgc_decode_merge([dev(p) for p in sp], agg, acc, outp, ratio)
        want_agg, want_out, want_acc = oracle.sparse_decode_merge(sp, n, a0, ratio)
        np.testing.assert_array_equal(host(agg), want_agg, err_msg="sparse merge " + where)
        check_sparse(host(outp), want_out, "sparse merge payload " + where)
        np.testing.assert_array_equal(host(acc), want_acc, err_msg="sparse merge accumulator " + where)


def test_batches_of_random_tensor_tables(hp):
    rng = seeded(2027)
    for alg in ("tbq", "terngrad", "dgc", "graddrop"):
        for table in range(8):
            ns = sizes(rng, int(rng.integers(2, 25)), top=600_000)
            ratio = 0.01 if alg == "graddrop" else 0.001
            ts, data = [], []
            for n in ns:
                g, u = rng.normal(0, 0.02 if alg == "tbq" else 1e-3, n).astype(F), rng.random(n, dtype=F)
                nbytes = {"tbq": hp.tbq_payload_bytes(n), "terngrad": hp.terngrad_payload_bytes(n, 512),
                          "dgc": hp.sparse_payload_bytes(n, ratio), "graddrop": hp.sparse_payload_bytes(n, ratio)}[alg]
                t = {"gradient": dev(g), "out": torch.full((n,), 7.0, device="cuda"), "compressed": payload(nbytes)}
                if alg == "tbq":
                    t["residual"] = torch.zeros(n, device="cuda")
                elif alg == "terngrad":
                    t["uniform"] = dev(u)
                elif alg == "dgc":
                    t["momentum"], t["accumulator"] = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
                else:
                    t["accumulator"] = torch.zeros(n, device="cuda")
                ts.append(t)
                data.append((g, u))
            b = hp.Batch(alg, ts, threshold=0.05, bucket=512, momentum_factor=0.9, ratio=ratio)
            b.encode()
            b.decode()
            for i, (t, n, (g, u)) in enumerate(zip(ts, ns, data)):
                where = f"{alg} table {table} tensor {i} n={n}"
                z = np.zeros(n, F)
                got = host(t["compressed"])
                if alg == "tbq":
                    want = oracle.tbq_encode(g, z, 0.05)[0]
                    np.testing.assert_array_equal(got, want, err_msg=where)
                    ref = oracle.tbq_decode(want, n)
                elif alg == "terngrad":
                    want = oracle.terngrad_encode(g, u, 512)
                    np.testing.assert_array_equal(got, want, err_msg=where)
                    ref = oracle.terngrad_decode(want, n)
                elif alg == "dgc":
                    want = oracle.dgc_encode(g, z, z, 0.9, ratio)[0]
                    check_sparse(got, want, where)
                    ref = oracle.sparse_decode(want, n)
                else:
                    want = oracle.graddrop_encode(g, z, ratio)[0]
                    check_sparse(got, want, where)
                    ref = oracle.sparse_decode(want, n)
                np.testing.assert_array_equal(host(t["out"]), ref, err_msg="decode " + where)
            b.close()


def test_views_buckets_and_dense_merges_random_cases(hp):
    """What the cases above hold fixed: fp32 tensors that start 0-3 elements into their
    allocation (4-byte aligned only), TernGrad bucket sizes of any value, dense merges of
    1-16 peers with and without a local gradient (TernGrad peers partly with bucket sizes of
    their own), and the min/max quantiser at every bit width."""
    rng = seeded(2028)
    for case, n in enumerate(sizes(rng, 60, top=700_000)):
        bucket = int(rng.choice([int(rng.integers(1, 6000)), 256, 512, 768, 1024, 4096, 8192,
                                 int(rng.integers(6000, 200000))]))
        P = int(rng.integers(1, 17))
        off = int(rng.integers(0, 4))
        where = f"case {case}: n={n} bucket={bucket} peers={P} offset={off}"

        def view(a):
            t = torch.empty(n + off, device="cuda")
            v = t[off:]
            v.copy_(torch.from_numpy(np.ascontiguousarray(a, dtype=F)))
            return v

        g, u = rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F)
        pay = payload(hp.terngrad_payload_bytes(n, bucket))
        hp.terngrad_encode(view(g), view(u), pay, bucket)
        want = oracle.terngrad_encode(g, u, bucket)
        np.testing.assert_array_equal(host(pay), want, err_msg="terngrad " + where)
        out = view(np.full(n, 7, F))
        hp.terngrad_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.terngrad_decode(want, n), err_msg="terngrad decode " + where)

        pays = []
        for _ in range(P):
            b = bucket if rng.random() < 0.8 else int(rng.integers(1, 3000))
            pays.append(oracle.terngrad_encode(rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F), b))
        local = rng.normal(0, 1e-3, n).astype(F) if rng.random() < 0.5 else None
        loc = (lambda: None if local is None else view(local))
        agg = view(np.full(n, 7, F))
        hp.terngrad_decode_merge([dev(p) for p in pays], agg, local=loc())
        np.testing.assert_array_equal(host(agg), oracle.terngrad_decode_merge(pays, n, local=local),
                                      err_msg="terngrad merge " + where)
        z = np.zeros(n, F)
        pays = [oracle.onebit_encode(rng.normal(0, 10 ** rng.uniform(-4, 0), n).astype(F), z)[0] for _ in range(P)]
        agg = view(np.full(n, 7, F))
        hp.onebit_decode_merge([dev(p) for p in pays], agg, local=loc())
        np.testing.assert_array_equal(host(agg), oracle.onebit_decode_merge(pays, n, local=local),
                                      err_msg="onebit merge " + where)
        tau = float(F(rng.uniform(0.01, 0.1)))
        pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), z, tau)[0] for _ in range(P)]
        agg = view(np.full(n, 7, F))
        hp.tbq_decode_merge([dev(p) for p in pays], agg, local=loc())
        np.testing.assert_array_equal(host(agg), oracle.tbq_decode_merge(pays, n, None, 0.0, local=local),
                                      err_msg="tbq merge " + where)

        b = int(rng.choice([1, 2, 4, 8]))
        pay = payload(hp.compll_payload_bytes(n, b))
        hp.compll_terngrad_encode(view(g), view(u), pay, b)
        want = oracle.compll_encode(g, u, b)
        np.testing.assert_array_equal(host(pay), want, err_msg=f"min/max quantiser b={b} " + where)
        count = hp.compll_decoded_count(n, b)
        out = torch.full((count + off + 1,), 7.0, device="cuda")[off:off + count]
        hp.compll_terngrad_decode(pay, out)
        ref = oracle.compll_decode(want, count)
        assert len(ref) == count, (len(ref), count, where)
        np.testing.assert_array_equal(host(out), ref, err_msg=f"min/max decode b={b} " + where)

        ratio = float(10 ** rng.uniform(-3, -1))
        m = float(F(rng.uniform(0.0, 0.99)))
        mom0, acc0 = rng.normal(0, 1e-3, n).astype(F), rng.normal(0, 1e-3, n).astype(F)
        mom, acc = view(mom0), view(acc0)
        pay = payload(hp.sparse_payload_bytes(n, ratio))
        hp.dgc_encode(view(g), mom, acc, pay, m, ratio)
        want, mom_ref, acc_ref = oracle.dgc_encode(g, mom0, acc0, m, ratio)
        check_sparse(host(pay), want, "dgc " + where)
        np.testing.assert_array_equal(host(mom), mom_ref, err_msg="dgc momentum " + where)
        np.testing.assert_array_equal(host(acc), acc_ref, err_msg="dgc accumulator " + where)
        out = view(np.full(n, 7, F))
        hp.dgc_decode(pay, out)
        np.testing.assert_array_equal(host(out), oracle.sparse_decode(want, n), err_msg="sparse decode " + where)
        sp = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), z, ratio)[0] for _ in range(P)]
        agg, acc, outp = view(np.full(n, 7, F)), view(acc0), payload(hp.sparse_payload_bytes(n, ratio))
        hp.dgc_decode_merge([dev(p) for p in sp], agg, acc, outp, ratio, local=loc())
        want_agg, want_out, want_acc = oracle.sparse_decode_merge(sp, n, acc0, ratio, local=local)
        np.testing.assert_array_equal(host(agg), want_agg, err_msg="sparse merge " + where)
        check_sparse(host(outp), want_out, "sparse merge payload " + where)
        np.testing.assert_array_equal(host(acc), want_acc, err_msg="sparse merge accumulator " + where)


def test_seeded_quantisers_random_cases(hp):
    """The encoders that draw their own noise, at random sizes, bucket sizes, bit widths, seeds
    and view offsets, per tensor and as a table: equal to the oracle run on oracle.uniform_draws."""
    rng = seeded(2029)
    for case, n in enumerate(sizes(rng, 60, top=700_000)):
        bucket = int(rng.choice([int(rng.integers(1, 6000)), 256, 512, 1024, 4096, int(rng.integers(6000, 200000))]))
        seed, off, b = int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 4)), int(rng.choice([1, 2, 4, 8]))
        where = f"case {case}: n={n} bucket={bucket} seed={seed} offset={off} b={b}"
        g = rng.normal(0, 1e-3, n).astype(F)
        t = torch.empty(n + off, device="cuda")
        gv = t[off:]
        gv.copy_(torch.from_numpy(g))
        u = oracle.uniform_draws(seed, n)
        pay = payload(hp.terngrad_payload_bytes(n, bucket))
        hp.terngrad_encode_seeded(gv, pay, bucket, seed)
        np.testing.assert_array_equal(host(pay), oracle.terngrad_encode(g, u, bucket), err_msg="terngrad " + where)
        pay = payload(hp.compll_payload_bytes(n, b))
        hp.compll_terngrad_encode_seeded(gv, pay, b, seed)
        np.testing.assert_array_equal(host(pay), oracle.compll_encode(g, u, b), err_msg="min/max quantiser " + where)
    for table in range(6):
        ns = sizes(rng, int(rng.integers(2, 25)), top=400_000)
        bucket, seed = int(rng.choice([512, 100, 777, 5000])), int(rng.integers(0, 2 ** 63))
        gs = [rng.normal(0, 1e-3, n).astype(F) for n in ns]
        ts = [{"gradient": dev(g), "compressed": payload(hp.terngrad_payload_bytes(g.size, bucket))} for g in gs]
        bt = hp.Batch("terngrad", ts, bucket=bucket)
        bt.encode(seed=seed)
        for k, (tt, g) in enumerate(zip(ts, gs)):
            want = oracle.terngrad_encode(g, oracle.uniform_draws(seed, g.size, k), bucket)
            np.testing.assert_array_equal(host(tt["compressed"]), want, err_msg=f"table {table} tensor {k} n={g.size} bucket={bucket}")
        bt.close()


SPECIALS = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, -3e-42, 1.4e-45, np.finfo(F).max, -np.finfo(F).max,
                     np.finfo(F).tiny, -np.finfo(F).tiny], F)


def feq(got, want, msg=""):
    """Equal as floats, NaN matching NaN, and the sign of zero respected."""
    np.testing.assert_array_equal(got, want, err_msg=msg)
    z = want == 0
    np.testing.assert_array_equal(np.signbit(got[z]), np.signbit(want[z]), err_msg=msg + " (sign of zero)")


def sprinkled(rng, n, sigma):
    """N(0, sigma) data with special values at random places (about one in fifty, and the ends)."""
    g = rng.normal(0, sigma, n).astype(F)
    k = max(1, n // 50)
    at = np.concatenate([rng.integers(0, n, k), [0, n - 1]])
    g[at] = rng.choice(SPECIALS, at.size)
    return g


def test_special_values_random_cases(hp):
    """NaN, infinities, signed zeros, denormals and FLT_MAX at random places of tensors of random
    sizes, through the encoders that have no per-tensor sum (TBQ, TernGrad at any bucket size,
    DGC, GradDrop), their decoders and the merges, state carried over two steps."""
    rng = seeded(2030)
    for case, n in enumerate(sizes(rng, 50, top=500_000)):
        bucket = int(rng.choice([int(rng.integers(1, 6000)), 256, 512, 1024, 4096, int(rng.integers(6000, 100000))]))
        ratio, P = float(10 ** rng.uniform(-3, -1.5)), int(rng.integers(1, 9))
        where = f"case {case}: n={n} bucket={bucket} ratio={ratio:.3g} peers={P}"
        r_ref, mom_ref, acc_ref, gacc_ref = sprinkled(rng, n, 0.02), np.zeros(n, F), np.zeros(n, F), np.zeros(n, F)
        r, mom, acc, gacc = dev(r_ref), dev(mom_ref), dev(acc_ref), dev(gacc_ref)
        out = torch.full((n,), 7.0, device="cuda")
        for step in range(2):
            g, u = sprinkled(rng, n, 0.02), rng.random(n, dtype=F)
            pay = payload(hp.tbq_payload_bytes(n))
            hp.tbq_encode(dev(g), r, pay, 0.05)
            want, r_ref = oracle.tbq_encode(g, r_ref, 0.05)
            np.testing.assert_array_equal(host(pay), want, err_msg="tbq " + where)
            feq(host(r), r_ref, "tbq residual " + where)
            hp.tbq_decode(pay, out)
            feq(host(out), oracle.tbq_decode(want, n), "tbq decode " + where)
            pay = payload(hp.terngrad_payload_bytes(n, bucket))
            hp.terngrad_encode(dev(g), dev(u), pay, bucket)
            want = oracle.terngrad_encode(g, u, bucket)
            got, nb = host(pay), (n + bucket - 1) // bucket
            feq(got[16:16 + 4 * nb].view(F), want[16:16 + 4 * nb].view(F), "terngrad scales " + where)
            np.testing.assert_array_equal(got[:16], want[:16], err_msg="terngrad header " + where)
            off = 16 + oracle.terngrad_scale_bytes(n, bucket)
            np.testing.assert_array_equal(got[off:], want[off:], err_msg="terngrad codes " + where)
            hp.terngrad_decode(pay, out)
            feq(host(out), oracle.terngrad_decode(want, n), "terngrad decode " + where)
            gs = sprinkled(rng, n, 1e-3)
            pay = payload(hp.sparse_payload_bytes(n, ratio))
            hp.dgc_encode(dev(gs), mom, acc, pay, 0.9, ratio)
            want, mom_ref, acc_ref = oracle.dgc_encode(gs, mom_ref, acc_ref, 0.9, ratio)
            gp, wp = oracle.sparse_unpack(host(pay)), oracle.sparse_unpack(want)
            assert gp[:3] == wp[:3] and gp[3].view(np.uint32) == wp[3].view(np.uint32), ("dgc " + where, gp[:4], wp[:4])
            np.testing.assert_array_equal(gp[4], wp[4], err_msg="dgc indices " + where)
            feq(gp[5], wp[5], "dgc values " + where)
            feq(host(mom), mom_ref, "dgc momentum " + where)
            feq(host(acc), acc_ref, "dgc accumulator " + where)
            hp.dgc_decode(pay, out)
            feq(host(out), oracle.sparse_decode(want, n), "sparse decode " + where)
            pay = payload(hp.sparse_payload_bytes(n, ratio))
            hp.graddrop_encode(dev(gs), gacc, pay, ratio)
            want, gacc_ref = oracle.graddrop_encode(gs, gacc_ref, ratio)
            gp, wp = oracle.sparse_unpack(host(pay)), oracle.sparse_unpack(want)
            assert gp[:3] == wp[:3] and gp[3].view(np.uint32) == wp[3].view(np.uint32), ("graddrop " + where, gp[:4], wp[:4])
            np.testing.assert_array_equal(gp[4], wp[4], err_msg="graddrop indices " + where)
            feq(gp[5], wp[5], "graddrop values " + where)
            feq(host(gacc), gacc_ref, "graddrop accumulator " + where)
        # merges of peers that carry such values
        z = np.zeros(n, F)
        tp = [oracle.tbq_encode(sprinkled(rng, n, 0.04), z, 0.05)[0] for _ in range(P)]
        r0 = sprinkled(rng, n, 0.02)
        agg, res, outp = torch.full((n,), 7.0, device="cuda"), dev(r0), payload(hp.tbq_payload_bytes(n))
        hp.tbq_decode_merge([dev(p) for p in tp], agg, res, outp, 0.05)
        want_agg, want_out, want_r = oracle.tbq_decode_merge(tp, n, r0, 0.05)
        feq(host(agg), want_agg, "tbq merge " + where)
        np.testing.assert_array_equal(host(outp), want_out, err_msg="tbq merge payload " + where)
        feq(host(res), want_r, "tbq merge residual " + where)
        tg = [oracle.terngrad_encode(sprinkled(rng, n, 1e-3), rng.random(n, dtype=F), bucket) for _ in range(P)]
        hp.terngrad_decode_merge([dev(p) for p in tg], agg)
        feq(host(agg), oracle.terngrad_decode_merge(tg, n), "terngrad merge " + where)
        sp = [oracle.graddrop_encode(sprinkled(rng, n, 1e-3), z, ratio)[0] for _ in range(P)]
        a0 = sprinkled(rng, n, 1e-4)
        acc2, outp = dev(a0), payload(hp.sparse_payload_bytes(n, ratio))
        hp.dgc_decode_merge([dev(p) for p in sp], agg, acc2, outp, ratio)
        want_agg, want_out, want_acc = oracle.sparse_decode_merge(sp, n, a0, ratio)
        feq(host(agg), want_agg, "sparse merge " + where)
        gp, wp = oracle.sparse_unpack(host(outp)), oracle.sparse_unpack(want_out)
        assert gp[:3] == wp[:3] and gp[3].view(np.uint32) == wp[3].view(np.uint32), ("sparse merge payload " + where, gp[:4], wp[:4])
        np.testing.assert_array_equal(gp[4], wp[4], err_msg="sparse merge indices " + where)
        feq(gp[5], wp[5], "sparse merge values " + where)
        feq(host(acc2), want_acc, "sparse merge accumulator " + where)


def test_merge_batches_of_random_chunk_tables(hp):
    """MergeBatch over tables of chunks of random sizes: every dense algorithm and the sparse
    merge, 1-16 peers, with and without the re-encode, some chunks starting from a local
    gradient, some re-encoding chunks without an aggregate buffer, run twice on the same table."""
    rng = seeded(2031)
    for table in range(10):
        alg = ("tbq", "onebit", "terngrad", "dgc")[table % 4]
        P = int(rng.integers(1, 17))
        reenc = alg in ("tbq", "dgc") and rng.random() < 0.7
        tau, ratio = float(F(rng.uniform(0.01, 0.1))), float(10 ** rng.uniform(-3, -1.5))
        bucket = int(rng.choice([512, 256, 100, 3000, 5000]))
        ns = sizes(rng, int(rng.integers(2, 14)), top=600_000)
        chunks, pays_all, locals_, states = [], [], [], []
        z = lambda n: np.zeros(n, F)
        for n in ns:
            if alg == "tbq":
                pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), z(n), tau)[0] for _ in range(P)]
            elif alg == "onebit":
                pays = [oracle.onebit_encode(rng.normal(0, 1e-2, n).astype(F), z(n))[0] for _ in range(P)]
            elif alg == "terngrad":
                pays = [oracle.terngrad_encode(rng.normal(0, 1e-3, n).astype(F), rng.random(n, dtype=F), bucket) for _ in range(P)]
            else:
                pays = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), z(n), ratio)[0] for _ in range(P)]
            local = rng.normal(0, 1e-2, n).astype(F) if rng.random() < 0.4 else None
            st = rng.normal(0, 1e-3, n).astype(F)
            c = {"compressed": [dev(p) for p in pays]}
            if not (reenc and rng.random() < 0.3):
                c["aggregate"] = torch.full((n,), 7.0, device="cuda")
            else:
                c["aggregate"] = None
            if reenc:
                nb = hp.tbq_payload_bytes(n) if alg == "tbq" else hp.sparse_payload_bytes(n, ratio)
                c["state"], c["out_compressed"] = dev(st), payload(nb)
            if local is not None:
                c["local"] = dev(local)
            chunks.append(c); pays_all.append(pays); locals_.append(local); states.append(st)
        mb = hp.MergeBatch(alg, chunks, threshold=tau, bucket=bucket, ratio=ratio)
        for rnd in range(2):
            mb.run()
            for k, (c, n, pays, local) in enumerate(zip(chunks, ns, pays_all, locals_)):
                where = f"table {table} ({alg}, {P} peers, re-encode {reenc}) round {rnd} chunk {k} n={n}"
                if alg == "tbq":
                    want = oracle.tbq_decode_merge(pays, n, states[k] if reenc else None, tau if reenc else 0.0, local=local)
                elif alg == "onebit":
                    want = oracle.onebit_decode_merge(pays, n, local=local)
                elif alg == "terngrad":
                    want = oracle.terngrad_decode_merge(pays, n, local=local)
                else:
                    want = oracle.sparse_decode_merge(pays, n, states[k] if reenc else None, ratio if reenc else 0.0, local=local)
                agg, outp, st = want if reenc else (want, None, None)
                if c["aggregate"] is not None:
                    np.testing.assert_array_equal(host(c["aggregate"]), agg, err_msg="aggregate " + where)
                if reenc:
                    if alg == "tbq":
                        np.testing.assert_array_equal(host(c["out_compressed"]), outp, err_msg="payload " + where)
                    else:
                        check_sparse(host(c["out_compressed"]), outp, "payload " + where)
                    np.testing.assert_array_equal(host(c["state"]), st, err_msg="state " + where)
                    states[k] = st  # the next round starts from the state this one left
        mb.close()
