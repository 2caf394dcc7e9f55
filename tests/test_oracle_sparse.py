"""Pins the oracle's DGC / GradDrop sparsifiers and the decode-and-merge step:
thresholds against numpy order statistics of the stated sample, selected sets
by brute force in Python, the conservation identity, momentum masking, the
overflow rule, and merges against sums of single decodes.  The reference holds
no source or fixture for these operators."""
import numpy as np
import pytest

import oracle

F = np.float32


def brute_select(a, ratio):
    """Pure-Python statement of the selection rule on an accumulated tensor."""
    n = a.size
    S = 100 if n >= 262144 else 1
    ns = n // S
    cap = oracle.sparse_capacity(n, ratio)
    if ns == 0:
        return [], F(0), cap
    sample = np.abs(a[[j * S + S // 2 for j in range(ns)]])
    k = max(1, int(np.ceil(ratio * ns)))
    thr = np.sort(sample)[::-1][k - 1]
    mag = np.abs(a)
    sel = [i for i in range(n) if mag[i] >= thr and mag[i] > 0]
    if len(sel) > cap:
        thr = np.sort(mag)[::-1][cap - 1]
        above = [i for i in range(n) if mag[i] > thr]
        ties = [i for i in range(n) if mag[i] == thr][: cap - len(above)]
        sel = sorted(above + ties)
    return sel, F(thr), cap


def test_capacity_and_sizes():
    assert oracle.sparse_capacity(10, 0.001) == 64
    assert oracle.sparse_capacity(1000, 0.5) == 1024  # min(n, 2000) = 1000 -> round up to 64s
    assert oracle.sparse_capacity(1 << 20, 0.001) == 4224  # ceil(4194.304)=4195 -> 4224
    assert oracle.sparse_payload_bytes(1 << 20, 0.001) == 16 + 8 * 4224
    assert oracle.sparse_sample_stride(262143) == 1 and oracle.sparse_sample_stride(262144) == 100
    assert oracle.sparse_sample_k(262144, 0.001) == 3  # ceil(0.001*2621)
    assert oracle.sparse_sample_k(64, 0.001) == 1


def test_graddrop_hand_kat():
    # n=8, ratio 0.25 -> sample = whole tensor, k = 2, threshold = 2nd largest |acc'|
    g = np.array([0.5, -3.0, 0.25, 2.0, -2.0, 0.0, 1.0, -0.1], dtype=F)
    acc = np.array([0.0, 1.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0], dtype=F)
    # acc' = [.5,-2,.25,2,-2,0,1,-.1]; |.| sorted desc: 2,2,2,1.. -> thr = 2 -> ties all selected
    pay, acc2 = oracle.graddrop_encode(g, acc, 0.25)
    nnz, n, cap, thr, idx, val = oracle.sparse_unpack(pay)
    assert (nnz, n, cap) == (3, 8, 64) and thr == F(2.0)
    np.testing.assert_array_equal(idx, [1, 3, 4])
    np.testing.assert_array_equal(val, np.array([-2.0, 2.0, -2.0], dtype=F))
    np.testing.assert_array_equal(acc2, np.array([0.5, 0, 0.25, 0, 0, 0, 1.0, -0.1], dtype=F))
    np.testing.assert_array_equal(
        oracle.sparse_decode(pay, 8), np.array([0, -2.0, 0, 2.0, -2.0, 0, 0, 0], dtype=F)
    )


def test_dgc_hand_kat_momentum_and_masking():
    g = np.array([1.0, 0.5, -4.0, 0.25], dtype=F)
    mom = np.array([1.0, -1.0, 0.0, 2.0], dtype=F)
    acc = np.array([0.0, 3.0, 0.5, 0.0], dtype=F)
    # mom' = .5*mom+g = [1.5, 0, -4, 1.25]; acc' = [1.5, 3, -3.5, 1.25]; k=ceil(.25*4)=1 -> thr 3.5
    pay, mom2, acc2 = oracle.dgc_encode(g, mom, acc, 0.5, 0.25)
    nnz, n, cap, thr, idx, val = oracle.sparse_unpack(pay)
    assert nnz == 1 and thr == F(3.5)
    np.testing.assert_array_equal(idx, [2])
    np.testing.assert_array_equal(val, np.array([-3.5], dtype=F))
    np.testing.assert_array_equal(mom2, np.array([1.5, 0.0, 0.0, 1.25], dtype=F))
    np.testing.assert_array_equal(acc2, np.array([1.5, 3.0, 0.0, 1.25], dtype=F))


def test_dgc_momentum_is_two_roundings_not_fma():
    # m*mom is inexact; an fma would keep the low bits and give a different sum
    m, mo, g = F(0.9), F(1.0000001), F(-0.9)
    prod = F(m * mo)
    want = F(prod + g)
    fma = F(np.float64(m) * np.float64(mo) + np.float64(g))
    assert want != fma  # the case distinguishes the two
    # a second, larger element takes the single selected slot so element 0 is not masked
    _, mom2, _ = oracle.dgc_encode(
        np.array([g, 100.0], dtype=F), np.array([mo, 0.0], dtype=F), np.zeros(2, F), m, 0.5
    )
    assert mom2[0] == want and mom2[1] == 0


@pytest.mark.parametrize("n,ratio", [(1, 0.001), (63, 0.01), (1000, 0.001), (5000, 0.01), (262143, 0.001), (262144, 0.001), (300001, 0.01)])
def test_graddrop_against_brute_force(n, ratio):
    rng = np.random.default_rng(n)
    g = rng.normal(0, 1e-3, n).astype(F)
    acc = rng.normal(0, 1e-3, n).astype(F)
    a = (acc + g).astype(F)
    sel, thr, cap = brute_select(a, ratio)
    pay, acc2 = oracle.graddrop_encode(g, acc, ratio)
    nnz, n_, cap_, thr_, idx, val = oracle.sparse_unpack(pay)
    assert (n_, cap_) == (n, cap) and thr_ == thr
    assert nnz == len(sel)
    np.testing.assert_array_equal(idx, sel)
    assert (np.diff(idx) > 0).all()
    np.testing.assert_array_equal(val, a[sel])
    # conservation: what was sent plus what stayed is exactly acc'
    dec = oracle.sparse_decode(pay, n)
    np.testing.assert_array_equal(np.where(dec != 0, dec, acc2), a)
    assert not acc2[sel].any()
    # independent check of the threshold: numpy partition on the stated sample
    S = 100 if n >= 262144 else 1
    samp = np.abs(a[S // 2 :: S][: n // S])
    k = max(1, int(np.ceil(ratio * (n // S))))
    assert oracle.sparse_threshold(a, ratio) == np.partition(samp, samp.size - k)[samp.size - k]


def test_dgc_against_brute_force_three_steps():
    n, m, ratio = 70000, F(0.9), 0.001
    rng = np.random.default_rng(3)
    mom = np.zeros(n, F)
    acc = np.zeros(n, F)
    for step in range(3):
        g = rng.normal(0, 1e-3, n).astype(F)
        mom_want = (F(m) * mom).astype(F) + g
        a = (acc + mom_want).astype(F)
        sel, thr, cap = brute_select(a, ratio)
        pay, mom, acc = oracle.dgc_encode(g, mom, acc, m, ratio)
        nnz, _, _, thr_, idx, val = oracle.sparse_unpack(pay)
        assert thr_ == thr
        np.testing.assert_array_equal(idx, sel)
        np.testing.assert_array_equal(val, a[sel])
        mom_want[sel] = 0
        a[sel] = 0
        np.testing.assert_array_equal(mom, mom_want)
        np.testing.assert_array_equal(acc, a)


def test_overflow_ties_take_lowest_indices():
    n = 1000
    g = np.full(n, 0.5, F)
    pay, acc2 = oracle.graddrop_encode(g, np.zeros(n, F), 0.001)
    nnz, _, cap, thr, idx, val = oracle.sparse_unpack(pay)
    assert cap == 64 and nnz == 64 and thr == F(0.5)
    np.testing.assert_array_equal(idx, np.arange(64))
    assert (acc2[:64] == 0).all() and (acc2[64:] == F(0.5)).all()


def test_overflow_rethresholds_on_whole_tensor():
    # sample positions (j*100+50) hold small values, everything else is large:
    # the sampled threshold admits far more than capacity
    n = 262144
    rng = np.random.default_rng(11)
    a = rng.uniform(1.0, 2.0, n).astype(F) * rng.choice([-1, 1], n).astype(F)
    a[50::100] = rng.uniform(0.001, 0.002, a[50::100].size).astype(F)
    sel, thr, cap = brute_select(a, 0.001)
    assert len(sel) == cap
    pay, acc2 = oracle.graddrop_encode(a, np.zeros(n, F), 0.001)
    nnz, _, cap_, thr_, idx, val = oracle.sparse_unpack(pay)
    assert nnz == cap == cap_ and thr_ == thr
    assert thr_ == np.sort(np.abs(a))[::-1][cap - 1]
    np.testing.assert_array_equal(idx, sel)


def test_all_zero_tensor_selects_nothing():
    pay, acc2 = oracle.graddrop_encode(np.zeros(500, F), np.zeros(500, F), 0.01)
    nnz, _, _, thr, idx, _ = oracle.sparse_unpack(pay)
    assert nnz == 0 and thr == 0 and idx.size == 0
    assert not oracle.sparse_decode(pay, 500).any()


def test_sparse_decode_ignores_bad_entries():
    pay = np.zeros(16 + 8 * 64, np.uint8)
    pay[:16].view(np.uint32)[:3] = [3, 10, 64]
    pay[16:28].view(np.int32)[:] = [2, 99, -1]
    pay[16 + 256 : 16 + 256 + 12].view(F)[:] = [1.5, 2.5, 3.5]
    want = np.zeros(10, F)
    want[2] = 1.5
    np.testing.assert_array_equal(oracle.sparse_decode(pay, 10), want)


# ---------------------------------------------------------------- merges
def test_tbq_merge_equals_sum_of_decodes_and_count_identity():
    n, P, tau = 5003, 8, F(0.05)
    rng = np.random.default_rng(5)
    pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(P)]
    decs = [oracle.tbq_decode(p, n) for p in pays]
    agg = oracle.tbq_decode_merge(pays, n)
    seq = np.zeros(n, F)
    for d in decs:
        seq = (seq + d).astype(F)
    np.testing.assert_array_equal(agg, seq)
    cnt = sum((d > 0).astype(int) - (d < 0).astype(int) for d in decs)
    np.testing.assert_allclose(agg, cnt * np.float64(tau), rtol=1e-5, atol=0)
    # fused re-encode = encode of the aggregate with the aggregator's residual
    r0 = rng.normal(0, 0.01, n).astype(F)
    agg2, out, r = oracle.tbq_decode_merge(pays, n, r0, tau)
    np.testing.assert_array_equal(agg2, agg)
    want_pay, want_r = oracle.tbq_encode(agg, r0, tau)
    np.testing.assert_array_equal(out, want_pay)
    np.testing.assert_array_equal(r, want_r)


def test_onebit_and_terngrad_merge_equal_sum_of_decodes():
    n, P = 1500, 4
    rng = np.random.default_rng(6)
    ob = [oracle.onebit_encode(rng.normal(0, 1, n).astype(F), np.zeros(n, F))[0] for _ in range(P)]
    tg = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), 512) for _ in range(P)]
    for pays, dec, mrg in ((ob, oracle.onebit_decode, oracle.onebit_decode_merge), (tg, oracle.terngrad_decode, oracle.terngrad_decode_merge)):
        seq = np.zeros(n, F)
        for p in pays:
            seq = (seq + dec(p, n)).astype(F)
        np.testing.assert_array_equal(mrg(pays, n), seq)


def test_sparse_merge_scatter_add_with_duplicates():
    n, P, ratio = 20000, 8, 0.01
    rng = np.random.default_rng(8)
    pays = []
    for p in range(P):
        g = rng.normal(0, 1e-3, n).astype(F)
        g[:50] += 1.0  # every peer selects the same leading entries -> duplicates
        pays.append(oracle.graddrop_encode(g, np.zeros(n, F), ratio)[0])
    agg = oracle.sparse_decode_merge(pays, n)
    dense = np.zeros(n, np.float64)
    for p in pays:
        dense += oracle.sparse_decode(p, n)
    np.testing.assert_allclose(agg, dense, rtol=1e-5, atol=1e-12)
    assert (agg[:50] > 7.5).all()
    acc0 = rng.normal(0, 1e-3, n).astype(F)
    agg2, out, acc = oracle.sparse_decode_merge(pays, n, acc0, ratio)
    np.testing.assert_array_equal(agg2, agg)
    want_pay, want_acc = oracle.graddrop_encode(agg, acc0, ratio)
    np.testing.assert_array_equal(out, want_pay)
    np.testing.assert_array_equal(acc, want_acc)


def test_merges_that_start_from_a_local_gradient():
    """A ring hop / a server that is also a worker: the sum starts from the aggregator's own
    uncompressed gradient, the peers are added to it in peer order; independent restatement
    with numpy float32 adds, element for element, and the re-encode sees that sum."""
    n, P, tau, ratio = 7001, 3, F(0.05), 0.01
    rng = np.random.default_rng(21)
    local = rng.normal(0, 0.03, n).astype(F)
    local[:4] = [0.0, -0.0, np.inf, 1e-40]
    tb = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(P)]
    ob = [oracle.onebit_encode(rng.normal(0, 1, n).astype(F), np.zeros(n, F))[0] for _ in range(P)]
    tg = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), 512) for _ in range(P)]
    sp = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), ratio)[0] for _ in range(P)]
    for pays, dec, mrg in ((tb, oracle.tbq_decode, oracle.tbq_decode_merge), (ob, oracle.onebit_decode, oracle.onebit_decode_merge),
                           (tg, oracle.terngrad_decode, oracle.terngrad_decode_merge),
                           (sp, oracle.sparse_decode, oracle.sparse_decode_merge)):
        seq = local.copy()
        for p in pays:
            d = dec(p, n)
            if mrg is oracle.sparse_decode_merge:  # only the listed elements are touched: -0 and NaN patterns survive elsewhere
                idx = oracle.sparse_unpack(p)[4]
                seq[idx] = (seq[idx] + d[idx]).astype(F)
            else:
                seq = (seq + d).astype(F)
        got = mrg(pays, n, local=local)
        np.testing.assert_array_equal(got.view(np.uint32), seq.view(np.uint32))
        # without a local gradient the start is +0
        np.testing.assert_array_equal(mrg(pays, n, local=np.zeros(n, F)), mrg(pays, n))
    r0 = rng.normal(0, 0.01, n).astype(F)
    agg, out, r = oracle.tbq_decode_merge(tb, n, r0, tau, local=local)
    finite = np.isfinite(agg)
    want_pay, want_r = oracle.tbq_encode(agg, r0, tau)
    np.testing.assert_array_equal(out, want_pay)
    np.testing.assert_array_equal(r[finite], want_r[finite])
    loc2 = np.where(np.isfinite(local), local, 0).astype(F)
    agg, out, acc = oracle.sparse_decode_merge(sp, n, r0, ratio, local=loc2)
    want_pay, want_acc = oracle.graddrop_encode(agg, r0, ratio)
    np.testing.assert_array_equal(out, want_pay)
    np.testing.assert_array_equal(acc, want_acc)
