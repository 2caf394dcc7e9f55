"""Decode-and-merge that starts from the aggregator's own uncompressed gradient (a ring
hop, a server that is also a worker): every entry point against the oracle, bit for bit."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32
SIZES = [1, 1000, 4096, 100003, (1 << 20) + 5]


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def offset_view(a):
    """The same values at an address that is only 4-byte aligned."""
    buf = torch.empty(a.size + 1, dtype=torch.float32, device="cuda")
    buf[1:].copy_(torch.from_numpy(a))
    return buf[1:]


def same_pairs(got, want):
    *hg, ig, vg = oracle.sparse_unpack(got)
    *hw, iw, vw = oracle.sparse_unpack(want)
    assert hg == hw
    np.testing.assert_array_equal(ig, iw)
    np.testing.assert_array_equal(vg, vw)


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("npeers", [1, 3, 9])
def test_tbq_hop(hp, n, npeers):
    rng = np.random.default_rng(n + npeers)
    tau = F(0.05)
    pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(npeers)]
    local = rng.normal(0, 0.03, n).astype(F)
    r0 = rng.normal(0, 0.01, n).astype(F)
    d_pays = [dev(p) for p in pays]
    # sum only
    agg = torch.empty(n, device="cuda")
    hp.tbq_decode_merge(d_pays, agg, local=dev(local))
    np.testing.assert_array_equal(host(agg), oracle.tbq_decode_merge(pays, n, local=local))
    # sum + re-encode, the local gradient at a 4-byte-aligned address, the aggregate in the local buffer itself
    want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, r0, tau, local=local)
    for loc in (dev(local), offset_view(local)):
        r, out = dev(r0), torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
        agg = torch.empty(n, device="cuda")
        hp.tbq_decode_merge(d_pays, agg, r, out, float(tau), local=loc)
        np.testing.assert_array_equal(host(agg), want_agg)
        np.testing.assert_array_equal(host(out), want_out)
        np.testing.assert_array_equal(host(r), want_r)
    inplace, r, out = dev(local), dev(r0), torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.tbq_decode_merge(d_pays, inplace, r, out, float(tau), local=inplace)
    np.testing.assert_array_equal(host(inplace), want_agg)
    np.testing.assert_array_equal(host(out), want_out)
    # only the payload to send on
    r, out = dev(r0), torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.tbq_decode_merge(d_pays, None, r, out, float(tau), local=dev(local))
    np.testing.assert_array_equal(host(out), want_out)
    np.testing.assert_array_equal(host(r), want_r)


@pytest.mark.parametrize("n", SIZES)
def test_onebit_and_terngrad_merges_start_from_local(hp, n):
    rng = np.random.default_rng(n)
    local = rng.normal(0, 1, n).astype(F)
    ob = [oracle.onebit_encode(rng.normal(0, 1, n).astype(F), np.zeros(n, F))[0] for _ in range(4)]
    tg = [oracle.terngrad_encode(rng.normal(0, 1, n).astype(F), rng.random(n, dtype=F), 512) for _ in range(4)]
    for loc in (dev(local), offset_view(local)):
        agg = torch.empty(n, device="cuda")
        hp.onebit_decode_merge([dev(p) for p in ob], agg, local=loc)
        np.testing.assert_array_equal(host(agg), oracle.onebit_decode_merge(ob, n, local=local))
        hp.terngrad_decode_merge([dev(p) for p in tg], agg, local=loc)
        np.testing.assert_array_equal(host(agg), oracle.terngrad_decode_merge(tg, n, local=local))


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("npeers", [1, 8])
def test_sparse_hop(hp, n, npeers):
    rng = np.random.default_rng(3 * n + npeers)
    ratio = 0.01
    pays = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), ratio)[0] for _ in range(npeers)]
    local = rng.normal(0, 1e-3, n).astype(F)
    a0 = rng.normal(0, 1e-3, n).astype(F)
    d_pays = [dev(p) for p in pays]
    agg = torch.empty(n, device="cuda")
    hp.dgc_decode_merge(d_pays, agg, ratio=ratio, local=dev(local))
    np.testing.assert_array_equal(host(agg).view(np.uint32), oracle.sparse_decode_merge(pays, n, local=local).view(np.uint32))
    want_agg, want_out, want_acc = oracle.sparse_decode_merge(pays, n, a0, ratio, local=local)
    for loc in (dev(local), offset_view(local)):
        acc, out = dev(a0), torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
        agg = torch.empty(n, device="cuda")
        hp.dgc_decode_merge(d_pays, agg, acc, out, ratio, local=loc)
        np.testing.assert_array_equal(host(agg), want_agg)
        same_pairs(host(out), want_out)
        np.testing.assert_array_equal(host(acc), want_acc)
    acc, out = dev(a0), torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    hp.dgc_decode_merge(d_pays, None, acc, out, ratio, local=dev(local))
    same_pairs(host(out), want_out)
    np.testing.assert_array_equal(host(acc), want_acc)


@pytest.mark.parametrize("alg", ["tbq", "dgc"])
def test_merge_batch_chunks_with_and_without_local(hp, alg):
    """One launch sequence over chunks of which some start from a local gradient and some from zero."""
    rng = np.random.default_rng(11)
    sizes = [5000, 4096, 70001, 1 << 20, 12]
    tau, ratio = F(0.05), 0.01
    chunks, wants = [], []
    for k, n in enumerate(sizes):
        if alg == "tbq":
            pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(3)]
        else:
            pays = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), ratio)[0] for _ in range(3)]
        local = rng.normal(0, 0.02 if alg == "tbq" else 1e-3, n).astype(F) if k % 2 == 0 else None
        st = rng.normal(0, 0.01 if alg == "tbq" else 1e-3, n).astype(F)
        nb = hp.tbq_payload_bytes(n) if alg == "tbq" else hp.sparse_payload_bytes(n, ratio)
        c = {"compressed": [dev(p) for p in pays], "aggregate": torch.empty(n, device="cuda"), "state": dev(st),
             "out_compressed": torch.zeros(nb, dtype=torch.uint8, device="cuda")}
        if local is not None:
            c["local"] = dev(local)
        chunks.append(c)
        wants.append(oracle.tbq_decode_merge(pays, n, st, tau, local=local) if alg == "tbq"
                     else oracle.sparse_decode_merge(pays, n, st, ratio, local=local))
    mb = hp.MergeBatch(alg, chunks, threshold=float(tau), ratio=ratio)
    mb.run()
    for c, (agg, out, st) in zip(chunks, wants):
        np.testing.assert_array_equal(host(c["aggregate"]), agg)
        if alg == "tbq":
            np.testing.assert_array_equal(host(c["out_compressed"]), out)
        else:
            same_pairs(host(c["out_compressed"]), out)
        np.testing.assert_array_equal(host(c["state"]), st)
    mb.close()


def test_empty_chunk_and_argument_checks(hp):
    pay = torch.zeros(16, dtype=torch.uint8, device="cuda")
    agg = torch.empty(0, device="cuda")
    hp.tbq_decode_merge([pay], agg, local=torch.empty(0, device="cuda"))
    with pytest.raises(ValueError, match="local"):
        hp.tbq_decode_merge([torch.zeros(hp.tbq_payload_bytes(8), dtype=torch.uint8, device="cuda")], torch.empty(8, device="cuda"),
                            local=torch.empty(7, device="cuda"))
    with pytest.raises(TypeError):
        hp.onebit_decode_merge([torch.zeros(hp.onebit_payload_bytes(8), dtype=torch.uint8, device="cuda")],
                               torch.empty(8, device="cuda"), local=torch.empty(8, device="cuda", dtype=torch.float64))


@pytest.mark.parametrize("n", [100003, (1 << 20) + 5])
def test_more_peers_than_one_call_takes_are_merged_in_two_calls(hp, n):
    """One call takes at most 16 peers.  Twenty are merged by two calls, the second starting
    from the first one's aggregate (`local`) and carrying the re-encode: the additions happen
    in the same order as in one sum over all twenty, so aggregate, re-encoded payload and state
    equal the oracle's for twenty peers bit for bit - dense (TBQ) and sparse."""
    rng = np.random.default_rng(n)
    P, first = 20, 16
    tau = F(0.05)
    pays = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), np.zeros(n, F), tau)[0] for _ in range(P)]
    r0 = rng.normal(0, 0.01, n).astype(F)
    want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, r0, tau)
    d = [dev(p) for p in pays]
    agg, res = torch.empty(n, device="cuda"), dev(r0)
    outp = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.tbq_decode_merge(d[:first], agg)
    hp.tbq_decode_merge(d[first:], agg, res, outp, tau, local=agg)  # aggregate may be the same buffer as local
    np.testing.assert_array_equal(host(agg), want_agg)
    np.testing.assert_array_equal(host(outp), want_out)
    np.testing.assert_array_equal(host(res), want_r)
    # sparse: twenty GradDrop payloads, re-encoded at 1 %
    sp = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), 0.01)[0] for _ in range(P)]
    a0 = rng.normal(0, 1e-4, n).astype(F)
    want_agg, want_out, want_acc = oracle.sparse_decode_merge(sp, n, a0, 0.01)
    d = [dev(p) for p in sp]
    agg, acc = torch.empty(n, device="cuda"), dev(a0)
    outp = torch.zeros(hp.sparse_payload_bytes(n, 0.01), dtype=torch.uint8, device="cuda")
    hp.dgc_decode_merge(d[:first], agg)
    hp.dgc_decode_merge(d[first:], agg, acc, outp, 0.01, local=agg)
    np.testing.assert_array_equal(host(agg), want_agg)
    np.testing.assert_array_equal(host(acc), want_acc)
    same_pairs(host(outp), want_out)
