"""Host threads: the library keeps no state between calls except what the caller hands it
(and two atomic counters), so calls from different host threads on different buffers and
streams may run at the same time.  Four threads, each with a stream of its own, run
different operators over and over while the others do the same; every result is held
against the CPU oracle's, computed beforehand.  (ctypes releases the interpreter lock for
the duration of a call, so the calls do overlap on the host.)"""
import threading

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32
ROUNDS = 12


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _tbq_job(hp, seed):
    n = 300007 + seed
    rng = np.random.default_rng(seed)
    gs = [rng.normal(0, 0.03, n).astype(F) for _ in range(3)]
    want, r = [], np.zeros(n, F)
    for g in gs:
        pay, r = oracle.tbq_encode(g, r, 0.05)
        want.append((pay, r.copy(), oracle.tbq_decode(pay, n)))

    def run():
        r_gpu = torch.zeros(n, device="cuda")
        for g, (pay_w, r_w, out_w) in zip(gs, want):
            pay = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
            out = torch.empty(n, device="cuda")
            hp.tbq_encode(dev(g), r_gpu, pay, 0.05)
            hp.tbq_decode(pay, out)
            torch.cuda.current_stream().synchronize()
            assert np.array_equal(pay.cpu().numpy(), pay_w) and np.array_equal(r_gpu.cpu().numpy(), r_w)
            assert np.array_equal(out.cpu().numpy(), out_w)

    return run


def _onebit_job(hp, seed):
    n = 200003 + seed
    rng = np.random.default_rng(seed)
    g, r0 = rng.normal(0, 1e-3, n).astype(F), rng.normal(0, 1e-3, n).astype(F)

    def run():
        r = dev(r0)
        pay = torch.zeros(hp.onebit_payload_bytes(n), dtype=torch.uint8, device="cuda")
        hp.onebit_encode(dev(g), r, pay)  # per-stream workspace inside the binding
        torch.cuda.current_stream().synchronize()
        got = pay.cpu().numpy()
        s = got[:4].view(F)[0]
        assert abs(float(s) - float(oracle.onebit_scale(g, r0))) <= 1e-5 * float(s)
        pay_w, r_w = oracle.onebit_encode(g, r0, scale=s)
        assert np.array_equal(got, pay_w) and np.array_equal(r.cpu().numpy(), r_w)

    return run


def _dgc_job(hp, seed):
    n = 400009 + seed
    rng = np.random.default_rng(seed)
    g = rng.normal(0, 1e-3, n).astype(F)
    pay_w, mom_w, acc_w = oracle.dgc_encode(g, np.zeros(n, F), np.zeros(n, F), 0.9, 0.001)
    out_w = oracle.sparse_decode(pay_w, n)
    want = oracle.sparse_unpack(pay_w)

    def run():
        mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
        pay = torch.zeros(hp.dgc_payload_bytes(n, 0.001), dtype=torch.uint8, device="cuda")
        out = torch.empty(n, device="cuda")
        hp.dgc_encode(dev(g), mom, acc, pay, 0.9, 0.001)
        hp.dgc_decode(pay, out)
        torch.cuda.current_stream().synchronize()
        got = oracle.sparse_unpack(pay.cpu().numpy())
        assert got[:3] == want[:3] and np.array_equal(got[4], want[4]) and np.array_equal(got[5], want[5])
        assert np.array_equal(mom.cpu().numpy(), mom_w) and np.array_equal(acc.cpu().numpy(), acc_w)
        assert np.array_equal(out.cpu().numpy(), out_w)

    return run


def _sparse_merge_job(hp, seed):
    """The per-tensor sparse merge draws a number from a process-wide counter on every call."""
    n = 250001 + seed
    rng = np.random.default_rng(seed)
    pays = [oracle.graddrop_encode(rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F), 0.01)[0] for _ in range(4)]
    agg_w, out_w, acc_w = oracle.sparse_decode_merge(pays, n, np.zeros(n, F), 0.01)
    want = oracle.sparse_unpack(out_w)

    def run():
        agg, acc = torch.empty(n, device="cuda"), torch.zeros(n, device="cuda")
        outp = torch.zeros(hp.sparse_payload_bytes(n, 0.01), dtype=torch.uint8, device="cuda")
        hp.dgc_decode_merge([dev(p) for p in pays], agg, acc, outp, 0.01)
        torch.cuda.current_stream().synchronize()
        got = oracle.sparse_unpack(outp.cpu().numpy())
        assert np.array_equal(agg.cpu().numpy(), agg_w) and np.array_equal(acc.cpu().numpy(), acc_w)
        assert got[:3] == want[:3] and np.array_equal(got[4], want[4]) and np.array_equal(got[5], want[5])

    return run


def test_four_host_threads_on_their_own_streams():
    import hipress_amd as hp

    hp._lib.lib()
    jobs = [_tbq_job(hp, 1), _onebit_job(hp, 2), _dgc_job(hp, 3), _sparse_merge_job(hp, 4)]
    for job in jobs:  # once alone: a wrong expectation must not pass for a race
        job()
    torch.cuda.synchronize()
    errors, start = [], threading.Barrier(len(jobs))

    def worker(k, job):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                start.wait(timeout=60)
                for _ in range(ROUNDS):
                    job()
        except BaseException as exc:  # reported by the main thread
            errors.append((k, repr(exc)))

    threads = [threading.Thread(target=worker, args=(k, job)) for k, job in enumerate(jobs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    torch.cuda.synchronize()
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors
