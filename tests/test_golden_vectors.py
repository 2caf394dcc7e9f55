"""Committed vectors (tests/golden/operator_vectors.npz, written by
tests/golden/make_operator_vectors.py): every operator on small fixed cases.  The CPU part
holds the oracle to them, so the oracle cannot drift; the GPU part holds the library to them
directly, so oracle and kernels cannot drift together (a bit order, a header field, a tie
rule changed on both sides would pass every live comparison)."""
import hashlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

F = np.float32
V = np.load(os.path.join(ROOT, "tests", "golden", "operator_vectors.npz"), allow_pickle=False)
N, NS, PEERS = 5003, 300007, 3


def digest(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8)


def same(a, b):
    return a.shape == b.shape and np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


def sparse_gradient(tag, step):
    """The gradient of a sparse case: stored for the small one, regenerated for the large one
    (skipped when this platform's generator gives other bits than the fixture was made from)."""
    import torch

    from hipress_amd import datagen

    if tag == "small":
        return V[f"sparse_small_gradient_{step}"]
    g = datagen.normal(NS, torch.device("cpu"), 9, step, 1e-3).numpy().astype(F)
    if not np.array_equal(digest(g), V[f"sparse_large_gradient_digest_{step}"]):
        pytest.skip("this platform's float64 log/cos move an input of the large fixture by a unit")
    return g


def merge_peers(prefix):
    return [V[f"{prefix}_{p}"] for p in range(PEERS)]


# ------------------------------------------------------------------ the oracle against the vectors
def test_oracle_tbq():
    r = np.zeros(N, F)
    for step in range(3):
        pay, r = oracle.tbq_encode(V[f"tbq_gradient_{step}"], r, 0.05)
        assert same(pay, V[f"tbq_payload_{step}"]) and same(r, V[f"tbq_residual_{step}"])
        assert same(oracle.tbq_decode(pay, N), V[f"tbq_decoded_{step}"])


def test_oracle_onebit():
    r = V["onebit_residual_in"]
    for step in range(2):
        pay, r = oracle.onebit_encode(V[f"onebit_gradient_{step}"], r)
        assert same(pay, V[f"onebit_payload_{step}"]) and same(r, V[f"onebit_residual_{step}"])
        assert same(oracle.onebit_decode(pay, N), V[f"onebit_decoded_{step}"])


def test_oracle_terngrad_and_minmax_quantiser():
    g, u = V["terngrad_gradient"], V["terngrad_uniform"]
    for bucket in (512, 100):
        pay = oracle.terngrad_encode(g, u, bucket)
        assert same(pay, V[f"terngrad_payload_b{bucket}"])
        assert same(oracle.terngrad_decode(pay, N), V[f"terngrad_decoded_b{bucket}"])
    for b in (1, 2, 4, 8):
        pay = oracle.compll_encode(g, u, b)
        assert same(pay, V[f"compll_payload_b{b}"]) and same(oracle.compll_decode(pay, N), V[f"compll_decoded_b{b}"])


@pytest.mark.parametrize("tag", ["small", "large"])
def test_oracle_sparse(tag):
    n = N if tag == "small" else NS
    mom, acc, acc_gd = np.zeros(n, F), np.zeros(n, F), np.zeros(n, F)
    for step in range(2):
        g = sparse_gradient(tag, step)
        pay, mom, acc = oracle.dgc_encode(g, mom, acc, 0.9, 0.001)
        assert same(pay, V[f"dgc_{tag}_payload_{step}"])
        assert same(digest(mom), V[f"dgc_{tag}_momentum_digest_{step}"]) and same(digest(acc), V[f"dgc_{tag}_accumulator_digest_{step}"])
        assert same(digest(oracle.sparse_decode(pay, n)), V[f"dgc_{tag}_decoded_digest_{step}"])
        pay, acc_gd = oracle.graddrop_encode(g, acc_gd, 0.01)
        assert same(pay, V[f"graddrop_{tag}_payload_{step}"]) and same(digest(acc_gd), V[f"graddrop_{tag}_accumulator_digest_{step}"])


def test_oracle_merges():
    agg, outp, res = oracle.tbq_decode_merge(merge_peers("merge_tbq_peer"), N, np.zeros(N, F), 0.05)
    assert same(agg, V["merge_tbq_aggregate"]) and same(outp, V["merge_tbq_out_payload"]) and same(res, V["merge_tbq_residual"])
    agg, outp, acc = oracle.sparse_decode_merge(merge_peers("merge_sparse_peer"), NS, np.zeros(NS, F), 0.01)
    assert same(digest(agg), V["merge_sparse_aggregate_digest"]) and same(digest(acc), V["merge_sparse_accumulator_digest"])
    assert same(outp, V["merge_sparse_out_payload"])


def test_vectors_hold_what_the_wire_format_says():
    """Spot checks that need neither side: header fields and sizes of the stored payloads."""
    p = V["tbq_payload_0"]
    assert p.size == 16 + 4 * ((N + 15) // 16) and p[:4].view(F)[0] == F(0.05) and p[4:8].view(np.uint32)[0] == N
    p = V["onebit_payload_0"]
    assert p.size == 16 + 4 * ((N + 31) // 32) and p[4:8].view(np.uint32)[0] == N and not p[8:16].any()
    p = V["terngrad_payload_b512"]
    assert p[:8].view(np.uint32).tolist() == [N, 512]
    p = V["compll_payload_b2"]
    assert p[0] == 2 and p[1] == N % 4 and p.size == 10 + (2 * N + 7) // 8
    for name in ("dgc_large_payload_0", "graddrop_large_payload_1", "merge_sparse_out_payload"):
        nnz, n, cap = V[name][:12].view(np.uint32)
        assert n == NS and 0 < nnz <= cap and V[name].size == 16 + 8 * cap
        idx = V[name][16:16 + 4 * nnz].view(np.int32)
        assert (np.diff(idx) > 0).all() and idx[0] >= 0 and idx[-1] < NS  # ascending index order


# ------------------------------------------------------------------ the library against the vectors
@pytest.fixture(scope="module")
def hp():
    import torch

    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch

    torch.cuda.synchronize()
    return t.cpu().numpy()


def new_payload(nbytes):
    import torch

    return torch.full((int(nbytes),), 0xAB, dtype=torch.uint8, device="cuda")


@pytest.mark.gpu
def test_library_tbq(hp):
    import torch

    r = torch.zeros(N, device="cuda")
    for step in range(3):
        pay, out = new_payload(hp.tbq_payload_bytes(N)), torch.empty(N, device="cuda")
        hp.tbq_encode(dev(V[f"tbq_gradient_{step}"]), r, pay, 0.05)
        hp.tbq_decode(pay, out)
        assert same(host(pay), V[f"tbq_payload_{step}"]) and same(host(r), V[f"tbq_residual_{step}"])
        assert same(host(out), V[f"tbq_decoded_{step}"])


@pytest.mark.gpu
def test_library_onebit(hp):
    import torch

    r_ref = V["onebit_residual_in"]
    r = dev(r_ref)
    for step in range(2):
        g = V[f"onebit_gradient_{step}"]
        pay, out = new_payload(hp.onebit_payload_bytes(N)), torch.empty(N, device="cuda")
        hp.onebit_encode(dev(g), r, pay)
        hp.onebit_decode(pay, out)
        got, want = host(pay), V[f"onebit_payload_{step}"]
        s, s_want = got[:4].view(F)[0], want[:4].view(F)[0]
        assert abs(float(s) - float(s_want)) <= 1e-5 * float(s_want)
        assert same(got[4:], want[4:])  # n, the reserved words and every sign bit do not depend on the scale's last bits
        if s == s_want:
            assert same(host(r), V[f"onebit_residual_{step}"]) and same(host(out), V[f"onebit_decoded_{step}"])
        else:  # a last-bit difference of the scale: the stored residual is reached within 1e-5 of the scale
            assert np.all(np.abs(host(r) - V[f"onebit_residual_{step}"]) <= 1e-5 * float(s_want))
        # the next step starts from the stored residual on both sides
        r = dev(V[f"onebit_residual_{step}"])


@pytest.mark.gpu
def test_library_terngrad_and_minmax_quantiser(hp):
    import torch

    g, u = dev(V["terngrad_gradient"]), dev(V["terngrad_uniform"])
    for bucket in (512, 100):
        pay, out = new_payload(hp.terngrad_payload_bytes(N, bucket)), torch.empty(N, device="cuda")
        hp.terngrad_encode(g, u, pay, bucket)
        hp.terngrad_decode(pay, out)
        assert same(host(pay), V[f"terngrad_payload_b{bucket}"]) and same(host(out), V[f"terngrad_decoded_b{bucket}"])
    for b in (1, 2, 4, 8):
        want = V[f"compll_payload_b{b}"]
        pay = new_payload(want.size)
        hp.compll_terngrad_encode(g, u, pay, b)
        got = host(pay)
        # min and max are order-free, so the header and with it every code are bit-exact
        assert same(got, want)
        out = torch.full((N,), 7.0, device="cuda")
        hp.compll_terngrad_decode(pay, out)
        dec = V[f"compll_decoded_b{b}"]
        k = hp.compll_decoded_count(N, b)  # the reference's count, short of N for some widths
        assert dec.size == k and same(host(out)[:k], dec) and (host(out)[k:] == 7.0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["small", "large"])
def test_library_sparse(hp, tag):
    import torch

    n = N if tag == "small" else NS
    mom, acc, acc_gd = (torch.zeros(n, device="cuda") for _ in range(3))
    for step in range(2):
        g = dev(sparse_gradient(tag, step))
        pay, out = new_payload(hp.dgc_payload_bytes(n, 0.001)), torch.empty(n, device="cuda")
        hp.dgc_encode(g, mom, acc, pay, 0.9, 0.001)
        hp.dgc_decode(pay, out)
        want = V[f"dgc_{tag}_payload_{step}"]
        nnz = int(want[:4].view(np.uint32)[0])
        got = host(pay)
        cap = int(want[8:12].view(np.uint32)[0])
        assert same(got[:16], want[:16])
        assert same(got[16:16 + 4 * nnz], want[16:16 + 4 * nnz])  # indices
        assert same(got[16 + 4 * cap:16 + 4 * cap + 4 * nnz], want[16 + 4 * cap:16 + 4 * cap + 4 * nnz])  # values
        assert same(digest(host(mom)), V[f"dgc_{tag}_momentum_digest_{step}"])
        assert same(digest(host(acc)), V[f"dgc_{tag}_accumulator_digest_{step}"])
        assert same(digest(host(out)), V[f"dgc_{tag}_decoded_digest_{step}"])
        pay = new_payload(hp.graddrop_payload_bytes(n, 0.01))
        hp.graddrop_encode(g, acc_gd, pay, 0.01)
        want = V[f"graddrop_{tag}_payload_{step}"]
        nnz, cap = int(want[:4].view(np.uint32)[0]), int(want[8:12].view(np.uint32)[0])
        got = host(pay)
        assert same(got[:16], want[:16]) and same(got[16:16 + 4 * nnz], want[16:16 + 4 * nnz])
        assert same(got[16 + 4 * cap:16 + 4 * cap + 4 * nnz], want[16 + 4 * cap:16 + 4 * cap + 4 * nnz])
        assert same(digest(host(acc_gd)), V[f"graddrop_{tag}_accumulator_digest_{step}"])


@pytest.mark.gpu
def test_library_merges(hp):
    import torch

    agg, res = torch.empty(N, device="cuda"), torch.zeros(N, device="cuda")
    outp = new_payload(hp.tbq_payload_bytes(N))
    hp.tbq_decode_merge([dev(p) for p in merge_peers("merge_tbq_peer")], agg, res, outp, 0.05)
    assert same(host(agg), V["merge_tbq_aggregate"]) and same(host(outp), V["merge_tbq_out_payload"])
    assert same(host(res), V["merge_tbq_residual"])
    agg, acc = torch.empty(NS, device="cuda"), torch.zeros(NS, device="cuda")
    outp = new_payload(hp.sparse_payload_bytes(NS, 0.01))
    hp.dgc_decode_merge([dev(p) for p in merge_peers("merge_sparse_peer")], agg, acc, outp, 0.01)
    assert same(digest(host(agg)), V["merge_sparse_aggregate_digest"]) and same(digest(host(acc)), V["merge_sparse_accumulator_digest"])
    want = V["merge_sparse_out_payload"]
    nnz, cap = int(want[:4].view(np.uint32)[0]), int(want[8:12].view(np.uint32)[0])
    got = host(outp)
    assert same(got[:16], want[:16]) and same(got[16:16 + 4 * nnz], want[16:16 + 4 * nnz])
    assert same(got[16 + 4 * cap:16 + 4 * cap + 4 * nnz], want[16 + 4 * cap:16 + 4 * cap + 4 * nnz])
