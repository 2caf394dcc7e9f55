"""The all-cores (OpenMP) build of the oracle, which only the benchmark's CPU-baseline leg
times, computes what the scalar build computes: same payloads and state bit for bit (the
onebit scale, a sum, within rounding of the order it is taken in)."""
import numpy as np
import pytest

import oracle

F = np.float32


@pytest.fixture()
def both(monkeypatch):
    scalar, omp = oracle.lib(), oracle.omp_lib()
    assert omp.hpo_threads() >= 1 and scalar.hpo_threads() == 1

    def run(fn, *args, **kw):
        monkeypatch.setattr(oracle, "_lib", scalar)
        a = fn(*args, **kw)
        monkeypatch.setattr(oracle, "_lib", omp)
        b = fn(*args, **kw)
        monkeypatch.setattr(oracle, "_lib", scalar)
        return a, b

    return run


def same(a, b):
    a = a if isinstance(a, tuple) else (a,)
    b = b if isinstance(b, tuple) else (b,)
    assert len(a) == len(b)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(np.asarray(x).view(np.uint8) if isinstance(x, np.ndarray) else x,
                                      np.asarray(y).view(np.uint8) if isinstance(y, np.ndarray) else y)


@pytest.mark.parametrize("n", [1, 37, 4099, 300007])
def test_dense_quantisers(both, n):
    rng = np.random.default_rng(n)
    g, r, u = rng.normal(0, 0.02, n).astype(F), rng.normal(0, 0.01, n).astype(F), rng.random(n, dtype=F)
    a, b = both(oracle.tbq_encode, g, r, 0.05)
    same(a, b)
    same(*both(oracle.tbq_decode, a[0], n))
    sa, sb = both(oracle.onebit_scale, g, r)
    assert abs(float(sa) - float(sb)) <= 1e-6 * float(sa)
    a, b = both(oracle.onebit_encode, g, r, scale=sa)
    same(a, b)
    same(*both(oracle.onebit_decode, a[0], n))
    for bucket in (512, 100):  # 100: buckets share words, the loop must stay sequential
        a, b = both(oracle.terngrad_encode, g, u, bucket)
        same(a, b)
        same(*both(oracle.terngrad_decode, a, n))
    for bits in (1, 2, 4, 8):
        a, b = both(oracle.compll_encode, g, u, bits)
        same(a, b)
        same(*both(oracle.compll_decode, a, n))


@pytest.mark.parametrize("n,ratio", [(5000, 0.01), (300007, 0.001), (300007, 0.01)])
def test_sparsifiers_and_merges(both, n, ratio):
    rng = np.random.default_rng(n)
    g, z = rng.normal(0, 1e-3, n).astype(F), np.zeros(n, F)
    a, b = both(oracle.dgc_encode, g, z, z, 0.9, ratio)
    same(a, b)
    same(*both(oracle.sparse_decode, a[0], n))
    same(*both(oracle.graddrop_encode, g, z, ratio))
    pays = [oracle.dgc_encode(rng.normal(0, 1e-3, n).astype(F), z, z, 0.9, ratio)[0] for _ in range(3)]
    same(*both(oracle.sparse_decode_merge, pays, n, z, ratio))
    tp = [oracle.tbq_encode(rng.normal(0, 0.04, n).astype(F), z, 0.05)[0] for _ in range(3)]
    same(*both(oracle.tbq_decode_merge, tp, n, z, 0.05))
    ob = [oracle.onebit_encode(rng.normal(0, 0.04, n).astype(F), z)[0] for _ in range(3)]
    same(*both(oracle.onebit_decode_merge, ob, n))
    tg = [oracle.terngrad_encode(rng.normal(0, 0.04, n).astype(F), rng.random(n, dtype=F), 512) for _ in range(3)]
    same(*both(oracle.terngrad_decode_merge, tg, n))
