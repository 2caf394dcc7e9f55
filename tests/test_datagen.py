"""The counter-based input generator: its integer core against SplitMix64's published
outputs and a plain-integer restatement, the float transforms against what they must
produce, and the independence of a value from everything but (seed, tensor, element)."""
import math

import numpy as np
import torch

from hipress_amd import datagen as D
from hipress_amd import workloads as W


def test_splitmix64_known_answers():
    # the first outputs of SplitMix64 seeded with 0, as published with the generator
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC, 0x1B39896A51A8749B]
    x = 0
    for w in want:
        assert D.mix_int(x) == w
        x = (x + D.GOLDEN) & ((1 << 64) - 1)


def test_tensor_arithmetic_equals_the_integer_restatement():
    xs = [0, 1, 2, 12345, (1 << 63) - 1, 1 << 63, (1 << 64) - 1, 0xDEADBEEFCAFEF00D]
    t = torch.tensor([D._signed(x) for x in xs], dtype=torch.int64)
    got = [int(v) & ((1 << 64) - 1) for v in D.mix(t)]
    assert got == [D.mix_int(x) for x in xs]
    # words(): element i of tensor t is mix(key + i * GOLDEN)
    key = D.tensor_key(7, 3)
    w = D.words(7, 3, 5, "cpu", start=1000)
    for k in range(5):
        assert int(w[k]) & ((1 << 64) - 1) == D.mix_int((key + (1000 + k) * D.GOLDEN) & ((1 << 64) - 1))


def test_values_depend_on_seed_tensor_and_element_only():
    a = D.normal(10000, "cpu", 5, tensor=2, sigma=0.5)
    b = D.normal(4000, "cpu", 5, tensor=2, sigma=0.5)
    assert torch.equal(a[:4000], b)  # a longer tensor starts with the shorter one
    chunk = D._CHUNK
    try:  # and the chunking of the generation does not show
        D._CHUNK = 777
        c = D.normal(10000, "cpu", 5, tensor=2, sigma=0.5)
    finally:
        D._CHUNK = chunk
    assert torch.equal(a, c)
    assert not torch.equal(a, D.normal(10000, "cpu", 6, tensor=2, sigma=0.5))
    assert not torch.equal(a, D.normal(10000, "cpu", 5, tensor=3, sigma=0.5))
    # sets: tensor k of a set does not depend on the sizes of the others
    s1 = W.normal_set([100, 2000, 300], "cpu", 0, sigma=1e-3)
    s2 = W.normal_set([7, 2000], "cpu", 0, sigma=1e-3)
    assert torch.equal(s1[1], s2[1])


def test_uniform_is_24_bits_in_the_half_open_interval():
    u = D.uniform(200000, "cpu", 1)
    assert u.dtype == torch.float32 and float(u.min()) >= 0.0 and float(u.max()) < 1.0
    k = u.double() * (1 << 24)
    assert torch.equal(k, k.round())  # every value is a multiple of 2**-24
    assert abs(float(u.mean()) - 0.5) < 0.005
    w = D.words(1, 0, 10, "cpu")
    for i in range(10):
        assert float(u[i]) == ((int(w[i]) & ((1 << 64) - 1)) >> 40) / (1 << 24)


def test_normal_is_box_muller_of_the_word():
    n = 400000
    g = D.normal(n, "cpu", 3, tensor=1, sigma=2.0).double().numpy()
    w = D.words(3, 1, 8, "cpu")
    for i in range(8):
        z = int(w[i]) & ((1 << 64) - 1)
        u1, u2 = ((z >> 40) + 1) / (1 << 24), ((z >> 16) & 0xFFFFFF) / (1 << 24)
        ref = np.float32(math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)) * np.float32(2.0)
        assert abs(g[i] - float(ref)) <= 1e-6 * max(1.0, abs(float(ref)))
    assert abs(g.mean()) < 0.02 and abs(g.std() - 2.0) < 0.02
    assert abs((np.abs(g) > 2.0 * 3.2905).mean() - 0.001) < 0.0004  # the 0.1 % tail DGC selects from
    assert np.isfinite(g).all()


def test_heavy_tailed_and_log_sigma_sets():
    (g,) = W.heavy_tailed_set([300000], "cpu", 0)
    frac = float((g.abs() > 6e-3).float().mean())  # beyond 6 sigma of the bulk: Laplace draws only
    assert 0.003 < frac < 0.008
    sets = W.normal_set([50000] * 6, "cpu", 0, log_sigma_range=(-4.0, -2.0))
    sig = [float(t.std()) for t in sets]
    assert all(0.9e-4 < s < 1.1e-2 for s in sig) and len({round(math.log10(s), 2) for s in sig}) > 3


import pytest


@pytest.mark.gpu
def test_device_and_host_generate_the_same_values():
    n = 3_000_000
    assert torch.equal(D.uniform(n, "cuda", 9, 4).cpu(), D.uniform(n, "cpu", 9, 4))
    assert torch.equal(D.bernoulli(n, "cuda", 9, 4, 0.01).cpu(), D.bernoulli(n, "cpu", 9, 4, 0.01))
    a, b = D.normal(n, "cuda", 9, 4, 1e-3).cpu(), D.normal(n, "cpu", 9, 4, 1e-3)
    # the float64 logarithm and cosine of two libraries may differ in the last place, which
    # moves the float32 result by one unit for a vanishing share of the elements
    differ = (a != b)
    assert int(differ.sum()) <= n // 100000
    assert torch.allclose(a, b, rtol=2e-7, atol=0)
