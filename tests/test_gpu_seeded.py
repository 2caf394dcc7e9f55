"""The stochastic quantisers called with a seed instead of a noise tensor: the kernels draw
u_i = uniform_draws(seed, tensor)[i] themselves, so every result must equal, byte for byte,
what the oracle makes of the same gradient and those draws."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
F = np.float32


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


def view(a, off):
    """The array on the GPU, `off` elements into its allocation (4-byte aligned only for off % 4 != 0)."""
    t = torch.empty(a.size + off, device="cuda")
    v = t[off:]
    v.copy_(torch.from_numpy(a))
    return v


@pytest.mark.parametrize("seed,tensor", [(0, 0), (1, 0), (2 ** 64 - 1, 2 ** 32 - 1), (77, 390)])
@pytest.mark.parametrize("n,off", [(0, 0), (1, 0), (4095, 1), (4096, 0), (1000003, 3)])
def test_uniform_fill_writes_the_oracles_draws(hp, seed, tensor, n, off):
    buf = torch.full((n + off + 8,), 7.0, device="cuda")
    hp.uniform_fill(buf[off:off + n], seed, tensor)
    got = host(buf)
    np.testing.assert_array_equal(got[off:off + n], oracle.uniform_draws(seed, n, tensor))
    assert (got[:off] == 7).all() and (got[off + n:] == 7).all()


@pytest.mark.parametrize("bucket", [512, 256, 1024, 100, 4096, 5000, 1 << 20])
@pytest.mark.parametrize("n,off", [(1, 0), (4097, 0), (300001, 1), (1000003, 0)])
def test_terngrad_seeded_equals_the_explicit_noise(hp, n, off, bucket):
    rng = np.random.default_rng(n + bucket)
    g = rng.normal(0, 1e-3, n).astype(F)
    seed = int(rng.integers(0, 2 ** 63))
    want = oracle.terngrad_encode(g, oracle.uniform_draws(seed, n), bucket)
    pay = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode_seeded(view(g, off), pay, bucket, seed)
    np.testing.assert_array_equal(host(pay), want)
    # the same through the explicit entry point with the draws written out
    u = torch.empty(n, device="cuda")
    hp.uniform_fill(u, seed)
    pay2 = payload(hp.terngrad_payload_bytes(n, bucket))
    hp.terngrad_encode(dev(g), u, pay2, bucket)
    np.testing.assert_array_equal(host(pay2), want)
    # another seed, another payload (beyond a handful of elements)
    if n > 1000:
        hp.terngrad_encode_seeded(dev(g), pay2, bucket, seed + 1)
        assert (host(pay2) != want).any()


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("n,off", [(1, 0), (4099, 1), (1000003, 0)])
def test_minmax_quantiser_seeded_equals_the_explicit_noise(hp, n, off, b):
    rng = np.random.default_rng(n * 8 + b)
    g = rng.normal(0, 1e-3, n).astype(F)
    seed = int(rng.integers(0, 2 ** 63))
    want = oracle.compll_encode(g, oracle.uniform_draws(seed, n), b)
    pay = payload(hp.compll_payload_bytes(n, b))
    hp.compll_terngrad_encode_seeded(view(g, off), pay, b, seed)
    got = host(pay)
    # min and max are exact, so is everything derived from them
    np.testing.assert_array_equal(got, want)
    pay2 = payload(hp.compll_payload_bytes(n, b))
    hp.TernGradEncode(dev(g), pay2, b, seed=seed)  # the reference's operator name, no noise tensor
    np.testing.assert_array_equal(host(pay2), want)


def test_reference_named_operator_without_noise_follows_torchs_seed(hp):
    n = 50000
    g = dev(np.random.default_rng(0).normal(0, 1e-3, n).astype(F))
    pays = [payload(hp.compll_payload_bytes(n, 2)) for _ in range(4)]
    torch.manual_seed(123)
    hp.TernGradEncode(g, pays[0], 2)
    hp.TernGradEncode(g, pays[1], 2)
    torch.manual_seed(123)
    hp.TernGradEncode(g, pays[2], 2)
    hp.TernGradEncode(g, pays[3], 2)
    a, b, c, d = (host(p) for p in pays)
    np.testing.assert_array_equal(a, c)
    np.testing.assert_array_equal(b, d)
    assert (a != b).any()  # every call draws anew


@pytest.mark.parametrize("bucket", [512, 100, 6000])
def test_seeded_batch_gives_every_tensor_draws_of_its_own(hp, bucket):
    rng = np.random.default_rng(bucket)
    sizes = [4096 * 3 + 17, 1, 0, 4096, 12345, 70001, 300000]
    gs = [rng.normal(0, 1e-3, n).astype(F) for n in sizes]
    tensors = [{"gradient": dev(g), "out": torch.full((g.size,), 7.0, device="cuda"),
                "compressed": payload(hp.terngrad_payload_bytes(g.size, bucket))} for g in gs]
    b = hp.Batch("terngrad", tensors, bucket=bucket)
    assert b.seeded
    for seed in (5, 6):
        b.encode(seed=seed)
        b.decode()
        for k, (t, g) in enumerate(zip(tensors, gs)):
            want = oracle.terngrad_encode(g, oracle.uniform_draws(seed, g.size, k), bucket)
            np.testing.assert_array_equal(host(t["compressed"]), want, err_msg=f"seed {seed} tensor {k}")
            np.testing.assert_array_equal(host(t["out"]), oracle.terngrad_decode(want, g.size), err_msg=f"decode, tensor {k}")
    b.close()


def test_batches_take_a_seed_exactly_when_they_have_no_noise_tensors(hp):
    import ctypes

    from hipress_amd import _lib

    n = 5000
    g, u = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    mk = lambda with_u: {"gradient": g, "compressed": payload(hp.terngrad_payload_bytes(n, 512)), **({"uniform": u} if with_u else {})}
    with pytest.raises(_lib.HipressError) as e:  # some with, some without
        hp.Batch("terngrad", [mk(True), mk(False)], bucket=512)
    assert e.value.code == -1
    L = _lib.lib()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    drawn, plain = hp.Batch("terngrad", [mk(False)], bucket=512), hp.Batch("terngrad", [mk(True)], bucket=512)
    assert L.hipress_batch_encode(drawn._h, st) == -4
    assert L.hipress_batch_encode_seeded(plain._h, 1, st) == -4
    tb = hp.Batch("tbq", [{"gradient": g, "residual": torch.zeros(n, device="cuda"), "compressed": payload(hp.tbq_payload_bytes(n))}], threshold=0.05)
    assert L.hipress_batch_encode_seeded(tb._h, 1, st) == -4
    for b in (drawn, plain, tb):
        b.close()
    # a table of empty tensors has nothing to draw for: the plain call serves it, with or without noise tensors
    e = torch.zeros(0, device="cuda")
    empty = hp.Batch("terngrad", [{"gradient": e, "compressed": payload(hp.terngrad_payload_bytes(0, 512))}], bucket=512)
    assert not empty.seeded
    empty.encode()
    empty.close()


def test_planned_set_without_noise_tensors(hp):
    """Partitions of one gradient are tensors of their own in the table: each draws with its own
    number, so no two partitions round alike."""
    from hipress_amd import planner

    n, k, bucket, seed = 1_000_000, 4, 512, 99
    g = np.random.default_rng(1).normal(0, 1e-3, n).astype(F)
    ps = hp.PlannedSet("terngrad", [("w", n, True, k)], {"w": dev(g)}, bucket=bucket)
    ps.encode(seed=seed)
    ps.decode()
    ref = np.empty(n, F)
    for i, (off, length) in enumerate(planner.partition_bounds(n, k)):
        want = oracle.terngrad_encode(g[off:off + length], oracle.uniform_draws(seed, length, i), bucket)
        np.testing.assert_array_equal(host(ps.compressed["w"][i]), want, err_msg=f"partition {i}")
        ref[off:off + length] = oracle.terngrad_decode(want, length)
    np.testing.assert_array_equal(host(ps.out["w"]), ref)
    ps.close()


def test_seeded_terngrad_is_unbiased_over_seeds(hp):
    """What the noise is for: averaged over many seeds the decoded value of every element
    approaches the gradient (E[code] = g / s when u is uniform).  256 seeds, every element
    that is kept often enough for a normal bound within 5.5 standard errors, no drift over the
    tensor, and the spread of independent draws."""
    n, bucket, seeds = 20000, 512, 256
    g = np.random.default_rng(3).normal(0, 1e-3, n).astype(F)
    gd, pay, out = dev(g), payload(hp.terngrad_payload_bytes(n, bucket)), torch.empty(n, device="cuda")
    acc = torch.zeros(n, device="cuda", dtype=torch.float64)
    for seed in range(seeds):
        hp.terngrad_encode_seeded(gd, pay, bucket, seed)
        hp.terngrad_decode(pay, out)
        acc += out.double()
    mean = host(acc) / seeds
    s = np.empty(n)
    for b0 in range(0, n, bucket):
        s[b0:b0 + bucket] = np.abs(g[b0:b0 + bucket]).max()
    p = np.abs(g) / s                                  # the probability that an element is kept
    se = s * np.sqrt(p * (1 - p) / seeds) + 1e-12      # standard error of the mean of seeds draws of +-s or 0
    z = (mean - g) / se
    near_normal = (p * seeds >= 10) & ((1 - p) * seeds >= 10)  # elsewhere the count of kept draws is too skewed for a z bound
    assert near_normal.sum() > n // 2 and np.abs(z[near_normal]).max() < 5.5, np.abs(z[near_normal]).max()
    assert abs(z.mean()) < 5 / np.sqrt(n)              # no common drift
    assert 0.9 < z.std() < 1.1                         # and the spread of independent draws
