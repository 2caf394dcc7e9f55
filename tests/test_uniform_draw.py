"""The noise the encoders draw themselves when called with a seed (hipress_amd/csrc/uniform_draw.h).
It is a definition of this library's own (the reference seeds its generator from the clock,
/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode_body.h:119), so what pins it is
agreement between three statements of it that share no code - the header the kernels compile (built
for the host with g++), the oracle's C restatement, and big-integer arithmetic here - plus the one
published constant on the way (the first SplitMix64 output) and what a uniform draw must satisfy."""
import os
import subprocess

import numpy as np
import pytest

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
M32, M64 = (1 << 32) - 1, (1 << 64) - 1


def mix32(x):
    x ^= x >> 17
    x = (x * 0xED5AD4BB) & M32
    x ^= x >> 11
    x = (x * 0xAC4C1B51) & M32
    x ^= x >> 15
    x = (x * 0x31848BAB) & M32
    x ^= x >> 14
    return x


def splitmix_out(state):
    z = state & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def tensor_key(seed, tensor):
    z = splitmix_out(seed + 0x9E3779B97F4A7C15)
    return mix32(((z & M32) ^ (z >> 32)) + tensor * 0x9E3779B9 & M32)


def draws(seed, tensor, n):
    k = tensor_key(seed, tensor)
    return np.array([(mix32(i ^ k) >> 8) / 2.0 ** 24 for i in range(n)], np.float64)


CASES = [(0, 0), (1, 0), (0, 1), (12345678901234567890, 7), (M64, M32), (2 ** 63, 390)]


def test_the_seed_fold_starts_from_the_published_splitmix64_output():
    # SplitMix64 seeded with 0 gives 0xe220a8397b1dcdaf first (Steele, Lea, Flood 2014; the
    # reference implementation's test vector): the state it is computed from is 0 + the increment
    assert splitmix_out(0x9E3779B97F4A7C15) == 0xE220A8397B1DCDAF
    assert tensor_key(0, 0) == mix32(0xE220A839 ^ 0x7B1DCDAF)
    assert oracle.uniform_tensor_key(0, 0) == tensor_key(0, 0)


# key and first four draws (as 24-bit integers) of four (seed, tensor) pairs, written down once all
# three statements agreed: a later change to any of them, or to all of them together, shows here
KNOWN = {
    (0, 0): (0x092F2145, [13811539, 2065571, 15705468, 8840272]),
    (1, 0): (0xB84203CC, [9904259, 5622144, 12988182, 16505780]),
    (0, 1): (0x24D05459, [7309036, 16073506, 8752362, 6634831]),
    (12345678901234567890, 7): (0x5DA3BDDE, [15492225, 11940634, 2635990, 5572268]),
}


def test_known_answers():
    for (seed, tensor), (key, first) in KNOWN.items():
        assert oracle.uniform_tensor_key(seed, tensor) == key == tensor_key(seed, tensor)
        assert [int(x * 2 ** 24) for x in oracle.uniform_draws(seed, 4, tensor)] == first


@pytest.mark.parametrize("seed,tensor", CASES)
def test_oracle_equals_the_big_integer_restatement(seed, tensor):
    assert oracle.uniform_tensor_key(seed, tensor) == tensor_key(seed, tensor)
    np.testing.assert_array_equal(oracle.uniform_draws(seed, 300, tensor).astype(np.float64), draws(seed, tensor, 300))


def test_the_header_the_kernels_compile_equals_the_oracle(tmp_path):
    exe = str(tmp_path / "uniform_draw_check")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-ffp-contract=off",
                           "-I", os.path.join(ROOT, "hipress_amd", "csrc"),
                           os.path.join(ROOT, "tests", "csrc", "uniform_draw_check.cpp"), "-o", exe])
    args = [str(x) for seed, tensor in CASES for x in (seed, tensor, 500)]
    lines = subprocess.run([exe] + args, capture_output=True, text=True, check=True).stdout.splitlines()
    assert len(lines) == len(CASES)
    for (seed, tensor), line in zip(CASES, lines):
        words = [int(w) for w in line.split()]
        assert words[0] == oracle.uniform_tensor_key(seed, tensor), (seed, tensor)
        got = np.array(words[1:], np.uint32).view(np.float32)
        np.testing.assert_array_equal(got, oracle.uniform_draws(seed, 500, tensor), err_msg=f"seed {seed} tensor {tensor}")


def test_draws_are_uniform_on_the_24_bit_grid_below_one():
    u = oracle.uniform_draws(2024, 1 << 22).astype(np.float64)
    assert u.min() >= 0.0 and u.max() < 1.0
    assert np.all(u * 2 ** 24 == np.floor(u * 2 ** 24))
    n = u.size
    assert abs(u.mean() - 0.5) < 4 / np.sqrt(12 * n)
    assert abs(u.var() - 1 / 12) < 1e-3
    counts = np.bincount((u * 256).astype(np.int64), minlength=256)
    chi2 = ((counts - n / 256) ** 2 / (n / 256)).sum()
    assert chi2 < 255 + 5 * np.sqrt(2 * 255)  # five sigma of a chi-square with 255 degrees of freedom
    assert abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 5 / np.sqrt(n)  # neighbours do not follow each other


def test_tensors_and_seeds_draw_apart():
    a = oracle.uniform_draws(5, 100000, 0)
    for other in (oracle.uniform_draws(5, 100000, 1), oracle.uniform_draws(6, 100000, 0)):
        assert (a == other).mean() < 1e-3
        assert abs(np.corrcoef(a, other)[0, 1]) < 0.02
    # every element index of a tensor has a draw of its own: a key only relabels them (a bijection)
    k = oracle.uniform_tensor_key(5, 0)
    idx = np.arange(1 << 16, dtype=np.uint64)
    assert len({mix32(int(i) ^ k) for i in idx[:4096]}) == 4096
