"""Counter-based synthetic inputs: element i of tensor t of a set drawn with seed s is a
function of (s, t, i) alone, so the values do not depend on the order in which tensors
are generated, on the device they are generated on, or on the random-number engine of
any library.

The integer part is SplitMix64 (the 64-bit finaliser Vigna published with xoshiro): the
key of a tensor is mix(mix(seed) + tensor), the word of element i is mix(key + i * GOLDEN)
with GOLDEN = 0x9E3779B97F4A7C15.  It runs on int64 tensors, whose additions and
multiplications wrap like unsigned 64-bit arithmetic.  From one word come
  * a uniform in [0, 1): the top 24 bits times 2**-24 (exact in float32, never 1.0);
  * a standard normal by Box-Muller in float64 from the top 24 bits (offset to (0, 1]) and
    the next 24 bits, rounded once to float32.  Logarithm, square root and cosine are the
    library's: two libraries can disagree in the last place of the float64 result, which
    changes the float32 value for about one element in 10**8.
"""
import math

import torch

_MASK64 = (1 << 64) - 1
GOLDEN = 0x9E3779B97F4A7C15
_M1 = 0xBF58476D1CE4E5B9
_M2 = 0x94D049BB133111EB


def _signed(x):
    """The int64 with the bit pattern of the unsigned 64-bit x."""
    x &= _MASK64
    return x - (1 << 64) if x >> 63 else x


def mix_int(x):
    """SplitMix64's output function of the state x + GOLDEN, on Python integers."""
    z = (x + GOLDEN) & _MASK64
    z = ((z ^ (z >> 30)) * _M1) & _MASK64
    z = ((z ^ (z >> 27)) * _M2) & _MASK64
    return z ^ (z >> 31)


def _lsr(z, k):
    """Logical right shift of an int64 tensor."""
    return (z >> k) & ((1 << (64 - k)) - 1)


def mix(x):
    """mix_int on an int64 tensor (bit patterns of unsigned 64-bit words)."""
    z = x + _signed(GOLDEN)
    z = (z ^ _lsr(z, 30)) * _signed(_M1)
    z = (z ^ _lsr(z, 27)) * _signed(_M2)
    return z ^ _lsr(z, 31)


def tensor_key(seed, tensor):
    return mix_int((mix_int(seed & _MASK64) + tensor) & _MASK64)


def words(seed, tensor, n, device, start=0):
    """The 64-bit words of elements start .. start + n - 1 of tensor `tensor` (int64 bit patterns)."""
    i = torch.arange(start, start + n, dtype=torch.int64, device=device)
    return mix(i * _signed(GOLDEN) + _signed(tensor_key(seed, tensor)))


_CHUNK = 1 << 24  # elements generated at a time (bounds the int64 / float64 temporaries)


def _fill(n, device, seed, tensor, fn):
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, _CHUNK):
        k = min(_CHUNK, n - lo)
        out[lo:lo + k] = fn(words(seed, tensor, k, device, lo))
    return out


def uniform(n, device, seed, tensor=0):
    """U[0, 1) float32 from 24 bits per element: 1.0 is never produced."""
    return _fill(n, device, seed, tensor, lambda w: _lsr(w, 40).to(torch.float32) * (1.0 / (1 << 24)))


def normal(n, device, seed, tensor=0, sigma=1.0):
    """N(0, sigma) float32 (Box-Muller in float64, one rounding to float32, then the scale)."""
    def f(w):
        u1 = (_lsr(w, 40) + 1).to(torch.float64) * (1.0 / (1 << 24))          # (0, 1]
        u2 = (_lsr(w, 16) & 0xFFFFFF).to(torch.float64) * (1.0 / (1 << 24))   # [0, 1)
        g = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2)
        return g.to(torch.float32) * sigma
    return _fill(n, device, seed, tensor, f)


def bernoulli(n, device, seed, tensor, p):
    """True with probability p (24-bit resolution)."""
    thr = int(round(p * (1 << 24)))
    out = torch.empty(n, dtype=torch.bool, device=device)
    for lo in range(0, n, _CHUNK):
        k = min(_CHUNK, n - lo)
        out[lo:lo + k] = _lsr(words(seed, tensor, k, device, lo), 40) < thr
    return out


def scalar_uniform(seed, tensor):
    """One U[0, 1) double for a tensor (e.g. its own sigma), from the tensor's key."""
    return (mix_int(tensor_key(seed, tensor)) >> 11) * (1.0 / (1 << 53))
