// Uniform draws made inside a kernel, for the stochastic quantisers called without a noise
// tensor.  Element i of tensor t (its place in a batch's table; 0 for a per-tensor call) of a
// call with seed s takes
//     u = (mix32(i ^ tensor_key(uniform_key(s), t)) >> 8) * 2^-24,
// a value on the 24-bit grid in [0, 1): exact in binary32, never 1.  mix32 is a bijection on 32-bit
// words (three multiplications, four xor-shifts: the "triple32" constants, whose output bits each
// flip with probability 1/2 +- 0.02 when an input bit does; the cheaper two-multiplication mixers
// leave consecutive indices visibly clumped: 4 M draws fell into 256 bins with twice the spread of
// a random sample), so
// over the 2^32 element indices of the largest tensor every grid value is drawn equally often;
// uniform_key folds the 64-bit seed to 32 bits on the host with the SplitMix64 finaliser, and
// tensor_key gives every tensor of a batch draws of its own (two tensors, or two partitions of
// one, would otherwise round alike element by element).  A counter-based generator: no state,
// the draw depends on nothing but (seed, t, i), so the same call gives the same payload wherever
// and however the kernel runs, and a CPU restatement can reproduce it.
// Plain C++ on purpose: the same lines run on the device, in the host part of the library and
// in a host-side unit test.
#pragma once
#include <cstdint>

#if defined(__HIPCC__)
#define HP_UD_FN __host__ __device__ __forceinline__
#else
#define HP_UD_FN inline
#endif

namespace hp {

HP_UD_FN uint32_t mix32(uint32_t x) {
    x ^= x >> 17;
    x *= 0xed5ad4bbu;
    x ^= x >> 11;
    x *= 0xac4c1b51u;
    x ^= x >> 15;
    x *= 0x31848babu;
    x ^= x >> 14;
    return x;
}

HP_UD_FN uint32_t uniform_key(uint64_t seed) {
    uint64_t z = seed + 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return (uint32_t)(z ^ (z >> 32));
}

HP_UD_FN uint32_t tensor_key(uint32_t key, uint32_t tensor) { return mix32(key + tensor * 0x9e3779b9u); }

// i: element index, key: the tensor's key
HP_UD_FN float uniform_at(uint32_t i, uint32_t key) { return (float)(mix32(i ^ key) >> 8) * 5.9604644775390625e-08f; }

}  // namespace hp
