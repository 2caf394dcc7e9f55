// Primitive library for operators generated from the CompLL operator language
// (hipress_amd/compll): the device-side pieces every generated operator is put
// together from, written for gfx950.  It takes the place of the Thrust calls
// the reference's generator emits (thrust::reduce / thrust::transform /
// thrust::copy in /root/reference/src/CompLL/GCGen/output/TernGradEncode/
// TernGradEncode_body.h:110-125), with three differences that matter on this
// hardware: several folds over the same vector share one sweep, scalars that
// come out of a reduction or a payload header stay on the device (no host
// round trip between launches), and packed codes are produced in place behind
// the header instead of in a temporary that is copied.
//
// Conventions.  A generated operator has a struct of host-known values (`Args`,
// passed to every kernel by value) and a struct of device-computed scalars
// (`Dev`, in the caller's workspace).  The user-written lambdas become static
// member functions of small structs that take both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "uniform_draw.h"

namespace cl {

typedef float f4 __attribute__((ext_vector_type(4)));
// 16 bytes at any dword address: one global_load_dwordx4 / global_store_dwordx4 either way,
// so float vectors need only the alignment of a float
typedef f4 f4u __attribute__((aligned(4)));

constexpr int kBlock = 256;   // threads per workgroup (four wave64 wavefronts)
constexpr int kTile = 4096;   // elements per workgroup in the sweeps
constexpr int kFinalBlock = 1024;

// ---- packed codes ---------------------------------------------------------------
// uint<bits> vectors live in bytes: code i at bit (i mod 8/bits)*bits of byte
// floor(i*bits/8), the placement the reference's decoder reads
// (/root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode_body.h:44).
// bits is one of 1, 2, 4, 8.
__device__ __forceinline__ bool valid_bits(int bits) { return bits == 1 || bits == 2 || bits == 4 || bits == 8; }

__device__ __forceinline__ int log2_per_byte(int bits) { return bits == 1 ? 3 : (bits == 2 ? 2 : (bits == 4 ? 1 : 0)); }

__device__ __forceinline__ unsigned get_code(const uint8_t* bytes, long long i, int bits) {
    const int sh = log2_per_byte(bits);
    return ((unsigned)bytes[i >> sh] >> ((int)(i & ((1 << sh) - 1)) * bits)) & ((1u << bits) - 1u);
}

// Conversion of a computed value to uint<bits>: saturating, NaN gives 0.
__device__ __forceinline__ unsigned to_code(float x, int bits) {
    const float top = (float)((1u << bits) - 1u);
    return x >= top ? (unsigned)top : (x > 0.f ? (unsigned)x : 0u);
}
__device__ __forceinline__ unsigned to_code(long long x, int bits) {
    const long long top = (1ll << bits) - 1;
    return (unsigned)(x < 0 ? 0 : (x > top ? top : x));
}
__device__ __forceinline__ unsigned to_code(int x, int bits) { return to_code((long long)x, bits); }
__device__ __forceinline__ unsigned to_code(unsigned x, int bits) { return to_code((long long)x, bits); }

// ---- header fields at any byte offset ----------------------------------------------
template <class T>
__device__ __forceinline__ void put(uint8_t* p, T v) {
    uint8_t raw[sizeof(T)];
    __builtin_memcpy(raw, &v, sizeof(T));
    for (unsigned k = 0; k < sizeof(T); ++k) p[k] = raw[k];
}
template <class T>
__device__ __forceinline__ T get(const uint8_t* p) {
    uint8_t raw[sizeof(T)];
    for (unsigned k = 0; k < sizeof(T); ++k) raw[k] = p[k];
    T v;
    __builtin_memcpy(&v, raw, sizeof(T));
    return v;
}

// ---- rounding noise -------------------------------------------------------------------
// random<float>(lo, hi) of the language reads an explicit uniform[0,1) tensor at
// the element being mapped, so that an operator is a function of its inputs; without such
// a tensor (NULL) the value is drawn from the call's key and the element's index
// (uniform_draw.h), which the caller's seed fixes: still a function of the inputs.
__device__ __forceinline__ float uniform_from(float u, float lo, float hi) { return lo + (hi - lo) * u; }
__device__ __forceinline__ float uniform_draw(const float* u, unsigned key, long long i, float lo, float hi) {
    return uniform_from(u ? u[i] : hp::uniform_at((uint32_t)i, key), lo, hi);
}

struct Nothing {
    template <class Args, class Dev>
    static __device__ void run(const Args&, Dev&) {}
};

// ---- serial block ------------------------------------------------------------------------
// Scalar statements that depend on device values (and header reads / writes) run
// in one thread between the sweeps.
template <class Args, class Dev, class Body>
__global__ void serial_kernel(Args a, Dev* d) {
    if (blockIdx.x == 0 && threadIdx.x == 0) Body::run(a, *d);
}

// ---- streamed operands ---------------------------------------------------------------------
// A lane owns four consecutive indices of each of four rows of 256 of its
// wavefront's 1024.  Fn::stream(a, k), k < Fn::NS, are the float vectors a lambda
// reads at its own index; they are loaded as 16-byte vectors, whole rows per wavefront.  A
// stream without a vector (NULL: the noise of random<float> when the caller passed a seed and
// no noise tensor; Fn::UNIFORM names that stream, -1: none) is drawn instead, element i taking
// hp::uniform_at(i, a.ukey).
// KEEP: plain loads, which leave their lines on the chip for the sweep that follows; the others are
// streamed.  (The empty statement keeps the compiler from folding the two otherwise identical
// branches into one, which would drop the streaming hint from both.)
template <class Args, class Fn, bool KEEP>
__device__ __forceinline__ void load_streams_as(const Args& a, long long base, long long count, f4 (&x)[Fn::NS > 0 ? Fn::NS : 1][4]) {
#pragma unroll
    for (int k = 0; k < Fn::NS; ++k) {
        const float* p = Fn::stream(a, k);
        const bool vec_ok = (reinterpret_cast<uintptr_t>(p) & 3u) == 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long long e = base + j * 256;
            if (k == Fn::UNIFORM && p == nullptr) {  // the same for every lane of the launch
                const uint32_t i = (uint32_t)e;
                x[k][j].x = e < count ? hp::uniform_at(i, a.ukey) : 0.f;
                x[k][j].y = e + 1 < count ? hp::uniform_at(i + 1u, a.ukey) : 0.f;
                x[k][j].z = e + 2 < count ? hp::uniform_at(i + 2u, a.ukey) : 0.f;
                x[k][j].w = e + 3 < count ? hp::uniform_at(i + 3u, a.ukey) : 0.f;
            } else if (e + 3 < count && vec_ok) {
                if (KEEP) {
                    asm volatile("");
                    x[k][j] = *reinterpret_cast<const f4u*>(p + e);
                } else {
                    x[k][j] = __builtin_nontemporal_load(reinterpret_cast<const f4u*>(p + e));
                }
            } else {
                x[k][j].x = e < count ? p[e] : 0.f;
                x[k][j].y = e + 1 < count ? p[e + 1] : 0.f;
                x[k][j].z = e + 2 < count ? p[e + 2] : 0.f;
                x[k][j].w = e + 3 < count ? p[e + 3] : 0.f;
            }
        }
    }
}
template <class Args, class Fn>
__device__ __forceinline__ void load_streams(const Args& a, long long base, long long count, f4 (&x)[Fn::NS > 0 ? Fn::NS : 1][4],
                                             bool keep = false) {
    if (keep) load_streams_as<Args, Fn, true>(a, base, count, x);
    else load_streams_as<Args, Fn, false>(a, base, count, x);
}

// A sweep that follows a reduce over the same vectors walks its tiles backwards (in groups of
// eight, so that consecutive workgroups still go to the eight XCDs in turn), and the reduce
// reads its last tiles with plain loads: a plain load leaves its line in the memory-side
// Infinity Cache (256 MiB), which a streamed load passes by, so the sweep begins with data
// that is still on the chip.  After a reduce over one vector the tail is as large as that
// cache; with more vectors 32 MiB in all (beyond that the plain loads cost the reduce what
// the sweep gains).
// (Build-time overrides for A/B measurements, as in common.h of the hand-written kernels.)
#ifndef HP_CACHE_TAIL_ONE_MIB
#define HP_CACHE_TAIL_ONE_MIB 256
#endif
#ifndef HP_CACHE_TAIL_MANY_MIB
#define HP_CACHE_TAIL_MANY_MIB 32
#endif
#ifndef HP_SECOND_PASS_REVERSED
#define HP_SECOND_PASS_REVERSED 1
#endif
__device__ __forceinline__ unsigned tile_reversed(unsigned b, unsigned nblocks) {
    const unsigned groups = nblocks >> 3, g = b >> 3;
    return (HP_SECOND_PASS_REVERSED) && g < groups ? (groups - 1 - g) * 8 + (b & 7u) : b;
}
__device__ __forceinline__ bool in_cache_tail(unsigned b, unsigned nblocks, unsigned streams) {
    const unsigned bytes = (streams <= 1u ? (unsigned)HP_CACHE_TAIL_ONE_MIB : (unsigned)HP_CACHE_TAIL_MANY_MIB) << 20;
    return b + bytes / ((streams ? streams : 1u) * (unsigned)kTile * 4u) >= nblocks && bytes != 0u;
}

// ---- reduce --------------------------------------------------------------------------------
// Folds::K folds over one float vector in one sweep.  Folds provides
//   static float init(const Args&, const Dev&, int k)
//   static float apply(const Args&, const Dev&, int k, float acc, float x)   (the user's lambda)
//   static void  store(Dev&, int k, float value)
// reduce(v, init, f) is f folded over init and the elements; as in any parallel
// reduce f has to be associative and commutative, and the order in which elements
// meet is this kernel's business.  init enters exactly once, at the very end, so f
// need not be idempotent in it (a sum with a non-zero init stays correct).
// Src says what is folded: count(a, d), NS / stream(a, k) and call(a, d, i, s) as for a
// map - a stored vector is the lambda that returns its one streamed operand, a
// mapped vector that is never stored is computed here, on the way into the fold.
template <class Args, class Dev, class Folds, class Src>
__global__ __launch_bounds__(kBlock) void reduce_tiles_kernel(Args a, const Dev* d, float* partial) {
    __shared__ float wave_acc[4][Folds::K];
    __shared__ int wave_any[4];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = Src::count(a, *d);
    const long long base = (long long)blockIdx.x * kTile + wave * 1024 + lane * 4;
    f4 in[Src::NS > 0 ? Src::NS : 1][4];
    load_streams<Args, Src>(a, base, n, in, in_cache_tail(blockIdx.x, gridDim.x, Src::NS));
    f4 x[4];
    unsigned ok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256;
        const long long left = n - e;
        ok[j] = left >= 4 ? 0xfu : (left <= 0 ? 0u : ((1u << left) - 1u));
        float s[4][Src::NS > 0 ? Src::NS : 1];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int k = 0; k < Src::NS; ++k) s[c][k] = in[k][j][c];
        if (ok[j] == 0xfu) {
            x[j].x = Src::call(a, *d, e, s[0]);
            x[j].y = Src::call(a, *d, e + 1, s[1]);
            x[j].z = Src::call(a, *d, e + 2, s[2]);
            x[j].w = Src::call(a, *d, e + 3, s[3]);
        } else {
            x[j].x = (ok[j] & 1u) ? Src::call(a, *d, e, s[0]) : 0.f;
            x[j].y = (ok[j] & 2u) ? Src::call(a, *d, e + 1, s[1]) : 0.f;
            x[j].z = (ok[j] & 4u) ? Src::call(a, *d, e + 2, s[2]) : 0.f;
            x[j].w = (ok[j] & 8u) ? Src::call(a, *d, e + 3, s[3]) : 0.f;
        }
    }
    float acc[Folds::K];
    bool any;  // whether acc holds at least one element yet
    if ((long long)(blockIdx.x + 1) * kTile <= n) {
        // a full tile: every lane has all sixteen elements, nothing to keep track of
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) acc[k] = x[0].x;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float xs[4] = {x[j].x, x[j].y, x[j].z, x[j].w};
#pragma unroll
            for (int c = (j == 0 ? 1 : 0); c < 4; ++c)
#pragma unroll
                for (int k = 0; k < Folds::K; ++k) acc[k] = Folds::apply(a, *d, k, acc[k], xs[c]);
        }
#pragma unroll
        for (int m = 1; m < 64; m <<= 1)
#pragma unroll
            for (int k = 0; k < Folds::K; ++k) acc[k] = Folds::apply(a, *d, k, acc[k], __shfl_xor(acc[k], m, 64));
        any = true;
    } else {
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) acc[k] = 0.f;
        any = false;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float xs[4] = {x[j].x, x[j].y, x[j].z, x[j].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const bool have = (ok[j] >> c) & 1u;
#pragma unroll
                for (int k = 0; k < Folds::K; ++k)
                    acc[k] = have ? (any ? Folds::apply(a, *d, k, acc[k], xs[c]) : xs[c]) : acc[k];
                any = any || have;
            }
        }
#pragma unroll
        for (int m = 1; m < 64; m <<= 1) {
            const bool other_any = __shfl_xor((int)any, m, 64) != 0;
#pragma unroll
            for (int k = 0; k < Folds::K; ++k) {
                const float other = __shfl_xor(acc[k], m, 64);
                acc[k] = (any && other_any) ? Folds::apply(a, *d, k, acc[k], other) : (any ? acc[k] : other);
            }
            any = any || other_any;
        }
    }
    if (lane == 0) {
        wave_any[wave] = any;
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) wave_acc[wave][k] = acc[k];
    }
    __syncthreads();
    if (threadIdx.x == 0) {  // the first wavefront of a launched tile always holds an element
        float t[Folds::K];
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) t[k] = wave_acc[0][k];
        for (int w = 1; w < 4; ++w)
            if (wave_any[w]) {
#pragma unroll
                for (int k = 0; k < Folds::K; ++k) t[k] = Folds::apply(a, *d, k, t[k], wave_acc[w][k]);
            }
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) partial[(long long)blockIdx.x * Folds::K + k] = t[k];
    }
}

// One workgroup folds the per-tile results (every tile of a launch holds at least
// one element), combines them with the initial values and stores the K results.
// With no tile at all the results are the initial values.
// After::run: the scalar statements that follow the reduce in the program, if any.
template <class Args, class Dev, class Folds, class After>
__global__ __launch_bounds__(kFinalBlock) void reduce_final_kernel(Args a, Dev* d, const float* partial, unsigned ntiles) {
    constexpr int kWaves = kFinalBlock / 64;
    __shared__ float wave_acc[kWaves][Folds::K];
    __shared__ int wave_any[kWaves];
    float acc[Folds::K];
#pragma unroll
    for (int k = 0; k < Folds::K; ++k) acc[k] = 0.f;
    bool any = false;
    unsigned t = threadIdx.x;
    for (; t + 3 * kFinalBlock < ntiles; t += 4 * kFinalBlock) {  // four rows of loads in flight per lane
        float p[4][Folds::K];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int k = 0; k < Folds::K; ++k) p[u][k] = partial[(long long)(t + u * kFinalBlock) * Folds::K + k];
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) {
            const float q = Folds::apply(a, *d, k, Folds::apply(a, *d, k, p[0][k], p[1][k]),
                                         Folds::apply(a, *d, k, p[2][k], p[3][k]));
            acc[k] = any ? Folds::apply(a, *d, k, acc[k], q) : q;
        }
        any = true;
    }
    for (; t < ntiles; t += kFinalBlock) {
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) {
            const float p = partial[(long long)t * Folds::K + k];
            acc[k] = any ? Folds::apply(a, *d, k, acc[k], p) : p;
        }
        any = true;
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const bool other_any = __shfl_xor((int)any, m, 64) != 0;
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) {
            const float other = __shfl_xor(acc[k], m, 64);
            acc[k] = (any && other_any) ? Folds::apply(a, *d, k, acc[k], other) : (any ? acc[k] : other);
        }
        any = any || other_any;
    }
    if ((threadIdx.x & 63u) == 0) {
        wave_any[threadIdx.x >> 6] = any;
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) wave_acc[threadIdx.x >> 6][k] = acc[k];
    }
    __syncthreads();
    if (threadIdx.x == 0) {  // lanes are filled from thread 0 upwards, so wavefront 0 holds a value whenever any does
        for (int w = 1; w < kWaves; ++w)
            if (wave_any[w]) {
#pragma unroll
                for (int k = 0; k < Folds::K; ++k) acc[k] = Folds::apply(a, *d, k, acc[k], wave_acc[w][k]);
            }
#pragma unroll
        for (int k = 0; k < Folds::K; ++k) {
            const float init = Folds::init(a, *d, k);
            Folds::store(*d, k, any ? Folds::apply(a, *d, k, init, acc[k]) : init);
        }
        After::run(a, *d);
    }
}

// ---- map ---------------------------------------------------------------------------------------
// Fn describes the mapped lambda:
//   count(a, d)              length of the range
//   NS, stream(a, k)         the float vectors the lambda reads at its own index (its
//                            random draws among them); the kernel loads them as 16-byte
//                            vectors, whole rows per wavefront, and hands the lambda values
//   call(a, d, i, s)         the lambda; s[k] is the element of stream k at index i
//   bits(a, d)               (packed maps) width of the codes
// A lane owns four consecutive indices of each of four rows of 256, as in the other
// operators of this library.

// Before::run: scalar statements that precede the sweep and may be run again freely.
// Every workgroup runs them into its own copy of the device scalars and works from
// that copy; the first workgroup also publishes it.  With Nothing the scalars are
// read where they are.
template <class Args, class Dev, class Before>
__device__ __forceinline__ const Dev* device_scalars(const Args& a, Dev* d, Dev* mine) {
    if (std::is_same<Before, Nothing>::value) return d;
    if (threadIdx.x == 0) {
        *mine = *d;
        Before::run(a, *mine);
        if (blockIdx.x == 0) *d = *mine;
    }
    __syncthreads();
    return mine;
}

// out[i] = Fn::call(...) for i < min(count, cap).
template <class Args, class Dev, class Fn, class Before>
__global__ __launch_bounds__(kBlock) void map_float_kernel(Args a, Dev* dglobal, float* out, long long cap) {
    __shared__ Dev mine;
    const Dev* d = device_scalars<Args, Dev, Before>(a, dglobal, &mine);
    long long count = Fn::count(a, *d);
    if (count > cap) count = cap;
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long base = (long long)blockIdx.x * kTile + wave * 1024 + lane * 4;
    const bool vec_ok = (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    f4 x[Fn::NS > 0 ? Fn::NS : 1][4];
    load_streams<Args, Fn>(a, base, count, x);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256;
        float s[4][Fn::NS > 0 ? Fn::NS : 1];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int k = 0; k < Fn::NS; ++k) s[c][k] = x[k][j][c];
        if (e + 3 < count && vec_ok) {  // the common case carries no per-element test
            f4 q;
            q.x = Fn::call(a, *d, e, s[0]);
            q.y = Fn::call(a, *d, e + 1, s[1]);
            q.z = Fn::call(a, *d, e + 2, s[2]);
            q.w = Fn::call(a, *d, e + 3, s[3]);
            __builtin_nontemporal_store(q, reinterpret_cast<f4u*>(out + e));
        } else {
            for (int c = 0; c < 4; ++c)
                if (e + c < count) out[e + c] = Fn::call(a, *d, e + c, s[c]);
        }
    }
}

// bytes[...] = packed Fn::call(...) for i < count.  A lane's four codes of a row are
// 4 * bits bits: half a byte, one, two or four bytes; with 1-bit codes two lanes share
// a byte and the even one writes it.  The pad bits of the last byte are written as zero.
template <class Args, class Dev, class Fn, class Before>
__global__ __launch_bounds__(kBlock) void map_packed_kernel(Args a, Dev* dglobal, uint8_t* bytes, long long cap_bytes) {
    __shared__ Dev mine;
    const Dev* d = device_scalars<Args, Dev, Before>(a, dglobal, &mine);
    const int bits = Fn::bits(a, *d);
    if (!valid_bits(bits)) return;
    const long long count = Fn::count(a, *d);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long base = (long long)tile_reversed(blockIdx.x, gridDim.x) * kTile + wave * 1024 + lane * 4;
    if (base - lane * 4 >= count) return;  // the whole wavefront leaves together
    f4 x[Fn::NS > 0 ? Fn::NS : 1][4];
    load_streams<Args, Fn>(a, base, count, x);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256;
        float s[4][Fn::NS > 0 ? Fn::NS : 1];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int k = 0; k < Fn::NS; ++k) s[c][k] = x[k][j][c];
        unsigned chunk = 0;
        if (e + 3 < count) {  // the common case carries no per-element test
#pragma unroll
            for (int c = 0; c < 4; ++c) chunk |= to_code(Fn::call(a, *d, e + c, s[c]), bits) << (c * bits);
        } else {
            for (int c = 0; c < 4; ++c)
                if (e + c < count) chunk |= to_code(Fn::call(a, *d, e + c, s[c]), bits) << (c * bits);
        }
        if (bits == 8) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (e + c < count && e + c < cap_bytes) bytes[e + c] = (uint8_t)(chunk >> (8 * c));
        } else if (bits == 4) {
            if (e < count && e / 2 < cap_bytes) bytes[e / 2] = (uint8_t)chunk;
            if (e + 2 < count && e / 2 + 1 < cap_bytes) bytes[e / 2 + 1] = (uint8_t)(chunk >> 8);
        } else if (bits == 2) {
            if (e < count && e / 4 < cap_bytes) bytes[e / 4] = (uint8_t)chunk;
        } else {
            const unsigned other = (unsigned)__shfl_xor((int)chunk, 1, 64);
            if ((lane & 1u) == 0 && e < count && e / 8 < cap_bytes) bytes[e / 8] = (uint8_t)(chunk | (other << 4));
        }
    }
}

// Two maps over the same range in one sweep: packed codes and a float vector (the shape
// of a quantiser that also updates its error-feedback residual).  Fn provides count,
// NS / stream for the operands of both lambdas, bits, call_codes and call_values.  All
// operands of a thread are loaded before its first store, so the float output may be
// one of the operands (an update in place).
template <class Args, class Dev, class Fn, class Before>
__global__ __launch_bounds__(kBlock) void map_fused_kernel(Args a, Dev* dglobal, uint8_t* bytes, long long cap_bytes,
                                                           float* out) {
    __shared__ Dev mine;
    const Dev* d = device_scalars<Args, Dev, Before>(a, dglobal, &mine);
    const int bits = Fn::bits(a, *d);
    if (!valid_bits(bits)) return;
    const long long count = Fn::count(a, *d);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long base = (long long)tile_reversed(blockIdx.x, gridDim.x) * kTile + wave * 1024 + lane * 4;
    if (base - lane * 4 >= count) return;  // the whole wavefront leaves together
    const bool vec_ok = (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    f4 x[Fn::NS > 0 ? Fn::NS : 1][4];
    load_streams<Args, Fn>(a, base, count, x);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256;
        float s[4][Fn::NS > 0 ? Fn::NS : 1];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int k = 0; k < Fn::NS; ++k) s[c][k] = x[k][j][c];
        unsigned chunk = 0;
        if (e + 3 < count) {
            f4 q;
#pragma unroll
            for (int c = 0; c < 4; ++c) chunk |= to_code(Fn::call_codes(a, *d, e + c, s[c]), bits) << (c * bits);
            q.x = Fn::call_values(a, *d, e, s[0]);
            q.y = Fn::call_values(a, *d, e + 1, s[1]);
            q.z = Fn::call_values(a, *d, e + 2, s[2]);
            q.w = Fn::call_values(a, *d, e + 3, s[3]);
            if (vec_ok) {
                __builtin_nontemporal_store(q, reinterpret_cast<f4u*>(out + e));
            } else {
                out[e] = q.x;
                out[e + 1] = q.y;
                out[e + 2] = q.z;
                out[e + 3] = q.w;
            }
        } else {
            for (int c = 0; c < 4; ++c)
                if (e + c < count) {
                    chunk |= to_code(Fn::call_codes(a, *d, e + c, s[c]), bits) << (c * bits);
                    out[e + c] = Fn::call_values(a, *d, e + c, s[c]);
                }
        }
        if (bits == 8) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (e + c < count && e + c < cap_bytes) bytes[e + c] = (uint8_t)(chunk >> (8 * c));
        } else if (bits == 4) {
            if (e < count && e / 2 < cap_bytes) bytes[e / 2] = (uint8_t)chunk;
            if (e + 2 < count && e / 2 + 1 < cap_bytes) bytes[e / 2 + 1] = (uint8_t)(chunk >> 8);
        } else if (bits == 2) {
            if (e < count && e / 4 < cap_bytes) bytes[e / 4] = (uint8_t)chunk;
        } else {
            const unsigned other = (unsigned)__shfl_xor((int)chunk, 1, 64);
            if ((lane & 1u) == 0 && e < count && e / 8 < cap_bytes) bytes[e / 8] = (uint8_t)(chunk | (other << 4));
        }
    }
}

}  // namespace cl
