// Shared device/host definitions for the gfx950 gradient-compression kernels.
//
// Work decomposition used by every dense kernel: a tensor is cut into tiles of
// kTile = 4096 consecutive elements; one 256-thread workgroup (four wave64
// wavefronts) owns a tile, wavefront w owns the 1024 consecutive elements
// [w*1024, +1024) of it, and in step j (0..3) lane l of that wavefront holds the
// four elements at offset j*256 + 4*l as one 16-byte vector.  Every global
// access of a wavefront is therefore one contiguous, fully used 1 KiB row, and
// the 2-bit (1-bit) codes of four (eight) neighbouring lanes form one dense
// uint32 word.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "uniform_draw.h"

namespace hp {

typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;       // threads per workgroup
constexpr int kWaveTile = 1024;   // elements per wavefront per tile
constexpr int kTile = 4096;       // elements per workgroup
constexpr int kHeaderBytes = 16;
constexpr int kMaxPeers = 16;
constexpr int kSampleStride = 100;      // sparse: every 100th element of a large tensor is a sample
constexpr long long kSampleFrom = 262144;  // sparse: tensors at least this large are sampled
// sparse: the threshold's 31 key bits are found 12 + 12 + 7 at a time, one histogram each
constexpr unsigned kSelBins = 4096, kSelBinsLast = 128;
constexpr unsigned kSelShift0 = 19, kSelShift1 = 7;
constexpr unsigned kSelHistWords = 2 * kSelBins + kSelBinsLast;  // per tensor

// One tensor (or one chunk) as the kernels see it.  Batched launches index a
// device-resident array of these through a tile map; single-tensor launches
// carry one by value in the kernel arguments.
struct Seg {
    const float* g;    // gradient in
    float* s0;         // residual (onebit, tbq) | momentum (dgc; NULL for graddrop)
    float* s1;         // accumulator (dgc, graddrop)
    const float* u;    // uniform noise (terngrad)
    uint8_t* pay;      // payload base (header)
    float* out;        // decode output / aggregate
    unsigned long long n;
    unsigned int tile0;      // index of this tensor's first tile among all tiles of the launch
    unsigned int ntiles;     // tiles of this tensor
    unsigned int words_off;  // byte offset of the packed words from the payload base
    unsigned int bucket;     // terngrad bucket size
    unsigned int aligned;    // 1 when the 16-byte vector path may be used (every fp32 pointer a multiple of 4)
    unsigned int cap;        // sparse capacity
    float f0;                // tbq threshold | dgc momentum factor
    unsigned int ks;         // sparse: rank of the threshold inside the sample
    unsigned int sstride;    // sparse: sample stride
    unsigned int ns;         // sparse: sample count
    unsigned long long ws0;  // sparse: element offset of this tensor's sample slice
    unsigned int id;         // index of this tensor in the launch's table
    unsigned int nsblk;      // sparse: workgroups the select passes spend on this tensor
    unsigned int ncblk;      // sparse decode: workgroups of 1024 payload slots
    unsigned int pad0;
    unsigned long long pay_bytes;  // size of the payload buffer (decode-side bounds checks)
};

// Peers of one chunk for decode-and-merge.
struct MergeSeg {
    const uint8_t* peer[kMaxPeers];
    unsigned long long peer_bytes[kMaxPeers];  // size of each peer's buffer
    unsigned int peer_slots[kMaxPeers];  // sparse: pairs each peer's buffer has room for
    Seg s;  // out = aggregate, s0 = aggregator residual (tbq), pay = re-encoded payload
    Seg r;  // sparse re-encode of the aggregate (GradDrop descriptor: s1 = accumulator, pay = out payload)
};

// where(k) = {tensor index, tile index inside the tensor} of tile k of the launch;
// seg(i) = descriptor of tensor i, whose id is i and whose tiles are the launch's
// tiles tile0 .. tile0 + ntiles - 1, so k = tile0 + tile index.
struct SingleSrc {
    Seg seg;
    unsigned base;  // first tile of this launch when a tensor's tiles are spread over several launches
    __device__ __forceinline__ const Seg& get(unsigned& tile, unsigned blk) const {
        tile = blk + base;
        return seg;
    }
    __device__ __forceinline__ uint2 where(unsigned blk) const { return make_uint2(0u, blk); }
    __device__ __forceinline__ const Seg& at(unsigned) const { return seg; }
};

struct BatchSrc {
    const Seg* segs;
    const uint2* map;  // per workgroup: {tensor index, tile index inside the tensor}
    __device__ __forceinline__ const Seg& get(unsigned& tile, unsigned blk) const {
        uint2 m = map[blk];
        tile = m.y;
        return segs[m.x];
    }
    __device__ __forceinline__ uint2 where(unsigned blk) const { return map[blk]; }
    __device__ __forceinline__ const Seg& at(unsigned i) const { return segs[i]; }
};

// Per-tensor (not per-tile) launches: workgroup i works on tensor i.
struct SingleSegSrc {
    Seg seg;
    __device__ __forceinline__ const Seg& at(unsigned) const { return seg; }
};

struct BatchSegSrc {
    const Seg* segs;
    __device__ __forceinline__ const Seg& at(unsigned i) const { return segs[i]; }
};

struct MergeSingleSegSrc {
    MergeSeg seg;
    __device__ __forceinline__ const MergeSeg& at(unsigned) const { return seg; }
};

struct MergeBatchSegSrc {
    const MergeSeg* segs;
    __device__ __forceinline__ const MergeSeg& at(unsigned i) const { return segs[i]; }
};

struct MergeSingleSrc {
    MergeSeg seg;
    __device__ __forceinline__ const MergeSeg& get(unsigned& tile, unsigned blk) const {
        tile = blk;
        return seg;
    }
};

struct MergeBatchSrc {
    const MergeSeg* segs;
    const uint2* map;
    __device__ __forceinline__ const MergeSeg& get(unsigned& tile, unsigned blk) const {
        uint2 m = map[blk];
        tile = m.y;
        return segs[m.x];
    }
};

#ifdef __HIPCC__
// ---- memory access ---------------------------------------------------------
// Streaming data is touched exactly once, so loads and stores carry the
// non-temporal hint.  The fp32 arrays need only be 4-byte aligned: a 16-byte access to
// global memory is one instruction at any dword address (the vector type below says
// "aligned to 4", and the compiler emits the same global_load_dwordx4 / global_store_dwordx4
// for it as for a 16-byte aligned one), so a view that starts a few floats into an
// allocation takes the same path as the allocation itself.
typedef f4 f4u __attribute__((aligned(4)));
__device__ __forceinline__ f4 ld4(const float* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const f4u*>(p));
}
__device__ __forceinline__ void st4(float* p, f4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<f4u*>(p));
}
// Element-wise variants for partial tiles.
__device__ __forceinline__ f4 ld4_guard(const float* p, long long e, long long n) {
    f4 v = {0.f, 0.f, 0.f, 0.f};
    if (e < n) v.x = p[e];
    if (e + 1 < n) v.y = p[e + 1];
    if (e + 2 < n) v.z = p[e + 2];
    if (e + 3 < n) v.w = p[e + 3];
    return v;
}
__device__ __forceinline__ void st4_guard(float* p, long long e, long long n, f4 v) {
    if (e < n) p[e] = v.x;
    if (e + 1 < n) p[e + 1] = v.y;
    if (e + 2 < n) p[e + 2] = v.z;
    if (e + 3 < n) p[e + 3] = v.w;
}
template <bool FAST>
__device__ __forceinline__ f4 load4(const float* p, long long e, long long n) {
    if (FAST) return ld4(p + e);
    return ld4_guard(p, e, n);
}
template <bool FAST>
__device__ __forceinline__ void store4(float* p, long long e, long long n, f4 v) {
    if (FAST) st4(p + e, v);
    else st4_guard(p, e, n, v);
}
// The noise of the stochastic quantisers for the four elements from e on: read from the noise
// tensor, or (DRAW) drawn from the tensor's key and the element's index (uniform_draw.h).
template <bool FAST, bool DRAW>
__device__ __forceinline__ f4 noise4(const float* u, long long e, long long n, unsigned key) {
    if (DRAW) {
        const uint32_t i = (uint32_t)e;  // element counts fit 32 bits
        f4 v;
        v.x = uniform_at(i, key);
        v.y = uniform_at(i + 1u, key);
        v.z = uniform_at(i + 2u, key);
        v.w = uniform_at(i + 3u, key);
        if (!FAST) {  // places beyond the tensor draw 0, as they read 0 from a noise tensor
            if (e + 3 >= n) v.w = 0.f;
            if (e + 2 >= n) v.z = 0.f;
            if (e + 1 >= n) v.y = 0.f;
            if (e >= n) v.x = 0.f;
        }
        return v;
    }
    return load4<FAST>(u, e, n);
}
// bit k set when element e+k exists
__device__ __forceinline__ unsigned valid4(long long e, long long n) {
    long long left = n - e;
    return left >= 4 ? 0xfu : (left <= 0 ? 0u : ((1u << left) - 1u));
}

// ---- occupancy --------------------------------------------------------------------
// The plain streaming kernels move most bytes with four wavefronts per SIMD, not with the
// eight their few registers would allow.  Naming a high register as clobbered makes the
// kernel claim 104 of the 512 vector registers of a SIMD lane, which is that limit; set
// this way it is worth about 1 % over the same limit set with idle LDS at launch (TBQ
// encode 270 -> 266 us on the VGG19 set), which the kernels that do better with five
// workgroups per CU, or with a limit that depends on the launch's size, still use.
__device__ __forceinline__ void four_waves_per_simd() { asm volatile("" ::: "v103"); }

// ---- workgroup -> tile order ----------------------------------------------------
// Consecutive workgroup ids are dealt to the eight XCDs in turn, so with the plain
// order every XCD (and its L2) writes every eighth 16 KiB tile.  Kernels that mostly
// write do better when an XCD's tiles are neighbours: of every 64 consecutive tiles,
// XCD x takes tiles 8x .. 8x+7.  The tail that does not fill a group of 64 keeps
// the plain order.  A permutation of [0, nblocks).
__device__ __forceinline__ unsigned xcd_grouped(unsigned b, unsigned nblocks) {
    return b < (nblocks & ~63u) ? ((b & ~63u) | ((b & 7u) << 3) | ((b >> 3) & 7u)) : b;
}

// Two-pass operators (a reduction over the tensor, then the pass that needs its result) read
// the same arrays twice.  What the first pass read last can still be on the chip when the
// second pass starts: not in the L2s (the counter of L2-to-fabric read traffic, FETCH_SIZE,
// reads the same with and without what follows) but in the memory-side Infinity Cache behind
// them (256 MiB, shared by all XCDs), which a streamed (non-temporal) load passes by and a
// plain load fills.  So the first pass reads the last tiles of its launch with plain loads
// (cache_tail) and the second pass walks the launch backwards (xcd_reversed), in groups of
// eight so that consecutive workgroups still go to the eight XCDs in turn.  Both halves are
// needed: on the same GPU, alternating libraries, the quantise pass of onebit over the VGG19
// set takes 256.8 us with both, 262.6 us with only the reversed order and 259.7 us with
// neither; the code pass of the min/max quantiser over 102.8 M elements 133.0 us with a
// 32 MiB tail and the reversed order, 136.2 us with the order alone, 134.8 us with neither.
// How much to leave behind depends on what the second pass does besides re-reading.  After
// one read stream (the min/max quantiser) the gain grows up to the cache's size: tails of
// 0 / 32 / 64 / 128 / 192 / 256 / 384 MiB take min/max + code pass 192.7 / 190.3 / 189.3 /
// 187.9 / 186.3 / 185.3 / 186.7 us (the plain loads cost the first pass 1 us per 64 MiB, the
// second pass gains 2.5).  After two read streams whose second pass also writes one of them
// back (onebit) nothing is gained beyond 32 MiB: what the second pass saves, the first loses.
//
// Tuning constants, overridable at build time for A/B measurements
// (python -m hipress_amd.build --define HP_CACHE_TAIL_ONE_MIB=0 ...): MiB read with plain loads
// at the end of a first pass over one / over several fp32 arrays (0 = none), and whether the
// second pass is walked backwards.
#ifndef HP_CACHE_TAIL_ONE_MIB
#define HP_CACHE_TAIL_ONE_MIB 256
#endif
#ifndef HP_CACHE_TAIL_MANY_MIB
#define HP_CACHE_TAIL_MANY_MIB 32
#endif
#ifndef HP_SECOND_PASS_REVERSED
#define HP_SECOND_PASS_REVERSED 1
#endif
// A permutation of [0, nblocks).
__device__ __forceinline__ unsigned xcd_reversed(unsigned b, unsigned nblocks) {
    const unsigned groups = nblocks >> 3, g = b >> 3;
    return (HP_SECOND_PASS_REVERSED) && g < groups ? (groups - 1 - g) * 8 + (b & 7u) : b;
}
// True for the last tiles of a launch that reads `streams` fp32 arrays: plain loads there.
__device__ __forceinline__ bool cache_tail(unsigned b, unsigned nblocks, unsigned streams) {
    const unsigned bytes = (streams <= 1u ? (unsigned)HP_CACHE_TAIL_ONE_MIB : (unsigned)HP_CACHE_TAIL_MANY_MIB) << 20;
    return b + bytes / ((streams ? streams : 1u) * kTile * 4u) >= nblocks && bytes != 0u;
}
// (The empty statement keeps the compiler from folding a branch of such loads into an
// otherwise identical branch of streamed ones, which would make all of them plain.)
__device__ __forceinline__ f4 ld4_keep(const float* p) {
    asm volatile("");
    return *reinterpret_cast<const f4u*>(p);
}

// ---- bucket arithmetic --------------------------------------------------------
// Element first + off (off < 8192) lies in bucket q, at place r inside it, given that element
// `first` lies in bucket q0 at place r0 and buckets hold B elements: a 32-bit division, or a
// comparison when a bucket is longer than the stretch looked at.  The 64-bit division that
// places `first` is done once per wavefront on uniform values; per element it would cost more
// than everything else a decoder does.
struct BucketPos {
    long long q;
    unsigned long long r;
};
__device__ __forceinline__ BucketPos bucket_pos(long long q0, unsigned long long r0, unsigned off, unsigned long long B) {
    const unsigned long long x = r0 + off;
    BucketPos p;
    if (B <= 8192ull) {
        const unsigned xq = (unsigned)x / (unsigned)B;
        p.q = q0 + xq;
        p.r = x - (unsigned long long)xq * B;
    } else {
        const bool over = x >= B;
        p.q = q0 + (over ? 1 : 0);
        p.r = over ? x - B : x;
    }
    return p;
}

// ---- cross-lane -------------------------------------------------------------
// quad_perm broadcast of lane k of every group of four lanes (DPP, no LDS traffic)
template <int K>
__device__ __forceinline__ unsigned quad_bcast(unsigned x) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, K * 0x55, 0xf, 0xf, false);
}
// Four neighbouring lanes each hold 8 bits; all four receive the 32-bit word
// with lane (4q+k)'s byte at bits [8k, 8k+8).
__device__ __forceinline__ unsigned quad_pack8(unsigned byte) {
    return quad_bcast<0>(byte) | (quad_bcast<1>(byte) << 8) | (quad_bcast<2>(byte) << 16) |
           (quad_bcast<3>(byte) << 24);
}
// Eight neighbouring lanes each hold 4 bits; all eight receive the word with
// lane (8o+k)'s nibble at bits [4k, 4k+4).
__device__ __forceinline__ unsigned oct_pack4(unsigned nib, unsigned lane) {
    unsigned h = quad_bcast<0>(nib) | (quad_bcast<1>(nib) << 4) | (quad_bcast<2>(nib) << 8) |
                 (quad_bcast<3>(nib) << 12);
    unsigned o = (unsigned)__shfl_xor((int)h, 4, 64);
    return (lane & 4u) ? (o | (h << 16)) : (h | (o << 16));
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
    return x;
}
// Maximum over the 64 lanes, the same value in every lane: data-parallel-primitive steps
// inside every row of 16 lanes, then across the rows (a maximum does not depend on the
// order it is taken in).  All 64 lanes must be active.
__device__ __forceinline__ float wave_max(float x) {
#define HP_MAX_STEP(CTRL, ROWS)                                                                                   \
    {                                                                                                             \
        const float y = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), CTRL, ROWS, 0xf, false)); \
        x = y > x ? y : x;                                                                                        \
    }
    HP_MAX_STEP(0xB1, 0xf)   // quad_perm [1,0,3,2]
    HP_MAX_STEP(0x4E, 0xf)   // quad_perm [2,3,0,1]
    HP_MAX_STEP(0x141, 0xf)  // row_half_mirror
    HP_MAX_STEP(0x140, 0xf)  // row_mirror
    HP_MAX_STEP(0x142, 0xa)  // row_bcast:15 into rows 1, 3
    HP_MAX_STEP(0x143, 0xc)  // row_bcast:31 into rows 2, 3
#undef HP_MAX_STEP
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}
// Inclusive prefix sum over the 64 lanes in six data-parallel-primitive steps:
// four shifts inside every row of 16 lanes, then lane 15 of rows 0 and 2 is added
// to the row after it, then lane 31 to the upper two rows.  All 64 lanes must be active
// where it is called (a lane that is switched off would be read as garbage by its
// neighbours).
__device__ __forceinline__ unsigned wave_incl_scan_u(unsigned x) {
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, true);   // row_shr:1
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, true);   // row_shr:2
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, true);   // row_shr:4
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, true);   // row_shr:8
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return x;
}
// Sum over the 64 lanes, the same value (wavefront-uniform) in every lane.
// The same for unsigned keys.
__device__ __forceinline__ unsigned wave_umax(unsigned x) {
#define HP_UMAX_STEP(CTRL, ROWS)                                                                       \
    {                                                                                                 \
        const unsigned y = (unsigned)__builtin_amdgcn_update_dpp((int)x, (int)x, CTRL, ROWS, 0xf, false); \
        x = y > x ? y : x;                                                                            \
    }
    HP_UMAX_STEP(0xB1, 0xf)   // quad_perm [1,0,3,2]
    HP_UMAX_STEP(0x4E, 0xf)   // quad_perm [2,3,0,1]
    HP_UMAX_STEP(0x141, 0xf)  // row_half_mirror
    HP_UMAX_STEP(0x140, 0xf)  // row_mirror
    HP_UMAX_STEP(0x142, 0xa)  // row_bcast:15 into rows 1, 3
    HP_UMAX_STEP(0x143, 0xc)  // row_bcast:31 into rows 2, 3
#undef HP_UMAX_STEP
    return (unsigned)__builtin_amdgcn_readlane((int)x, 63);
}
__device__ __forceinline__ unsigned wave_sum_u(unsigned x) {
    return (unsigned)__builtin_amdgcn_readlane((int)wave_incl_scan_u(x), 63);
}
#endif  // __HIPCC__

// ---- occupancy caps ----------------------------------------------------------------
// A launch may ask for dynamic LDS that no kernel touches, only to cap how many
// workgroups share a CU (160 KiB of LDS each).  The plain streaming kernels move more
// bytes per second with four or five workgroups per CU than with eight: fewer tiles
// in flight keep the addresses the memory controllers see closer together.  Kernels
// with a chain of dependent loads before their stores want every wave they can get
// and ask for none.  Values chosen per kernel from measurements on MI355X.
constexpr unsigned kLdsFor5 = 32 * 1024;  // five workgroups per CU
constexpr unsigned kLdsFor4 = 40 * 1024;  // four

// ---- host-side launch description -----------------------------------------------
struct Launch {
    bool single;          // true: seg by value, grid = seg.ntiles
    Seg seg;              // single
    const Seg* dsegs;     // batch: device table
    const uint2* dmap;    // batch: device tile map
    const uint2* dsmap;   // batch, sparse: device map of sample tiles
    const uint2* dcmap;   // batch, sparse decode: device map of payload-slot tiles
    unsigned ntiles;      // workgroups to launch
    unsigned nstiles;     // batch, sparse: sample tiles
    unsigned nctiles;     // batch, sparse decode: payload-slot tiles
    unsigned nsegs;       // tensors in the table (1 for single)
    unsigned long long expect_pairs;  // sparse encode: pairs the launch is expected to select (ratio x elements)
};

struct MergeLaunch {
    bool single;
    MergeSeg seg;
    const MergeSeg* dsegs;
    const uint2* dmap;
    unsigned ntiles;
    unsigned nsegs;
    int npeers;
    bool reencode;
    bool aggregate;  // some chunk of the launch writes its fp32 sum
    bool local;      // some chunk of the launch starts its sum from a local gradient
    unsigned* tgflags;  // terngrad batch (its descriptors name the bucket size): one word per chunk, does a header disagree
    bool bucket256;     // and that size is a multiple of 256
};

}  // namespace hp
