// Sampled-threshold sparsifiers for gfx950: DGC and GradDrop encode, the shared
// sparse decode, and the tile-owner sparse decode-and-merge.
//
// Encode is seven launches over the whole tensor set:
//   0. accumulate   one streaming pass: mom' = m*mom + g, acc' = acc + mom'
//                   (GradDrop: acc' = acc + g), written back; the |acc'| keys at
//                   the sample positions are gathered and every 64-element group
//                   leaves a record on the way: its largest |acc'| with value and
//                   place, and a bound on its second largest;
//   1-3. select     the k-th largest sample key of every tensor by radix
//                   selection, 12 + 12 + 7 bits from the top: every pass is one
//                   launch over all sample tiles that adds LDS histograms into a
//                   per-tensor global one; which digit holds the k-th key is
//                   worked out from the finished histogram by every workgroup of
//                   the NEXT launch (the last digit by count and scan), so all
//                   that workgroups hand each other travels across a kernel
//                   boundary;
//   4. count        per-tile counts of keys above / equal to the threshold: a
//                   group whose record shows no or one such key is counted from
//                   the record, only the others are read again;
//   5. scan         one workgroup per tensor turns the counts into output
//                   offsets, writes the header and, if more than `capacity`
//                   elements qualify, re-thresholds on the whole tensor;
//   6. emit         the selected (index, value) pairs are written in ascending
//                   index order, from the record for single-pair groups and from
//                   one more read for the others, the accumulator (and momentum)
//                   being zeroed at those places.
// |x| is handled as the integer key bits(x) & 0x7fffffff, which orders like |x|.
#include "common.h"
#include "flat_pairs.h"
#include "launch.h"

namespace hp {

constexpr unsigned kNoQuota = 0xffffffffu;
constexpr int kSampleTile = 4096;  // sample keys per workgroup in the select passes

__device__ __forceinline__ unsigned key_of(float x) { return __float_as_uint(x) & 0x7fffffffu; }

__device__ __forceinline__ unsigned umax(unsigned a, unsigned b) { return a > b ? a : b; }
__device__ __forceinline__ unsigned umin(unsigned a, unsigned b) { return a < b ? a : b; }

// What a group record says about threshold thr: `flagged` when the group holds a
// selected element at all, `multi` when it may hold more than one (the group has
// to be read), otherwise its only selected element is the recorded one.
struct GroupView {
    unsigned key;   // largest key of the group
    bool flagged, multi;
};
__device__ __forceinline__ GroupView view_group(uint2 rec, unsigned thr) {
    GroupView v;
    v.key = rec.x & 0x7fffffffu;
    v.flagged = v.key >= thr && v.key > 0u;
    v.multi = v.flagged && (rec.y & ~63u) >= thr;
    return v;
}

// max over the 16 lanes of a DPP row; every lane of the row gets the result
__device__ __forceinline__ unsigned row_max16(unsigned x) {
    x = umax(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
    x = umax(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
    x = umax(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xf, 0xf, false));  // row_half_mirror
    x = umax(x, (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xf, 0xf, false));  // row_mirror
    return x;
}

__device__ __forceinline__ unsigned popc_lt(unsigned long long m, unsigned lane) {
    return __popcll(m & ((1ull << lane) - 1ull));
}

// per-tensor control words of the select passes: what the digit picks of passes 1 and 2
// found, written by the first workgroup of the tensor in that pass and read by the launch
// after it
enum { kCtlPrefix1 = 0, kCtlK1 = 1, kCtlPrefix2 = 2, kCtlK2 = 3, kCtlWords = 8 };

// ---- 0. accumulate -------------------------------------------------------------

// y / kSampleStride for y < 1024 + kSampleStride
__device__ __forceinline__ unsigned sample_quot(unsigned y) {
    static_assert(kSampleStride == 100, "the multiplier below is the one for 100");
    return __umul24(y, 5243u) >> 19;
}

// gload(j, e) supplies the four gradient values of step j (element e): global
// memory for the encoders, the LDS tile of merged peers for decode-and-merge.
// aload(j, e) supplies the accumulator values the same way (decode-and-merge
// loads them before it starts merging, to have them in flight early).
template <bool FAST, bool DGC, class GLoad, class ALoad>
__device__ __forceinline__ void sparse_accum_tile(const Seg& s, unsigned tile, const SparseWs& ws, GLoad gload,
                                                  ALoad aload) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const float mf = s.f0;
    uint32_t* sample = ws.sample + s.ws0;
    // the first sample position q0*S + S/2 at or behind the wavefront's first element, and its
    // distance off0 < S from that element: the same in every lane, so scalar arithmetic
    const unsigned long long wbase =
        (unsigned long long)tile * kTile + (unsigned)__builtin_amdgcn_readfirstlane((int)wave) * kWaveTile;
    const unsigned long long q0 = (wbase + (kSampleStride - 1 - kSampleStride / 2)) / kSampleStride;
    const unsigned off0 = (unsigned)(q0 * kSampleStride + kSampleStride / 2 - wbase);
    f4 g[4], a[4], m[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = gload(j, e);
        a[j] = aload(j, e);
        if (DGC) m[j] = load4<FAST>(s.s0, e, n);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        f4 acc;
        if (DGC) {
            f4 mm;  // a rounded product, then a rounded sum: never a fused multiply-add
            mm.x = __fadd_rn(__fmul_rn(mf, m[j].x), g[j].x);
            mm.y = __fadd_rn(__fmul_rn(mf, m[j].y), g[j].y);
            mm.z = __fadd_rn(__fmul_rn(mf, m[j].z), g[j].z);
            mm.w = __fadd_rn(__fmul_rn(mf, m[j].w), g[j].w);
            store4<FAST>(s.s0, e, n, mm);
            acc = a[j] + mm;
        } else {
            acc = a[j] + g[j];
        }
        store4<FAST>(s.s1, e, n, acc);
        unsigned k0 = key_of(acc.x), k1 = key_of(acc.y), k2 = key_of(acc.z), k3 = key_of(acc.w);
        if (!FAST) {
            unsigned v = valid4(e, n);
            k0 = (v & 1u) ? k0 : 0u;
            k1 = (v & 2u) ? k1 : 0u;
            k2 = (v & 4u) ? k2 : 0u;
            k3 = (v & 8u) ? k3 : 0u;
        }
        {   // group record: the largest key with its value and place, and a bound on the runner-up
            const unsigned lo1 = umax(k0, k1), lo2 = umin(k0, k1), plo = k1 > k0 ? 1u : 0u;
            const unsigned hi1 = umax(k2, k3), hi2 = umin(k2, k3), phi = k3 > k2 ? 3u : 2u;
            const bool bw = hi1 > lo1;
            const unsigned l1 = bw ? hi1 : lo1, lp = bw ? phi : plo;       // this lane's largest key and its place
            const unsigned l2 = bw ? umax(lo1, hi2) : umax(hi1, lo2);     // and its second largest
            const unsigned m1 = row_max16(l1);
            const unsigned rowbits = (unsigned)(__ballot(l1 == m1) >> (lane & 48u)) & 0xffffu;  // never empty
            const bool own = (lane & 15u) == (unsigned)__ffs((int)rowbits) - 1u;
            const unsigned m2 = row_max16(own ? l2 : l1);
            if (own) {
                const float top = lp == 0 ? acc.x : (lp == 1 ? acc.y : (lp == 2 ? acc.z : acc.w));
                ws.grec[(unsigned long long)(s.tile0 + tile) * 64 + wave * 16 + j * 4 + (lane >> 4)] =
                    make_uint2(__float_as_uint(top), (((m2 + 63u) >> 6) << 6) | ((lane & 15u) * 4 + lp));
            }
        }
        if (s.sstride == 1) {  // small tensor: every element is a sample
            if (e < n) sample[e] = k0;
            if (e + 1 < n) sample[e + 1] = k1;
            if (e + 2 < n) sample[e + 2] = k2;
            if (e + 3 < n) sample[e + 3] = k3;
        } else {  // sample positions are q*S + S/2; at most one falls into [e, e+4)
            // first sample at or behind this step's four elements, counted from the wavefront's
            // first sample: x + S-1 - off0 < 1024 + S, so the quotient by S is a 24-bit
            // multiply and a shift
            const unsigned x = (unsigned)j * 256u + lane * 4u;
            const unsigned t = sample_quot(x + (unsigned)kSampleStride - 1u - off0);
            const unsigned at = off0 + t * (unsigned)kSampleStride;  // place of that sample in the wavefront's 1024
            if (at < x + 4u && q0 + t < s.ns) {
                const unsigned d = at - x;
                sample[q0 + t] = d == 0 ? k0 : (d == 1 ? k1 : (d == 2 ? k2 : k3));
            }
        }
    }
}

// Tile 0 of a tensor resets that tensor's select-pass state.
__device__ __forceinline__ void sparse_reset_select(const Seg& s, const SparseWs& ws) {
    uint32_t* h = ws.hist + (unsigned long long)s.id * kSelHistWords;
    for (unsigned i = threadIdx.x; i < kSelHistWords; i += kBlock) h[i] = 0;
    if (threadIdx.x < kCtlWords) ws.ctl[s.id * kCtlWords + threadIdx.x] = 0u;
    if (threadIdx.x == 0) {
        ws.thr[2 * s.id] = 0;
        ws.thr[2 * s.id + 1] = kNoQuota;
    }
}

template <class Src, bool DGC>
__global__ __launch_bounds__(kBlock) void sparse_accum_kernel(Src src, SparseWs ws) {
    if (!DGC) four_waves_per_simd();  // with the momentum streams the kernel does best unlimited
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (tile == 0) sparse_reset_select(s, ws);
    const long long n = (long long)s.n;
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n)
        sparse_accum_tile<true, DGC>(s, tile, ws, [&](int, long long e) { return load4<true>(s.g, e, n); },
                                     [&](int, long long e) { return load4<true>(s.s1, e, n); });
    else
        sparse_accum_tile<false, DGC>(s, tile, ws, [&](int, long long e) { return load4<false>(s.g, e, n); },
                                      [&](int, long long e) { return load4<false>(s.s1, e, n); });
}

// ---- 1-3. select -----------------------------------------------------------------

// Which of 4096 bins holds the k-th largest key (bins walked from the top), and the rank
// of that key inside the bin: every thread of a 256-thread workgroup gets {bin, rank} in
// res[] after the call.  Thread t owns the 16 bins [4096 - 16 (t + 1), 4096 - 16 t).  If the
// counts fall short of k the lowest bin is taken.
__device__ __forceinline__ void block_pick4096(const uint32_t* gh, unsigned k, unsigned (&xw)[4], unsigned (&res)[2]) {
    const uint4* p = reinterpret_cast<const uint4*>(gh + kSelBins - 16 * (threadIdx.x + 1));
    const uint4 q0 = p[0], q1 = p[1], q2 = p[2], q3 = p[3];
    const unsigned c[16] = {q3.w, q3.z, q3.y, q3.x, q2.w, q2.z, q2.y, q2.x, q1.w, q1.z, q1.y, q1.x, q0.w, q0.z, q0.y, q0.x};
    unsigned mine = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) mine += c[j];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned incl = wave_incl_scan_u(mine);
    if (lane == 63) xw[wave] = incl;
    __syncthreads();
    unsigned before = incl - mine;
    for (unsigned w = 0; w < wave; ++w) before += xw[w];
    k = k ? k : 1u;
    // exactly one thread owns the chunk that holds rank k (the last one takes what is left)
    const bool owner = (k > before && k <= before + mine) || (threadIdx.x == kBlock - 1 && k > before + mine);
    if (owner) {
        unsigned kk = k - before, j = 0;
#pragma unroll
        for (int i = 0; i < 15; ++i) {
            const bool stay = j == (unsigned)i && kk > c[i];  // not in bin i from the top: move on
            kk -= stay ? c[i] : 0u;
            j += stay ? 1u : 0u;
        }
        res[0] = kSelBins - 1 - 16 * threadIdx.x - j;
        res[1] = kk;
    }
    __syncthreads();
}

// The last digit (128 bins) by one wavefront, all 64 lanes active: lane l owns bins
// 127 - 2l and 126 - 2l.  Returns the threshold key, the same value in every lane.
__device__ __forceinline__ unsigned wave_pick_threshold(const SparseWs& ws, unsigned id, unsigned lane) {
    const uint2 pk = *reinterpret_cast<const uint2*>(ws.ctl + id * kCtlWords + kCtlPrefix2);
    const uint2 v = *reinterpret_cast<const uint2*>(ws.hist + (unsigned long long)id * kSelHistWords + 2 * kSelBins + 126 - 2 * lane);
    const unsigned mine = v.x + v.y;
    const unsigned incl = wave_incl_scan_u(mine), before = incl - mine;
    const unsigned k = pk.y ? pk.y : 1u;
    const bool owner = (k > before && k <= before + mine) || (lane == 63 && k > before + mine);
    const unsigned d = (k - before) <= v.y ? 127u - 2 * lane : 126u - 2 * lane;
    const unsigned src = (unsigned)__ffsll((long long)__ballot(owner)) - 1u;
    return pk.x | (unsigned)__builtin_amdgcn_readlane((int)d, (int)__builtin_amdgcn_readfirstlane((int)src));
}

// One radix pass.  Workgroup = one tile of kSampleTile sample keys of one tensor.  Pass 0
// counts the top 12 bits of every key; pass 1 first works out, from pass 0's finished
// histogram, which of those digits holds the k-th largest key, and counts the next 12 bits
// of the keys that carry it; pass 2 does the same for the last 7 bits.  Nothing is read
// that another workgroup of the same launch writes: the adds go to this pass's histogram,
// which only the next launch reads, and what the first workgroup of a tensor records of
// its pick (every workgroup of the tensor computes the same) is likewise for the launch
// after it.
template <class Src, int PASS>
__global__ __launch_bounds__(kBlock) void sparse_select_kernel(Src src, SparseWs ws) {
    constexpr unsigned NB = PASS == 2 ? kSelBinsLast : kSelBins;
    constexpr unsigned SHIFT = PASS == 0 ? kSelShift0 : (PASS == 1 ? kSelShift1 : 0u);
    constexpr unsigned ABOVE = PASS == 0 ? 0u : (PASS == 1 ? (0x7fffffffu >> kSelShift0) << kSelShift0
                                                           : (0x7fffffffu >> kSelShift1) << kSelShift1);
    __shared__ unsigned lh[NB];
    __shared__ unsigned xw[4], res[2];
    unsigned stile;
    const Seg s = src.get(stile, blockIdx.x);
    const uint32_t* keys = ws.sample + s.ws0;
    uint32_t* ctl = ws.ctl + s.id * kCtlWords;
    uint32_t* hist = ws.hist + (unsigned long long)s.id * kSelHistWords;
    uint32_t* gh = hist + PASS * kSelBins;
    for (unsigned i = threadIdx.x; i < NB; i += kBlock) lh[i] = 0;
    // all sixteen keys of a thread are requested before anything else is waited for
    const unsigned long long lo = (unsigned long long)stile * kSampleTile;
    unsigned key[kSampleTile / kBlock];
#pragma unroll
    for (int j = 0; j < kSampleTile / kBlock; ++j) {
        const unsigned long long i = lo + j * kBlock + threadIdx.x;
        key[j] = i < s.ns ? keys[i] : 0u;
    }
    unsigned prefix = 0;
    if (PASS > 0) {
        const unsigned pprev = PASS == 1 ? 0u : ctl[kCtlPrefix1];
        const unsigned kprev = PASS == 1 ? s.ks : ctl[kCtlK1];
        block_pick4096(hist + (PASS - 1) * kSelBins, kprev, xw, res);
        prefix = pprev | (res[0] << (PASS == 1 ? kSelShift0 : kSelShift1));
        if (stile == 0 && threadIdx.x == 0) {
            ctl[PASS == 1 ? kCtlPrefix1 : kCtlPrefix2] = prefix;
            ctl[PASS == 1 ? kCtlK1 : kCtlK2] = res[1];
        }
    } else {
        __syncthreads();
    }
    // Zero keys (and the 0 that stands for a key past the end) are left out: they are the
    // smallest there is, a pick that runs short of counts takes the lowest bin anyway, and a
    // sample that is mostly zeros (the sum of sparse payloads) would otherwise send every
    // lane to the same LDS word.
#pragma unroll
    for (int j = 0; j < kSampleTile / kBlock; ++j)
        if (key[j] != 0u && (key[j] & ABOVE) == prefix) atomicAdd(&lh[(key[j] >> SHIFT) & (NB - 1)], 1u);
    __syncthreads();
    for (unsigned i = threadIdx.x; i < NB; i += kBlock) {
        const unsigned c = lh[i];
        if (c) atomicAdd(&gh[i], c);  // no result is asked for: the next launch reads the sums
    }
}

// ---- 4. count ---------------------------------------------------------------------

// The 16 lanes of a DPP row read one 64-element group as 16-byte vectors; a
// wavefront therefore works on four flagged groups per load instruction.
__device__ __forceinline__ f4 load_group4(const float* p, long long e, long long n, bool aligned) {
    if (aligned && e + 3 < n) return *reinterpret_cast<const f4u*>(p + e);
    return ld4_guard(p, e, n);
}

// Takes the lowest set bit out of m: its index, or 64 when m is empty.
__device__ __forceinline__ unsigned pop_bit(unsigned long long& m) {
    unsigned i = m ? (unsigned)__ffsll((long long)m) - 1 : 64u;
    m &= m - 1;
    return i;
}

__device__ __forceinline__ unsigned pick_row(unsigned row, unsigned a, unsigned b, unsigned c, unsigned d) {
    return row == 0 ? a : (row == 1 ? b : (row == 2 ? c : d));
}

// Counts, for tile `tile` (4096 elements) of tensor s, the keys above and equal
// to thr; lane l looks at the record of 64-element group l and only groups that
// may hold more than one such key are read, eight per round, the next round's
// loads in flight while this round is counted.  Wavefront-uniform result.
__device__ __forceinline__ void count_tile(const Seg& s, uint2 rec, unsigned tile, unsigned thr, unsigned lane,
                                           unsigned& gt, unsigned& eq) {
    const long long n = (long long)s.n;
    const bool aligned = s.aligned != 0;
    const float* acc = s.s1;
    const GroupView gv = view_group(rec, thr);
    unsigned long long mask = __ballot(gv.multi);
    const unsigned row = lane >> 4;
    const long long base = (long long)tile * kTile + (lane & 15u) * 4;
    const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    // a group with a single selected element is counted from its record alone
    const bool single = gv.flagged && !gv.multi;
    unsigned cg = single && gv.key > thr, ce = single && gv.key == thr;
    auto fetch = [&](f4& va, f4& vb) {
        unsigned a0 = pop_bit(mask), a1 = pop_bit(mask), a2 = pop_bit(mask), a3 = pop_bit(mask);
        unsigned b0 = pop_bit(mask), b1 = pop_bit(mask), b2 = pop_bit(mask), b3 = pop_bit(mask);
        unsigned ga = pick_row(row, a0, a1, a2, a3), gb = pick_row(row, b0, b1, b2, b3);
        va = zero4;
        vb = zero4;
        if (ga < 64u) va = load_group4(acc, base + ga * 64, n, aligned);
        if (gb < 64u) vb = load_group4(acc, base + gb * 64, n, aligned);
    };
    auto tally = [&](f4 v) {
        unsigned k;
        k = key_of(v.x); cg += k > thr; ce += (k == thr) & (k > 0u);
        k = key_of(v.y); cg += k > thr; ce += (k == thr) & (k > 0u);
        k = key_of(v.z); cg += k > thr; ce += (k == thr) & (k > 0u);
        k = key_of(v.w); cg += k > thr; ce += (k == thr) & (k > 0u);
    };
    f4 va, vb;
    bool have = mask != 0;
    if (have) fetch(va, vb);
    while (have) {
        f4 na = zero4, nb = zero4;
        const bool more = mask != 0;
        if (more) fetch(na, nb);
        tally(va);
        tally(vb);
        va = na;
        vb = nb;
        have = more;
    }
    gt = wave_sum_u(cg);
    eq = wave_sum_u(ce);
}

// One wavefront per tile, four tiles per workgroup.
template <class Src>
__global__ __launch_bounds__(kBlock) void sparse_count_kernel(Src src, SparseWs ws, unsigned total_tiles) {
    // the wavefront's index as a scalar: what is addressed by it is then fetched by scalar loads
    const unsigned lane = threadIdx.x & 63u, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned gt_idx = blockIdx.x * 4 + wave;
    if (gt_idx >= total_tiles) return;
    // the record needs nothing but the tile's place in the launch, the threshold (the pick
    // of the last digit from pass 2's histogram) only the tensor's index: neither waits for
    // the descriptor
    const uint2 rec = ws.grec[(unsigned long long)gt_idx * 64 + lane];
    const uint2 m = src.where(gt_idx);
    const unsigned thr = wave_pick_threshold(ws, m.x, lane);
    const Seg s = src.at(m.x);
    unsigned gt, eq;
    count_tile(s, rec, m.y, thr, lane, gt, eq);
    if (lane == 0) *reinterpret_cast<uint2*>(ws.counts + (unsigned long long)gt_idx * 2) = make_uint2(gt, eq);
}

// ---- 5. scan ----------------------------------------------------------------------

// In-place exclusive scan of nw {above, equal} pairs by one workgroup of
// kScanBlock threads; returns the totals to every thread.  Each wavefront owns a
// contiguous span.  The first sweep adds the span up, sixteen loads in flight per
// lane, and leaves the pairs in LDS as 16 + 16 bits (a tile holds at most 4096 of
// either kind); the second sweep scans 256 pairs at a time from there, so only its
// stores touch memory.  Tensors beyond kScanStage tiles read memory twice.
constexpr int kScanBlock = 1024;
constexpr int kScanWaves = kScanBlock / 64;
constexpr unsigned kScanStage = 32768;  // pairs that stay in LDS between the sweeps: 128 KiB
constexpr int kScanBatch = 16;          // loads in flight per lane in the first sweep

__device__ __forceinline__ void block_scan_pairs(uint32_t* c, unsigned nw, unsigned (&sh)[2][kScanWaves],
                                                 uint32_t* stage, unsigned& tot_gt, unsigned& tot_eq) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint2* c2 = reinterpret_cast<uint2*>(c);
    const bool staged = nw <= kScanStage;
    const bool wide = (reinterpret_cast<unsigned long long>(c) & 15ull) == 0;  // a tensor may start at an odd tile
    const unsigned span = ((nw + kScanWaves - 1) / kScanWaves + 63u) & ~63u;
    const unsigned lo = wave * span < nw ? wave * span : nw;
    const unsigned hi = lo + span < nw ? lo + span : nw;
    unsigned sg = 0, se = 0;
    for (unsigned i0 = lo + lane; i0 < hi; i0 += kScanBatch * 64) {
        uint2 v[kScanBatch];
#pragma unroll
        for (int r = 0; r < kScanBatch; ++r) v[r] = i0 + r * 64 < hi ? c2[i0 + r * 64] : make_uint2(0u, 0u);
#pragma unroll
        for (int r = 0; r < kScanBatch; ++r) {
            sg += v[r].x;
            se += v[r].y;
            if (staged && i0 + r * 64 < hi) stage[i0 + r * 64] = v[r].x | (v[r].y << 16);
        }
    }
    sg = wave_sum_u(sg);
    se = wave_sum_u(se);
    __syncthreads();  // sh may still be read from a previous call
    if (lane == 0) {
        sh[0][wave] = sg;
        sh[1][wave] = se;
    }
    __syncthreads();
    unsigned bg = 0, be = 0;
    tot_gt = 0;
    tot_eq = 0;
#pragma unroll
    for (int w = 0; w < kScanWaves; ++w) {
        unsigned g = sh[0][w], e = sh[1][w];
        if ((unsigned)w < wave) {
            bg += g;
            be += e;
        }
        tot_gt += g;
        tot_eq += e;
    }
    // 256 pairs per trip: every lane owns four consecutive pairs, adds them up on its
    // own, and one wavefront scan per kind of the lane sums places them (the scan's
    // instructions, not memory, bound this kernel: one compute unit works through the
    // largest tensor).  A wavefront reads back only what it staged itself.
    for (unsigned i0 = lo; i0 < hi; i0 += 256) {
        const unsigned i = i0 + lane * 4;
        uint2 v[4];
        if (staged) {
            const uint4 p = *reinterpret_cast<const uint4*>(&stage[i]);  // lo is a multiple of 64
            const unsigned w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = i + r < hi ? make_uint2(w[r] & 0xffffu, w[r] >> 16) : make_uint2(0u, 0u);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = i + r < hi ? c2[i + r] : make_uint2(0u, 0u);
        }
        const unsigned lg = v[0].x + v[1].x + v[2].x + v[3].x, le = v[0].y + v[1].y + v[2].y + v[3].y;
        const unsigned ig = wave_incl_scan_u(lg), ie = wave_incl_scan_u(le);
        uint2 x[4];
        x[0] = make_uint2(bg + ig - lg, be + ie - le);
#pragma unroll
        for (int r = 1; r < 4; ++r) x[r] = make_uint2(x[r - 1].x + v[r - 1].x, x[r - 1].y + v[r - 1].y);
        if (i + 3 < hi && wide) {  // two 16-byte stores
            *reinterpret_cast<uint4*>(&c2[i]) = make_uint4(x[0].x, x[0].y, x[1].x, x[1].y);
            *reinterpret_cast<uint4*>(&c2[i + 2]) = make_uint4(x[2].x, x[2].y, x[3].x, x[3].y);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (i + r < hi) c2[i + r] = x[r];
        }
        bg += (unsigned)__builtin_amdgcn_readlane((int)ig, 63);
        be += (unsigned)__builtin_amdgcn_readlane((int)ie, 63);
    }
    __syncthreads();
}

// k-th largest (k >= 1) key among the keys a workgroup enumerates with visit(f)
// (which must call f(key) for every candidate, the same set each time it is
// invoked).  8-bit digits from the top; 16 interleaved histograms keep the LDS
// atomics of neighbouring lanes apart.  Only the overflow path uses it.
struct RadixScratch {
    unsigned hist[16][257];
    unsigned prefix, k;
};

template <class Visit>
__device__ __forceinline__ unsigned block_kth_largest(RadixScratch& sc, unsigned k, Visit visit) {
    unsigned prefix = 0, mask = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (unsigned i = threadIdx.x; i < 16 * 257; i += blockDim.x) (&sc.hist[0][0])[i] = 0;
        __syncthreads();
        visit([&](unsigned key) {
            if ((key & mask) == prefix) atomicAdd(&sc.hist[threadIdx.x & 15u][(key >> shift) & 255u], 1u);
        });
        __syncthreads();
        if (threadIdx.x < 256) {  // fold the 16 copies, one bin per thread
            unsigned t = threadIdx.x;
            unsigned c = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r) c += sc.hist[r][t];
            sc.hist[0][t] = c;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned kk = k;
            int d = 255;
            for (; d > 0; --d) {
                unsigned c = sc.hist[0][d];
                if (kk <= c) break;
                kk -= c;
            }
            sc.prefix = prefix | ((unsigned)d << shift);
            sc.k = kk;
        }
        __syncthreads();
        prefix = sc.prefix;
        k = sc.k;
        mask |= 0xffu << shift;
        __syncthreads();
    }
    return prefix;
}

template <class SegSrc>
__global__ __launch_bounds__(kScanBlock) void sparse_scan_kernel(SegSrc src, SparseWs ws) {
    __shared__ unsigned sh[2][kScanWaves];
    __shared__ RadixScratch sc;
    __shared__ __attribute__((aligned(16))) uint32_t stage[kScanStage + 256];  // a trip may read past the last pair
    const Seg s = src.at(blockIdx.x);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned nw = s.ntiles;
    uint32_t* c = ws.counts + (unsigned long long)s.tile0 * 2;
    unsigned thr = wave_pick_threshold(ws, s.id, lane);  // every wavefront works out the same value
    unsigned quota = kNoQuota;
    unsigned tot_gt, tot_eq;
    block_scan_pairs(c, nw, sh, stage, tot_gt, tot_eq);
    unsigned long long total = (unsigned long long)tot_gt + tot_eq;
    if (total > s.cap && tot_gt < s.cap) {
        // More candidates than slots, but only because of ties at the threshold (gradients
        // clipped by value do this): the capacity-th largest key of the tensor is the threshold
        // itself, so it stays, the tile counts stand, and the ties are taken in ascending index
        // order until the slots are full.
        quota = s.cap - tot_gt;
        total = s.cap;
    } else if (total > s.cap) {
        // More keys above the threshold than slots (the sample misjudged the tensor): the
        // threshold becomes the capacity-th largest key of the whole tensor (all of those keys
        // are >= the sampled threshold, hence inside flagged groups), found by this one
        // workgroup; ties at the new threshold are rationed as above.
        const unsigned old = thr;
        const long long n = (long long)s.n;
        const uint2* grec = ws.grec + (unsigned long long)s.tile0 * 64;
        // a wavefront per tile: lane l looks at the record of group l, then the flagged groups are
        // read eight at a time (lane l their element l), all eight loads in flight together
        thr = block_kth_largest(sc, s.cap, [&](auto f) {
            for (unsigned t = wave; t < nw; t += kScanWaves) {
                const unsigned gm = grec[(unsigned long long)t * 64 + lane].x & 0x7fffffffu;
                unsigned long long m = __ballot(gm >= old && gm > 0u);
                const long long tb = (long long)t * kTile + lane;
                while (m) {
                    unsigned key[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const unsigned gi = pop_bit(m);
                        const long long e = tb + (long long)gi * 64;
                        key[u] = (gi < 64u && e < n) ? key_of(s.s1[e]) : 0u;
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (key[u] >= old && key[u] > 0u) f(key[u]);
                }
            }
        });
        for (unsigned t = wave; t < nw; t += kScanWaves) {
            unsigned gt, eq;
            count_tile(s, grec[(unsigned long long)t * 64 + lane], t, thr, lane, gt, eq);
            if (lane == 0) {
                c[2 * t] = gt;
                c[2 * t + 1] = eq;
            }
        }
        __syncthreads();
        block_scan_pairs(c, nw, sh, stage, tot_gt, tot_eq);
        quota = s.cap - tot_gt;
        total = s.cap;
    }
    if (threadIdx.x == 0) {
        ws.thr[2 * s.id] = thr;
        ws.thr[2 * s.id + 1] = quota;
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = (uint32_t)total;
        h[1] = (uint32_t)s.n;
        h[2] = s.cap;
        h[3] = thr;  // bit pattern of the threshold value
    }
}

// ---- 6. emit ----------------------------------------------------------------------

// inclusive prefix sum over the 16 lanes of a DPP row
__device__ __forceinline__ unsigned row_scan16(unsigned x) {
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, true);  // row_shr:1
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, true);  // row_shr:2
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, true);  // row_shr:4
    x += (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, true);  // row_shr:8
    return x;
}

// The 4-byte store that clears a selected element.  A plain store leaves a partly written
// line in the cache hierarchy, which is the cheaper way as long as one launch clears no more
// than about two million elements: the lines stay on chip until the next accumulate pass
// overwrites them whole.  Beyond that they are pushed out piecemeal under the following
// kernels (measured on MI355X: the next accumulate pass loses 4 %), and a store that goes
// straight through costs less (STREAM).
template <bool STREAM>
__device__ __forceinline__ void clear_element(float* p) {
    if (STREAM) __builtin_nontemporal_store(0.f, p);
    else *p = 0.f;
}

template <class Src, bool STREAM>
__global__ __launch_bounds__(kBlock) void sparse_emit_kernel(Src src, SparseWs ws, unsigned total_tiles) {
    // the wavefront's index as a scalar: what is addressed by it is then fetched by scalar loads
    const unsigned lane = threadIdx.x & 63u, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned gt_idx = blockIdx.x * 4 + wave;
    if (gt_idx >= total_tiles) return;
    // record and offsets need nothing but the tile's place in the launch, threshold and
    // quota only the tensor's index: none of them waits for the descriptor
    const uint2 rec = ws.grec[(unsigned long long)gt_idx * 64 + lane];
    const uint2 before = *reinterpret_cast<const uint2*>(ws.counts + (unsigned long long)gt_idx * 2);
    const uint2 m = src.where(gt_idx);
    const uint2 tq = *reinterpret_cast<const uint2*>(ws.thr + 2 * m.x);
    const Seg s = src.at(m.x);
    const unsigned tile = m.y, thr = tq.x, quota = tq.y;
    const long long n = (long long)s.n;
    const unsigned G = before.x, E = before.y;
    unsigned pos = G + (E < quota ? E : quota);  // pairs written by earlier tiles
    int32_t* idx = reinterpret_cast<int32_t*>(s.pay + kHeaderBytes);
    float* val = reinterpret_cast<float*>(s.pay + kHeaderBytes + 4ull * s.cap);
    const GroupView gv = view_group(rec, thr);
    if (quota == kNoQuota) {
        // Usual case: everything at or above the threshold is taken.  Lane l speaks for
        // group l.  A group with one selected element yields its pair straight from the
        // record; groups that may hold more are read, four per round: row r of the
        // wavefront reads the r-th of them, positions come from a row prefix sum of the
        // per-lane counts, the totals of the rows before and the single-pair groups
        // below.  The next round's loads are issued before this round's stores (they
        // touch different groups), so rounds overlap.
        const unsigned long long smask = __ballot(gv.flagged && !gv.multi);
        unsigned long long mask = __ballot(gv.multi);
        const unsigned pos0 = pos;
        unsigned from_multi = 0;  // pairs of read groups below group `lane`
        const unsigned row = lane >> 4;
        const bool aligned = s.aligned != 0;
        const long long base = (long long)tile * kTile + (lane & 15u) * 4;
        const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
        unsigned gi = 64u, c0 = 64u, c1 = 64u, c2 = 64u, c3 = 64u;  // this round's groups (64: none)
        f4 v = zero4;
        bool more = mask != 0;
        if (more) {
            c0 = pop_bit(mask); c1 = pop_bit(mask); c2 = pop_bit(mask); c3 = pop_bit(mask);
            gi = pick_row(row, c0, c1, c2, c3);
            if (gi < 64u) v = load_group4(s.s1, base + gi * 64, n, aligned);
        }
        while (more) {
            more = mask != 0;
            unsigned gi_next = 64u, n0 = 64u, n1 = 64u, n2 = 64u, n3 = 64u;
            f4 v_next = zero4;
            if (more) {
                n0 = pop_bit(mask); n1 = pop_bit(mask); n2 = pop_bit(mask); n3 = pop_bit(mask);
                gi_next = pick_row(row, n0, n1, n2, n3);
                if (gi_next < 64u) v_next = load_group4(s.s1, base + gi_next * 64, n, aligned);
            }
            const long long e = base + gi * 64;
            unsigned k0 = key_of(v.x), k1 = key_of(v.y), k2 = key_of(v.z), k3 = key_of(v.w);
            unsigned s0 = (k0 >= thr) & (k0 > 0u), s1 = (k1 >= thr) & (k1 > 0u);
            unsigned s2 = (k2 >= thr) & (k2 > 0u), s3 = (k3 >= thr) & (k3 > 0u);
            unsigned c = s0 + s1 + s2 + s3;
            unsigned incl = row_scan16(c);
            unsigned t0 = (unsigned)__builtin_amdgcn_readlane((int)incl, 15);
            unsigned t1 = (unsigned)__builtin_amdgcn_readlane((int)incl, 31);
            unsigned t2 = (unsigned)__builtin_amdgcn_readlane((int)incl, 47);
            unsigned t3 = (unsigned)__builtin_amdgcn_readlane((int)incl, 63);
            unsigned p = pos + (incl - c) + (row > 0 ? t0 : 0u) + (row > 1 ? t1 : 0u) + (row > 2 ? t2 : 0u) +
                         (gi < 64u ? popc_lt(smask, gi) : 0u);
            if (c && p + c <= s.cap) {  // the scan guarantees room; the test only guards the buffer
                f4 keep = v;
                if (s0) { idx[p] = (int32_t)e; val[p] = v.x; keep.x = 0.f; ++p; }
                if (s1) { idx[p] = (int32_t)(e + 1); val[p] = v.y; keep.y = 0.f; ++p; }
                if (s2) { idx[p] = (int32_t)(e + 2); val[p] = v.z; keep.z = 0.f; ++p; }
                if (s3) { idx[p] = (int32_t)(e + 3); val[p] = v.w; keep.w = 0.f; ++p; }
                if (aligned && e + 3 < n) {
                    *reinterpret_cast<f4u*>(s.s1 + e) = keep;
                    if (s.s0) {
                        f4 m = *reinterpret_cast<const f4u*>(s.s0 + e);
                        m.x = s0 ? 0.f : m.x; m.y = s1 ? 0.f : m.y; m.z = s2 ? 0.f : m.z; m.w = s3 ? 0.f : m.w;
                        *reinterpret_cast<f4u*>(s.s0 + e) = m;
                    }
                } else {
                    if (s0) { clear_element<STREAM>(&s.s1[e]); if (s.s0) clear_element<STREAM>(&s.s0[e]); }
                    if (s1) { clear_element<STREAM>(&s.s1[e + 1]); if (s.s0) clear_element<STREAM>(&s.s0[e + 1]); }
                    if (s2) { clear_element<STREAM>(&s.s1[e + 2]); if (s.s0) clear_element<STREAM>(&s.s0[e + 2]); }
                    if (s3) { clear_element<STREAM>(&s.s1[e + 3]); if (s.s0) clear_element<STREAM>(&s.s0[e + 3]); }
                }
            }
            pos += t0 + t1 + t2 + t3;
            from_multi += (lane > c0 ? t0 : 0u) + (lane > c1 ? t1 : 0u) + (lane > c2 ? t2 : 0u) + (lane > c3 ? t3 : 0u);
            gi = gi_next;
            v = v_next;
            c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        }
        if (gv.flagged && !gv.multi) {
            const unsigned p = pos0 + popc_lt(smask, lane) + from_multi;
            const long long e = (long long)tile * kTile + lane * 64 + (rec.y & 63u);
            if (p < s.cap) {
                idx[p] = (int32_t)e;
                val[p] = __uint_as_float(rec.x);
                clear_element<STREAM>(&s.s1[e]);
                if (s.s0) clear_element<STREAM>(&s.s0[e]);
            }
        }
        return;
    }
    unsigned long long mask = __ballot(gv.flagged);
    // Overflow case: ties at the threshold are rationed in index order, one group
    // of 64 at a time across the whole wavefront.
    unsigned eq_seen = E;
    const long long base = (long long)tile * kTile + lane;
    while (mask) {
        unsigned gi = pop_bit(mask);
        long long e = base + gi * 64;
        float v = e < n ? s.s1[e] : 0.f;
        unsigned key = key_of(v);
        bool is_eq = key == thr && key > 0u;
        unsigned long long m_eq = __ballot(is_eq);
        bool sel = key > thr || (is_eq && eq_seen + popc_lt(m_eq, lane) < quota);
        unsigned long long m_sel = __ballot(sel);
        if (sel) {
            unsigned p = pos + popc_lt(m_sel, lane);
            if (p < s.cap) {
                idx[p] = (int32_t)e;
                val[p] = v;
                clear_element<STREAM>(&s.s1[e]);
                if (s.s0) clear_element<STREAM>(&s.s0[e]);
            }
        }
        pos += __popcll(m_sel);
        eq_seen += __popcll(m_eq);
    }
}

// ---- decode: zero fill + scatter ------------------------------------------------------

template <bool FAST>
__device__ __forceinline__ void zero_tile(float* out, long long n, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const f4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) store4<FAST>(out, base + j * 256 + lane * 4, n, z);
}

template <class Src>
__global__ __launch_bounds__(kBlock) void zero_fill_kernel(Src src) {
    unsigned tile;
    const Seg s = src.get(tile, xcd_grouped(blockIdx.x, gridDim.x));
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) zero_tile<true>(s.out, (long long)s.n, tile);
    else zero_tile<false>(s.out, (long long)s.n, tile);
}

// Reads the header of a sparse payload that has room for `slots` pairs; returns
// the number of usable pairs (0 when the header does not fit the buffer).
__device__ __forceinline__ unsigned sparse_header(const uint8_t* pay, unsigned slots, const int32_t*& idx,
                                                  const float*& val) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(pay);
    unsigned nnz = h[0], cap = h[2];
    if (cap > slots) return 0;
    idx = reinterpret_cast<const int32_t*>(pay + kHeaderBytes);
    val = reinterpret_cast<const float*>(pay + kHeaderBytes + 4ull * cap);
    return nnz < cap ? nnz : cap;
}

// One workgroup per 1024 slots of a tensor's payload; workgroups past nnz exit.
constexpr int kSlotTile = 1024;

// out[idx[j]] = val[j] for the 1024 slots of slot tile ct
__device__ __forceinline__ void scatter_slots(const Seg& s, unsigned ct) {
    const int32_t* idx;
    const float* val;
    const unsigned nnz = sparse_header(s.pay, s.cap, idx, val);
    const unsigned long long lo = (unsigned long long)ct * kSlotTile;
#pragma unroll
    for (int k = 0; k < kSlotTile / kBlock; ++k) {
        unsigned long long j = lo + k * kBlock + threadIdx.x;
        if (j < nnz) {
            long long i = idx[j];
            if (i >= 0 && i < (long long)s.n) s.out[i] = val[j];
        }
    }
}

template <class Src>
__global__ __launch_bounds__(kBlock) void sparse_scatter_kernel(Src src) {
    unsigned ct;
    const Seg s = src.get(ct, blockIdx.x);
    scatter_slots(s, ct);
}

// ---- decode with tile pointers (launches over a tensor table) -------------------------
// A payload in ascending index order holds the pairs of a 4096-element tile as one
// contiguous run.  The index kernel walks the payload once, records where every
// tile's run starts and notices disorder; the tile kernel then builds each output
// tile in LDS (zeros plus the tile's pairs) and writes it once, so no line of the
// output is written twice.  For a tensor whose payload is not in order every tile
// looks through the whole payload instead of a run: correct, and slow in proportion
// to tiles x pairs (this library's encoders, like the reference's, emit ascending
// indices; the per-tensor decode scatters and does not care about order).

// One workgroup per 1024 slots.  ptr[t] (t < ntiles) = first slot whose index lies in
// tile t or later.  Slot j starts every tile after the tile of slot j-1 up to its
// own; long stretches of empty tiles are queued and filled by the whole workgroup.
template <class Src>
__global__ __launch_bounds__(kBlock) void sparse_decode_index_kernel(Src src, uint32_t* tptr, uint32_t* disorder,
                                                                     unsigned epoch) {
    __shared__ unsigned gap_first[kSlotTile + 2], gap_count[kSlotTile + 2], gap_value[kSlotTile + 2];
    __shared__ unsigned ngaps;
    unsigned ct;
    const Seg s = src.get(ct, blockIdx.x);
    const int32_t* idx;
    const float* val;
    const unsigned nnz = sparse_header(s.pay, s.cap, idx, val);
    const unsigned nt = s.ntiles;
    if (nt == 0) return;
    uint32_t* ptr = tptr + s.tile0;
    if (threadIdx.x == 0) ngaps = 0;
    __syncthreads();
    auto tile_of = [&](int32_t i) -> unsigned {  // indices outside the tensor count for the first / last tile
        if (i < 0) return 0u;
        unsigned t = (unsigned)i / kTile;
        return t < nt ? t : nt - 1;
    };
    auto start = [&](unsigned t0, unsigned t1, unsigned v) {  // ptr[t0, t1) = v
        if (t1 - t0 <= 8u) {
            for (unsigned t = t0; t < t1; ++t) ptr[t] = v;
        } else {
            unsigned g = atomicAdd(&ngaps, 1u);
            gap_first[g] = t0;
            gap_count[g] = t1 - t0;
            gap_value[g] = v;
        }
    };
    bool bad = false;
    const unsigned long long lo = (unsigned long long)ct * kSlotTile;
#pragma unroll
    for (int k = 0; k < kSlotTile / kBlock; ++k) {
        const unsigned long long j = lo + k * kBlock + threadIdx.x;
        if (j < nnz) {
            const int32_t cur = idx[j];
            const unsigned tc = tile_of(cur);
            unsigned first = 0;
            if (j) {
                const int32_t prev = idx[j - 1];
                bad |= prev > cur;
                first = tile_of(prev) + 1;
            }
            if (tc + 1 > first) start(first, tc + 1, (unsigned)j);
            if (j == nnz - 1 && tc + 1 < nt) start(tc + 1, nt, nnz);
        }
    }
    if (ct == 0 && threadIdx.x == 0 && nnz == 0 && nt) start(0, nt, 0u);
    if (bad) disorder[s.id] = epoch;  // every writer stores the same value
    __syncthreads();
    const unsigned ng = ngaps;
    for (unsigned g = 0; g < ng; ++g)
        for (unsigned t = threadIdx.x; t < gap_count[g]; t += kBlock) ptr[gap_first[g] + t] = gap_value[g];
}

template <class Src>
__global__ __launch_bounds__(kBlock) void sparse_decode_tile_kernel(Src src, const uint32_t* tptr,
                                                                    const uint32_t* disorder, unsigned epoch) {
    __shared__ __attribute__((aligned(16))) float lds[kTile];
    unsigned tile;
    const Seg s = src.get(tile, xcd_grouped(blockIdx.x, gridDim.x));
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long t_lo = (long long)tile * kTile, t_hi = t_lo + kTile < n ? t_lo + kTile : n;
    const int32_t* idx;
    const float* val;
    const unsigned nnz = sparse_header(s.pay, s.cap, idx, val);
    unsigned lo = 0, hi = nnz;  // a payload out of order: every pair is looked at
    if (disorder[s.id] != epoch) {
        lo = tptr[s.tile0 + tile];
        hi = tile + 1 < s.ntiles ? tptr[s.tile0 + tile + 1] : nnz;
        if (hi > nnz) hi = nnz;
        if (lo > hi) lo = hi;
    }
    const bool fast = s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n;
    const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    if (lo == hi) {  // nothing lands in this tile
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            long long e = t_lo + wave * kWaveTile + j * 256 + lane * 4;
            if (fast) st4(s.out + e, zero4);
            else st4_guard(s.out, e, n, zero4);
        }
        return;
    }
    // the first round of pairs is requested before the LDS tile is cleared
    unsigned j0 = lo + threadIdx.x;
    long long i0 = -1;
    float v0 = 0.f;
    if (j0 < hi) {
        i0 = idx[j0];
        v0 = val[j0];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<f4*>(&lds[wave * kWaveTile + j * 256 + lane * 4]) = zero4;
    __syncthreads();
    if (i0 >= t_lo && i0 < t_hi) lds[i0 - t_lo] = v0;
    for (unsigned j = j0 + kBlock; j < hi; j += kBlock) {
        long long i = idx[j];
        if (i >= t_lo && i < t_hi) lds[i - t_lo] = val[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = t_lo + wave * kWaveTile + j * 256 + lane * 4;
        f4 v = *reinterpret_cast<const f4*>(&lds[wave * kWaveTile + j * 256 + lane * 4]);
        if (fast) st4(s.out + e, v);
        else st4_guard(s.out, e, n, v);
    }
}

// ---- sparse decode-and-merge -------------------------------------------------------
// Pairs arrive in ascending index order, so the pairs of one 4096-element tile are
// one contiguous run of every peer's payload.  An index launch walks the payloads once,
// 1024 slots per workgroup: where the tile number changes from one pair to the next a
// run ends and the next begins, and the workgroup that sees it writes both facts into
// the run records of the tiles concerned (begin and end of one record may come from
// different workgroups).  A record holds the addresses of the run's first index and
// value and the address just behind its last index, at a place that depends on nothing
// but the tile's number in the launch (the merge launch's grid is the launch's tiles).
// The merge kernel then gives every tile to one workgroup, which asks for the records
// before anything else, adds the peers' runs into an LDS tile in peer order, writes the
// aggregate once and, if asked, continues with the GradDrop-style re-encode pass on the
// values it already holds.  Summation order per element is the peer order, as in a
// sequential implementation.
// A payload that is not in order: the workgroup that notices stamps every record of that
// (chunk, peer) with the call's epoch, and a merge workgroup that finds the stamp looks
// through the peer's whole payload instead of a run (correct, slow).  The stamp is never
// cleared, only compared with the epoch, which differs from call to call: whatever an
// earlier call or uninitialised memory left there can at worst send a sorted payload
// down the slow path, never the other way round.

// One workgroup per 1024 payload slots of one (chunk, peer); blockIdx.y and .z number the slice.
template <class MSegSrc>
__global__ __launch_bounds__(kBlock) void sparse_merge_index_kernel(MSegSrc src, PeerRun* runs, int npeers,
                                                                    unsigned total_tiles, unsigned epoch) {
    __shared__ unsigned gap_first[kSlotTile + 2], gap_count[kSlotTile + 2], gap_value[kSlotTile + 2];
    __shared__ unsigned ngaps, bad;
    const unsigned chunk = blockIdx.x / npeers, p = blockIdx.x % npeers, slice = blockIdx.z * gridDim.y + blockIdx.y;
    const MergeSeg& m = src.at(chunk);
    const int32_t* idx;
    const float* val;
    const unsigned nnz = sparse_header(m.peer[p], m.peer_slots[p], idx, val);
    const unsigned nt = m.s.ntiles;
    // heads of all tiles of the launch first, then the runs peer by peer
    PeerRun* rec = runs + (unsigned long long)(1 + p) * total_tiles + m.s.tile0;  // record of tile t: rec[t]
    if (slice == 0 && p == 0) {  // the chunk's tile heads
        for (unsigned t = threadIdx.x; t < nt; t += kBlock) {
            TileHead h;
            h.acc = m.r.s1 ? m.r.s1 + (unsigned long long)t * kTile : nullptr;
            h.fast = m.s.aligned && (!m.r.s1 || m.r.aligned) && (unsigned long long)(t + 1) * kTile <= m.s.n;
            h.pad[0] = h.pad[1] = h.pad[2] = h.pad[3] = h.pad[4] = 0;
            *reinterpret_cast<TileHead*>(runs + m.s.tile0 + t) = h;
        }
    }
    const unsigned long long lo = (unsigned long long)slice * kSlotTile;
    if (lo >= nnz && !(slice == 0 && nnz == 0)) return;  // nothing in this slice
    if (threadIdx.x == 0) {
        ngaps = 0;
        bad = 0;
    }
    __syncthreads();
    auto tile_of = [&](int32_t i) -> unsigned {  // indices outside the chunk count for the first / last tile
        if (i < 0) return 0u;
        const unsigned t = (unsigned)i / kTile;
        return t < nt ? t : nt - 1;
    };
    // tiles t0 .. t1-1 begin at slot v, and the tiles before them end there
    auto mark = [&](unsigned t, unsigned v) {
        rec[t].idx = idx + v;
        rec[t].val = val + v;
        if (t) rec[t - 1].end = idx + v;
    };
    auto start = [&](unsigned t0, unsigned t1, unsigned v) {
        if (t1 - t0 <= 8u) {
            for (unsigned t = t0; t < t1; ++t) mark(t, v);
        } else {  // a long stretch of empty tiles: left to the whole workgroup
            const unsigned g = atomicAdd(&ngaps, 1u);
            gap_first[g] = t0;
            gap_count[g] = t1 - t0;
            gap_value[g] = v;
        }
    };
    bool disorder = false;
#pragma unroll
    for (int k = 0; k < kSlotTile / kBlock; ++k) {
        const unsigned long long j = lo + k * kBlock + threadIdx.x;
        if (j < nnz) {
            const int32_t cur = idx[j];
            const unsigned tc = tile_of(cur);
            unsigned first = 0;
            if (j) {
                const int32_t prev = idx[j - 1];
                disorder |= prev > cur;
                first = tile_of(prev) + 1;
            }
            if (tc + 1 > first) start(first, tc + 1, (unsigned)j);
            if (j == nnz - 1) {  // nothing is left for the tiles behind this pair's
                if (tc + 1 < nt) start(tc + 1, nt, nnz);
                rec[nt - 1].end = idx + nnz;
            }
        }
    }
    if (slice == 0 && nnz == 0 && threadIdx.x == 0) {
        start(0, nt, 0u);
        rec[nt - 1].end = idx;
    }
    if (disorder) bad = 1;  // every writer stores 1
    __syncthreads();
    const unsigned ng = ngaps;
    for (unsigned g = 0; g < ng; ++g)
        for (unsigned t = threadIdx.x; t < gap_count[g]; t += kBlock) mark(gap_first[g] + t, gap_value[g]);
    if (bad)
        for (unsigned t = threadIdx.x; t < nt; t += kBlock) rec[t].disorder = epoch;
}

template <class MSrc, bool REENC, bool LOCAL>
__global__ __launch_bounds__(kBlock) void sparse_merge_kernel(MSrc src, SparseWs ws, const PeerRun* runs, int npeers,
                                                              unsigned epoch) {
    __shared__ __attribute__((aligned(16))) float lds[kTile];
    __shared__ const int32_t* pidx[kMaxPeers];
    __shared__ const float* pval[kMaxPeers];
    __shared__ unsigned pcnt[kMaxPeers];
    // What this tile needs first lies where the tile's number in the launch says, so it is
    // asked for before the descriptor: the head (where the accumulator tile starts) and the
    // peers' runs.  The accumulator tile of the re-encode is requested as soon as the head is
    // there and is in flight while the peers are merged.
    const unsigned gtile = xcd_grouped(blockIdx.x, gridDim.x);
    const TileHead head = *reinterpret_cast<const TileHead*>(runs + gtile);
    PeerRun run;
    run.idx = run.end = nullptr;
    run.val = nullptr;
    run.disorder = epoch + 1u;
    if ((int)threadIdx.x < npeers) run = runs[(unsigned long long)(1 + threadIdx.x) * gridDim.x + gtile];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const bool fast = head.fast != 0;
    f4 apre[4];
    if (REENC && fast) {
#pragma unroll
        for (int j = 0; j < 4; ++j) apre[j] = ld4(head.acc + wave * kWaveTile + j * 256 + lane * 4);
    }
    unsigned tile;
    const MergeSeg& m = src.get(tile, gtile);
    const Seg s = m.s;
    const Seg r = m.r;  // re-encode descriptor of this chunk: same tile numbering
    const long long n = (long long)s.n;
    const long long t_lo = (long long)tile * kTile, t_hi = t_lo + kTile < n ? t_lo + kTile : n;
    if (REENC && !fast) {
#pragma unroll
        for (int j = 0; j < 4; ++j) apre[j] = ld4_guard(r.s1, t_lo + wave * kWaveTile + j * 256 + lane * 4, n);
    }
    // the sum starts from zero, or from the aggregator's own uncompressed gradient
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned at = wave * kWaveTile + j * 256 + lane * 4;
        f4 v = {0.f, 0.f, 0.f, 0.f};
        if (LOCAL && s.g) v = fast ? ld4(s.g + t_lo + at) : ld4_guard(s.g, t_lo + at, n);
        *reinterpret_cast<f4*>(&lds[at]) = v;
    }
    if ((int)threadIdx.x < npeers) {
        if (run.disorder == epoch) {  // this peer's payload was seen out of order: every pair is looked at
            const unsigned nnz = sparse_header(m.peer[threadIdx.x], m.peer_slots[threadIdx.x], run.idx, run.val);
            run.end = run.idx + nnz;
        }
        pidx[threadIdx.x] = run.idx;
        pval[threadIdx.x] = run.val;
        pcnt[threadIdx.x] = run.end > run.idx ? (unsigned)(run.end - run.idx) : 0u;
    }
    __syncthreads();
    // The pairs of all peers, flattened peer by peer (64-bit positions: flat_pairs.h), are
    // dealt out one per thread, so a whole round is one memory round trip; they are then
    // added peer by peer (sums must follow the peer order; within a peer the indices are
    // distinct).
    using u64 = unsigned long long;
    const u64 total = flat_total(pcnt, (unsigned)npeers);
    for (u64 base = 0; base < total; base += kBlock) {
        const u64 f = base + threadIdx.x;
        unsigned myp = 0;
        u64 before = 0;
        flat_advance(pcnt, (unsigned)npeers, f, myp, before);
        const bool have = f < total;
        long long i = -1;
        float v = 0.f;
        if (have) {
            i = pidx[myp][f - before];
            v = pval[myp][f - before];
        }
        const bool inside = have && i >= t_lo && i < t_hi;
        // peers present in this round (uniform): first and last flat entry of the round
        unsigned pfirst = 0;
        u64 acc0 = 0;
        flat_advance(pcnt, (unsigned)npeers, base, pfirst, acc0);
        const u64 lastf = (base + kBlock < total ? base + kBlock : total) - 1;
        unsigned plast = pfirst;
        u64 acc1 = acc0;
        flat_advance(pcnt, (unsigned)npeers, lastf, plast, acc1);
        for (unsigned p = pfirst; p <= plast; ++p) {
            if (inside && myp == p) atomicAdd(&lds[i - t_lo], v);
            __syncthreads();
        }
    }
    __syncthreads();
    auto from_lds = [&](int j, long long) { return *reinterpret_cast<const f4*>(&lds[wave * kWaveTile + j * 256 + lane * 4]); };
    if (s.out) {  // a re-encoding call may leave the aggregate out
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            long long e = t_lo + wave * kWaveTile + j * 256 + lane * 4;
            if (fast) st4(s.out + e, from_lds(j, e));
            else st4_guard(s.out, e, n, from_lds(j, e));
        }
    }
    if (REENC) {
        if (tile == 0) sparse_reset_select(r, ws);
        auto from_pre = [&](int j, long long) { return apre[j]; };
        if (fast) sparse_accum_tile<true, false>(r, tile, ws, from_lds, from_pre);
        else sparse_accum_tile<false, false>(r, tile, ws, from_lds, from_pre);
    }
}

// =============================================================================
// launchers
// =============================================================================

constexpr unsigned kAccumTilesPerLaunch = 49152;
// Pairs one emit launch is expected to write from which on its clearing stores go straight
// through (clear_element): 1.4-2.0 million are neutral or up to 1 % slower that way, 2.9
// million and more 1.5-4.5 % faster (GradDrop steps of 143-335 M elements at 0.5-2 % kept).
constexpr unsigned long long kEmitStreamFrom = 1ull << 21;

// The same table of tensors, workgroup 0 starting at tile `base` of the launch.
static SingleSrc offset_src(const SingleSrc& s, unsigned base) { return SingleSrc{s.seg, s.base + base}; }
static BatchSrc offset_src(const BatchSrc& s, unsigned base) { return BatchSrc{s.segs, s.map + base}; }

template <class Src, class SegSrcT>
static hipError_t sparse_encode_src(const Src& src, const Src& ssrc_tiles, const SegSrcT& ssrc, unsigned ntiles,
                                    unsigned nstiles, unsigned nsegs, bool dgc, unsigned long long expect_pairs,
                                    const SparseWs& ws, int phase, hipStream_t st) {
    auto on = [&](int p) { return phase < 0 || phase == p || (phase == kSparseAfterAccum && p > 0); };
    const unsigned g4 = (ntiles + 3) / 4;
    if (on(0)) {
        // A launch of this kernel over much more than 40,000 tiles slows down as it goes (6.4 TB/s
        // over the first 35,000 tiles, 5.9 TB/s as the average over 82,000; the plain dense
        // encoders show no such decay), so a long one is issued in equal parts of at most
        // kAccumTilesPerLaunch tiles: 3 % off the accumulate pass of the BERT-large set.
        const unsigned parts = (ntiles + kAccumTilesPerLaunch - 1) / kAccumTilesPerLaunch, per = (ntiles + parts - 1) / parts;
        for (unsigned base = 0; base < ntiles; base += per) {
            const unsigned cnt = ntiles - base < per ? ntiles - base : per;
            const Src part = offset_src(src, base);
            if (dgc) hipLaunchKernelGGL((sparse_accum_kernel<Src, true>), dim3(cnt), dim3(kBlock), 0, st, part, ws);
            else hipLaunchKernelGGL((sparse_accum_kernel<Src, false>), dim3(cnt), dim3(kBlock), 0, st, part, ws);
        }
    }
    if (on(1) && nstiles) hipLaunchKernelGGL((sparse_select_kernel<Src, 0>), dim3(nstiles), dim3(kBlock), 0, st, ssrc_tiles, ws);
    if (on(2) && nstiles) hipLaunchKernelGGL((sparse_select_kernel<Src, 1>), dim3(nstiles), dim3(kBlock), 0, st, ssrc_tiles, ws);
    if (on(3) && nstiles) hipLaunchKernelGGL((sparse_select_kernel<Src, 2>), dim3(nstiles), dim3(kBlock), 0, st, ssrc_tiles, ws);
    if (on(4)) hipLaunchKernelGGL((sparse_count_kernel<Src>), dim3(g4), dim3(kBlock), 0, st, src, ws, ntiles);
    if (on(5)) hipLaunchKernelGGL((sparse_scan_kernel<SegSrcT>), dim3(nsegs), dim3(kScanBlock), 0, st, ssrc, ws);
    if (on(6)) {
        if (expect_pairs > kEmitStreamFrom)
            hipLaunchKernelGGL((sparse_emit_kernel<Src, true>), dim3(g4), dim3(kBlock), 0, st, src, ws, ntiles);
        else
            hipLaunchKernelGGL((sparse_emit_kernel<Src, false>), dim3(g4), dim3(kBlock), 0, st, src, ws, ntiles);
    }
    return hipGetLastError();
}

// phase < 0 runs the whole sequence; 0..6 run one launch of it (accumulate,
// three select passes, count, scan, emit); kSparseAfterAccum runs launches 1..6.
hipError_t launch_sparse_encode(const Launch& L, bool dgc, const SparseWs& ws, int phase, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single)
        return sparse_encode_src(SingleSrc{L.seg}, SingleSrc{L.seg}, SingleSegSrc{L.seg}, L.ntiles, L.seg.nsblk, 1, dgc,
                                 L.expect_pairs, ws, phase, st);
    return sparse_encode_src(BatchSrc{L.dsegs, L.dmap}, BatchSrc{L.dsegs, L.dsmap}, BatchSegSrc{L.dsegs}, L.ntiles,
                             L.nstiles, L.nsegs, dgc, L.expect_pairs, ws, phase, st);
}

hipError_t launch_sparse_decode(const Launch& L, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {
        SingleSrc src{L.seg};
        hipLaunchKernelGGL((zero_fill_kernel<SingleSrc>), dim3(L.ntiles), dim3(kBlock), kLdsFor5, st, src);
        if (L.seg.ncblk)
            hipLaunchKernelGGL((sparse_scatter_kernel<SingleSrc>), dim3(L.seg.ncblk), dim3(kBlock), 0, st, src);
    } else {
        BatchSrc src{L.dsegs, L.dmap};
        hipLaunchKernelGGL((zero_fill_kernel<BatchSrc>), dim3(L.ntiles), dim3(kBlock), kLdsFor5, st, src);
        BatchSrc csrc{L.dsegs, L.dcmap};
        if (L.nctiles)
            hipLaunchKernelGGL((sparse_scatter_kernel<BatchSrc>), dim3(L.nctiles), dim3(kBlock), 0, st, csrc);
    }
    return hipGetLastError();
}

// Decode of a tensor table through tile pointers: tptr has one word per tile of the
// launch, disorder one word per tensor; epoch must differ from call to call.
// few_pairs: most tiles receive no or a handful of pairs, so the tile kernel is a plain
// stream of stores and runs with the occupancy cap of one.  With tens of pairs per tile
// every workgroup waits on a chain of loads first; five workgroups per CU still move
// more bytes then (6-13 %) as long as the launch writes less than about 1 GiB, and fewer
// beyond (5-9 % at 1.3-1.6 GiB, measured on MI355X: the crossover is at 65,536 tiles), so
// the cap is applied below 57,344 tiles only.  The cap of the few-pairs case pays up to
// 262,144 tiles (4 GiB written: +10 % at 98,304 tiles, +1.5 % at 262,144) and costs 9 % at
// 393,216.
constexpr unsigned kTileCapTiles = 57344, kFewPairsCapTiles = 262144;
hipError_t launch_sparse_decode_indexed(const Launch& L, uint32_t* tptr, uint32_t* disorder, unsigned epoch,
                                        bool few_pairs, hipStream_t st) {
    if (L.ntiles == 0 || L.single) return hipSuccess;
    BatchSrc csrc{L.dsegs, L.dcmap};
    if (L.nctiles)
        hipLaunchKernelGGL((sparse_decode_index_kernel<BatchSrc>), dim3(L.nctiles), dim3(kBlock), 0, st, csrc, tptr,
                           disorder, epoch);
    BatchSrc src{L.dsegs, L.dmap};
    hipLaunchKernelGGL((sparse_decode_tile_kernel<BatchSrc>), dim3(L.ntiles), dim3(kBlock),
                       few_pairs ? (L.ntiles <= kFewPairsCapTiles ? kLdsFor4 - 4 * kTile : 0u)
                                 : (L.ntiles <= kTileCapTiles ? kLdsFor5 - 4 * kTile : 0u),
                       st, src, tptr, disorder, epoch);
    return hipGetLastError();
}

// Index launch (phase 0) + tile-owner merge (phase 1); phase < 0 runs both.  With
// L.reencode the merge kernel also runs launch 0 of the GradDrop-style re-encode
// (the caller follows with launch_sparse_encode, kSparseAfterAccum).  runs: records as
// described at PeerRun; slices: the largest peer buffer's slots / 1024, rounded up; epoch:
// a number no earlier call on these records used.
hipError_t launch_sparse_merge(const MergeLaunch& L, const SparseWs& ws, PeerRun* runs, unsigned slices, unsigned epoch,
                               int phase, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    const bool index = phase < 0 || phase == 0, merge = phase < 0 || phase == 1;
    if (slices == 0) slices = 1;
    const unsigned sy = slices < 65535u ? slices : 65535u, sz = (slices + sy - 1) / sy;  // a grid dimension ends at 65535
    // A merge that reads the accumulator and writes it and the aggregate (one read, two write
    // streams) moves 3-6 % more bytes with four workgroups per CU than with the seven its own
    // LDS tile allows (measured on MI355X on the VGG19 chunks and on 400 chunks of 1 Mi, with the
    // buffers allocated chunk by chunk and kind by kind); without the aggregate (one read, one
    // write stream) it is 10 % slower capped, so only the former is.
    const unsigned cap = L.aggregate ? 16u * 1024u : 0u;
    auto merge_launch = [&](auto src) {
        using S = decltype(src);
        dim3 g(L.ntiles), b(kBlock);
        if (L.reencode && L.local)
            hipLaunchKernelGGL((sparse_merge_kernel<S, true, true>), g, b, cap, st, src, ws, runs, L.npeers, epoch);
        else if (L.reencode)
            hipLaunchKernelGGL((sparse_merge_kernel<S, true, false>), g, b, cap, st, src, ws, runs, L.npeers, epoch);
        else if (L.local)
            hipLaunchKernelGGL((sparse_merge_kernel<S, false, true>), g, b, 0, st, src, ws, runs, L.npeers, epoch);
        else
            hipLaunchKernelGGL((sparse_merge_kernel<S, false, false>), g, b, 0, st, src, ws, runs, L.npeers, epoch);
    };
    if (L.single) {
        MergeSingleSegSrc isrc{L.seg};
        if (index)
            hipLaunchKernelGGL((sparse_merge_index_kernel<MergeSingleSegSrc>), dim3(L.npeers, sy, sz), dim3(kBlock), 0, st,
                               isrc, runs, L.npeers, L.ntiles, epoch);
        if (merge) merge_launch(MergeSingleSrc{L.seg});
    } else {
        MergeBatchSegSrc isrc{L.dsegs};
        if (index)
            hipLaunchKernelGGL((sparse_merge_index_kernel<MergeBatchSegSrc>), dim3(L.nsegs * L.npeers, sy, sz), dim3(kBlock),
                               0, st, isrc, runs, L.npeers, L.ntiles, epoch);
        if (merge) merge_launch(MergeBatchSrc{L.dsegs, L.dmap});
    }
    return hipGetLastError();
}

}  // namespace hp
