// Dense decode-and-merge for gfx950: the payloads of up to 16 peers are decoded
// and summed in peer order into one fp32 aggregate in a single streaming pass;
// for TBQ the aggregate can be re-encoded for the next hop in the same pass
// (aggregator residual read and written once, aggregate never read back).
#include "common.h"
#include "launch.h"
#include "../../include/hipress_amd.h"

namespace hp {

__device__ __forceinline__ float code_val(unsigned c, float s) {
    return c == 1u ? s : (c == 2u ? -s : 0.f);
}

__device__ __forceinline__ f4 expand_codes(unsigned byte, float sc) {
    f4 o;
    o.x = code_val(byte & 3u, sc);
    o.y = code_val((byte >> 2) & 3u, sc);
    o.z = code_val((byte >> 4) & 3u, sc);
    o.w = code_val((byte >> 6) & 3u, sc);
    return o;
}

// The same sum for a scale that is finite and not negative ("plain": its bits, read as an unsigned
// number, lie below those of +Inf), at two thirds of the instructions.  A code is then worth a
// multiplier 0, +1 or -1, and agg + value is one fused multiply-add: the product is exact, so the
// result is rounded once like the addition of +-s, and a code of 0 adds the product +0 like the
// addition of 0.f (sc = NaN or an infinity would turn 0 * sc into NaN, a negative sc into -0:
// those scales take expand_codes).  The multipliers of a byte's four codes are made together as
// two-bit signed fields: 00 -> 00, 01 -> 01, 10 -> 11, and the unused 11 -> 00.  Used for TBQ
// peers, whose scale is one number per peer (8 peers over the VGG19 chunks without re-encode
// 200 -> 184 us); with TernGrad's per-bucket scales the decision costs more than it saves
// (377 -> 396 us per lane, 409 us per wavefront and peer).
__device__ __forceinline__ bool plain_scale(float sc) { return __float_as_uint(sc) < 0x7f800000u; }

__device__ __forceinline__ unsigned code_multipliers(unsigned byte) {
    const unsigned hi = byte >> 1;
    const unsigned one = (byte ^ hi) & 0x55u;    // exactly one bit of the code set: the low bit of the field
    const unsigned neg = hi & ~byte & 0x55u;     // code 10: also the high bit
    return one | (neg << 1);
}

__device__ __forceinline__ f4 add_codes_plain(f4 agg, unsigned byte, float sc) {
    const int m = (int)code_multipliers(byte);
    agg.x = __fmaf_rn((float)(int)__builtin_amdgcn_sbfe(m, 0, 2), sc, agg.x);
    agg.y = __fmaf_rn((float)(int)__builtin_amdgcn_sbfe(m, 2, 2), sc, agg.y);
    agg.z = __fmaf_rn((float)(int)__builtin_amdgcn_sbfe(m, 4, 2), sc, agg.z);
    agg.w = __fmaf_rn((float)(int)__builtin_amdgcn_sbfe(m, 6, 2), sc, agg.w);
    return agg;
}

__device__ __forceinline__ unsigned tbq_q(float v, float tau, float& keep) {
    unsigned c = v >= tau ? 1u : (v <= -tau ? 2u : 0u);
    keep = c == 1u ? v - tau : (c == 2u ? v + tau : v);
    return c;
}

// LOCAL: some chunk of the launch starts its sum from a local gradient (Seg::g).
template <bool FAST, int ALG, bool REENC, bool LOCAL>
__device__ __forceinline__ void merge_tile(const MergeSeg& m, unsigned tile, int npeers) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const Seg s = m.s;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    f4 agg[4], rpre[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // the sum starts from zero, or from the aggregator's own uncompressed gradient
        agg[j] = (f4){0.f, 0.f, 0.f, 0.f};
        if (LOCAL && s.g) agg[j] = load4<FAST>(s.g, base + j * 256 + lane * 4, n);
        // the aggregator's residual is requested first: it is in flight while the peers are added
        if (REENC) rpre[j] = load4<FAST>(s.s0, base + j * 256 + lane * 4, n);
    }
    // Up to eight peers at a time.  First everything that comes from memory is requested:
    // per peer one word per lane (the 1024 elements of the wavefront are 64 two-bit or 32
    // one-bit words) and the scalar of its header.  Then the peers are added one after the
    // other, each lane taking the word it needs from the lane that loaded it.
    constexpr int kPeerChunk = 8;
    for (int p0 = 0; p0 < npeers; p0 += kPeerChunk) {
        uint32_t wq[kPeerChunk];
        float sc[kPeerChunk];                // onebit: scale, tbq: threshold
        bool use[kPeerChunk];
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            wq[q] = 0u;
            sc[q] = 0.f;
            use[q] = p0 + q < npeers;
            if (!use[q]) continue;
            const uint8_t* pay = m.peer[p0 + q];
            const uint32_t* h = reinterpret_cast<const uint32_t*>(pay);
            if (ALG == HIPRESS_ONEBIT) {
                sc[q] = __uint_as_float(h[0]);
                const uint32_t* words = reinterpret_cast<const uint32_t*>(pay + kHeaderBytes);
                const long long widx = (base >> 5) + lane;
                if (lane < 32u && (FAST || widx < ((n + 31) >> 5))) wq[q] = words[widx];
            } else {
                const long long nwords = (n + 15) >> 4;
                const uint32_t* words;
                if (ALG == HIPRESS_TBQ) {
                    sc[q] = __uint_as_float(h[0]);
                    words = reinterpret_cast<const uint32_t*>(pay + kHeaderBytes);
                } else {
                    static_assert(ALG != HIPRESS_TERNGRAD, "terngrad has a tile function of its own");
                    words = nullptr;
                }
                const long long widx = (base >> 4) + lane;
                if (FAST || widx < nwords) wq[q] = words[widx];
            }
        }
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            if (!use[q]) continue;  // wavefront-uniform
            const bool plain = ALG == HIPRESS_TBQ && plain_scale(sc[q]);  // the same for the whole launch of a peer
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (ALG == HIPRESS_ONEBIT) {
                    const uint32_t w = (uint32_t)__shfl((int)wq[q], j * 8 + (int)(lane >> 3), 64);
                    const unsigned nib = (w >> (4 * (lane & 7u))) & 0xfu;
                    f4 d;
                    d.x = (nib & 1u) ? sc[q] : -sc[q];
                    d.y = (nib & 2u) ? sc[q] : -sc[q];
                    d.z = (nib & 4u) ? sc[q] : -sc[q];
                    d.w = (nib & 8u) ? sc[q] : -sc[q];
                    agg[j] = agg[j] + d;
                } else {
                    const uint32_t w = (uint32_t)__shfl((int)wq[q], j * 16 + (int)(lane >> 2), 64);
                    const unsigned byte = (w >> (8 * (lane & 3u))) & 0xffu;
                    if (ALG == HIPRESS_TBQ) {
                        if (plain) agg[j] = add_codes_plain(agg[j], byte, sc[q]);
                        else agg[j] = agg[j] + expand_codes(byte, sc[q]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (s.out) store4<FAST>(s.out, base + j * 256 + lane * 4, n, agg[j]);  // a re-encoding call may leave the aggregate out
    if (REENC) {
        const float tau = s.f0;
        uint32_t* owords = reinterpret_cast<uint32_t*>(s.pay + kHeaderBytes);
        unsigned myword = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            long long e = base + j * 256 + lane * 4;
            f4 v = rpre[j] + agg[j];
            f4 keep;
            float k;
            unsigned byte = 0, c;
            c = tbq_q(v.x, tau, k); keep.x = k; byte |= c;
            c = tbq_q(v.y, tau, k); keep.y = k; byte |= c << 2;
            c = tbq_q(v.z, tau, k); keep.z = k; byte |= c << 4;
            c = tbq_q(v.w, tau, k); keep.w = k; byte |= c << 6;
            if (!FAST) {
                unsigned vm = valid4(e, n);
                byte &= ((vm & 1u) * 0x03u) | ((vm >> 1 & 1u) * 0x0cu) | ((vm >> 2 & 1u) * 0x30u) |
                        ((vm >> 3 & 1u) * 0xc0u);
            }
            store4<FAST>(s.s0, e, n, keep);
            unsigned w = quad_pack8(byte);
            myword = ((lane & 3u) == (unsigned)j) ? w : myword;
        }
        long long widx = (base >> 4) + (lane & 3u) * 16 + (lane >> 2);
        if (FAST || widx < (long long)((n + 15) >> 4)) owords[widx] = myword;
    }
}

// ---- TernGrad peers --------------------------------------------------------------------
// A TernGrad payload keeps one scale per bucket between its header and its words, so where the
// words start, and which scale an element takes, follow from the bucket size in the header.
// Everything here is arranged so that this costs one round trip to memory and a handful of
// instructions per wavefront and tile, not per peer or per element:
//  * n and the bucket size are 32-bit quantities; a power of two divides by shifting;
//  * the peers of a launch normally share one bucket size.  The launch may name it
//    (Seg::bucket; otherwise the first peer's header does), the geometry for it - where the words
//    start, which bucket and place the wavefront's and each lane's first elements have - is
//    worked out once, and words and scales of all peers are asked for from it straight away,
//    together with the headers.  A header that names another size decides: that peer alone is
//    set up again from its own header.
struct TgGeom {
    unsigned long long words_off;  // byte offset of the packed words from the payload base
    unsigned q0, r0;               // bucket of the wavefront's first element, and that element's place in it
    bool ok;                       // the bucket size is usable
};

__device__ __forceinline__ TgGeom tg_geom(unsigned B, unsigned n32, unsigned b32) {
    TgGeom g;
    g.ok = B >= 1u;
    unsigned nb = 0u;
    g.q0 = g.r0 = 0u;
    if (g.ok) {
        if ((B & (B - 1u)) == 0u) {
            const unsigned sh = (unsigned)__ffs((int)B) - 1u;
            nb = (n32 >> sh) + ((n32 & (B - 1u)) != 0u);
            g.q0 = b32 >> sh;
            g.r0 = b32 & (B - 1u);
        } else {
            nb = n32 / B + (n32 % B != 0u);
            g.q0 = b32 / B;
            g.r0 = b32 - g.q0 * B;
        }
    }
    g.words_off = kHeaderBytes + ((4ull * nb + 15ull) & ~15ull);
    return g;
}

// Bucket (pq) and place in it (pr) of the lane's first element in each of the four steps.
__device__ __forceinline__ void tg_positions(const TgGeom& g, unsigned B, unsigned lane, unsigned (&pq)[4], unsigned (&pr)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if ((B & 255u) == 0u) {
            // a step of 256 aligned elements lies inside one bucket, at most three on from the wavefront's first
            const unsigned long long x = (unsigned long long)g.r0 + (unsigned)(j * 256);
            pq[j] = g.q0 + (unsigned)(x >= B) + (unsigned)(x >= 2ull * B) + (unsigned)(x >= 3ull * B);
            pr[j] = 0u;  // not used: every element of the step shares the bucket
        } else {
            const BucketPos bp = bucket_pos(g.q0, g.r0, (unsigned)(j * 256) + lane * 4u, B);
            pq[j] = (unsigned)bp.q;
            pr[j] = (unsigned)bp.r;
        }
    }
}

// Asks for one peer's word and for the scales of the lane's first elements; false when the
// payload cannot hold what its bucket size implies (such a peer adds nothing).
template <bool FAST>
__device__ __forceinline__ bool tg_request(const uint8_t* pay, unsigned long long pay_bytes, const TgGeom& g,
                                           const unsigned (&pq)[4], long long n, long long base, unsigned lane,
                                           uint32_t& word, float (&sc)[4]) {
    const long long nwords = (n + 15) >> 4;
    word = 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) sc[j] = 0.f;
    if (!g.ok || g.words_off + 4ull * (unsigned long long)nwords > pay_bytes) return false;
    const uint32_t* words = reinterpret_cast<const uint32_t*>(pay + g.words_off);
    const float* scales = reinterpret_cast<const float*>(pay + kHeaderBytes);
    const long long widx = (base >> 4) + lane;
    if (FAST || widx < nwords) word = words[widx];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (base + j * 256 + lane * 4 < n) sc[j] = scales[pq[j]];
    return true;
}

// The tile function for a launch whose bucket size is named by the host (a batch).  With a multiple of
// 256 (512, the usual one, among them) a step's 256 elements share a bucket, so nothing below
// looks at single elements; and with any size no peer is set up a second time - which is what makes
// the general function further down take 121 registers and 365 us for 8 peers over the VGG19 chunks,
// against 94 registers and 235 us here.  It holds no code for a peer whose header names another bucket size
// and does not even read the headers (eight more scalar loads per wavefront and tile cost 35 us):
// a launch of one wavefront per chunk looks at them first and flags the chunks in which some
// header disagrees (terngrad_headers_kernel); a flagged chunk's tiles store nothing here - the flag
// is asked for at the start and looked at before the stores - and are written by a third launch,
// a few workgroups per chunk that run the general function over the flagged chunks' tiles and
// return at once from the others (terngrad_others_kernel).
// B256: the bucket size is a multiple of 256; otherwise it is any size, the lane's first elements are
// placed by division and four elements that straddle a bucket border look their scales up one by one
// (8 peers, buckets of 100: 411 us in the general function, 324 us here).
template <bool FAST, bool LOCAL, bool B256>
__device__ __forceinline__ void merge_tile_terngrad_lean(const MergeSeg& m, unsigned tile, int npeers, const unsigned* flags) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const Seg s = m.s;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    if (base >= n) return;
    const unsigned B = s.bucket;  // named by the host, at least 1 (B256: a multiple of 256)
    const unsigned flagged = flags[s.id];
    const TgGeom g = tg_geom(B, (unsigned)n, (unsigned)base);
    unsigned pq[4], pr[4];
    if (B256) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned long long x = (unsigned long long)g.r0 + (unsigned)(j * 256);
            pq[j] = g.q0 + (unsigned)(x >= B) + (unsigned)(x >= 2ull * B) + (unsigned)(x >= 3ull * B);
            pr[j] = 0u;
        }
    } else {
        tg_positions(g, B, lane, pq, pr);
    }
    f4 agg[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        agg[j] = (f4){0.f, 0.f, 0.f, 0.f};
        if (LOCAL && s.g) agg[j] = load4<FAST>(s.g, base + j * 256 + lane * 4, n);
    }
    constexpr int kPeerChunk = 8;
    for (int p0 = 0; p0 < npeers; p0 += kPeerChunk) {
        uint32_t wq[kPeerChunk];
        float tsc[kPeerChunk][4];
        unsigned usemask = 0u;
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            wq[q] = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j) tsc[q][j] = 0.f;
            if (p0 + q >= npeers) continue;
            if (tg_request<FAST>(m.peer[p0 + q], m.peer_bytes[p0 + q], g, pq, n, base, lane, wq[q], tsc[q])) usemask |= 1u << q;
        }
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            if (!((usemask >> q) & 1u)) continue;  // wavefront-uniform
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = (uint32_t)__shfl((int)wq[q], j * 16 + (int)(lane >> 2), 64);
                const unsigned byte = (w >> (8 * (lane & 3u))) & 0xffu;
                if (B256 || (B & 255u) == 0u || (unsigned long long)pr[j] + 3ull < B) {
                    agg[j] = agg[j] + expand_codes(byte, tsc[q][j]);  // the four share a bucket; codes beyond n are 0
                } else {
                    const float* scales = reinterpret_cast<const float*>(m.peer[p0 + q] + kHeaderBytes);
                    const long long e = base + j * 256 + lane * 4;
                    unsigned bq = pq[j], br = pr[j];
                    float sck = tsc[q][j], dv[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const unsigned c = (byte >> (2 * k)) & 3u;
                        dv[k] = (e + k < n && c) ? code_val(c, sck) : 0.f;
                        if (++br == B) {  // the next element begins a bucket: its scale is looked up here
                            br = 0u;
                            ++bq;
                            if (k < 3 && e + k + 1 < n) sck = scales[bq];
                        }
                    }
                    f4 d;
                    d.x = dv[0]; d.y = dv[1]; d.z = dv[2]; d.w = dv[3];
                    agg[j] = agg[j] + d;
                }
            }
        }
    }
    if (flagged) return;  // wavefront-uniform: the third launch writes this chunk's tiles
#pragma unroll
    for (int j = 0; j < 4; ++j) store4<FAST>(s.out, base + j * 256 + lane * 4, n, agg[j]);
}

template <bool FAST, bool LOCAL>
__device__ __forceinline__ void merge_tile_terngrad(const MergeSeg& m, unsigned tile, int npeers) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const Seg s = m.s;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    if (base >= n) return;
    const unsigned n32 = (unsigned)n, b32 = (unsigned)base;
    f4 agg[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        agg[j] = (f4){0.f, 0.f, 0.f, 0.f};
        if (LOCAL && s.g) agg[j] = load4<FAST>(s.g, base + j * 256 + lane * 4, n);
    }
    constexpr int kPeerChunk = 8;  // two or four at a time are no faster: the adds, not the loads, bound this kernel
    for (int p0 = 0; p0 < npeers; p0 += kPeerChunk) {
        unsigned hb[kPeerChunk];  // bucket sizes as the headers have them
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            hb[q] = 0u;
            if (p0 + q < npeers) hb[q] = reinterpret_cast<const uint32_t*>(m.peer[p0 + q])[1];
        }
        // the size the peers are expected to share: named by the launch, else the first header's
        const unsigned B0 = s.bucket ? s.bucket : (unsigned)__builtin_amdgcn_readfirstlane((int)hb[0]);
        const TgGeom g0 = tg_geom(B0, n32, b32);
        unsigned pq0[4], pr0[4];
        tg_positions(g0, B0 ? B0 : 1u, lane, pq0, pr0);
        uint32_t wq[kPeerChunk];
        float tsc[kPeerChunk][4];
        unsigned usemask = 0u;
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            wq[q] = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j) tsc[q][j] = 0.f;
            if (p0 + q < npeers && tg_request<FAST>(m.peer[p0 + q], m.peer_bytes[p0 + q], g0, pq0, n, base, lane, wq[q], tsc[q]))
                usemask |= 1u << q;
        }
        // the headers have their say: a peer of another bucket size is set up again from its own
        unsigned ownmask = 0u;
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            if (p0 + q < npeers && hb[q] != B0) {  // wavefront-uniform, rare
                const TgGeom g = tg_geom(hb[q], n32, b32);
                unsigned pq[4], pr[4];
                tg_positions(g, hb[q] ? hb[q] : 1u, lane, pq, pr);
                usemask &= ~(1u << q);
                if (tg_request<FAST>(m.peer[p0 + q], m.peer_bytes[p0 + q], g, pq, n, base, lane, wq[q], tsc[q])) usemask |= 1u << q;
                ownmask |= 1u << q;
            }
        }
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            if (!((usemask >> q) & 1u)) continue;  // wavefront-uniform
            const bool own = (ownmask >> q) & 1u;
            const unsigned B = own ? hb[q] : B0;
            unsigned pq[4], pr[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                pq[j] = pq0[j];
                pr[j] = pr0[j];
            }
            if (own) tg_positions(tg_geom(B, n32, b32), B, lane, pq, pr);
            const float* scales = reinterpret_cast<const float*>(m.peer[p0 + q] + kHeaderBytes);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = (uint32_t)__shfl((int)wq[q], j * 16 + (int)(lane >> 2), 64);
                const unsigned byte = (w >> (8 * (lane & 3u))) & 0xffu;
                if ((B & 255u) == 0u || (unsigned long long)pr[j] + 3ull < B) {
                    // the lane's four elements share a bucket (codes beyond n are 0)
                    agg[j] = agg[j] + expand_codes(byte, tsc[q][j]);
                } else {
                    const long long e = base + j * 256 + lane * 4;
                    unsigned bq = pq[j], br = pr[j];
                    float sck = tsc[q][j], dv[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const unsigned c = (byte >> (2 * k)) & 3u;
                        dv[k] = (e + k < n && c) ? code_val(c, sck) : 0.f;
                        if (++br == B) {  // the next element begins a bucket: its scale is looked up here
                            br = 0u;
                            ++bq;
                            if (k < 3 && e + k + 1 < n) sck = scales[bq];
                        }
                    }
                    f4 d;
                    d.x = dv[0]; d.y = dv[1]; d.z = dv[2]; d.w = dv[3];
                    agg[j] = agg[j] + d;
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) store4<FAST>(s.out, base + j * 256 + lane * 4, n, agg[j]);
}

// LEAN (TernGrad only): 1 the lean tile function for bucket sizes that are multiples of 256, 2 the one for any
// size, 0 the general function; flags: one word per chunk, not zero where a header disagrees.
template <class MSrc, int ALG, bool REENC, bool LOCAL, int LEAN = 0>
__global__ __launch_bounds__(kBlock) void dense_merge_kernel(MSrc src, int npeers, const unsigned* flags) {
    unsigned tile;
    const MergeSeg& m = src.get(tile, blockIdx.x);
    if (REENC && tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(m.s.pay);
        h[0] = __float_as_uint(m.s.f0);
        h[1] = (uint32_t)m.s.n;
        h[2] = 0;
        h[3] = 0;
    }
    const bool fast = m.s.aligned && (unsigned long long)(tile + 1) * kTile <= m.s.n;
    if constexpr (ALG == HIPRESS_TERNGRAD) {
        if constexpr (LEAN != 0) {
            if (fast) merge_tile_terngrad_lean<true, LOCAL, LEAN == 1>(m, tile, npeers, flags);
            else merge_tile_terngrad_lean<false, LOCAL, LEAN == 1>(m, tile, npeers, flags);
        } else {
            if (fast) merge_tile_terngrad<true, LOCAL>(m, tile, npeers);
            else merge_tile_terngrad<false, LOCAL>(m, tile, npeers);
        }
    } else {
        if (fast) merge_tile<true, ALG, REENC, LOCAL>(m, tile, npeers);
        else merge_tile<false, ALG, REENC, LOCAL>(m, tile, npeers);
    }
}

// One wavefront per chunk: flags[chunk] = some peer's header names another bucket size than the launch.
template <class SegSrc>
__global__ __launch_bounds__(64) void terngrad_headers_kernel(SegSrc src, int npeers, unsigned* flags) {
    const MergeSeg& m = src.at(blockIdx.x);
    const unsigned B = m.s.bucket;
    unsigned differ = 0u;
    for (int p = (int)threadIdx.x; p < npeers; p += 64) differ |= reinterpret_cast<const uint32_t*>(m.peer[p])[1] ^ B;
    const bool any = __any(differ != 0u);
    if (threadIdx.x == 0) flags[m.s.id] = any ? 1u : 0u;
}

// The general function over the tiles of the flagged chunks; gridDim.y workgroups share a chunk's tiles.
template <class SegSrc, bool LOCAL>
__global__ __launch_bounds__(kBlock) void terngrad_others_kernel(SegSrc src, int npeers, const unsigned* flags) {
    const MergeSeg& m = src.at(blockIdx.x);
    if (!flags[m.s.id]) return;
    for (unsigned tile = blockIdx.y; tile < m.s.ntiles; tile += gridDim.y) {
        if (m.s.aligned && (unsigned long long)(tile + 1) * kTile <= m.s.n) merge_tile_terngrad<true, LOCAL>(m, tile, npeers);
        else merge_tile_terngrad<false, LOCAL>(m, tile, npeers);
    }
}

template <class MSrc, bool LOCAL>
static hipError_t dense_merge_src(const MSrc& src, const MergeLaunch& L, int alg, hipStream_t st) {
    dim3 g(L.ntiles), b(kBlock);
    if (alg == HIPRESS_ONEBIT)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_ONEBIT, false, LOCAL>), g, b, 0, st, src, L.npeers, static_cast<const unsigned*>(nullptr));
    else if (alg == HIPRESS_TERNGRAD && L.tgflags) {  // a batch: its descriptors name the bucket size
        const MergeBatchSegSrc segs{L.dsegs};
        hipLaunchKernelGGL((terngrad_headers_kernel<MergeBatchSegSrc>), dim3(L.nsegs), dim3(64), 0, st, segs, L.npeers, L.tgflags);
        if (L.bucket256)
            hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TERNGRAD, false, LOCAL, 1>), g, b, 0, st, src, L.npeers, L.tgflags);
        else
            hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TERNGRAD, false, LOCAL, 2>), g, b, 0, st, src, L.npeers, L.tgflags);
        hipLaunchKernelGGL((terngrad_others_kernel<MergeBatchSegSrc, LOCAL>), dim3(L.nsegs, 8), b, 0, st, segs, L.npeers, L.tgflags);
    }
    else if (alg == HIPRESS_TERNGRAD)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TERNGRAD, false, LOCAL>), g, b, 0, st, src, L.npeers, static_cast<const unsigned*>(nullptr));
    else if (L.reencode)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TBQ, true, LOCAL>), g, b, 0, st, src, L.npeers, static_cast<const unsigned*>(nullptr));
    else
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TBQ, false, LOCAL>), g, b, 0, st, src, L.npeers, static_cast<const unsigned*>(nullptr));
    return hipGetLastError();
}

hipError_t launch_dense_merge(const MergeLaunch& L, int alg, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {
        if (L.local) return dense_merge_src<MergeSingleSrc, true>(MergeSingleSrc{L.seg}, L, alg, st);
        return dense_merge_src<MergeSingleSrc, false>(MergeSingleSrc{L.seg}, L, alg, st);
    }
    if (L.local) return dense_merge_src<MergeBatchSrc, true>(MergeBatchSrc{L.dsegs, L.dmap}, L, alg, st);
    return dense_merge_src<MergeBatchSrc, false>(MergeBatchSrc{L.dsegs, L.dmap}, L, alg, st);
}

}  // namespace hp
