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
        const float* scales[kPeerChunk];     // terngrad
        long long bucket[kPeerChunk];
        bool use[kPeerChunk];
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            wq[q] = 0u;
            sc[q] = 0.f;
            scales[q] = nullptr;
            bucket[q] = 1;
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
                    // bucket size from the header; a header that does not fit the buffer adds nothing
                    const long long B = h[1];
                    const unsigned long long nb = B >= 1 ? ((unsigned long long)n + B - 1) / B : 0;
                    const unsigned long long off = kHeaderBytes + ((4 * nb + 15) & ~15ull);
                    if (B < 1 || off + 4 * (unsigned long long)nwords > m.peer_bytes[p0 + q]) {
                        use[q] = false;
                        continue;
                    }
                    bucket[q] = B;
                    scales[q] = reinterpret_cast<const float*>(pay + kHeaderBytes);
                    words = reinterpret_cast<const uint32_t*>(pay + off);
                }
                const long long widx = (base >> 4) + lane;
                if (FAST || widx < nwords) wq[q] = words[widx];
            }
        }
#pragma unroll
        for (int q = 0; q < kPeerChunk; ++q) {
            if (!use[q]) continue;  // wavefront-uniform
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
                        agg[j] = agg[j] + expand_codes(byte, sc[q]);
                    } else {
                        const long long e = base + j * 256 + lane * 4, B = bucket[q];
                        f4 d;
                        d.x = e < n ? code_val(byte & 3u, scales[q][e / B]) : 0.f;
                        d.y = e + 1 < n ? code_val((byte >> 2) & 3u, scales[q][(e + 1) / B]) : 0.f;
                        d.z = e + 2 < n ? code_val((byte >> 4) & 3u, scales[q][(e + 2) / B]) : 0.f;
                        d.w = e + 3 < n ? code_val((byte >> 6) & 3u, scales[q][(e + 3) / B]) : 0.f;
                        agg[j] = agg[j] + d;
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

template <class MSrc, int ALG, bool REENC, bool LOCAL>
__global__ __launch_bounds__(kBlock) void dense_merge_kernel(MSrc src, int npeers) {
    unsigned tile;
    const MergeSeg& m = src.get(tile, blockIdx.x);
    if (REENC && tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(m.s.pay);
        h[0] = __float_as_uint(m.s.f0);
        h[1] = (uint32_t)m.s.n;
        h[2] = 0;
        h[3] = 0;
    }
    if (m.s.aligned && (unsigned long long)(tile + 1) * kTile <= m.s.n) merge_tile<true, ALG, REENC, LOCAL>(m, tile, npeers);
    else merge_tile<false, ALG, REENC, LOCAL>(m, tile, npeers);
}

template <class MSrc, bool LOCAL>
static hipError_t dense_merge_src(const MSrc& src, const MergeLaunch& L, int alg, hipStream_t st) {
    dim3 g(L.ntiles), b(kBlock);
    if (alg == HIPRESS_ONEBIT)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_ONEBIT, false, LOCAL>), g, b, 0, st, src, L.npeers);
    else if (alg == HIPRESS_TERNGRAD)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TERNGRAD, false, LOCAL>), g, b, 0, st, src, L.npeers);
    else if (L.reencode)
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TBQ, true, LOCAL>), g, b, 0, st, src, L.npeers);
    else
        hipLaunchKernelGGL((dense_merge_kernel<MSrc, HIPRESS_TBQ, false, LOCAL>), g, b, 0, st, src, L.npeers);
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
