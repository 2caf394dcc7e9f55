// Dense quantisers for gfx950: TBQ, onebit and TernGrad encode/decode.
// Every kernel is a streaming pass bounded by HBM bandwidth; see common.h for the
// tile / wavefront / lane decomposition all of them share.
#include "common.h"
#include "launch.h"

namespace hp {

// =============================================================================
// TBQ
// =============================================================================

// v -> code (0, 1 = +tau, 2 = -tau) and the residual that stays behind.
__device__ __forceinline__ unsigned tbq_quant(float v, float tau, float& keep) {
    unsigned c = v >= tau ? 1u : (v <= -tau ? 2u : 0u);
    keep = c == 1u ? v - tau : (c == 2u ? v + tau : v);
    return c;
}

__device__ __forceinline__ float code_value(unsigned c, float s) {
    return c == 1u ? s : (c == 2u ? -s : 0.f);
}

// Quantises the four elements of one lane, returns their 8 code bits.
template <bool FAST>
__device__ __forceinline__ unsigned tbq_quant4(f4 v, float tau, unsigned valid, f4& keep) {
    unsigned byte = 0;
    float k;
    unsigned c;
    c = tbq_quant(v.x, tau, k); keep.x = k; byte |= c;
    c = tbq_quant(v.y, tau, k); keep.y = k; byte |= c << 2;
    c = tbq_quant(v.z, tau, k); keep.z = k; byte |= c << 4;
    c = tbq_quant(v.w, tau, k); keep.w = k; byte |= c << 6;
    if (!FAST) {  // elements past the end produce pad code 0
        unsigned m = ((valid & 1u) * 0x03u) | ((valid >> 1 & 1u) * 0x0cu) | ((valid >> 2 & 1u) * 0x30u) |
                     ((valid >> 3 & 1u) * 0xc0u);
        byte &= m;
    }
    return byte;
}

// Shared tail of TBQ encode and of the fused re-encode in decode-and-merge:
// v[j] are this lane's 16 values; writes residual and packed words.
template <bool FAST>
__device__ __forceinline__ void tbq_emit(const f4 (&v)[4], float tau, float* res, uint32_t* words,
                                         long long wbase_elem, long long n, unsigned lane) {
    unsigned myword = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = wbase_elem + j * 256 + lane * 4;
        f4 keep;
        unsigned byte = tbq_quant4<FAST>(v[j], tau, FAST ? 0xfu : valid4(e, n), keep);
        store4<FAST>(res, e, n, keep);
        unsigned w = quad_pack8(byte);
        myword = ((lane & 3u) == (unsigned)j) ? w : myword;
    }
    // lane 4q+j holds the word of step j, quad q
    long long widx = (wbase_elem >> 4) + (lane & 3u) * 16 + (lane >> 2);
    if (FAST || widx < (long long)((n + 15) >> 4)) words[widx] = myword;
}

template <bool FAST>
__device__ __forceinline__ void tbq_encode_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const float tau = s.f0;
    f4 g[4], r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        r[j] = load4<FAST>(s.s0, e, n);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = r[j] + g[j];
    tbq_emit<FAST>(r, tau, s.s0, reinterpret_cast<uint32_t*>(s.pay + kHeaderBytes), base, n, lane);
}

template <class Src>
__global__ __launch_bounds__(kBlock) void tbq_encode_kernel(Src src) {
    four_waves_per_simd();
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = __float_as_uint(s.f0);
        h[1] = (uint32_t)s.n;
        h[2] = 0;
        h[3] = 0;
    }
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) tbq_encode_tile<true>(s, tile);
    else tbq_encode_tile<false>(s, tile);
}

// Expands the 8 code bits of one lane to four values of magnitude sc.
__device__ __forceinline__ f4 expand2(unsigned byte, float sc) {
    f4 o;
    o.x = code_value(byte & 3u, sc);
    o.y = code_value((byte >> 2) & 3u, sc);
    o.z = code_value((byte >> 4) & 3u, sc);
    o.w = code_value((byte >> 6) & 3u, sc);
    return o;
}

// The byte of 2-bit codes that lane `lane` needs in step j of a wavefront whose
// first element is wbase_elem (a multiple of 1024).
template <bool FAST>
__device__ __forceinline__ unsigned fetch_byte2(const uint32_t* words, long long wbase_elem, int j,
                                                unsigned lane, long long nwords) {
    long long widx = (wbase_elem >> 4) + j * 16 + (lane >> 2);
    uint32_t w = (FAST || widx < nwords) ? words[widx] : 0u;
    return (w >> (8 * (lane & 3u))) & 0xffu;
}

template <bool FAST>
__device__ __forceinline__ void tbq_decode_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const uint32_t* words = reinterpret_cast<const uint32_t*>(s.pay + kHeaderBytes);
    const float tau = *reinterpret_cast<const float*>(s.pay);
    const long long nwords = (n + 15) >> 4;
    unsigned b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = fetch_byte2<FAST>(words, base, j, lane, nwords);
#pragma unroll
    for (int j = 0; j < 4; ++j) store4<FAST>(s.out, base + j * 256 + lane * 4, n, expand2(b[j], tau));
}

template <class Src>
__global__ __launch_bounds__(kBlock) void tbq_decode_kernel(Src src) {
    four_waves_per_simd();
    unsigned tile;
    const Seg s = src.get(tile, xcd_grouped(blockIdx.x, gridDim.x));
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) tbq_decode_tile<true>(s, tile);
    else tbq_decode_tile<false>(s, tile);
}

// =============================================================================
// onebit
// =============================================================================

__device__ __forceinline__ float abs4sum(f4 v) {
    return (fabsf(v.x) + fabsf(v.y)) + (fabsf(v.z) + fabsf(v.w));
}

// Pass 1: one partial sum of |r+g| per tile, in a fixed order (deterministic).
// KEEP: plain loads, for the tiles the quantise pass is to find on the chip (cache_tail).
template <bool FAST, bool KEEP = false>
__device__ __forceinline__ float onebit_abs_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    f4 g[4], r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = KEEP ? ld4_keep(s.g + e) : load4<FAST>(s.g, e, n);
        r[j] = KEEP ? ld4_keep(s.s0 + e) : load4<FAST>(s.s0, e, n);
    }
    float a = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) a += abs4sum(r[j] + g[j]);
    return a;
}

template <class Src>
__global__ __launch_bounds__(kBlock) void onebit_abs_kernel(Src src, float* partial) {
    four_waves_per_simd();
    __shared__ float wsum[4];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    float a;
    const bool whole = s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n;
    if (whole && cache_tail(blockIdx.x, gridDim.x, 2)) a = onebit_abs_tile<true, true>(s, tile);
    else if (whole) a = onebit_abs_tile<true>(s, tile);
    else a = onebit_abs_tile<false>(s, tile);
    a = wave_sum(a);
    if ((threadIdx.x & 63u) == 0) wsum[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) partial[s.tile0 + tile] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}

// Pass 2: one workgroup of 1024 threads per tensor adds that tensor's partials in
// double, in a fixed order, and writes the header {scale, n, 0, 0} (and the
// scale-state word of the deferred variant).
constexpr int kScaleBlock = 1024;

__device__ __forceinline__ double wave_sum_d(double x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
    return x;
}

template <class Src>
__global__ __launch_bounds__(kScaleBlock) void onebit_scale_kernel(Src src, const float* partial) {
    __shared__ double red[kScaleBlock / 64];
    const Seg s = src.at(blockIdx.x);
    const float* p = partial + s.tile0;
    const unsigned nt = s.ntiles;
    double a0 = 0.0, a1 = 0.0, a2 = 0.0, a3 = 0.0;
    unsigned t = threadIdx.x;
    for (; t + 3 * kScaleBlock < nt; t += 4 * kScaleBlock) {
        float x0 = p[t], x1 = p[t + kScaleBlock], x2 = p[t + 2 * kScaleBlock], x3 = p[t + 3 * kScaleBlock];
        a0 += (double)x0;
        a1 += (double)x1;
        a2 += (double)x2;
        a3 += (double)x3;
    }
    for (; t < nt; t += kScaleBlock) a0 += (double)p[t];
    double a = wave_sum_d((a0 + a1) + (a2 + a3));
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        double tot = 0.0;
        for (int w = 0; w < kScaleBlock / 64; ++w) tot += red[w];
        float sc = s.n ? (float)(tot / (double)s.n) : 0.f;
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = __float_as_uint(sc);
        h[1] = (uint32_t)s.n;
        h[2] = 0;
        h[3] = 0;
        if (s.s1) *s.s1 = sc;
    }
}

template <bool FAST>
__device__ __forceinline__ void onebit_quant_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const float sc = *reinterpret_cast<const float*>(s.pay);
    uint32_t* words = reinterpret_cast<uint32_t*>(s.pay + kHeaderBytes);
    f4 g[4], r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        r[j] = load4<FAST>(s.s0, e, n);
    }
    unsigned myword = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        f4 v = r[j] + g[j];
        unsigned b0 = v.x >= 0.f, b1 = v.y >= 0.f, b2 = v.z >= 0.f, b3 = v.w >= 0.f;
        f4 keep;
        keep.x = v.x - (b0 ? sc : -sc);
        keep.y = v.y - (b1 ? sc : -sc);
        keep.z = v.z - (b2 ? sc : -sc);
        keep.w = v.w - (b3 ? sc : -sc);
        unsigned nib = b0 | (b1 << 1) | (b2 << 2) | (b3 << 3);
        if (!FAST) nib &= valid4(e, n);
        store4<FAST>(s.s0, e, n, keep);
        unsigned w = oct_pack4(nib, lane);
        myword = ((lane & 7u) == (unsigned)j) ? w : myword;
    }
    // lane 8o+j (j < 4) holds the word of step j, octet o
    long long widx = (base >> 5) + (lane & 7u) * 8 + (lane >> 3);
    if ((lane & 7u) < 4u && (FAST || widx < (long long)((n + 31) >> 5))) words[widx] = myword;
}

// The launch is walked from its end towards its start: the pass that summed |r+g| finished
// there and left its last tiles in the Infinity Cache (xcd_reversed, cache_tail).
template <class Src>
__global__ __launch_bounds__(kBlock) void onebit_quant_kernel(Src src) {
    four_waves_per_simd();
    unsigned tile;
    const Seg s = src.get(tile, xcd_reversed(blockIdx.x, gridDim.x));
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) onebit_quant_tile<true>(s, tile);
    else onebit_quant_tile<false>(s, tile);
}

// ---- deferred residual ----------------------------------------------------------
// The two-pass encode above reads gradient and residual twice because the scale
// must be known before r' = v - d can be written.  The deferred variant keeps
// the state buffer one step behind: it stores v (the value before the scale was
// subtracted) together with that step's scale in a one-word side buffer, and the
// NEXT call forms r = v_prev - d(v_prev, s_prev) on the fly before adding the new
// gradient - the same two roundings in the same order, so every bit matches the
// two-pass operator.  One pass per step: read g and state, write state and bits.
template <bool FAST>
__device__ __forceinline__ float onebit_deferred_tile(const Seg& s, unsigned tile, float sp) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    uint32_t* words = reinterpret_cast<uint32_t*>(s.pay + kHeaderBytes);
    f4 g[4], v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        v[j] = load4<FAST>(s.s0, e, n);
    }
    unsigned myword = 0;
    float a = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        f4 r;  // residual the two-pass operator would have stored last step
        r.x = v[j].x - (v[j].x >= 0.f ? sp : -sp);
        r.y = v[j].y - (v[j].y >= 0.f ? sp : -sp);
        r.z = v[j].z - (v[j].z >= 0.f ? sp : -sp);
        r.w = v[j].w - (v[j].w >= 0.f ? sp : -sp);
        f4 nv = r + g[j];
        unsigned nib = (nv.x >= 0.f) | ((nv.y >= 0.f) << 1) | ((nv.z >= 0.f) << 2) | ((nv.w >= 0.f) << 3);
        if (!FAST) {
            unsigned vm = valid4(e, n);
            nib &= vm;
            nv.x = (vm & 1u) ? nv.x : 0.f;
            nv.y = (vm & 2u) ? nv.y : 0.f;
            nv.z = (vm & 4u) ? nv.z : 0.f;
            nv.w = (vm & 8u) ? nv.w : 0.f;
        }
        a += abs4sum(nv);
        store4<FAST>(s.s0, e, n, nv);
        unsigned w = oct_pack4(nib, lane);
        myword = ((lane & 7u) == (unsigned)j) ? w : myword;
    }
    long long widx = (base >> 5) + (lane & 7u) * 8 + (lane >> 3);
    if ((lane & 7u) < 4u && (FAST || widx < (long long)((n + 31) >> 5))) words[widx] = myword;
    return a;
}

template <class Src>
__global__ __launch_bounds__(kBlock) void onebit_deferred_kernel(Src src, float* partial) {
    __shared__ float wsum[4];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    const float sp = *s.s1;  // last step's scale (0 before the first step)
    float a;
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) a = onebit_deferred_tile<true>(s, tile, sp);
    else a = onebit_deferred_tile<false>(s, tile, sp);
    a = wave_sum(a);
    if ((threadIdx.x & 63u) == 0) wsum[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) partial[s.tile0 + tile] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}

// out = v - d(v, scale): the residual the two-pass operator holds after the same steps.
template <bool FAST>
__device__ __forceinline__ void onebit_materialize_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const float sp = *s.s1;
    f4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = load4<FAST>(s.s0, base + j * 256 + lane * 4, n);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f4 r;
        r.x = v[j].x - (v[j].x >= 0.f ? sp : -sp);
        r.y = v[j].y - (v[j].y >= 0.f ? sp : -sp);
        r.z = v[j].z - (v[j].z >= 0.f ? sp : -sp);
        r.w = v[j].w - (v[j].w >= 0.f ? sp : -sp);
        store4<FAST>(s.out, base + j * 256 + lane * 4, n, r);
    }
}

template <class Src>
__global__ __launch_bounds__(kBlock) void onebit_materialize_kernel(Src src) {
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) onebit_materialize_tile<true>(s, tile);
    else onebit_materialize_tile<false>(s, tile);
}

template <bool FAST>
__device__ __forceinline__ void onebit_decode_tile(const Seg& s, unsigned tile) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const uint32_t* words = reinterpret_cast<const uint32_t*>(s.pay + kHeaderBytes);
    const float sc = *reinterpret_cast<const float*>(s.pay);
    const long long nwords = (n + 31) >> 5;
    unsigned nib[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long widx = (base >> 5) + j * 8 + (lane >> 3);
        uint32_t w = (FAST || widx < nwords) ? words[widx] : 0u;
        nib[j] = (w >> (4 * (lane & 7u))) & 0xfu;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f4 o;
        o.x = (nib[j] & 1u) ? sc : -sc;
        o.y = (nib[j] & 2u) ? sc : -sc;
        o.z = (nib[j] & 4u) ? sc : -sc;
        o.w = (nib[j] & 8u) ? sc : -sc;
        store4<FAST>(s.out, base + j * 256 + lane * 4, n, o);
    }
}

template <class Src>
__global__ __launch_bounds__(kBlock) void onebit_decode_kernel(Src src) {
    four_waves_per_simd();
    unsigned tile;
    const Seg s = src.get(tile, xcd_grouped(blockIdx.x, gridDim.x));
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) onebit_decode_tile<true>(s, tile);
    else onebit_decode_tile<false>(s, tile);
}

// =============================================================================
// TernGrad
// =============================================================================

__device__ __forceinline__ float absmax4(f4 v) {
    return fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
}

__device__ __forceinline__ unsigned tern_code(float g, float u, float s) {
    float t = u * s;
    return t < fabsf(g) ? (g < 0.f ? 2u : 1u) : 0u;
}

__device__ __forceinline__ unsigned tern_code4(f4 g, f4 u, float s) {
    return tern_code(g.x, u.x, s) | (tern_code(g.y, u.y, s) << 2) | (tern_code(g.z, u.z, s) << 4) |
           (tern_code(g.w, u.w, s) << 6);
}

// Bucket sizes 256, 512 and 1024 divide a wavefront's 1024 elements, so the
// bucket maximum is a wavefront reduction over values already in registers and
// the whole encode is a single pass.  BPW = buckets per wavefront tile.
template <bool FAST, int BPW, bool DRAW>
__device__ __forceinline__ void terngrad_encode_tile(const Seg& s, unsigned tile, unsigned key) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    if (base >= n) return;
    float* scales = reinterpret_cast<float*>(s.pay + kHeaderBytes);
    uint32_t* words = reinterpret_cast<uint32_t*>(s.pay + s.words_off);
    f4 g[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        u[j] = noise4<FAST, DRAW>(s.u, e, n, key);
    }
    float sc[4];
    constexpr int SPB = 4 / BPW;  // steps per bucket
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        float m = 0.f;
#pragma unroll
        for (int k = 0; k < SPB; ++k) m = fmaxf(m, absmax4(g[b * SPB + k]));
        m = wave_max(m);
#pragma unroll
        for (int k = 0; k < SPB; ++k) sc[b * SPB + k] = m;
        long long bidx = (base / (256 * SPB)) + b;
        if (lane == 0 && bidx * (256 * SPB) < n) scales[bidx] = m;
    }
    unsigned myword = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        unsigned byte = tern_code4(g[j], u[j], sc[j]);  // pad elements are 0: u*s < 0 is false
        unsigned w = quad_pack8(byte);
        myword = ((lane & 3u) == (unsigned)j) ? w : myword;
    }
    long long widx = (base >> 4) + (lane & 3u) * 16 + (lane >> 2);
    if (FAST || widx < (long long)((n + 15) >> 4)) words[widx] = myword;
}

// The scale array is padded to 16 bytes; the pad entries are written as zero.
__device__ __forceinline__ void terngrad_zero_scale_pad(const Seg& s, unsigned tile) {
    if (tile == 0 && threadIdx.x < 4) {
        unsigned long long nb = (s.n + s.bucket - 1) / s.bucket;
        unsigned long long i = nb + threadIdx.x;
        if (i < ((nb + 3) & ~3ull)) reinterpret_cast<float*>(s.pay + kHeaderBytes)[i] = 0.f;
    }
}

// DRAW: the noise is drawn in the kernel from `key` (the call's), the tensor's place in the
// launch's table and the element's index; otherwise it is read from the tensor the descriptor
// names and `key` is not used.
template <class Src, int BPW, bool DRAW>
__global__ __launch_bounds__(kBlock) void terngrad_encode_kernel(Src src, unsigned key) {
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = (uint32_t)s.n;
        h[1] = s.bucket;
        h[2] = 0;
        h[3] = 0;
    }
    terngrad_zero_scale_pad(s, tile);
    const unsigned tkey = DRAW ? tensor_key(key, s.id) : 0u;
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) terngrad_encode_tile<true, BPW, DRAW>(s, tile, tkey);
    else terngrad_encode_tile<false, BPW, DRAW>(s, tile, tkey);
}

// Any other bucket size up to a tile (4096): still a single pass.  A tile's elements lie in
// the buckets b_first .. b_last; the first of them may have begun in the tile before and the
// last may end in the tile behind, by less than a bucket each, so the workgroup also reads
// those two stretches of the gradient (nothing else of the neighbours) and so knows the
// maximum of every bucket its own elements need.  Maxima meet in LDS as integer keys (the
// bit pattern of |g| orders like |g|; values that are no number leave no key, as fmaxf
// passes them over).  A bucket's scale is written by the tile it begins in.
constexpr unsigned kAnyBucketMax = kTile;  // beyond a tile: the three-launch path, whose tiles lie in at most two buckets
constexpr unsigned kAnyBuckets = kTile + 2;  // bucket size 1: every element its own, plus none hanging over

__device__ __forceinline__ unsigned umax32(unsigned a, unsigned b) { return a > b ? a : b; }

__device__ __forceinline__ unsigned absmax_key(float x) {
    const unsigned k = __float_as_uint(x) & 0x7fffffffu;
    return k > 0x7f800000u ? 0u : k;  // NaN contributes nothing
}

template <bool FAST, bool DRAW>
__device__ __forceinline__ void terngrad_encode_any_tile(const Seg& s, unsigned tile, unsigned* mx, unsigned key) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const unsigned B = s.bucket;
    const long long t0 = (long long)tile * kTile, t1 = t0 + kTile < n ? t0 + kTile : n;
    const long long b_first = t0 / B, b_last = (t1 - 1) / B;
    const long long start = b_first * B;                                         // <= t0
    const long long end = (b_last + 1) * B < n ? (b_last + 1) * B : n;           // >= t1
    const unsigned nb = (unsigned)(b_last - b_first + 1);
    const unsigned head = (unsigned)(t0 - start);                                // elements of bucket b_first in front of the tile
    float* scales = reinterpret_cast<float*>(s.pay + kHeaderBytes);
    uint32_t* words = reinterpret_cast<uint32_t*>(s.pay + s.words_off);
    for (unsigned i = threadIdx.x; i < nb; i += kBlock) mx[i] = 0u;
    // the tile's own elements, requested before anything waits
    const long long base = t0 + wave * kWaveTile;
    f4 g[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        u[j] = noise4<FAST, DRAW>(s.u, e, n, key);
    }
    __syncthreads();
    // what hangs over from the neighbours: fewer than B elements on either side
    // (every wavefront folds its share before it touches the shared word)
    if (start < t0) {
        unsigned k = 0u;
        for (long long i = start + threadIdx.x; i < t0; i += kBlock) k = umax32(k, absmax_key(s.g[i]));
        k = wave_umax(k);
        if (lane == 0) atomicMax(&mx[0], k);
    }
    if (t1 < end) {
        unsigned k = 0u;
        for (long long i = t1 + threadIdx.x; i < end; i += kBlock) k = umax32(k, absmax_key(s.g[i]));
        k = wave_umax(k);
        if (lane == 0) atomicMax(&mx[nb - 1], k);
    }
    // local bucket and place inside it of each step's first element: one 32-bit division per step
    unsigned lb[4], rem[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned x = head + wave * kWaveTile + j * 256 + lane * 4;  // < 2 * kTile
        lb[j] = x / B;
        rem[j] = x - lb[j] * B;
        const float v[4] = {g[j].x, g[j].y, g[j].z, g[j].w};
        const long long e = base + j * 256 + lane * 4;
        const bool shared = rem[j] + 3u < B;  // the four elements share a bucket
        if (!shared) {
            unsigned b = lb[j], r = rem[j];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (e + k < n) atomicMax(&mx[b], absmax_key(v[k]));
                if (++r == B) { r = 0; ++b; }
            }
        }
        const bool mine = shared && e < n;  // elements beyond n were loaded as zero
        const unsigned key = mine ? absmax_key(absmax4(g[j])) : 0u;
        if (B >= 128u) {
            // the step's 256 elements lie in at most three buckets, lane 0's and the two after it: one
            // fold over the wavefront and one shared-memory maximum each, instead of one per lane
            const unsigned first = (unsigned)__builtin_amdgcn_readfirstlane((int)lb[j]);
#pragma unroll
            for (unsigned d = 0; d < 3u; ++d) {
                const bool here = mine && lb[j] == first + d;
                if (__ballot(here)) {  // wavefront-uniform
                    const unsigned m = wave_umax(here ? key : 0u);
                    if (lane == 0) atomicMax(&mx[first + d], m);
                }
            }
        } else if (mine) {
            atomicMax(&mx[lb[j]], key);
        }
    }
    __syncthreads();
    // scales of the buckets that begin in this tile
    for (unsigned i = (head ? 1u : 0u) + threadIdx.x; i < nb; i += kBlock) scales[b_first + i] = __uint_as_float(mx[i]);
    if (base >= n) return;
    unsigned myword = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        unsigned byte;
        if (rem[j] + 3u < B) {
            byte = tern_code4(g[j], u[j], __uint_as_float(mx[lb[j]]));  // pad elements are 0: u*s < 0 is false
        } else {
            const float gv[4] = {g[j].x, g[j].y, g[j].z, g[j].w}, uv[4] = {u[j].x, u[j].y, u[j].z, u[j].w};
            unsigned b = lb[j], r = rem[j];
            byte = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                // a pad element may index one bucket past the last: its code is 0 whatever the scale
                const float sc = b < nb ? __uint_as_float(mx[b]) : 0.f;
                byte |= tern_code(gv[k], uv[k], sc) << (2 * k);
                if (++r == B) { r = 0; ++b; }
            }
        }
        const unsigned w = quad_pack8(byte);
        myword = ((lane & 3u) == (unsigned)j) ? w : myword;
    }
    const long long widx = (base >> 4) + (lane & 3u) * 16 + (lane >> 2);
    if (FAST || widx < (long long)((n + 15) >> 4)) words[widx] = myword;
}

template <class Src, bool DRAW>
__global__ __launch_bounds__(kBlock) void terngrad_encode_any_kernel(Src src, unsigned key) {
    __shared__ unsigned mx[kAnyBuckets];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = (uint32_t)s.n;
        h[1] = s.bucket;
        h[2] = 0;
        h[3] = 0;
    }
    terngrad_zero_scale_pad(s, tile);
    if ((unsigned long long)tile * kTile >= s.n) return;  // an empty tensor has one tile and nothing in it
    const unsigned tkey = DRAW ? tensor_key(key, s.id) : 0u;
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) terngrad_encode_any_tile<true, DRAW>(s, tile, mx, tkey);
    else terngrad_encode_any_tile<false, DRAW>(s, tile, mx, tkey);
}

// Bucket sizes beyond a tile, up to the whole tensor: a tile then lies in at most two buckets, and a
// bucket's maximum is gathered over many tiles.  Three launches, no device-wide read-modify-write
// (which, a hundred thousand of them on the few cache lines of a short scale array, took a
// millisecond).  1: every tile folds the magnitudes of its two parts, as bit patterns (which order
// like the magnitudes; a maximum does not depend on the order it is taken in), into two words that
// it parks at the start of the payload's word area, words 2t and 2t + 1 for tile t: that area holds
// 256 words per tile and is written only by launch 3.  (A tensor of a single tile lies in one
// bucket and parks one word.)  2: the workgroup of the tile in which a bucket begins folds the
// parked words of the tiles the bucket covers and writes its scale; the first tile also writes the
// header.  3: a second pass over the gradient quantises with the finished scales.
struct BigBucketTile {
    unsigned b0;              // bucket of the tile's first element
    unsigned long long bnd;   // elements of the tile in front of the next bucket (kTile or more: none follows)
};
__device__ __forceinline__ BigBucketTile big_bucket_tile(unsigned tile, unsigned B) {
    BigBucketTile t;
    const unsigned t0 = tile * (unsigned)kTile;  // the element count fits 32 bits
    t.b0 = t0 / B;
    t.bnd = ((unsigned long long)t.b0 + 1ull) * B - t0;
    return t;
}

// maximum over the workgroup of what lane 0 of each wavefront holds; red: one word per wavefront
__device__ __forceinline__ unsigned block_umax(unsigned wave_value, unsigned* red) {
    if ((threadIdx.x & 63u) == 0u) red[threadIdx.x >> 6] = wave_value;
    __syncthreads();
    unsigned m = red[0];
#pragma unroll
    for (int w = 1; w < kBlock / 64; ++w) m = umax32(m, red[w]);
    __syncthreads();
    return m;
}

template <bool FAST>
__device__ __forceinline__ void terngrad_partial_big_tile(const Seg& s, unsigned tile, unsigned* red) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const BigBucketTile t = big_bucket_tile(tile, s.bucket);
    f4 g[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) g[j] = load4<FAST>(s.g, base + j * 256 + lane * 4, n);  // beyond n: zero, which adds nothing
    unsigned ka = 0u, kb = 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned li = wave * kWaveTile + j * 256 + lane * 4;
        const float v[4] = {g[j].x, g[j].y, g[j].z, g[j].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const unsigned key = absmax_key(v[k]);
            if (li + k < t.bnd) ka = umax32(ka, key);
            else kb = umax32(kb, key);
        }
    }
    ka = block_umax(wave_umax(ka), red);
    kb = block_umax(wave_umax(kb), red);
    if (threadIdx.x == 0) {
        uint32_t* parked = reinterpret_cast<uint32_t*>(s.pay + s.words_off);
        if (s.n > (unsigned long long)kTile) {
            parked[2ull * tile] = ka;
            parked[2ull * tile + 1ull] = kb;
        } else {
            parked[0] = ka;
        }
    }
}

template <class Src>
__global__ __launch_bounds__(kBlock) void terngrad_partial_big_kernel(Src src) {
    __shared__ unsigned red[kBlock / 64];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if ((unsigned long long)tile * kTile >= s.n) return;  // an empty tensor has one tile and nothing in it
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) terngrad_partial_big_tile<true>(s, tile, red);
    else terngrad_partial_big_tile<false>(s, tile, red);
}

template <class Src>
__global__ __launch_bounds__(kBlock) void terngrad_scale_big_kernel(Src src) {
    __shared__ unsigned red[kBlock / 64];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    if (tile == 0 && threadIdx.x == 0) {
        uint32_t* h = reinterpret_cast<uint32_t*>(s.pay);
        h[0] = (uint32_t)s.n;
        h[1] = s.bucket;
        h[2] = 0;
        h[3] = 0;
    }
    terngrad_zero_scale_pad(s, tile);
    const unsigned long long B = s.bucket, lo = (unsigned long long)tile * kTile;
    const unsigned long long hi = lo + kTile < s.n ? lo + kTile : s.n;
    const unsigned long long first = (lo + B - 1) / B;  // the bucket that begins at or after lo
    const unsigned long long e0 = first * B;
    if (e0 >= hi) return;  // no bucket begins in this tile
    const unsigned long long e1 = e0 + B < s.n ? e0 + B : s.n;
    const unsigned long long last_tile = (e1 - 1) / kTile;
    const uint32_t* parked = reinterpret_cast<const uint32_t*>(s.pay + s.words_off);
    unsigned k = 0u;
    if (s.n > (unsigned long long)kTile) {
        // this tile holds the bucket's beginning: in its second part unless the bucket begins with the
        // tile; every further tile the bucket reaches holds it in its first part
        for (unsigned long long t = tile + threadIdx.x; t <= last_tile; t += kBlock)
            k = umax32(k, parked[2ull * t + ((t == tile && e0 != lo) ? 1ull : 0ull)]);
    } else if (threadIdx.x == 0) {
        k = parked[0];
    }
    k = block_umax(wave_umax(k), red);
    if (threadIdx.x == 0) reinterpret_cast<float*>(s.pay + kHeaderBytes)[first] = __uint_as_float(k);
}

template <bool FAST, bool DRAW>
__device__ __forceinline__ void terngrad_quant_big_tile(const Seg& s, unsigned tile, unsigned key) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    if (base >= n) return;
    const BigBucketTile t = big_bucket_tile(tile, s.bucket);
    const float* scales = reinterpret_cast<const float*>(s.pay + kHeaderBytes);
    uint32_t* words = reinterpret_cast<uint32_t*>(s.pay + s.words_off);
    f4 g[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256 + lane * 4;
        g[j] = load4<FAST>(s.g, e, n);
        u[j] = noise4<FAST, DRAW>(s.u, e, n, key);
    }
    const float sa = scales[t.b0];
    const float sb = (unsigned long long)tile * kTile + t.bnd < (unsigned long long)n && t.bnd < (unsigned long long)kTile ? scales[t.b0 + 1u] : 0.f;
    unsigned myword = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned li = wave * kWaveTile + j * 256 + lane * 4;
        unsigned byte;
        if (li + 3u < t.bnd) {
            byte = tern_code4(g[j], u[j], sa);  // pad elements are 0: u*s < 0 is false
        } else if (li >= t.bnd) {
            byte = tern_code4(g[j], u[j], sb);
        } else {
            const float gv[4] = {g[j].x, g[j].y, g[j].z, g[j].w}, uv[4] = {u[j].x, u[j].y, u[j].z, u[j].w};
            byte = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) byte |= tern_code(gv[k], uv[k], li + k < t.bnd ? sa : sb) << (2 * k);
        }
        const unsigned w = quad_pack8(byte);
        myword = ((lane & 3u) == (unsigned)j) ? w : myword;
    }
    const long long widx = (base >> 4) + (lane & 3u) * 16 + (lane >> 2);
    if (FAST || widx < (long long)((n + 15) >> 4)) words[widx] = myword;
}

template <class Src, bool DRAW>
__global__ __launch_bounds__(kBlock) void terngrad_quant_big_kernel(Src src, unsigned key) {
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    const unsigned tkey = DRAW ? tensor_key(key, s.id) : 0u;
    if (s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n) terngrad_quant_big_tile<true, DRAW>(s, tile, tkey);
    else terngrad_quant_big_tile<false, DRAW>(s, tile, tkey);
}

// Decode.  The bucket size is in the payload header, and with it the place of the
// packed words behind the scale array; a header that does not fit the buffer
// decodes to zeros.  A launch whose host side knows the bucket size (descriptor
// field `bucket`, with `words_off` already checked against the buffer) starts its
// loads from that and only compares the header with it afterwards, so the header
// is not on the path to the first load; on a mismatch the header decides.
// BUCKET256 means the bucket size is a multiple of 256, so one step of a
// wavefront (256 aligned elements) lies inside one bucket.
template <bool FAST, bool BUCKET256>
__device__ __forceinline__ void terngrad_decode_tile(const Seg& s, unsigned tile, long long B,
                                                     const uint32_t* words, bool verify) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    if (base >= n) return;
    const float* scales = reinterpret_cast<const float*>(s.pay + kHeaderBytes);
    const long long nwords = words ? (n + 15) >> 4 : 0;
    const uint32_t header_bucket = verify ? reinterpret_cast<const uint32_t*>(s.pay)[1] : 0u;
    unsigned b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long widx = (base >> 4) + j * 16 + (lane >> 2);
        uint32_t w = widx < nwords ? words[widx] : 0u;
        b[j] = (w >> (8 * (lane & 3u))) & 0xffu;
    }
    float sc4[4] = {0.f, 0.f, 0.f, 0.f};
    // the tile's first element: its bucket and its place in it (not needed when every step lies in one bucket)
    const long long tile0 = (long long)tile * kTile;
    const long long tq0 = BUCKET256 ? 0 : tile0 / B;
    const unsigned long long tr0 = BUCKET256 ? 0ull : (unsigned long long)(tile0 - tq0 * B);
    if (BUCKET256) {
        // one division per wavefront: the four steps start 0, 256, 512, 768 elements
        // further on and B >= 256, so each step is at most three buckets ahead
        const long long q0 = base / B, r0 = base - q0 * B;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long long x = r0 + j * 256;
            const long long q = q0 + (x >= B) + (x >= 2 * B) + (x >= 3 * B);
            sc4[j] = (base + j * 256 < n && words) ? scales[q] : 0.f;
        }
    }
    if (verify && header_bucket != (uint32_t)B) return;  // the caller falls back to the header
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        f4 o;
        if (BUCKET256) {
            o = expand2(b[j], sc4[j]);
        } else {
            // bucket of the lane's first element from the tile's; the other three follow by counting
            const BucketPos bp = bucket_pos(tq0, tr0, (unsigned)(wave * kWaveTile + j * 256 + lane * 4), (unsigned long long)B);
            long long q = bp.q;
            unsigned long long r = bp.r;
            float ov[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const unsigned c = (b[j] >> (2 * k)) & 3u;
                ov[k] = (e + k < n && c) ? code_value(c, scales[q]) : 0.f;
                if (++r == (unsigned long long)B) { r = 0; ++q; }
            }
            o.x = ov[0]; o.y = ov[1]; o.z = ov[2]; o.w = ov[3];
        }
        store4<FAST>(s.out, e, n, o);
    }
}

// Where the packed words of a TernGrad payload start, or NULL when the header's
// bucket size does not fit the buffer.
__device__ __forceinline__ const uint32_t* terngrad_words(const uint8_t* pay, unsigned long long pay_bytes,
                                                           unsigned long long n, long long& B) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(pay);
    B = h[1];
    if (B < 1) { B = 1; return nullptr; }
    unsigned long long nb = (n + B - 1) / B;
    unsigned long long off = kHeaderBytes + ((4 * nb + 15) & ~15ull);
    if (off + 4 * ((n + 15) >> 4) > pay_bytes) return nullptr;
    return reinterpret_cast<const uint32_t*>(pay + off);
}

// ANY_BUCKET: the launch may meet bucket sizes that are no multiple of 256 on full tiles and
// carries the vector-store path for them.  A launch whose descriptors all name a multiple of
// 256 runs the kernel without it, which is 5 % faster on its own path for being smaller (the
// decode of the VGG19 set 80 against 84 us); a payload that names another size after all is
// still decoded, element by element.
template <class Src, bool ANY_BUCKET>
__global__ __launch_bounds__(kBlock) void terngrad_decode_kernel(Src src) {
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    const bool fast = s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n;
    if (s.bucket && (s.bucket & 255u) == 0) {
        const uint32_t* words = reinterpret_cast<const uint32_t*>(s.pay + s.words_off);
        if (fast) terngrad_decode_tile<true, true>(s, tile, s.bucket, words, true);
        else terngrad_decode_tile<false, true>(s, tile, s.bucket, words, true);
        if (reinterpret_cast<const uint32_t*>(s.pay)[1] == s.bucket) return;
    }
    long long B;
    const uint32_t* words = terngrad_words(s.pay, s.pay_bytes, s.n, B);
    const bool b256 = (B & 255) == 0;
    if (fast && b256) terngrad_decode_tile<true, true>(s, tile, B, words, false);
    else if (b256) terngrad_decode_tile<false, true>(s, tile, B, words, false);
    else if (ANY_BUCKET && fast) terngrad_decode_tile<true, false>(s, tile, B, words, false);
    else terngrad_decode_tile<false, false>(s, tile, B, words, false);
}

// =============================================================================
// launchers
// =============================================================================

#define HP_LAUNCH(KERNEL, LDS, L, st, ...)                                                        \
    do {                                                                                      \
        if ((L).ntiles == 0) return hipSuccess;                                               \
        if ((L).single) {                                                                     \
            SingleSrc src{(L).seg};                                                           \
            hipLaunchKernelGGL((KERNEL<SingleSrc>), dim3((L).ntiles), dim3(kBlock), LDS, st, src, \
                               ##__VA_ARGS__);                                                \
        } else {                                                                              \
            BatchSrc src{(L).dsegs, (L).dmap};                                                \
            hipLaunchKernelGGL((KERNEL<BatchSrc>), dim3((L).ntiles), dim3(kBlock), LDS, st, src, \
                               ##__VA_ARGS__);                                                \
        }                                                                                     \
        return hipGetLastError();                                                             \
    } while (0)

// The TBQ and onebit decoders limit themselves to four wavefronts per SIMD by the registers
// they claim, at every size (92 -> 80 us on the VGG19 set behind their encoders; at 1.5 and
// 3 G elements the same as unlimited or 10 % better).  The TernGrad table decode does better
// with five workgroups per CU, set with idle LDS, and only while the payload it reads
// (per_tile bytes for every 4096 elements) still fits the 256 MiB memory-side cache, where
// the encoder left it: beyond that such a cap costs 15 %.
static unsigned decode_cap(const Launch& L, unsigned per_tile) {
    return (unsigned long long)L.ntiles * per_tile <= (192ull << 20) ? kLdsFor5 : 0u;
}

hipError_t launch_tbq_encode(const Launch& L, hipStream_t st) { HP_LAUNCH(tbq_encode_kernel, 0u, L, st); }
hipError_t launch_tbq_decode(const Launch& L, hipStream_t st) { HP_LAUNCH(tbq_decode_kernel, 0u, L, st); }
hipError_t launch_onebit_decode(const Launch& L, hipStream_t st) {
    HP_LAUNCH(onebit_decode_kernel, 0u, L, st);
}
// A single-tensor call learns the bucket size from the header on the device, a chain of
// dependent loads that wants full occupancy; a table launch carries it in the descriptors.
hipError_t launch_terngrad_decode(const Launch& L, unsigned bucket, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {  // the bucket size is in the payload's header, on the device
        SingleSrc src{L.seg};
        hipLaunchKernelGGL((terngrad_decode_kernel<SingleSrc, true>), dim3(L.ntiles), dim3(kBlock), 0u, st, src);
    } else {
        BatchSrc src{L.dsegs, L.dmap};
        const unsigned lds = decode_cap(L, kTile / 4);
        if (bucket && (bucket & 255u) == 0u)
            hipLaunchKernelGGL((terngrad_decode_kernel<BatchSrc, false>), dim3(L.ntiles), dim3(kBlock), lds, st, src);
        else
            hipLaunchKernelGGL((terngrad_decode_kernel<BatchSrc, true>), dim3(L.ntiles), dim3(kBlock), lds, st, src);
    }
    return hipGetLastError();
}

static hipError_t onebit_abs(const Launch& L, float* partial, hipStream_t st) {
    HP_LAUNCH(onebit_abs_kernel, 0u, L, st, partial);
}
static hipError_t onebit_quant(const Launch& L, hipStream_t st) { HP_LAUNCH(onebit_quant_kernel, 0u, L, st); }

static hipError_t onebit_scale(const Launch& L, const float* partial, hipStream_t st) {
    if (L.single) {
        SingleSegSrc src{L.seg};
        hipLaunchKernelGGL((onebit_scale_kernel<SingleSegSrc>), dim3(1), dim3(kScaleBlock), 0, st, src, partial);
    } else {
        BatchSegSrc src{L.dsegs};
        hipLaunchKernelGGL((onebit_scale_kernel<BatchSegSrc>), dim3(L.nsegs), dim3(kScaleBlock), 0, st, src, partial);
    }
    return hipGetLastError();
}

// partial: one float per tile of the launch.  phase < 0 runs the whole sequence,
// 0 / 1 / 2 run only the magnitude sum / the scale / the quantisation launch.
hipError_t launch_onebit_encode(const Launch& L, float* partial, int phase, hipStream_t st) {
    hipError_t e;
    if (L.ntiles && (phase < 0 || phase == 0)) {
        if ((e = onebit_abs(L, partial, st)) != hipSuccess) return e;
    }
    if (phase < 0 || phase == 1) {
        if ((e = onebit_scale(L, partial, st)) != hipSuccess) return e;
    }
    if (L.ntiles && (phase < 0 || phase == 2)) {
        if ((e = onebit_quant(L, st)) != hipSuccess) return e;
    }
    return hipSuccess;
}

static hipError_t onebit_deferred(const Launch& L, float* partial, hipStream_t st) {
    HP_LAUNCH(onebit_deferred_kernel, kLdsFor5, L, st, partial);
}

// phase < 0: both launches; 0: the fused pass; 1: the scale.
hipError_t launch_onebit_encode_deferred(const Launch& L, float* partial, int phase, hipStream_t st) {
    hipError_t e;
    if (L.ntiles && (phase < 0 || phase == 0)) {
        if ((e = onebit_deferred(L, partial, st)) != hipSuccess) return e;
    }
    if (phase < 0 || phase == 1) {
        if ((e = onebit_scale(L, partial, st)) != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_onebit_materialize(const Launch& L, hipStream_t st) { HP_LAUNCH(onebit_materialize_kernel, kLdsFor5, L, st); }

template <class Src, bool DRAW>
static hipError_t terngrad_encode_src(const Src& src, unsigned ntiles, unsigned bucket, unsigned key, hipStream_t st) {
    const dim3 g(ntiles), b(kBlock);
    if (bucket == 256) hipLaunchKernelGGL((terngrad_encode_kernel<Src, 4, DRAW>), g, b, kLdsFor5, st, src, key);
    else if (bucket == 512) hipLaunchKernelGGL((terngrad_encode_kernel<Src, 2, DRAW>), g, b, kLdsFor5, st, src, key);
    else if (bucket == 1024) hipLaunchKernelGGL((terngrad_encode_kernel<Src, 1, DRAW>), g, b, kLdsFor5, st, src, key);
    else if (bucket <= kAnyBucketMax) hipLaunchKernelGGL((terngrad_encode_any_kernel<Src, DRAW>), g, b, 0, st, src, key);
    else {
        hipLaunchKernelGGL((terngrad_partial_big_kernel<Src>), g, b, 0, st, src);
        hipLaunchKernelGGL((terngrad_scale_big_kernel<Src>), g, b, 0, st, src);
        hipLaunchKernelGGL((terngrad_quant_big_kernel<Src, DRAW>), g, b, kLdsFor5, st, src, key);
    }
    return hipGetLastError();
}

// All tensors of one launch share the bucket size.  draw: the noise is drawn in the kernels from
// `key` (uniform_draw.h) instead of being read from the tensors the descriptors name.
hipError_t launch_terngrad_encode(const Launch& L, unsigned bucket, bool draw, unsigned key, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {
        if (draw) return terngrad_encode_src<SingleSrc, true>(SingleSrc{L.seg}, L.ntiles, bucket, key, st);
        return terngrad_encode_src<SingleSrc, false>(SingleSrc{L.seg}, L.ntiles, bucket, 0u, st);
    }
    if (draw) return terngrad_encode_src<BatchSrc, true>(BatchSrc{L.dsegs, L.dmap}, L.ntiles, bucket, key, st);
    return terngrad_encode_src<BatchSrc, false>(BatchSrc{L.dsegs, L.dmap}, L.ntiles, bucket, 0u, st);
}

// out[i] = the draw an encoder makes for element i of the tensor with this key.
__global__ __launch_bounds__(kBlock) void uniform_fill_kernel(float* out, unsigned long long n, unsigned key, unsigned aligned) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long base = (long long)blockIdx.x * kTile + wave * kWaveTile;
    const bool fast = aligned && (unsigned long long)(blockIdx.x + 1) * kTile <= n;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long long e = base + j * 256 + lane * 4;
        const f4 v = noise4<true, true>(nullptr, e, (long long)n, key);
        if (fast) st4(out + e, v);
        else st4_guard(out, e, (long long)n, v);
    }
}

hipError_t launch_uniform_fill(float* out, unsigned long long n, unsigned key, hipStream_t st) {
    if (n == 0) return hipSuccess;
    const unsigned ntiles = (unsigned)((n + kTile - 1) / kTile);
    hipLaunchKernelGGL(uniform_fill_kernel, dim3(ntiles), dim3(kBlock), 0, st, out, n, key,
                       (unsigned)((reinterpret_cast<uintptr_t>(out) & 3u) == 0));
    return hipGetLastError();
}

}  // namespace hp
