// The in-tree CompLL operator (min/max b-bit stochastic quantiser, 10-byte header)
// for gfx950, as its DSL source states it
// (/root/reference/src/CompLL/GCGen/pse/TernGradEncode.pse:22-33,
//  /root/reference/src/CompLL/GCGen/pse/TernGradDecode.pse:1-14):
//   encode: max/min reduction, gap = (max-min)/(2^b-1), code_i = floor((g_i-min)/gap + u_i),
//           payload [b:u8][tail:u8][min:f32][max:f32] then codes, code i at bit
//           (i mod 8/b)*b of byte floor(i*b/8) - the placement the decoder reads
//           (TernGradDecode_body.h:44);
//   decode: count = (8*csz - 80)/b - tail elements, out_i = code_i*gap + min
//           (TernGradDecode_body.h:65-72).
// Three launches for encode (per-tile min/max, per-tensor header, quantise), one
// for decode; same tile / wavefront / lane decomposition as the other operators.
#include "common.h"
#include "launch.h"

namespace hp {

constexpr float kMaxInit = -99999.0f, kMinInit = 99999.0f;  // the DSL's reduce() initial values

__device__ __forceinline__ float load_f32_bytes(const uint8_t* p) {
    return __uint_as_float((unsigned)p[0] | ((unsigned)p[1] << 8) | ((unsigned)p[2] << 16) | ((unsigned)p[3] << 24));
}
__device__ __forceinline__ void store_f32_bytes(uint8_t* p, float x) {
    unsigned u = __float_as_uint(x);
    p[0] = (uint8_t)u;
    p[1] = (uint8_t)(u >> 8);
    p[2] = (uint8_t)(u >> 16);
    p[3] = (uint8_t)(u >> 24);
}

template <class Src>
__global__ __launch_bounds__(kBlock) void compll_minmax_kernel(Src src, float* partial) {
    four_waves_per_simd();  // a read-only sweep: 61 -> 57 us on 102.8 M elements
    __shared__ float wmx[4], wmn[4];
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const bool fast = s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n;
    const bool keep = fast && cache_tail(blockIdx.x, gridDim.x, 1);  // left on the chip for the code pass
    float mx = kMaxInit, mn = kMinInit;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        f4 v = keep ? ld4_keep(s.g + e) : (fast ? ld4(s.g + e) : ld4_guard(s.g, e, n));
        unsigned ok = fast ? 0xfu : valid4(e, n);
        if (ok & 1u) { mx = v.x > mx ? v.x : mx; mn = v.x < mn ? v.x : mn; }
        if (ok & 2u) { mx = v.y > mx ? v.y : mx; mn = v.y < mn ? v.y : mn; }
        if (ok & 4u) { mx = v.z > mx ? v.z : mx; mn = v.z < mn ? v.z : mn; }
        if (ok & 8u) { mx = v.w > mx ? v.w : mx; mn = v.w < mn ? v.w : mn; }
    }
    mx = wave_max(mx);
    mn = -wave_max(-mn);
    if (lane == 0) {
        wmx[wave] = mx;
        wmn[wave] = mn;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        partial[2 * (s.tile0 + tile)] = fmaxf(fmaxf(wmx[0], wmx[1]), fmaxf(wmx[2], wmx[3]));
        partial[2 * (s.tile0 + tile) + 1] = fminf(fminf(wmn[0], wmn[1]), fminf(wmn[2], wmn[3]));
    }
}

constexpr int kHeaderBlock = 1024;

template <class SegSrc>
__global__ __launch_bounds__(kHeaderBlock) void compll_header_kernel(SegSrc src, const float* partial) {
    __shared__ float smx[kHeaderBlock / 64], smn[kHeaderBlock / 64];
    const Seg s = src.at(blockIdx.x);
    const unsigned nt = s.ntiles;
    const float2* p2 = reinterpret_cast<const float2*>(partial) + s.tile0;
    float mx = kMaxInit, mn = kMinInit;
    unsigned t = threadIdx.x;
    for (; t + 3 * kHeaderBlock < nt; t += 4 * kHeaderBlock) {  // four loads in flight per lane
        float2 v0 = p2[t], v1 = p2[t + kHeaderBlock], v2 = p2[t + 2 * kHeaderBlock], v3 = p2[t + 3 * kHeaderBlock];
        mx = fmaxf(fmaxf(mx, v0.x), fmaxf(fmaxf(v1.x, v2.x), v3.x));
        mn = fminf(fminf(mn, v0.y), fminf(fminf(v1.y, v2.y), v3.y));
    }
    for (; t < nt; t += kHeaderBlock) {
        float2 v = p2[t];
        mx = fmaxf(mx, v.x);
        mn = fminf(mn, v.y);
    }
    mx = wave_max(mx);
    mn = -wave_max(-mn);
    if ((threadIdx.x & 63u) == 0) {
        smx[threadIdx.x >> 6] = mx;
        smn[threadIdx.x >> 6] = mn;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kHeaderBlock / 64; ++w) {
            mx = fmaxf(mx, smx[w]);
            mn = fminf(mn, smn[w]);
        }
        const unsigned b = s.bucket;  // bit width
        s.pay[0] = (uint8_t)b;
        s.pay[1] = (uint8_t)(s.n % (1ull << b));  // the DSL's tail = size % (1 << bitwidth)
        store_f32_bytes(s.pay + 2, mn);
        store_f32_bytes(s.pay + 6, mx);
    }
}

__device__ __forceinline__ unsigned compll_code(float g, float u, float mn, float gap, float top) {
    if (!(gap > 0.f)) return 0u;
    float f = floorf((g - mn) / gap + u);
    return !(f > 0.f) ? 0u : (f >= top ? (unsigned)top : (unsigned)f);  // NaN -> 0
}

// DRAW: the noise is drawn in the kernel from `key` and the element's index (uniform_draw.h);
// otherwise it is read from the tensor the descriptor names.
template <class Src, int B, bool DRAW>
__global__ __launch_bounds__(kBlock) void compll_quant_kernel(Src src, unsigned key) {
    unsigned tile;
    const Seg s = src.get(tile, xcd_reversed(blockIdx.x, gridDim.x));  // begins where the min/max pass ended
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const long long n = (long long)s.n;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const bool fast = s.aligned && (unsigned long long)(tile + 1) * kTile <= s.n;
    const float mn = load_f32_bytes(s.pay + 2), mx = load_f32_bytes(s.pay + 6);
    constexpr float top = (float)((1 << B) - 1);
    const float gap = (mx - mn) / top;
    uint8_t* Q = s.pay + 10;
    const long long nbytes = (n * B + 7) / 8;
    const unsigned tkey = DRAW ? tensor_key(key, s.id) : 0u;
    f4 g[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        g[j] = fast ? ld4(s.g + e) : ld4_guard(s.g, e, n);
        u[j] = DRAW ? noise4<true, true>(nullptr, e, n, tkey) : (fast ? ld4(s.u + e) : ld4_guard(s.u, e, n));  // codes beyond n are masked below
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        unsigned ok = fast ? 0xfu : valid4(e, n);
        unsigned c0 = (ok & 1u) ? compll_code(g[j].x, u[j].x, mn, gap, top) : 0u;
        unsigned c1 = (ok & 2u) ? compll_code(g[j].y, u[j].y, mn, gap, top) : 0u;
        unsigned c2 = (ok & 4u) ? compll_code(g[j].z, u[j].z, mn, gap, top) : 0u;
        unsigned c3 = (ok & 8u) ? compll_code(g[j].w, u[j].w, mn, gap, top) : 0u;
        if (B == 8) {
            if (ok & 1u) Q[e] = (uint8_t)c0;
            if (ok & 2u) Q[e + 1] = (uint8_t)c1;
            if (ok & 4u) Q[e + 2] = (uint8_t)c2;
            if (ok & 8u) Q[e + 3] = (uint8_t)c3;
        } else if (B == 4) {
            if (ok & 1u) Q[e / 2] = (uint8_t)(c0 | (c1 << 4));
            if (ok & 4u) Q[e / 2 + 1] = (uint8_t)(c2 | (c3 << 4));
        } else if (B == 2) {
            if (ok & 1u) Q[e / 4] = (uint8_t)(c0 | (c1 << 2) | (c2 << 4) | (c3 << 6));
        } else {  // B == 1: two neighbouring lanes share a byte
            unsigned nib = c0 | (c1 << 1) | (c2 << 2) | (c3 << 3);
            unsigned other = (unsigned)__builtin_amdgcn_update_dpp(0, (int)nib, 0xB1, 0xf, 0xf, false);  // quad_perm [1,0,3,2]
            if ((lane & 1u) == 0 && e / 8 < nbytes && (ok & 1u)) Q[e / 8] = (uint8_t)(nib | (other << 4));
        }
    }
}

// Decode follows the reference literally: the element count comes from the payload
// length and the tail byte; at most n (the caller's buffer) elements are written.
template <class Src>
__global__ __launch_bounds__(kBlock) void compll_decode_kernel(Src src) {
    unsigned tile;
    const Seg s = src.get(tile, blockIdx.x);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned b = s.pay[0], tail = s.pay[1];
    if (b != 1 && b != 2 && b != 4 && b != 8) return;
    const float mn = load_f32_bytes(s.pay + 2), mx = load_f32_bytes(s.pay + 6);
    const float gap = (mx - mn) / (float)((1u << b) - 1u);
    long long count = (8 * (long long)s.pay_bytes - 80) / (long long)b - (long long)tail;
    if (count > (long long)s.n) count = (long long)s.n;
    const uint8_t* Q = s.pay + 10;
    const long long base = (long long)tile * kTile + wave * kWaveTile;
    const unsigned mask = (1u << b) - 1u;
    const bool vec = s.aligned != 0;
    unsigned bits[4];  // the 4*b code bits of this lane's four elements, per step
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        bits[j] = 0;
        if (e < count) {  // e is a multiple of 4, so its codes start on a byte (b >= 2) or nibble (b == 1) boundary
            const long long byte0 = e * b / 8;
            if (b == 8) {
                bits[j] = Q[byte0];
                if (e + 1 < count) bits[j] |= (unsigned)Q[byte0 + 1] << 8;
                if (e + 2 < count) bits[j] |= (unsigned)Q[byte0 + 2] << 16;
                if (e + 3 < count) bits[j] |= (unsigned)Q[byte0 + 3] << 24;
            } else if (b == 4) {
                bits[j] = Q[byte0];
                if (e + 2 < count) bits[j] |= (unsigned)Q[byte0 + 1] << 8;
            } else if (b == 2) {
                bits[j] = Q[byte0];
            } else {
                bits[j] = (Q[byte0] >> ((e & 4) ? 4 : 0)) & 0xfu;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long long e = base + j * 256 + lane * 4;
        if (e >= count) continue;
        f4 o;
        o.x = __fadd_rn(__fmul_rn((float)(bits[j] & mask), gap), mn);
        o.y = __fadd_rn(__fmul_rn((float)((bits[j] >> b) & mask), gap), mn);
        o.z = __fadd_rn(__fmul_rn((float)((bits[j] >> (2 * b)) & mask), gap), mn);
        o.w = __fadd_rn(__fmul_rn((float)((bits[j] >> (3 * b)) & mask), gap), mn);
        if (vec && e + 3 < count) st4(s.out + e, o);
        else st4_guard(s.out, e, count, o);
    }
}

template <class Src, class SegSrcT, bool DRAW>
static hipError_t compll_encode_src(const Src& src, const SegSrcT& ssrc, unsigned ntiles, unsigned nsegs, int b,
                                    float* partial, unsigned key, hipStream_t st) {
    hipLaunchKernelGGL((compll_minmax_kernel<Src>), dim3(ntiles), dim3(kBlock), 0, st, src, partial);
    hipLaunchKernelGGL((compll_header_kernel<SegSrcT>), dim3(nsegs), dim3(kHeaderBlock), 0, st, ssrc, partial);
    if (b == 1) hipLaunchKernelGGL((compll_quant_kernel<Src, 1, DRAW>), dim3(ntiles), dim3(kBlock), 0, st, src, key);
    else if (b == 2) hipLaunchKernelGGL((compll_quant_kernel<Src, 2, DRAW>), dim3(ntiles), dim3(kBlock), 0, st, src, key);
    else if (b == 4) hipLaunchKernelGGL((compll_quant_kernel<Src, 4, DRAW>), dim3(ntiles), dim3(kBlock), 0, st, src, key);
    else hipLaunchKernelGGL((compll_quant_kernel<Src, 8, DRAW>), dim3(ntiles), dim3(kBlock), 0, st, src, key);
    return hipGetLastError();
}

// partial: two floats per tile.  draw: the noise comes from `key`, not from the descriptors' tensors.
hipError_t launch_compll_encode(const Launch& L, int bitwidth, float* partial, bool draw, unsigned key, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {
        if (draw) return compll_encode_src<SingleSrc, SingleSegSrc, true>(SingleSrc{L.seg}, SingleSegSrc{L.seg}, L.ntiles, 1, bitwidth, partial, key, st);
        return compll_encode_src<SingleSrc, SingleSegSrc, false>(SingleSrc{L.seg}, SingleSegSrc{L.seg}, L.ntiles, 1, bitwidth, partial, 0u, st);
    }
    if (draw) return compll_encode_src<BatchSrc, BatchSegSrc, true>(BatchSrc{L.dsegs, L.dmap}, BatchSegSrc{L.dsegs}, L.ntiles, L.nsegs, bitwidth, partial, key, st);
    return compll_encode_src<BatchSrc, BatchSegSrc, false>(BatchSrc{L.dsegs, L.dmap}, BatchSegSrc{L.dsegs}, L.ntiles, L.nsegs, bitwidth, partial, 0u, st);
}

hipError_t launch_compll_decode(const Launch& L, hipStream_t st) {
    if (L.ntiles == 0) return hipSuccess;
    if (L.single) {
        SingleSrc src{L.seg};
        hipLaunchKernelGGL((compll_decode_kernel<SingleSrc>), dim3(L.ntiles), dim3(kBlock), 0, st, src);
    } else {
        BatchSrc src{L.dsegs, L.dmap};
        hipLaunchKernelGGL((compll_decode_kernel<BatchSrc>), dim3(L.ntiles), dim3(kBlock), 0, st, src);
    }
    return hipGetLastError();
}

}  // namespace hp
