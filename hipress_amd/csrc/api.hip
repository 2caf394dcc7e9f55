// C ABI of libhipress_amd.so: argument validation, tensor descriptors, batched
// launch objects.  Kernels live in dense.hip, sparse.hip and merge.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/hipress_amd.h"
#include "common.h"
#include "launch.h"

using namespace hp;

namespace {

constexpr int64_t kSampleTile = 4096;    // sample keys per workgroup of the select passes

inline bool mis(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }
// The 16-byte vector path of the kernels needs dword alignment only (common.h: f4u), which
// every fp32 pointer has once it has passed the 4-byte check.
inline bool vec_ok(const void* p) { return !mis(p, 4); }
inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline unsigned tiles_of(int64_t n) { return n <= 0 ? 1u : (unsigned)((n + kTile - 1) / kTile); }
inline bool bad_n(int64_t n) { return n < 0 || n > HIPRESS_MAX_N; }
// sparse payloads carry int32 indices
inline bool bad_sparse_n(int64_t n) { return n < 0 || n > HIPRESS_SPARSE_MAX_N; }
inline bool is_sparse(int alg) { return alg == HIPRESS_DGC || alg == HIPRESS_GRADDROP; }

inline int64_t words_bytes(int64_t n, int bits) {
    int per = 32 / bits;
    return 4 * ((n + per - 1) / per);
}

inline int64_t tg_scale_bytes(int64_t n, int64_t bucket) { return round_up(4 * ((n + bucket - 1) / bucket), 16); }

struct SparsePlan {
    int64_t cap, stride, ns, ks;
};

inline SparsePlan sparse_plan(int64_t n, double ratio) {
    SparsePlan p;
    int64_t want = (int64_t)std::ceil(4.0 * ratio * (double)n);
    if (want > n) want = n;
    if (want < 64) want = 64;
    p.cap = round_up(want, 64);
    p.stride = n >= kSampleFrom ? kSampleStride : 1;
    p.ns = n / p.stride;
    p.ks = (int64_t)std::ceil(ratio * (double)p.ns);
    if (p.ks < 1) p.ks = 1;
    if (p.ks > p.ns) p.ks = p.ns;
    return p;
}

inline bool bad_ratio(double r) { return !(r > 0.0 && r <= 1.0); }

// Workspace of a sparse launch: six uint32 arrays, each starting on a 256-byte boundary.
struct SparseWsLayout {
    int64_t sample_off, grec_off, counts_off, thr_off, hist_off, ctl_off, bytes;
};

inline SparseWsLayout sparse_ws_layout(int64_t total_ns, int64_t total_tiles, int64_t nsegs) {
    SparseWsLayout l;
    int64_t off = 0;
    l.sample_off = off;
    off += round_up(4 * total_ns, 256);
    l.grec_off = off;
    off += round_up(8 * 64 * total_tiles, 256);
    l.counts_off = off;
    off += round_up(4 * 2 * total_tiles, 256);
    l.thr_off = off;
    off += round_up(4 * 2 * nsegs, 256);
    l.hist_off = off;
    off += round_up(4 * (int64_t)kSelHistWords * nsegs, 256);
    l.ctl_off = off;
    off += round_up(4 * 8 * nsegs, 256);
    l.bytes = off;
    return l;
}

inline SparseWs sparse_ws_at(void* base, const SparseWsLayout& l) {
    uint8_t* b = static_cast<uint8_t*>(base);
    SparseWs w;
    w.sample = reinterpret_cast<uint32_t*>(b + l.sample_off);
    w.grec = reinterpret_cast<uint2*>(b + l.grec_off);
    w.counts = reinterpret_cast<uint32_t*>(b + l.counts_off);
    w.thr = reinterpret_cast<uint32_t*>(b + l.thr_off);
    w.hist = reinterpret_cast<uint32_t*>(b + l.hist_off);
    w.ctl = reinterpret_cast<uint32_t*>(b + l.ctl_off);
    return w;
}

// Index part of a sparse merge workspace: per tile a head and one run record per peer.
inline int64_t merge_index_bytes(int64_t ntiles, int64_t npeers) {
    return round_up((int64_t)sizeof(PeerRun) * ntiles * kMergeRecs((unsigned)npeers), 256);
}

// Sparse merges stamp records with a number that differs from call to call (0 is never used).
inline unsigned next_epoch(std::atomic<unsigned>& counter) {
    unsigned e = counter.fetch_add(1u, std::memory_order_relaxed) + 1u;
    if (e == 0) e = counter.fetch_add(1u, std::memory_order_relaxed) + 1u;
    return e;
}
std::atomic<unsigned> g_merge_epoch{0};  // per-tensor calls (their workspace belongs to the caller)

inline unsigned slices_of(unsigned slots) { return (unsigned)(((uint64_t)slots + 1023) / 1024); }

inline int hiperr(hipError_t e) { return e == hipSuccess ? HIPRESS_OK : HIPRESS_ERR_HIP; }

// ---- descriptor builders: validate one tensor and fill its Seg -------------------------

int payload_need(int alg, int64_t n, const hipress_params& pr, int64_t* need) {
    switch (alg) {
        case HIPRESS_ONEBIT:
        case HIPRESS_ONEBIT_DEFERRED: *need = HIPRESS_HEADER_BYTES + words_bytes(n, 1); return HIPRESS_OK;
        case HIPRESS_TBQ: *need = HIPRESS_HEADER_BYTES + words_bytes(n, 2); return HIPRESS_OK;
        case HIPRESS_TERNGRAD:
            if (pr.bucket < 1) return HIPRESS_ERR_PARAM;
            *need = HIPRESS_HEADER_BYTES + tg_scale_bytes(n, pr.bucket) + words_bytes(n, 2);
            return HIPRESS_OK;
        case HIPRESS_DGC:
        case HIPRESS_GRADDROP:
            if (bad_ratio(pr.ratio)) return HIPRESS_ERR_PARAM;
            *need = HIPRESS_HEADER_BYTES + 8 * sparse_plan(n, pr.ratio).cap;
            return HIPRESS_OK;
    }
    return HIPRESS_ERR_PARAM;
}

int check_params(int alg, const hipress_params& pr) {
    switch (alg) {
        case HIPRESS_ONEBIT:
        case HIPRESS_ONEBIT_DEFERRED: return HIPRESS_OK;
        case HIPRESS_TBQ: return (pr.threshold >= 0.f && std::isfinite(pr.threshold)) ? HIPRESS_OK : HIPRESS_ERR_PARAM;
        case HIPRESS_TERNGRAD: return pr.bucket >= 1 ? HIPRESS_OK : HIPRESS_ERR_PARAM;
        case HIPRESS_DGC:
            if (!std::isfinite(pr.momentum_factor)) return HIPRESS_ERR_PARAM;
            return bad_ratio(pr.ratio) ? HIPRESS_ERR_PARAM : HIPRESS_OK;
        case HIPRESS_GRADDROP: return bad_ratio(pr.ratio) ? HIPRESS_ERR_PARAM : HIPRESS_OK;
    }
    return HIPRESS_ERR_PARAM;
}

// Fills the fields of `s` that do not depend on the tensor's place in a launch.
// drawn: the stochastic rounding's noise is drawn in the kernel, so no noise tensor is asked for.
int build_encode_seg(int alg, const hipress_tensor& t, const hipress_params& pr, Seg* s, bool drawn = false) {
    std::memset(s, 0, sizeof(Seg));
    if (bad_n(t.n) || (is_sparse(alg) && bad_sparse_n(t.n))) return HIPRESS_ERR_SIZE;
    int rc = check_params(alg, pr);
    if (rc) return rc;
    if (!t.payload) return HIPRESS_ERR_NULL;
    if (mis(t.payload, 16)) return HIPRESS_ERR_ALIGN;
    int64_t need;
    if ((rc = payload_need(alg, t.n, pr, &need))) return rc;
    if (t.payload_bytes < need) return HIPRESS_ERR_SIZE;
    const bool need_s0 = alg != HIPRESS_TERNGRAD;
    const bool need_s1 = alg == HIPRESS_DGC || alg == HIPRESS_ONEBIT_DEFERRED;
    const bool need_u = alg == HIPRESS_TERNGRAD && !drawn;
    if (t.n > 0) {
        if (!t.grad || (need_s0 && !t.state0) || (need_s1 && !t.state1) || (need_u && !t.uniform)) return HIPRESS_ERR_NULL;
    }
    if (alg == HIPRESS_ONEBIT_DEFERRED && !t.state1) return HIPRESS_ERR_NULL;  // the scale word is always read
    if (mis(t.grad, 4) || mis(t.state0, 4) || mis(t.state1, 4) || mis(t.uniform, 4)) return HIPRESS_ERR_ALIGN;
    s->g = t.grad;
    s->pay = static_cast<uint8_t*>(t.payload);
    s->n = (unsigned long long)t.n;
    s->ntiles = tiles_of(t.n);
    s->aligned = vec_ok(t.grad);
    switch (alg) {
        case HIPRESS_ONEBIT:
        case HIPRESS_ONEBIT_DEFERRED:
        case HIPRESS_TBQ:
            s->s0 = t.state0;
            s->s1 = alg == HIPRESS_ONEBIT_DEFERRED ? t.state1 : nullptr;
            s->aligned = s->aligned && vec_ok(t.state0);
            s->f0 = pr.threshold;
            s->words_off = HIPRESS_HEADER_BYTES;
            break;
        case HIPRESS_TERNGRAD: {
            s->u = drawn ? nullptr : t.uniform;
            s->aligned = s->aligned && (drawn || vec_ok(t.uniform));
            s->bucket = (unsigned)pr.bucket;
            int64_t off = HIPRESS_HEADER_BYTES + tg_scale_bytes(t.n, pr.bucket);
            if (off > 0xffffffffLL) return HIPRESS_ERR_SIZE;
            s->words_off = (unsigned)off;
            break;
        }
        case HIPRESS_DGC:
        case HIPRESS_GRADDROP: {
            if (alg == HIPRESS_DGC) {
                s->s0 = t.state0;
                s->s1 = t.state1;
                s->f0 = pr.momentum_factor;
                s->aligned = s->aligned && vec_ok(t.state0) && vec_ok(t.state1);
            } else {
                s->s0 = nullptr;
                s->s1 = t.state0;
                s->aligned = s->aligned && vec_ok(t.state0);
            }
            SparsePlan p = sparse_plan(t.n, pr.ratio);
            s->cap = (unsigned)p.cap;
            s->sstride = (unsigned)p.stride;
            s->ns = (unsigned)p.ns;
            s->ks = (unsigned)p.ks;
            s->nsblk = (unsigned)((p.ns + kSampleTile - 1) / kSampleTile);
            break;
        }
    }
    return HIPRESS_OK;
}

int build_decode_seg(int alg, const void* payload, int64_t payload_bytes, float* out, int64_t n, Seg* s) {
    std::memset(s, 0, sizeof(Seg));
    if (bad_n(n) || (is_sparse(alg) && bad_sparse_n(n))) return HIPRESS_ERR_SIZE;
    if (!payload || (n > 0 && !out)) return HIPRESS_ERR_NULL;
    if (mis(payload, 16) || mis(out, 4)) return HIPRESS_ERR_ALIGN;
    if (payload_bytes < HIPRESS_HEADER_BYTES) return HIPRESS_ERR_SIZE;
    s->pay = const_cast<uint8_t*>(static_cast<const uint8_t*>(payload));
    s->pay_bytes = (unsigned long long)payload_bytes;
    s->out = out;
    s->n = (unsigned long long)n;
    s->ntiles = tiles_of(n);
    s->aligned = vec_ok(out);
    s->words_off = HIPRESS_HEADER_BYTES;
    switch (alg) {
        case HIPRESS_ONEBIT:
        case HIPRESS_ONEBIT_DEFERRED:
            if (payload_bytes < HIPRESS_HEADER_BYTES + words_bytes(n, 1)) return HIPRESS_ERR_SIZE;
            break;
        case HIPRESS_TBQ:
            if (payload_bytes < HIPRESS_HEADER_BYTES + words_bytes(n, 2)) return HIPRESS_ERR_SIZE;
            break;
        case HIPRESS_TERNGRAD:
            // the bucket size lives in the header on the device; the caller-side
            // size check is done by the variant that knows the bucket
            break;
        case HIPRESS_DGC:
        case HIPRESS_GRADDROP: {
            int64_t slots = (payload_bytes - HIPRESS_HEADER_BYTES) / 8;
            s->cap = (unsigned)(slots > 0xffffffffLL ? 0xffffffffLL : slots);
            s->ncblk = (unsigned)(((int64_t)s->cap + 1023) / 1024);
            break;
        }
        default: return HIPRESS_ERR_PARAM;
    }
    return HIPRESS_OK;
}

// TernGrad decode needs the bucket size to place the words; the host passes it.
int finish_terngrad_decode_seg(Seg* s, int64_t payload_bytes, int32_t bucket) {
    if (bucket < 1) return HIPRESS_ERR_PARAM;
    int64_t off = HIPRESS_HEADER_BYTES + tg_scale_bytes((int64_t)s->n, bucket);
    if (off > 0xffffffffLL) return HIPRESS_ERR_SIZE;
    if (payload_bytes < off + words_bytes((int64_t)s->n, 2)) return HIPRESS_ERR_SIZE;
    s->bucket = (unsigned)bucket;
    s->words_off = (unsigned)off;
    return HIPRESS_OK;
}

// Pairs a sparse encode of this tensor is expected to select: the sample's rank times the stride.
inline unsigned long long expected_pairs(const Seg& s) { return (unsigned long long)s.ks * s.sstride; }

Launch single_launch(const Seg& s) {
    Launch L;
    std::memset(&L, 0, sizeof L);
    L.single = true;
    L.seg = s;
    L.seg.tile0 = 0;
    L.seg.id = 0;
    L.seg.ws0 = 0;
    L.ntiles = s.ntiles;
    L.nsegs = 1;
    L.expect_pairs = expected_pairs(s);
    return L;
}

template <class T>
int upload(const std::vector<T>& v, T** dptr) {
    *dptr = nullptr;
    if (v.empty()) return HIPRESS_OK;
    if (hipMalloc(reinterpret_cast<void**>(dptr), v.size() * sizeof(T)) != hipSuccess) return HIPRESS_ERR_HIP;
    if (hipMemcpy(*dptr, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return HIPRESS_ERR_HIP;
    return HIPRESS_OK;
}

// Assigns tile ranges to the tensors of a launch and builds the workgroup -> (tensor, tile) map.
template <class S, class GetSeg>
int layout_tiles(std::vector<S>& segs, GetSeg seg_of, std::vector<uint2>& map, unsigned* total) {
    uint64_t t = 0;
    for (size_t i = 0; i < segs.size(); ++i) {
        Seg& s = seg_of(segs[i]);
        s.tile0 = (unsigned)t;
        s.id = (unsigned)i;
        t += s.ntiles;
        if (t > 0x7fffffffull) return HIPRESS_ERR_SIZE;
    }
    map.resize((size_t)t);
    size_t k = 0;
    for (size_t i = 0; i < segs.size(); ++i) {
        Seg& s = seg_of(segs[i]);
        for (unsigned j = 0; j < s.ntiles; ++j) map[k++] = make_uint2((unsigned)i, j);
    }
    *total = (unsigned)t;
    return HIPRESS_OK;
}

// Sparse launches: gives every tensor its slice of the sample array and builds the
// workgroup -> (tensor, sample tile) map of the select passes.
int64_t layout_samples(std::vector<Seg>& segs, std::vector<uint2>& smap) {
    uint64_t off = 0;
    smap.clear();
    for (size_t i = 0; i < segs.size(); ++i) {
        Seg& s = segs[i];
        s.ws0 = off;
        off += (s.ns + 3u) & ~3ull;
        for (unsigned j = 0; j < s.nsblk; ++j) smap.push_back(make_uint2((unsigned)i, j));
    }
    return (int64_t)off;
}

}  // namespace

// ============================================================================
// batch objects
// ============================================================================

struct hipress_batch {
    int alg = 0;
    hipress_params params{};
    std::vector<Seg> enc, dec;
    bool can_encode = false, can_decode = false;
    bool drawn = false;  // terngrad: no tensor brings a noise tensor, the encode call brings a seed
    Seg* d_enc = nullptr;
    Seg* d_dec = nullptr;
    uint2* d_map = nullptr;
    uint2* d_smap = nullptr;  // sparse: sample tiles
    uint2* d_cmap = nullptr;  // sparse decode: payload-slot tiles
    uint32_t* d_tptr = nullptr;      // sparse decode: first payload slot of every tile
    uint32_t* d_disorder = nullptr;  // sparse decode: per tensor, the epoch in which its payload was last seen out of order
    unsigned epoch = 0;
    unsigned ntiles = 0, nstiles = 0, nctiles = 0;
    void* ws = nullptr;  // onebit: one float per tile; sparse: SparseWsLayout
    SparseWsLayout swl{};
    unsigned long long expect_pairs = 0;  // sparse encode: sum over the tensors
};

struct hipress_merge_batch {
    int alg = 0;
    hipress_params params{};
    int npeers = 0;
    bool reencode = false;
    bool aggregate = false;  // some chunk writes its fp32 sum
    bool local = false;      // some chunk starts from a local gradient
    std::vector<MergeSeg> segs;
    std::vector<Seg> renc;  // sparse re-encode descriptors
    MergeSeg* d_segs = nullptr;
    Seg* d_renc = nullptr;
    uint2* d_map = nullptr;
    uint2* d_smap = nullptr;
    unsigned ntiles = 0, nstiles = 0;
    void* ws = nullptr;
    SparseWsLayout swl{};
    void* iws = nullptr;  // sparse: per tile a head and one run record per peer
    unsigned* tgflags = nullptr;  // terngrad: per chunk, does some peer's header disagree with the batch's bucket size
    unsigned slices = 1;  // sparse: the largest peer buffer's slots / 1024, rounded up
    unsigned long long expect_pairs = 0;  // sparse re-encode: sum over the chunks
    std::atomic<unsigned> epoch{0};
    unsigned cur_epoch = 0;
};

extern "C" {

int hipress_version(void) { return 120; }

const char* hipress_strerror(int code) {
    switch (code) {
        case HIPRESS_OK: return "ok";
        case HIPRESS_ERR_NULL: return "a required pointer is NULL";
        case HIPRESS_ERR_SIZE: return "element count out of range or buffer too small";
        case HIPRESS_ERR_ALIGN: return "pointer not sufficiently aligned";
        case HIPRESS_ERR_PARAM: return "parameter out of range";
        case HIPRESS_ERR_HIP: return "HIP runtime error";
        case HIPRESS_ERR_WORKSPACE: return "workspace missing or too small";
    }
    return "unknown error";
}

// ---- sizes -----------------------------------------------------------------------

int64_t hipress_onebit_payload_bytes(int64_t n) {
    return bad_n(n) ? HIPRESS_ERR_SIZE : HIPRESS_HEADER_BYTES + words_bytes(n, 1);
}
int64_t hipress_tbq_payload_bytes(int64_t n) {
    return bad_n(n) ? HIPRESS_ERR_SIZE : HIPRESS_HEADER_BYTES + words_bytes(n, 2);
}
int64_t hipress_terngrad_payload_bytes(int64_t n, int32_t bucket) {
    if (bad_n(n)) return HIPRESS_ERR_SIZE;
    if (bucket < 1) return HIPRESS_ERR_PARAM;
    return HIPRESS_HEADER_BYTES + tg_scale_bytes(n, bucket) + words_bytes(n, 2);
}
int64_t hipress_sparse_capacity(int64_t n, double ratio) {
    if (bad_sparse_n(n)) return HIPRESS_ERR_SIZE;
    if (bad_ratio(ratio)) return HIPRESS_ERR_PARAM;
    return sparse_plan(n, ratio).cap;
}
int64_t hipress_sparse_payload_bytes(int64_t n, double ratio) {
    int64_t c = hipress_sparse_capacity(n, ratio);
    return c < 0 ? c : HIPRESS_HEADER_BYTES + 8 * c;
}
int64_t hipress_onebit_workspace_bytes(int64_t n) {
    return bad_n(n) ? HIPRESS_ERR_SIZE : round_up(4 * (int64_t)tiles_of(n), 256);
}
int64_t hipress_sparse_workspace_bytes(int64_t n, double ratio) {
    if (bad_sparse_n(n)) return HIPRESS_ERR_SIZE;
    if (bad_ratio(ratio)) return HIPRESS_ERR_PARAM;
    return sparse_ws_layout(sparse_plan(n, ratio).ns, tiles_of(n), 1).bytes;
}

// ---- TBQ -------------------------------------------------------------------------

int hipress_tbq_encode(const float* grad, float* residual, int64_t n, void* payload, int64_t payload_bytes,
                       float threshold, void* stream) {
    hipress_tensor t{grad, residual, nullptr, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    pr.threshold = threshold;
    Seg s;
    int rc = build_encode_seg(HIPRESS_TBQ, t, pr, &s);
    if (rc) return rc;
    return hiperr(launch_tbq_encode(single_launch(s), static_cast<hipStream_t>(stream)));
}

int hipress_tbq_decode(const void* payload, int64_t payload_bytes, float* out, int64_t n, void* stream) {
    Seg s;
    int rc = build_decode_seg(HIPRESS_TBQ, payload, payload_bytes, out, n, &s);
    if (rc) return rc;
    return hiperr(launch_tbq_decode(single_launch(s), static_cast<hipStream_t>(stream)));
}

// ---- onebit ------------------------------------------------------------------------

int hipress_onebit_encode(const float* grad, float* residual, int64_t n, void* payload, int64_t payload_bytes,
                          void* workspace, int64_t workspace_bytes, void* stream) {
    hipress_tensor t{grad, residual, nullptr, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    Seg s;
    int rc = build_encode_seg(HIPRESS_ONEBIT, t, pr, &s);
    if (rc) return rc;
    if (!workspace || workspace_bytes < hipress_onebit_workspace_bytes(n)) return HIPRESS_ERR_WORKSPACE;
    if (mis(workspace, 16)) return HIPRESS_ERR_ALIGN;
    return hiperr(launch_onebit_encode(single_launch(s), static_cast<float*>(workspace), -1, static_cast<hipStream_t>(stream)));
}

// hipress_onebit_encode without a workspace argument: the per-tile partial sums go to
// a file-scope device array, so the call needs no memory beyond inputs and outputs.
// Every GPU holds its own copy of the array at its own address; that address is asked
// for once per device (the first call on it) and kept.  The array's name is a
// host-side stand-in, not a device address, so only the looked-up pointer is handed to
// kernels.  The magnitude-sum launch writes partial[0, tiles) before the scale launch
// reads them, so whatever an earlier call left there is never seen and nothing has to
// be cleared.
constexpr int kStaticMaxDevices = 64;
constexpr int64_t kStaticTiles = HIPRESS_ONEBIT_STATIC_MAX_N / kTile;
static_assert(HIPRESS_ONEBIT_STATIC_MAX_N % kTile == 0 && kStaticTiles == 65536,
              "a tensor of HIPRESS_ONEBIT_STATIC_MAX_N elements fills the array exactly");
static __device__ __align__(256) float scratch[kStaticTiles];
static std::atomic<float*> scratch_ptr[kStaticMaxDevices];

// The array of the CURRENT device; a stream that belongs to another device is refused
// (its kernels would run where this pointer means nothing).
static int static_scratch(hipStream_t stream, float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticMaxDevices) return HIPRESS_ERR_HIP;
    // 0, 1 and 2 are the default, legacy and per-thread stream handles: always the current device's
    if (reinterpret_cast<uintptr_t>(stream) > 2) {
        int sdev = -1;
        if (hipStreamGetDevice(stream, &sdev) != hipSuccess) return HIPRESS_ERR_HIP;
        if (sdev != dev) return HIPRESS_ERR_PARAM;
    }
    float* p = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)) != hipSuccess || !p) return HIPRESS_ERR_HIP;
        scratch_ptr[dev].store(p, std::memory_order_release);  // threads that race here look up the same address
    }
    *out = p;
    return HIPRESS_OK;
}

int hipress_onebit_encode_static(const float* grad, float* residual, int64_t n, void* payload, int64_t payload_bytes,
                                 void* stream) {
    if (n > HIPRESS_ONEBIT_STATIC_MAX_N) return HIPRESS_ERR_SIZE;
    hipress_tensor t{grad, residual, nullptr, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    Seg s;
    int rc = build_encode_seg(HIPRESS_ONEBIT, t, pr, &s);
    if (rc) return rc;
    float* partial = nullptr;
    if ((rc = static_scratch(static_cast<hipStream_t>(stream), &partial))) return rc;
    return hiperr(launch_onebit_encode(single_launch(s), partial, -1, static_cast<hipStream_t>(stream)));
}

int hipress_onebit_decode(const void* payload, int64_t payload_bytes, float* out, int64_t n, void* stream) {
    Seg s;
    int rc = build_decode_seg(HIPRESS_ONEBIT, payload, payload_bytes, out, n, &s);
    if (rc) return rc;
    return hiperr(launch_onebit_decode(single_launch(s), static_cast<hipStream_t>(stream)));
}

int hipress_onebit_encode_deferred(const float* grad, float* state, float* scale_state, int64_t n, void* payload,
                                   int64_t payload_bytes, void* workspace, int64_t workspace_bytes, void* stream) {
    hipress_tensor t{grad, state, scale_state, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    Seg s;
    int rc = build_encode_seg(HIPRESS_ONEBIT_DEFERRED, t, pr, &s);
    if (rc) return rc;
    if (!workspace || workspace_bytes < hipress_onebit_workspace_bytes(n)) return HIPRESS_ERR_WORKSPACE;
    if (mis(workspace, 16)) return HIPRESS_ERR_ALIGN;
    return hiperr(launch_onebit_encode_deferred(single_launch(s), static_cast<float*>(workspace), -1,
                                                static_cast<hipStream_t>(stream)));
}

int hipress_onebit_residual(const float* state, const float* scale_state, int64_t n, float* residual, void* stream) {
    if (bad_n(n)) return HIPRESS_ERR_SIZE;
    if (!scale_state || (n > 0 && (!state || !residual))) return HIPRESS_ERR_NULL;
    if (mis(state, 4) || mis(scale_state, 4) || mis(residual, 4)) return HIPRESS_ERR_ALIGN;
    Seg s;
    std::memset(&s, 0, sizeof s);
    s.s0 = const_cast<float*>(state);
    s.s1 = const_cast<float*>(scale_state);
    s.out = residual;
    s.n = (unsigned long long)n;
    s.ntiles = tiles_of(n);
    s.aligned = vec_ok(state) && vec_ok(residual);
    return hiperr(launch_onebit_materialize(single_launch(s), static_cast<hipStream_t>(stream)));
}

// ---- TernGrad ----------------------------------------------------------------------

int hipress_terngrad_encode(const float* grad, const float* uniform, int64_t n, void* payload,
                            int64_t payload_bytes, int32_t bucket, void* stream) {
    hipress_tensor t{grad, nullptr, nullptr, uniform, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    pr.bucket = bucket;
    Seg s;
    int rc = build_encode_seg(HIPRESS_TERNGRAD, t, pr, &s);
    if (rc) return rc;
    return hiperr(launch_terngrad_encode(single_launch(s), (unsigned)bucket, false, 0u, static_cast<hipStream_t>(stream)));
}

int hipress_terngrad_encode_seeded(const float* grad, int64_t n, void* payload, int64_t payload_bytes, int32_t bucket,
                                   uint64_t seed, void* stream) {
    hipress_tensor t{grad, nullptr, nullptr, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    pr.bucket = bucket;
    Seg s;
    int rc = build_encode_seg(HIPRESS_TERNGRAD, t, pr, &s, true);
    if (rc) return rc;
    return hiperr(launch_terngrad_encode(single_launch(s), (unsigned)bucket, true, uniform_key(seed),
                                         static_cast<hipStream_t>(stream)));
}

int hipress_uniform_fill(float* out, int64_t n, uint64_t seed, uint32_t tensor, void* stream) {
    if (bad_n(n)) return HIPRESS_ERR_SIZE;
    if (n > 0 && !out) return HIPRESS_ERR_NULL;
    if (mis(out, 4)) return HIPRESS_ERR_ALIGN;
    return hiperr(launch_uniform_fill(out, (unsigned long long)n, tensor_key(uniform_key(seed), tensor),
                                      static_cast<hipStream_t>(stream)));
}

// The bucket size is read from the payload header on the device and the scale
// array that precedes the words is located with it there (checked against
// payload_bytes on the device); the host-side check covers header and words.
int hipress_terngrad_decode(const void* payload, int64_t payload_bytes, float* out, int64_t n, void* stream) {
    Seg s;
    int rc = build_decode_seg(HIPRESS_TERNGRAD, payload, payload_bytes, out, n, &s);
    if (rc) return rc;
    if (payload_bytes < HIPRESS_HEADER_BYTES + words_bytes(n, 2)) return HIPRESS_ERR_SIZE;
    return hiperr(launch_terngrad_decode(single_launch(s), 0u, static_cast<hipStream_t>(stream)));
}

// ---- the in-tree CompLL operator -------------------------------------------------------

int64_t hipress_compll_payload_bytes(int64_t n, int32_t bitwidth) {
    if (bad_n(n)) return HIPRESS_ERR_SIZE;
    if (bitwidth != 1 && bitwidth != 2 && bitwidth != 4 && bitwidth != 8) return HIPRESS_ERR_PARAM;
    return 10 + (n * bitwidth + 7) / 8;
}

// What hipress_compll_decode writes for a payload hipress_compll_encode made of n
// elements: (8 * code bytes) / b - tail with tail = n mod 2^b, never more than n.
int64_t hipress_compll_decoded_count(int64_t n, int32_t bitwidth) {
    int64_t bytes = hipress_compll_payload_bytes(n, bitwidth);
    if (bytes < 0) return bytes;
    int64_t count = (8 * (bytes - 10)) / bitwidth - (n % (1LL << bitwidth));
    if (count < 0) count = 0;
    return count < n ? count : n;
}

int64_t hipress_compll_workspace_bytes(int64_t n) {
    return bad_n(n) ? HIPRESS_ERR_SIZE : round_up(8 * (int64_t)tiles_of(n), 256);
}

static int compll_encode_impl(const float* grad, const float* uniform, bool drawn, uint64_t seed, int64_t n,
                              void* compressed, int64_t compressed_bytes, int32_t bitwidth, void* workspace,
                              int64_t workspace_bytes, void* stream) {
    int64_t need = hipress_compll_payload_bytes(n, bitwidth);
    if (need < 0) return (int)need;
    if (!compressed || (n > 0 && (!grad || (!drawn && !uniform)))) return HIPRESS_ERR_NULL;
    if (mis(grad, 4) || mis(uniform, 4)) return HIPRESS_ERR_ALIGN;
    if (compressed_bytes < need) return HIPRESS_ERR_SIZE;
    if (!workspace || workspace_bytes < hipress_compll_workspace_bytes(n)) return HIPRESS_ERR_WORKSPACE;
    if (mis(workspace, 16)) return HIPRESS_ERR_ALIGN;
    Seg s;
    std::memset(&s, 0, sizeof s);
    s.g = grad;
    s.u = drawn ? nullptr : uniform;
    s.pay = static_cast<uint8_t*>(compressed);
    s.n = (unsigned long long)n;
    s.ntiles = tiles_of(n);
    s.aligned = vec_ok(grad) && (drawn || vec_ok(uniform));
    s.bucket = (unsigned)bitwidth;
    return hiperr(launch_compll_encode(single_launch(s), bitwidth, static_cast<float*>(workspace), drawn,
                                       drawn ? uniform_key(seed) : 0u, static_cast<hipStream_t>(stream)));
}

int hipress_compll_encode(const float* grad, const float* uniform, int64_t n, void* compressed,
                          int64_t compressed_bytes, int32_t bitwidth, void* workspace, int64_t workspace_bytes,
                          void* stream) {
    return compll_encode_impl(grad, uniform, false, 0, n, compressed, compressed_bytes, bitwidth, workspace,
                              workspace_bytes, stream);
}

int hipress_compll_encode_seeded(const float* grad, int64_t n, void* compressed, int64_t compressed_bytes,
                                 int32_t bitwidth, uint64_t seed, void* workspace, int64_t workspace_bytes,
                                 void* stream) {
    return compll_encode_impl(grad, nullptr, true, seed, n, compressed, compressed_bytes, bitwidth, workspace,
                              workspace_bytes, stream);
}

int hipress_compll_decode(const void* compressed, int64_t compressed_bytes, float* out, int64_t n, void* stream) {
    if (bad_n(n)) return HIPRESS_ERR_SIZE;
    if (!compressed || (n > 0 && !out)) return HIPRESS_ERR_NULL;
    if (mis(out, 4)) return HIPRESS_ERR_ALIGN;
    if (compressed_bytes < 10) return HIPRESS_ERR_SIZE;
    Seg s;
    std::memset(&s, 0, sizeof s);
    s.pay = const_cast<uint8_t*>(static_cast<const uint8_t*>(compressed));
    s.pay_bytes = (unsigned long long)compressed_bytes;
    s.out = out;
    s.n = (unsigned long long)n;
    s.ntiles = tiles_of(n);
    s.aligned = vec_ok(out);
    return hiperr(launch_compll_decode(single_launch(s), static_cast<hipStream_t>(stream)));
}

// ---- DGC / GradDrop ------------------------------------------------------------------

static int sparse_encode_single(int alg, const hipress_tensor& t, const hipress_params& pr, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    Seg s;
    int rc = build_encode_seg(alg, t, pr, &s);
    if (rc) return rc;
    SparseWsLayout l = sparse_ws_layout(s.ns, s.ntiles, 1);
    if (!workspace || workspace_bytes < l.bytes) return HIPRESS_ERR_WORKSPACE;
    if (mis(workspace, 16)) return HIPRESS_ERR_ALIGN;
    return hiperr(launch_sparse_encode(single_launch(s), alg == HIPRESS_DGC, sparse_ws_at(workspace, l), -1,
                                       static_cast<hipStream_t>(stream)));
}

int hipress_dgc_encode(const float* grad, float* momentum, float* accumulator, int64_t n, void* payload,
                       int64_t payload_bytes, float momentum_factor, double ratio, void* workspace,
                       int64_t workspace_bytes, void* stream) {
    hipress_tensor t{grad, momentum, accumulator, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    pr.momentum_factor = momentum_factor;
    pr.ratio = ratio;
    return sparse_encode_single(HIPRESS_DGC, t, pr, workspace, workspace_bytes, stream);
}

int hipress_graddrop_encode(const float* grad, float* accumulator, int64_t n, void* payload,
                            int64_t payload_bytes, double ratio, void* workspace, int64_t workspace_bytes,
                            void* stream) {
    hipress_tensor t{grad, accumulator, nullptr, nullptr, payload, nullptr, n, payload_bytes};
    hipress_params pr{};
    pr.ratio = ratio;
    return sparse_encode_single(HIPRESS_GRADDROP, t, pr, workspace, workspace_bytes, stream);
}

int hipress_sparse_decode(const void* payload, int64_t payload_bytes, float* out, int64_t n, void* stream) {
    Seg s;
    int rc = build_decode_seg(HIPRESS_DGC, payload, payload_bytes, out, n, &s);
    if (rc) return rc;
    return hiperr(launch_sparse_decode(single_launch(s), static_cast<hipStream_t>(stream)));
}

// ---- decode-and-merge ------------------------------------------------------------------

// reencode: the call also re-encodes the sum; only then may the aggregate be left out.
// local: the aggregator's own uncompressed gradient the sum starts from, or NULL (zero).
static int build_merge_seg(int alg, const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                           const float* local, float* aggregate, int64_t n, bool reencode, MergeSeg* m) {
    std::memset(m, 0, sizeof(MergeSeg));
    if (bad_n(n) || (is_sparse(alg) && bad_sparse_n(n))) return HIPRESS_ERR_SIZE;
    if (npeers < 1 || npeers > HIPRESS_MAX_PEERS) return HIPRESS_ERR_PARAM;
    if (!payloads || !payload_bytes || (n > 0 && !aggregate && !reencode)) return HIPRESS_ERR_NULL;
    if (mis(aggregate, 4) || mis(local, 4)) return HIPRESS_ERR_ALIGN;
    for (int p = 0; p < npeers; ++p) {
        if (!payloads[p]) return HIPRESS_ERR_NULL;
        if (mis(payloads[p], 16)) return HIPRESS_ERR_ALIGN;
        int64_t need = HIPRESS_HEADER_BYTES;
        if (alg == HIPRESS_ONEBIT) need += words_bytes(n, 1);
        else if (alg == HIPRESS_TBQ || alg == HIPRESS_TERNGRAD) need += words_bytes(n, 2);
        if (payload_bytes[p] < need) return HIPRESS_ERR_SIZE;
        m->peer[p] = static_cast<const uint8_t*>(payloads[p]);
        m->peer_bytes[p] = (unsigned long long)payload_bytes[p];
        int64_t slots = (payload_bytes[p] - HIPRESS_HEADER_BYTES) / 8;
        m->peer_slots[p] = (unsigned)(slots > 0xffffffffLL ? 0xffffffffLL : slots);
    }
    m->s.g = n > 0 ? local : nullptr;
    m->s.out = aggregate;
    m->s.n = (unsigned long long)n;
    m->s.ntiles = tiles_of(n);
    m->s.aligned = vec_ok(aggregate) && vec_ok(local);
    return HIPRESS_OK;
}

// The state buffer asks for the re-encode; an empty chunk has no state buffer to point at,
// so there the output payload does.
static bool wants_reencode(const float* state, const void* out_payload, int64_t n) {
    return state != nullptr || (n == 0 && out_payload != nullptr);
}

static MergeLaunch single_merge_launch(const MergeSeg& m, int npeers, bool reencode) {
    MergeLaunch L;
    std::memset(&L, 0, sizeof L);
    L.single = true;
    L.seg = m;
    L.ntiles = m.s.ntiles;
    L.nsegs = 1;
    L.npeers = npeers;
    L.reencode = reencode;
    L.aggregate = m.s.out != nullptr;
    L.local = m.s.g != nullptr;
    return L;
}

static int add_tbq_reencode(MergeSeg* m, float* residual, void* out_payload, int64_t out_payload_bytes, float threshold) {
    if (!out_payload) return HIPRESS_ERR_NULL;
    if (mis(out_payload, 16) || mis(residual, 4)) return HIPRESS_ERR_ALIGN;
    if (!(threshold >= 0.f && std::isfinite(threshold))) return HIPRESS_ERR_PARAM;
    if (out_payload_bytes < HIPRESS_HEADER_BYTES + words_bytes((int64_t)m->s.n, 2)) return HIPRESS_ERR_SIZE;
    m->s.s0 = residual;
    m->s.pay = static_cast<uint8_t*>(out_payload);
    m->s.f0 = threshold;
    m->s.aligned = m->s.aligned && vec_ok(residual);
    return HIPRESS_OK;
}

int hipress_tbq_decode_merge(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                             float* aggregate, int64_t n, float* residual, void* out_payload,
                             int64_t out_payload_bytes, float threshold, void* stream) {
    return hipress_tbq_decode_merge_local(payloads, payload_bytes, npeers, nullptr, aggregate, n, residual, out_payload,
                                          out_payload_bytes, threshold, stream);
}

int hipress_tbq_decode_merge_local(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                   const float* local, float* aggregate, int64_t n, float* residual, void* out_payload,
                                   int64_t out_payload_bytes, float threshold, void* stream) {
    MergeSeg m;
    const bool reenc = wants_reencode(residual, out_payload, n);
    int rc = build_merge_seg(HIPRESS_TBQ, payloads, payload_bytes, npeers, local, aggregate, n, reenc, &m);
    if (rc) return rc;
    if (reenc && (rc = add_tbq_reencode(&m, residual, out_payload, out_payload_bytes, threshold))) return rc;
    return hiperr(launch_dense_merge(single_merge_launch(m, npeers, reenc), HIPRESS_TBQ,
                                     static_cast<hipStream_t>(stream)));
}

int hipress_onebit_decode_merge(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                float* aggregate, int64_t n, void* stream) {
    return hipress_onebit_decode_merge_local(payloads, payload_bytes, npeers, nullptr, aggregate, n, stream);
}

int hipress_onebit_decode_merge_local(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                      const float* local, float* aggregate, int64_t n, void* stream) {
    MergeSeg m;
    int rc = build_merge_seg(HIPRESS_ONEBIT, payloads, payload_bytes, npeers, local, aggregate, n, false, &m);
    if (rc) return rc;
    return hiperr(launch_dense_merge(single_merge_launch(m, npeers, false), HIPRESS_ONEBIT,
                                     static_cast<hipStream_t>(stream)));
}

int hipress_terngrad_decode_merge(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                  float* aggregate, int64_t n, void* stream) {
    return hipress_terngrad_decode_merge_local(payloads, payload_bytes, npeers, nullptr, aggregate, n, stream);
}

int hipress_terngrad_decode_merge_local(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                        const float* local, float* aggregate, int64_t n, void* stream) {
    MergeSeg m;
    int rc = build_merge_seg(HIPRESS_TERNGRAD, payloads, payload_bytes, npeers, local, aggregate, n, false, &m);
    if (rc) return rc;
    return hiperr(launch_dense_merge(single_merge_launch(m, npeers, false), HIPRESS_TERNGRAD,
                                     static_cast<hipStream_t>(stream)));
}

int64_t hipress_sparse_merge_workspace_bytes(int64_t n, int32_t npeers, double ratio, int32_t reencode) {
    if (bad_sparse_n(n)) return HIPRESS_ERR_SIZE;
    if (npeers < 1 || npeers > HIPRESS_MAX_PEERS) return HIPRESS_ERR_PARAM;
    int64_t bytes = merge_index_bytes(tiles_of(n), npeers);
    if (reencode) {
        if (bad_ratio(ratio)) return HIPRESS_ERR_PARAM;
        bytes += sparse_ws_layout(sparse_plan(n, ratio).ns, tiles_of(n), 1).bytes;
    }
    return bytes;
}

int hipress_sparse_decode_merge(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                float* aggregate, int64_t n, float* accumulator, void* out_payload,
                                int64_t out_payload_bytes, double ratio, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    return hipress_sparse_decode_merge_local(payloads, payload_bytes, npeers, nullptr, aggregate, n, accumulator,
                                             out_payload, out_payload_bytes, ratio, workspace, workspace_bytes, stream);
}

int hipress_sparse_decode_merge_local(const void* const* payloads, const int64_t* payload_bytes, int32_t npeers,
                                      const float* local, float* aggregate, int64_t n, float* accumulator,
                                      void* out_payload, int64_t out_payload_bytes, double ratio, void* workspace,
                                      int64_t workspace_bytes, void* stream) {
    MergeSeg m;
    const bool reenc = wants_reencode(accumulator, out_payload, n);
    int rc = build_merge_seg(HIPRESS_DGC, payloads, payload_bytes, npeers, local, aggregate, n, reenc, &m);
    if (rc) return rc;
    SparseWsLayout l{};
    const int64_t ibytes = merge_index_bytes(m.s.ntiles, npeers);
    int64_t need = ibytes;
    if (reenc) {
        // the gradient of this descriptor is never read (the merge kernel takes the sum from LDS): any valid pointer passes its checks
        hipress_tensor t{aggregate ? aggregate : accumulator, accumulator, nullptr, nullptr, out_payload, nullptr, n, out_payload_bytes};
        hipress_params pr{};
        pr.ratio = ratio;
        if ((rc = build_encode_seg(HIPRESS_GRADDROP, t, pr, &m.r))) return rc;
        l = sparse_ws_layout(m.r.ns, m.r.ntiles, 1);
        need += l.bytes;
    }
    if (!workspace || workspace_bytes < need) return HIPRESS_ERR_WORKSPACE;
    if (mis(workspace, 16)) return HIPRESS_ERR_ALIGN;
    uint8_t* wsb = static_cast<uint8_t*>(workspace);
    PeerRun* runs = reinterpret_cast<PeerRun*>(wsb);
    SparseWs ws{};
    if (reenc) ws = sparse_ws_at(wsb + ibytes, l);
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned slices = 1;
    for (int p = 0; p < npeers; ++p) slices = std::max(slices, slices_of(m.peer_slots[p]));
    hipError_t e = launch_sparse_merge(single_merge_launch(m, npeers, reenc), ws, runs, slices, next_epoch(g_merge_epoch), -1, st);
    if (e != hipSuccess) return HIPRESS_ERR_HIP;
    if (reenc) e = launch_sparse_encode(single_launch(m.r), false, ws, kSparseAfterAccum, st);
    return hiperr(e);
}

// ---- batches ---------------------------------------------------------------------------

int hipress_batch_destroy(hipress_batch* b) {
    if (!b) return HIPRESS_OK;
    (void)hipFree(b->d_enc);
    (void)hipFree(b->d_dec);
    (void)hipFree(b->d_map);
    (void)hipFree(b->d_smap);
    (void)hipFree(b->d_cmap);
    (void)hipFree(b->d_tptr);
    (void)hipFree(b->d_disorder);
    (void)hipFree(b->ws);
    delete b;
    return HIPRESS_OK;
}

static int batch_create_impl(hipress_batch** out, int32_t alg, const hipress_tensor* tensors, int32_t count,
                             const hipress_params* params) {
    if (!out || !params || (count > 0 && !tensors)) return HIPRESS_ERR_NULL;
    *out = nullptr;
    if (count < 0) return HIPRESS_ERR_SIZE;
    if (alg < HIPRESS_ONEBIT || alg > HIPRESS_ONEBIT_DEFERRED) return HIPRESS_ERR_PARAM;
    int rc = check_params(alg, *params);
    if (rc) return rc;
    hipress_batch* b = new (std::nothrow) hipress_batch;
    if (!b) return HIPRESS_ERR_HIP;
    b->alg = alg;
    b->params = *params;
    const bool sparse = alg == HIPRESS_DGC || alg == HIPRESS_GRADDROP;
    // A batch may be built for encode, for decode, or for both: a side is enabled
    // when every tensor carries the buffers that side needs.
    bool enc_ok = true, dec_ok = true;
    for (int i = 0; i < count; ++i) {
        const hipress_tensor& t = tensors[i];
        if (t.n > 0 && !t.grad) enc_ok = false;
        if (t.n > 0 && !t.out) dec_ok = false;
    }
    if (!enc_ok && !dec_ok) { delete b; return HIPRESS_ERR_NULL; }
    if (alg == HIPRESS_TERNGRAD && enc_ok) {
        // either every tensor brings its noise, or none does and the encode calls bring a seed
        int with = 0, without = 0;
        for (int i = 0; i < count; ++i)
            if (tensors[i].n > 0) (tensors[i].uniform ? with : without)++;
        if (with && without) { delete b; return HIPRESS_ERR_NULL; }
        b->drawn = without > 0;
    }
    b->can_encode = enc_ok;
    b->can_decode = dec_ok;
    struct Guard {  // frees the half-built batch on every way out but the last
        hipress_batch* b;
        ~Guard() { hipress_batch_destroy(b); }
    } guard{b};
    auto fail = [](int code) { return code; };
    for (int i = 0; i < count; ++i) {
        const hipress_tensor& t = tensors[i];
        Seg s;
        if (enc_ok) {
            if ((rc = build_encode_seg(alg, t, *params, &s, b->drawn))) return fail(rc);
            b->enc.push_back(s);
        }
        if (dec_ok) {
            if ((rc = build_decode_seg(alg, t.payload, t.payload_bytes, t.out, t.n, &s))) return fail(rc);
            if (alg == HIPRESS_TERNGRAD && (rc = finish_terngrad_decode_seg(&s, t.payload_bytes, params->bucket))) return fail(rc);
            b->dec.push_back(s);
        }
    }
    std::vector<uint2> map;
    auto ident = [](Seg& s) -> Seg& { return s; };
    if (enc_ok && (rc = layout_tiles(b->enc, ident, map, &b->ntiles))) return fail(rc);
    if (dec_ok && (rc = layout_tiles(b->dec, ident, map, &b->ntiles))) return fail(rc);
    if (enc_ok && sparse) {
        std::vector<uint2> smap;
        int64_t total_ns = layout_samples(b->enc, smap);
        for (const Seg& s : b->enc) b->expect_pairs += expected_pairs(s);
        b->nstiles = (unsigned)smap.size();
        b->swl = sparse_ws_layout(total_ns, b->ntiles, count);
        if (b->swl.bytes && hipMalloc(&b->ws, (size_t)b->swl.bytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        if ((rc = upload(smap, &b->d_smap))) return fail(rc);
    } else if (enc_ok && (alg == HIPRESS_ONEBIT || alg == HIPRESS_ONEBIT_DEFERRED)) {
        if (hipMalloc(&b->ws, (size_t)round_up(4 * (int64_t)(b->ntiles ? b->ntiles : 1), 256)) != hipSuccess) return fail(HIPRESS_ERR_HIP);
    }
    if (dec_ok && sparse) {
        std::vector<uint2> cmap;
        for (size_t i = 0; i < b->dec.size(); ++i)
            for (unsigned j = 0; j < b->dec[i].ncblk; ++j) cmap.push_back(make_uint2((unsigned)i, j));
        b->nctiles = (unsigned)cmap.size();
        if ((rc = upload(cmap, &b->d_cmap))) return fail(rc);
        const size_t tptr_bytes = 4 * (size_t)(b->ntiles ? b->ntiles : 1), flag_bytes = 4 * (size_t)(count ? count : 1);
        if (hipMalloc(reinterpret_cast<void**>(&b->d_tptr), tptr_bytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        if (hipMalloc(reinterpret_cast<void**>(&b->d_disorder), flag_bytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        if (hipMemset(b->d_disorder, 0, flag_bytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
    }
    if ((rc = upload(b->enc, &b->d_enc))) return fail(rc);
    if ((rc = upload(b->dec, &b->d_dec))) return fail(rc);
    if ((rc = upload(map, &b->d_map))) return fail(rc);
    guard.b = nullptr;
    *out = b;
    return HIPRESS_OK;
}

// Host allocations of the set-up (descriptor vectors, maps) may fail with an exception,
// which must not leave a C function: it is reported as an error code instead.
int hipress_batch_create(hipress_batch** out, int32_t alg, const hipress_tensor* tensors, int32_t count,
                         const hipress_params* params) {
    try {
        return batch_create_impl(out, alg, tensors, count, params);
    } catch (...) {
        if (out) *out = nullptr;
        return HIPRESS_ERR_HIP;
    }
}

static Launch batch_launch(const hipress_batch* b, bool encode) {
    Launch L;
    std::memset(&L, 0, sizeof L);
    L.single = false;
    L.dsegs = encode ? b->d_enc : b->d_dec;
    L.dmap = b->d_map;
    L.dsmap = b->d_smap;
    L.dcmap = b->d_cmap;
    L.ntiles = b->ntiles;
    L.nstiles = b->nstiles;
    L.nctiles = b->nctiles;
    L.nsegs = (unsigned)(encode ? b->enc.size() : b->dec.size());
    L.expect_pairs = b->expect_pairs;
    return L;
}

static int batch_encode_impl(hipress_batch* b, int phase, void* stream, bool seeded = false, uint64_t seed = 0) {
    if (!b) return HIPRESS_ERR_NULL;
    if (!b->can_encode) return HIPRESS_ERR_NULL;
    if (seeded != b->drawn) return HIPRESS_ERR_PARAM;  // a seed goes with a batch without noise tensors, and only with it
    if (b->enc.empty()) return HIPRESS_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    Launch L = batch_launch(b, true);
    switch (b->alg) {
        case HIPRESS_ONEBIT:
            if (phase > 2) return HIPRESS_ERR_PARAM;
            return hiperr(launch_onebit_encode(L, static_cast<float*>(b->ws), phase, st));
        case HIPRESS_ONEBIT_DEFERRED:
            if (phase > 1) return HIPRESS_ERR_PARAM;
            return hiperr(launch_onebit_encode_deferred(L, static_cast<float*>(b->ws), phase, st));
        case HIPRESS_TBQ:
            if (phase > 0) return HIPRESS_ERR_PARAM;
            return hiperr(launch_tbq_encode(L, st));
        case HIPRESS_TERNGRAD:
            if (phase > 0) return HIPRESS_ERR_PARAM;
            return hiperr(launch_terngrad_encode(L, (unsigned)b->params.bucket, b->drawn, b->drawn ? uniform_key(seed) : 0u, st));
        case HIPRESS_DGC:
        case HIPRESS_GRADDROP:
            if (phase > 6) return HIPRESS_ERR_PARAM;
            return hiperr(launch_sparse_encode(L, b->alg == HIPRESS_DGC, sparse_ws_at(b->ws, b->swl), phase, st));
    }
    return HIPRESS_ERR_PARAM;
}

int hipress_batch_encode(hipress_batch* b, void* stream) { return batch_encode_impl(b, -1, stream); }

int hipress_batch_encode_seeded(hipress_batch* b, uint64_t seed, void* stream) {
    return batch_encode_impl(b, -1, stream, true, seed);
}

int hipress_batch_encode_phase(hipress_batch* b, int32_t phase, void* stream) {
    if (phase < 0) return HIPRESS_ERR_PARAM;
    return batch_encode_impl(b, phase, stream);
}

int hipress_batch_decode(hipress_batch* b, void* stream) {
    if (!b) return HIPRESS_ERR_NULL;
    if (!b->can_decode) return HIPRESS_ERR_NULL;
    if (b->dec.empty()) return HIPRESS_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    Launch L = batch_launch(b, false);
    switch (b->alg) {
        case HIPRESS_ONEBIT:
        case HIPRESS_ONEBIT_DEFERRED: return hiperr(launch_onebit_decode(L, st));
        case HIPRESS_TBQ: return hiperr(launch_tbq_decode(L, st));
        case HIPRESS_TERNGRAD: return hiperr(launch_terngrad_decode(L, (unsigned)b->params.bucket, st));
        case HIPRESS_DGC:
        case HIPRESS_GRADDROP:
            if (++b->epoch == 0) b->epoch = 1;  // the flags start at 0, which no call uses
            return hiperr(launch_sparse_decode_indexed(L, b->d_tptr, b->d_disorder, b->epoch,
                                                       b->params.ratio * kTile <= 8.0, st));
    }
    return HIPRESS_ERR_PARAM;
}

// ---- merge batches ---------------------------------------------------------------------

int hipress_merge_batch_destroy(hipress_merge_batch* b) {
    if (!b) return HIPRESS_OK;
    (void)hipFree(b->d_segs);
    (void)hipFree(b->iws);
    (void)hipFree(b->tgflags);
    (void)hipFree(b->d_renc);
    (void)hipFree(b->d_map);
    (void)hipFree(b->d_smap);
    (void)hipFree(b->ws);
    delete b;
    return HIPRESS_OK;
}

static int merge_batch_create_impl(hipress_merge_batch** out, int32_t alg, const hipress_merge_chunk* chunks,
                                   int32_t count, int32_t npeers, const hipress_params* params) {
    if (!out || !params || (count > 0 && !chunks)) return HIPRESS_ERR_NULL;
    *out = nullptr;
    if (count < 0) return HIPRESS_ERR_SIZE;
    if (alg < HIPRESS_ONEBIT || alg > HIPRESS_GRADDROP) return HIPRESS_ERR_PARAM;
    if (npeers < 1 || npeers > HIPRESS_MAX_PEERS) return HIPRESS_ERR_PARAM;
    hipress_merge_batch* b = new (std::nothrow) hipress_merge_batch;
    if (!b) return HIPRESS_ERR_HIP;
    b->alg = alg;
    b->params = *params;
    b->npeers = npeers;
    const bool sparse = alg == HIPRESS_DGC || alg == HIPRESS_GRADDROP;
    struct Guard {  // frees the half-built batch on every way out but the last
        hipress_merge_batch* b;
        ~Guard() { hipress_merge_batch_destroy(b); }
    } guard{b};
    auto fail = [](int code) { return code; };
    int rc;
    bool any_state = false, all_state = true;
    for (int i = 0; i < count; ++i) {
        if (wants_reencode(chunks[i].state, chunks[i].out_payload, chunks[i].n)) any_state = true;
        else all_state = false;
    }
    if (any_state && !all_state) return fail(HIPRESS_ERR_NULL);  // re-encode is all chunks or none
    if (any_state && (alg == HIPRESS_ONEBIT || alg == HIPRESS_TERNGRAD)) return fail(HIPRESS_ERR_PARAM);
    b->reencode = any_state;
    for (int i = 0; i < count; ++i) {
        const hipress_merge_chunk& c = chunks[i];
        MergeSeg m;
        if ((rc = build_merge_seg(alg, c.payloads, c.payload_bytes, npeers, c.local, c.aggregate, c.n, b->reencode, &m))) return fail(rc);
        // terngrad: the bucket size the peers are expected to have used lets the kernel ask for their
        // words before it has seen their headers (which still decide when they say otherwise)
        if (alg == HIPRESS_TERNGRAD && params->bucket >= 1) m.s.bucket = (unsigned)params->bucket;
        if (b->reencode && alg == HIPRESS_TBQ) {
            if ((rc = add_tbq_reencode(&m, c.state, c.out_payload, c.out_payload_bytes, params->threshold))) return fail(rc);
        }
        if (b->reencode && sparse) {
            hipress_tensor t{c.aggregate ? c.aggregate : c.state, c.state, nullptr, nullptr, c.out_payload, nullptr, c.n, c.out_payload_bytes};
            Seg s;
            if ((rc = build_encode_seg(HIPRESS_GRADDROP, t, *params, &s))) return fail(rc);
            b->renc.push_back(s);
        }
        b->aggregate = b->aggregate || m.s.out != nullptr;
        b->local = b->local || m.s.g != nullptr;
        b->segs.push_back(m);
    }
    std::vector<uint2> map;
    if ((rc = layout_tiles(b->segs, [](MergeSeg& m) -> Seg& { return m.s; }, map, &b->ntiles))) return fail(rc);
    if (!b->renc.empty()) {
        std::vector<uint2> map2;
        unsigned nt2;
        if ((rc = layout_tiles(b->renc, [](Seg& s) -> Seg& { return s; }, map2, &nt2))) return fail(rc);
        std::vector<uint2> smap;
        int64_t total_ns = layout_samples(b->renc, smap);
        for (const Seg& s : b->renc) b->expect_pairs += expected_pairs(s);
        b->nstiles = (unsigned)smap.size();
        b->swl = sparse_ws_layout(total_ns, b->ntiles, count);
        if (b->swl.bytes && hipMalloc(&b->ws, (size_t)b->swl.bytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        if ((rc = upload(smap, &b->d_smap))) return fail(rc);
        for (size_t i = 0; i < b->segs.size(); ++i) b->segs[i].r = b->renc[i];  // the merge kernel runs their first launch
    }
    if (sparse) {
        const size_t ibytes = (size_t)merge_index_bytes(b->ntiles ? b->ntiles : 1, npeers);
        if (hipMalloc(&b->iws, ibytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        if (hipMemset(b->iws, 0, ibytes) != hipSuccess) return fail(HIPRESS_ERR_HIP);
        for (const MergeSeg& m : b->segs)
            for (int p = 0; p < npeers; ++p) b->slices = std::max(b->slices, slices_of(m.peer_slots[p]));
    }
    if (alg == HIPRESS_TERNGRAD && params->bucket >= 1 && !b->segs.empty()) {
        // the lean merge kernels (every descriptor names this bucket size): one flag per chunk, written by every run
        if (hipMalloc(reinterpret_cast<void**>(&b->tgflags), 4 * b->segs.size()) != hipSuccess) return fail(HIPRESS_ERR_HIP);
    }
    if ((rc = upload(b->segs, &b->d_segs))) return fail(rc);
    if ((rc = upload(b->renc, &b->d_renc))) return fail(rc);
    if ((rc = upload(map, &b->d_map))) return fail(rc);
    guard.b = nullptr;
    *out = b;
    return HIPRESS_OK;
}

int hipress_merge_batch_create(hipress_merge_batch** out, int32_t alg, const hipress_merge_chunk* chunks,
                               int32_t count, int32_t npeers, const hipress_params* params) {
    try {
        return merge_batch_create_impl(out, alg, chunks, count, npeers, params);
    } catch (...) {
        if (out) *out = nullptr;
        return HIPRESS_ERR_HIP;
    }
}

// phase < 0: everything.  Sparse: 0 index, 1 merge (+ accumulate of the re-encode),
// 2 the remaining re-encode launches.  Dense: 0.
static int merge_batch_run_impl(hipress_merge_batch* b, int phase, void* stream) {
    if (!b) return HIPRESS_ERR_NULL;
    if (b->segs.empty()) return HIPRESS_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    MergeLaunch L;
    std::memset(&L, 0, sizeof L);
    L.single = false;
    L.dsegs = b->d_segs;
    L.dmap = b->d_map;
    L.ntiles = b->ntiles;
    L.nsegs = (unsigned)b->segs.size();
    L.npeers = b->npeers;
    L.reencode = b->reencode;
    L.aggregate = b->aggregate;
    L.local = b->local;
    L.tgflags = b->tgflags;
    L.bucket256 = b->params.bucket >= 256 && b->params.bucket % 256 == 0;
    if (b->alg == HIPRESS_DGC || b->alg == HIPRESS_GRADDROP) {
        if (phase > 2) return HIPRESS_ERR_PARAM;
        PeerRun* runs = static_cast<PeerRun*>(b->iws);
        SparseWs ws{};
        if (b->reencode) ws = sparse_ws_at(b->ws, b->swl);
        hipError_t e = hipSuccess;
        // the index and the merge launch of one run share an epoch, also when a caller asks for them one by one
        if (phase <= 0) b->cur_epoch = next_epoch(b->epoch);
        if (phase < 0 || phase < 2) e = launch_sparse_merge(L, ws, runs, b->slices, b->cur_epoch, phase, st);
        if (e != hipSuccess) return HIPRESS_ERR_HIP;
        if (b->reencode && (phase < 0 || phase == 2)) {
            Launch R;
            std::memset(&R, 0, sizeof R);
            R.single = false;
            R.dsegs = b->d_renc;
            R.dmap = b->d_map;  // same tensors, same tile numbering
            R.dsmap = b->d_smap;
            R.nstiles = b->nstiles;
            R.ntiles = b->ntiles;
            R.nsegs = (unsigned)b->renc.size();
            R.expect_pairs = b->expect_pairs;
            e = launch_sparse_encode(R, false, ws, kSparseAfterAccum, st);
        }
        return hiperr(e);
    }
    if (phase > 0) return HIPRESS_ERR_PARAM;
    return hiperr(launch_dense_merge(L, b->alg, st));
}

int hipress_merge_batch_run(hipress_merge_batch* b, void* stream) { return merge_batch_run_impl(b, -1, stream); }

int hipress_merge_batch_run_phase(hipress_merge_batch* b, int32_t phase, void* stream) {
    if (phase < 0) return HIPRESS_ERR_PARAM;
    return merge_batch_run_impl(b, phase, stream);
}

}  // extern "C"
