/*
 * CPU oracle for the HiPress gradient-compression hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may link, import or
 * call this file: it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have a scalar, obviously-sequential statement of every
 * operator to compare the HIP kernels with.
 *
 * Provenance of the arithmetic.  The reference checkout carries source for one
 * compressor only, the CompLL-generated min/max stochastic quantiser
 *   /root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode_body.h:99-126
 *   /root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode_body.h:48-74
 * and names the five built-in algorithms (onebit, TBQ, TernGrad, DGC, GradDrop,
 * /root/reference/README.md:9) whose operator sources live in submodules that
 * are empty directories here (/root/reference/.gitmodules:1-12:
 * torch-hipress-extension, hipress-mxnet, tensorflow-ops, CCO; no pinned
 * revision is recoverable).  What the checkout does fix, and what every
 * function below follows, is
 *   - the bit-placement rule for packed codes: code i of width b sits at bit
 *     (i mod 8/b)*b of byte floor(i*b/8), i.e. least-significant first
 *     (TernGradDecode_body.h:44).  hpo_get_code()/hpo_put_code() restate it on
 *     little-endian uint32 words, which is the same byte image;
 *   - header-then-codes payloads sized by the caller
 *     (TernGradEncode_body.h:114,120-123);
 *   - in-place operators over caller-allocated buffers, encode
 *     (gradient, compressed, params), decode (compressed, gradient)
 *     (TernGradEncode.cc:10-24, TernGradDecode.cc:10-24).
 * The arithmetic of the five built-in compressors and of the decode-and-merge
 * step is restated from their published algorithms (1-bit SGD, threshold
 * two-bit quantisation, TernGrad, Deep Gradient Compression, Gradient
 * Dropping) with the choices listed beside each function.
 *
 * PARITY STATUS.  The reference holds no test, golden vector or fixture for
 * this path, and the operator sources are absent, so with respect to the
 * reference's numbers every function here except the bit-placement helpers is
 * "parity unpinned".  They are pinned instead by hand-worked known answers,
 * closed forms, invariants and brute force in tests/test_oracle_*.py.
 * hpo_get_code/hpo_put_code, hpo_compll_decode and hpo_lcg_uniform are pinned
 * against the reference text (TernGradDecode_body.h:44,65-72;
 * naive_random.hpp:40-68); hpo_compll_encode follows the DSL source of the
 * in-tree operator and is pinned by its header layout, grid-point round trips
 * through hpo_compll_decode and a float64 closed form.
 *
 * Build: gcc -O3 -ffp-contract=off -fno-fast-math (see oracle/Makefile).  All
 * arithmetic is IEEE binary32 round-to-nearest with no contraction.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define HPO_HEADER_BYTES 16

/* The same source builds the all-cores variant of the CPU baseline (-fopenmp
 * -DHPO_OMP, libhipress_oracle_omp.so).  Loops whose iterations are independent
 * are shared between the cores: the quantisers run one packed word (or one bucket
 * of whole words, or one byte) per iteration so that iterations never share a
 * word, element-wise loops run as they are, counts are reductions.  What depends
 * on order stays sequential in both builds: the radix selection of a threshold and
 * the walk that emits the selected pairs in ascending index order.  Without
 * HPO_OMP the pragmas vanish and every loop is sequential. */
#ifdef HPO_OMP
#define HPO_PRAGMA(x) _Pragma(#x)
#define HPO_PARALLEL_FOR HPO_PRAGMA(omp parallel for schedule(static))
#define HPO_PARALLEL_FOR_IF(c) HPO_PRAGMA(omp parallel for schedule(static) if (c))
#define HPO_PARALLEL_SUM(v) HPO_PRAGMA(omp parallel for schedule(static) reduction(+ : v))
#define HPO_PARALLEL_MINMAX(a, b) HPO_PRAGMA(omp parallel for schedule(static) reduction(max : a) reduction(min : b))
int hpo_threads(void);
#else
#define HPO_PARALLEL_FOR
#define HPO_PARALLEL_FOR_IF(c)
#define HPO_PARALLEL_SUM(v)
#define HPO_PARALLEL_MINMAX(a, b)
#endif

/* ------------------------------------------------------------------ */
/* wire rule                                                          */
/* ------------------------------------------------------------------ */

/* Code i of width b: bits [b*(i mod 32/b), +b) of little-endian word
 * floor(i*b/32).  Same byte image as TernGradDecode_body.h:44
 * (byte floor(i*b/8), shift (i mod 8/b)*b). */
uint32_t hpo_get_code(const uint32_t *words, int64_t i, int b)
{
    int per = 32 / b;
    return (words[i / per] >> ((i % per) * b)) & ((1u << b) - 1u);
}

void hpo_put_code(uint32_t *words, int64_t i, int b, uint32_t code)
{
    int per = 32 / b;
    uint32_t mask = ((1u << b) - 1u) << ((i % per) * b);
    words[i / per] = (words[i / per] & ~mask) | ((code << ((i % per) * b)) & mask);
}

static int64_t words_for(int64_t n, int b)
{
    int per = 32 / b;
    return (n + per - 1) / per;
}

static int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

/* ------------------------------------------------------------------ */
/* payload sizes                                                      */
/* ------------------------------------------------------------------ */

int64_t hpo_onebit_payload_bytes(int64_t n) { return HPO_HEADER_BYTES + 4 * words_for(n, 1); }
int64_t hpo_tbq_payload_bytes(int64_t n) { return HPO_HEADER_BYTES + 4 * words_for(n, 2); }

int64_t hpo_terngrad_scale_bytes(int64_t n, int64_t bucket)
{
    int64_t nb = (n + bucket - 1) / bucket;
    return round_up(4 * nb, 16);
}

int64_t hpo_terngrad_payload_bytes(int64_t n, int64_t bucket)
{
    return HPO_HEADER_BYTES + hpo_terngrad_scale_bytes(n, bucket) + 4 * words_for(n, 2);
}

/* Slots reserved for (index, value) pairs: four times the expected count,
 * never fewer than 64 and never more than n, rounded up to a multiple of 64. */
int64_t hpo_sparse_capacity(int64_t n, double ratio)
{
    int64_t want = (int64_t)ceil(4.0 * ratio * (double)n);
    if (want > n) want = n;
    if (want < 64) want = 64;
    return round_up(want, 64);
}

int64_t hpo_sparse_payload_bytes(int64_t n, double ratio)
{
    return HPO_HEADER_BYTES + 8 * hpo_sparse_capacity(n, ratio);
}

/* ------------------------------------------------------------------ */
/* TBQ: threshold two-bit quantisation with error feedback            */
/* ------------------------------------------------------------------ */

/* v = r + g; v >= tau -> code 1, r' = v - tau; v <= -tau -> code 2,
 * r' = v + tau; otherwise code 0, r' = v.  NaN compares false -> code 0.
 * Payload: {f32 tau, u32 n, 0, 0} then ceil(n/16) words, pad codes 0. */
void hpo_tbq_encode(const float *g, float *r, int64_t n, uint8_t *payload, float tau)
{
    uint32_t *hdr = (uint32_t *)payload;
    uint32_t *w = (uint32_t *)(payload + HPO_HEADER_BYTES);
    int64_t nw = words_for(n, 2);
    memcpy(&hdr[0], &tau, 4);
    hdr[1] = (uint32_t)n;
    hdr[2] = 0;
    hdr[3] = 0;
    /* one word (16 codes) at a time, so that the OpenMP build can share the loop */
    HPO_PARALLEL_FOR
    for (int64_t k = 0; k < nw; ++k) {
        int64_t hi = 16 * k + 16 < n ? 16 * k + 16 : n;
        w[k] = 0;
        for (int64_t i = 16 * k; i < hi; ++i) {
            float v = r[i] + g[i];
            uint32_t code = 0;
            if (v >= tau) {
                code = 1;
                v = v - tau;
            } else if (v <= -tau) {
                code = 2;
                v = v + tau;
            }
            r[i] = v;
            hpo_put_code(w, i, 2, code);
        }
    }
}

static float tbq_value(uint32_t code, float tau)
{
    return code == 1 ? tau : (code == 2 ? -tau : 0.0f);
}

/* code 0 -> 0, 1 -> +tau, 2 -> -tau, 3 -> 0; tau comes from the header. */
void hpo_tbq_decode(const uint8_t *payload, float *out, int64_t n)
{
    float tau;
    const uint32_t *w = (const uint32_t *)(payload + HPO_HEADER_BYTES);
    memcpy(&tau, payload, 4);
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i)
        out[i] = tbq_value(hpo_get_code(w, i, 2), tau);
}

/* ------------------------------------------------------------------ */
/* onebit: sign quantisation, per-tensor mean-magnitude scale         */
/* ------------------------------------------------------------------ */

/* Scale s = (sum |r+g|) / n, accumulated in double and rounded once to
 * binary32 (any summation order is acceptable to within 1e-5 relative);
 * n = 0 gives 0. */
float hpo_onebit_scale(const float *g, const float *r, int64_t n)
{
    double acc = 0.0;
    HPO_PARALLEL_SUM(acc)
    for (int64_t i = 0; i < n; ++i) {
        float v = r[i] + g[i];
        acc += (double)fabsf(v);
    }
    return n > 0 ? (float)(acc / (double)n) : 0.0f;
}

/* Given the scale: bit = (v >= 0); d = bit ? +s : -s; r' = v - d.
 * Payload {f32 s, u32 n, 0, 0} then ceil(n/32) words, pad bits 0. */
void hpo_onebit_encode_with_scale(const float *g, float *r, int64_t n, uint8_t *payload, float s)
{
    uint32_t *hdr = (uint32_t *)payload;
    uint32_t *w = (uint32_t *)(payload + HPO_HEADER_BYTES);
    int64_t nw = words_for(n, 1);
    memcpy(&hdr[0], &s, 4);
    hdr[1] = (uint32_t)n;
    hdr[2] = 0;
    hdr[3] = 0;
    HPO_PARALLEL_FOR
    for (int64_t k = 0; k < nw; ++k) {
        int64_t hi = 32 * k + 32 < n ? 32 * k + 32 : n;
        w[k] = 0;
        for (int64_t i = 32 * k; i < hi; ++i) {
            float v = r[i] + g[i];
            uint32_t bit = v >= 0.0f ? 1u : 0u;
            float d = bit ? s : -s;
            r[i] = v - d;
            hpo_put_code(w, i, 1, bit);
        }
    }
}

void hpo_onebit_encode(const float *g, float *r, int64_t n, uint8_t *payload)
{
    hpo_onebit_encode_with_scale(g, r, n, payload, hpo_onebit_scale(g, r, n));
}

void hpo_onebit_decode(const uint8_t *payload, float *out, int64_t n)
{
    float s;
    const uint32_t *w = (const uint32_t *)(payload + HPO_HEADER_BYTES);
    memcpy(&s, payload, 4);
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i)
        out[i] = hpo_get_code(w, i, 1) ? s : -s;
}

/* ------------------------------------------------------------------ */
/* TernGrad: stochastic ternarisation, per-bucket max-abs scale       */
/* ------------------------------------------------------------------ */

/* Buckets of `bucket` consecutive elements over the flattened tensor (last
 * one may be short).  s_k = max |g_i| over bucket k (NaN never wins a
 * comparison).  Element i is kept iff u_i * s_k < |g_i| (one binary32
 * multiply), so P(keep) = |g_i| / s_k for u uniform on [0,1).
 * code = keep ? (g_i < 0 ? 2 : 1) : 0.  No residual.
 * Payload {u32 n, u32 bucket, 0, 0}, f32 scale[nb] padded to 16 B, words. */
void hpo_terngrad_encode(const float *g, const float *u, int64_t n, uint8_t *payload, int64_t bucket)
{
    uint32_t *hdr = (uint32_t *)payload;
    float *scale = (float *)(payload + HPO_HEADER_BYTES);
    int64_t sb = hpo_terngrad_scale_bytes(n, bucket);
    uint32_t *w = (uint32_t *)(payload + HPO_HEADER_BYTES + sb);
    int64_t nb = (n + bucket - 1) / bucket;
    hdr[0] = (uint32_t)n;
    hdr[1] = (uint32_t)bucket;
    hdr[2] = 0;
    hdr[3] = 0;
    memset(scale, 0, sb);
    memset(w, 0, 4 * words_for(n, 2));
    /* buckets of whole words (a multiple of 16 codes) never share a word */
    HPO_PARALLEL_FOR_IF(bucket % 16 == 0)
    for (int64_t k = 0; k < nb; ++k) {
        int64_t lo = k * bucket, hi = lo + bucket < n ? lo + bucket : n;
        float s = 0.0f;
        for (int64_t i = lo; i < hi; ++i) {
            float a = fabsf(g[i]);
            if (a > s) s = a;
        }
        scale[k] = s;
        for (int64_t i = lo; i < hi; ++i) {
            float a = fabsf(g[i]);
            float t = u[i] * s;
            uint32_t code = 0;
            if (t < a) code = g[i] < 0.0f ? 2u : 1u;
            hpo_put_code(w, i, 2, code);
        }
    }
}

void hpo_terngrad_decode(const uint8_t *payload, float *out, int64_t n)
{
    const uint32_t *hdr = (const uint32_t *)payload;
    int64_t bucket = hdr[1];
    const float *scale = (const float *)(payload + HPO_HEADER_BYTES);
    const uint32_t *w = (const uint32_t *)(payload + HPO_HEADER_BYTES + hpo_terngrad_scale_bytes(n, bucket));
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i) {
        float s = scale[i / bucket];
        out[i] = tbq_value(hpo_get_code(w, i, 2), s);
    }
}

/* ------------------------------------------------------------------ */
/* DGC / GradDrop: sampled-threshold top-k sparsification             */
/* ------------------------------------------------------------------ */

static uint32_t abs_key(float x)
{
    uint32_t k;
    memcpy(&k, &x, 4);
    return k & 0x7fffffffu; /* |x| as an order-preserving integer (NaN sorts above inf) */
}

static float key_value(uint32_t k)
{
    float x;
    memcpy(&x, &k, 4);
    return x;
}

/* k-th largest (k >= 1) of m unsigned keys by counting on 8-bit digits from
 * the top; the result is a value, so it does not depend on any ordering of
 * equal keys.  keys[] is overwritten. */
static uint32_t kth_largest(uint32_t *keys, int64_t m, int64_t k)
{
    uint32_t prefix = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        int64_t hist[256];
        int64_t kept = 0;
        int d;
        memset(hist, 0, sizeof hist);
        for (int64_t i = 0; i < m; ++i) hist[(keys[i] >> shift) & 255u]++;
        for (d = 255; d > 0; --d) {
            if (k <= hist[d]) break;
            k -= hist[d];
        }
        prefix |= (uint32_t)d << shift;
        for (int64_t i = 0; i < m; ++i)
            if (((keys[i] >> shift) & 255u) == (uint32_t)d) keys[kept++] = keys[i];
        m = kept;
    }
    return prefix;
}

/* Sample stride: every 100th element (a 1 % sample) once the tensor reaches
 * 262144 elements, the compression threshold the reference's launch lines use
 * (/root/reference/README.md:45); smaller tensors are their own sample. */
int64_t hpo_sparse_sample_stride(int64_t n) { return n >= 262144 ? 100 : 1; }

int64_t hpo_sparse_sample_count(int64_t n)
{
    int64_t S = hpo_sparse_sample_stride(n);
    return n / S;
}

int64_t hpo_sparse_sample_k(int64_t n, double ratio)
{
    int64_t ns = hpo_sparse_sample_count(n);
    int64_t k = (int64_t)ceil(ratio * (double)ns);
    if (k < 1) k = 1;
    if (k > ns) k = ns;
    return k;
}

/* Threshold = k_s-th largest |a| over sample positions j*S + S/2. */
float hpo_sparse_threshold(const float *a, int64_t n, double ratio)
{
    int64_t S = hpo_sparse_sample_stride(n);
    int64_t ns = n / S;
    uint32_t *keys;
    uint32_t t;
    if (ns <= 0) return 0.0f;
    keys = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)ns);
    for (int64_t j = 0; j < ns; ++j) keys[j] = abs_key(a[j * S + S / 2]);
    t = kth_largest(keys, ns, hpo_sparse_sample_k(n, ratio));
    free(keys);
    return key_value(t);
}

/* Select every i with |a_i| >= thr and |a_i| > 0, in ascending i.  If more
 * than `capacity` qualify, thr becomes the capacity-th largest |a| of the
 * whole tensor; everything above it is kept and elements equal to it are
 * kept in ascending index order until the slots are full.  Selected
 * positions are zeroed in a[] and, when given, in mom[] (momentum-factor
 * masking).  Payload {u32 nnz, u32 n, u32 capacity, f32 thr}, i32
 * idx[capacity], f32 val[capacity]; unused slots are left untouched. */
static void sparse_select(float *a, float *mom, int64_t n, uint8_t *payload, double ratio)
{
    uint32_t *hdr = (uint32_t *)payload;
    int64_t cap = hpo_sparse_capacity(n, ratio);
    int32_t *idx = (int32_t *)(payload + HPO_HEADER_BYTES);
    float *val = (float *)(payload + HPO_HEADER_BYTES + 4 * cap);
    float thr = hpo_sparse_threshold(a, n, ratio);
    uint32_t tk = abs_key(thr);
    int64_t count = 0, eq_quota = INT64_MAX, nnz = 0;

    HPO_PARALLEL_SUM(count)
    for (int64_t i = 0; i < n; ++i) {
        uint32_t k = abs_key(a[i]);
        if (k >= tk && k > 0) count++;
    }
    if (count > cap) {
        uint32_t *keys = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n);
        int64_t gt = 0;
        HPO_PARALLEL_FOR
        for (int64_t i = 0; i < n; ++i) keys[i] = abs_key(a[i]);
        tk = kth_largest(keys, n, cap);
        free(keys);
        thr = key_value(tk);
        HPO_PARALLEL_SUM(gt)
        for (int64_t i = 0; i < n; ++i)
            if (abs_key(a[i]) > tk) gt++;
        eq_quota = cap - gt;
    }
    for (int64_t i = 0; i < n; ++i) {
        uint32_t k = abs_key(a[i]);
        int take = 0;
        if (k == 0) continue;
        if (k > tk) take = 1;
        else if (k == tk && eq_quota > 0) {
            take = 1;
            eq_quota--;
        }
        if (take) {
            idx[nnz] = (int32_t)i;
            val[nnz] = a[i];
            nnz++;
            a[i] = 0.0f;
            if (mom) mom[i] = 0.0f;
        }
    }
    hdr[0] = (uint32_t)nnz;
    hdr[1] = (uint32_t)n;
    hdr[2] = (uint32_t)cap;
    memcpy(&hdr[3], &thr, 4);
}

/* DGC with momentum correction: mom' = m*mom + g (a multiply rounded to
 * binary32, then an add rounded to binary32), acc' = acc + mom', then
 * sampled-threshold selection on acc' with momentum-factor masking. */
void hpo_dgc_encode(const float *g, float *mom, float *acc, int64_t n, uint8_t *payload, float m,
                    double ratio)
{
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i) {
        float p = m * mom[i]; /* rounded product: the build disables contraction */
        float u = p + g[i];
        mom[i] = u;
        acc[i] = acc[i] + u;
    }
    sparse_select(acc, mom, n, payload, ratio);
}

/* GradDrop: acc' = acc + g, same selection, `ratio` is the kept fraction
 * (drop ratio 0.99 = ratio 0.01). */
void hpo_graddrop_encode(const float *g, float *acc, int64_t n, uint8_t *payload, double ratio)
{
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i) acc[i] = acc[i] + g[i];
    sparse_select(acc, NULL, n, payload, ratio);
}

/* Zero-fill then scatter; entries past n or past capacity are ignored. */
void hpo_sparse_decode(const uint8_t *payload, float *out, int64_t n)
{
    const uint32_t *hdr = (const uint32_t *)payload;
    int64_t nnz = hdr[0], cap = hdr[2];
    const int32_t *idx = (const int32_t *)(payload + HPO_HEADER_BYTES);
    const float *val = (const float *)(payload + HPO_HEADER_BYTES + 4 * cap);
    if (nnz > cap) nnz = cap;
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i) out[i] = 0.0f;
    for (int64_t j = 0; j < nnz; ++j)
        if (idx[j] >= 0 && idx[j] < n) out[idx[j]] = val[j];
}

/* ------------------------------------------------------------------ */
/* decode-and-merge                                                   */
/* ------------------------------------------------------------------ */

/* The aggregate starts from zero, or from the aggregator's own uncompressed
 * gradient `local` (a ring hop, a server that is also a worker); the peers are
 * then added to it in peer order.  agg may be the same buffer as local. */
static void merge_start(float *agg, const float *local, int64_t n)
{
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i) agg[i] = local ? local[i] : 0.0f;
}

/* agg[i] = ((start + d_1[i]) + d_2[i]) + ... in peer order, binary32, start = 0
 * or local[i].  If r is not NULL the aggregate is re-encoded for the next hop
 * with the aggregator's own residual r and threshold tau into out_payload. */
void hpo_tbq_decode_merge_local(const uint8_t *const *payloads, int npeers, const float *local, float *agg,
                                int64_t n, float *r, uint8_t *out_payload, float tau)
{
    merge_start(agg, local, n);
    for (int p = 0; p < npeers; ++p) {
        float t;
        const uint32_t *w = (const uint32_t *)(payloads[p] + HPO_HEADER_BYTES);
        memcpy(&t, payloads[p], 4);
        HPO_PARALLEL_FOR
        for (int64_t i = 0; i < n; ++i) agg[i] = agg[i] + tbq_value(hpo_get_code(w, i, 2), t);
    }
    if (r) hpo_tbq_encode(agg, r, n, out_payload, tau);
}

void hpo_tbq_decode_merge(const uint8_t *const *payloads, int npeers, float *agg, int64_t n, float *r,
                          uint8_t *out_payload, float tau)
{
    hpo_tbq_decode_merge_local(payloads, npeers, NULL, agg, n, r, out_payload, tau);
}

void hpo_onebit_decode_merge_local(const uint8_t *const *payloads, int npeers, const float *local, float *agg,
                                   int64_t n)
{
    merge_start(agg, local, n);
    for (int p = 0; p < npeers; ++p) {
        float s;
        const uint32_t *w = (const uint32_t *)(payloads[p] + HPO_HEADER_BYTES);
        memcpy(&s, payloads[p], 4);
        HPO_PARALLEL_FOR
        for (int64_t i = 0; i < n; ++i) agg[i] = agg[i] + (hpo_get_code(w, i, 1) ? s : -s);
    }
}

void hpo_onebit_decode_merge(const uint8_t *const *payloads, int npeers, float *agg, int64_t n)
{
    hpo_onebit_decode_merge_local(payloads, npeers, NULL, agg, n);
}

void hpo_terngrad_decode_merge_local(const uint8_t *const *payloads, int npeers, const float *local, float *agg,
                                     int64_t n)
{
    merge_start(agg, local, n);
    for (int p = 0; p < npeers; ++p) {
        const uint32_t *hdr = (const uint32_t *)payloads[p];
        int64_t bucket = hdr[1];
        const float *scale = (const float *)(payloads[p] + HPO_HEADER_BYTES);
        const uint32_t *w =
            (const uint32_t *)(payloads[p] + HPO_HEADER_BYTES + hpo_terngrad_scale_bytes(n, bucket));
        HPO_PARALLEL_FOR
        for (int64_t i = 0; i < n; ++i)
            agg[i] = agg[i] + tbq_value(hpo_get_code(w, i, 2), scale[i / bucket]);
    }
}

void hpo_terngrad_decode_merge(const uint8_t *const *payloads, int npeers, float *agg, int64_t n)
{
    hpo_terngrad_decode_merge_local(payloads, npeers, NULL, agg, n);
}

/* Start from zero or from `local`, then scatter-ADD every peer's pairs in peer
 * order and slot order (duplicates across peers sum).  If acc is not NULL the
 * aggregate is re-sparsified for the next hop GradDrop-style with the
 * aggregator's residual acc: acc' = acc + agg, select, zero. */
void hpo_sparse_decode_merge_local(const uint8_t *const *payloads, int npeers, const float *local, float *agg,
                                   int64_t n, float *acc, uint8_t *out_payload, double ratio)
{
    merge_start(agg, local, n);
    for (int p = 0; p < npeers; ++p) {
        const uint32_t *hdr = (const uint32_t *)payloads[p];
        int64_t nnz = hdr[0], cap = hdr[2];
        const int32_t *idx = (const int32_t *)(payloads[p] + HPO_HEADER_BYTES);
        const float *val = (const float *)(payloads[p] + HPO_HEADER_BYTES + 4 * cap);
        if (nnz > cap) nnz = cap;
        for (int64_t j = 0; j < nnz; ++j)
            if (idx[j] >= 0 && idx[j] < n) agg[idx[j]] = agg[idx[j]] + val[j];
    }
    if (acc) hpo_graddrop_encode(agg, acc, n, out_payload, ratio);
}

void hpo_sparse_decode_merge(const uint8_t *const *payloads, int npeers, float *agg, int64_t n,
                             float *acc, uint8_t *out_payload, double ratio)
{
    hpo_sparse_decode_merge_local(payloads, npeers, NULL, agg, n, acc, out_payload, ratio);
}

/* ------------------------------------------------------------------ */
/* CompLL generated-operator wire format (10-byte header)             */
/* ------------------------------------------------------------------ */

/* Decode of the in-tree generated operator, as written
 * (TernGradDecode_body.h:48-74): header [bitwidth:u8][tail:u8][min:f32]
 * [max:f32] at byte offsets 0,1,2,6, codes from byte 10;
 * gap = (max-min)/((1<<b)-1); count = (8*csz - 80)/b - tail;
 * out[i] = code_i*gap + min with code_i at bit (i mod 8/b)*b of byte
 * floor(i*b/8).  Returns the element count written (at most out_cap). */
int64_t hpo_compll_decode(const uint8_t *compressed, int64_t csz, float *out, int64_t out_cap)
{
    uint8_t b = compressed[0], tail = compressed[1];
    float mn, mx, gap;
    const uint8_t *Q = compressed + 10;
    int64_t count;
    memcpy(&mn, compressed + 2, 4);
    memcpy(&mx, compressed + 6, 4);
    gap = (mx - mn) / (float)((1 << b) - 1);
    count = (8 * csz - 80) / b - tail;
    if (count > out_cap) count = out_cap;
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < count; ++i) {
        uint32_t code = (Q[i * b / 8] >> ((i % (8 / b)) * b)) & ((1u << b) - 1u);
        out[i] = (float)code * gap + mn;
    }
    return count < 0 ? 0 : count;
}

/* Encode of the in-tree CompLL operator as its DSL source states it
 * (/root/reference/src/CompLL/GCGen/pse/TernGradEncode.pse:22-33), not as the
 * generator mis-translated it (the generated functor walks output bytes as if
 * they were element indices and shifts codes in from the wrong end,
 * TernGradEncode_body.h:48-59):
 *   max = reduce(g, -99999, greater), min = reduce(g, 99999, smaller) in float;
 *   gap = (max - min) / ((1<<b) - 1);  tail = n % (1<<b) kept as uint8;
 *   code_i = floor((g_i - min) / gap + u_i), u_i an explicit uniform[0,1) draw in
 *   place of random<float>(0,1), limited to [0, 2^b - 1]; gap == 0 gives code 0, and so
 *   does a value that is no number (a NaN gradient, or Inf/Inf when the range is infinite);
 *   code i is stored where the decoder reads it: bit (i mod 8/b)*b of byte
 *   floor(i*b/8) after the 10-byte header [b][tail][min][max]
 *   (TernGradEncode_body.h:114,120-123; TernGradDecode_body.h:44).
 * b must divide 8.  Returns the payload length 10 + ceil(n*b/8). */
int64_t hpo_compll_payload_bytes(int64_t n, int b) { return 10 + (n * b + 7) / 8; }

int64_t hpo_compll_encode(const float *g, const float *u, int64_t n, uint8_t *compressed, int b)
{
    float mx = -99999.0f, mn = 99999.0f, gap;
    int64_t nbytes = (n * b + 7) / 8;
    uint8_t *Q = compressed + 10;
    uint8_t tail = (uint8_t)(n % (1 << b));
    uint32_t top = (1u << b) - 1u;
    int per = 8 / b;
    HPO_PARALLEL_MINMAX(mx, mn)
    for (int64_t i = 0; i < n; ++i) {
        if (g[i] > mx) mx = g[i];
        if (g[i] < mn) mn = g[i];
    }
    gap = (mx - mn) / (float)top;
    compressed[0] = (uint8_t)b;
    compressed[1] = tail;
    memcpy(compressed + 2, &mn, 4);
    memcpy(compressed + 6, &mx, 4);
    /* one output byte (8/b codes) per iteration, so that iterations never share a byte */
    HPO_PARALLEL_FOR
    for (int64_t k = 0; k < nbytes; ++k) {
        int64_t hi = (k + 1) * per < n ? (k + 1) * per : n;
        uint8_t q = 0;
        for (int64_t i = k * per; i < hi; ++i) {
            uint32_t code = 0;
            if (gap > 0.0f) {
                float r = (g[i] - mn) / gap + u[i];
                float f = floorf(r);
                code = !(f > 0.0f) ? 0u : (f >= (float)top ? top : (uint32_t)f); /* NaN -> 0 */
            }
            q |= (uint8_t)(code << ((i % per) * b));
        }
        Q[k] = q;
    }
    return 10 + nbytes;
}

/* The reference's generator for its rounding noise
 * (/root/reference/src/CompLL/GCGen/output/naive_random.hpp:40-68): a 32-bit
 * linear congruential sequence x <- 1103515245*x + 12345, mapped to [lo, hi] by
 * float(x / (4294967295.0 / (hi - lo))) + lo (the division in double).  Fills
 * out[0..n) with consecutive draws starting from `seed`. */
void hpo_lcg_uniform(uint32_t seed, float lo, float hi, float *out, int64_t n)
{
    uint32_t x = seed;
    double scale = 4294967295.0 / (double)(hi - lo);
    for (int64_t i = 0; i < n; ++i) {
        x = 1103515245u * x + 12345u;
        out[i] = (float)((double)x / scale) + lo;
    }
}

/* The noise the encoders draw themselves when they are called with a seed instead of a
 * noise tensor (include/hipress_amd.h, hipress_terngrad_encode_seeded).  A definition of
 * this library's own, with no counterpart in the reference, whose generator is seeded from
 * the clock (TernGradEncode_body.h:119): element i of tensor t takes the top 24 bits of
 * h(i xor k) as a fraction, h being the 32-bit mixer "triple32" (xor-shift 17, times
 * 0xed5ad4bb, xor-shift 11, times 0xac4c1b51, xor-shift 15, times 0x31848bab, xor-shift 14)
 * and k = h(fold(seed) +
 * t * 0x9e3779b9), where fold xors the two halves of the SplitMix64 output function
 * applied to seed + 0x9e3779b97f4a7c15.  Pinned by tests/test_uniform_draw.py: the
 * published first SplitMix64 output, an independent big-integer restatement, and the
 * header the kernels compile, built for the host. */
static uint32_t hpo_triple32(uint32_t x)
{
    x = x ^ (x >> 17);
    x = x * 0xed5ad4bbU;
    x = x ^ (x >> 11);
    x = x * 0xac4c1b51U;
    x = x ^ (x >> 15);
    x = x * 0x31848babU;
    x = x ^ (x >> 14);
    return x;
}

uint32_t hpo_uniform_tensor_key(uint64_t seed, uint32_t tensor)
{
    uint64_t z = seed + 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    z = z ^ (z >> 31);
    uint32_t folded = (uint32_t)(z & 0xffffffffULL) ^ (uint32_t)(z >> 32);
    return hpo_triple32(folded + tensor * 0x9e3779b9U);
}

void hpo_uniform_draws(uint64_t seed, uint32_t tensor, float *out, int64_t n)
{
    const uint32_t k = hpo_uniform_tensor_key(seed, tensor);
    HPO_PARALLEL_FOR
    for (int64_t i = 0; i < n; ++i)
        out[i] = (float)(hpo_triple32((uint32_t)i ^ k) >> 8) / 16777216.0f;
}

/* Threads the all-cores build runs its parallel loops on (1 for the plain build). */
#ifdef HPO_OMP
#include <omp.h>
int hpo_threads(void) { return omp_get_max_threads(); }
#else
int hpo_threads(void) { return 1; }
#endif
