/*
 * hipress_amd — C ABI of the MI355X (gfx950) gradient-compression operators.
 *
 * One shared library, libhipress_amd.so, exports everything declared here with
 * C linkage.  All pointers named grad/residual/momentum/accumulator/uniform/
 * payload/out/aggregate/workspace are DEVICE pointers owned by the caller (fp32
 * arrays 4-byte aligned - a view a few floats into a flat buffer runs on the same
 * 16-byte vector path as the buffer itself; payloads and workspaces 16-byte aligned);
 * `stream` is a hipStream_t passed as void* (NULL = the default stream), the
 * way the reference carries its stream
 * (/root/reference/src/CompLL/GCGen/output/get_policy_general.h:125-133,
 *  /root/reference/src/CompLL/GCGen/output/get_stream_mxnet.h:19-25).
 * Every call only enqueues work on `stream` and returns; nothing here
 * synchronises with the host or allocates device memory, except
 * hipress_batch_create / hipress_merge_batch_create (set-up time) and their
 * destroy calls.  Like the reference's bodies, the library starts no threads and keeps
 * no state between calls beyond what the caller passes in (two atomic counters and
 * the array of hipress_onebit_encode_static aside): calls from different host
 * threads may overlap as long as their buffers, workspaces and batch objects are
 * distinct.
 *
 * The per-tensor entry points replace the reference's generated operator body
 *   void <Func>_body<policy_t>(float* gradient, int32 _gradient_size,
 *                              uint8* compressed, int32 _compressed_size,
 *                              <scalars>, policy_t policy, void* stream)
 * (/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode_body.h:99-109,
 *  /root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode_body.h:48-57)
 * which the framework wrappers call with raw pointers and element counts
 * (TernGradEncode_wrapper.h:42-70, TernGradDecode_wrapper.h:40-67): encode takes
 * (gradient, [state...], compressed, scalars), decode takes (compressed,
 * gradient); both buffers are caller-allocated and updated in place
 * (TernGradEncode.cc:10-24, TernGradDecode.cc:10-24).  Differences: sizes are
 * int64, error-feedback state buffers are explicit arguments, and errors come
 * back as negative return codes instead of a fatal CHECK.
 *
 * Payload layout (all little-endian, payload base 16-byte aligned):
 *   16-byte header, then dense uint32 words.  Code i of width b occupies bits
 *   [b*(i mod 32/b), +b) of word floor(i*b/32) — the byte image the reference
 *   decoder reads (TernGradDecode_body.h:44).  Pad codes are 0.
 *     onebit   {f32 scale, u32 n, 0, 0}            words: ceil(n/32)
 *     tbq      {f32 tau,   u32 n, 0, 0}            words: ceil(n/16)
 *     terngrad {u32 n, u32 bucket, 0, 0} f32 scale[ceil(n/bucket)] (padded to
 *              16 B) then words: ceil(n/16)
 *     dgc/graddrop {u32 nnz, u32 n, u32 capacity, f32 thr} i32 idx[capacity]
 *              f32 val[capacity]; pairs are in ascending index order
 *   2-bit codes: 0 -> 0, 1 -> +scale, 2 -> -scale, 3 -> 0 (never produced).
 */
#ifndef HIPRESS_AMD_H_
#define HIPRESS_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPRESS_OK 0
#define HIPRESS_ERR_NULL (-1)      /* a required pointer is NULL */
#define HIPRESS_ERR_SIZE (-2)      /* n out of range, or a buffer is too small */
#define HIPRESS_ERR_ALIGN (-3)     /* pointer not aligned (fp32: 4 B, payload/workspace: 16 B) */
#define HIPRESS_ERR_PARAM (-4)     /* scalar parameter out of range */
#define HIPRESS_ERR_HIP (-5)       /* the HIP runtime reported an error */
#define HIPRESS_ERR_WORKSPACE (-6) /* workspace missing or too small */

#define HIPRESS_HEADER_BYTES 16
#define HIPRESS_MAX_PEERS 16
#define HIPRESS_MAX_N 4294967295LL /* n is carried as u32 in payload headers */
/* DGC, GradDrop, hipress_sparse_decode and hipress_sparse_decode_merge (and batches of
 * them) carry element indices as int32 in the payload: a larger n is HIPRESS_ERR_SIZE. */
#define HIPRESS_SPARSE_MAX_N 2147483647LL

enum hipress_alg {
    HIPRESS_ONEBIT = 0,
    HIPRESS_TBQ = 1,
    HIPRESS_TERNGRAD = 2,
    HIPRESS_DGC = 3,
    HIPRESS_GRADDROP = 4,
    HIPRESS_ONEBIT_DEFERRED = 5 /* batches only: state0 = state, state1 = one-word scale state */
};

int hipress_version(void);
const char *hipress_strerror(int code);

/* ---- sizes (host-only arithmetic; negative return = error code) ---------- */
int64_t hipress_onebit_payload_bytes(int64_t n);
int64_t hipress_tbq_payload_bytes(int64_t n);
int64_t hipress_terngrad_payload_bytes(int64_t n, int32_t bucket);
int64_t hipress_sparse_capacity(int64_t n, double ratio);
int64_t hipress_sparse_payload_bytes(int64_t n, double ratio);
int64_t hipress_onebit_workspace_bytes(int64_t n);
int64_t hipress_sparse_workspace_bytes(int64_t n, double ratio);
int64_t hipress_sparse_merge_workspace_bytes(int64_t n, int32_t npeers, double ratio, int32_t reencode);

/* ---- TBQ: threshold two-bit quantisation with error feedback ------------- */
/* Replaces <Func>_body for the built-in "tbq" algorithm
 * (/root/reference/README.md:9,45).  residual is read and overwritten. */
int hipress_tbq_encode(const float *grad, float *residual, int64_t n, void *payload,
                       int64_t payload_bytes, float threshold, void *stream);
int hipress_tbq_decode(const void *payload, int64_t payload_bytes, float *out, int64_t n,
                       void *stream);

/* ---- onebit: sign bits, per-tensor mean-magnitude scale, error feedback --- */
/* Replaces <Func>_body for "onebit" (/root/reference/README.md:9).  Where the
 * reference body blocks the host on each thrust::reduce result
 * (TernGradEncode_body.h:115-116), the scale here stays on the device.  The scale is
 * mean|r + g|, summed per 4096-element tile in fp32 (fixed order: the same bits on
 * every run) and over the tiles in fp64; a tile whose magnitudes sum beyond FLT_MAX
 * therefore yields an infinite scale where an fp64 sum would still be finite. */
int hipress_onebit_encode(const float *grad, float *residual, int64_t n, void *payload,
                          int64_t payload_bytes, void *workspace, int64_t workspace_bytes,
                          void *stream);
int hipress_onebit_decode(const void *payload, int64_t payload_bytes, float *out, int64_t n,
                          void *stream);

/* hipress_onebit_encode for callers that cannot allocate device memory (code under
 * HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc): same
 * arguments without the workspace, same payload and residual bit for bit.  The
 * per-tile partial sums live in a device array inside the library (256 KiB per GPU,
 * held until the process ends), which limits n to HIPRESS_ONEBIT_STATIC_MAX_N
 * (larger n: HIPRESS_ERR_SIZE).  The call allocates and frees nothing; the first call
 * on a device looks up that device's copy of the array (hipGetSymbolAddress), so make
 * it once before a capture begins.  The array used is the one of the CURRENT device
 * (hipGetDevice at the time of the call): `stream` must belong to that device, and a
 * stream of another device is refused with HIPRESS_ERR_PARAM before anything is
 * enqueued.  All calls on one GPU share the array: calls that
 * overlap there (different streams without ordering) race; calls on one stream, or
 * ordered by events, are safe.  No counterpart in the reference. */
#define HIPRESS_ONEBIT_STATIC_MAX_N 268435456LL /* 2^28 elements = 65,536 tiles of 4096 */
int hipress_onebit_encode_static(const float *grad, float *residual, int64_t n, void *payload,
                                 int64_t payload_bytes, void *stream);

/* onebit with a deferred residual: one pass per step instead of two.  `state`
 * holds v = r + g of the LAST step (initially the residual itself) and
 * `scale_state` (one float, initially 0) that step's scale; each call first forms
 * the residual r = v - (v >= 0 ? s : -s) on the fly, exactly as the two-pass
 * operator would have stored it, then proceeds as hipress_onebit_encode.  Payloads
 * are identical to hipress_onebit_encode's; hipress_onebit_residual writes the
 * residual that operator would hold into `residual`.  No counterpart in the
 * reference: an extension for callers that do not read the residual between steps. */
int hipress_onebit_encode_deferred(const float *grad, float *state, float *scale_state, int64_t n,
                                   void *payload, int64_t payload_bytes, void *workspace,
                                   int64_t workspace_bytes, void *stream);
int hipress_onebit_residual(const float *state, const float *scale_state, int64_t n,
                            float *residual, void *stream);

/* ---- TernGrad: stochastic ternarisation, per-bucket max-abs scale ---------- */
/* Replaces TernGradEncode_body / TernGradDecode_body for "terngrad"
 * (/root/reference/README.md:9,276).  The rounding noise is an explicit
 * uniform[0,1) tensor instead of the body's clock-seeded generator
 * (TernGradEncode_body.h:49,119). */
int hipress_terngrad_encode(const float *grad, const float *uniform, int64_t n, void *payload,
                            int64_t payload_bytes, int32_t bucket, void *stream);
int hipress_terngrad_decode(const void *payload, int64_t payload_bytes, float *out, int64_t n,
                            void *stream);
/* The same encoder with the noise drawn inside the kernel, as the body this replaces draws
 * its own (TernGradEncode_body.h:49,119: a generator per output byte, seeded from the
 * clock): no noise tensor to fill, keep and read, 4 of the encoder's 8.26 bytes per element
 * less.  Where the reference's seed is the time of the call, here the caller passes it, so
 * that a call can be repeated: element i takes
 *     u_i = (mix32(i ^ tensor_key(uniform_key(seed), tensor)) >> 8) * 2^-24,
 * a counter-based draw on the 24-bit grid in [0, 1) (hipress_amd/csrc/uniform_draw.h states
 * the three functions; tensor = 0 here, the tensor's place in the table for a batch), and
 * the payload equals, byte for byte, that of hipress_terngrad_encode with those values as
 * its noise tensor.  hipress_uniform_fill writes them out (for a check, or for a peer that
 * needs the tensor).  Use a new seed every step.  A call captured in a HIP graph replays
 * the seed it was captured with. */
int hipress_terngrad_encode_seeded(const float *grad, int64_t n, void *payload,
                                   int64_t payload_bytes, int32_t bucket, uint64_t seed,
                                   void *stream);
int hipress_uniform_fill(float *out, int64_t n, uint64_t seed, uint32_t tensor, void *stream);

/* ---- the in-tree CompLL operator, in its own wire format ---------------------- */
/* Replaces TernGradEncode_body / TernGradDecode_body as generated in the tree
 * (/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode_body.h:99-126,
 *  /root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode_body.h:48-74),
 * with the semantics of their DSL sources (pse/TernGradEncode.pse:22-33): payload
 * [bitwidth:u8][tail:u8][min:f32][max:f32] then b-bit codes, code i at bit
 * (i mod 8/b)*b of byte floor(i*b/8); bitwidth in {1,2,4,8}; no alignment is
 * required of `compressed`.  The rounding noise is an explicit uniform[0,1)
 * tensor.  Decode writes (8*compressed_bytes - 80)/b - tail elements, as the
 * reference does (TernGradDecode_body.h:70-72), but never more than n.  With the
 * encoder's tail = n mod 2^b (TernGradEncode_body.h:118) that count is SMALLER than n
 * for some n (b = 2: two short when n mod 4 = 3; b = 4: up to 15; b = 8: n mod 256 short
 * when n is no multiple of 256): out[count, n) is then left as the caller passed it.
 * hipress_compll_decoded_count(n, bitwidth) is that count for a payload encoded from n
 * elements (host arithmetic only). */
int64_t hipress_compll_payload_bytes(int64_t n, int32_t bitwidth);
int64_t hipress_compll_decoded_count(int64_t n, int32_t bitwidth);
int64_t hipress_compll_workspace_bytes(int64_t n);
int hipress_compll_encode(const float *grad, const float *uniform, int64_t n, void *compressed,
                          int64_t compressed_bytes, int32_t bitwidth, void *workspace,
                          int64_t workspace_bytes, void *stream);
/* The encoder with the signature of the body it replaces, (gradient, size, compressed, size,
 * bitwidth, ..., stream), plus the seed that the reference takes from the clock
 * (TernGradEncode_body.h:119): the noise is drawn in the kernel as described at
 * hipress_terngrad_encode_seeded (tensor = 0), and the result equals hipress_compll_encode
 * with hipress_uniform_fill's values as its noise tensor. */
int hipress_compll_encode_seeded(const float *grad, int64_t n, void *compressed,
                                 int64_t compressed_bytes, int32_t bitwidth, uint64_t seed,
                                 void *workspace, int64_t workspace_bytes, void *stream);
int hipress_compll_decode(const void *compressed, int64_t compressed_bytes, float *out, int64_t n,
                          void *stream);

/* ---- DGC / GradDrop: sampled-threshold sparsification ---------------------- */
/* Replace <Func>_body for "dgc" and "graddrop" (/root/reference/README.md:9,162).
 * ratio is the kept fraction (DGC 0.001; GradDrop drop ratio 0.99 = 0.01). */
int hipress_dgc_encode(const float *grad, float *momentum, float *accumulator, int64_t n,
                       void *payload, int64_t payload_bytes, float momentum_factor, double ratio,
                       void *workspace, int64_t workspace_bytes, void *stream);
int hipress_graddrop_encode(const float *grad, float *accumulator, int64_t n, void *payload,
                            int64_t payload_bytes, double ratio, void *workspace,
                            int64_t workspace_bytes, void *stream);
/* One decoder for both: zero-fill out[n], then scatter the pairs. */
int hipress_sparse_decode(const void *payload, int64_t payload_bytes, float *out, int64_t n,
                          void *stream);

/* ---- decode-and-merge (the aggregation step of CaSync, README.md:7) -------- */
/* payloads / payload_bytes are HOST arrays of npeers entries (device pointers
 * and sizes).  aggregate[n] receives the sum of the decoded peers.  With a
 * non-NULL residual (tbq) or accumulator (sparse) the aggregate is re-encoded
 * for the next hop into out_payload in the same pass; such a call may pass
 * aggregate = NULL when only the re-encoded payload is wanted (an aggregator that
 * forwards the sum and applies no update itself): the sum is then never written
 * as fp32, which saves 4 of the step's bytes per element.  Payload and state come
 * out the same either way.  (An empty chunk, n = 0, has no state buffer to point at:
 * there a non-NULL out_payload asks for the re-encode, which writes the header.) */
int hipress_tbq_decode_merge(const void *const *payloads, const int64_t *payload_bytes,
                             int32_t npeers, float *aggregate, int64_t n, float *residual,
                             void *out_payload, int64_t out_payload_bytes, float threshold,
                             void *stream);
int hipress_onebit_decode_merge(const void *const *payloads, const int64_t *payload_bytes,
                                int32_t npeers, float *aggregate, int64_t n, void *stream);
int hipress_terngrad_decode_merge(const void *const *payloads, const int64_t *payload_bytes,
                                  int32_t npeers, float *aggregate, int64_t n, void *stream);
/* Sparse payloads must hold their pairs in ascending index order (the encoders
 * here write them so); a payload that does not is still merged correctly, but
 * every tile then looks through that peer's whole payload: time grows with
 * tiles x pairs (168 chunks of 4 MB with 8 x 1,100 pairs each: 2.5 ms instead of
 * 0.4 ms; one 400 MB chunk with 4 x 100,000 pairs: 27 ms).  workspace: hipress_sparse_merge_workspace_bytes(n, npeers, ratio,
 * accumulator != NULL); it needs no initialisation.  Every call stamps what it
 * finds out of order with a number of its own (a process-wide counter), which a
 * HIP graph freezes: in replays a peer whose payload was once out of order keeps
 * taking the slow path (results stay correct). */
int hipress_sparse_decode_merge(const void *const *payloads, const int64_t *payload_bytes,
                                int32_t npeers, float *aggregate, int64_t n, float *accumulator,
                                void *out_payload, int64_t out_payload_bytes, double ratio,
                                void *workspace, int64_t workspace_bytes, void *stream);

/* The same merges starting from the aggregator's own uncompressed gradient instead of
 * zero: aggregate[i] = ((local[i] + d_1[i]) + d_2[i]) + ..., peers added in order.  One
 * hop of a ring (the payload that arrived, the local gradient, the re-encoded payload to
 * send on), or a server that is also a worker and need not compress its own share.
 * local = NULL is the plain merge; aggregate may be the same buffer as local.  More
 * than HIPRESS_MAX_PEERS payloads are merged by several calls, each after the first
 * with local = the aggregate so far (and only the last with the re-encode): the
 * additions happen in the same order as in one sum over all peers, so the result is
 * the same bit for bit.  No counterpart in the reference checkout (CaSync's sources
 * are not part of it). */
int hipress_tbq_decode_merge_local(const void *const *payloads, const int64_t *payload_bytes,
                                   int32_t npeers, const float *local, float *aggregate, int64_t n,
                                   float *residual, void *out_payload, int64_t out_payload_bytes,
                                   float threshold, void *stream);
int hipress_onebit_decode_merge_local(const void *const *payloads, const int64_t *payload_bytes,
                                      int32_t npeers, const float *local, float *aggregate,
                                      int64_t n, void *stream);
int hipress_terngrad_decode_merge_local(const void *const *payloads, const int64_t *payload_bytes,
                                        int32_t npeers, const float *local, float *aggregate,
                                        int64_t n, void *stream);
int hipress_sparse_decode_merge_local(const void *const *payloads, const int64_t *payload_bytes,
                                      int32_t npeers, const float *local, float *aggregate,
                                      int64_t n, float *accumulator, void *out_payload,
                                      int64_t out_payload_bytes, double ratio, void *workspace,
                                      int64_t workspace_bytes, void *stream);

/* ---- batched launches over a whole gradient set ---------------------------- */
/* A training step compresses every tensor of the model; a batch object holds a
 * device-resident table of the tensors so that one launch sequence covers all of
 * them (the per-tensor calls cost one launch sequence each).  Fields a given
 * algorithm does not use may be NULL.  A batch owns scratch memory on the device, so
 * calls on one batch must not overlap (one stream, or ordered by events); distinct
 * batches are independent.  All calls only enqueue kernels: they may be captured in a
 * HIP graph.  The batched sparse decode expects ascending indices, as this library's and
 * the reference's encoders emit them; a payload out of order still decodes correctly,
 * but every tile of that tensor then looks through its whole payload (time grows with
 * tiles x pairs; hipress_sparse_decode scatters and does not care about order).  The
 * decode passes a per-call counter to its kernels, which a graph freezes: in replays a
 * tensor whose payload was once found out of order keeps taking that slow path
 * (results stay correct). */
typedef struct hipress_tensor {
    const float *grad;    /* encode input, fp32[n] */
    float *state0;        /* residual (onebit, tbq) | momentum (dgc) | accumulator (graddrop) */
    float *state1;        /* accumulator (dgc) */
    const float *uniform; /* terngrad rounding noise, fp32[n] */
    void *payload;        /* compressed buffer */
    float *out;           /* decode output, fp32[n] */
    int64_t n;
    int64_t payload_bytes;
} hipress_tensor;

typedef struct hipress_params {
    float threshold;       /* tbq */
    int32_t bucket;        /* terngrad */
    float momentum_factor; /* dgc */
    float reserved;
    double ratio;          /* dgc, graddrop */
} hipress_params;

typedef struct hipress_batch hipress_batch;

int hipress_batch_create(hipress_batch **out, int32_t alg, const hipress_tensor *tensors,
                         int32_t count, const hipress_params *params);
int hipress_batch_encode(hipress_batch *batch, void *stream);
/* For a terngrad batch none of whose tensors names a noise tensor (`uniform` NULL in all of
 * them; a batch with some and not others is refused): the noise is drawn in the kernel from
 * this seed, tensor k of the table with tensor = k (hipress_terngrad_encode_seeded).
 * hipress_batch_encode and hipress_batch_encode_phase refuse such a batch, and this
 * call any other (HIPRESS_ERR_PARAM). */
int hipress_batch_encode_seeded(hipress_batch *batch, uint64_t seed, void *stream);
int hipress_batch_decode(hipress_batch *batch, void *stream);
/* Measurement aid: enqueues only launch number `phase` of the encode sequence, so
 * that a caller can bracket one kernel with events.  onebit: 0 magnitude sum,
 * 1 scale, 2 quantise; tbq, terngrad: 0; dgc, graddrop: 0 accumulate, 1-3 the
 * three radix-select passes of the threshold, 4 count, 5 scan, 6 emit.  Running every phase in order equals
 * hipress_batch_encode.  No counterpart in the reference. */
int hipress_batch_encode_phase(hipress_batch *batch, int32_t phase, void *stream);
int hipress_batch_destroy(hipress_batch *batch);

/* One chunk of the aggregation step: npeers payloads of the same n. */
typedef struct hipress_merge_chunk {
    const void *payloads[HIPRESS_MAX_PEERS];
    int64_t payload_bytes[HIPRESS_MAX_PEERS];
    float *aggregate;    /* fp32[n] */
    float *state;        /* aggregator residual (tbq) / accumulator (sparse), or NULL */
    void *out_payload;   /* re-encoded payload when state != NULL */
    int64_t out_payload_bytes;
    int64_t n;
    const float *local;  /* fp32[n] the sum starts from (the aggregator's own gradient), or NULL */
} hipress_merge_chunk;

typedef struct hipress_merge_batch hipress_merge_batch;

/* params: threshold (tbq re-encode), ratio (sparse re-encode), and for terngrad `bucket`, the
 * bucket size the peers are expected to have used: the merge then works from it without
 * waiting for the payload headers (8 peers over 168 chunks of 4 MB: 235 us against 365 us
 * through hipress_terngrad_decode_merge, which learns the size from the headers).  The
 * headers still decide: a chunk in which some peer's header names another size is summed
 * from the headers, correctly and more slowly. */
int hipress_merge_batch_create(hipress_merge_batch **out, int32_t alg,
                               const hipress_merge_chunk *chunks, int32_t count, int32_t npeers,
                               const hipress_params *params);
int hipress_merge_batch_run(hipress_merge_batch *batch, void *stream);
/* Measurement aid, like hipress_batch_encode_phase.  dgc / graddrop: 0 tile index of
 * the peers' payloads, 1 merge (with the first launch of the re-encode fused in),
 * 2 the remaining launches of the re-encode; onebit, tbq, terngrad: 0.  No
 * counterpart in the reference. */
int hipress_merge_batch_run_phase(hipress_merge_batch *batch, int32_t phase, void *stream);
int hipress_merge_batch_destroy(hipress_merge_batch *batch);

#ifdef __cplusplus
}
#endif
#endif /* HIPRESS_AMD_H_ */
