// Host-callable launchers; each one only enqueues kernels on the given stream.
#pragma once
#include "common.h"

namespace hp {

hipError_t launch_tbq_encode(const Launch& L, hipStream_t st);
hipError_t launch_tbq_decode(const Launch& L, hipStream_t st);
hipError_t launch_onebit_encode(const Launch& L, float* partial, int phase, hipStream_t st);
hipError_t launch_onebit_decode(const Launch& L, hipStream_t st);
hipError_t launch_onebit_encode_deferred(const Launch& L, float* partial, int phase, hipStream_t st);
hipError_t launch_onebit_materialize(const Launch& L, hipStream_t st);
hipError_t launch_terngrad_encode(const Launch& L, unsigned bucket, hipStream_t st);
hipError_t launch_terngrad_decode(const Launch& L, hipStream_t st);

// The in-tree CompLL operator (10-byte header, b-bit min/max quantiser).
hipError_t launch_compll_encode(const Launch& L, int bitwidth, float* partial, hipStream_t st);
hipError_t launch_compll_decode(const Launch& L, hipStream_t st);

// Dense decode-and-merge; alg is a hipress_alg value (onebit, tbq, terngrad).
hipError_t launch_dense_merge(const MergeLaunch& L, int alg, hipStream_t st);

// Sparse (DGC / GradDrop) pipeline.  ws is the launch's workspace.
struct SparseWs {
    uint32_t* sample;   // |acc'| keys at the sample positions, all tensors back to back
    uint2* grec;        // per 64-element group (64 per tile): {bits of the acc' value with the largest |.|,
                        //  (upper bound of the second-largest key, multiple of 64) | position of the largest}
    uint32_t* counts;   // per tile {above, equal} counts, then their exclusive scans
    uint32_t* thr;      // per tensor {threshold key, equal-quota}
    uint32_t* hist;     // per tensor 3 x 2048 bins, one histogram per select pass
    uint32_t* ctl;      // per tensor 8 words: select prefix, remaining rank, done counters
};
hipError_t launch_sparse_encode(const Launch& L, bool dgc, const SparseWs& ws, int phase, hipStream_t st);
hipError_t launch_sparse_decode(const Launch& L, hipStream_t st);
hipError_t launch_sparse_decode_indexed(const Launch& L, uint32_t* tptr, uint32_t* disorder, unsigned epoch,
                                        bool few_pairs, hipStream_t st);
constexpr int kSparseAfterAccum = 100;  // launch_sparse_encode phase: everything after the accumulate launch
hipError_t launch_sparse_merge(const MergeLaunch& L, const SparseWs& ws, uint32_t* tileptr, uint32_t* unsorted,
                               int phase, hipStream_t st);

}  // namespace hp
