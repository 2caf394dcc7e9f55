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
hipError_t launch_terngrad_encode(const Launch& L, unsigned bucket, bool draw, unsigned key, hipStream_t st);  // draw: noise from key, not from the tensors
hipError_t launch_uniform_fill(float* out, unsigned long long n, unsigned key, hipStream_t st);
hipError_t launch_terngrad_decode(const Launch& L, unsigned bucket, hipStream_t st);  // bucket: what the launch's descriptors name, 0 = unknown

// The in-tree CompLL operator (10-byte header, b-bit min/max quantiser).
hipError_t launch_compll_encode(const Launch& L, int bitwidth, float* partial, bool draw, unsigned key, hipStream_t st);
hipError_t launch_compll_decode(const Launch& L, hipStream_t st);

// Dense decode-and-merge; alg is a hipress_alg value (onebit, tbq, terngrad).
hipError_t launch_dense_merge(const MergeLaunch& L, int alg, hipStream_t st);

// Sparse (DGC / GradDrop) pipeline.  ws is the launch's workspace.
struct SparseWs {
    uint32_t* sample;   // |acc'| keys at the sample positions, all tensors back to back
    uint2* grec;        // per 64-element group (64 per tile): {bits of the acc' value with the largest |.|,
                        //  (upper bound of the second-largest key, multiple of 64) | position of the largest}
    uint32_t* counts;   // per tile {above, equal} counts, then their exclusive scans
    uint32_t* thr;      // per tensor {threshold key, equal-quota}, written by the scan launch
    uint32_t* hist;     // per tensor 4096 + 4096 + 128 bins, one histogram per select pass
    uint32_t* ctl;      // per tensor 8 words: key prefix and remaining rank after the first and the second digit
};
hipError_t launch_sparse_encode(const Launch& L, bool dgc, const SparseWs& ws, int phase, hipStream_t st);
hipError_t launch_sparse_decode(const Launch& L, hipStream_t st);
hipError_t launch_sparse_decode_indexed(const Launch& L, uint32_t* tptr, uint32_t* disorder, unsigned epoch,
                                        bool few_pairs, hipStream_t st);
constexpr int kSparseAfterAccum = 100;  // launch_sparse_encode phase: everything after the accumulate launch
// Sparse decode-and-merge: what the index launch leaves for the merge launch, records of
// 32 bytes: the heads of all T tiles of the launch, then every peer's runs for those tiles
// (record of peer p, tile t at (1 + p) * T + t), kMergeRecs(npeers) * T records in all.
struct PeerRun {
    const int32_t* idx;  // first index of the run
    const float* val;    // first value of the run
    const int32_t* end;  // just behind the run's last index
    unsigned disorder;   // == the call's epoch: this peer's payload is not in order, ignore the run
    unsigned pad;        // 32 bytes: one record is two 16-byte loads
};
struct TileHead {
    const float* acc;    // re-encode: the tile's first accumulator element (NULL without re-encode)
    unsigned fast;       // 1: whole tile, every pointer 16-byte aligned
    unsigned pad[5];
};
static_assert(sizeof(PeerRun) == 32 && sizeof(TileHead) == 32, "merge records are 32 bytes");
constexpr unsigned kMergeRecs(unsigned npeers) { return npeers + 1; }
hipError_t launch_sparse_merge(const MergeLaunch& L, const SparseWs& ws, PeerRun* runs, unsigned slices, unsigned epoch,
                               int phase, hipStream_t st);

}  // namespace hp
