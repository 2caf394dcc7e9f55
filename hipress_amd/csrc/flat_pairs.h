// Positions among the pairs of several peers laid end to end, peer after peer.
//
// The sparse merge deals the pairs of all peers of a tile out to its threads by such a
// flat position.  A peer contributes up to 2^31 - 1 pairs (a payload found out of order is
// looked through whole) and there are up to sixteen peers, so positions are 64-bit.
// Plain C++ on purpose: the same lines run on the device and in a host-side unit test.
#pragma once

#if defined(__HIPCC__)
#define HP_HOST_DEVICE __host__ __device__ __forceinline__
#else
#define HP_HOST_DEVICE inline
#endif

namespace hp {

// Total number of pairs.
HP_HOST_DEVICE unsigned long long flat_total(const unsigned* count, unsigned npeers) {
    unsigned long long total = 0;
    for (unsigned p = 0; p < npeers; ++p) total += count[p];
    return total;
}

// Moves (peer, before) forward to the peer that holds flat position f, where `before` is the
// number of pairs of all peers in front of `peer`.  Positions at or beyond the total stay
// with the last peer.  Start from (0, 0), or from the result for a smaller position.
HP_HOST_DEVICE void flat_advance(const unsigned* count, unsigned npeers, unsigned long long f, unsigned& peer,
                                 unsigned long long& before) {
    while (peer + 1 < npeers && f >= before + count[peer]) before += count[peer++];
}

}  // namespace hp
