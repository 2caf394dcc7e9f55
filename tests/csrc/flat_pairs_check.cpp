// Host-side check of the flat pair positions the sparse merge deals out (flat_pairs.h):
// compiled with g++ by tests/test_flat_pairs.py, no GPU involved.
#include <cstdio>
#include <cstdlib>

#include "flat_pairs.h"

typedef unsigned long long u64;

static int failures = 0;
#define CHECK(cond)                                                   \
    do {                                                              \
        if (!(cond)) {                                                \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);    \
            ++failures;                                               \
        }                                                             \
    } while (0)

// the peer and offset of position f by the definition: walk the peers
static void by_definition(const unsigned* cnt, unsigned np, u64 f, unsigned* peer, u64* off) {
    u64 left = f;
    for (unsigned p = 0; p < np; ++p) {
        if (left < cnt[p] || p + 1 == np) {
            *peer = p;
            *off = left;
            return;
        }
        left -= cnt[p];
    }
}

int main() {
    // small: every position of a ragged set, empty peers included
    {
        const unsigned cnt[6] = {3, 0, 0, 5, 1, 0};
        CHECK(hp::flat_total(cnt, 6) == 9);
        for (u64 f = 0; f < 9; ++f) {
            unsigned p = 0, wp;
            u64 before = 0, woff;
            hp::flat_advance(cnt, 6, f, p, before);
            by_definition(cnt, 6, f, &wp, &woff);
            // an empty peer never holds a position
            CHECK(cnt[p] > 0 && f - before < cnt[p]);
            CHECK(p == wp && f - before == woff);
        }
        // resuming from an earlier position gives the same answer as starting afresh
        unsigned p = 0;
        u64 before = 0;
        hp::flat_advance(cnt, 6, 2, p, before);
        hp::flat_advance(cnt, 6, 8, p, before);
        CHECK(p == 4 && before == 8);
    }
    // sixteen peers with 2^31 - 1 pairs each: the total and the positions exceed 32 bits
    {
        unsigned cnt[16];
        for (int i = 0; i < 16; ++i) cnt[i] = 2147483647u;
        const u64 total = hp::flat_total(cnt, 16);
        CHECK(total == 16ull * 2147483647ull);
        CHECK(total > 0xffffffffull);
        const u64 probes[] = {0ull, 2147483646ull, 2147483647ull, 4294967295ull, 4294967296ull, 3ull * 2147483647ull - 1,
                              3ull * 2147483647ull, total - 256, total - 1};
        for (u64 f : probes) {
            unsigned p = 0, wp;
            u64 before = 0, woff;
            hp::flat_advance(cnt, 16, f, p, before);
            by_definition(cnt, 16, f, &wp, &woff);
            CHECK(p == wp && f - before == woff && woff < 2147483647ull);
            CHECK(p == (unsigned)(f / 2147483647ull));
        }
        // the rounds of 256 positions cover [0, total) without wrapping: count them
        u64 rounds = 0;
        for (u64 base = total - 1024; base < total; base += 256) ++rounds;
        CHECK(rounds == 4);
    }
    // four peers just above 2^30 pairs each: the smallest case a 32-bit total gets wrong
    {
        const unsigned cnt[4] = {(1u << 30) + 7, (1u << 30) + 9, (1u << 30) + 11, (1u << 30) + 13};
        const u64 total = hp::flat_total(cnt, 4);
        CHECK(total == 4ull * (1ull << 30) + 40);
        CHECK((unsigned)total != total);
        unsigned p = 0;
        u64 before = 0;
        hp::flat_advance(cnt, 4, total - 1, p, before);
        CHECK(p == 3 && total - 1 - before == cnt[3] - 1);
    }
    if (failures) return 1;
    std::printf("flat pair positions ok\n");
    return 0;
}
