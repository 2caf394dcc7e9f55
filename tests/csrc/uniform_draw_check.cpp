// Host build of the header the kernels draw their noise with: prints the key and the first draws of
// every (seed, tensor) given on the command line, as integers, for tests/test_uniform_draw.py.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "uniform_draw.h"

int main(int argc, char** argv) {
    for (int a = 1; a + 2 < argc; a += 3) {
        const uint64_t seed = std::strtoull(argv[a], nullptr, 0);
        const uint32_t tensor = (uint32_t)std::strtoul(argv[a + 1], nullptr, 0);
        const uint32_t count = (uint32_t)std::strtoul(argv[a + 2], nullptr, 0);
        const uint32_t key = hp::tensor_key(hp::uniform_key(seed), tensor);
        std::printf("%" PRIu32, key);
        for (uint32_t i = 0; i < count; ++i) {
            const float u = hp::uniform_at(i, key);
            uint32_t bits;
            std::memcpy(&bits, &u, 4);
            std::printf(" %" PRIu32, bits);
        }
        std::printf("\n");
    }
    return 0;
}
