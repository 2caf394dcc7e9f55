/* A C99 consumer of include/hipress_amd.h, as the reference's operator wrapper would be
 * (it would include the header and call the body's replacement with raw pointers).
 * Prints what it sees; tests/test_abi_c_consumer.py compares. Touches no GPU. */
#include <inttypes.h>
#include <stddef.h>
#include <stdio.h>

#include "hipress_amd.h"

#define FIELD(type, f) printf("offset " #type "." #f " %zu\n", offsetof(type, f))

int main(void) {
    const int64_t ns[4] = {0, 1, 262144, 102760448};
    int i;
    printf("version %d\n", hipress_version());
    for (i = 0; i < 4; ++i)
        printf("sizes %" PRId64 " %" PRId64 " %" PRId64 " %" PRId64 " %" PRId64 " %" PRId64 " %" PRId64 "\n", ns[i],
               hipress_onebit_payload_bytes(ns[i]), hipress_tbq_payload_bytes(ns[i]),
               hipress_terngrad_payload_bytes(ns[i], 512), hipress_sparse_capacity(ns[i], 0.001),
               hipress_sparse_payload_bytes(ns[i], 0.001), hipress_compll_payload_bytes(ns[i], 2));
    printf("sizeof hipress_tensor %zu\nsizeof hipress_params %zu\nsizeof hipress_merge_chunk %zu\n",
           sizeof(hipress_tensor), sizeof(hipress_params), sizeof(hipress_merge_chunk));
    FIELD(hipress_tensor, grad); FIELD(hipress_tensor, state0); FIELD(hipress_tensor, state1);
    FIELD(hipress_tensor, uniform); FIELD(hipress_tensor, payload); FIELD(hipress_tensor, out);
    FIELD(hipress_tensor, n); FIELD(hipress_tensor, payload_bytes);
    FIELD(hipress_params, threshold); FIELD(hipress_params, bucket); FIELD(hipress_params, momentum_factor);
    FIELD(hipress_params, reserved); FIELD(hipress_params, ratio);
    FIELD(hipress_merge_chunk, payloads); FIELD(hipress_merge_chunk, payload_bytes);
    FIELD(hipress_merge_chunk, aggregate); FIELD(hipress_merge_chunk, state); FIELD(hipress_merge_chunk, out_payload);
    FIELD(hipress_merge_chunk, out_payload_bytes); FIELD(hipress_merge_chunk, n); FIELD(hipress_merge_chunk, local);
    /* validated on the host before any launch: no device is needed for these */
    printf("null_encode %d\n", hipress_tbq_encode(NULL, NULL, 16, NULL, 100, 0.05f, NULL));
    printf("null_decode %d\n", hipress_tbq_decode(NULL, 100, NULL, 16, NULL));
    printf("too_large %d\n", (int)hipress_tbq_payload_bytes(HIPRESS_MAX_N + 1));
    printf("strerror %s\n", hipress_strerror(HIPRESS_ERR_NULL));
    return 0;
}
