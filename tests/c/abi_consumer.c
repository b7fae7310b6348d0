/* A plain C consumer of the library: proves that morphkv.h is valid C (no C++ or
 * torch types in the signatures) and that a C program links against
 * libmorphkv.so and gets the documented status codes.  Host-only entry points:
 * nothing here needs a GPU. */
#include <stdio.h>
#include <string.h>

#include "morphkv.h"

#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            fprintf(stderr, "abi_consumer: %s failed (line %d): %s\n", #cond, __LINE__, \
                    mkv_last_error());                                       \
            return 1;                                                        \
        }                                                                    \
    } while (0)

int main(void) {
    uint64_t k0 = 0, v0 = 0;
    int64_t seg = 0;
    mkv_pool pool;

    CHECK(mkv_version() >= 1);
    CHECK(mkv_sizeof_pool() == (int)sizeof(mkv_pool));

    /* segment carving arithmetic: 256-byte aligned start behind the quantized bytes,
     * as many whole K+V blocks as fit, V base right after the K blocks */
    CHECK(mkv_pool_carve_segment(1000, 4000, 300, 2, 2, 4, 8, &k0, &seg, &v0) == MKV_OK);
    CHECK(k0 == 1536 && seg == 6 && v0 == 1536 + 6 * 256);
    CHECK(mkv_pool_carve_segment(0, 1000, 600, 2, 2, 4, 8, &k0, &seg, &v0) == MKV_ENOSPC);
    CHECK(strstr(mkv_last_error(), "No space available") != NULL);

    /* strided segment table */
    memset(&pool, 0, sizeof pool);
    CHECK(mkv_pool_set_strided(&pool, (void*)(uintptr_t)(1u << 30), (void*)(uintptr_t)((1u << 30) + 4096),
                               1000, 2, 3) == MKV_OK);
    CHECK(pool.num_segments == 3);
    CHECK((uintptr_t)pool.k_seg[2] == (uintptr_t)(1u << 30) - 2 * 2000);
    CHECK(mkv_pool_set_strided(&pool, NULL, NULL, 1000, 2, MKV_MAX_SEGMENTS + 1) == MKV_EINVAL);

    /* argument validation comes before any launch */
    CHECK(mkv_append_decode(NULL, NULL, NULL, NULL, 0, NULL, NULL, 1, 0, NULL) == MKV_EINVAL);
    CHECK(mkv_fill_zero(NULL, 64, NULL) == MKV_EINVAL);

    printf("abi_consumer: ok (version %d, sizeof(mkv_pool) %d)\n", mkv_version(), mkv_sizeof_pool());
    return 0;
}
