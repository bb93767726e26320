/* A plain C client of the C ABI: what a C or cgo-style host sees.  Uses only the
 * entry points that need no GPU (version, chunk scheduler, algorithm selection,
 * workspace sizing, error reporting), checks them against values worked out by
 * hand from the reference's rules, and prints "ok".
 *   chunkize:     csrc/backend/AllreduceAlgos.cpp:22-34
 *   select_algo:  csrc/backend/ProcessGroupMCCL.cpp:134-145 */
#include <stdio.h>
#include <string.h>

#include "mcclx.h"

#define CHECK(c)                                                    \
    do {                                                            \
        if (!(c)) {                                                 \
            fprintf(stderr, "FAILED line %d: %s\n", __LINE__, #c);  \
            return 1;                                               \
        }                                                           \
    } while (0)

int main(void) {
    CHECK(mcclx_abi_version() == MCCLX_ABI_VERSION);
    CHECK(sizeof(mcclx_seg) == 88);

    /* C2: 6,553,600 bf16 wire elements over 3 ranks -> 2,184,534 / 2,184,534 / 2,184,532 */
    mcclx_chunk ch[3];
    CHECK(mcclx_chunkize(6553600, 2, 3, ch) == MCCLX_OK);
    CHECK(ch[0].elem_count == 2184534 && ch[1].elem_count == 2184534 && ch[2].elem_count == 2184532);
    CHECK(ch[1].byte_off == 2184534ull * 2 && ch[2].elem_start == 2 * 2184534ll);
    /* 3 elements over 5 ranks: the last two chunks are empty (test_ring_chunks.cpp:66-72) */
    mcclx_chunk small[5];
    CHECK(mcclx_chunkize(3, 4, 5, small) == MCCLX_OK);
    CHECK(small[2].elem_count == 1 && small[3].elem_count == 0 && small[4].elem_count == 0);
    CHECK(mcclx_chunkize(3, 4, 0, small) != MCCLX_OK);
    CHECK(strncmp(mcclx_last_error(), "[MCCL] ", 7) == 0);

    /* auto: wire bytes <= 262144 -> tree (inclusive), above -> ring */
    CHECK(mcclx_select_algo(NULL, -1, 262144, 65536, 3) == MCCLX_ALGO_TREE);
    CHECK(mcclx_select_algo("auto", -1, 262145, 65537, 3) == MCCLX_ALGO_RING);
    CHECK(mcclx_select_algo("auto", 1024, 2048, 512, 2) == MCCLX_ALGO_RING);
    CHECK(mcclx_select_algo("butterfly", -1, 1 << 20, 1 << 18, 3) == MCCLX_ALGO_BUTTERFLY);
    CHECK(mcclx_select_algo("ring", -1, 8, 2, 3) == MCCLX_ALGO_TREE);       /* numel < world */
    CHECK(mcclx_select_algo("butterfly", -1, 8, 2, 3) == MCCLX_ALGO_TREE);
    CHECK(mcclx_select_algo("no-such-algorithm", -1, 1 << 20, 1 << 18, 3) == MCCLX_ALGO_TREE);

    /* compute entry points refuse a null context instead of crashing */
    float x[4] = {0};
    CHECK(mcclx_reduce(NULL, x, x, MCCLX_F32, 4, MCCLX_SUM) == MCCLX_ERR_STATE);
    CHECK(mcclx_queue_drain(NULL) == MCCLX_ERR_STATE);
    CHECK(strstr(mcclx_last_error(), "mcclx_init") != NULL);

    mcclx_replay rp;
    memset(&rp, 0, sizeof rp);
    rp.world = 3; rp.algo = MCCLX_ALGO_BUTTERFLY; rp.op = MCCLX_AVG; rp.dtype = MCCLX_F32;
    rp.wire_bf16 = 1; rp.mode = MCCLX_REPLAY_FUSED; rp.numel = 6553600;
    CHECK(mcclx_replay_workspace_bytes(&rp) >= 3ull * 6553600 * 2);   /* one bf16 copy per rank */
    puts("ok");
    return 0;
}
