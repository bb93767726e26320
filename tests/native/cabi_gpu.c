/* A plain C client of the C ABI on the GPU, with no HIP or torch in sight: buffers
 * come from mcclx_host_alloc (pinned host memory the GPU reads and writes in
 * place), the C2-shaped fused fold and the reference's four kernel calls run on
 * them, and the results are checked on the host against values worked out here
 * with the reference's recipe (encode = round to nearest even, add in fp32, round,
 * multiply by the truncated bf16 constant, round, decode).
 *   metal_reduce_op_view / metal_scale_inplace_view: csrc/metal/MetalKernels.mm:628-674
 *   wire codec:                                      csrc/backend/ProcessGroupMCCL.cpp:131-132,179-183 */
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "mcclx.h"

#define CHECK(c)                                                                       \
    do {                                                                               \
        if (!(c)) {                                                                    \
            fprintf(stderr, "FAILED line %d: %s  [%s]\n", __LINE__, #c, mcclx_last_error()); \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint16_t enc(float f) {  /* torch/headeronly/util/BFloat16.h:100-114 */
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static float dec(uint16_t h) { return u2f((uint32_t)h << 16); }

int main(void) {
    enum { N = 100003 };
    mcclx_ctx* ctx = NULL;
    CHECK(mcclx_init(0, &ctx) == MCCLX_OK);
    CHECK(mcclx_device_cus(ctx) > 0);

    void *h_own, *d_own, *h_p1, *d_p1, *h_p2, *d_p2, *h_out, *d_out, *h_w, *d_w;
    CHECK(mcclx_host_alloc(ctx, N * 4, &h_own, &d_own) == MCCLX_OK);
    CHECK(mcclx_host_alloc(ctx, N * 2, &h_p1, &d_p1) == MCCLX_OK);
    CHECK(mcclx_host_alloc(ctx, N * 2, &h_p2, &d_p2) == MCCLX_OK);
    CHECK(mcclx_host_alloc(ctx, N * 4, &h_out, &d_out) == MCCLX_OK);
    CHECK(mcclx_host_alloc(ctx, N * 2, &h_w, &d_w) == MCCLX_OK);
    float* own = (float*)h_own; uint16_t* p1 = (uint16_t*)h_p1; uint16_t* p2 = (uint16_t*)h_p2;
    float* out = (float*)h_out; uint16_t* w = (uint16_t*)h_w;
    uint64_t s = 0x6D63636C00000000ull;
    for (int i = 0; i < N; ++i) {  /* xorshift values in about +-1e-3, a few large ones */
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        own[i] = ((int32_t)(s & 0xFFFFF) - 0x80000) * 2e-9f * ((i % 997 == 0) ? 1e5f : 1.0f);
        p1[i] = enc(((int32_t)((s >> 20) & 0xFFFFF) - 0x80000) * 2e-9f);
        p2[i] = enc(((int32_t)((s >> 40) & 0xFFFFF) - 0x80000) * 2e-9f);
    }

    /* the fused C2 step: own fp32 + two bf16 peers, x 1/3 (view constant), fp32 out + bf16 wire copy */
    mcclx_plan plan;
    memset(&plan, 0, sizeof plan);
    plan.dtype = MCCLX_BF16; plan.io = MCCLX_IO_OWN_FIRST_F32; plan.k = 3; plan.topo = MCCLX_TOPO_FOLD;
    plan.op = MCCLX_SUM; plan.acc = MCCLX_ACC_STEP; plan.scale_mode = MCCLX_SCALE_VIEW; plan.scale = 1.0 / 3.0;
    mcclx_seg seg;
    memset(&seg, 0, sizeof seg);
    seg.out = d_out; seg.wire_out = d_w; seg.in[0] = d_own; seg.in[1] = d_p1; seg.in[2] = d_p2; seg.count = N;
    CHECK(mcclx_fold(ctx, &plan, &seg) == MCCLX_OK);
    CHECK(mcclx_queue_drain(ctx) == MCCLX_OK);
    const float third = u2f(f2u((float)(1.0 / 3.0)) & 0xFFFF0000u);  /* 0x3EAA0000 */
    CHECK(f2u(third) == 0x3EAA0000u);
    for (int i = 0; i < N; ++i) {
        uint16_t a = enc(own[i]);
        a = enc(dec(a) + dec(p1[i]));
        a = enc(dec(a) + dec(p2[i]));
        a = enc(dec(a) * third);
        if (w[i] != a || f2u(out[i]) != ((uint32_t)a << 16)) {
            fprintf(stderr, "fold differs at %d: got %08x / %04x want %04x\n", i, f2u(out[i]), w[i], a);
            return 1;
        }
    }

    /* the reference's own calls, one for one: dst += src (fp32), then dst *= 1/2 */
    float* a32 = out; float* b32 = own;
    for (int i = 0; i < N; ++i) a32[i] = (float)i * 0.5f;
    CHECK(mcclx_reduce(ctx, d_out, d_own, MCCLX_F32, N, MCCLX_SUM) == MCCLX_OK);
    CHECK(mcclx_scale(ctx, d_out, MCCLX_F32, N, 0.5, MCCLX_SCALE_VIEW) == MCCLX_OK);
    uint64_t ticket = 0;
    CHECK(mcclx_event_record(ctx, &ticket) == MCCLX_OK && ticket != 0);
    CHECK(mcclx_event_wait(ctx, ticket) == MCCLX_OK);
    for (int i = 0; i < N; ++i) {
        float want = ((float)i * 0.5f + b32[i]) * 0.5f;
        if (f2u(a32[i]) != f2u(want)) { fprintf(stderr, "reduce/scale differs at %d\n", i); return 1; }
    }

    /* errors come back as codes with the reference's message prefix */
    CHECK(mcclx_reduce(ctx, d_out, d_own, MCCLX_F32, N, 17) == MCCLX_ERR_UNSUPPORTED);
    CHECK(strstr(mcclx_last_error(), "[MCCL] Unsupported ReduceOp: 17") != NULL);
    CHECK(mcclx_reduce(ctx, d_out, NULL, MCCLX_F32, N, MCCLX_SUM) == MCCLX_ERR_INVALID);

    CHECK(mcclx_host_free(ctx, h_own) == MCCLX_OK && mcclx_host_free(ctx, h_p1) == MCCLX_OK);
    CHECK(mcclx_host_free(ctx, h_p2) == MCCLX_OK && mcclx_host_free(ctx, h_out) == MCCLX_OK);
    CHECK(mcclx_host_free(ctx, h_w) == MCCLX_OK);
    CHECK(mcclx_destroy(ctx) == MCCLX_OK);
    puts("ok");
    return 0;
}
