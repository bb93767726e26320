/*
 * mccl_oracle.c -- CPU restatement of the reference's per-rank reduction path.
 * TEST INFRASTRUCTURE ONLY (see mccl_oracle.h).  All reference citations are
 * paths inside the dormlab/mccl checkout.
 *
 * Build: gcc -O3 -march=x86-64-v3 -ffp-contract=off -fno-fast-math -fopenmp -fPIC -shared
 * IEEE fp32 arithmetic, denormals preserved, no FMA contraction: that is the
 * meaning of "the reference's CPU path" for a code base whose only arithmetic
 * is in GPU kernels.
 */
#include "mccl_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_PAR_FOR(threads) _Pragma("omp parallel for schedule(static) num_threads(threads) if ((threads) > 1)")

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

size_t orc_elem_size(int dtype) { return dtype == ORC_F32 ? 4u : 2u; }

/* ------------------------------------------------------------------ chunking */

/* AllreduceAlgos.cpp:22-34: per = ceil(numel/world); chunk i spans
 * [min(i*per, numel), min((i+1)*per, numel)); the tail chunk may be short or
 * empty. */
void orc_chunkize(int64_t numel, size_t elem_size, int world, orc_chunk* out) {
    int64_t per = (numel + world - 1) / world;
    for (int i = 0; i < world; ++i) {
        int64_t s = (int64_t)i * per;
        int64_t e = (int64_t)(i + 1) * per;
        if (s > numel) s = numel;
        if (e > numel) e = numel;
        out[i].elem_start = s;
        out[i].elem_count = e - s;
        out[i].byte_off = (uint64_t)s * elem_size;
        out[i].byte_len = (uint64_t)(e - s) * elem_size;
    }
}

/* -------------------------------------------------------------- scalar codec */

static inline uint32_t f32_bits(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float x;
    memcpy(&x, &u, 4);
    return x;
}

/* torch/headeronly/util/BFloat16.h:100-114 (round_to_nearest_even), the CPU
 * meaning of `t.to(at::kBFloat16)` at ProcessGroupMCCL.cpp:131-132: any NaN
 * becomes 0x7FC0; otherwise add 0x7FFF plus the lowest kept bit and truncate. */
uint16_t orc_f32_to_bf16(float x) {
    uint32_t u = f32_bits(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
    return (uint16_t)((u + bias) >> 16);
}

/* BFloat16.h: f32_from_bits -- the bf16 pattern is the top half of the fp32
 * pattern (ProcessGroupMCCL.cpp:181, `work.to(fp32)`). */
float orc_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 <- binary64, round to nearest even in ONE rounding, as the
 * AArch64 `(__fp16)scale` conversion at MetalKernels.mm:387,656 does. */
uint16_t orc_f64_to_f16(double x) {
    uint64_t u;
    memcpy(&u, &x, 8);
    uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    int64_t exp = (int64_t)((u >> 52) & 0x7FF);
    uint64_t man = u & 0xFFFFFFFFFFFFFull;
    if (exp == 0x7FF) {
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7E00u | (uint16_t)(man >> 42)); /* quiet NaN, top payload bits */
    }
    int64_t e = exp - 1023 + 15; /* biased half exponent */
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    uint64_t sig = man | (exp ? (1ull << 52) : 0); /* 53-bit significand */
    int shift;                                     /* bits to drop */
    if (e <= 0) {
        if (e < -11) return sign; /* below half of the smallest subnormal */
        shift = 42 + (int)(1 - e);
        e = 0;
    } else {
        shift = 42;
    }
    uint64_t kept = sig >> shift;
    uint64_t rem = sig & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (kept & 1))) kept += 1;
    /* kept holds the implicit bit when e > 0; adding e-1 to the exponent
     * field and letting the carry ripple handles mantissa overflow, including
     * subnormal -> normal and max-finite -> Inf. */
    uint32_t out;
    if (e > 0)
        out = (uint32_t)(((uint64_t)(e - 1) << 10) + kept);
    else
        out = (uint32_t)kept;
    if (out >= 0x7C00u) out = 0x7C00u;
    return (uint16_t)(sign | out);
}

/* binary16 <- binary32: exact widening to binary64 first, so one rounding. */
uint16_t orc_f32_to_f16(float x) { return orc_f64_to_f16((double)x); }

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0x1F) return bits_f32(sign | 0x7F800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24, exact in fp32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* ------------------------------------------------------- whole-buffer codec */

void orc_encode_bf16(uint16_t* dst, const float* src, size_t n, int threads) {
    ORC_PAR_FOR(threads)
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16(src[i]);
}

void orc_decode_bf16(float* dst, const uint16_t* src, size_t n, int threads) {
    ORC_PAR_FOR(threads)
    for (size_t i = 0; i < n; ++i) dst[i] = orc_bf16_to_f32(src[i]);
}

/* ------------------------------------------------------------- element ops */

/* Metal Shading Language, common functions: min(x,y) "returns y if y < x,
 * otherwise x"; max(x,y) "returns y if x < y, otherwise x" (shaders.metal:65-72
 * apply them with x = dst, y = src).  NaN operands make the comparison false,
 * so dst is kept; Apple GPUs under fast-math leave that case undefined, hence
 * "parity unpinned" for NaN inputs. */
static inline float op_f32(float a, float b, int op) {
    switch (op) {
        case ORC_SUM:
        case ORC_AVG: return a + b;
        case ORC_PRODUCT: return a * b;
        case ORC_MIN: return (b < a) ? b : a;
        default: return (a < b) ? b : a; /* ORC_MAX */
    }
}

/* shaders.metal:219-228: bfloat arithmetic rounds after every operation;
 * float add/mul then RNE to bf16 equals the correctly rounded bf16 result
 * (24 >= 2*8+2 significand bits, so the double rounding is innocuous).
 * min/max go through float and back (shaders.metal:9-16). */
static inline uint16_t op_bf16(uint16_t a, uint16_t b, int op) {
    return orc_f32_to_bf16(op_f32(orc_bf16_to_f32(a), orc_bf16_to_f32(b), op));
}

/* shaders.metal:207-216: half arithmetic; float op then RNE to half is the
 * correctly rounded half result for add and mul (24 >= 2*11+2). */
static inline uint16_t op_f16(uint16_t a, uint16_t b, int op) {
    return orc_f32_to_f16(op_f32(orc_f16_to_f32(a), orc_f16_to_f32(b), op));
}

static int op_ok(int op) {
    return op == ORC_SUM || op == ORC_AVG || op == ORC_PRODUCT || op == ORC_MIN || op == ORC_MAX;
}

/* metal_reduce_op_view, MetalKernels.mm:628-640 + select_op_pipeline :606-624:
 * SUM and AVG both run accumulate_chunk_*; the aligned / unaligned / tail
 * branches of binary_vec_op (shaders.metal:159-187) compute the same
 * per-element result, so one loop restates all three. */
int orc_reduce(void* dst, const void* src, int dtype, size_t count, int op, int threads) {
    if (!op_ok(op)) return -1;
    if (dtype == ORC_F32) {
        float* d = (float*)dst;
        const float* s = (const float*)src;
        if (op == ORC_SUM || op == ORC_AVG) {
            ORC_PAR_FOR(threads)
            for (size_t i = 0; i < count; ++i) d[i] = d[i] + s[i];
        } else {
            ORC_PAR_FOR(threads)
            for (size_t i = 0; i < count; ++i) d[i] = op_f32(d[i], s[i], op);
        }
    } else if (dtype == ORC_BF16) {
        uint16_t* d = (uint16_t*)dst;
        const uint16_t* s = (const uint16_t*)src;
        if (op == ORC_SUM || op == ORC_AVG) {
            ORC_PAR_FOR(threads)
            for (size_t i = 0; i < count; ++i)
                d[i] = orc_f32_to_bf16(orc_bf16_to_f32(d[i]) + orc_bf16_to_f32(s[i]));
        } else {
            ORC_PAR_FOR(threads)
            for (size_t i = 0; i < count; ++i) d[i] = op_bf16(d[i], s[i], op);
        }
    } else if (dtype == ORC_F16) {
        uint16_t* d = (uint16_t*)dst;
        const uint16_t* s = (const uint16_t*)src;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) d[i] = op_f16(d[i], s[i], op);
    } else {
        return -1;
    }
    return 0;
}

/* The scalar each scale kernel is handed.
 *   f32 : (float)scale                         MetalKernels.mm:396,664
 *   f16 : (__fp16)scale from double            MetalKernels.mm:387,656
 *   bf16: view variant  bits((float)scale)>>16 MetalKernels.mm:659-662 (truncation)
 *         tensor variant c10::BFloat16((float)scale)  MetalKernels.mm:390-392 (RNE) */
uint32_t orc_scale_constant_bits(int dtype, double scale, int scale_mode) {
    float f = (float)scale;
    if (dtype == ORC_F32) return f32_bits(f);
    if (dtype == ORC_F16) return orc_f64_to_f16(scale);
    if (scale_mode == ORC_SCALE_VIEW) return f32_bits(f) >> 16;
    return orc_f32_to_bf16(f);
}

/* scale_inplace_{f32,f16,bf16}, shaders.metal:233-332: buf[i] = buf[i] * s in
 * the buffer's own type (one rounding per element for the 16-bit types). */
int orc_scale(void* buf, int dtype, size_t count, double scale, int scale_mode, int threads) {
    uint32_t cb = orc_scale_constant_bits(dtype, scale, scale_mode);
    if (dtype == ORC_F32) {
        float s = bits_f32(cb);
        float* b = (float*)buf;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) b[i] = b[i] * s;
    } else if (dtype == ORC_BF16) {
        float s = orc_bf16_to_f32((uint16_t)cb);
        uint16_t* b = (uint16_t*)buf;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) b[i] = orc_f32_to_bf16(orc_bf16_to_f32(b[i]) * s);
    } else if (dtype == ORC_F16) {
        float s = orc_f16_to_f32((uint16_t)cb);
        uint16_t* b = (uint16_t*)buf;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) b[i] = orc_f32_to_f16(orc_f16_to_f32(b[i]) * s);
    } else {
        return -1;
    }
    return 0;
}

/* accumulate_scale_{f32,f16,bf16}, shaders.metal:447-551, constants per
 * metal_accumulate_and_scale (MetalKernels.mm:408-458, tensor variant). */
int orc_accumulate_scale(void* dst, const void* src, int dtype, size_t count, double scale,
                         int threads) {
    uint32_t cb = orc_scale_constant_bits(dtype, scale, ORC_SCALE_TENSOR);
    if (dtype == ORC_F32) {
        float s = bits_f32(cb);
        float* d = (float*)dst;
        const float* a = (const float*)src;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) {
            float t = d[i] + a[i];
            d[i] = t * s;
        }
    } else if (dtype == ORC_BF16) {
        float s = orc_bf16_to_f32((uint16_t)cb);
        uint16_t* d = (uint16_t*)dst;
        const uint16_t* a = (const uint16_t*)src;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) {
            uint16_t t = orc_f32_to_bf16(orc_bf16_to_f32(d[i]) + orc_bf16_to_f32(a[i]));
            d[i] = orc_f32_to_bf16(orc_bf16_to_f32(t) * s);
        }
    } else if (dtype == ORC_F16) {
        float s = orc_f16_to_f32((uint16_t)cb);
        uint16_t* d = (uint16_t*)dst;
        const uint16_t* a = (const uint16_t*)src;
        ORC_PAR_FOR(threads)
        for (size_t i = 0; i < count; ++i) {
            uint16_t t = orc_f32_to_f16(orc_f16_to_f32(d[i]) + orc_f16_to_f32(a[i]));
            d[i] = orc_f32_to_f16(orc_f16_to_f32(t) * s);
        }
    } else {
        return -1;
    }
    return 0;
}

/* ------------------------------------------------ in-memory blocking "mesh" */

/* Stands in for PeerMesh::send/recv (PeerMesh.cpp:293-301): one FIFO per
 * ordered (from, to) pair; send stores a snapshot of the bytes, recv pops the
 * oldest one.  Message order per pair is what the TCP stream guarantees. */
typedef struct orc_msg {
    struct orc_msg* next;
    size_t len;
    unsigned char data[];
} orc_msg;

typedef struct {
    int world;
    orc_msg** head; /* world*world */
    orc_msg** tail;
} orc_mesh;

static int mesh_init(orc_mesh* m, int world) {
    m->world = world;
    m->head = (orc_msg**)calloc((size_t)world * world, sizeof(orc_msg*));
    m->tail = (orc_msg**)calloc((size_t)world * world, sizeof(orc_msg*));
    return (m->head && m->tail) ? 0 : -1;
}
static void mesh_free(orc_mesh* m) {
    for (int i = 0; i < m->world * m->world; ++i) {
        orc_msg* p = m->head[i];
        while (p) {
            orc_msg* n = p->next;
            free(p);
            p = n;
        }
    }
    free(m->head);
    free(m->tail);
}
static int mesh_send(orc_mesh* m, int from, int to, const void* buf, size_t len) {
    orc_msg* msg = (orc_msg*)malloc(sizeof(orc_msg) + len);
    if (!msg) return -1;
    msg->next = NULL;
    msg->len = len;
    if (len) memcpy(msg->data, buf, len);
    int q = from * m->world + to;
    if (m->tail[q])
        m->tail[q]->next = msg;
    else
        m->head[q] = msg;
    m->tail[q] = msg;
    return 0;
}
static int mesh_recv(orc_mesh* m, int to, int from, void* buf, size_t len) {
    int q = from * m->world + to;
    orc_msg* msg = m->head[q];
    if (!msg || msg->len != len) return -1; /* would block / framing error */
    if (len) memcpy(buf, msg->data, len);
    m->head[q] = msg->next;
    if (!m->head[q]) m->tail[q] = NULL;
    free(msg);
    return 0;
}

/* ---------------------------------------------------------------- schedules */

typedef struct {
    int world;
    unsigned char** t;    /* rank tensors */
    unsigned char** recv; /* per-rank recv scratch (ProcessGroupMCCL.cpp:152-162) */
    int dtype;
    int64_t numel;
    size_t esize;
    int op;
    int threads;
    orc_mesh mesh;
} orc_world;

#define TRY(x)            \
    do {                  \
        if ((x) != 0) return -1; \
    } while (0)

/* allreduce_ring, AllreduceAlgos.cpp:52-92.  Within a step every rank's send
 * (a std::thread in the reference) reads a chunk that no rank writes during
 * that step, so "all sends, then all recv+reduce" is an equivalent order. */
static int sched_ring(orc_world* w) {
    int N = w->world;
    if (w->numel < N) return -1; /* AllreduceAlgos.cpp:55 */
    orc_chunk* c = (orc_chunk*)malloc(sizeof(orc_chunk) * N);
    orc_chunkize(w->numel, w->esize, N, c);
    int rc = 0;
    for (int k = 0; k < N - 1 && !rc; ++k) { /* :62-75 reduce-scatter */
        for (int r = 0; r < N; ++r) {
            int send_idx = (r - k + N) % N;
            rc |= mesh_send(&w->mesh, r, (r + 1) % N, w->t[r] + c[send_idx].byte_off,
                            c[send_idx].byte_len);
        }
        for (int r = 0; r < N && !rc; ++r) {
            int recv_idx = (r - k - 1 + N) % N;
            rc |= mesh_recv(&w->mesh, r, (r - 1 + N) % N, w->recv[r], c[recv_idx].byte_len);
            rc |= orc_reduce(w->t[r] + c[recv_idx].byte_off, w->recv[r], w->dtype,
                             (size_t)c[recv_idx].elem_count, w->op, w->threads);
        }
    }
    for (int k = 0; k < N - 1 && !rc; ++k) { /* :77-86 allgather */
        for (int r = 0; r < N; ++r) {
            int send_idx = (r - k + 1 + N) % N;
            rc |= mesh_send(&w->mesh, r, (r + 1) % N, w->t[r] + c[send_idx].byte_off,
                            c[send_idx].byte_len);
        }
        for (int r = 0; r < N && !rc; ++r) {
            int recv_idx = (r - k + N) % N;
            rc |= mesh_recv(&w->mesh, r, (r - 1 + N) % N, w->t[r] + c[recv_idx].byte_off,
                            c[recv_idx].byte_len);
        }
    }
    free(c);
    return rc ? -1 : 0;
}

/* allreduce_tree, AllreduceAlgos.cpp:94-132: binomial reduce to rank 0, then
 * binomial broadcast. */
static int sched_tree(orc_world* w) {
    int N = w->world;
    size_t nbytes = (size_t)w->numel * w->esize;
    char* active = (char*)malloc((size_t)N);
    memset(active, 1, (size_t)N);
    int rc = 0;
    for (int mask = 1; mask < N && !rc; mask <<= 1) { /* :100-114 */
        for (int r = 0; r < N; ++r)
            if (active[r] && (r & mask)) {
                rc |= mesh_send(&w->mesh, r, r - mask, w->t[r], nbytes);
                active[r] = 0;
            }
        for (int r = 0; r < N && !rc; ++r)
            if (active[r] && !(r & mask)) {
                int src = r + mask;
                if (src < N) {
                    rc |= mesh_recv(&w->mesh, r, src, w->recv[r], nbytes);
                    rc |= orc_reduce(w->t[r], w->recv[r], w->dtype, (size_t)w->numel, w->op,
                                     w->threads);
                }
            }
    }
    int top_mask = 1;
    while (top_mask * 2 < N) top_mask <<= 1; /* :116-117 */
    for (int mask = top_mask; mask >= 1 && !rc; mask >>= 1) { /* :119-126 */
        int two = mask << 1;
        for (int r = 0; r < N; ++r)
            if ((r % two) == 0 && (r + mask) < N)
                rc |= mesh_send(&w->mesh, r, r + mask, w->t[r], nbytes);
        for (int r = 0; r < N && !rc; ++r)
            if ((r % two) == mask) rc |= mesh_recv(&w->mesh, r, r - mask, w->t[r], nbytes);
    }
    free(active);
    return rc ? -1 : 0;
}

/* allreduce_butterfly, AllreduceAlgos.cpp:134-206. */
static int sched_butterfly(orc_world* w) {
    int N = w->world;
    if (w->numel < N) return -1; /* :137 */
    orc_chunk* c = (orc_chunk*)malloc(sizeof(orc_chunk) * N);
    orc_chunkize(w->numel, w->esize, N, c);
    int rc = 0;
    for (int r = 0; r < N; ++r) /* :151-169 phase 1 sends */
        for (int p = 0; p < N; ++p)
            if (p != r) rc |= mesh_send(&w->mesh, r, p, w->t[r] + c[p].byte_off, c[p].byte_len);
    for (int r = 0; r < N && !rc; ++r) {
        int slot = 0;
        for (int p = 0; p < N; ++p) { /* recvs land in slot order = ascending peer */
            if (p == r) continue;
            rc |= mesh_recv(&w->mesh, r, p, w->recv[r] + (size_t)slot * c[r].byte_len,
                            c[r].byte_len);
            slot++;
        }
        for (int s = 0; s < N - 1 && !rc; ++s) /* :172-180 */
            rc |= orc_reduce(w->t[r] + c[r].byte_off, w->recv[r] + (size_t)s * c[r].byte_len,
                             w->dtype, (size_t)c[r].elem_count, w->op, w->threads);
    }
    for (int r = 0; r < N && !rc; ++r) /* :185-200 phase 2 */
        for (int p = 0; p < N; ++p)
            if (p != r) rc |= mesh_send(&w->mesh, r, p, w->t[r] + c[r].byte_off, c[r].byte_len);
    for (int r = 0; r < N && !rc; ++r)
        for (int p = 0; p < N; ++p)
            if (p != r) rc |= mesh_recv(&w->mesh, r, p, w->t[r] + c[p].byte_off, c[p].byte_len);
    free(c);
    return rc ? -1 : 0;
}

int orc_allreduce(int algo, int world, void* const* bufs, int dtype, int64_t numel, int op,
                  int threads) {
    if (world < 1 || numel < 0 || !op_ok(op)) return -1;
    if (world == 1) return 0; /* ProcessGroupMCCL.cpp:107 */
    orc_world w;
    w.world = world;
    w.dtype = dtype;
    w.numel = numel;
    w.esize = orc_elem_size(dtype);
    w.op = op;
    w.threads = threads;
    w.t = (unsigned char**)malloc(sizeof(void*) * world);
    w.recv = (unsigned char**)malloc(sizeof(void*) * world);
    int64_t per = (numel + world - 1) / world;
    /* scratch sizing, ProcessGroupMCCL.cpp:152-162 */
    size_t scratch = algo == ORC_ALGO_RING        ? (size_t)per * w.esize
                     : algo == ORC_ALGO_BUTTERFLY ? (size_t)(world - 1) * per * w.esize
                                                  : (size_t)numel * w.esize;
    for (int r = 0; r < world; ++r) {
        w.t[r] = (unsigned char*)bufs[r];
        w.recv[r] = (unsigned char*)malloc(scratch ? scratch : 1);
    }
    int rc = mesh_init(&w.mesh, world);
    if (!rc) {
        if (algo == ORC_ALGO_RING)
            rc = sched_ring(&w);
        else if (algo == ORC_ALGO_BUTTERFLY)
            rc = sched_butterfly(&w);
        else
            rc = sched_tree(&w);
    }
    /* AVG tail, AllreduceAlgos.cpp:88-91,128-131,202-205: view-variant scale of
     * the whole tensor on every rank. */
    if (!rc && op == ORC_AVG)
        for (int r = 0; r < world; ++r)
            orc_scale(w.t[r], dtype, (size_t)numel, 1.0 / (double)world, ORC_SCALE_VIEW, threads);
    mesh_free(&w.mesh);
    for (int r = 0; r < world; ++r) free(w.recv[r]);
    free(w.t);
    free(w.recv);
    return rc;
}

/* ProcessGroupMCCL.cpp:134-145 (+ :173-176: any other string runs tree). */
int orc_select_algo(const char* env_algo, int64_t tree_below, uint64_t wire_nbytes, int64_t numel,
                    int world) {
    int algo;
    if (!env_algo || strcmp(env_algo, "auto") == 0) {
        uint64_t below = tree_below < 0 ? 256ull * 1024 : (uint64_t)tree_below;
        algo = (wire_nbytes <= below) ? ORC_ALGO_TREE : ORC_ALGO_RING;
    } else if (strcmp(env_algo, "ring") == 0) {
        algo = ORC_ALGO_RING;
    } else if (strcmp(env_algo, "butterfly") == 0) {
        algo = ORC_ALGO_BUTTERFLY;
    } else {
        algo = ORC_ALGO_TREE;
    }
    if (algo == ORC_ALGO_RING && numel < world) algo = ORC_ALGO_TREE;
    if (algo == ORC_ALGO_BUTTERFLY && (world < 2 || numel < world)) algo = ORC_ALGO_TREE;
    return algo;
}

int orc_pg_allreduce(int world, void* const* bufs, int dtype, int64_t numel, int op,
                     int wire_bf16, const char* env_algo, int64_t tree_below, int* algo_out,
                     int threads) {
    if (world == 1) return 0;
    int use_wire = wire_bf16 && dtype == ORC_F32; /* :131 */
    int wdtype = use_wire ? ORC_BF16 : dtype;
    int algo = orc_select_algo(env_algo, tree_below, (uint64_t)numel * orc_elem_size(wdtype),
                               numel, world);
    if (algo_out) *algo_out = algo;
    if (!use_wire) return orc_allreduce(algo, world, bufs, dtype, numel, op, threads);
    void** wt = (void**)malloc(sizeof(void*) * world);
    for (int r = 0; r < world; ++r) {
        wt[r] = malloc((size_t)numel * 2 + 2);
        orc_encode_bf16((uint16_t*)wt[r], (const float*)bufs[r], (size_t)numel, threads);
    }
    int rc = orc_allreduce(algo, world, wt, ORC_BF16, numel, op, threads);
    for (int r = 0; r < world; ++r) {
        if (!rc) orc_decode_bf16((float*)bufs[r], (const uint16_t*)wt[r], (size_t)numel, threads);
        free(wt[r]);
    }
    free(wt);
    return rc;
}

/* _reduce_scatter_base, ProcessGroupMCCL.cpp:331-390: out = own share, then one
 * binary reduce per peer in ascending peer order, then the tensor-variant
 * scale for AVG (:384-386). */
int orc_reduce_scatter(int world, void* const* outs, const void* const* ins, int dtype,
                       int64_t chunk_numel, int op, int threads) {
    if (!op_ok(op)) return -1;
    size_t cb = (size_t)chunk_numel * orc_elem_size(dtype);
    for (int r = 0; r < world; ++r) {
        memmove(outs[r], (const unsigned char*)ins[r] + (size_t)r * cb, cb);
        if (world == 1) continue; /* :333-337 */
        for (int p = 0; p < world; ++p) {
            if (p == r) continue;
            orc_reduce(outs[r], (const unsigned char*)ins[p] + (size_t)r * cb, dtype,
                       (size_t)chunk_numel, op, threads);
        }
        if (op == ORC_AVG)
            orc_scale(outs[r], dtype, (size_t)chunk_numel, 1.0 / (double)world, ORC_SCALE_TENSOR,
                      threads);
    }
    return 0;
}

int orc_reduce_scatter_f32acc(int world, void* const* outs, const void* const* ins,
                              int64_t chunk_numel, int op, int threads) {
    if (op != ORC_SUM && op != ORC_AVG) return -1;
    float s = (float)(1.0 / (double)world);
    for (int r = 0; r < world; ++r) {
        uint16_t* o = (uint16_t*)outs[r];
        ORC_PAR_FOR(threads)
        for (int64_t i = 0; i < chunk_numel; ++i) {
            float acc = orc_bf16_to_f32(((const uint16_t*)ins[r])[(size_t)r * chunk_numel + i]);
            for (int p = 0; p < world; ++p) {
                if (p == r) continue;
                acc = acc + orc_bf16_to_f32(((const uint16_t*)ins[p])[(size_t)r * chunk_numel + i]);
            }
            if (op == ORC_AVG) acc = acc * s;
            o[i] = orc_f32_to_bf16(acc);
        }
    }
    return 0;
}

void orc_allgather(int world, void* const* outs, const void* const* ins, size_t chunk_nbytes) {
    for (int r = 0; r < world; ++r)
        for (int p = 0; p < world; ++p)
            memmove((unsigned char*)outs[r] + (size_t)p * chunk_nbytes, ins[p], chunk_nbytes);
}

void orc_wire_fold_chunk(float* out, const float* own, const uint16_t* const* peers, int npeers,
                         size_t n, int own_last, int do_scale, double scale, uint16_t* tmp,
                         uint16_t* wire_out, int threads) {
    if (!own_last) {
        orc_encode_bf16(tmp, own, n, threads);
        for (int p = 0; p < npeers; ++p) orc_reduce(tmp, peers[p], ORC_BF16, n, ORC_SUM, threads);
    } else {
        /* ring order: the travelling partial sum starts as the first peer's
         * chunk, the owner's own data is added last (AllreduceAlgos.cpp:62-75);
         * a + b is commutative bit for bit, so dst/src roles do not matter. */
        memcpy(tmp, peers[0], n * 2);
        for (int p = 1; p < npeers; ++p) orc_reduce(tmp, peers[p], ORC_BF16, n, ORC_SUM, threads);
        uint16_t* enc = (uint16_t*)malloc(n * 2 + 2);
        orc_encode_bf16(enc, own, n, threads);
        orc_reduce(tmp, enc, ORC_BF16, n, ORC_SUM, threads);
        free(enc);
    }
    if (do_scale) orc_scale(tmp, ORC_BF16, n, scale, ORC_SCALE_VIEW, threads);
    orc_decode_bf16(out, tmp, n, threads);
    if (wire_out) memcpy(wire_out, tmp, n * 2);
}
