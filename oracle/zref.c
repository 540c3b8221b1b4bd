/* CPU oracle: a plain-C restatement of the reference's src/ref path.
 * TEST INFRASTRUCTURE ONLY: see zref.h. Build with -ffp-contract=off: the
 * reference's decoders and microkernel are defined by separately rounded
 * multiplies, subtracts and adds. */
#define _GNU_SOURCE
#include "zref.h"

#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ---- block geometry: src/gguf/gguf.zig:69-109 ------------------------------ */

int zref_layout(int type, uint32_t *block_elems, uint32_t *block_bytes) {
    uint32_t e, b;
    switch (type) {
    case ZREF_F32: e = 1; b = 4; break;
    case ZREF_F16: case ZREF_BF16: e = 1; b = 2; break;
    case ZREF_Q8_0: e = 32; b = 34; break;
    case ZREF_Q3_K: e = 256; b = 110; break;
    case ZREF_Q4_K: e = 256; b = 144; break;
    case ZREF_Q5_K: e = 256; b = 176; break;
    case ZREF_Q6_K: e = 256; b = 210; break;
    case ZREF_IQ4_XS: e = 256; b = 136; break;
    default: return 0;
    }
    if (block_elems) *block_elems = e;
    if (block_bytes) *block_bytes = b;
    return 1;
}

/* ---- scalar conversions ----------------------------------------------------- */

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline uint32_t rd32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static inline float bits_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

/* src/ref/tensor.zig:45-47: the f16 widened to f32, which is exact. */
float zref_half(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ff;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* Subnormal: man * 2^-24, exact in f32. */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112) << 23) | (man << 13));
}

/* src/ref/matmul.zig:250-255. */
float zref_bf16_round(float v) {
    uint32_t bits = f32_bits(v);
    uint32_t r = bits + (0x7fffu + ((bits >> 16) & 1u));
    return bits_f32(r & 0xffff0000u);
}

/* src/ref/ops.zig:49-51. */
float zref_silu(float x) { return x / (1.0f + expf(-x)); }

/* src/ref/ops.zig:25-41: squares rounded to f32, summed and divided in f64,
 * then an f32 mean, add, sqrt and reciprocal; x * scale, then * w. */
void zref_rms_norm(float *x, const float *weight, size_t n, float eps) {
    double sum = 0;
    for (size_t i = 0; i < n; i++) {
        float square = x[i] * x[i];
        sum += square;
    }
    float mean = (float)(sum / (double)n);
    float scale = 1.0f / sqrtf(mean + eps);
    for (size_t i = 0; i < n; i++) {
        float t = x[i] * scale;
        x[i] = t * weight[i];
    }
}

/* ---- decoders: src/ref/tensor.zig ------------------------------------------- */

/* src/ref/tensor.zig:94-98. */
void zref_scale_min_k4(unsigned j, const uint8_t q[12], uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

void zref_pack_scale_min_k4(unsigned j, uint8_t q[12], uint8_t sc, uint8_t m) {
    if (j < 4) {
        q[j] = (uint8_t)((q[j] & 0xC0) | (sc & 63));
        q[j + 4] = (uint8_t)((q[j + 4] & 0xC0) | (m & 63));
    } else {
        q[j + 4] = (uint8_t)((sc & 0xF) | ((m & 0xF) << 4));
        q[j - 4] = (uint8_t)((q[j - 4] & 63) | ((sc >> 4) << 6));
        q[j] = (uint8_t)((q[j] & 63) | ((m >> 4) << 6));
    }
}

/* src/ref/tensor.zig:49-53: one f32 multiply per weight. */
static void q8_0_block(const uint8_t *b, float *y) {
    float d = zref_half(rd16(b));
    for (int i = 0; i < 32; i++) y[i] = (float)(int8_t)b[2 + i] * d;
}

/* src/ref/tensor.zig:100-116: d1 = d*sc, m1 = dmin*m (one rounding each),
 * then d1*q - m1 as a multiply followed by a subtract. */
static void q4_k_block(const uint8_t *b, float *y) {
    float d = zref_half(rd16(b));
    float min = zref_half(rd16(b + 2));
    const uint8_t *scales = b + 4;
    for (unsigned j = 0; j < 4; j++) {
        const uint8_t *q = b + 16 + 32 * j;
        uint8_t sc1, mn1, sc2, mn2;
        zref_scale_min_k4(2 * j, scales, &sc1, &mn1);
        zref_scale_min_k4(2 * j + 1, scales, &sc2, &mn2);
        float d1 = d * (float)sc1;
        float m1 = min * (float)mn1;
        float d2 = d * (float)sc2;
        float m2 = min * (float)mn2;
        for (int l = 0; l < 32; l++) {
            float p = d1 * (float)(q[l] & 0xF);
            y[64 * j + l] = p - m1;
        }
        for (int l = 0; l < 32; l++) {
            float p = d2 * (float)(q[l] >> 4);
            y[64 * j + 32 + l] = p - m2;
        }
    }
}

/* src/ref/tensor.zig:55-92: sixteen 6-bit scales (low four bits in bytes
 * 0..7 by nibble, top two in bytes 8..11), dl = d * (scale - 32), weight l of
 * half n and shift j = dl * (two bits 2j of qs[32n + l], minus 4 unless bit
 * 4n + j of hmask[l] is set). */
static void q3_k_scales(const uint8_t *b, int8_t scales[16]) {
    uint32_t aux[4];
    for (int i = 0; i < 3; i++) aux[i] = rd32(b + 96 + 4 * i);
    const uint32_t kmask1 = 0x03030303u, kmask2 = 0x0f0f0f0fu;
    uint32_t tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
    aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
    aux[0] = (aux[0] & kmask2) | (((tmp >> 0) & kmask1) << 4);
    aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
    for (int i = 0; i < 16; i++) scales[i] = (int8_t)((aux[i / 4] >> (8 * (i % 4))) & 0xff);
}

static void q3_k_block(const uint8_t *b, float *y) {
    const uint8_t *hm = b;
    float d_all = zref_half(rd16(b + 108));
    int8_t scales[16];
    q3_k_scales(b, scales);
    size_t out = 0;
    unsigned is = 0;
    uint8_t m = 1;
    for (unsigned n = 0; n < 2; n++) {
        const uint8_t *q = b + 32 + 32 * n;
        unsigned shift = 0;
        for (unsigned j = 0; j < 4; j++) {
            for (unsigned h = 0; h < 2; h++) {
                float dl = d_all * (float)((int)scales[is++] - 32);
                for (unsigned l = 0; l < 16; l++) {
                    int lo = (q[l + 16 * h] >> shift) & 3;
                    int v = lo - ((hm[l + 16 * h] & m) ? 0 : 4);
                    y[out++] = dl * (float)v;
                }
            }
            shift += 2;
            m = (uint8_t)(m << 1);
        }
    }
}

/* src/ref/tensor.zig:118-138: Q4_K with a fifth bit per weight from qh
 * (bit 2j of qh[l] for the low sub-block of chunk j, bit 2j + 1 for the high). */
static void q5_k_block(const uint8_t *b, float *y) {
    float d = zref_half(rd16(b));
    float min = zref_half(rd16(b + 2));
    const uint8_t *scales = b + 4;
    const uint8_t *qh = b + 16;
    for (unsigned j = 0; j < 4; j++) {
        const uint8_t *ql = b + 48 + 32 * j;
        uint8_t bit_lo = (uint8_t)(1u << (2 * j)), bit_hi = (uint8_t)(2u << (2 * j));
        uint8_t sc1, mn1, sc2, mn2;
        zref_scale_min_k4(2 * j, scales, &sc1, &mn1);
        zref_scale_min_k4(2 * j + 1, scales, &sc2, &mn2);
        float d1 = d * (float)sc1;
        float m1 = min * (float)mn1;
        float d2 = d * (float)sc2;
        float m2 = min * (float)mn2;
        for (int l = 0; l < 32; l++) {
            float p = d1 * (float)((ql[l] & 0xF) + ((qh[l] & bit_lo) ? 16 : 0));
            y[64 * j + l] = p - m1;
        }
        for (int l = 0; l < 32; l++) {
            float p = d2 * (float)((ql[l] >> 4) + ((qh[l] & bit_hi) ? 16 : 0));
            y[64 * j + 32 + l] = p - m2;
        }
    }
}

/* src/ref/tensor.zig:140-160: d * sc * q evaluated left to right, two
 * roundings; q = low nibble | two high bits << 4, minus 32. */
static void q6_k_block(const uint8_t *b, float *y) {
    float d = zref_half(rd16(b + 208));
    for (unsigned n = 0; n < 2; n++) {
        const uint8_t *ql = b + 64 * n;
        const uint8_t *qh = b + 128 + 32 * n;
        const int8_t *sc = (const int8_t *)(b + 192 + 8 * n);
        float *out = y + 128 * n;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            float t1 = d * (float)sc[is], t2 = d * (float)sc[is + 2], t3 = d * (float)sc[is + 4], t4 = d * (float)sc[is + 6];
            out[l] = t1 * (float)q1;
            out[l + 32] = t2 * (float)q2;
            out[l + 64] = t3 * (float)q3;
            out[l + 96] = t4 * (float)q4;
        }
    }
}

/* src/ref/tensor.zig:162-181: d (f16), scales_h (u16), scales_l[4], qs[128]; each
 * group of 32 has a signed six-bit scale biased by 32 and sixteen bytes of
 * indices into a nonlinear table, low nibbles first, then high nibbles. */
static void iq4_xs_block(const uint8_t *b, float *y) {
    static const int8_t values[16] = { -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113 };
    float d = zref_half(rd16(b));
    uint32_t scales_h = rd16(b + 2);
    for (unsigned group = 0; group < 8; group++) {
        uint32_t low = (b[4 + group / 2] >> (4 * (group % 2))) & 15;
        uint32_t high = (scales_h >> (2 * group)) & 3;
        int scale = (int)(low | (high << 4)) - 32;
        float dl = d * (float)scale;
        const uint8_t *qs = b + 8 + 16 * group;
        for (unsigned j = 0; j < 16; j++) {
            y[32 * group + j] = dl * (float)values[qs[j] & 15];
            y[32 * group + 16 + j] = dl * (float)values[qs[j] >> 4];
        }
    }
}

/* src/ref/tensor.zig:21-43. */
int zref_dequantize(int type, const uint8_t *bytes, float *out, size_t n) {
    switch (type) {
    case ZREF_Q8_0:
        for (size_t i = 0; i < n / 32; i++) q8_0_block(bytes + i * 34, out + i * 32);
        return 0;
    case ZREF_Q3_K:
        for (size_t i = 0; i < n / 256; i++) q3_k_block(bytes + i * 110, out + i * 256);
        return 0;
    case ZREF_Q4_K:
        for (size_t i = 0; i < n / 256; i++) q4_k_block(bytes + i * 144, out + i * 256);
        return 0;
    case ZREF_Q5_K:
        for (size_t i = 0; i < n / 256; i++) q5_k_block(bytes + i * 176, out + i * 256);
        return 0;
    case ZREF_Q6_K:
        for (size_t i = 0; i < n / 256; i++) q6_k_block(bytes + i * 210, out + i * 256);
        return 0;
    case ZREF_IQ4_XS:
        if (n % 256) return -1;
        for (size_t i = 0; i < n / 256; i++) iq4_xs_block(bytes + i * 136, out + i * 256);
        return 0;
    case ZREF_F32:
        for (size_t i = 0; i < n; i++) out[i] = bits_f32(rd32(bytes + 4 * i));
        return 0;
    case ZREF_F16:
        for (size_t i = 0; i < n; i++) out[i] = zref_half(rd16(bytes + 2 * i));
        return 0;
    case ZREF_BF16:
        for (size_t i = 0; i < n; i++) out[i] = bits_f32((uint32_t)rd16(bytes + 2 * i) << 16);
        return 0;
    default:
        return -1;
    }
}

/* ---- fork-join pool: src/ref/pool.zig:76-122 --------------------------------
 * Persistent workers; parallel_for splits [0, n) into contiguous ranges, the
 * caller taking the range after all workers' ranges. */

typedef void (*range_fn)(void *ctx, size_t first, size_t last);

typedef struct pool {
    unsigned workers; /* threads besides the caller */
    pthread_t *threads;
    pthread_mutex_t mu;
    pthread_cond_t wake, done;
    unsigned long generation;
    unsigned pending;
    int stop;
    range_fn fn;
    void *ctx;
    size_t n, chunk;
} pool;

typedef struct { pool *p; unsigned index; } worker_arg;

static void run_range(pool *p, unsigned index) {
    size_t first = (size_t)index * p->chunk;
    if (first >= p->n) return;
    size_t last = first + p->chunk;
    if (last > p->n) last = p->n;
    p->fn(p->ctx, first, last);
}

static void *worker_main(void *argp) {
    worker_arg *arg = (worker_arg *)argp;
    pool *p = arg->p;
    unsigned index = arg->index;
    free(arg);
    unsigned long seen = 0;
    for (;;) {
        pthread_mutex_lock(&p->mu);
        while (p->generation == seen && !p->stop) pthread_cond_wait(&p->wake, &p->mu);
        if (p->stop) { pthread_mutex_unlock(&p->mu); return NULL; }
        seen = p->generation;
        pthread_mutex_unlock(&p->mu);
        run_range(p, index);
        pthread_mutex_lock(&p->mu);
        if (--p->pending == 0) pthread_cond_signal(&p->done);
        pthread_mutex_unlock(&p->mu);
    }
}

static pool *pool_create(unsigned threads) {
    pool *p = (pool *)calloc(1, sizeof *p);
    p->workers = threads > 0 ? threads - 1 : 0;
    pthread_mutex_init(&p->mu, NULL);
    pthread_cond_init(&p->wake, NULL);
    pthread_cond_init(&p->done, NULL);
    p->threads = (pthread_t *)calloc(p->workers ? p->workers : 1, sizeof(pthread_t));
    for (unsigned i = 0; i < p->workers; i++) {
        worker_arg *a = (worker_arg *)malloc(sizeof *a);
        a->p = p; a->index = i;
        pthread_create(&p->threads[i], NULL, worker_main, a);
    }
    return p;
}

/* One cached pool per thread count requested, kept for the process's life as
 * the reference keeps its pool for the run. */
static pool *pool_get(unsigned threads) {
    static pool *cache[8];
    static unsigned counts[8];
    static pthread_mutex_t mu = PTHREAD_MUTEX_INITIALIZER;
    if (threads == 0) threads = 1;
    pthread_mutex_lock(&mu);
    pool *found = NULL;
    for (int i = 0; i < 8; i++) {
        if (cache[i] && counts[i] == threads) { found = cache[i]; break; }
    }
    if (!found) {
        for (int i = 0; i < 8; i++) {
            if (!cache[i]) { cache[i] = found = pool_create(threads); counts[i] = threads; break; }
        }
    }
    pthread_mutex_unlock(&mu);
    if (!found) { fprintf(stderr, "zref: too many distinct pool sizes\n"); abort(); }
    return found;
}

/* src/ref/pool.zig:79-101. */
static void parallel_for(pool *p, size_t n, size_t align_to, size_t min_chunk, void *ctx, range_fn fn) {
    size_t thread_count = (size_t)p->workers + 1;
    size_t by_chunk = n / (min_chunk ? min_chunk : 1);
    size_t parts = thread_count < by_chunk ? thread_count : by_chunk;
    if (parts < 1) parts = 1;
    size_t chunk = (n + parts - 1) / parts;
    chunk = (chunk + align_to - 1) / align_to * align_to;
    if (parts == 1 || p->workers == 0) { fn(ctx, 0, n); return; }
    pthread_mutex_lock(&p->mu);
    p->fn = fn; p->ctx = ctx; p->n = n; p->chunk = chunk;
    p->pending = p->workers;
    p->generation++;
    pthread_cond_broadcast(&p->wake);
    pthread_mutex_unlock(&p->mu);
    run_range(p, p->workers);
    pthread_mutex_lock(&p->mu);
    while (p->pending != 0) pthread_cond_wait(&p->done, &p->mu);
    pthread_mutex_unlock(&p->mu);
}

/* src/main.zig:438-448. */
unsigned zref_default_threads(void) {
    const char *env = getenv("ZLLM_THREADS");
    if (env) {
        long v = strtol(env, NULL, 10);
        if (v > 0) return (unsigned)v;
    }
    long logical = sysconf(_SC_NPROCESSORS_ONLN);
    if (logical < 1) logical = 1;
    FILE *f = fopen("/sys/devices/system/cpu/smt/active", "r");
    if (!f) return (unsigned)logical;
    int c = fgetc(f);
    fclose(f);
    if (c == '1') return (unsigned)(logical / 2 > 0 ? logical / 2 : 1);
    return (unsigned)logical;
}

/* ---- matrix multiply: src/ref/matmul.zig ------------------------------------ */

#define PANEL 32
#define BLOCK_ROWS 8

struct zref_matrix {
    float *data; /* packed panels for f32/f16/bf16, NULL for quantized */
    size_t n, k;
    int type;
    const uint8_t *quant; /* raw rows for quantized types */
};

/* src/ref/matmul.zig:111-133: rows [p*32, p*32+32) decoded k-major, rows past
 * n zero, decoded in pieces of 256 elements. */
static void pack_panel(int type, const uint8_t *bytes, size_t n, size_t k, size_t p, float *dst) {
    uint32_t be, bb;
    zref_layout(type, &be, &bb);
    size_t row_bytes = k / be * bb;
    float buf[256];
    for (size_t col = 0; col < PANEL; col++) {
        size_t j = p * PANEL + col;
        if (j >= n) {
            for (size_t i = 0; i < k; i++) dst[i * PANEL + col] = 0;
            continue;
        }
        const uint8_t *src = bytes + j * row_bytes;
        for (size_t start = 0; start < k; start += 256) {
            size_t len = k - start < 256 ? k - start : 256;
            size_t b0 = start / be * bb;
            zref_dequantize(type, src + b0, buf, len);
            for (size_t i = 0; i < len; i++) dst[(start + i) * PANEL + col] = buf[i];
        }
    }
}

typedef struct { zref_matrix *m; const uint8_t *bytes; } pack_ctx;

static void pack_run(void *ctxp, size_t first, size_t last) {
    pack_ctx *c = (pack_ctx *)ctxp;
    for (size_t p = first; p < last; p++)
        pack_panel(c->m->type, c->bytes, c->m->n, c->m->k, p, c->m->data + p * PANEL * c->m->k);
}

static size_t panels_of(const zref_matrix *m) { return (m->n + PANEL - 1) / PANEL; }

/* src/ref/matmul.zig:56-82. */
zref_matrix *zref_matrix_init(int type, const uint8_t *bytes, size_t n, size_t k, unsigned threads) {
    uint32_t be, bb;
    if (!zref_layout(type, &be, &bb) || k % be != 0) return NULL;
    zref_matrix *m = (zref_matrix *)calloc(1, sizeof *m);
    m->n = n; m->k = k; m->type = type;
    if (type == ZREF_Q8_0 || type == ZREF_Q3_K || type == ZREF_Q4_K || type == ZREF_Q5_K || type == ZREF_Q6_K) {
        m->quant = bytes;
        return m;
    }
    size_t n_panels = panels_of(m);
    if (posix_memalign((void **)&m->data, 64, n_panels * PANEL * k * sizeof(float)) != 0) { free(m); return NULL; }
    pack_ctx ctx = { m, bytes };
    parallel_for(pool_get(threads), n_panels, 1, 1, &ctx, pack_run);
    return m;
}

void zref_matrix_free(zref_matrix *m) {
    if (!m) return;
    free(m->data);
    free(m);
}

/* src/ref/matmul.zig:94-106. */
void zref_matrix_row(const zref_matrix *m, size_t j, float *out) {
    if (m->quant) {
        uint32_t be, bb;
        zref_layout(m->type, &be, &bb);
        size_t row_bytes = m->k / be * bb;
        zref_dequantize(m->type, m->quant + j * row_bytes, out, m->k);
        return;
    }
    const float *base = m->data + (j / PANEL) * PANEL * m->k + j % PANEL;
    for (size_t i = 0; i < m->k; i++) out[i] = base[i * PANEL];
}

typedef struct {
    float *out;
    const float *x;
    const zref_matrix *w;
    size_t rows;
} mm_ctx;

/* src/ref/matmul.zig:262-294: R tokens x 32 outputs; for each i the panel's
 * 32-wide weight row times one broadcast activation per token, accumulated
 * with a separate multiply and add; outputs clipped to n. */
#define MICROKERNEL(R)                                                                     \
    static void microkernel_##R(const mm_ctx *c, const float *wp, size_t p, size_t t0) {   \
        size_t k = c->w->k;                                                                \
        float acc[R][PANEL];                                                               \
        const float *xp[R];                                                                \
        for (int a = 0; a < R; a++) {                                                      \
            xp[a] = c->x + (t0 + a) * k;                                                   \
            for (int cc = 0; cc < PANEL; cc++) acc[a][cc] = 0;                             \
        }                                                                                  \
        for (size_t i = 0; i < k; i++) {                                                   \
            const float *w = wp + i * PANEL;                                               \
            for (int a = 0; a < R; a++) {                                                  \
                float xb = xp[a][i];                                                       \
                for (int cc = 0; cc < PANEL; cc++) {                                       \
                    float prod = xb * w[cc];                                               \
                    acc[a][cc] = acc[a][cc] + prod;                                        \
                }                                                                          \
            }                                                                              \
        }                                                                                  \
        size_t n = c->w->n;                                                                \
        size_t j0 = p * PANEL;                                                             \
        size_t cols = n - j0 < PANEL ? n - j0 : PANEL;                                     \
        for (int a = 0; a < R; a++) memcpy(c->out + (t0 + a) * n + j0, acc[a], cols * sizeof(float)); \
    }

MICROKERNEL(1)
MICROKERNEL(2)
MICROKERNEL(3)
MICROKERNEL(4)
MICROKERNEL(5)
MICROKERNEL(6)
MICROKERNEL(7)
MICROKERNEL(8)

/* src/ref/matmul.zig:135-145: each thread's panel buffer, grown as needed and
 * kept for the life of the thread. */
static __thread float *panel_buf;
static __thread size_t panel_buf_len;

static float *thread_panel(size_t k) {
    if (panel_buf_len < PANEL * k) {
        free(panel_buf);
        if (posix_memalign((void **)&panel_buf, 64, PANEL * k * sizeof(float)) != 0) abort();
        panel_buf_len = PANEL * k;
    }
    return panel_buf;
}

/* src/ref/matmul.zig:177-192. */
static void mm_run(void *ctxp, size_t first, size_t last) {
    const mm_ctx *c = (const mm_ctx *)ctxp;
    for (size_t p = first; p < last; p++) {
        const float *wp;
        if (c->w->quant) {
            float *buf = thread_panel(c->w->k);
            pack_panel(c->w->type, c->w->quant, c->w->n, c->w->k, p, buf);
            wp = buf;
        } else {
            wp = c->w->data + p * PANEL * c->w->k;
        }
        for (size_t t = 0; t < c->rows; t += BLOCK_ROWS) {
            size_t r = c->rows - t < BLOCK_ROWS ? c->rows - t : BLOCK_ROWS;
            switch (r) {
            case 1: microkernel_1(c, wp, p, t); break;
            case 2: microkernel_2(c, wp, p, t); break;
            case 3: microkernel_3(c, wp, p, t); break;
            case 4: microkernel_4(c, wp, p, t); break;
            case 5: microkernel_5(c, wp, p, t); break;
            case 6: microkernel_6(c, wp, p, t); break;
            case 7: microkernel_7(c, wp, p, t); break;
            default: microkernel_8(c, wp, p, t); break;
            }
        }
    }
}

/* src/ref/matmul.zig:160-195 (Activations.f32). */
void zref_matmul(float *out, const float *x, const zref_matrix *w, size_t rows, unsigned threads) {
    mm_ctx ctx = { out, x, w, rows };
    parallel_for(pool_get(threads), panels_of(w), 1, 1, &ctx, mm_run);
}

typedef struct { float *gate; const float *up; size_t ff; } act_ctx;

static void act_run(void *ctxp, size_t first, size_t last) {
    act_ctx *c = (act_ctx *)ctxp;
    for (size_t i = first * c->ff; i < last * c->ff; i++) c->gate[i] = zref_silu(c->gate[i]) * c->up[i];
}

/* src/ref/dense.zig:179-195: gate and up multiplies, then silu(g)*u split by
 * token rows across the pool. */
void zref_gate_up_silu(float *act, const float *x, const zref_matrix *w, size_t half, size_t rows, unsigned threads) {
    float *gu = (float *)malloc(rows * w->n * sizeof(float));
    zref_matmul(gu, x, w, rows, threads);
    float *up = (float *)malloc(rows * half * sizeof(float));
    for (size_t t = 0; t < rows; t++) {
        memcpy(act + t * half, gu + t * w->n, half * sizeof(float));
        memcpy(up + t * half, gu + t * w->n + half, half * sizeof(float));
    }
    act_ctx ctx = { act, up, half };
    parallel_for(pool_get(threads), rows, 1, 1, &ctx, act_run);
    free(up);
    free(gu);
}

/* src/kernels/draft.wgsl:1-4. */
uint32_t zref_argmax(const float *v, size_t n) {
    uint32_t at = 0;
    for (size_t i = 1; i < n; i++)
        if (v[i] > v[at]) at = (uint32_t)i;
    return at;
}

/* ---- GPU-side layouts --------------------------------------------------------- */

/* src/kernels/kernels.zig:144-160. */
uint64_t zref_row_bytes(int type, uint64_t k) {
    if (type == ZREF_Q8_0) return (k + k / 16 + 15) & ~(uint64_t)15;
    uint32_t be, bb;
    if (!zref_layout(type, &be, &bb)) return 0;
    if (type == ZREF_Q6_K) bb = 224;  /* blockStride: padded to 16 bytes by repad */
    if (type == ZREF_IQ4_XS) bb = 144;
    if (type == ZREF_Q3_K) bb = 128;  /* repacked into eight 16-byte units */
    return k / be * bb;
}

/* src/kernels/repack_q3_k.wgsl:30-75. */
static uint32_t q3_scale(const uint8_t *sb, uint32_t i) {
    uint32_t k = i % 4, g = i / 4;
    uint32_t low = (sb[4 * (g % 2) + k] >> (4 * (g / 2))) & 0xf;
    uint32_t high = (sb[8 + k] >> (2 * g)) & 3;
    return low | (high << 4);
}

void zref_repack_q3_k(const uint8_t *src, uint8_t *dst, size_t blocks) {
    for (size_t unit = 0; unit < blocks * 8; unit++) {
        const uint8_t *b = src + (unit / 8) * 110;
        uint32_t s = (uint32_t)(unit % 8), half = s / 4, j = s % 4;
        uint32_t l0 = 0, l1 = 0, hw = 0;
        for (uint32_t l = 0; l < 32; l++) {
            uint32_t q = (b[32 + 32 * half + l] >> (2 * j)) & 3;
            uint32_t h = (b[l] >> (4 * half + j)) & 1;
            uint32_t e = l / 4, byte = l % 4;
            if (e < 4) l0 |= q << (8 * byte + 2 * e);
            else l1 |= q << (8 * byte + 2 * (e - 4));
            hw |= h << (8 * byte + e);
        }
        uint32_t sc0 = (q3_scale(b + 96, 8 * half + 2 * j) + 224) & 0xff;
        uint32_t sc1 = (q3_scale(b + 96, 8 * half + 2 * j + 1) + 224) & 0xff;
        uint32_t d = (uint32_t)b[108] | ((uint32_t)b[109] << 8);
        uint32_t words[4] = { l0, l1, hw, sc0 | (sc1 << 8) | (d << 16) };
        for (int w = 0; w < 4; w++)
            for (int i = 0; i < 4; i++) dst[unit * 16 + 4 * w + i] = (uint8_t)(words[w] >> (8 * i));
    }
}

/* src/kernels/repack_q8_0.wgsl:26-51. */
void zref_repack_q8_0(const uint8_t *src, uint8_t *dst, size_t rows, size_t k) {
    size_t stride = (size_t)zref_row_bytes(ZREF_Q8_0, k);
    size_t blocks = k / 32;
    for (size_t r = 0; r < rows; r++) {
        const uint8_t *raw = src + r * blocks * 34;
        uint8_t *row = dst + r * stride;
        memset(row, 0, stride);
        for (size_t b = 0; b < blocks; b++) {
            memcpy(row + 32 * b, raw + 34 * b + 2, 32);
            row[k + 2 * b] = raw[34 * b];
            row[k + 2 * b + 1] = raw[34 * b + 1];
        }
    }
}

/* src/kernels/kernels.zig:285-295. */
void zref_matmul_slices(uint32_t n, uint32_t k, uint32_t *count, uint32_t *k_slice) {
    const uint32_t tile_n = 128, target = 256, min_slice = 512;
    uint32_t tiles = (n + tile_n - 1) / tile_n;
    uint32_t want = (target + tiles - 1) / tiles;
    uint32_t hi = k / min_slice > 1 ? k / min_slice : 1;
    uint32_t c = want < 1 ? 1 : (want > hi ? hi : want);
    uint32_t ks = (k + c - 1) / c;
    ks = (ks + 31) / 32 * 32;
    *count = (k + ks - 1) / ks;
    *k_slice = ks;
}

/* ---- float64 formula checker: src/kernels/check.zig ---------------------------- */

typedef struct { double *want; const float *x; const float *w; size_t rows, n, k; } f64_ctx;

static void f64_run(void *ctxp, size_t first, size_t last) {
    f64_ctx *c = (f64_ctx *)ctxp;
    for (size_t j = first; j < last; j++) {
        const float *wr = c->w + j * c->k;
        for (size_t t = 0; t < c->rows; t++) {
            const float *xr = c->x + t * c->k;
            double s = 0;
            for (size_t i = 0; i < c->k; i++) s += (double)xr[i] * (double)wr[i];
            c->want[t * c->n + j] = s;
        }
    }
}

void zref_matmul_f64(double *want, const float *x, const float *w, size_t rows, size_t n, size_t k, unsigned threads) {
    f64_ctx ctx = { want, x, w, rows, n, k };
    parallel_for(pool_get(threads), n, 1, 1, &ctx, f64_run);
}

/* ---- activations rounded to 8-bit blocks: the quantized prefill multiply --------- */

/* x >= 0 rounded to binary16 precision (nearest, ties to even) and widened
 * back, as src/kernels/quantize_q8.wgsl:52-60 does on raw bits. Values above
 * the f16 range do not occur: x is a block maximum divided by 127. */
float zref_f16_round(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if (((u >> 23) & 0xffu) < 113u) {
        /* Below f16's normal range: multiples of 2^-24. */
        return nearbyintf(x * 16777216.0f) * (1.0f / 16777216.0f);
    }
    u = (u + 0xfffu + ((u >> 13) & 1u)) & 0xffffe000u;
    memcpy(&x, &u, 4);
    return x;
}

/* ggml's nearest_int: the f32 addition rounds ties to even
 * (src/ref/matmul.zig:217-219,240-242). */
static int32_t nearest_int(float y) {
    float s = y + 12582912.0f;
    int32_t bits;
    memcpy(&bits, &s, 4);
    return bits - 0x4b400000;
}

/* src/ref/matmul.zig:197-247 with the integers and block scales kept apart
 * (src/kernels/quantize_q8.wgsl:11-22): x[i] ~ q[i] * d[i / block]. */
int zref_quantize_q8(const float *x, size_t n, unsigned block, int8_t *q, float *d) {
    if ((block != 32 && block != 256) || n % block != 0) return -1;
    for (size_t b = 0; b < n; b += block) {
        const float *v = x + b;
        if (block == 32) {
            float amax = 0;
            for (unsigned i = 0; i < 32; i++) {
                float a = fabsf(v[i]);
                if (a > amax) amax = a;
            }
            float d32 = amax / 127.0f;
            float id = amax != 0 ? 127.0f / amax : 0.0f;
            d[b / 32] = zref_f16_round(d32);
            for (unsigned i = 0; i < 32; i++) {
                float scaled = v[i] * id;
                q[b + i] = (int8_t)nearest_int(scaled);
            }
        } else {
            float amax = 0, max = 0;
            for (unsigned i = 0; i < 256; i++) {
                float a = fabsf(v[i]);
                if (a > amax) {
                    amax = a;
                    max = v[i];
                }
            }
            if (amax == 0) {
                d[b / 256] = 0;
                memset(q + b, 0, 256);
                continue;
            }
            float iscale = -127.0f / max;
            d[b / 256] = 1.0f / iscale;
            for (unsigned i = 0; i < 256; i++) {
                float scaled = iscale * v[i];
                int32_t r = nearest_int(scaled);
                q[b + i] = (int8_t)(r < 127 ? r : 127);
            }
        }
    }
    return 0;
}

/* src/ref/matmul.zig:197-247: a row rounded as the multiply will see it. */
int zref_round_like_llama(int type, float *x, size_t n) {
    if (type == ZREF_Q8_0 || type == ZREF_Q3_K || type == ZREF_Q4_K || type == ZREF_Q5_K || type == ZREF_Q6_K ||
        type == ZREF_IQ4_XS) {
        unsigned block = type == ZREF_Q8_0 ? 32 : 256;
        int8_t *q = malloc(n);
        float *d = malloc((n / block + 1) * sizeof(float));
        int r = q && d ? zref_quantize_q8(x, n, block, q, d) : -1;
        if (r == 0)
            for (size_t i = 0; i < n; i++) x[i] = (float)q[i] * d[i / block];
        free(q);
        free(d);
        return r;
    }
    if (type == ZREF_BF16) {
        for (size_t i = 0; i < n; i++) x[i] = zref_bf16_round(x[i]);
        return 0;
    }
    if (type == ZREF_F16) {
        for (size_t i = 0; i < n; i++) {
            float a = zref_f16_round(fabsf(x[i]));
            x[i] = copysignf(a, x[i]);
        }
        return 0;
    }
    return type == ZREF_F32 ? 0 : -1;
}

/* src/kernels/quantize_q8.wgsl:1-9,66-104: rows of k values computed by
 * `mode` (0: x; 1: RMSNorm(x) * nw; 2: silu(gate) * up over rows of gate | up),
 * then rounded block by block. */
int zref_quantize_q8_rows(const float *x, size_t rows, size_t k, unsigned block, unsigned mode, float eps,
                          const float *nw, int8_t *q, float *d) {
    float *row = malloc(k * sizeof(float));
    if (!row) return -1;
    int r = 0;
    for (size_t t = 0; t < rows && r == 0; t++) {
        if (mode == 2) {
            const float *g = x + t * 2 * k, *u = g + k;
            for (size_t i = 0; i < k; i++) row[i] = zref_silu(g[i]) * u[i];
        } else {
            memcpy(row, x + t * k, k * sizeof(float));
            if (mode == 1) zref_rms_norm(row, nw, k, eps);
        }
        r = zref_quantize_q8(row, k, block, q + t * k, d + t * (k / block));
    }
    free(row);
    return r;
}

/* Unit u (32 weights) of a 256-weight block as the int8 prefill multiply sees
 * it: signed integers q, a scale for each half of sixteen and a minimum
 * (src/kernels/quant/q3_k.wgsl, q4_k.wgsl, q5_k.wgsl, q6_k.wgsl: head, scales,
 * quad_i8). b is the block as the file stores it. */
static void kquant_unit(int type, const uint8_t *b, unsigned u, int32_t q[32], float *s0, float *s1, float *mn) {
    if (type == ZREF_Q4_K || type == ZREF_Q5_K) {
        float d = zref_half(rd16(b)), dmin = zref_half(rd16(b + 2));
        uint8_t sc, m;
        zref_scale_min_k4(u, b + 4, &sc, &m);
        const uint8_t *qs = b + (type == ZREF_Q4_K ? 16 : 48) + 32 * (u / 2);
        for (unsigned i = 0; i < 32; i++) {
            q[i] = u & 1 ? qs[i] >> 4 : qs[i] & 0xF;
            if (type == ZREF_Q5_K) q[i] += ((b[16 + i] >> u) & 1) << 4;
        }
        *s0 = *s1 = d * (float)sc;
        *mn = dmin * (float)m;
    } else if (type == ZREF_Q6_K) {
        unsigned n = u / 4, c = u % 4;
        float d = zref_half(rd16(b + 208));
        const uint8_t *ql = b + 64 * n + 32 * (c % 2), *qh = b + 128 + 32 * n;
        const int8_t *sc = (const int8_t *)(b + 192 + 8 * n + 2 * c);
        for (unsigned i = 0; i < 32; i++)
            q[i] = (int32_t)(((ql[i] >> (4 * (c / 2))) & 0xF) | (((qh[i] >> (2 * c)) & 3) << 4)) - 32;
        *s0 = d * (float)sc[0];
        *s1 = d * (float)sc[1];
        *mn = 0.f;
    } else {  /* ZREF_Q3_K */
        unsigned n = u / 4, j = u % 4;
        float d = zref_half(rd16(b + 108));
        int8_t scales[16];
        q3_k_scales(b, scales);
        for (unsigned i = 0; i < 32; i++)
            q[i] = (int32_t)((b[32 + 32 * n + i] >> (2 * j)) & 3) - (((b[i] >> (4 * n + j)) & 1) ? 0 : 4);
        *s0 = d * (float)((int)scales[8 * n + 2 * j] - 32);
        *s1 = d * (float)((int)scales[8 * n + 2 * j + 1] - 32);
        *mn = 0.f;
    }
}

/* out[t][j] = sum over 32-weight units of dx * (s0 * sum(q * qx) over the first
 * sixteen + s1 * the same over the second sixteen - m * sum(qx))
 * (src/kernels/matmul_quant.wgsl:1-9,130-160), the integer sums exact and the
 * scaled terms added in double. Weights are file-layout blocks (Q8_0: 34
 * bytes; Q3_K 110; Q4_K 144; Q5_K 176; Q6_K 210); dx has one scale per 32
 * (Q8_0) or 256 (the K formats) activations. */
int zref_matmul_q8(int type, const uint8_t *w, const int8_t *qx, const float *dx, size_t rows, size_t n, size_t k, double *out) {
    size_t bb;
    switch (type) {
    case ZREF_Q8_0: bb = 34; break;
    case ZREF_Q3_K: bb = 110; break;
    case ZREF_Q4_K: bb = 144; break;
    case ZREF_Q5_K: bb = 176; break;
    case ZREF_Q6_K: bb = 210; break;
    default: return -1;
    }
    for (size_t t = 0; t < rows; t++) {
        const int8_t *xr = qx + t * k;
        for (size_t j = 0; j < n; j++) {
            double sum = 0;
            if (type == ZREF_Q8_0) {
                const uint8_t *row = w + j * (k / 32) * bb;
                for (size_t u = 0; u < k / 32; u++) {
                    const uint8_t *b = row + u * bb;
                    int32_t dot = 0;
                    for (unsigned i = 0; i < 32; i++) dot += (int32_t)(int8_t)b[2 + i] * xr[u * 32 + i];
                    sum += (double)dx[t * (k / 32) + u] * ((double)zref_half(rd16(b)) * dot);
                }
            } else {
                const uint8_t *row = w + j * (k / 256) * bb;
                for (size_t blk = 0; blk < k / 256; blk++) {
                    for (unsigned u = 0; u < 8; u++) {
                        int32_t q[32], dot0 = 0, dot1 = 0, xs = 0;
                        float s0, s1, mn;
                        kquant_unit(type, row + blk * bb, u, q, &s0, &s1, &mn);
                        for (unsigned i = 0; i < 32; i++) {
                            int32_t xv = xr[blk * 256 + u * 32 + i];
                            if (i < 16) dot0 += q[i] * xv;
                            else dot1 += q[i] * xv;
                            xs += xv;
                        }
                        sum += (double)dx[t * (k / 256) + blk] * ((double)s0 * dot0 + (double)s1 * dot1 - (double)mn * xs);
                    }
                }
            }
            out[t * n + j] = sum;
        }
    }
    return 0;
}
