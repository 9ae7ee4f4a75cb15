/*
 * CPU baseline of the "dequantise, then FP32 GEMM" branch of the reference's Gguf.linear - TEST / BENCHMARK
 * INFRASTRUCTURE ONLY (loaded by tests/ and by bench.py's cpu_baseline leg; the product never links it).
 *
 * What the reference's CPU backend runs for a K-quant weight at more than one row, or any weight beyond
 * jitnn.gguf.tiledRows rows (ops/Gguf.java:90-96): y = x.matmul(dequantize(w), false, true), i.e.
 *   1. Gguf.Dequantize.reference (ops/Gguf.java:127-133): the scalar per-value decode on ONE thread (the operator has no
 *      cpu() kernel, so CpuExecutor.host falls back to its reference, engine/CpuExecutor.java:233-239) - jo_dequantize;
 *   2. MatMul.cpu -> CpuKernels.matmul (ops/CpuKernels.java:89-108): both operands packed on every call (the dequantised
 *      weight is not persistent, so its packing is not cached) and Gemm.compute (cpu/Gemm.java:541-573):
 *        packA: panels of MR = 6 rows of x; packB: panels of NR = 2 vectors of weight rows (cpu/Gemm.java:121-176);
 *        tiles of at most 16 A panels x 256 / NR B panels, cut finer until there are 2 x threads of them or a tile
 *        would hold fewer than 2^20 multiply-adds (cpu/Gemm.java:543-556; defaults JitnnConfig.java:247-256);
 *        per tile: K in blocks of KC = 256, B panel outer, A panel inner, a 6 x NR register tile of vector FMAs, stored on
 *        the first K block and added to C afterwards (cpu/Gemm.java:575-640);
 *      parallel loops over at most `threads` contiguous chunks (cpu/Cpu.java:81-103), threads = the physical cores of one
 *      socket by default (cpu/Cpu.java:221-225).
 * The vector is the widest the machine has, as FloatVector.SPECIES_PREFERRED is (cpu/Gemm.java:40): 16 floats with
 * AVX-512, 8 with AVX2 + FMA, else 4-float SSE arithmetic without fused multiply-add.
 * The summation order (K blocks of 256, FP32 FMAs) is the reference's; its exact bits are not pinned by any
 * reference-held vector (tests check this file against the FP64 oracle within FP32 rounding).
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define JO_API __attribute__((visibility("default")))

int jo_dequantize(int fmt, const uint8_t *w, long numel, float *y); /* jitnn_oracle.c */

enum { MR = 6, KC = 256, MC_PANELS = 16, NC = 256 };
static const long TILE_MIN_MACS = 1L << 20;
static const int PACK_GRAIN = 1 << 15;

static double now_s(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

/* ---- Cpu.parallelFor: [0, n) in at most `threads` contiguous chunks of at least `grain` indices */
typedef void (*range_fn)(void *ctx, int from, int to);
typedef struct {
    range_fn fn;
    void *ctx;
    int from, to;
} chunk_t;

static void *chunk_main(void *p) {
    chunk_t *c = (chunk_t *)p;
    c->fn(c->ctx, c->from, c->to);
    return NULL;
}

static void parallel_for(int n, int grain, int threads, range_fn fn, void *ctx) {
    long byg = n / (long)(grain > 1 ? grain : 1);
    int chunks = (int)(byg < 1 ? 1 : byg);
    if (chunks > threads) chunks = threads;
    if (chunks <= 1) {
        fn(ctx, 0, n);
        return;
    }
    pthread_t tid[256];
    chunk_t ch[256];
    if (chunks > 256) chunks = 256;
    for (int c = 0; c < chunks; c++) {
        ch[c].fn = fn;
        ch[c].ctx = ctx;
        ch[c].from = (int)((long)n * c / chunks);
        ch[c].to = (int)((long)n * (c + 1) / chunks);
    }
    for (int c = 1; c < chunks; c++) pthread_create(&tid[c], NULL, chunk_main, &ch[c]);
    chunk_main(&ch[0]);
    for (int c = 1; c < chunks; c++) pthread_join(tid[c], NULL);
}

static int panels(int rows, int w) { return (rows + w - 1) / w; }

/* ---- pack: src is row-major [rows, k] (value (x, q) at x * k + q); panel p holds rows p*w .. p*w + w - 1 as
 * dst[p * k * w + q * w + c] (Gemm.packPanel, the strided branch: a row of the source is not contiguous across the panel) */
typedef struct {
    const float *src;
    float *dst;
    int rows, k, w;
} pack_ctx;

static void pack_range(void *p, int from, int to) {
    pack_ctx *c = (pack_ctx *)p;
    for (int pn = from; pn < to; pn++) {
        int x0 = pn * c->w;
        int valid = c->rows - x0 < c->w ? c->rows - x0 : c->w;
        float *base = c->dst + (size_t)pn * c->k * c->w;
        for (int col = 0; col < c->w; col++) {
            if (col >= valid) {
                for (int q = 0; q < c->k; q++) base[(size_t)q * c->w + col] = 0.f;
                continue;
            }
            const float *s = c->src + (size_t)(x0 + col) * c->k;
            for (int q = 0; q < c->k; q++) base[(size_t)q * c->w + col] = s[q];
        }
    }
}

static void pack(const float *src, int rows, int k, int w, float *dst, int threads) {
    pack_ctx c = {src, dst, rows, k, w};
    int grain = PACK_GRAIN / (k * w > 1 ? k * w : 1);
    if (grain < 1) grain = 1;
    parallel_for(panels(rows, w), grain, threads, pack_range, &c);
}

/* ---- the 6 x NR micro-kernel in three vector widths */
typedef void (*kernel_fn)(const float *ap, const float *bp, int kc, float *out /* MR x NR */);

__attribute__((target("avx512f"))) static void kernel_avx512(const float *ap, const float *bp, int kc, float *out) {
    __m512 c[MR][2];
    for (int i = 0; i < MR; i++) c[i][0] = c[i][1] = _mm512_setzero_ps();
    for (int q = 0; q < kc; q++) {
        const __m512 b0 = _mm512_loadu_ps(bp), b1 = _mm512_loadu_ps(bp + 16);
        for (int i = 0; i < MR; i++) {
            const __m512 a = _mm512_set1_ps(ap[i]);
            c[i][0] = _mm512_fmadd_ps(a, b0, c[i][0]);
            c[i][1] = _mm512_fmadd_ps(a, b1, c[i][1]);
        }
        ap += MR;
        bp += 32;
    }
    for (int i = 0; i < MR; i++) {
        _mm512_storeu_ps(out + i * 32, c[i][0]);
        _mm512_storeu_ps(out + i * 32 + 16, c[i][1]);
    }
}

__attribute__((target("avx2,fma"))) static void kernel_avx2(const float *ap, const float *bp, int kc, float *out) {
    __m256 c[MR][2];
    for (int i = 0; i < MR; i++) c[i][0] = c[i][1] = _mm256_setzero_ps();
    for (int q = 0; q < kc; q++) {
        const __m256 b0 = _mm256_loadu_ps(bp), b1 = _mm256_loadu_ps(bp + 8);
        for (int i = 0; i < MR; i++) {
            const __m256 a = _mm256_set1_ps(ap[i]);
            c[i][0] = _mm256_fmadd_ps(a, b0, c[i][0]);
            c[i][1] = _mm256_fmadd_ps(a, b1, c[i][1]);
        }
        ap += MR;
        bp += 16;
    }
    for (int i = 0; i < MR; i++) {
        _mm256_storeu_ps(out + i * 16, c[i][0]);
        _mm256_storeu_ps(out + i * 16 + 8, c[i][1]);
    }
}

static void kernel_sse(const float *ap, const float *bp, int kc, float *out) {
    __m128 c[MR][2];
    for (int i = 0; i < MR; i++) c[i][0] = c[i][1] = _mm_setzero_ps();
    for (int q = 0; q < kc; q++) {
        const __m128 b0 = _mm_loadu_ps(bp), b1 = _mm_loadu_ps(bp + 4);
        for (int i = 0; i < MR; i++) {
            const __m128 a = _mm_set1_ps(ap[i]);
            c[i][0] = _mm_add_ps(_mm_mul_ps(a, b0), c[i][0]);
            c[i][1] = _mm_add_ps(_mm_mul_ps(a, b1), c[i][1]);
        }
        ap += MR;
        bp += 8;
    }
    for (int i = 0; i < MR; i++) {
        _mm_storeu_ps(out + i * 8, c[i][0]);
        _mm_storeu_ps(out + i * 8 + 4, c[i][1]);
    }
}

/* lanes of the widest vector: 16, 8 or 4 */
JO_API int jo_cpu_vector_lanes(void) {
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f")) return 16;
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) return 8;
    return 4;
}

typedef struct {
    const float *ap, *bp;
    float *c;
    int m, n, k, nr, pm, pn, fm, fn, tn;
    kernel_fn kernel;
} tile_ctx;

/* Gemm.tile over A panels [ip0, ip1) and B panels [jp0, jp1): C [m, n] row-major, ldc = n */
static void tile_range(void *p, int from, int to) {
    tile_ctx *t = (tile_ctx *)p;
    float out[MR * 32];
    const int nr = t->nr;
    for (int ti_tj = from; ti_tj < to; ti_tj++) {
        const int ti = ti_tj / t->tn, tj = ti_tj % t->tn;
        const int ip0 = ti * t->fm, ip1 = (ti + 1) * t->fm < t->pm ? (ti + 1) * t->fm : t->pm;
        const int jp0 = tj * t->fn, jp1 = (tj + 1) * t->fn < t->pn ? (tj + 1) * t->fn : t->pn;
        for (int pc = 0; pc < t->k; pc += KC) {
            const int kc = t->k - pc < KC ? t->k - pc : KC;
            const int first = pc == 0;
            for (int jp = jp0; jp < jp1; jp++) {
                const float *bo = t->bp + ((size_t)jp * t->k + pc) * nr;
                for (int ip = ip0; ip < ip1; ip++) {
                    t->kernel(t->ap + ((size_t)ip * t->k + pc) * MR, bo, kc, out);
                    const int i0 = ip * MR, j0 = jp * nr;
                    const int rows = t->m - i0 < MR ? t->m - i0 : MR, cols = t->n - j0 < nr ? t->n - j0 : nr;
                    for (int r = 0; r < rows; r++) {
                        float *crow = t->c + (size_t)(i0 + r) * t->n + j0;
                        if (first) {
                            for (int j = 0; j < cols; j++) crow[j] = out[r * nr + j];
                        } else {
                            for (int j = 0; j < cols; j++) crow[j] = crow[j] + out[r * nr + j];
                        }
                    }
                }
            }
        }
    }
}

/* C [m, n] = A [m, k] B [n, k]^T: pack both, then Gemm.compute.  Returns 0, or -2 when out of memory. */
JO_API int jo_cpu_gemm_nt(const float *a, const float *b, float *c, int m, int n, int k, int threads) {
    const int lanes = jo_cpu_vector_lanes(), nr = 2 * lanes;
    const int pm = panels(m, MR), pn = panels(n, nr);
    float *ap = (float *)malloc(sizeof(float) * (size_t)pm * (k > 1 ? k : 1) * MR);
    float *bp = (float *)malloc(sizeof(float) * (size_t)pn * (k > 1 ? k : 1) * nr);
    if (!ap || !bp) {
        free(ap);
        free(bp);
        return -2;
    }
    if (threads < 1) threads = 1;
    pack(a, m, k, MR, ap, threads);
    pack(b, n, k, nr, bp, threads);
    int mcp = MC_PANELS < pm ? MC_PANELS : pm;
    int ncp = NC / nr > 1 ? NC / nr : 1;
    if (ncp > pn) ncp = pn;
    const long macs = (long)m * n * (k > 1 ? k : 1);
    long want = macs / TILE_MIN_MACS;
    if (want > 2L * threads) want = 2L * threads;
    if (want < 1) want = 1;
    while ((long)panels(pm, mcp) * panels(pn, ncp) < want && (mcp > 1 || ncp > 1)) {
        if ((mcp >= ncp * 2 && mcp > 1) || ncp == 1) mcp = (mcp + 1) / 2;
        else ncp = (ncp + 1) / 2;
    }
    tile_ctx t = {ap, bp, c, m, n, k, nr, pm, pn, mcp, ncp, panels(pn, ncp),
                  lanes == 16 ? kernel_avx512 : lanes == 8 ? kernel_avx2 : kernel_sse};
    const int tm = panels(pm, mcp);
    const long work = 2L * m * n * (k > 1 ? k : 1);
    parallel_for(tm * t.tn, work < (1 << 16) ? tm * t.tn : 1, threads, tile_range, &t);
    free(ap);
    free(bp);
    return 0;
}

/* Gguf.linear's dequantise + GEMM branch: y [rows, n] = x [rows, k] . dequantize(w [n, k])^T (+ bias).
 * seconds[0] = the dequantiser (one thread), seconds[1] = packing + GEMM (`threads` threads); seconds may be NULL. */
JO_API int jo_dequant_gemm(int fmt, const float *x, const uint8_t *w, const float *bias, float *y, int rows, int n, int k, int threads,
                           double *seconds) {
    float *wd = (float *)malloc(sizeof(float) * (size_t)n * k);
    if (!wd) return -2;
    const double t0 = now_s();
    int rc = jo_dequantize(fmt, w, (long)n * k, wd);
    const double t1 = now_s();
    if (rc == 0) rc = jo_cpu_gemm_nt(x, wd, y, rows, n, k, threads);
    if (rc == 0 && bias) { /* y.add(bias): a second elementwise operator (ops/Gguf.java:97) */
        for (int r = 0; r < rows; r++)
            for (int c = 0; c < n; c++) y[(size_t)r * n + c] = y[(size_t)r * n + c] + bias[c];
    }
    const double t2 = now_s();
    if (seconds) {
        seconds[0] = t1 - t0;
        seconds[1] = t2 - t1;
    }
    free(wd);
    return rc;
}
