/*
 * CPU oracle for the GGUF quantised-weight linear path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, what the reference's host
 * ("reference" / CPU backend) implementation computes for the path, so that the HIP library can be
 * checked against it.  Nothing in the shipped library calls it: only tests/, the smoke check and the
 * benchmark's cpu_baseline leg load liboracle.so.
 *
 * Build with -ffp-contract=off and without -ffast-math: Java never fuses a*b+c and evaluates float
 * expressions strictly left to right in binary32, and the dequantised values must match bit for bit.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference root).
 * Pinning status (what fixes each function besides this restatement) is listed at the bottom.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define JO_API __attribute__((visibility("default")))

/* ggml type ids as stored in GGUF files: jitnn-gguf/src/main/java/ai/beestream/jitnn/gguf/GgmlType.java:27-65 */
enum { JO_Q4_0 = 2, JO_Q4_1 = 3, JO_Q5_0 = 6, JO_Q5_1 = 7, JO_Q8_0 = 8, JO_Q2_K = 10, JO_Q3_K = 11, JO_Q4_K = 12, JO_Q5_K = 13, JO_Q6_K = 14 };

/* values per block / bytes per block: jitnn-core/src/main/java/ai/beestream/jitnn/DType.java:75-98 */
JO_API int jo_block_values(int fmt) {
    switch (fmt) {
    case JO_Q8_0: case JO_Q4_0: case JO_Q4_1: case JO_Q5_0: case JO_Q5_1: return 32;
    case JO_Q4_K: case JO_Q5_K: case JO_Q6_K: case JO_Q2_K: case JO_Q3_K: return 256;
    default: return 0;
    }
}

JO_API int jo_block_bytes(int fmt) {
    switch (fmt) {
    case JO_Q8_0: return 34;
    case JO_Q4_0: return 18;
    case JO_Q4_1: return 20;
    case JO_Q4_K: return 144;
    case JO_Q5_K: return 176;
    case JO_Q6_K: return 210;
    case JO_Q5_0: return 22;
    case JO_Q5_1: return 24;
    case JO_Q2_K: return 84;
    case JO_Q3_K: return 110;
    default: return 0;
    }
}

/* ---- IEEE binary16 <-> binary32 (tornado-api HalfFloat semantics: decode exact, encode RNE) ---- */

JO_API float jo_half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

JO_API uint16_t jo_float_to_half(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7fffffffu;
    if (abs >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x200u | ((abs >> 13) & 0x3ffu) : 0));
    }
    if (abs >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (abs < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
        if (abs < 0x33000000u) { /* < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
            return (uint16_t)sign;
        }
        int e = (int)(abs >> 23);               /* biased binary32 exponent */
        uint32_t man = (abs & 0x7fffffu) | 0x800000u;
        int shift = 126 - e;                     /* 14 .. 24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q);
    }
    uint32_t e = (abs >> 23) - 112;
    uint32_t man = abs & 0x7fffffu;
    uint32_t h = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) {
        h++; /* carries into the exponent correctly */
    }
    return (uint16_t)(sign | h);
}

static inline int u8(const uint8_t *w, long at) { return w[at]; }
static inline int i8(const uint8_t *w, long at) { return (int8_t)w[at]; }
static inline float f16(const uint8_t *w, long at) { return jo_half_to_float((uint16_t)(w[at] | (w[at + 1] << 8))); }

/* jitnn-core/src/main/java/ai/beestream/jitnn/kernels/GgufKernels.java:74-83 */
static int scale_min(const uint8_t *w, long s, int j, int part) {
    if (j < 4) {
        return u8(w, s + j + 4 * part) % 64;
    }
    int low = part == 0 ? u8(w, s + j + 4) % 16 : u8(w, s + j + 4) / 16;
    return low + (u8(w, s + j - 4 + 4 * part) / 64) * 16;
}

/* GgufKernels.java:85-91 */
static float q4_0(const uint8_t *w, long i) {
    long base = (i / 32) * 18;
    int e = (int)(i % 32);
    int b = u8(w, base + 2 + e % 16);
    int q = e < 16 ? b % 16 : b / 16;
    return (float)(q - 8) * f16(w, base);
}

/* GgufKernels.java:93-99 */
static float q4_1(const uint8_t *w, long i) {
    long base = (i / 32) * 20;
    int e = (int)(i % 32);
    int b = u8(w, base + 4 + e % 16);
    int q = e < 16 ? b % 16 : b / 16;
    float p = (float)q * f16(w, base);
    return p + f16(w, base + 2);
}

/* GgufKernels.java:101-111 */
static float q4_k(const uint8_t *w, long i) {
    long base = (i / 256) * 144;
    int e = (int)(i % 256);
    int j = e / 64;
    int half = (e % 64) / 32;
    int l = e % 32;
    int sub = 2 * j + half;
    int b = u8(w, base + 16 + 32 * j + l);
    int q = half == 0 ? b % 16 : b / 16;
    float a = f16(w, base) * (float)scale_min(w, base + 4, sub, 0);
    a = a * (float)q;
    float m = f16(w, base + 2) * (float)scale_min(w, base + 4, sub, 1);
    return a - m;
}

/* GgufKernels.java:113-125 */
static float q5_k(const uint8_t *w, long i) {
    long base = (i / 256) * 176;
    int e = (int)(i % 256);
    int j = e / 64;
    int half = (e % 64) / 32;
    int l = e % 32;
    int sub = 2 * j + half;
    int b = u8(w, base + 48 + 32 * j + l);
    int q = half == 0 ? b % 16 : b / 16;
    int hbit = (u8(w, base + 16 + l) / (1 << sub)) % 2;
    q = q + 16 * hbit;
    float a = f16(w, base) * (float)scale_min(w, base + 4, sub, 0);
    a = a * (float)q;
    float m = f16(w, base + 2) * (float)scale_min(w, base + 4, sub, 1);
    return a - m;
}

/* GgufKernels.java:127-140 */
static float q6_k(const uint8_t *w, long i) {
    long base = (i / 256) * 210;
    int e = (int)(i % 256);
    int n = e / 128;
    int r = e % 128;
    int k = r / 32;
    int l = r % 32;
    int lb = u8(w, base + 64 * n + l + (k % 2) * 32);
    int low = k < 2 ? lb % 16 : lb / 16;
    int hb = (u8(w, base + 128 + 32 * n + l) / (1 << (2 * k))) % 4;
    int q = low + 16 * hb - 32;
    int sc = i8(w, base + 192 + 8 * n + l / 16 + 2 * k);
    float a = f16(w, base + 208) * (float)sc;
    return a * (float)q;
}

/* GgufKernels.java:143-145 */
static int bit32(const uint8_t *w, long at, int bit) { return (u8(w, at + bit / 8) / (1 << (bit % 8))) % 2; }

/* GgufKernels.java:148-154 */
static float q5_0(const uint8_t *w, long i) {
    long base = (i / 32) * 22;
    int e = (int)(i % 32);
    int b = u8(w, base + 6 + e % 16);
    int q = (e < 16 ? b % 16 : b / 16) + 16 * bit32(w, base + 2, e);
    return (float)(q - 16) * f16(w, base);
}

/* GgufKernels.java:157-163 */
static float q5_1(const uint8_t *w, long i) {
    long base = (i / 32) * 24;
    int e = (int)(i % 32);
    int b = u8(w, base + 8 + e % 16);
    int q = (e < 16 ? b % 16 : b / 16) + 16 * bit32(w, base + 4, e);
    float p = (float)q * f16(w, base);
    return p + f16(w, base + 2);
}

/* GgufKernels.java:166-175 */
static float q2_k(const uint8_t *w, long i) {
    long base = (i / 256) * 84;
    int e = (int)(i % 256);
    int n = e / 128;
    int j = (e % 128) / 32;
    int l = e % 32;
    int sc = u8(w, base + n * 8 + j * 2 + l / 16);
    int q = (u8(w, base + 16 + n * 32 + l) / (1 << (2 * j))) % 4;
    float a = f16(w, base + 80) * (float)(sc % 16);
    a = a * (float)q;
    float m = f16(w, base + 82) * (float)(sc / 16);
    return a - m;
}

/* GgufKernels.java:181-185 */
static int scale3(const uint8_t *w, long s, int is) {
    int low = is < 8 ? u8(w, s + is) % 16 : u8(w, s + is - 8) / 16;
    int high = (u8(w, s + 8 + is % 4) / (1 << (2 * (is / 4)))) % 4;
    return low + 16 * high;
}

/* GgufKernels.java:188-198 */
static float q3_k(const uint8_t *w, long i) {
    long base = (i / 256) * 110;
    int e = (int)(i % 256);
    int n = e / 128;
    int j = (e % 128) / 32;
    int l = e % 32;
    int is = n * 8 + j * 2 + l / 16;
    int q = (u8(w, base + 32 + n * 32 + l) / (1 << (2 * j))) % 4;
    int high = (u8(w, base + l) / (1 << (4 * n + j))) % 2;
    float a = f16(w, base + 108) * (float)(scale3(w, base + 96, is) - 32);
    return a * (float)(q - (high == 1 ? 0 : 4));
}

/* Q8_0 element: jitnn-core/src/main/java/ai/beestream/jitnn/ops/Quant.java:137-144, Tensor.java:546-553 */
static float q8_0(const uint8_t *w, long i) {
    long base = (i / 32) * 34;
    return f16(w, base) * (float)i8(w, base + 2 + i % 32);
}

/* GgufKernels.value (GgufKernels.java:201-223) extended with Q8_0; fmt is the ggml type id. NaN for unknown formats. */
JO_API float jo_value(int fmt, const uint8_t *w, long i) {
    switch (fmt) {
    case JO_Q4_0: return q4_0(w, i);
    case JO_Q4_1: return q4_1(w, i);
    case JO_Q4_K: return q4_k(w, i);
    case JO_Q5_K: return q5_k(w, i);
    case JO_Q6_K: return q6_k(w, i);
    case JO_Q5_0: return q5_0(w, i);
    case JO_Q5_1: return q5_1(w, i);
    case JO_Q2_K: return q2_k(w, i);
    case JO_Q3_K: return q3_k(w, i);
    case JO_Q8_0: return q8_0(w, i);
    default: return NAN;
    }
}

/* Gguf.Dequantize.reference (ops/Gguf.java:127-133), Quant.Dequantize.reference (ops/Quant.java:137-144),
 * Tensor.toFloatArray on block tensors (Tensor.java:539-555): y[i] = value(w, i). */
JO_API int jo_dequantize(int fmt, const uint8_t *w, long numel, float *y) {
    if (jo_block_values(fmt) == 0) {
        return -1;
    }
    for (long i = 0; i < numel; i++) {
        y[i] = jo_value(fmt, w, i);
    }
    return 0;
}

/* Gguf.MatVec.reference (ops/Gguf.java:187-205): per output column the row is decoded to double once,
 * then each input row accumulates in double, j ascending; y[r*n+c] = (float)acc.  No bias here. */
JO_API int jo_matvec_ref(int fmt, const float *x, const uint8_t *w, float *y, int rows, int n, int k) {
    if (jo_block_values(fmt) == 0 || k % jo_block_values(fmt) != 0) {
        return -1;
    }
    double *wr = (double *)malloc(sizeof(double) * (size_t)k);
    if (!wr) {
        return -2;
    }
    for (int c = 0; c < n; c++) {
        for (int j = 0; j < k; j++) {
            wr[j] = (double)jo_value(fmt, w, (long)c * k + j);
        }
        for (int r = 0; r < rows; r++) {
            double acc = 0;
            for (int j = 0; j < k; j++) {
                acc += wr[j] * (double)x[(long)r * k + j];
            }
            y[(long)r * n + c] = (float)acc;
        }
    }
    free(wr);
    return 0;
}

/* Quant.LinearQ8.reference (ops/Quant.java:171-187): the bias seeds the double accumulator;
 * each term is (double)f16(d) * q * x evaluated left to right in double. */
JO_API int jo_linear_q8_ref(const float *x, const uint8_t *w, const float *bias, float *y, int m, int n, int k) {
    if (k % 32 != 0) {
        return -1;
    }
    int blocks = k / 32;
    for (int i = 0; i < m; i++) {
        for (int r = 0; r < n; r++) {
            double acc = bias ? (double)bias[r] : 0.0;
            for (int j = 0; j < k; j++) {
                long off = ((long)r * blocks + j / 32) * 34;
                double t = (double)f16(w, off) * (double)i8(w, off + 2 + j % 32);
                acc += t * (double)x[(long)i * k + j];
            }
            y[(long)i * n + r] = (float)acc;
        }
    }
    return 0;
}

/* MatMul.reference with tb=1 (ops/MatMul.java:597-625): C[m,n] = A[m,k] . B[n,k]^T, double accumulation. */
JO_API void jo_matmul_nt_ref(const float *a, const float *b, float *c, int m, int n, int k) {
    for (int i = 0; i < m; i++) {
        for (int j = 0; j < n; j++) {
            double acc = 0;
            for (int p = 0; p < k; p++) {
                acc += (double)a[(long)i * k + p] * (double)b[(long)j * k + p];
            }
            c[(long)i * n + j] = (float)acc;
        }
    }
}

/* Gguf.linear as the host executes it (ops/Gguf.java:76-98): Q8_0 -> Quant.linear (bias inside the
 * accumulator); rows==1 for the five matvec formats, or rows<=tiled_rows for Q4_0/Q4_1/Q5_K -> matvec;
 * otherwise dequantise + matmul(x, W^T); then the bias is added as a separate FP32 add (Gguf.java:97).
 * Both non-Q8 branches give (float)(double dot) before the bias, so they are computed the same way here. */
JO_API int jo_gguf_linear(int fmt, const float *x, const uint8_t *w, const float *bias, float *y, int rows, int n, int k) {
    if (fmt == JO_Q8_0) {
        return jo_linear_q8_ref(x, w, bias, y, rows, n, k);
    }
    int rc = jo_matvec_ref(fmt, x, w, y, rows, n, k);
    if (rc != 0) {
        return rc;
    }
    if (bias) {
        for (int r = 0; r < rows; r++) {
            for (int c = 0; c < n; c++) {
                y[(long)r * n + c] = y[(long)r * n + c] + bias[c];
            }
        }
    }
    return 0;
}

/* Quant.Quantize.reference (ops/Quant.java:102-118): per 32 values amax in double, d=(float)(amax/127.0),
 * stored as binary16 (RNE); the quants divide by the unrounded float d in double and round half away
 * from zero, clamped to +-127; an all-zero block stores d=0 and zeros. */
JO_API int jo_quantize_q8_0_ref(const float *x, long numel, uint8_t *q) {
    if (numel % 32 != 0) {
        return -1;
    }
    for (long b = 0; b < numel / 32; b++) {
        double amax = 0;
        for (int l = 0; l < 32; l++) {
            double a = fabs((double)x[b * 32 + l]);
            amax = a > amax ? a : amax; /* Math.max; NaN inputs are outside the reference's tests */
        }
        float d = (float)(amax / 127.0);
        uint16_t h = jo_float_to_half(d);
        q[b * 34] = (uint8_t)(h & 0xff);
        q[b * 34 + 1] = (uint8_t)(h >> 8);
        for (int l = 0; l < 32; l++) {
            double s = d > 0 ? (double)x[b * 32 + l] / (double)d : 0.0;
            long v = s >= 0 ? (long)(s + 0.5) : -(long)(-s + 0.5);
            v = v < -127 ? -127 : (v > 127 ? 127 : v);
            q[b * 34 + 2 + l] = (uint8_t)(int8_t)v;
        }
    }
    return 0;
}

/*
 * Pinning status (tests/test_oracle_*.py):
 *  - jo_value / jo_dequantize, all ten formats: bit-exact against expect.<T> in the reference's
 *    fixture.gguf and against the gguf_dequant_* goldens (five formats); brute-force over every byte
 *    value against an independent numpy restatement of ggml's published shift/mask unpacking.
 *  - jo_matvec_ref / jo_gguf_linear: gguf_linear_* goldens (15 cases) within 1 ulp (goldens are
 *    (float)(fp64 dot + bias); the reference rounds the dot to float before adding the bias);
 *    GgufChecks' recipe with java.util.Random restated; unit-vector inputs reproduce columns bit-exactly.
 *  - jo_linear_q8_ref: fixture w.Q8_0/expect.Q8_0 with the FP64-dot recipe; all-ones x -> row sums.
 *  - jo_half_to_float / jo_float_to_half: all 65536 halves round-trip; numpy float16 agreement.
 *  - jo_quantize_q8_0_ref: closed form and invariants only (|x - dq| <= d/2 (+ fp16 rounding of d),
 *    zero block, +-127 at the maximum); no reference-held vector of quantiser output exists, so exact
 *    bytes on .5 ties are "parity unpinned".
 *  - jo_matmul_nt_ref: matmul_t01_* goldens.
 */
