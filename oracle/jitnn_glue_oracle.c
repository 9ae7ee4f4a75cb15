/*
 * CPU oracle for the decode-step glue around the quantised linears (RMSNorm, RoPE, grouped-query
 * attention over an FP32 KV cache, SiLU/SwiGLU, residual add).
 *
 * TEST INFRASTRUCTURE ONLY (see jitnn_oracle.c).  Each function follows the reference's host
 * "reference" method: double arithmetic, FP32 storage.  Paths are relative to the reference root,
 * prefix jitnn-core/src/main/java/ai/beestream/jitnn/.
 *
 * Pinned by the reference's goldens (tests/test_oracle_glue.py): rms_norm*, rope_heads, rope_half,
 * rope_offset, rope_long, sdpa, sdpa_causal, sdpa_head128, sdpa_bthd_causal, silu, silu_tails, swiglu.
 * jo_attention_decode (one query token against a cache, grouped heads) is the same reference with
 * T=1 and every cached key visible; it is pinned through jo_sdpa on sdpa_bthd_causal's last query row
 * and by equality with jo_sdpa on repeated heads (F.repeatHeads, F.java:588-624).
 */
#include <math.h>
#include <stdlib.h>

#define JO_API __attribute__((visibility("default")))

/* RowNorm.reference, RMS branch (ops/RowNorm.java:286-306): is = 1/sqrt(mean(x^2)+eps); y = x*is*w. */
JO_API void jo_rms_norm(const float *x, const float *w, float *y, int rows, int cols, double eps) {
    for (int r = 0; r < rows; r++) {
        double sq = 0;
        for (int c = 0; c < cols; c++) {
            double d = x[(long)r * cols + c];
            sq += d * d;
        }
        double is = 1 / sqrt(sq / cols + eps);
        for (int c = 0; c < cols; c++) {
            double v = (double)x[(long)r * cols + c] * is * (double)w[c];
            y[(long)r * cols + c] = (float)v;
        }
    }
}

/* Rope.tables (ops/Rope.java:86-102): cos/sin of t * base^(-2i/D) in double, stored FP32.
 * base arrives as the float the reference holds, widened to double (Math.pow(float, double)). */
JO_API void jo_rope_tables(int positions, int dim, float base, float *cosv, float *sinv) {
    int half = dim / 2;
    for (int t = 0; t < positions; t++) {
        for (int i = 0; i < half; i++) {
            double frequency = pow((double)base, -2.0 * i / dim);
            double angle = t * frequency;
            cosv[(long)t * half + i] = (float)cos(angle);
            sinv[(long)t * half + i] = (float)sin(angle);
        }
    }
}

/* Rope.reference (ops/Rope.java:126-150) on x [rows, dim] where row / group % seq + offset is the
 * position: group = heads sharing a token's position (1 for plain rope). */
JO_API void jo_rope(const float *x, float *out, const float *cosv, const float *sinv, long rows, int seq, int dim, int group,
                    int offset, int interleaved) {
    int half = dim / 2;
    for (long row = 0; row < rows; row++) {
        long t = (row / group) % seq + offset;
        for (int p = 0; p < half; p++) {
            long ia = interleaved ? row * dim + 2 * p : row * dim + p;
            long ib = interleaved ? ia + 1 : ia + half;
            double c = cosv[t * half + p];
            double s = sinv[t * half + p];
            double a = x[ia];
            double b = x[ib];
            out[ia] = (float)(a * c - b * s);
            out[ib] = (float)(a * s + b * c);
        }
    }
}

/* RefMath SILU (ops/RefMath.java:114): x / (1 + exp(-x)) in double. */
JO_API void jo_silu(const float *x, float *y, long n) {
    for (long i = 0; i < n; i++) {
        double v = x[i];
        y[i] = (float)(v / (1 + exp(-v)));
    }
}

/* F.swiglu (F.java:1159-1161): silu(gate) rounded to FP32, then an FP32 multiply by up. */
JO_API void jo_swiglu(const float *gate, const float *up, float *y, long n) {
    for (long i = 0; i < n; i++) {
        double v = gate[i];
        float s = (float)(v / (1 + exp(-v)));
        y[i] = s * up[i];
    }
}

/* FlashAttention.reference (ops/FlashAttention.java:538-626) for contiguous problems:
 * q [z, t, d], k [z, s, d], v [z, s, dv], o [z, t, dv]; causal hides key j > query i. */
JO_API int jo_sdpa(const float *q, const float *k, const float *v, float *o, int z, int t, int s, int d, int dv, int causal,
                   double scale) {
    double *row = (double *)malloc(sizeof(double) * (size_t)s);
    if (!row) {
        return -2;
    }
    for (int zi = 0; zi < z; zi++) {
        for (int i = 0; i < t; i++) {
            const float *qi = q + ((long)zi * t + i) * d;
            double m = -INFINITY;
            for (int j = 0; j < s; j++) {
                if (causal && j > i) {
                    row[j] = -INFINITY;
                    continue;
                }
                const float *kj = k + ((long)zi * s + j) * d;
                double dot = 0;
                for (int c = 0; c < d; c++) {
                    dot += (double)qi[c] * (double)kj[c];
                }
                row[j] = dot * scale;
                m = row[j] > m ? row[j] : m;
            }
            double sum = 0;
            for (int j = 0; j < s; j++) {
                row[j] = row[j] == -INFINITY ? 0 : exp(row[j] - m);
                sum += row[j];
            }
            for (int j = 0; j < s; j++) {
                row[j] /= sum;
            }
            for (int c = 0; c < dv; c++) {
                double acc = 0;
                for (int j = 0; j < s; j++) {
                    acc += row[j] * (double)v[((long)zi * s + j) * dv + c];
                }
                o[((long)zi * t + i) * dv + c] = (float)acc;
            }
        }
    }
    free(row);
    return 0;
}

/* One new token against a cache in [S, KV, D] order (the BTHD layout of F.scaledDotProductAttentionBTHD,
 * F.java:588-600, batch 1): query head h reads key/value head h / (heads / kv_heads) (F.repeatHeads).
 * q [heads, d]; kc, vc [s, kv_heads, d] with all s entries visible (the causal mask of the last row). */
JO_API int jo_attention_decode(const float *q, const float *kc, const float *vc, float *o, int heads, int kv_heads, int s, int d,
                               double scale) {
    double *row = (double *)malloc(sizeof(double) * (size_t)s);
    if (!row) {
        return -2;
    }
    int group = heads / kv_heads;
    for (int h = 0; h < heads; h++) {
        int g = h / group;
        double m = -INFINITY;
        for (int j = 0; j < s; j++) {
            const float *kj = kc + ((long)j * kv_heads + g) * d;
            double dot = 0;
            for (int c = 0; c < d; c++) {
                dot += (double)q[(long)h * d + c] * (double)kj[c];
            }
            row[j] = dot * scale;
            m = row[j] > m ? row[j] : m;
        }
        double sum = 0;
        for (int j = 0; j < s; j++) {
            row[j] = exp(row[j] - m);
            sum += row[j];
        }
        for (int j = 0; j < s; j++) {
            row[j] /= sum;
        }
        for (int c = 0; c < d; c++) {
            double acc = 0;
            for (int j = 0; j < s; j++) {
                acc += row[j] * (double)vc[((long)j * kv_heads + g) * d + c];
            }
            o[(long)h * d + c] = (float)acc;
        }
    }
    free(row);
    return 0;
}

/* Residual add (Binary add reference): FP32 a + b. */
JO_API void jo_add(const float *a, const float *b, float *y, long n) {
    for (long i = 0; i < n; i++) {
        y[i] = a[i] + b[i];
    }
}
