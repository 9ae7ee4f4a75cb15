// Bit-exact dequantisation of raw GGUF blocks to FP32 and the Q8_0 quantiser.
//
// The arithmetic follows the reference's per-value decode operation by operation in binary32 with no fused
// multiply-add (this translation unit is built with -ffp-contract=off): the integer fields are unpacked
// with shifts and masks, which give the same integers as the reference's division/remainder form, and the
// float expression is evaluated left to right exactly as written there
// (reference: core/kernels/GgufKernels.java:61-140, core/ops/Quant.java:137-144).
#pragma once
#include "common.h"

namespace jitnn {

// 6-bit scale (part 0) or min (part 1) of sub-block j from the 12 scale bytes at s (GgufKernels.java:74-83).
__device__ __forceinline__ int k4_scale_min(const uint8_t *s, int j, int part) {
    if (j < 4) return s[j + 4 * part] & 63;
    int low = part == 0 ? (s[j + 4] & 15) : (s[j + 4] >> 4);
    return low | ((s[j - 4 + 4 * part] >> 6) << 4);
}

// Four consecutive values i..i+3 (i % 4 == 0) of a tensor: they share block, sub-block, nibble half and scale.
template <int FMT>
__device__ __forceinline__ float4 dequant4(const uint8_t *w, size_t i) {
    float o[4];
    if constexpr (FMT == F_Q4_0) {
        const uint8_t *b = w + (i >> 5) * 18;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = b[2 + ((e + t) & 15)];
            int q = e < 16 ? (v & 15) : (v >> 4);
            o[t] = (float)(q - 8) * d;
        }
    } else if constexpr (FMT == F_Q4_1) {
        const uint8_t *b = w + (i >> 5) * 20;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b)), m = h2f(ld16(b + 2));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = b[4 + ((e + t) & 15)];
            int q = e < 16 ? (v & 15) : (v >> 4);
            float p = (float)q * d;
            o[t] = p + m;
        }
    } else if constexpr (FMT == F_Q8_0) {
        const uint8_t *b = w + (i >> 5) * 34;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b));
#pragma unroll
        for (int t = 0; t < 4; ++t) o[t] = d * (float)(int)(int8_t)b[2 + e + t];
    } else if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        constexpr int NB = FMT == F_Q4_K ? 144 : 176, QS = FMT == F_Q4_K ? 16 : 48;
        const uint8_t *b = w + (i >> 8) * NB;
        const int e = (int)(i & 255);
        const int j = e >> 6, half = (e & 63) >> 5, l = e & 31, sub = 2 * j + half;
        const float ds = h2f(ld16(b)) * (float)k4_scale_min(b + 4, sub, 0);
        const float m = h2f(ld16(b + 2)) * (float)k4_scale_min(b + 4, sub, 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = b[QS + 32 * j + l + t];
            int q = half == 0 ? (v & 15) : (v >> 4);
            if constexpr (FMT == F_Q5_K) q += 16 * ((b[16 + l + t] >> sub) & 1);
            float a = ds * (float)q;
            o[t] = a - m;
        }
    } else if constexpr (FMT == F_Q5_0 || FMT == F_Q5_1) {
        // 22 / 24 bytes: f16 d (, f16 m), 32 fifth bits, 16 bytes of nibbles; value e: nibble e % 16 (low for e < 16) + 16 *
        // bit e, then (q - 16) * d or q * d + m (GgufKernels.java:143-163)
        constexpr int NB = FMT == F_Q5_0 ? 22 : 24, QH = FMT == F_Q5_0 ? 2 : 4, QS = QH + 4;
        const uint8_t *b = w + (i >> 5) * NB;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int v = b[QS + ((e + t) & 15)];
            const int q = (e < 16 ? (v & 15) : (v >> 4)) + 16 * ((b[QH + ((e + t) >> 3)] >> ((e + t) & 7)) & 1);
            if constexpr (FMT == F_Q5_0) {
                o[t] = (float)(q - 16) * d;
            } else {
                const float p = (float)q * d;
                o[t] = p + h2f(ld16(b + 2));
            }
        }
    } else if constexpr (FMT == F_Q2_K) {
        // 84 bytes: 16 scale bytes (low nibble scale, high nibble min), 64 bytes of 2-bit quants, f16 d, f16 dmin
        // (GgufKernels.java:166-175)
        const uint8_t *b = w + (i >> 8) * 84;
        const int e = (int)(i & 255);
        const int n = e >> 7, j = (e & 127) >> 5, l = e & 31;
        const int sc = b[n * 8 + j * 2 + (l >> 4)];
        const float ds = h2f(ld16(b + 80)) * (float)(sc & 15);
        const float m = h2f(ld16(b + 82)) * (float)(sc >> 4);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int q = (b[16 + n * 32 + l + t] >> (2 * j)) & 3;
            const float a = ds * (float)q;
            o[t] = a - m;
        }
    } else if constexpr (FMT == F_Q3_K) {
        // 110 bytes: 32 bytes of high bits, 64 bytes of 2-bit quants, 12 bytes of 6-bit scales, f16 d
        // (GgufKernels.java:181-198)
        const uint8_t *b = w + (i >> 8) * 110;
        const int e = (int)(i & 255);
        const int n = e >> 7, j = (e & 127) >> 5, l = e & 31;
        const int is = n * 8 + j * 2 + (l >> 4);
        const int low = is < 8 ? (b[96 + is] & 15) : (b[96 + is - 8] >> 4);
        const int high = (b[96 + 8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const float a = h2f(ld16(b + 108)) * (float)(low + 16 * high - 32);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int q = (b[32 + n * 32 + l + t] >> (2 * j)) & 3;
            const int hb = (b[l + t] >> (4 * n + j)) & 1;
            o[t] = a * (float)(q - (hb == 1 ? 0 : 4));
        }
    } else {  // F_Q6_K
        const uint8_t *b = w + (i >> 8) * 210;
        const int e = (int)(i & 255);
        const int n = e >> 7, k = (e & 127) >> 5, l = e & 31;
        const int sc = (int)(int8_t)b[192 + 8 * n + (l >> 4) + 2 * k];
        const float a = h2f(ld16(b + 208)) * (float)sc;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int lb = b[64 * n + l + t + (k & 1) * 32];
            int low = k < 2 ? (lb & 15) : (lb >> 4);
            int hb = (b[128 + 32 * n + l + t] >> (2 * k)) & 3;
            o[t] = a * (float)(low + 16 * hb - 32);
        }
    }
    return make_float4(o[0], o[1], o[2], o[3]);
}

template <int FMT>
__global__ void __launch_bounds__(256) dequant_kernel(const uint8_t *__restrict__ w, float *__restrict__ y, size_t quads) {
    for (size_t f = (size_t)blockIdx.x * blockDim.x + threadIdx.x; f < quads; f += (size_t)gridDim.x * blockDim.x) {
        reinterpret_cast<float4 *>(y)[f] = dequant4<FMT>(w, f * 4);
    }
}

// Rows token[t] of a block-quantised table [vocab, k], dequantised bit-exactly into x [tokens, k] (the embedding lookup of
// a model whose token table is quantised).  grid = tokens.
template <int FMT>
__global__ void __launch_bounds__(256) dequant_rows_kernel(const uint8_t *__restrict__ w, const int *__restrict__ tokens, float *__restrict__ x, int k) {
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const uint8_t *wr = w + (size_t)tokens[blockIdx.x] * rowbytes;
    float4 *xr = reinterpret_cast<float4 *>(x + (size_t)blockIdx.x * k);
    for (int f = threadIdx.x; f < (k >> 2); f += 256) xr[f] = dequant4<FMT>(wr, (size_t)f * 4);
}

// Plain GEMV for the formats without a tuned kernel: one wave per weight row, every lane dequantises quads of the row
// with the bit-exact decoder and multiplies them with up to eight activation rows; a fixed DPP tree adds the lanes.
//   y[b, row] = sum_k W[row, k] x[b, k] (+ bias[row]), b < rows <= 8.  grid: any; waves take rows round-robin.
template <int FMT>
__global__ void __launch_bounds__(256) gemv_plain_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x, const float *__restrict__ bias,
                                                          float *__restrict__ y, int n, int k, int rows) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    for (int row = blockIdx.x * 4 + wave; row < n; row += gridDim.x * 4) {
        const uint8_t *wr = W + (size_t)row * rowbytes;
        float acc[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[b] = 0.f;
        for (int f = lane; f < (k >> 2); f += 64) {
            const float4 v = dequant4<FMT>(wr, (size_t)f * 4);
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                if (b < rows) {
                    const float4 xv = reinterpret_cast<const float4 *>(x + (size_t)b * k)[f];
                    acc[b] = __builtin_fmaf(v.w, xv.w, __builtin_fmaf(v.z, xv.z, __builtin_fmaf(v.y, xv.y, __builtin_fmaf(v.x, xv.x, acc[b]))));
                }
            }
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            if (b < rows) {
                const float t = wave_sum(acc[b]);
                if (lane == 0) y[(size_t)b * n + row] = bias ? t + bias[row] : t;
            }
        }
    }
}

// Two of the formats without kernels of their own hold exactly the values of a format that has them, block by block and
// element by element, and are rewritten into it once, when the weight is uploaded:
//   Q5_0 (q - 16) d, q of five bits (kernels/GgufKernels.java:147-153)  ->  Q8_0 with the same d and the int8 quant q - 16;
//   Q3_K d (sc - 32) (q - 4 or q), sc of six bits per 16 values, q of two bits (kernels/GgufKernels.java:185-198)  ->  Q6_K
//   with the same d, the int8 scale sc - 32 and the 6-bit quant q' + 32, q' = q - 4 or q: Q6_K's element order, its scale
//   index 8 n + 2 k + l / 16 and its product d * sc * q (kernels/GgufKernels.java:126-138) are Q3_K's own.
// The same floats multiply in the same order, so every value - and the dequantiser's output - keeps its bits.
// One thread per block.
static __global__ void __launch_bounds__(256) transcode_q5_0_to_q8_0_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, size_t blocks) {
    for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks; b += (size_t)gridDim.x * blockDim.x) {
        const uint8_t *s = src + b * 22;
        uint8_t *d = dst + b * 34;
        d[0] = s[0];
        d[1] = s[1];
        const uint32_t qh = (uint32_t)s[2] | ((uint32_t)s[3] << 8) | ((uint32_t)s[4] << 16) | ((uint32_t)s[5] << 24);
        for (int e = 0; e < 32; ++e) {
            const int byte = s[6 + (e & 15)], q = (e < 16 ? byte & 15 : byte >> 4) + 16 * (int)((qh >> e) & 1u);
            d[2 + e] = (uint8_t)(int8_t)(q - 16);
        }
    }
}

static __global__ void __launch_bounds__(256) transcode_q3_k_to_q6_k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, size_t blocks) {
    for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks; b += (size_t)gridDim.x * blockDim.x) {
        const uint8_t *s = src + b * 110;  // hmask[32], qs[64], scales[12], d
        uint8_t *d = dst + b * 210;        // ql[128], qh[64], scales[16], d
        for (int i = 0; i < 192; ++i) d[i] = 0;
        for (int e = 0; e < 256; ++e) {
            const int n = e >> 7, j = (e & 127) >> 5, l = e & 31;
            const int q = (s[32 + n * 32 + l] >> (2 * j)) & 3, high = (s[l] >> (4 * n + j)) & 1;
            const int q6 = q - (high ? 0 : 4) + 32;  // 28 .. 35
            d[64 * n + l + (j & 1) * 32] |= (uint8_t)((q6 & 15) << (j < 2 ? 0 : 4));
            d[128 + 32 * n + l] |= (uint8_t)((q6 >> 4) << (2 * j));
        }
        for (int is = 0; is < 16; ++is) {  // the 6-bit scale `is`: low four bits from bytes 0..7, high two from bytes 8..11
            const int low = is < 8 ? s[96 + is] & 15 : s[96 + is - 8] >> 4, hi2 = (s[96 + 8 + (is & 3)] >> (2 * (is >> 2))) & 3;
            d[192 + is] = (uint8_t)(int8_t)(low + 16 * hi2 - 32);
        }
        d[208] = s[108];
        d[209] = s[109];
    }
}

// FP32 -> Q8_0, one thread per block of 32 values, in the reference quantiser's arithmetic
// (core/ops/Quant.java:102-118): amax in double, d = (float)(amax / 127.0) stored as binary16 (round to
// nearest even), quants = round-half-away(x / (double)d) with the unrounded float d, clamped to +-127.
static __global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x, uint8_t *__restrict__ q, size_t blocks) {
    for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks; b += (size_t)gridDim.x * blockDim.x) {
        const float *xb = x + b * 32;
        float v[32];
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            float4 t = reinterpret_cast<const float4 *>(xb)[l];
            v[4 * l] = t.x; v[4 * l + 1] = t.y; v[4 * l + 2] = t.z; v[4 * l + 3] = t.w;
        }
        double amax = 0;
#pragma unroll
        for (int l = 0; l < 32; ++l) {
            double a = fabs((double)v[l]);
            amax = a > amax ? a : amax;
        }
        const float d = (float)(amax / 127.0);
        uint8_t *o = q + b * 34;
        *reinterpret_cast<uint16_t *>(o) = __half_as_ushort(__float2half_rn(d));
#pragma unroll
        for (int l = 0; l < 32; ++l) {
            double s = d > 0 ? (double)v[l] / (double)d : 0.0;
            long long r = s >= 0 ? (long long)(s + 0.5) : -(long long)(-s + 0.5);
            r = r < -127 ? -127 : (r > 127 ? 127 : r);
            o[2 + l] = (uint8_t)(int8_t)r;
        }
    }
}

}  // namespace jitnn
