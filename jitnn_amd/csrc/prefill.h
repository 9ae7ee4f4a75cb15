// Many-row linear (prefill, batches beyond the GEMV range) on raw GGUF blocks: y[M, N] = x[M, K] W[N, K]^T.
//
// This is the one shape on the path that is a real dense contraction, so it runs on the matrix cores:
//   1. x_to_f16_kernel turns each activation row into FP16 with a power-of-two row scale that puts its largest
//      magnitude in [2^13, 2^14) (no overflow for any FP32 input, no loss of small rows to FP16 subnormals);
//   2. prefill_mfma_kernel: a workgroup of four waves owns a 128 (weight rows) x 128 (tokens) output tile and
//      walks K in steps of 64.  Per step every thread dequantises 32 weights of one row from the raw blocks
//      (FP32 arithmetic of the dequantiser, then one rounding to FP16) into LDS, the FP16 activations of the
//      step are copied beside them, and each wave issues 16 v_mfma_f32_32x32x16_f16 on its 64 x 64 quadrant,
//      accumulating in FP32.  The epilogue undoes the row scale and adds the bias.
// Both FP16 roundings are relative 2^-11, so the result stays well inside the 2e-3 bar of the MFMA path.
#pragma once
#include "common.h"
#include "dequant.h"

namespace jitnn {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int PF_BN = 128, PF_BM = 128, PF_BK = 64, PF_LD = PF_BK + 8;  // LDS row pitch in halves: 144 bytes, conflict-free 16-byte reads

// One workgroup per activation row: amax, scale = 2^(13 - floor(log2 amax)), FP16 copy, 1/scale for the epilogue.
__global__ void __launch_bounds__(256) x_to_f16_kernel(const float *__restrict__ x, _Float16 *__restrict__ xh, float *__restrict__ inv_scale,
                                                        int k) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * k;
    float m = 0.f;
    for (int i = threadIdx.x; i < k; i += 256) m = fmaxf(m, fabsf(xr[i]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float scale = 1.f;
    if (m > 0.f && m < 3.0e38f) {
        int e;
        frexpf(m, &e);  // m = f * 2^e, f in [0.5, 1)
        scale = ldexpf(1.f, 14 - e);
    }
    _Float16 *o = xh + (size_t)blockIdx.x * k;
    for (int i = threadIdx.x; i < k; i += 256) o[i] = (_Float16)(xr[i] * scale);
    if (threadIdx.x == 0) inv_scale[blockIdx.x] = 1.f / scale;
}

// 32 consecutive weights of a row, starting at value k0 (k0 % 32 == 0), in the dequantiser's FP32 arithmetic.
template <int FMT>
__device__ __forceinline__ void dequant32(const uint8_t *row, int k0, float (&o)[32]) {
    if constexpr (FMT == F_Q4_0 || FMT == F_Q4_1) {
        constexpr int NB = FMT == F_Q4_0 ? 18 : 20, QS = FMT == F_Q4_0 ? 2 : 4;
        const uint8_t *b = row + (size_t)(k0 >> 5) * NB;
        const float d = h2f(ld16(b));
        const u32x4 q = FMT == F_Q4_0 ? ld128<2>(b + QS) : ld128<4>(b + QS);
        const float m = FMT == F_Q4_1 ? h2f(ld16(b + 2)) : 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t byte = (q[i >> 2] >> (8 * (i & 3))) & 0xffu;
            if constexpr (FMT == F_Q4_0) {
                o[i] = (float)((int)(byte & 15u) - 8) * d;
                o[16 + i] = (float)((int)(byte >> 4) - 8) * d;
            } else {
                o[i] = (float)(byte & 15u) * d + m;
                o[16 + i] = (float)(byte >> 4) * d + m;
            }
        }
    } else if constexpr (FMT == F_Q8_0) {
        const uint8_t *b = row + (size_t)(k0 >> 5) * 34;
        const float d = h2f(ld16(b));
        const u32x4 q0 = ld128<2>(b + 2), q1 = ld128<2>(b + 18);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = i < 16 ? q0[i >> 2] : q1[(i - 16) >> 2];
            o[i] = d * (float)(int)(int8_t)((w >> (8 * (i & 3))) & 0xffu);
        }
    } else if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        constexpr int NB = FMT == F_Q4_K ? 144 : 176, QS = FMT == F_Q4_K ? 16 : 48;
        const uint8_t *b = row + (size_t)(k0 >> 8) * NB;
        const int e = k0 & 255, j = e >> 6, half = (e >> 5) & 1, sub = 2 * j + half;
        const u32x4 h = ld128<16>(b);
        const u32x4 q0 = ld128<16>(b + QS + 32 * j), q1 = ld128<16>(b + QS + 32 * j + 16);
        int sc, mn;
        {
            const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;
            const int i4 = sub & 3, sh = 8 * i4;
            if (sub < 4) {
                sc = (s0 >> sh) & 63;
                mn = (s1 >> sh) & 63;
            } else {
                sc = ((s2 >> sh) & 15) | (((s0 >> sh) >> 6 & 3) << 4);
                mn = ((s2 >> sh) >> 4 & 15) | (((s1 >> sh) >> 6 & 3) << 4);
            }
        }
        const float ds = h2f(h.x) * (float)sc, m = h2f(h.x >> 16) * (float)mn;
        u32x4 qh0 = {0, 0, 0, 0}, qh1 = {0, 0, 0, 0};
        if constexpr (FMT == F_Q5_K) {
            qh0 = ld128<16>(b + 16);
            qh1 = ld128<16>(b + 32);
        }
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = i < 16 ? q0[i >> 2] : q1[(i - 16) >> 2];
            uint32_t q = (w >> (8 * (i & 3) + 4 * half)) & 15u;
            if constexpr (FMT == F_Q5_K) {
                const uint32_t hw = i < 16 ? qh0[i >> 2] : qh1[(i - 16) >> 2];
                q += 16u * ((hw >> (8 * (i & 3) + sub)) & 1u);
            }
            o[i] = ds * (float)q - m;
        }
    } else {  // F_Q6_K
        const uint8_t *b = row + (size_t)(k0 >> 8) * 210;
        const int e = k0 & 255, n = e >> 7, kk = (e >> 5) & 3;
        const u32x4 l0 = ld128<2>(b + 64 * n + 32 * (kk & 1)), l1 = ld128<2>(b + 64 * n + 32 * (kk & 1) + 16);
        const u32x4 h0 = ld128<2>(b + 128 + 32 * n), h1 = ld128<2>(b + 128 + 32 * n + 16);
        const uint32_t scw = ld16(b + 192 + 8 * n + 2 * kk);
        const float d = h2f(ld16(b + 208));
        const float a0 = d * (float)(int)(int8_t)(scw & 0xffu), a1 = d * (float)(int)(int8_t)(scw >> 8);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t lw = i < 16 ? l0[i >> 2] : l1[(i - 16) >> 2];
            const uint32_t hw = i < 16 ? h0[i >> 2] : h1[(i - 16) >> 2];
            const int low = (lw >> (8 * (i & 3) + (kk < 2 ? 0 : 4))) & 15;
            const int hb = (hw >> (8 * (i & 3) + 2 * kk)) & 3;
            o[i] = (i < 16 ? a0 : a1) * (float)(low + 16 * hb - 32);
        }
    }
}

template <int FMT>
__global__ void __launch_bounds__(256) prefill_mfma_kernel(const uint8_t *__restrict__ W, const _Float16 *__restrict__ xh,
                                                            const float *__restrict__ inv_scale, const float *__restrict__ bias,
                                                            float *__restrict__ y, int m, int n, int k) {
    __shared__ _Float16 As[PF_BN * PF_LD];  // dequantised weights  [row][k]
    __shared__ _Float16 Bs[PF_BM * PF_LD];  // activations          [token][k]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * PF_BN, m0 = blockIdx.y * PF_BM;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    // dequantiser role: thread t fills weights [row t/2][32 * (t%2) ... +32) of the step
    const int drow = tid >> 1, dhalf = tid & 1;
    const uint8_t *wrow = W + (size_t)min(n0 + drow, n - 1) * rowbytes;
    // copier role: thread t copies 32 halves of token t/2
    const int xtok = min(m0 + drow, m - 1);
    const bool xlive = m0 + drow < m;
    const _Float16 *xrow = xh + (size_t)xtok * k;
    // MFMA role: wave (wr, wc) owns output rows [64 wr, +64) x tokens [64 wc, +64) as 2 x 2 tiles of 32 x 32
    const int wr = wave >> 1, wc = wave & 1;
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    for (int k0 = 0; k0 < k; k0 += PF_BK) {
        const int kk = k0 + 32 * dhalf;
        // ---- weights -> FP16 in LDS
        {
            float v[32];
            if (kk < k) {
                dequant32<FMT>(wrow, kk, v);
            } else {
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = 0.f;
            }
            f16x8 *dst = reinterpret_cast<f16x8 *>(&As[drow * PF_LD + 32 * dhalf]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                f16x8 p;
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] = (_Float16)v[8 * c + i];
                dst[c] = p;
            }
        }
        // ---- activations (already FP16) -> LDS
        {
            f16x8 *dst = reinterpret_cast<f16x8 *>(&Bs[drow * PF_LD + 32 * dhalf]);
            const f16x8 *src = reinterpret_cast<const f16x8 *>(xrow + kk);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                f16x8 p = {0, 0, 0, 0, 0, 0, 0, 0};
                if (xlive && kk < k) p = src[c];
                dst[c] = p;
            }
        }
        __syncthreads();
        // ---- 4 k-substeps of 16: lane l supplies row/token l%32, halves 8*(l/32) .. +8 of the substep
#pragma unroll
        for (int ks = 0; ks < PF_BK; ks += 16) {
            f16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = *reinterpret_cast<const f16x8 *>(&As[(64 * wr + 32 * i + (lane & 31)) * PF_LD + ks + 8 * (lane >> 5)]);
                b[i] = *reinterpret_cast<const f16x8 *>(&Bs[(64 * wc + 32 * i + (lane & 31)) * PF_LD + ks + 8 * (lane >> 5)]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // ---- epilogue: element r of a 32 x 32 accumulator is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int tok = m0 + 64 * wc + 32 * j + (lane & 31);
            if (tok >= m) continue;
            const float is = inv_scale[tok];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = n0 + 64 * wr + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < n) {
                    float v = acc[i][j][r] * is;
                    if (bias) v += bias[row];
                    y[(size_t)tok * n + row] = v;
                }
            }
        }
    }
}

}  // namespace jitnn
