// Many-row linear (prefill, batches beyond the GEMV range) on raw GGUF blocks: y[M, N] = x[M, K] W[N, K]^T.
//
// This is the one shape on the path that is a real dense contraction, so it runs on the matrix cores:
//   1. x_row_scale_kernel finds, per activation row, the power-of-two scale that puts its largest magnitude in
//      [2^13, 2^14) (no overflow for any FP32 input, no loss of small rows to FP16 subnormals), and
//      x_to_operand_kernel writes the scaled FP16 activations in the order the matrix cores consume them: 1 KiB per
//      (block of 32 tokens, step of 16 K values), 16 bytes per lane - a wave's B operand is one fully coalesced
//      128-bit load from L2, no LDS involved;
//   2. prefill_mfma_kernel: a workgroup of four waves owns a 128 (weight rows) x 256 (tokens) output tile and
//      walks K in steps of 64.  Per step every thread dequantises 32 weights of one row from the raw blocks into a
//      double-buffered LDS tile as FP16, and each wave issues 32 v_mfma_f32_32x32x16_f16 on its 128 x 64 slice
//      (weight operands from LDS, each used twice; activation operands from registers loaded two steps ahead, each
//      used four times - the shape that keeps both LDS and the vector L1 at half their bandwidth), accumulating in
//      FP32; the raw weight bytes are requested two steps ahead and decoded after the MFMAs are issued.  The epilogue
//      undoes the row scale and adds the bias.
// Both FP16 roundings are relative 2^-11, so the result stays well inside the 2e-3 bar of the MFMA path.
#pragma once
#include "common.h"
#include "dequant.h"
#include "tu.h"

namespace jitnn {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int PF_BN = 128, PF_BM = 256, PF_BK = 64, PF_LD = PF_BK + 8;  // LDS row pitch in halves: 144 bytes, conflict-free 16-byte reads
constexpr int PF_NARROW_ROWS = 128;  // calls of at most this many rows: two 32-row blocks per wave instead of four (prefill_mfma_body, RT)

// position of value i (0..3) of a group of four in the FP16 operands: 0, 2, 1, 3
__host__ __device__ constexpr int pf_perm4(int i) { return ((i & 1) << 1) | (i >> 1); }

// One workgroup per activation row: amax -> scale = 2^(13 - floor(log2 amax)) and 1/scale for the epilogue.
static __global__ void __launch_bounds__(256) x_row_scale_kernel(const float *__restrict__ x, float *__restrict__ scale, float *__restrict__ inv_scale,
                                                           int k) {
    __shared__ float red[4];
    const float4 *xr = reinterpret_cast<const float4 *>(x + (size_t)blockIdx.x * k);  // k is a multiple of 32
    float m = 0.f;
    for (int i = threadIdx.x; i < (k >> 2); i += 256) {
        const float4 v = xr[i];
        m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sc = 1.f;
    if (m > 0.f && m < 3.0e38f) {
        int e;
        frexpf(m, &e);  // m = f * 2^e, f in [0.5, 1)
        sc = ldexpf(1.f, 14 - e);
    }
    if (threadIdx.x == 0) {
        scale[blockIdx.x] = sc;
        inv_scale[blockIdx.x] = 1.f / sc;
    }
}

// Number of 16-value K steps the operand array holds per token block: K rounded up to whole steps of PF_BK.
__host__ __device__ constexpr int pf_ksteps(int k) { return (k + PF_BK - 1) / PF_BK * (PF_BK / 16); }

// FP16 activations in matrix-core operand order: xo[token block mb][K step ks][lane][8], lane l holding token
// 32 mb + l % 32, values 16 ks + 8 (l / 32) .. + 7, each group of four values in the order 0, 2, 1, 3 (the order in
// which the weight decoder produces FP16 pairs from a dword of quants; a dot product only needs both to agree).
// Tokens past m and values past k are zeros.  grid (token blocks, K / 64), 256 threads: one 16-byte piece each.
static __global__ void __launch_bounds__(256) x_to_operand_kernel(const float *__restrict__ x, const float *__restrict__ scale,
                                                            _Float16 *__restrict__ xo, int m, int k) {
    // 32 tokens x 64 values through LDS: the reads run along the token rows (256 contiguous bytes each), the writes
    // along the operand order (1 KiB per K step)
    __shared__ float4 tile[32][17];  // [token][16 quads + 1: the operand reads below walk down the tokens]
    const int t = threadIdx.x, tok0 = blockIdx.x * 32, k0 = blockIdx.y * 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int idx = t + 256 * i, r = idx >> 4, q = idx & 15, tok = tok0 + r, kk = k0 + 4 * q;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (tok < m && kk < k) {
            const float sc = scale[tok];
            v = *reinterpret_cast<const float4 *>(x + (size_t)tok * k + kk);
            v = make_float4(v.x * sc, v.y * sc, v.z * sc, v.w * sc);
        }
        tile[r][q] = v;
    }
    __syncthreads();
    const int lane = t & 63, ks = t >> 6;  // this thread's piece: token lane % 32, values 16 ks + 8 (lane / 32) .. + 7 of the tile
    const float4 a = tile[lane & 31][4 * ks + 2 * (lane >> 5)], b = tile[lane & 31][4 * ks + 2 * (lane >> 5) + 1];
    const f16x8 o = {(_Float16)a.x, (_Float16)a.z, (_Float16)a.y, (_Float16)a.w, (_Float16)b.x, (_Float16)b.z, (_Float16)b.y, (_Float16)b.w};
    reinterpret_cast<f16x8 *>(xo)[((size_t)blockIdx.x * pf_ksteps(k) + blockIdx.y * 4 + ks) * 64 + lane] = o;
}

// The two kernels above in one launch, for rows of up to XP_MAXK values: one workgroup per token keeps the row in
// registers between finding its scale and writing its FP16 pieces (16 bytes each, 512 bytes apart in operand order).
// Eight consecutive tokens share every 128-byte line of the operand array, and consecutive workgroups run on
// different XCDs, each with its own L2: the workgroup -> token map keeps the eight writers of a line on one XCD, so
// that the line leaves its L2 whole.  grid = padded tokens (a multiple of 64); padding tokens write zeros.
// J = 8-value pieces per thread: a row holds at most 256 J of them.
// MODE XP_NORM: the row is RMS-normalised first, x <- x * nw / sqrt(mean(x^2) + eps) (ops/RowNorm.java:286-306), for
// callers whose linear follows a norm (the layers of a model): the normalised activations exist only as these operands.
// MODE XP_SWIGLU: the row is silu(x) * nw, nw being a second [m, k] array (F.swiglu, F.java:1159-1161, in front of the
// down projection of an FFN): the gated activations exist only as these operands.
constexpr int XP_MAXJ = 8, XP_MAXK = XP_MAXJ * 256 * 8;
// MODE XP_NORM_JOIN: XP_NORM on a row that does not exist yet - the linear in front of it split K and left its slices
// unjoined: the row is x (the residual) + the slices part[z] [m, k] in slice order, exactly what prefill_join_kernel would
// have stored; it is written to xsum [m, k] on the way (the next residual) and normalised from the registers.
constexpr int XP_PLAIN = 0, XP_NORM = 1, XP_SWIGLU = 2, XP_NORM_JOIN = 3;
template <int J, int MODE>
__global__ void __launch_bounds__(256) x_prepare_kernel(const float *__restrict__ x, float *__restrict__ inv_scale, _Float16 *__restrict__ xo,
                                                         int m, int k, const float *__restrict__ nw, float eps, const float *__restrict__ part,
                                                         int splits, float *__restrict__ xsum) {
    constexpr bool NORM = MODE == XP_NORM || MODE == XP_NORM_JOIN;
    __shared__ float red[4];
    __shared__ float red2[4];
    const int b = blockIdx.x, tok = (b & ~63) | ((b & 7) << 3) | ((b >> 3) & 7), t = threadIdx.x;
    const int ksteps = pf_ksteps(k), npieces = 2 * ksteps;  // 8-value pieces of a row, zero padding included
    const float *xr = x + (size_t)min(tok, m - 1) * k;
    float4 v[J][2];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j) {  // unconditional loads (index clamped), so that all of them are in flight at once
        const int kk = 8 * (t + 256 * j);
        const float4 *src = reinterpret_cast<const float4 *>(xr + min(kk, k - 8));
        v[j][0] = src[0];
        v[j][1] = src[1];
    }
    float4 w[MODE != XP_PLAIN ? J : 1][2];
    if constexpr (MODE != XP_PLAIN) {
        const float *wr = MODE == XP_SWIGLU ? nw + (size_t)min(tok, m - 1) * k : nw;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const float4 *src = reinterpret_cast<const float4 *>(wr + min(8 * (t + 256 * j), k - 8));
            w[j][0] = src[0];
            w[j][1] = src[1];
        }
    }
    if constexpr (MODE == XP_NORM_JOIN) {
        const size_t row = (size_t)min(tok, m - 1) * k, slice = (size_t)m * k;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int kk = min(8 * (t + 256 * j), k - 8);
            float4 a[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) a[h] = reinterpret_cast<const float4 *>(part + row + kk)[h];
            for (int z = 1; z < splits; ++z) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 b = reinterpret_cast<const float4 *>(part + z * slice + row + kk)[h];
                    a[h] = make_float4(a[h].x + b.x, a[h].y + b.y, a[h].z + b.z, a[h].w + b.w);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                v[j][h] = make_float4(a[h].x + v[j][h].x, a[h].y + v[j][h].y, a[h].z + v[j][h].z, a[h].w + v[j][h].w);
                if (tok < m && 8 * (t + 256 * j) < k) reinterpret_cast<float4 *>(xsum + row + kk)[h] = v[j][h];
            }
        }
    }
    if constexpr (MODE == XP_SWIGLU) {
        auto sw = [](float g, float u) { return (g / (1.f + __expf(-g))) * u; };
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                v[j][h] = make_float4(sw(v[j][h].x, w[j][h].x), sw(v[j][h].y, w[j][h].y), sw(v[j][h].z, w[j][h].z), sw(v[j][h].w, w[j][h].w));
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const bool in = tok < m && 8 * (t + 256 * j) < k;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            if (!in) v[j][h] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if constexpr (NORM) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) ss += (v[j][h].x * v[j][h].x + v[j][h].y * v[j][h].y) + (v[j][h].z * v[j][h].z + v[j][h].w * v[j][h].w);
        ss = wave_sum(ss);
        if ((t & 63) == 0) red2[t >> 6] = ss;
        __syncthreads();
        const float is = 1.f / sqrtf(((red2[0] + red2[1]) + (red2[2] + red2[3])) / (float)k + eps);
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                v[j][h] = make_float4(v[j][h].x * is * w[j][h].x, v[j][h].y * is * w[j][h].y, v[j][h].z * is * w[j][h].z, v[j][h].w * is * w[j][h].w);
    }
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h)
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j][h].x), fabsf(v[j][h].y)), fmaxf(fabsf(v[j][h].z), fabsf(v[j][h].w))));
    amax = wave_max(amax);
    if ((t & 63) == 0) red[t >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sc = 1.f;
    if (amax > 0.f && amax < 3.0e38f) {
        int e;
        frexpf(amax, &e);
        sc = ldexpf(1.f, 14 - e);
    }
    if (t == 0 && tok < m) inv_scale[tok] = 1.f / sc;
    f16x8 *dst = reinterpret_cast<f16x8 *>(xo) + (size_t)(tok >> 5) * ksteps * 64 + (tok & 31);
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int p = t + 256 * j;  // values 8 p .. 8 p + 7: K step p / 2, lane half p % 2
        if (p < npieces) {
            const float4 a = v[j][0], c = v[j][1];
            dst[(size_t)(p >> 1) * 64 + 32 * (p & 1)] = f16x8{(_Float16)(a.x * sc), (_Float16)(a.z * sc), (_Float16)(a.y * sc), (_Float16)(a.w * sc),
                                                             (_Float16)(c.x * sc), (_Float16)(c.z * sc), (_Float16)(c.y * sc), (_Float16)(c.w * sc)};
        }
    }
}

// 32 consecutive weights of a row, starting at value k0 (k0 % 32 == 0), in two phases so that the loads of the next
// K step can be in flight while the matrix cores work on the current one: pf_load fetches the raw bytes, pf_decode
// turns them into FP32 values in the dequantiser's arithmetic.
template <int FMT>
struct PfRaw;
template <>
struct PfRaw<F_Q4_0> { u32x4 q; uint32_t d; };
template <>
struct PfRaw<F_Q4_1> { u32x4 q; uint32_t dm; };
template <>
struct PfRaw<F_Q8_0> { u32x4 q0, q1; uint32_t d; };
template <>
struct PfRaw<F_Q4_K> { u32x4 h, q0, q1; };
template <>
struct PfRaw<F_Q5_K> { u32x4 h, q0, q1, qh0, qh1; };
template <>
struct PfRaw<F_Q6_K> { u32x4 l0, l1, h0, h1; uint32_t sc, d; };
template <>
struct PfRaw<F_Q5_1> { u32x4 q; uint32_t dm, qh; };
template <>
struct PfRaw<F_Q2_K> { u32x4 q0, q1; uint32_t sc, dd; };

template <int FMT>
__device__ __forceinline__ void pf_load(PfRaw<FMT> &r, const uint8_t *row, int k0) {
    if constexpr (FMT == F_Q4_0) {
        const uint8_t *b = row + (size_t)(k0 >> 5) * 18;
        r.d = ld16(b);
        r.q = ld128<2>(b + 2);
    } else if constexpr (FMT == F_Q4_1) {
        const uint8_t *b = row + (size_t)(k0 >> 5) * 20;
        r.dm = ld32<4>(b);
        r.q = ld128<4>(b + 4);
    } else if constexpr (FMT == F_Q5_1) {  // 24 bytes: d, m, 32 fifth bits, 16 bytes of nibbles
        const uint8_t *b = row + (size_t)(k0 >> 5) * 24;
        r.dm = ld32<4>(b);
        r.qh = ld32<4>(b + 4);
        r.q = ld128<4>(b + 8);
    } else if constexpr (FMT == F_Q2_K) {  // 84 bytes: 16 scale bytes, 64 bytes of 2-bit quants, d, dmin
        const uint8_t *b = row + (size_t)(k0 >> 8) * 84;
        const int e = k0 & 255, n = e >> 7, j = (e & 127) >> 5;
        r.q0 = ld128<4>(b + 16 + 32 * n);
        r.q1 = ld128<4>(b + 16 + 32 * n + 16);
        r.sc = ld16(b + 8 * n + 2 * j);
        r.dd = ld32<4>(b + 80);
    } else if constexpr (FMT == F_Q8_0) {
        const uint8_t *b = row + (size_t)(k0 >> 5) * 34;
        r.d = ld16(b);
        r.q0 = ld128<2>(b + 2);
        r.q1 = ld128<2>(b + 18);
    } else if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        constexpr int NB = FMT == F_Q4_K ? 144 : 176, QS = FMT == F_Q4_K ? 16 : 48;
        const uint8_t *b = row + (size_t)(k0 >> 8) * NB;
        const int j = (k0 & 255) >> 6;
        r.h = ld128<16>(b);
        r.q0 = ld128<16>(b + QS + 32 * j);
        r.q1 = ld128<16>(b + QS + 32 * j + 16);
        if constexpr (FMT == F_Q5_K) {
            r.qh0 = ld128<16>(b + 16);
            r.qh1 = ld128<16>(b + 32);
        }
    } else {
        const uint8_t *b = row + (size_t)(k0 >> 8) * 210;
        const int e = k0 & 255, n = e >> 7, kk = (e >> 5) & 3;
        r.l0 = ld128<2>(b + 64 * n + 32 * (kk & 1));
        r.l1 = ld128<2>(b + 64 * n + 32 * (kk & 1) + 16);
        r.h0 = ld128<2>(b + 128 + 32 * n);
        r.h1 = ld128<2>(b + 128 + 32 * n + 16);
        r.sc = ld16(b + 192 + 8 * n + 2 * kk);
        r.d = ld16(b + 208);
    }
}

template <int FMT>
__device__ __forceinline__ void pf_decode(const PfRaw<FMT> &r, int k0, float (&o)[32]) {
    if constexpr (FMT == F_Q4_0 || FMT == F_Q4_1) {
        float d, m = 0.f;
        if constexpr (FMT == F_Q4_0) {
            d = h2f(r.d);
        } else {
            d = h2f(r.dm);
            m = h2f(r.dm >> 16);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t byte = (r.q[i >> 2] >> (8 * (i & 3))) & 0xffu;
            if constexpr (FMT == F_Q4_0) {
                o[i] = (float)((int)(byte & 15u) - 8) * d;
                o[16 + i] = (float)((int)(byte >> 4) - 8) * d;
            } else {
                o[i] = (float)(byte & 15u) * d + m;
                o[16 + i] = (float)(byte >> 4) * d + m;
            }
        }
    } else if constexpr (FMT == F_Q5_1) {  // (q_low + 16 bit e of qh) d + m (GgufKernels.java:155-163)
        const float d = h2f(r.dm), m = h2f(r.dm >> 16);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t byte = (r.q[i >> 2] >> (8 * (i & 3))) & 0xffu;
            const float lo = (float)((byte & 15u) + 16u * ((r.qh >> i) & 1u)) * d, hi = (float)((byte >> 4) + 16u * ((r.qh >> (16 + i)) & 1u)) * d;
            o[i] = lo + m;
            o[16 + i] = hi + m;
        }
    } else if constexpr (FMT == F_Q2_K) {  // d (scale nibble) q - dmin (min nibble), a scale byte per 16 values (GgufKernels.java:166-175)
        const int j = ((k0 & 127) >> 5);
        const float d = h2f(r.dd), dmin = h2f(r.dd >> 16);
        const float ds0 = d * (float)(r.sc & 15u), m0 = dmin * (float)((r.sc >> 4) & 15u);
        const float ds1 = d * (float)((r.sc >> 8) & 15u), m1 = dmin * (float)((r.sc >> 12) & 15u);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = i < 16 ? r.q0[i >> 2] : r.q1[(i - 16) >> 2];
            const float a = (i < 16 ? ds0 : ds1) * (float)((w >> (8 * (i & 3) + 2 * j)) & 3u);
            o[i] = a - (i < 16 ? m0 : m1);
        }
    } else if constexpr (FMT == F_Q8_0) {
        const float d = h2f(r.d);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = i < 16 ? r.q0[i >> 2] : r.q1[(i - 16) >> 2];
            o[i] = d * (float)(int)(int8_t)((w >> (8 * (i & 3))) & 0xffu);
        }
    } else if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        const int e = k0 & 255, j = e >> 6, half = (e >> 5) & 1, sub = 2 * j + half;
        int sc, mn;
        {
            const uint32_t s0 = r.h.y, s1 = r.h.z, s2 = r.h.w;
            const int sh = 8 * (sub & 3);
            if (sub < 4) {
                sc = (s0 >> sh) & 63;
                mn = (s1 >> sh) & 63;
            } else {
                sc = ((s2 >> sh) & 15) | (((s0 >> sh) >> 6 & 3) << 4);
                mn = ((s2 >> sh) >> 4 & 15) | (((s1 >> sh) >> 6 & 3) << 4);
            }
        }
        const float ds = h2f(r.h.x) * (float)sc, m = h2f(r.h.x >> 16) * (float)mn;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = i < 16 ? r.q0[i >> 2] : r.q1[(i - 16) >> 2];
            uint32_t q = (w >> (8 * (i & 3) + 4 * half)) & 15u;
            if constexpr (FMT == F_Q5_K) {
                const uint32_t hw = i < 16 ? r.qh0[i >> 2] : r.qh1[(i - 16) >> 2];
                q += 16u * ((hw >> (8 * (i & 3) + sub)) & 1u);
            }
            o[i] = ds * (float)q - m;
        }
    } else {  // F_Q6_K
        const int kk = ((k0 & 255) >> 5) & 3;
        const float d = h2f(r.d);
        const float a0 = d * (float)(int)(int8_t)(r.sc & 0xffu), a1 = d * (float)(int)(int8_t)(r.sc >> 8);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t lw = i < 16 ? r.l0[i >> 2] : r.l1[(i - 16) >> 2];
            const uint32_t hw = i < 16 ? r.h0[i >> 2] : r.h1[(i - 16) >> 2];
            const int low = (lw >> (8 * (i & 3) + (kk < 2 ? 0 : 4))) & 15;
            const int hb = (hw >> (8 * (i & 3) + 2 * kk)) & 3;
            o[i] = (i < 16 ? a0 : a1) * (float)(low + 16 * hb - 32);
        }
    }
}

// Half-precision decoders for the two formats of a Q4_K_M model: the quants become exact FP16 integers without a
// conversion instruction (a byte OR-ed under the exponent 0x6400 is 1024 + byte; the 1024, and Q6_K's 32, come off
// with one exact packed add), and the block scale is applied with packed FP16 arithmetic, two weights per
// instruction.  Pairs come out as (byte 0, byte 2), (byte 1, byte 3) of each dword of quants: the 0, 2, 1, 3 order
// the activations are stored in.  Rounding: the scale product d*sc is rounded to FP16 once more than in the FP32
// decoder, still far inside the 2e-3 bar of this path.
typedef union { uint32_t u; f16x2 h; } pf_h2;

__device__ __forceinline__ f16x2 pf_pair(uint32_t u) { pf_h2 t; t.u = u; return t.h; }
__device__ __forceinline__ uint32_t pf_bits(f16x2 h) { pf_h2 t; t.h = h; return t.u; }
// 0x64006400 (FP16 1024.0 twice) held in a VGPR, so that (v & mask) | magic is a single v_and_or_b32: the instruction
// takes one scalar or literal operand only, and the mask is one already
__device__ __forceinline__ uint32_t pf_magic() {
    uint32_t m = 0x64006400u;
    asm("" : "+v"(m));
    return m;
}

template <int FMT>
__device__ __forceinline__ void pf_decode_h(const PfRaw<FMT> &r, int k0, f16x8 (&o)[4]);

template <>
__device__ __forceinline__ void pf_decode_h<F_Q4_K>(const PfRaw<F_Q4_K> &r, int k0, f16x8 (&o)[4]) {
    const int e = k0 & 255, j = e >> 6, half = (e >> 5) & 1, sub = 2 * j + half;
    int sc, mn;
    {
        // the eight 6-bit scales and mins bytewise, then this thread's pair by a shift: no branch, so that the decode
        // stays in the basic block of the MFMAs it is interleaved with
        const uint32_t s0 = r.h.y, s1 = r.h.z, s2 = r.h.w;
        const uint32_t scA = s0 & 0x3f3f3f3fu, scB = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
        const uint32_t mnA = s1 & 0x3f3f3f3fu, mnB = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
        const int sh = 8 * (sub & 3);
        sc = ((sub < 4 ? scA : scB) >> sh) & 0xff;
        mn = ((sub < 4 ? mnA : mnB) >> sh) & 0xff;
    }
    const _Float16 ds = (_Float16)(h2f(r.h.x) * (float)sc), nm = (_Float16)(-(h2f(r.h.x >> 16) * (float)mn));
    const f16x2 ds2 = {ds, ds}, nm2 = {nm, nm}, off = {(_Float16)-1024.f, (_Float16)-1024.f};
    const uint32_t mg = pf_magic();
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        u32x4 out;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int w = 2 * c + t;
            const uint32_t v = (w < 4 ? r.q0[w] : r.q1[w - 4]) >> (4 * half);
            const f16x2 a = pf_pair((v & 0x000f000fu) | mg) + off;         // bytes 0, 2
            const f16x2 b = pf_pair(((v >> 8) & 0x000f000fu) | mg) + off;  // bytes 1, 3
            out[2 * t] = pf_bits(__builtin_elementwise_fma(a, ds2, nm2));
            out[2 * t + 1] = pf_bits(__builtin_elementwise_fma(b, ds2, nm2));
        }
        o[c] = __builtin_bit_cast(f16x8, out);
    }
}

// Q5_K: the Q4_K decoder with the fifth bit of every quant (bit `sub` of the qh byte of its position) put above the
// nibble before the exponent trick.
template <>
__device__ __forceinline__ void pf_decode_h<F_Q5_K>(const PfRaw<F_Q5_K> &r, int k0, f16x8 (&o)[4]) {
    const int e = k0 & 255, j = e >> 6, half = (e >> 5) & 1, sub = 2 * j + half;
    int sc, mn;
    {
        const uint32_t s0 = r.h.y, s1 = r.h.z, s2 = r.h.w;
        const uint32_t scA = s0 & 0x3f3f3f3fu, scB = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
        const uint32_t mnA = s1 & 0x3f3f3f3fu, mnB = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
        const int sh = 8 * (sub & 3);
        sc = ((sub < 4 ? scA : scB) >> sh) & 0xff;
        mn = ((sub < 4 ? mnA : mnB) >> sh) & 0xff;
    }
    const _Float16 ds = (_Float16)(h2f(r.h.x) * (float)sc), nm = (_Float16)(-(h2f(r.h.x >> 16) * (float)mn));
    const f16x2 ds2 = {ds, ds}, nm2 = {nm, nm}, off = {(_Float16)-1024.f, (_Float16)-1024.f};
    const uint32_t mg = pf_magic();
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        u32x4 out;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int w = 2 * c + t;
            const uint32_t v = (w < 4 ? r.q0[w] : r.q1[w - 4]) >> (4 * half);
            const uint32_t hb = ((w < 4 ? r.qh0[w] : r.qh1[w - 4]) >> sub) << 4;  // bit 4 of bytes 0 .. 3 at bits 4, 12, 20, 28
            const f16x2 a = pf_pair((v & 0x000f000fu) | (hb & 0x00100010u) | mg) + off;                // bytes 0, 2
            const f16x2 b = pf_pair(((v >> 8) & 0x000f000fu) | ((hb >> 8) & 0x00100010u) | mg) + off;  // bytes 1, 3
            out[2 * t] = pf_bits(__builtin_elementwise_fma(a, ds2, nm2));
            out[2 * t + 1] = pf_bits(__builtin_elementwise_fma(b, ds2, nm2));
        }
        o[c] = __builtin_bit_cast(f16x8, out);
    }
}

template <>
__device__ __forceinline__ void pf_decode_h<F_Q6_K>(const PfRaw<F_Q6_K> &r, int k0, f16x8 (&o)[4]) {
    const int kk = ((k0 & 255) >> 5) & 3;
    const float d = h2f(r.d);
    const _Float16 a0 = (_Float16)(d * (float)(int)(int8_t)(r.sc & 0xffu)), a1 = (_Float16)(d * (float)(int)(int8_t)(r.sc >> 8));
    const f16x2 off = {(_Float16)-1056.f, (_Float16)-1056.f};  // -1024 of the exponent trick, -32 of the format
    const uint32_t mg = pf_magic();
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        u32x4 out;
        const f16x2 sc2 = c < 2 ? f16x2{a0, a0} : f16x2{a1, a1};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int w = 2 * c + t;
            const uint32_t lw = (w < 4 ? r.l0[w] : r.l1[w - 4]) >> (kk < 2 ? 0 : 4);
            const uint32_t hw = (w < 4 ? r.h0[w] : r.h1[w - 4]) >> (2 * kk);
            const uint32_t q = (lw & 0x0f0f0f0fu) | ((hw << 4) & 0x30303030u);  // four 6-bit quants, one per byte
            out[2 * t] = pf_bits((pf_pair((q & 0x00ff00ffu) | mg) + off) * sc2);             // bytes 0, 2
            out[2 * t + 1] = pf_bits((pf_pair(((q >> 8) & 0x00ff00ffu) | mg) + off) * sc2);  // bytes 1, 3
        }
        o[c] = __builtin_bit_cast(f16x8, out);
    }
}

// The 256-value formats reach LDS in two hops.  A thread's 32 weights of a step are a few 16-byte fields scattered
// over its row's block, so fetching them straight from global memory makes every load instruction of a wave touch
// 32 to 64 cache lines (one or two per row), and the CU's one vector L1 spends more cycles on tag look-ups than the
// matrix cores spend on the step.  Instead the workgroup copies the whole blocks of its 128 rows once per 256 values
// (four steps), consecutive lanes taking consecutive 16-byte chunks of a row (CPR per row; a Q6_K block is 13
// chunks and a 2-byte tail), into a double-buffered LDS area with a row pitch of RP bytes (16 x odd: conflict-free
// 16-byte reads, and every field a decoder reads with one 16-byte load is 16-byte aligned relative to the block);
// each step's decoder then reads its fields from there.
template <int FMT>
struct PfStage { static constexpr bool ON = false; static constexpr int NB = 16, CPR = 1, RP = 16, TAIL = 0, ALIGN = 16, NRAW = 0; };
template <>
struct PfStage<F_Q4_K> { static constexpr bool ON = false; static constexpr int NB = 144, CPR = 9, RP = 144, TAIL = 0, ALIGN = 16, NRAW = 3; };
template <>
struct PfStage<F_Q5_K> { static constexpr bool ON = true; static constexpr int NB = 176, CPR = 11, RP = 176, TAIL = 0, ALIGN = 16, NRAW = 5; };
template <>
struct PfStage<F_Q6_K> { static constexpr bool ON = true; static constexpr int NB = 210, CPR = 13, RP = 240, TAIL = 1, ALIGN = 2, NRAW = 6; };

// dynamic LDS of prefill_mfma_kernel<FMT>: the FP16 weight tile of two steps, then the staged raw blocks of two
// groups of four steps
template <int FMT>
constexpr size_t pf_lds_bytes() { return (size_t)2 * PF_BN * PF_LD * 2 + (PfStage<FMT>::ON ? (size_t)2 * PF_BN * PfStage<FMT>::RP : 0); }

// pf_load from a staged block: b = the row's block in LDS, e = first value within the block (a multiple of 32)
template <int FMT>
__device__ __forceinline__ void pf_load_lds(PfRaw<FMT> &r, const uint8_t *b, int e) {
    auto q = [&](int off) { return *reinterpret_cast<const u32x4 *>(b + off); };
    if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        constexpr int QS = FMT == F_Q4_K ? 16 : 48;
        const int j = e >> 6;
        r.h = q(0);
        r.q0 = q(QS + 32 * j);
        r.q1 = q(QS + 32 * j + 16);
        if constexpr (FMT == F_Q5_K) {
            r.qh0 = q(16);
            r.qh1 = q(32);
        }
    } else {
        static_assert(FMT == F_Q6_K, "staged formats");
        const int n = e >> 7, kk = (e >> 5) & 3;
        r.l0 = q(64 * n + 32 * (kk & 1));
        r.l1 = q(64 * n + 32 * (kk & 1) + 16);
        r.h0 = q(128 + 32 * n);
        r.h1 = q(128 + 32 * n + 16);
        r.sc = *reinterpret_cast<const uint16_t *>(b + 192 + 8 * n + 2 * kk);
        r.d = *reinterpret_cast<const uint16_t *>(b + 208);
    }
}

// The work of one workgroup: row tile `tile` of the weight W [n, k] against token tile blockIdx.y, K slice `slice`.
// DUAL (the gate and up projections of a Llama FFN, F.swiglu, F.java:1159-1161): the tile is rows [64 tile, +64) of W in
// its first two 32-row blocks and the same rows of W2 [n, k] in the other two, so that a lane holds the gate and the up
// product of one output in the same element of two accumulators, and y [m, n] = silu(x W^T) * (x W2^T) - the two products
// never go to memory.  No K slices, no bias.
// RT = 4: wave w owns all four 32-row blocks of the tile x tokens [64 w, +64).  RT = 2, for calls of at most 128 rows (the
// token slices of waves 2 and 3 would be empty, half the matrix cores would multiply zeros): wave w owns the row blocks
// w % 2 and w % 2 + 2 - a gate and its up block when DUAL - x tokens [64 (w / 2), +64): half the products per wave and step.
template <int FMT, bool DUAL = false, int RT = 4>
__device__ __forceinline__ void prefill_mfma_body(const uint8_t *__restrict__ W, const _Float16 *__restrict__ xo, const float *__restrict__ inv_scale,
                                                  const float *__restrict__ bias, float *__restrict__ y, const int m, const int n, const int k,
                                                  const int split_steps, const int tile, const int slice, const uint8_t *__restrict__ W2 = nullptr) {
    using Stage = PfStage<FMT>;
    constexpr bool STAGED = Stage::ON;
    extern __shared__ __align__(16) uint8_t pf_smem[];  // pf_lds_bytes<FMT>()
    _Float16(*As)[PF_BN * PF_LD] = reinterpret_cast<_Float16(*)[PF_BN * PF_LD]>(pf_smem);  // dequantised weights [row][k], two steps
    uint8_t *Rs = pf_smem + 2 * PF_BN * PF_LD * 2;                                         // staged raw blocks [2][row][RP]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = tile * (DUAL ? PF_BN / 2 : PF_BN), m0 = blockIdx.y * PF_BM;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    // dequantiser role: thread t fills weights [row t/2][32 * (t%2) ... +32) of the step
    const int drow = tid >> 1, dhalf = tid & 1;
    const uint8_t *wrow = (DUAL && drow >= PF_BN / 2 ? W2 : W) + (size_t)min(n0 + (DUAL ? drow & (PF_BN / 2 - 1) : drow), n - 1) * rowbytes;
    // MFMA role: wave w owns all 128 output rows x tokens [64 w, +64) as 4 x 2 tiles of 32 x 32: every weight operand
    // read from LDS feeds two MFMAs, every activation operand loaded from L2 feeds four
    const int ksteps = pf_ksteps(k);
    // B operands of token blocks m0/32 + 2 w + {0, 1}: 16 bytes per lane, consecutive K steps 1 KiB apart (the operand
    // array is padded to whole tiles of PF_BM tokens, so both blocks exist)
    const int tslice = RT == 4 ? wave : wave >> 1;                    // this wave's 64 tokens of the tile
    auto rblock = [&](int i) { return RT == 4 ? i : (wave & 1) + 2 * i; };  // the 32-row block of acc[i]
    const f16x8 *xb = reinterpret_cast<const f16x8 *>(xo) + ((size_t)(m0 / 32 + 2 * tslice) * ksteps) * 64 + lane;
    f32x16 acc[RT][2];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // Software pipeline over K: the B operands of a step are requested two steps ahead (a step of 32 MFMAs per wave
    // is shorter than a trip to memory), and so are the raw weight bytes of the 32-value formats (raw[] alternates);
    // the 256-value formats request the blocks of the next four steps during the first of four, park them in
    // registers (stg) and hand them to LDS during the third.  The weights of step s+1 are decoded into registers
    // (ah) after the MFMAs of step s have been issued.  The B operands rotate through three sets, the FP16 tile
    // through two, the staged blocks have a period of four steps: the loop is unrolled six steps (twelve for the
    // staged formats) so that all of them are fixed registers and addresses.
    // Nothing in a step is conditional - requests past the last step repeat the last step, a half step past the end
    // of a row (K = 32 mod 64) re-reads the row's last block and meets the zeros the operand array holds there - so
    // that the compiler can count the outstanding loads exactly and a step waits only for the loads it consumes.
    f16x8 ah[4];
    PfRaw<FMT> raw[2];
    f16x8 bq[3][2][4];
    // this workgroup's K steps: all of them, or slice `slice` of split_steps steps when the launch splits K (then y
    // is the slice's own [m, n] array of partial sums, to be added up by prefill_join_kernel; a slice of a staged
    // format starts on a multiple of four steps)
    const int sbeg = slice * split_steps, nsteps = min((k + PF_BK - 1) / PF_BK, sbeg + split_steps);
    y += (size_t)slice * m * n;
    auto wk = [&](int s) { return min(min(s, nsteps - 1) * PF_BK + 32 * dhalf, k - 32); };  // first value this thread decodes in step s
    auto fetch_w = [&](PfRaw<FMT> &r, int s) { pf_load<FMT>(r, wrow, wk(s)); };
    auto fetch_b = [&](f16x8(&b)[2][4], int s) {
        const f16x8 *p = xb + (size_t)min(s, nsteps - 1) * 4 * 64;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) b[j][ks] = p[((size_t)j * ksteps + ks) * 64];
    };
    auto decode = [&](const PfRaw<FMT> &r, int kk) {  // raw -> FP16 registers, values of each group of four in the order 0, 2, 1, 3
        if constexpr (FMT == F_Q4_K || FMT == F_Q5_K || FMT == F_Q6_K) {
            pf_decode_h<FMT>(r, kk, ah);
        } else {
            float v[32];
            pf_decode<FMT>(r, kk, v);
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int i = 0; i < 8; ++i) ah[c][(i & ~3) | pf_perm4(i & 3)] = (_Float16)v[8 * c + i];
        }
    };
    // ---- staging of the 256-value formats: the two threads of a row take its even and its odd 16-byte chunks (every
    // address is the row's plus a constant); the odd thread of a Q6_K row ends with the block's last two bytes
    constexpr int NCH = STAGED ? (Stage::CPR + Stage::TAIL + 1) / 2 : 1, RBUF = PF_BN * Stage::RP;
    const int nblk = k >> 8;
    u32x4 stg[NCH];
    auto stage_fetch = [&](int blk) {  // block number blk of the row (clamped: past the end, the last again)
        const uint8_t *p = wrow + (size_t)min(blk, nblk - 1) * Stage::NB + 16 * dhalf;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (32 * i + 32 <= Stage::NB) {
                stg[i] = ld128<Stage::ALIGN>(p + 32 * i);
            } else if constexpr (Stage::TAIL) {  // 16 bytes for the even thread, 2 for the odd one
                const uint8_t *q = p + 32 * i - 14 * dhalf;  // odd: the block's last 16 bytes, the tail in its top half-word
                stg[i] = ld128<Stage::ALIGN>(q);
            } else {  // the even thread's last chunk; the odd thread repeats its previous one
                stg[i] = ld128<Stage::ALIGN>(p + 32 * i - 32 * dhalf);
            }
        }
    };
    auto stage_store = [&](int buf) {
        uint8_t *d = Rs + buf * RBUF + drow * Stage::RP + 16 * dhalf;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (32 * i + 32 <= Stage::NB) {
                *reinterpret_cast<u32x4 *>(d + 32 * i) = stg[i];
            } else if constexpr (Stage::TAIL) {
                if (dhalf == 0) *reinterpret_cast<u32x4 *>(d + 32 * i) = stg[i];
                else *reinterpret_cast<uint16_t *>(d + 32 * i) = (uint16_t)(stg[i].w >> 16);
            } else {
                if (dhalf == 0) *reinterpret_cast<u32x4 *>(d + 32 * i) = stg[i];
            }
        }
    };
    // one K step: publish the decoded weights, request the loads of step s+2, multiply, decode step s+1.  ph = s % 4.
    auto step = [&](int s, int ph, int buf, f16x8(&bcur)[2][4], f16x8(&bfar)[2][4], PfRaw<FMT> &rfar, const PfRaw<FMT> &rnext) {
        {
            f16x8 *da = reinterpret_cast<f16x8 *>(&As[buf][drow * PF_LD + 32 * dhalf]);
#pragma unroll
            for (int c = 0; c < 4; ++c) da[c] = ah[c];
        }
        __syncthreads();  // the one barrier of the step: the other buffer was read before the previous one
        PfRaw<FMT> rl;
        if constexpr (STAGED) {
            // the staged buffer of steps 4 S .. 4 S + 3 is number S % 2: written during step 4 S - 2, read (for the
            // decode of the step after) during steps 4 S - 1 .. 4 S + 2, every pair a barrier apart
            if (ph == 0) stage_fetch((s >> 2) + 1);
            if (ph == 2) stage_store(((s >> 2) + 1) & 1);
            pf_load_lds<FMT>(rl, Rs + (((s + 1) >> 2) & 1) * RBUF + drow * Stage::RP, 64 * ((ph + 1) & 3) + 32 * dhalf);
        } else {
            fetch_w(rfar, s + 2);
        }
        fetch_b(bfar, s + 2);
        // ---- 4 k-substeps of 16: lane l supplies row l%32, halves 8*(l/32) .. +8 of the substep.  The weight operands
        // of a substep are read from LDS while the MFMAs of the one before run (one wave per SIMD: nobody else hides
        // the LDS latency).
        const _Float16 *ap = &As[buf][(lane & 31) * PF_LD + 8 * (lane >> 5)];
        f16x8 a[2][RT];
#pragma unroll
        for (int i = 0; i < RT; ++i) a[0][i] = *reinterpret_cast<const f16x8 *>(ap + 32 * rblock(i) * PF_LD);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks < 3) {
#pragma unroll
                for (int i = 0; i < RT; ++i) a[(ks + 1) & 1][i] = *reinterpret_cast<const f16x8 *>(ap + 32 * rblock(i) * PF_LD + 16 * (ks + 1));
            }
#pragma unroll
            for (int i = 0; i < RT; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bcur[j][ks], a[ks & 1][i], acc[i][j], 0, 0, 0);
        }
        if constexpr (STAGED) decode(rl, 64 * ((ph + 1) & 3) + 32 * dhalf);
        else decode(rnext, wk(s + 1));
        // One wave per SIMD: nobody else fills the matrix pipe while this wave decodes, or the VALU while it multiplies.
        // Ask the scheduler for the interleaving by hand: 32 times one MFMA and a few decode instructions, every other
        // time also one LDS operand read and one of the step's global loads.  The loads are spread over the step on
        // purpose: issued in one burst after the barrier, the four waves' requests queue up at the CU's one
        // address unit and the waves stall at the issue while the matrix pipe idles.
        __builtin_amdgcn_sched_group_barrier(0x100, RT + Stage::NRAW, 0);
#pragma unroll
        for (int i = 0; i < 8 * RT; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, RT == 4 ? 4 : 8, 0);  // (the decode of a step is as long whatever RT is)
            if (i % 2 == 0 && i < 6 * RT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (RT == 2 || i % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
    };
    if constexpr (STAGED) {
        stage_fetch(sbeg >> 2);
        stage_store((sbeg >> 2) & 1);
        __syncthreads();
        pf_load_lds<FMT>(raw[0], Rs + ((sbeg >> 2) & 1) * RBUF + drow * Stage::RP, 32 * dhalf);
        fetch_b(bq[0], sbeg);
        fetch_b(bq[1], sbeg + 1);
        decode(raw[0], 32 * dhalf);
    } else {
        fetch_w(raw[0], sbeg);
        fetch_b(bq[0], sbeg);
        fetch_w(raw[1], sbeg + 1);
        fetch_b(bq[1], sbeg + 1);
        decode(raw[0], wk(sbeg));
    }
    constexpr int UNR = STAGED ? 12 : 6;  // lcm of the rotation periods: 3 operand sets, 2 tiles (and raw sets), 4 steps per staged block
    int s0 = sbeg;
    for (; s0 + UNR <= nsteps; s0 += UNR) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) step(s0 + u, u & 3, u & 1, bq[u % 3], bq[(u + 2) % 3], raw[u & 1], raw[(u + 1) & 1]);
    }
#pragma unroll
    for (int u = 0; u < UNR - 1; ++u)
        if (s0 + u < nsteps) step(s0 + u, u & 3, u & 1, bq[u % 3], bq[(u + 2) % 3], raw[u & 1], raw[(u + 1) & 1]);
    // ---- epilogue.  The activations went in as the first MFMA operand, so an accumulator holds a 32 (tokens) x 32
    // (weight rows) block of y: element r is token 8*(r/4) + 4*(lane/32) + r%4, weight row lane%32 - the 32 lanes of a
    // half wave store 32 consecutive floats of one token's output row.  The 32 token scales of the lane are read
    // first, in one batch (index clamped, so the loads are unconditional): a load between the stores would make
    // every store wait for the one before it, stores and loads being counted by the same counter.
    const int tok0 = m0 + 64 * tslice + 4 * (lane >> 5);
    float isc[2][16];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) isc[j][r] = inv_scale[min(tok0 + 32 * j + 8 * (r >> 2) + (r & 3), m - 1)];
    if constexpr (DUAL) {
        // (the same expression, on the same two floats, as the activation preparation that forms silu(gate) * up from
        // stored products: XP_SWIGLU)
        auto sw = [](float g, float u) { return (g / (1.f + __expf(-g))) * u; };
#pragma unroll
        for (int i = 0; i < RT / 2; ++i) {  // accumulators i (gate) and i + RT / 2 (up): row blocks rblock(i) and rblock(i) + 2
            const int row = n0 + 32 * rblock(i) + (lane & 31);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int tok = tok0 + 32 * j + 8 * (r >> 2) + (r & 3);
                    if (row < n && tok < m) y[(size_t)tok * n + row] = sw(acc[i][j][r] * isc[j][r], acc[i + RT / 2][j][r] * isc[j][r]);
                }
            }
        }
        return;
    }
    float bv[RT];
    {
        const float *bp = bias ? bias : inv_scale;  // some readable address when there is no bias: the value is dropped
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const float b = bp[bias ? min(n0 + 32 * rblock(i) + (lane & 31), n - 1) : 0];
            bv[i] = bias ? b : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int row = n0 + 32 * rblock(i) + (lane & 31);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int tok = tok0 + 32 * j + 8 * (r >> 2) + (r & 3);
                if (row < n && tok < m) y[(size_t)tok * n + row] = acc[i][j][r] * isc[j][r] + bv[i];
            }
        }
    }
}

// Up to three weights of one activation in one launch (the q, k and v projections of a layer): their row tiles are
// numbered one after the other along blockIdx.x, every workgroup works on its weight exactly as in a launch of its own.
__device__ __forceinline__ void pf_locate(const PfSegments &sg, int &seg, int &tile, int &slice) {
    seg = 0;
    int idx = blockIdx.x;
    if (idx >= sg.tiles[0] * sg.splits[0]) {
        idx -= sg.tiles[0] * sg.splits[0];
        seg = 1;
        if (idx >= sg.tiles[1] * sg.splits[1]) {
            idx -= sg.tiles[1] * sg.splits[1];
            seg = 2;
        }
    }
    slice = idx / sg.tiles[seg];
    tile = idx - slice * sg.tiles[seg];
}

// grid: (row tiles x K slices of all segments, token tiles); 256 threads; pf_lds_bytes<FMT>() of dynamic LDS.
//   sg.y[i]: [m, n[i]], or for a segment that splits K the first slice's array of partial sums (slice z at + z m n[i]);
//   bias: one segment only.
template <int FMT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) prefill_mfma_kernel(const PfSegments sg, const _Float16 *__restrict__ xo,
                                                            const float *__restrict__ inv_scale, const float *__restrict__ bias,
                                                            int m, int k) {
    int seg, tile, slice;
    pf_locate(sg, seg, tile, slice);
    if (m <= PF_NARROW_ROWS) prefill_mfma_body<FMT, false, 2>(sg.W[seg], xo, inv_scale, bias, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
    else prefill_mfma_body<FMT>(sg.W[seg], xo, inv_scale, bias, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
}

// The same for weights of two formats (a Q4_K_M layer keeps q and k as Q4_K and v as Q6_K): segments below first_b are
// FA, the others FB.  LDS: the larger of the two.
template <int FA, int FB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) prefill_mfma_mixed_kernel(const PfSegments sg, const int first_b,
                                                            const _Float16 *__restrict__ xo, const float *__restrict__ inv_scale,
                                                            int m, int k) {
    int seg, tile, slice;
    pf_locate(sg, seg, tile, slice);
    if (m <= PF_NARROW_ROWS) {
        if (seg < first_b) prefill_mfma_body<FA, false, 2>(sg.W[seg], xo, inv_scale, nullptr, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
        else prefill_mfma_body<FB, false, 2>(sg.W[seg], xo, inv_scale, nullptr, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
    } else if (seg < first_b) {
        prefill_mfma_body<FA>(sg.W[seg], xo, inv_scale, nullptr, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
    } else {
        prefill_mfma_body<FB>(sg.W[seg], xo, inv_scale, nullptr, sg.y[seg], m, sg.n[seg], k, sg.split_steps[seg], tile, slice);
    }
}

// y [m, n] = silu(x W^T) * (x W2^T) for two weights [n, k] of one format: grid (ceil(n / 64), token tiles).
template <int FMT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) prefill_mfma_dual_kernel(const uint8_t *__restrict__ W,
                                                                                                            const uint8_t *__restrict__ W2,
                                                                                                            const _Float16 *__restrict__ xo,
                                                                                                            const float *__restrict__ inv_scale,
                                                                                                            float *__restrict__ y, int m, int n, int k) {
    if (m <= PF_NARROW_ROWS) prefill_mfma_body<FMT, true, 2>(W, xo, inv_scale, nullptr, y, m, n, k, (k + PF_BK - 1) / PF_BK, blockIdx.x, 0, W2);
    else prefill_mfma_body<FMT, true>(W, xo, inv_scale, nullptr, y, m, n, k, (k + PF_BK - 1) / PF_BK, blockIdx.x, 0, W2);
}

// y[tok, row] = sum over the K slices of part[z][tok, row] (+ bias[row]) (+ res[tok, row]), slices in order: the second half of a
// split-K launch.  count4 = m * n / 4 (n is a multiple of 4 whenever the launch splits).
static __global__ void __launch_bounds__(256) prefill_join_kernel(const float *__restrict__ part, const float *__restrict__ bias,
                                                                   const float *__restrict__ res, float *__restrict__ y, size_t count4, int n, int splits) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count4; i += (size_t)gridDim.x * 256) {
        float4 a = reinterpret_cast<const float4 *>(part)[i];
        for (int z = 1; z < splits; ++z) {
            const float4 b = reinterpret_cast<const float4 *>(part)[(size_t)z * count4 + i];
            a.x += b.x;
            a.y += b.y;
            a.z += b.z;
            a.w += b.w;
        }
        if (bias) {
            const float4 b = *reinterpret_cast<const float4 *>(bias + (i * 4) % (size_t)n);
            a.x += b.x;
            a.y += b.y;
            a.z += b.z;
            a.w += b.w;
        }
        if (res) {  // a residual [m, n] rides along (the layers of a model: y = x + W a)
            const float4 b = reinterpret_cast<const float4 *>(res)[i];
            a.x += b.x;
            a.y += b.y;
            a.z += b.z;
            a.w += b.w;
        }
        reinterpret_cast<float4 *>(y)[i] = a;
    }
}

// The join for a launch of several segments: part holds, segment after segment, splits[i] arrays [m, n[i]] of partial
// sums; y[i][tok, row] = their sum in slice order.  n[i] multiples of 4.
static __global__ void __launch_bounds__(256) prefill_join_group_kernel(const float *__restrict__ part, const PfSegments sg, int m) {
    const size_t c0 = (size_t)m * sg.n[0] / 4, c1 = (size_t)m * sg.n[1] / 4, c2 = (size_t)m * sg.n[2] / 4;
    const size_t o1 = c0 * sg.splits[0], o2 = o1 + c1 * sg.splits[1];
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < c0 + c1 + c2; i += (size_t)gridDim.x * 256) {
        const int seg = (i >= c0) + (i >= c0 + c1);
        const size_t cnt = seg == 0 ? c0 : seg == 1 ? c1 : c2, local = i - (seg == 0 ? 0 : seg == 1 ? c0 : c0 + c1);
        const float4 *p = reinterpret_cast<const float4 *>(part) + (seg == 0 ? 0 : seg == 1 ? o1 : o2) + local;
        const int splits = sg.splits[seg];
        float4 a = p[0];
        for (int z = 1; z < splits; ++z) {
            const float4 b = p[(size_t)z * cnt];
            a.x += b.x;
            a.y += b.y;
            a.z += b.z;
            a.w += b.w;
        }
        reinterpret_cast<float4 *>(sg.y[seg])[local] = a;
    }
}

}  // namespace jitnn