// Many-row linear (prefill, batches beyond the GEMV range) on raw GGUF blocks: y[M, N] = x[M, K] W[N, K]^T.
//
// This is the one shape on the path that is a real dense contraction, so it runs on the matrix cores:
//   1. x_to_f16_kernel turns each activation row into FP16 with a power-of-two row scale that puts its largest
//      magnitude in [2^13, 2^14) (no overflow for any FP32 input, no loss of small rows to FP16 subnormals);
//   2. prefill_mfma_kernel: a workgroup of four waves owns a 128 (weight rows) x 128 (tokens) output tile and
//      walks K in steps of 64.  Per step every thread dequantises 32 weights of one row from the raw blocks
//      (FP32 arithmetic of the dequantiser, then one rounding to FP16) into LDS, the FP16 activations of the
//      step are copied beside them, and each wave issues 16 v_mfma_f32_32x32x16_f16 on its 64 x 64 quadrant,
//      accumulating in FP32; the loads of the next step are in flight meanwhile.  The epilogue undoes the row
//      scale and adds the bias.
// Both FP16 roundings are relative 2^-11, so the result stays well inside the 2e-3 bar of the MFMA path.
#pragma once
#include "common.h"
#include "dequant.h"

namespace jitnn {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int PF_BN = 128, PF_BM = 128, PF_BK = 64, PF_LD = PF_BK + 8;  // LDS row pitch in halves: 144 bytes, conflict-free 16-byte reads

// position of value i (0..3) of a group of four in the FP16 operands: 0, 2, 1, 3
__host__ __device__ constexpr int pf_perm4(int i) { return ((i & 1) << 1) | (i >> 1); }

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
    // within each group of four values the FP16 copy is stored in the order 0, 2, 1, 3 - the order in which the weight
    // decoder produces FP16 pairs from a dword of quants (bytes 0 and 2, then 1 and 3); a dot product does not care
    _Float16 *o = xh + (size_t)blockIdx.x * k;
    for (int i = threadIdx.x; i < k; i += 256) o[(i & ~3) | pf_perm4(i & 3)] = (_Float16)(xr[i] * scale);
    if (threadIdx.x == 0) inv_scale[blockIdx.x] = 1.f / scale;
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

template <int FMT>
__device__ __forceinline__ void pf_decode_h(const PfRaw<FMT> &r, int k0, f16x8 (&o)[4]);

template <>
__device__ __forceinline__ void pf_decode_h<F_Q4_K>(const PfRaw<F_Q4_K> &r, int k0, f16x8 (&o)[4]) {
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
    const _Float16 ds = (_Float16)(h2f(r.h.x) * (float)sc), nm = (_Float16)(-(h2f(r.h.x >> 16) * (float)mn));
    const f16x2 ds2 = {ds, ds}, nm2 = {nm, nm}, off = {(_Float16)-1024.f, (_Float16)-1024.f};
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const uint32_t v = (w < 4 ? r.q0[w] : r.q1[w - 4]) >> (4 * half);
        const f16x2 a = pf_pair((v & 0x000f000fu) | 0x64006400u) + off;         // bytes 0, 2
        const f16x2 b = pf_pair(((v >> 8) & 0x000f000fu) | 0x64006400u) + off;  // bytes 1, 3
        const f16x2 wa = a * ds2 + nm2, wb = b * ds2 + nm2;
        o[w >> 1][4 * (w & 1) + 0] = wa.x;
        o[w >> 1][4 * (w & 1) + 1] = wa.y;
        o[w >> 1][4 * (w & 1) + 2] = wb.x;
        o[w >> 1][4 * (w & 1) + 3] = wb.y;
    }
}

template <>
__device__ __forceinline__ void pf_decode_h<F_Q6_K>(const PfRaw<F_Q6_K> &r, int k0, f16x8 (&o)[4]) {
    const int kk = ((k0 & 255) >> 5) & 3;
    const float d = h2f(r.d);
    const _Float16 a0 = (_Float16)(d * (float)(int)(int8_t)(r.sc & 0xffu)), a1 = (_Float16)(d * (float)(int)(int8_t)(r.sc >> 8));
    const f16x2 off = {(_Float16)-1056.f, (_Float16)-1056.f};  // -1024 of the exponent trick, -32 of the format
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const uint32_t lw = (w < 4 ? r.l0[w] : r.l1[w - 4]) >> (kk < 2 ? 0 : 4);
        const uint32_t hw = (w < 4 ? r.h0[w] : r.h1[w - 4]) >> (2 * kk);
        const uint32_t q = (lw & 0x0f0f0f0fu) | ((hw << 4) & 0x30303030u);  // four 6-bit quants, one per byte
        const f16x2 sc2 = w < 4 ? f16x2{a0, a0} : f16x2{a1, a1};
        const f16x2 a = (pf_pair((q & 0x00ff00ffu) | 0x64006400u) + off) * sc2;         // bytes 0, 2
        const f16x2 b = (pf_pair(((q >> 8) & 0x00ff00ffu) | 0x64006400u) + off) * sc2;  // bytes 1, 3
        o[w >> 1][4 * (w & 1) + 0] = a.x;
        o[w >> 1][4 * (w & 1) + 1] = a.y;
        o[w >> 1][4 * (w & 1) + 2] = b.x;
        o[w >> 1][4 * (w & 1) + 3] = b.y;
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

    // Software pipeline over K: the raw weight bytes and the FP16 activations of step s+1 are loaded while the matrix
    // cores work on step s, and decoded into registers (ah, bh) after the MFMAs have been issued.
    f16x8 ah[4], bh[4];
    PfRaw<FMT> raw;
    auto fetch = [&](int k0) {  // issue the global loads of one step for this thread
        const int kk = k0 + 32 * dhalf;
        if (kk < k) {
            pf_load<FMT>(raw, wrow, kk);
            const f16x8 *src = reinterpret_cast<const f16x8 *>(xrow + kk);
#pragma unroll
            for (int c = 0; c < 4; ++c) bh[c] = src[c];
        }
    };
    auto decode = [&](int k0) {  // raw -> FP16 registers, values of each group of four in the order 0, 2, 1, 3
        const int kk = k0 + 32 * dhalf;
        if (kk < k) {
            if constexpr (FMT == F_Q4_K || FMT == F_Q6_K) {
                pf_decode_h<FMT>(raw, kk, ah);
            } else {
                float v[32];
                pf_decode<FMT>(raw, kk, v);
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int i = 0; i < 8; ++i) ah[c][(i & ~3) | pf_perm4(i & 3)] = (_Float16)v[8 * c + i];
            }
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) ah[c] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (!(xlive && kk < k)) bh[c] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    };
    fetch(0);
    decode(0);
    for (int k0 = 0; k0 < k; k0 += PF_BK) {
        {
            f16x8 *da = reinterpret_cast<f16x8 *>(&As[drow * PF_LD + 32 * dhalf]);
            f16x8 *db = reinterpret_cast<f16x8 *>(&Bs[drow * PF_LD + 32 * dhalf]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                da[c] = ah[c];
                db[c] = bh[c];
            }
        }
        __syncthreads();
        const bool more = k0 + PF_BK < k;
        if (more) fetch(k0 + PF_BK);
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
        if (more) decode(k0 + PF_BK);
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
