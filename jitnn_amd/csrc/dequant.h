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

// Four consecutive values i..i+3 (i % 4 == 0) of a tensor: they share block, sub-block, nibble half and scale.
template <int FMT>
__device__ __forceinline__ float4 dequant4(const uint8_t *w, size_t i) {
    float o[4];
    if constexpr (FMT == F_Q4_0) {
        const uint8_t *b = w + (i >> 5) * 18;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b));
        const uint32_t vs = ld32<2>(b + 2 + (e & 15));  // the four bytes of the quad at once
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = (vs >> (8 * t)) & 255;
            int q = e < 16 ? (v & 15) : (v >> 4);
            o[t] = (float)(q - 8) * d;
        }
    } else if constexpr (FMT == F_Q4_1) {
        const uint8_t *b = w + (i >> 5) * 20;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b)), m = h2f(ld16(b + 2));
        const uint32_t vs = ld32<4>(b + 4 + (e & 15));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = (vs >> (8 * t)) & 255;
            int q = e < 16 ? (v & 15) : (v >> 4);
            float p = (float)q * d;
            o[t] = p + m;
        }
    } else if constexpr (FMT == F_Q8_0) {
        const uint8_t *b = w + (i >> 5) * 34;
        const int e = (int)(i & 31);
        const float d = h2f(ld16(b));
        const uint32_t vs = ld32<2>(b + 2 + e);
#pragma unroll
        for (int t = 0; t < 4; ++t) o[t] = d * (float)(int)(int8_t)(uint8_t)(vs >> (8 * t));
    } else if constexpr (FMT == F_Q4_K || FMT == F_Q5_K) {
        constexpr int NB = FMT == F_Q4_K ? 144 : 176, QS = FMT == F_Q4_K ? 16 : 48;
        const uint8_t *b = w + (i >> 8) * NB;
        const int e = (int)(i & 255);
        const int j = e >> 6, half = (e & 63) >> 5, l = e & 31, sub = 2 * j + half;
        // d, dmin and the twelve scale bytes as four dwords; the 6-bit scale and min of sub-block `sub` (GgufKernels.java:74-83):
        // bytes sub and sub + 4 for sub < 4, else a nibble of byte sub + 4 with the top two bits of byte sub - 4 or sub
        const uint32_t dm = ld32<4>(b), s0 = ld32<4>(b + 4), s1 = ld32<4>(b + 8), s2 = ld32<4>(b + 12);
        const int sh = 8 * (sub & 3);
        const int sc = sub < 4 ? (s0 >> sh) & 63 : ((s2 >> sh) & 15) | (((s0 >> (sh + 6)) & 3) << 4);
        const int mn = sub < 4 ? (s1 >> sh) & 63 : ((s2 >> (sh + 4)) & 15) | (((s1 >> (sh + 6)) & 3) << 4);
        const float ds = h2f(dm) * (float)sc;
        const float m = h2f(dm >> 16) * (float)mn;
        const uint32_t vs = ld32<4>(b + QS + 32 * j + l);
        uint32_t hs = 0;
        if constexpr (FMT == F_Q5_K) hs = ld32<4>(b + 16 + l);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int v = (vs >> (8 * t)) & 255;
            int q = half == 0 ? (v & 15) : (v >> 4);
            if constexpr (FMT == F_Q5_K) q += 16 * ((((hs >> (8 * t)) & 255) >> sub) & 1);
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
        constexpr int AL = FMT == F_Q5_0 ? 2 : 4;
        const uint32_t vs = ld32<AL>(b + QS + (e & 15)), qh = ld32<AL>(b + QH);  // the quad's nibble bytes; bit e of qh is value e's
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int v = (vs >> (8 * t)) & 255;
            const int q = (e < 16 ? (v & 15) : (v >> 4)) + 16 * ((qh >> (e + t)) & 1);
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
        const uint32_t vs = ld32<4>(b + 16 + n * 32 + l);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int q = (vs >> (8 * t + 2 * j)) & 3;
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
        const uint32_t vs = ld32<2>(b + 32 + n * 32 + l), hs = ld32<2>(b + l);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int q = (vs >> (8 * t + 2 * j)) & 3;
            const int hb = (hs >> (8 * t + 4 * n + j)) & 1;
            o[t] = a * (float)(q - (hb == 1 ? 0 : 4));
        }
    } else {  // F_Q6_K
        const uint8_t *b = w + (i >> 8) * 210;
        const int e = (int)(i & 255);
        const int n = e >> 7, k = (e & 127) >> 5, l = e & 31;
        const int sc = (int)(int8_t)b[192 + 8 * n + (l >> 4) + 2 * k];
        const float a = h2f(ld16(b + 208)) * (float)sc;
        const uint32_t ls = ld32<2>(b + 64 * n + l + (k & 1) * 32), hs = ld32<2>(b + 128 + 32 * n + l);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int lb = (ls >> (8 * t)) & 255;
            int low = k < 2 ? (lb & 15) : (lb >> 4);
            int hb = (((hs >> (8 * t)) & 255) >> (2 * k)) & 3;
            o[t] = a * (float)(low + 16 * hb - 32);
        }
    }
    return make_float4(o[0], o[1], o[2], o[3]);
}

// Q6_K: a lane's four values need bytes from four fields of the block, and four narrow load instructions per wave and
// 1 KiB of output keep the CU's one address unit busier than the memory behind it.  A wave takes a whole block - 64
// quads - instead: thirteen lanes fetch its 208 bytes as 16-byte pieces and a fourteenth its last 16 bytes for the two of d
// (one load instruction, nothing read past the block), the pieces are parted through the wave's own LDS region, and every lane
// decodes its quad from there with the same expressions.
template <int FMT>
__global__ void __launch_bounds__(256) dequant_kernel(const uint8_t *__restrict__ w, float *__restrict__ y, size_t quads) {
    if constexpr (FMT == F_Q6_K) {
        __shared__ __align__(16) uint8_t stage[4][224];
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const size_t nblk = quads / 64, nwaves = (size_t)gridDim.x * 4;
        for (size_t blk = (size_t)blockIdx.x * 4 + wave; blk < nblk; blk += nwaves) {
            const uint8_t *b = w + blk * 210;
            if (lane < 14) {  // (the fourteenth lane: the block's last 16 bytes, d in the top half-word)
                const u32x4 c = ld128<2>(b + (lane < 13 ? 16 * lane : 194));
                if (lane < 13) *reinterpret_cast<u32x4 *>(&stage[wave][16 * lane]) = c;
                else *reinterpret_cast<uint16_t *>(&stage[wave][208]) = (uint16_t)(c.w >> 16);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // (the lanes of a wave run in step, LDS serves them in order)
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            reinterpret_cast<float4 *>(y)[blk * 64 + lane] = dequant4<FMT>(stage[wave], (size_t)lane * 4);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    } else {
        for (size_t f = (size_t)blockIdx.x * blockDim.x + threadIdx.x; f < quads; f += (size_t)gridDim.x * blockDim.x) {
            reinterpret_cast<float4 *>(y)[f] = dequant4<FMT>(w, f * 4);
        }
    }
}

// Rows token[t] of a block-quantised table [vocab, k], dequantised bit-exactly into x [tokens, k] (the embedding lookup of
// a model whose token table is quantised).  grid = tokens.  An id outside [0, vocab) reads nothing: its row is NaN.
template <int FMT>
__global__ void __launch_bounds__(256) dequant_rows_kernel(const uint8_t *__restrict__ w, const int *__restrict__ tokens, float *__restrict__ x, int k,
                                                            int vocab) {
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int id = tokens[blockIdx.x];
    float4 *xr = reinterpret_cast<float4 *>(x + (size_t)blockIdx.x * k);
    if (id < 0 || id >= vocab) {
        const float nan = __builtin_nanf("");
        for (int f = threadIdx.x; f < (k >> 2); f += 256) xr[f] = make_float4(nan, nan, nan, nan);
        return;
    }
    const uint8_t *wr = w + (size_t)id * rowbytes;
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

// FP32 -> Q8_0 in the reference quantiser's arithmetic (core/ops/Quant.java:102-118): amax in double, d = (float)(amax / 127.0)
// stored as binary16 (round to nearest even), quants = round-half-away(x / (double)d) with the unrounded float d, clamped
// to +-127.  One block of 32 values, the reference's expressions as they stand:
__device__ __forceinline__ void quantize_q8_0_block(const float *__restrict__ xb, uint8_t *__restrict__ o) {
    double amax = 0;
#pragma unroll 1  // (rolled: this is the rare path of the kernel below, and must not cost it registers)
    for (int l = 0; l < 32; ++l) {
        double a = fabs((double)xb[l]);
        amax = a > amax ? a : amax;
    }
    const float d = (float)(amax / 127.0);
    o[0] = (uint8_t)(__half_as_ushort(__float2half_rn(d)) & 0xff);
    o[1] = (uint8_t)(__half_as_ushort(__float2half_rn(d)) >> 8);
#pragma unroll 1
    for (int l = 0; l < 32; ++l) {
        double s = d > 0 ? (double)xb[l] / (double)d : 0.0;
        long long r = s >= 0 ? (long long)(s + 0.5) : -(long long)(-s + 0.5);
        r = r < -127 ? -127 : (r > 127 ? 127 : r);
        o[2 + l] = (uint8_t)(int8_t)r;
    }
}

// The kernel: a wave takes Q8Q_BLOCKS consecutive blocks per turn with coalesced 16-byte loads - eight lanes share a
// block -, finds the block maxima with three lane exchanges, lets one lane per block do the one FP64
// division of d, and writes the blocks through its own LDS region as whole dwords.  The 32 FP64 divisions per block of
// the reference's expression are not needed for its bits: with q = |x| / d the exact quotient of two floats and
// 0.5 <= q < 128, 2 q - (2 k + 1) is either zero or at least 2^-24 in magnitude (numerator and denominator are 24-bit
// integers times a power of two that leaves the difference of the cross products an integer), while the division, and
// the addition of 0.5 after it, each err by at most 2^-46: the reference's result IS the exact quotient rounded half
// away from zero.  So: a candidate from one FP32 multiplication (off by one at most), set right by the signs of
// fma(r + 1/2, d, -|x|) and fma(r - 1/2, d, -|x|) - an FMA rounds the exact value once, its sign is the exact sign.
// Blocks with a value that is not finite or beyond 2^100, or a maximum below 2^-100 (d near or in the subnormals), take
// the reference's expression itself.  grid: any; 256 threads.
constexpr int Q8Q_NI = 4, Q8Q_BLOCKS = 8 * Q8Q_NI;  // 16-byte loads per lane and blocks per wave and turn
static __global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x, uint8_t *__restrict__ q, size_t blocks) {
    constexpr int NI = Q8Q_NI, NB = Q8Q_BLOCKS;
    __shared__ __align__(16) uint8_t out_s[4][NB * 34];
    __shared__ float amax_s[4][NB], d_s[4][NB];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane >> 3, part = lane & 7;
    auto wave_sync = [] {  // the lanes of a wave run in step and LDS serves them in order: a fence for the compiler
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    for (size_t w0 = ((size_t)blockIdx.x * 4 + wave) * NB; w0 < blocks; w0 += (size_t)gridDim.x * 4 * NB) {
        const int nb = (int)(blocks - w0 < NB ? blocks - w0 : NB);
        const float *xw = x + w0 * 32;
        float4 v[NI];
        bool odd = false;  // a value outside the range the short form is proven for
#pragma unroll
        for (int i = 0; i < NI; ++i)  // block 8 i + sub of the wave's, values 4 part .. 4 part + 3; all requests before the first use,
            v[i] = *reinterpret_cast<const float4 *>(xw + (8 * i + sub < nb ? 256 * i + 4 * lane : 4 * part));  // none conditional
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            if (8 * i + sub >= nb) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            const float a0 = fabsf(v[i].x), a1 = fabsf(v[i].y), a2 = fabsf(v[i].z), a3 = fabsf(v[i].w);
            odd |= !(a0 <= 0x1p100f) | !(a1 <= 0x1p100f) | !(a2 <= 0x1p100f) | !(a3 <= 0x1p100f);
            float m = fmaxf(fmaxf(a0, a1), fmaxf(a2, a3));
            m = fmaxf(m, __shfl_xor(m, 1));
            m = fmaxf(m, __shfl_xor(m, 2));
            m = fmaxf(m, __shfl_xor(m, 4));
            if (part == 0) amax_s[wave][8 * i + sub] = m;
        }
        wave_sync();
        if (lane < NB) {  // one lane per block: the scale
            const float am = amax_s[wave][lane];
            odd |= am > 0.f && am < 0x1p-100f;
            const float d = (float)((double)am / 127.0);
            d_s[wave][lane] = d;
            *reinterpret_cast<uint16_t *>(&out_s[wave][34 * lane]) = __half_as_ushort(__float2half_rn(d));
        }
        if (__any(odd)) {  // (wave-uniform) the reference's expression, a block per lane, straight to memory
            if (lane < nb) quantize_q8_0_block(xw + 32 * lane, q + (w0 + lane) * 34);
            wave_sync();
            continue;
        }
        wave_sync();
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int blk = 8 * i + sub;
            const float d0 = d_s[wave][blk], d = d0 > 0.f ? d0 : 1.f, inv = 1.0f / d;  // (a block of zeros: any scale gives zeros)
            const float xs[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
            uint32_t packed = 0;  // bytes q + 128, by the float -> byte converter that also places the byte
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = fabsf(xs[e]);
                float r = rintf(a * inv);
                // |x| / d >= r + 1/2: one more; |x| / d < r - 1/2: one less (never both).  No clamp: |x| <= amax and d is
                // amax / 127 rounded to float, so the quotient stays below 127.5.
                const float step = __builtin_fmaf(r + 0.5f, d, -a) <= 0.f ? 1.f : (__builtin_fmaf(r - 0.5f, d, -a) > 0.f ? -1.f : 0.f);
                packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_copysignf(r + step, xs[e]) + 128.f, e, packed);
            }
            packed ^= 0x80808080u;  // q + 128 -> the two's complement byte of q
            uint16_t *o = reinterpret_cast<uint16_t *>(&out_s[wave][34 * blk + 2 + 4 * part]);  // 2-byte aligned
            o[0] = (uint16_t)packed;
            o[1] = (uint16_t)(packed >> 16);
        }
        wave_sync();
        uint8_t *qw = q + w0 * 34;  // a multiple of NB blocks: 4-byte aligned whenever q is
        if (nb == NB && (reinterpret_cast<uintptr_t>(qw) & 3) == 0) {
            for (int j = lane; j < NB * 34 / 4; j += 64) reinterpret_cast<uint32_t *>(qw)[j] = reinterpret_cast<const uint32_t *>(out_s[wave])[j];
        } else {
            for (int j = lane; j < nb * 34; j += 64) qw[j] = out_s[wave][j];
        }
        wave_sync();  // the next round's writes wait for these reads
    }
}

}  // namespace jitnn
