// Batch-1..8 GEMV on raw GGUF blocks for gfx950 (wave64).
//
// Work decomposition.  A weight row of K values is cut into "units", the piece one lane decodes per step:
//   Q4_K / Q5_K : (super-block, j)        64 values  = 32 qs bytes (+ header, + qh for Q5_K)
//   Q6_K        : (super-block, half, l0) 64 values  = 2 x 16 ql bytes + 16 qh bytes + 4 scales
//   Q4_0 / Q4_1 / Q8_0 : one block        32 values
// Lane L of a wavefront takes unit it*64+L of each of R rows, so one wave step reads R contiguous
// stretches of a row with 128-bit loads, and a K=4096 row is one step (two for the 32-value formats).
// Activations are staged once per workgroup into LDS in "unit order" (the 16-byte quads of a unit side by
// side, one quad of padding per unit so that 128-bit LDS reads of neighbouring lanes fall on different
// banks) together with the partial sums of x that the offset terms of the formats need
// (sum over 32 values for the min of Q4_K/Q5_K/Q4_1 and the -8 / +128 recentring of Q4_0 / Q8_0, over 16
// for the -32 of Q6_K), so the inner loop is: mask nibbles, convert bytes to float, FMA.
// Each lane accumulates in FP32 over its K/64 values, then the 64 partial sums are added by a fixed DPP
// tree: the result does not depend on the launch shape, and no atomics are used.
#pragma once
#include "common.h"

namespace jitnn {

// CV = 1: turn four masked nibbles (bytes 0x00..0x0f) into floats with two v_cvt_pk_f32_fp8: an E4M3 byte
// below 0x10 decodes to exactly q * 2^-9 (OCP) or q * 2^-10 (FNUZ) in both the subnormal and the first
// normal binade; the power of two (passed as nib) is folded into the block scale.
// CV = 0: four v_cvt_f32_ubyte, nib = 1.
template <int CV>
__device__ __forceinline__ void cvt4(uint32_t v, float &a, float &b, float &c, float &d) {
    if constexpr (CV == 1) {
        f32x2 p = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false);
        f32x2 q = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, true);
        a = p.x; b = p.y; c = q.x; d = q.y;
    } else {
        a = ub0(v); b = ub1(v); c = ub2(v); d = ub3(v);
    }
}

__device__ __forceinline__ float dot4(float a, float b, float c, float d, const float4 &x, float acc) {
    acc = __builtin_fmaf(a, x.x, acc);
    acc = __builtin_fmaf(b, x.y, acc);
    acc = __builtin_fmaf(c, x.z, acc);
    acc = __builtin_fmaf(d, x.w, acc);
    return acc;
}

template <int FMT>
struct Unit;

// ---------------------------------------------------------------------------------------------- Q4_K
// block_q4_K, 144 bytes: f16 d, f16 dmin, u8 scales[12], u8 qs[128]; value e of the block:
// j=e/64, low nibble of qs[32j + e%32] when e%64 < 32 else high nibble, sub-block 2j + (e%64)/32
// (reference: core/kernels/GgufKernels.java:101-111, 6-bit scale/min unpack :74-83).
template <>
struct Unit<F_Q4_K> {
    static constexpr int UV = 64, NS = 2, SG = 8;
    struct Raw { u32x4 h, q0, q1; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *sb = row + (size_t)(u >> 2) * 144;
        r.h = ld128<16>(sb);
        r.q0 = ld128<16>(sb + 16 + (u & 3) * 32);
        r.q1 = ld128<16>(sb + 32 + (u & 3) * 32);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    // scale and min of sub-blocks 2j and 2j+1 as packed byte pairs
    __device__ static __forceinline__ void scale_min(const u32x4 &h, int j, uint32_t &sc2, uint32_t &mn2) {
        int sh = (j & 1) * 16;
        uint32_t a = h.y >> sh, b = h.z >> sh, c = h.w >> sh;
        uint32_t sc_lo = a & 0x3f3fu, mn_lo = b & 0x3f3fu;
        uint32_t sc_hi = (c & 0x0f0fu) | (((a >> 6) & 0x0303u) << 4);
        uint32_t mn_hi = ((c >> 4) & 0x0f0fu) | (((b >> 6) & 0x0303u) << 4);
        sc2 = j < 2 ? sc_lo : sc_hi;
        mn2 = j < 2 ? mn_lo : mn_hi;
    }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        float sl[R][B], sh[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) sl[r][b] = sh[r][b] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            float4 xa[B], xb[B];
#pragma unroll
            for (int b = 0; b < B; ++b) {
                xa[b] = xu[b * bs + d];
                xb[b] = xu[b * bs + d + 8];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t v = d < 4 ? w[r].q0[d & 3] : w[r].q1[d & 3];
                float l0, l1, l2, l3, h0, h1, h2, h3;
                cvt4<CV>(v & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((v >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    sl[r][b] = dot4(l0, l1, l2, l3, xa[b], sl[r][b]);
                    sh[r][b] = dot4(h0, h1, h2, h3, xb[b], sh[r][b]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            uint32_t sc2, mn2;
            scale_min(w[r].h, u & 3, sc2, mn2);
            float d = h2f(w[r].h.x) * nib, dmin = h2f(w[r].h.x >> 16);
            float d0 = d * ub0(sc2), d1 = d * ub1(sc2);
            float m0 = dmin * ub0(mn2), m1 = dmin * ub1(mn2);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float t = __builtin_fmaf(d0, sl[r][b], d1 * sh[r][b]);
                float m = __builtin_fmaf(m0, su[b * ss], m1 * su[b * ss + 1]);
                acc[r][b] += t - m;
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q5_K
// block_q5_K, 176 bytes: f16 d, f16 dmin, u8 scales[12], u8 qh[32], u8 qs[128]; as Q4_K plus bit
// (2j + half) of qh[e%32] as the fifth bit (reference: core/kernels/GgufKernels.java:113-125).
template <>
struct Unit<F_Q5_K> {
    static constexpr int UV = 64, NS = 2, SG = 8;
    struct Raw { u32x4 h, qh0, qh1, q0, q1; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *sb = row + (size_t)(u >> 2) * 176;
        r.h = ld128<16>(sb);
        r.qh0 = ld128<16>(sb + 16);
        r.qh1 = ld128<16>(sb + 32);
        r.q0 = ld128<16>(sb + 48 + (u & 3) * 32);
        r.q1 = ld128<16>(sb + 64 + (u & 3) * 32);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        (void)nib;
        const int j2 = (u & 3) * 2;
        float sl[R][B], sh[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) sl[r][b] = sh[r][b] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            float4 xa[B], xb[B];
#pragma unroll
            for (int b = 0; b < B; ++b) {
                xa[b] = xu[b * bs + d];
                xb[b] = xu[b * bs + d + 8];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t v = d < 4 ? w[r].q0[d & 3] : w[r].q1[d & 3];
                uint32_t t = (d < 4 ? w[r].qh0[d & 3] : w[r].qh1[d & 3]) >> j2;
                uint32_t lo = (v & 0x0f0f0f0fu) | ((t << 4) & 0x10101010u);
                uint32_t hi = ((v >> 4) & 0x0f0f0f0fu) | ((t << 3) & 0x10101010u);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    sl[r][b] = dot4(ub0(lo), ub1(lo), ub2(lo), ub3(lo), xa[b], sl[r][b]);
                    sh[r][b] = dot4(ub0(hi), ub1(hi), ub2(hi), ub3(hi), xb[b], sh[r][b]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            uint32_t sc2, mn2;
            Unit<F_Q4_K>::scale_min(w[r].h, u & 3, sc2, mn2);
            float d = h2f(w[r].h.x), dmin = h2f(w[r].h.x >> 16);
            float d0 = d * ub0(sc2), d1 = d * ub1(sc2);
            float m0 = dmin * ub0(mn2), m1 = dmin * ub1(mn2);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float t = __builtin_fmaf(d0, sl[r][b], d1 * sh[r][b]);
                float m = __builtin_fmaf(m0, su[b * ss], m1 * su[b * ss + 1]);
                acc[r][b] += t - m;
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q6_K
// block_q6_K, 210 bytes: u8 ql[128], u8 qh[64], i8 scales[16], f16 d; value e: n=e/128, k=(e%128)/32,
// l=e%32; low 4 bits = nibble (low for k<2, high otherwise) of ql[64n + 32(k%2) + l], high 2 bits =
// (qh[32n + l] >> 2k) & 3, minus 32, times scales[8n + 2k + l/16] (reference:
// core/kernels/GgufKernels.java:127-140).  Blocks start on 2-byte boundaries only.
// Unit u = 4*sb + 2*n + l0/16 covers l in [l0, l0+16) for the four k: 64 values in four runs of 16.
template <>
struct Unit<F_Q6_K> {
    static constexpr int UV = 64, NS = 4, SG = 4;
    struct Raw { u32x4 ql0, ql1, qh; u32x2 sc; uint32_t d; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *sb = row + (size_t)(u >> 2) * 210;
        const int n = (u >> 1) & 1, l0 = (u & 1) * 16;
        r.ql0 = ld128<2>(sb + 64 * n + l0);
        r.ql1 = ld128<2>(sb + 64 * n + 32 + l0);
        r.qh = ld128<2>(sb + 128 + 32 * n + l0);
        r.sc = ld64<2>(sb + 192 + 8 * n);
        r.d = ld16(sb + 208);
    }
    // x quad f (values 4f..4f+3 of the row) -> unit and quad within the unit (quad 4k + (l%16)/4)
    __device__ static __forceinline__ void slot(int f, int &u, int &g) {
        int e = (f & 63) * 4;  // position in the super-block
        int n = e >> 7, k = (e & 127) >> 5, l = e & 31;
        u = (f >> 6) * 4 + n * 2 + (l >> 4);
        g = 4 * k + ((l & 15) >> 2);
    }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        (void)nib;
        float s[R][B][4];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b)
#pragma unroll
                for (int k = 0; k < 4; ++k) s[r][b][k] = 0.f;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float4 x0[B], x1[B], x2[B], x3[B];
#pragma unroll
            for (int b = 0; b < B; ++b) {
                x0[b] = xu[b * bs + p];
                x1[b] = xu[b * bs + 4 + p];
                x2[b] = xu[b * bs + 8 + p];
                x3[b] = xu[b * bs + 12 + p];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t a = w[r].ql0[p], c = w[r].ql1[p], h = w[r].qh[p];
                uint32_t q0 = (a & 0x0f0f0f0fu) | ((h << 4) & 0x30303030u);
                uint32_t q1 = (c & 0x0f0f0f0fu) | ((h << 2) & 0x30303030u);
                uint32_t q2 = ((a >> 4) & 0x0f0f0f0fu) | (h & 0x30303030u);
                uint32_t q3 = ((c >> 4) & 0x0f0f0f0fu) | ((h >> 2) & 0x30303030u);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s[r][b][0] = dot4(ub0(q0), ub1(q0), ub2(q0), ub3(q0), x0[b], s[r][b][0]);
                    s[r][b][1] = dot4(ub0(q1), ub1(q1), ub2(q1), ub3(q1), x1[b], s[r][b][1]);
                    s[r][b][2] = dot4(ub0(q2), ub1(q2), ub2(q2), ub3(q2), x2[b], s[r][b][2]);
                    s[r][b][3] = dot4(ub0(q3), ub1(q3), ub2(q3), ub3(q3), x3[b], s[r][b][3]);
                }
            }
        }
        const int sh = (u & 1) * 8;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float d = h2f(w[r].d);
            float c0 = (float)(int)(int8_t)(w[r].sc.x >> sh);
            float c1 = (float)(int)(int8_t)(w[r].sc.x >> (sh + 16));
            float c2 = (float)(int)(int8_t)(w[r].sc.y >> sh);
            float c3 = (float)(int)(int8_t)(w[r].sc.y >> (sh + 16));
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const float *sb = su + b * ss;
                float t = c0 * __builtin_fmaf(-32.f, sb[0], s[r][b][0]);
                t = __builtin_fmaf(c1, __builtin_fmaf(-32.f, sb[1], s[r][b][1]), t);
                t = __builtin_fmaf(c2, __builtin_fmaf(-32.f, sb[2], s[r][b][2]), t);
                t = __builtin_fmaf(c3, __builtin_fmaf(-32.f, sb[3], s[r][b][3]), t);
                acc[r][b] = __builtin_fmaf(d, t, acc[r][b]);
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q4_0
// block_q4_0, 18 bytes: f16 d, u8 qs[16]; value e: (nibble - 8) * d, low nibble of qs[e] for e < 16, high
// nibble of qs[e-16] otherwise (reference: core/kernels/GgufKernels.java:85-91).
template <>
struct Unit<F_Q4_0> {
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q; uint32_t d; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *b = row + (size_t)u * 18;
        r.d = ld16(b);
        r.q = ld128<2>(b + 2);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        (void)u;
        float s[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) s[r][b] = 0.f;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float4 xa[B], xb[B];
#pragma unroll
            for (int b = 0; b < B; ++b) {
                xa[b] = xu[b * bs + p];
                xb[b] = xu[b * bs + p + 4];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t v = w[r].q[p];
                float l0, l1, l2, l3, h0, h1, h2, h3;
                cvt4<CV>(v & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((v >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s[r][b] = dot4(l0, l1, l2, l3, xa[b], s[r][b]);
                    s[r][b] = dot4(h0, h1, h2, h3, xb[b], s[r][b]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float d = h2f(w[r].d);
#pragma unroll
            for (int b = 0; b < B; ++b)
                acc[r][b] = __builtin_fmaf(d, __builtin_fmaf(nib, s[r][b], -8.f * su[b * ss]), acc[r][b]);
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q4_1
// block_q4_1, 20 bytes: f16 d, f16 m, u8 qs[16]; value e: nibble * d + m (reference:
// core/kernels/GgufKernels.java:93-99).
template <>
struct Unit<F_Q4_1> {
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q; uint32_t dm; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *b = row + (size_t)u * 20;
        r.dm = ld32<4>(b);
        r.q = ld128<4>(b + 4);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        (void)u;
        float s[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) s[r][b] = 0.f;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float4 xa[B], xb[B];
#pragma unroll
            for (int b = 0; b < B; ++b) {
                xa[b] = xu[b * bs + p];
                xb[b] = xu[b * bs + p + 4];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t v = w[r].q[p];
                float l0, l1, l2, l3, h0, h1, h2, h3;
                cvt4<CV>(v & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((v >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s[r][b] = dot4(l0, l1, l2, l3, xa[b], s[r][b]);
                    s[r][b] = dot4(h0, h1, h2, h3, xb[b], s[r][b]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float d = h2f(w[r].dm) * nib, m = h2f(w[r].dm >> 16);
#pragma unroll
            for (int b = 0; b < B; ++b) acc[r][b] += __builtin_fmaf(d, s[r][b], m * su[b * ss]);
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q8_0
// block_q8_0, 34 bytes: f16 d, i8 qs[32]; value e: qs[e] * d (reference: core/ops/Quant.java:137-144).
// The signed bytes are flipped to unsigned (q + 128) so that one v_cvt_f32_ubyte converts them; the 128
// comes back out through the block sum of x.
template <>
struct Unit<F_Q8_0> {
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q0, q1; uint32_t d; };
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, int u) {
        const uint8_t *b = row + (size_t)u * 34;
        r.d = ld16(b);
        r.q0 = ld128<2>(b + 2);
        r.q1 = ld128<2>(b + 18);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const float4 *xu, int bs, const float *su, int ss,
                                               float (&acc)[R][B], float nib) {
        (void)u;
        (void)nib;
        float s[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) s[r][b] = 0.f;
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            float4 xa[B];
#pragma unroll
            for (int b = 0; b < B; ++b) xa[b] = xu[b * bs + p];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t v = (p < 4 ? w[r].q0[p & 3] : w[r].q1[p & 3]) ^ 0x80808080u;
#pragma unroll
                for (int b = 0; b < B; ++b) s[r][b] = dot4(ub0(v), ub1(v), ub2(v), ub3(v), xa[b], s[r][b]);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float d = h2f(w[r].d);
#pragma unroll
            for (int b = 0; b < B; ++b) acc[r][b] = __builtin_fmaf(d, __builtin_fmaf(-128.f, su[b * ss], s[r][b]), acc[r][b]);
        }
    }
};

// LDS bytes one staged K-chunk of `itc` wave steps takes for batch B.
template <int FMT>
__host__ __device__ constexpr size_t gemv_lds_bytes(int B, int itc) {
    return (size_t)B * itc * 64 * ((Unit<FMT>::UV / 4 + 1) * 16 + Unit<FMT>::NS * 4);
}

// y[b, row] = sum_k W[row, k] x[b, k] (+ bias[row]) for b < rows <= B.
//   grid: any number of workgroups of a multiple of 64 threads; waves take row groups of R rows round-robin.
//   itc : wave steps (64 units each) staged in LDS at a time; K beyond that is processed in further chunks,
//         each wave adding its partial sums to y (same wave, same order: deterministic).
template <int FMT, int B, int R, int CV>
__global__ void __launch_bounds__(512) gemv_lds_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                        const float *__restrict__ bias, float *__restrict__ y, int n, int k, int rows,
                                                        int itc, float nib) {
    using U = Unit<FMT>;
    constexpr int UQ = U::UV / 4, NS = U::NS, SG = U::SG;
    extern __shared__ float4 smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int units = k / U::UV;
    const int steps = (units + 63) >> 6;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int ngroups = (n + R - 1) / R;
    const int bs = itc * 64 * (UQ + 1);  // float4 stride between batch rows
    const int ss = itc * 64 * NS;        // float stride between batch rows of the partial sums
    float4 *xl = smem;
    float *sums = reinterpret_cast<float *>(xl + (size_t)B * bs);
    const int kq = k >> 2;  // quads per activation row

    for (int c0 = 0; c0 < steps; c0 += itc) {
        const int nit = min(itc, steps - c0);
        if (c0 > 0) __syncthreads();
        // ---- stage x[:, chunk] in unit order, with the partial sums of each group of SG quads
        const int f0 = c0 * 64 * UQ, f1 = (c0 + nit) * 64 * UQ;  // quad range of the chunk (may run past kq: zero fill)
        for (int b = 0; b < B; ++b) {
            for (int f = f0 + tid; f < f1; f += blockDim.x) {  // f1 - f0 is a multiple of 64: whole waves
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (f < kq && b < rows) v = reinterpret_cast<const float4 *>(x + (size_t)b * k)[f];
                int u, g;
                U::slot(f, u, g);
                u -= c0 * 64;
                xl[(size_t)b * bs + (size_t)u * (UQ + 1) + g] = v;
                float s = (v.x + v.y) + (v.z + v.w);
#pragma unroll
                for (int m = 1; m < SG; m <<= 1) s += __shfl_xor(s, m);
                if ((f & (SG - 1)) == 0) sums[(size_t)b * ss + u * NS + g / SG] = s;
            }
        }
        __syncthreads();
        // ---- row groups
        for (int rg = blockIdx.x * nwaves + wave; rg < ngroups; rg += gridDim.x * nwaves) {
            float acc[R][B];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int b = 0; b < B; ++b) acc[r][b] = 0.f;
            for (int it = 0; it < nit; ++it) {
                const int u = (c0 + it) * 64 + lane;
                const int uc = min(u, units - 1);  // lanes past the row end re-read the last unit against zeroed x
                typename U::Raw w[R];
#pragma unroll
                for (int r = 0; r < R; ++r) U::load(w[r], W + (size_t)min(rg * R + r, n - 1) * rowbytes, uc);
                U::template dot<B, R, CV>(w, uc, xl + (size_t)(it * 64 + lane) * (UQ + 1), bs, sums + (it * 64 + lane) * NS, ss, acc, nib);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    float t = wave_sum(acc[r][b]);
                    const int row = rg * R + r;
                    if (lane == 0 && row < n && b < rows) {
                        float *o = y + (size_t)b * n + row;
                        if (c0 == 0) {
                            *o = bias ? t + bias[row] : t;
                        } else {
                            *o += t;
                        }
                    }
                }
            }
        }
    }
}

}  // namespace jitnn
