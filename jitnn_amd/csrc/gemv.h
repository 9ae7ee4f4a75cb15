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

// Where a lane finds the activations of its unit: quad g (values 4g..4g+3 in unit order) and partial sum i of
// batch row b.  XLds reads them from the staged LDS copy; XReg holds them in registers (batch 1).
struct XLds {
    const float4 *xu;
    const float *su;
    int bs, ss;
    __device__ __forceinline__ float4 q(int b, int g) const { return xu[b * bs + g]; }
    __device__ __forceinline__ float s(int b, int i) const { return su[b * ss + i]; }
};
template <int UQ, int NS>
struct XReg {
    float4 x[UQ];
    float sm[NS];
    __device__ __forceinline__ float4 q(int, int g) const { return x[g]; }
    __device__ __forceinline__ float s(int, int i) const { return sm[i]; }
};
// the same for two batch rows (128 VGPRs of activations per lane)
template <int UQ, int NS>
struct XReg2 {
    float4 x[2][UQ];
    float sm[2][NS];
    __device__ __forceinline__ float4 q(int b, int g) const { return x[b][g]; }
    __device__ __forceinline__ float s(int b, int i) const { return sm[b][i]; }
};

template <int FMT>
struct Unit;

// ---------------------------------------------------------------------------------------------- Q4_K
// block_q4_K, 144 bytes: f16 d, f16 dmin, u8 scales[12], u8 qs[128]; value e of the block:
// j=e/64, low nibble of qs[32j + e%32] when e%64 < 32 else high nibble, sub-block 2j + (e%64)/32
// (reference: core/kernels/GgufKernels.java:101-111, 6-bit scale/min unpack :74-83).
template <>
struct Unit<F_Q4_K> {
    static constexpr int FMT = F_Q4_K;
    static constexpr int UV = 64, NS = 2, SG = 8;
    struct Raw { u32x4 h, q0, q1; };
    static constexpr int NOFF = 2;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) {
        o[0] = (uint32_t)(u >> 2) * 144u;
        o[1] = o[0] + 16u + (uint32_t)(u & 3) * 32u;
    }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.h = ld128<16>(row + o[0]);
        r.q0 = ld128<16>(row + o[1]);
        r.q1 = ld128<16>(row + o[1] + 16);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    // scale and min of sub-blocks 2j and 2j+1 as packed byte pairs (ggml's get_scale_min_k4 on two sub-blocks at
    // once): for j < 2 the low six bits of scale bytes 2j.. and 4+2j..; for j >= 2 a nibble of bytes 8+2(j-2)..
    // with the top two bits of bytes 2(j-2).. / 4+2(j-2)..  The three masks select the case without a branch.
    __device__ static __forceinline__ void scale_min(const u32x4 &h, int j, uint32_t &sc2, uint32_t &mn2) {
        const int sh = (j & 1) * 16;
        const uint32_t m1 = j < 2 ? 0x3f3fu : 0u, m2 = j < 2 ? 0u : 0x0f0fu, m3 = j < 2 ? 0u : 0x3030u;
        const uint32_t a = h.y >> sh, b = h.z >> sh, c = h.w >> sh;
        sc2 = (a & m1) | (c & m2) | ((a >> 2) & m3);
        mn2 = (b & m1) | ((c >> 4) & m2) | ((b >> 2) & m3);
    }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
        float sl[R][B], sh[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) sl[r][b] = sh[r][b] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            // decode the step's nibbles of every row first, then walk the batch rows: one pair of activation quads
            // is live at a time, whatever the batch size
            float lo[R][4], hi[R][4];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t v = d < 4 ? w[r].q0[d & 3] : w[r].q1[d & 3];
                cvt4<CV>(v & 0x0f0f0f0fu, lo[r][0], lo[r][1], lo[r][2], lo[r][3]);
                cvt4<CV>((v >> 4) & 0x0f0f0f0fu, hi[r][0], hi[r][1], hi[r][2], hi[r][3]);
            }
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const float4 xa = xs.q(b, d), xb = xs.q(b, d + 8);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    sl[r][b] = dot4(lo[r][0], lo[r][1], lo[r][2], lo[r][3], xa, sl[r][b]);
                    sh[r][b] = dot4(hi[r][0], hi[r][1], hi[r][2], hi[r][3], xb, sh[r][b]);
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
                float m = __builtin_fmaf(m0, xs.s(b, 0), m1 * xs.s(b, 1));
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
    static constexpr int FMT = F_Q5_K;
    static constexpr int UV = 64, NS = 2, SG = 8;
    struct Raw { u32x4 h, qh0, qh1, q0, q1; };
    static constexpr int NOFF = 2;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) {
        o[0] = (uint32_t)(u >> 2) * 176u;
        o[1] = o[0] + 48u + (uint32_t)(u & 3) * 32u;
    }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.h = ld128<16>(row + o[0]);
        r.qh0 = ld128<16>(row + o[0] + 16);
        r.qh1 = ld128<16>(row + o[0] + 32);
        r.q0 = ld128<16>(row + o[1]);
        r.q1 = ld128<16>(row + o[1] + 16);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
        (void)nib;
        const int j2 = (u & 3) * 2;
        float sl[R][B], sh[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) sl[r][b] = sh[r][b] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            uint32_t lo[R], hi[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t v = d < 4 ? w[r].q0[d & 3] : w[r].q1[d & 3];
                const uint32_t t = (d < 4 ? w[r].qh0[d & 3] : w[r].qh1[d & 3]) >> j2;
                lo[r] = (v & 0x0f0f0f0fu) | ((t << 4) & 0x10101010u);
                hi[r] = ((v >> 4) & 0x0f0f0f0fu) | ((t << 3) & 0x10101010u);
            }
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const float4 xa = xs.q(b, d), xb = xs.q(b, d + 8);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    sl[r][b] = dot4(ub0(lo[r]), ub1(lo[r]), ub2(lo[r]), ub3(lo[r]), xa, sl[r][b]);
                    sh[r][b] = dot4(ub0(hi[r]), ub1(hi[r]), ub2(hi[r]), ub3(hi[r]), xb, sh[r][b]);
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
                float m = __builtin_fmaf(m0, xs.s(b, 0), m1 * xs.s(b, 1));
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
    static constexpr int FMT = F_Q6_K;
    static constexpr int UV = 64, NS = 4, SG = 4;
    struct Raw { u32x4 ql0, ql1, qh; u32x2 sc; uint32_t d; };
    static constexpr int NOFF = 4;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) {
        const uint32_t sb = (uint32_t)(u >> 2) * 210u, n = (u >> 1) & 1, l0 = (u & 1) * 16;
        o[0] = sb + 64u * n + l0;  // ql (second half of the nibbles 32 bytes on)
        o[1] = sb + 32u * n + l0;  // qh, 128 bytes on
        o[2] = sb + 8u * n;        // scales, 192 bytes on
        o[3] = sb;                 // d, 208 bytes on
    }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.ql0 = ld128<2>(row + o[0]);
        r.ql1 = ld128<2>(row + o[0] + 32);
        r.qh = ld128<2>(row + o[1] + 128);
        r.sc = ld64<2>(row + o[2] + 192);
        r.d = ld16(row + o[3] + 208);
    }
    // x quad f (values 4f..4f+3 of the row) -> unit and quad within the unit (quad 4k + (l%16)/4)
    __device__ static __forceinline__ void slot(int f, int &u, int &g) {
        int e = (f & 63) * 4;  // position in the super-block
        int n = e >> 7, k = (e & 127) >> 5, l = e & 31;
        u = (f >> 6) * 4 + n * 2 + (l >> 4);
        g = 4 * k + ((l & 15) >> 2);
    }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
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
            uint32_t q0[R], q1[R], q2[R], q3[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t a = w[r].ql0[p], c = w[r].ql1[p], h = w[r].qh[p];
                q0[r] = (a & 0x0f0f0f0fu) | ((h << 4) & 0x30303030u);
                q1[r] = (c & 0x0f0f0f0fu) | ((h << 2) & 0x30303030u);
                q2[r] = ((a >> 4) & 0x0f0f0f0fu) | (h & 0x30303030u);
                q3[r] = ((c >> 4) & 0x0f0f0f0fu) | ((h >> 2) & 0x30303030u);
            }
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const float4 x0 = xs.q(b, p), x1 = xs.q(b, 4 + p), x2 = xs.q(b, 8 + p), x3 = xs.q(b, 12 + p);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    s[r][b][0] = dot4(ub0(q0[r]), ub1(q0[r]), ub2(q0[r]), ub3(q0[r]), x0, s[r][b][0]);
                    s[r][b][1] = dot4(ub0(q1[r]), ub1(q1[r]), ub2(q1[r]), ub3(q1[r]), x1, s[r][b][1]);
                    s[r][b][2] = dot4(ub0(q2[r]), ub1(q2[r]), ub2(q2[r]), ub3(q2[r]), x2, s[r][b][2]);
                    s[r][b][3] = dot4(ub0(q3[r]), ub1(q3[r]), ub2(q3[r]), ub3(q3[r]), x3, s[r][b][3]);
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
                float t = c0 * __builtin_fmaf(-32.f, xs.s(b, 0), s[r][b][0]);
                t = __builtin_fmaf(c1, __builtin_fmaf(-32.f, xs.s(b, 1), s[r][b][1]), t);
                t = __builtin_fmaf(c2, __builtin_fmaf(-32.f, xs.s(b, 2), s[r][b][2]), t);
                t = __builtin_fmaf(c3, __builtin_fmaf(-32.f, xs.s(b, 3), s[r][b][3]), t);
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
    static constexpr int FMT = F_Q4_0;
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q; uint32_t d; };
    static constexpr int NOFF = 1;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 18u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.d = ld16(row + o[0]);
        r.q = ld128<2>(row + o[0] + 2);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
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
                xa[b] = xs.q(b, p);
                xb[b] = xs.q(b, p + 4);
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
                acc[r][b] = __builtin_fmaf(d, __builtin_fmaf(nib, s[r][b], -8.f * xs.s(b, 0)), acc[r][b]);
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q4_1
// block_q4_1, 20 bytes: f16 d, f16 m, u8 qs[16]; value e: nibble * d + m (reference:
// core/kernels/GgufKernels.java:93-99).
template <>
struct Unit<F_Q4_1> {
    static constexpr int FMT = F_Q4_1;
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q; uint32_t dm; };
    static constexpr int NOFF = 1;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 20u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.dm = ld32<4>(row + o[0]);
        r.q = ld128<4>(row + o[0] + 4);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
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
                xa[b] = xs.q(b, p);
                xb[b] = xs.q(b, p + 4);
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
            for (int b = 0; b < B; ++b) acc[r][b] += __builtin_fmaf(d, s[r][b], m * xs.s(b, 0));
        }
    }
};

// ---------------------------------------------------------------------------------------------- Q8_0
// block_q8_0, 34 bytes: f16 d, i8 qs[32]; value e: qs[e] * d (reference: core/ops/Quant.java:137-144).
// The signed bytes are flipped to unsigned (q + 128) so that one v_cvt_f32_ubyte converts them; the 128
// comes back out through the block sum of x.
template <>
struct Unit<F_Q8_0> {
    static constexpr int FMT = F_Q8_0;
    static constexpr int UV = 32, NS = 1, SG = 8;
    struct Raw { u32x4 q0, q1; uint32_t d; };
    static constexpr int NOFF = 1;
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 34u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.d = ld16(row + o[0]);
        r.q0 = ld128<2>(row + o[0] + 2);
        r.q1 = ld128<2>(row + o[0] + 18);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 3; g = f & 7; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
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
            for (int b = 0; b < B; ++b) xa[b] = xs.q(b, p);
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
            for (int b = 0; b < B; ++b) acc[r][b] = __builtin_fmaf(d, __builtin_fmaf(-128.f, xs.s(b, 0), s[r][b]), acc[r][b]);
        }
    }
};

// ------------------------------------------------------------------------------------- pairs of 32-value blocks
// For rows whose block count is even, the 32-value formats are decoded two blocks per lane: a pair of blocks
// starts on a 4-byte boundary (36, 40 and 68 bytes), so the lane fetches it with aligned 128-bit loads and
// realigns the half-word-shifted quants of the first block with v_alignbit instead of issuing loads that
// straddle dwords.  The unit is 64 values like the k-quants': one wave step per 4096 values.
template <int FMT>
struct UnitPair;

// two block_q4_0: bytes 0-1 d0, 2-17 qs0, 18-19 d1, 20-35 qs1
template <>
struct UnitPair<F_Q4_0> {
    static constexpr int FMT = F_Q4_0;
    static constexpr int UV = 64, NS = 2, SG = 8, NOFF = 1;
    struct Raw { u32x4 a, b; uint32_t c; };
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 36u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.a = ld128<4>(row + o[0]);
        r.b = ld128<4>(row + o[0] + 16);
        r.c = ld32<4>(row + o[0] + 32);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
        (void)u;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t q0[4] = {__builtin_amdgcn_alignbit(w[r].a.y, w[r].a.x, 16), __builtin_amdgcn_alignbit(w[r].a.z, w[r].a.y, 16),
                                    __builtin_amdgcn_alignbit(w[r].a.w, w[r].a.z, 16), __builtin_amdgcn_alignbit(w[r].b.x, w[r].a.w, 16)};
            const uint32_t q1[4] = {w[r].b.y, w[r].b.z, w[r].b.w, w[r].c};
            float s0[B], s1[B];
#pragma unroll
            for (int b = 0; b < B; ++b) s0[b] = s1[b] = 0.f;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                float l0, l1, l2, l3, h0, h1, h2, h3;
                cvt4<CV>(q0[p] & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((q0[p] >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s0[b] = dot4(l0, l1, l2, l3, xs.q(b, p), s0[b]);
                    s0[b] = dot4(h0, h1, h2, h3, xs.q(b, p + 4), s0[b]);
                }
                cvt4<CV>(q1[p] & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((q1[p] >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s1[b] = dot4(l0, l1, l2, l3, xs.q(b, 8 + p), s1[b]);
                    s1[b] = dot4(h0, h1, h2, h3, xs.q(b, 12 + p), s1[b]);
                }
                }
            const float d0 = h2f(w[r].a.x), d1 = h2f(w[r].b.x >> 16);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float t = d0 * __builtin_fmaf(nib, s0[b], -8.f * xs.s(b, 0));
                acc[r][b] += __builtin_fmaf(d1, __builtin_fmaf(nib, s1[b], -8.f * xs.s(b, 1)), t);
            }
        }
    }
};

// two block_q4_1: bytes 0-3 d0 m0, 4-19 qs0, 20-23 d1 m1, 24-39 qs1
template <>
struct UnitPair<F_Q4_1> {
    static constexpr int FMT = F_Q4_1;
    static constexpr int UV = 64, NS = 2, SG = 8, NOFF = 1;
    struct Raw { u32x4 a, b; u32x2 c; };
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 40u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.a = ld128<4>(row + o[0]);
        r.b = ld128<4>(row + o[0] + 16);
        r.c = *reinterpret_cast<const u32x2 *>(row + o[0] + 32);  // 40u + 32 is a multiple of 8
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
        (void)u;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t q0[4] = {w[r].a.y, w[r].a.z, w[r].a.w, w[r].b.x};
            const uint32_t q1[4] = {w[r].b.z, w[r].b.w, w[r].c.x, w[r].c.y};
            float s0[B], s1[B];
#pragma unroll
            for (int b = 0; b < B; ++b) s0[b] = s1[b] = 0.f;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                float l0, l1, l2, l3, h0, h1, h2, h3;
                cvt4<CV>(q0[p] & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((q0[p] >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s0[b] = dot4(l0, l1, l2, l3, xs.q(b, p), s0[b]);
                    s0[b] = dot4(h0, h1, h2, h3, xs.q(b, p + 4), s0[b]);
                }
                cvt4<CV>(q1[p] & 0x0f0f0f0fu, l0, l1, l2, l3);
                cvt4<CV>((q1[p] >> 4) & 0x0f0f0f0fu, h0, h1, h2, h3);
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s1[b] = dot4(l0, l1, l2, l3, xs.q(b, 8 + p), s1[b]);
                    s1[b] = dot4(h0, h1, h2, h3, xs.q(b, 12 + p), s1[b]);
                }
                }
            const float d0 = h2f(w[r].a.x) * nib, m0 = h2f(w[r].a.x >> 16), d1 = h2f(w[r].b.y) * nib, m1 = h2f(w[r].b.y >> 16);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float t = __builtin_fmaf(d0, s0[b], m0 * xs.s(b, 0));
                t = __builtin_fmaf(d1, s1[b], t);
                acc[r][b] += __builtin_fmaf(m1, xs.s(b, 1), t);
            }
        }
    }
};

// two block_q8_0: bytes 0-1 d0, 2-33 qs0, 34-35 d1, 36-67 qs1
template <>
struct UnitPair<F_Q8_0> {
    static constexpr int FMT = F_Q8_0;
    static constexpr int UV = 64, NS = 2, SG = 8, NOFF = 1;
    struct Raw { u32x4 a, b, c, d; uint32_t e; };
    __device__ static __forceinline__ void offsets(int u, uint32_t (&o)[NOFF]) { o[0] = (uint32_t)u * 68u; }
    __device__ static __forceinline__ void load(Raw &r, const uint8_t *row, const uint32_t (&o)[NOFF]) {
        r.a = ld128<4>(row + o[0]);
        r.b = ld128<4>(row + o[0] + 16);
        r.c = ld128<4>(row + o[0] + 32);
        r.d = ld128<4>(row + o[0] + 48);
        r.e = ld32<4>(row + o[0] + 64);
    }
    __device__ static __forceinline__ void slot(int f, int &u, int &g) { u = f >> 4; g = f & 15; }

    template <int B, int R, int CV, class X>
    __device__ static __forceinline__ void dot(const Raw (&w)[R], int u, const X &xs, float (&acc)[R][B], float nib) {
        (void)u;
        (void)nib;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t v[17] = {w[r].a.x, w[r].a.y, w[r].a.z, w[r].a.w, w[r].b.x, w[r].b.y, w[r].b.z, w[r].b.w, w[r].c.x,
                                    w[r].c.y, w[r].c.z, w[r].c.w, w[r].d.x, w[r].d.y, w[r].d.z, w[r].d.w, w[r].e};
            float s0[B], s1[B];
#pragma unroll
            for (int b = 0; b < B; ++b) s0[b] = s1[b] = 0.f;
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const uint32_t a = __builtin_amdgcn_alignbit(v[p + 1], v[p], 16) ^ 0x80808080u;
                const uint32_t c = v[9 + p] ^ 0x80808080u;
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    s0[b] = dot4(ub0(a), ub1(a), ub2(a), ub3(a), xs.q(b, p), s0[b]);
                    s1[b] = dot4(ub0(c), ub1(c), ub2(c), ub3(c), xs.q(b, 8 + p), s1[b]);
                }
                }
            const float d0 = h2f(v[0]), d1 = h2f(v[8] >> 16);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float t = d0 * __builtin_fmaf(-128.f, xs.s(b, 0), s0[b]);
                acc[r][b] += __builtin_fmaf(d1, __builtin_fmaf(-128.f, xs.s(b, 1), s1[b]), t);
            }
        }
    }
};

// Batch-1 GEMV for rows of at most 4096 values: the activations live in registers.
//
// The vector is staged through LDS once per workgroup (coalesced global read, unit-order write), each lane
// then pulls the 64 floats of its own units (STEPS units of UV values, STEPS * UV = 64) and their partial
// sums into VGPRs and never touches LDS again.  Every wave walks the rows gw, gw + W, gw + 2W, ... (W = waves
// in the grid), one row per iteration, through a ring of PF + 1 register buffers: while one row is decoded
// the loads of the next PF rows are in flight, and a buffer is refilled as soon as its row is done.  The
// loads are unconditional (rows past the end re-read the last row) so that the hardware's in-order load
// counter can be waited on exactly; only the decode and the store are skipped for rows that do not exist.
// The first rows' loads are issued before the staging barrier, so HBM latency overlaps the staging too.
// Wave priority by the rows a wave still has to do.  The SIMD's arbiter serves its oldest wave first: of the waves
// that share a SIMD one runs ahead, and the others are left to finish alone at the issue rate of a single wave (about
// half of what two reach together).  With the priority stepping down as the last rows come up (more than 8, 4, 2 rows
// left), whoever is behind at a step is served first until it has caught up, and the waves of a SIMD finish together.
__device__ __forceinline__ void step_priority(int left) {
    if (left > 8) __builtin_amdgcn_s_setprio(3);
    else if (left > 4) __builtin_amdgcn_s_setprio(2);
    else if (left > 2) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

constexpr int XREG_THREADS = 256;  // workgroup size of gemv_xreg_kernel (compile-time: the staging is fully unrolled)

// Arguments of gemv_xreg_kernel.  Up to three matrices of the same format and row length share one launch and
// one activation vector (the q and k projections of a decode step): their rows are numbered one after the other.
struct XregArgs {
    const uint8_t *w[3];   // row segments: n[i] rows each, all [*, k] in the kernel's format
    float *y[3];           // outputs of the segments
    const float *bias[3];  // BIAS: added to the segment's rows (a residual rides here), else ignored
    int n[3];
    const uint8_t *w2;     // DUAL: second matrix of the shape of w[0]; the kernel writes silu(w[0] x) * (w2 x) to y[0]
    const float *x;        // [k]
    const float *nw;       // NORM: RMSNorm weight [k]; the kernel multiplies x by nw / sqrt(mean(x^2) + eps) while staging it
    float eps;
    int k;
    float nib;
    int rpw;  // rows the busiest wave sees (0: no priority steps)
};

// Extra template switches:
//   NORM  fuses the RMSNorm that precedes the linear (ops/RowNorm.java:286-306) into the staging of x;
//   DUAL  computes the SwiGLU gate of a Llama FFN (F.swiglu, F.java:1159-1161) from two matrices in one pass: the
//         ring alternates rows of w[0] (gate) and w2 (up), so NB = PF + 1 must be even.
// The body takes its workgroup number and the number of workgroups as arguments so that two of them, for two
// formats, can share one launch (gemv_xreg2_kernel).
template <class U, int CV, int PF, bool BIAS, bool NORM, bool DUAL>
__device__ __forceinline__ void gemv_xreg_body(const XregArgs &a, const int bid, const int nblocks) {
    constexpr int FMT = U::FMT, STEPS = 64 / U::UV;  // a lane keeps 64 activations: one 64-value unit or two of 32
    constexpr int UQ = U::UV / 4, NS = U::NS, SG = U::SG, NB = PF + 1;
    static_assert(!DUAL || NB % 2 == 0, "gate and up rows alternate in the ring");
    constexpr int RSTEP = DUAL ? NB / 2 : NB;  // rows a full turn of the ring advances
    __shared__ float4 xl[STEPS * 64 * (UQ + 1)];
    __shared__ float sums[STEPS * 64 * NS];
    __shared__ float red[XREG_THREADS / 64];
    constexpr int nwaves = XREG_THREADS / 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: row numbers, row pointers and the loop run on the SALU
    const int k = a.k, n = a.n[0] + a.n[1] + a.n[2];
    const int units = k / U::UV;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int stride = nblocks * nwaves;
    const int row0 = bid * nwaves + wave;
    int uc[STEPS];
    uint32_t off[STEPS][U::NOFF];  // byte offsets of this lane's fields within a row: the same for every row
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        uc[s] = min(s * 64 + lane, units - 1);  // lanes past the row end: last unit, zeroed x
        U::offsets(uc[s], off[s]);
    }
    // segment and local row of global row r (scalar)
    auto locate = [&](int r, int &seg, int &local) {
        seg = (r >= a.n[0]) + (r >= a.n[0] + a.n[1]);
        local = r - (seg > 0 ? a.n[0] : 0) - (seg > 1 ? a.n[1] : 0);
    };
    // loads of a buffer for row r of matrix `second ? w2 : w[seg]`; a row past the end is "loaded" from the first bytes
    // of the matrix by every lane (one cache line, no traffic) so that the number of loads in flight never depends on
    // the data
    auto fill = [&](typename U::Raw(&dst)[STEPS], float &bdst, int r, bool second) {
        const bool live = r < n;
        int seg = 0, local = 0;
        if (live) locate(r, seg, local);
        const uint8_t *rp = (DUAL && second ? a.w2 : a.w[seg]) + (size_t)local * rowbytes;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            uint32_t o[U::NOFF];
#pragma unroll
            for (int i = 0; i < U::NOFF; ++i) o[i] = live ? off[s][i] : 0u;
            U::load(dst[s], rp, o);
        }
        if (BIAS) bdst = a.bias[seg][local];
    };

    // ---- activations first: their loads (L2 hits) are issued ahead of the weight loads because the hardware counts
    // returning loads in order - waiting for x must not mean waiting for the first weight rows from HBM
    constexpr int QUADS = STEPS * 64 * UQ, PER = QUADS / XREG_THREADS;
    static_assert(QUADS % XREG_THREADS == 0, "whole passes");
    float4 xv[PER], nv[PER];
    {
        const int kq = k >> 2;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = tid + i * XREG_THREADS;
            xv[i] = f < kq ? reinterpret_cast<const float4 *>(a.x)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
            if (NORM) nv[i] = f < kq ? reinterpret_cast<const float4 *>(a.nw)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    typename U::Raw buf[NB][STEPS];
    float bv[NB];  // the bias of each buffered row rides with its loads, so waiting for it never drains younger loads
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        bv[b] = 0.f;
        fill(buf[b], bv[b], row0 + (DUAL ? b / 2 : b) * stride, DUAL && (b & 1));
    }
    if (NORM) {  // x <- x * nw / sqrt(mean(x^2) + eps): every workgroup normalises the whole vector for itself
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) ss += (xv[i].x * xv[i].x + xv[i].y * xv[i].y) + (xv[i].z * xv[i].z + xv[i].w * xv[i].w);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        const float is = 1.f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)k + a.eps);
#pragma unroll
        for (int i = 0; i < PER; ++i)
            xv[i] = make_float4(xv[i].x * is * nv[i].x, xv[i].y * is * nv[i].y, xv[i].z * is * nv[i].z, xv[i].w * is * nv[i].w);
    }
    // ---- stage x (and the partial sums) in unit order
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int f = tid + i * XREG_THREADS;
        int u, g;
        U::slot(f, u, g);
        xl[u * (UQ + 1) + g] = xv[i];
        const float sm = group_sum<SG>((xv[i].x + xv[i].y) + (xv[i].z + xv[i].w));
        if ((f & (SG - 1)) == 0) sums[u * NS + g / SG] = sm;
    }
    __syncthreads();
    XReg<UQ, NS> xs[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
        for (int g = 0; g < UQ; ++g) xs[s].x[g] = xl[(s * 64 + lane) * (UQ + 1) + g];
#pragma unroll
        for (int i = 0; i < NS; ++i) xs[s].sm[i] = sums[(s * 64 + lane) * NS + i];
    }

    int left = a.rpw;  // 0: the priority stays where it is
    step_priority(left);
    float gate = 0.f;  // DUAL: the gate row's result, held until the up row of the same index is done
    for (int base = row0; base < n; base += RSTEP * stride) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int row = base + (DUAL ? b / 2 : b) * stride;
            if (row < n) {  // wave-uniform
                float acc[1][1] = {{0.f}};
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    const typename U::Raw(&w1)[1] = reinterpret_cast<const typename U::Raw(&)[1]>(buf[b][s]);
                    U::template dot<1, 1, CV>(w1, uc[s], xs[s], acc, a.nib);
                }
                const float t = wave_sum(acc[0][0]);
                if (!DUAL || (b & 1)) step_priority(--left);
                if (DUAL) {
                    if ((b & 1) == 0) gate = t;
                    else if (lane == 0) a.y[0][row] = (gate / (1.f + __expf(-gate))) * t;
                } else {
                    int seg, local;
                    locate(row, seg, local);
                    if (lane == 0) a.y[seg][local] = BIAS ? t + bv[b] : t;
                }
            }
            fill(buf[b], bv[b], row + RSTEP * stride, DUAL && (b & 1));
        }
    }
}

template <class U, int CV, int PF, bool BIAS, bool NORM, bool DUAL>
__global__ void __launch_bounds__(XREG_THREADS) gemv_xreg_kernel(const XregArgs a) {
    gemv_xreg_body<U, CV, PF, BIAS, NORM, DUAL>(a, blockIdx.x, gridDim.x);
}

// Two sets of matrices in two formats over the same activations in one launch (the q / k and the v projections of a
// Q4_K_M layer): workgroups below `split` run the first set, the others the second, each exactly as its own launch
// would.  Always with the RMSNorm fused, never with bias or SwiGLU: that is the one place a decode step needs it.
template <class UA, int CVA, class UB, int CVB, int PF>
__global__ void __launch_bounds__(XREG_THREADS) gemv_xreg2_kernel(const XregArgs a, const XregArgs b, const int split) {
    if ((int)blockIdx.x < split) gemv_xreg_body<UA, CVA, PF, false, true, false>(a, blockIdx.x, split);
    else gemv_xreg_body<UB, CVB, PF, false, true, false>(b, blockIdx.x - split, gridDim.x - split);
}

// Batch 2, rows of at most 4096 values: gemv_xreg_kernel's scheme with the activations of both rows in registers.
// Every decoded weight meets two activations, so the kernel stays close to the batch-1 time where the FP32 kernel
// with activations in LDS and the matrix-core kernel (built for up to eight rows) both take half as long again.
//   x [2, k], y [2, n]; bias (BIAS) is added to both rows.
template <class U, int CV, int PF, bool BIAS>
__global__ void __launch_bounds__(XREG_THREADS) gemv_xreg_b2_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                                    const float *__restrict__ bias, float *__restrict__ y, int n, int k, float nib) {
    constexpr int FMT = U::FMT, STEPS = 64 / U::UV;
    constexpr int UQ = U::UV / 4, NS = U::NS, SG = U::SG, NB = PF + 1;
    __shared__ float4 xl[2][STEPS * 64 * (UQ + 1)];
    __shared__ float sums[2][STEPS * 64 * NS];
    constexpr int nwaves = XREG_THREADS / 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int units = k / U::UV;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int stride = gridDim.x * nwaves;
    const int row0 = blockIdx.x * nwaves + wave;
    int uc[STEPS];
    uint32_t off[STEPS][U::NOFF];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        uc[s] = min(s * 64 + lane, units - 1);  // lanes past the row end: last unit, zeroed x
        U::offsets(uc[s], off[s]);
    }
    auto fill = [&](typename U::Raw(&dst)[STEPS], float &bdst, int r) {
        const bool live = r < n;  // a row past the end is "loaded" from the first bytes of the matrix: one cache line
        const uint8_t *rp = W + (live ? (size_t)r * rowbytes : 0);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            uint32_t o[U::NOFF];
#pragma unroll
            for (int i = 0; i < U::NOFF; ++i) o[i] = live ? off[s][i] : 0u;
            U::load(dst[s], rp, o);
        }
        if (BIAS) bdst = bias[live ? r : 0];
    };
    // ---- activations first (their loads must not queue behind the first weight rows), then the ring's first rows
    constexpr int QUADS = STEPS * 64 * UQ, PER = QUADS / XREG_THREADS;
    static_assert(QUADS % XREG_THREADS == 0, "whole passes");
    float4 xv[2][PER];
    {
        const int kq = k >> 2;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int f = tid + i * XREG_THREADS;
                xv[b][i] = f < kq ? reinterpret_cast<const float4 *>(x + (size_t)b * k)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
    }
    typename U::Raw buf[NB][STEPS];
    float bv[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        bv[b] = 0.f;
        fill(buf[b], bv[b], row0 + b * stride);
    }
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = tid + i * XREG_THREADS;
            int u, g;
            U::slot(f, u, g);
            xl[b][u * (UQ + 1) + g] = xv[b][i];
            const float sm = group_sum<SG>((xv[b][i].x + xv[b][i].y) + (xv[b][i].z + xv[b][i].w));
            if ((f & (SG - 1)) == 0) sums[b][u * NS + g / SG] = sm;
        }
    __syncthreads();
    XReg2<UQ, NS> xs[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int g = 0; g < UQ; ++g) xs[s].x[b][g] = xl[b][(s * 64 + lane) * (UQ + 1) + g];
#pragma unroll
            for (int i = 0; i < NS; ++i) xs[s].sm[b][i] = sums[b][(s * 64 + lane) * NS + i];
        }

    int left = row0 < n ? (n - row0 + stride - 1) / stride : 0;  // rows of this wave
    step_priority(left);
    for (int base = row0; base < n; base += NB * stride) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int row = base + b * stride;
            if (row < n) {  // wave-uniform
                float acc[1][2] = {{0.f, 0.f}};
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    const typename U::Raw(&w1)[1] = reinterpret_cast<const typename U::Raw(&)[1]>(buf[b][s]);
                    U::template dot<2, 1, CV>(w1, uc[s], xs[s], acc, nib);
                }
                const float t0 = wave_sum(acc[0][0]), t1 = wave_sum(acc[0][1]);
                step_priority(--left);
                if (lane == 0) {
                    y[row] = BIAS ? t0 + bv[b] : t0;
                    y[(size_t)n + row] = BIAS ? t1 + bv[b] : t1;
                }
            }
            fill(buf[b], bv[b], row + NB * stride);
        }
    }
}

// Batch-1 GEMV for rows longer than 4096 values: the row is cut into slices of 4096 values, one per wave of
// the workgroup (a 14336-value row takes four waves, the last one half full), and each wave keeps the
// activations of its slice in registers exactly as gemv_xreg_kernel does.  All waves of a workgroup walk the
// same rows (blockIdx.x, + gridDim.x, ...) with the same prefetch ring; each leaves its partial sum of a row in
// LDS, and every KS_FLUSH rows (and at the end) the workgroup meets at a barrier where one thread per row adds
// the slices in slice order and writes y: a fixed summation order, no atomics.
//   launch: blockDim.x = 64 * slices, dynamic LDS = gemv_ksplit_lds_bytes<FMT>(slices).
constexpr int KS_FLUSH = 32;

template <class U>
__host__ __device__ constexpr size_t gemv_ksplit_lds_bytes(int slices) {
    constexpr int STEPS = 64 / U::UV;
    return (size_t)slices * STEPS * 64 * ((U::UV / 4 + 1) * 16 + U::NS * 4);
}

template <class U, int CV, int PF>
__global__ void __launch_bounds__(512) gemv_ksplit_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                            const float *__restrict__ bias, float *__restrict__ y, int n, int k, float nib) {
    constexpr int FMT = U::FMT, STEPS = 64 / U::UV;
    constexpr int UQ = U::UV / 4, NS = U::NS, SG = U::SG, NB = PF + 1;
    extern __shared__ float4 smem[];
    __shared__ float part[KS_FLUSH][8];  // at most 8 slices: rows of up to 32768 values
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slices = blockDim.x >> 6;
    float4 *xl = smem + (size_t)wave * STEPS * 64 * (UQ + 1);
    float *sums = reinterpret_cast<float *>(smem + (size_t)slices * STEPS * 64 * (UQ + 1)) + (size_t)wave * STEPS * 64 * NS;
    const int units = k / U::UV;
    const int ubase = wave * STEPS * 64;  // first unit of this wave's slice
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int stride = gridDim.x;
    const int row0 = blockIdx.x;
    int uc[STEPS];
    uint32_t off[STEPS][U::NOFF];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        uc[s] = min(ubase + s * 64 + lane, units - 1);  // lanes past the row end: last unit, zeroed x
        U::offsets(uc[s], off[s]);
    }
    auto fill = [&](typename U::Raw(&dst)[STEPS], int r) {
        const bool live = r < n;
        const uint8_t *rp = W + (live ? (size_t)r * rowbytes : 0);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            uint32_t o[U::NOFF];
#pragma unroll
            for (int i = 0; i < U::NOFF; ++i) o[i] = live ? off[s][i] : 0u;
            U::load(dst[s], rp, o);
        }
    };

    // ---- each wave stages its own slice of x: 16 quads per lane, issued ahead of the weight loads
    constexpr int PER = STEPS * UQ;  // quads per lane
    float4 xv[PER];
    {
        const int kq = k >> 2, fbase = ubase * UQ;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = fbase + i * 64 + lane;
            xv[i] = f < kq ? reinterpret_cast<const float4 *>(x)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    typename U::Raw buf[NB][STEPS];
#pragma unroll
    for (int b = 0; b < NB; ++b) fill(buf[b], row0 + b * stride);
    {
        const int fbase = ubase * UQ;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int f = fbase + i * 64 + lane;
            int u, g;
            U::slot(f, u, g);
            u -= ubase;
            xl[u * (UQ + 1) + g] = xv[i];
            const float sm = group_sum<SG>((xv[i].x + xv[i].y) + (xv[i].z + xv[i].w));
            if ((f & (SG - 1)) == 0) sums[u * NS + g / SG] = sm;
        }
    }
    __syncthreads();
    XReg<UQ, NS> xs[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
        for (int g = 0; g < UQ; ++g) xs[s].x[g] = xl[(s * 64 + lane) * (UQ + 1) + g];
#pragma unroll
        for (int i = 0; i < NS; ++i) xs[s].sm[i] = sums[(s * 64 + lane) * NS + i];
    }

    int done = 0;       // rows of this workgroup finished so far
    int flushed = 0;    // ... of which already written to y
    auto flush = [&]() {
        __syncthreads();
        const int cnt = done - flushed;
        if (tid < cnt) {
            const int row = row0 + (flushed + tid) * stride;
            float t = 0.f;
            for (int w = 0; w < slices; ++w) t += part[tid][w];
            y[row] = bias ? t + bias[row] : t;
        }
        __syncthreads();
        flushed = done;
    };
    for (int base = row0; base < n; base += NB * stride) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int row = base + b * stride;
            if (row < n) {  // workgroup-uniform
                float acc[1][1] = {{0.f}};
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    const typename U::Raw(&w1)[1] = reinterpret_cast<const typename U::Raw(&)[1]>(buf[b][s]);
                    U::template dot<1, 1, CV>(w1, uc[s], xs[s], acc, nib);
                }
                float t = wave_sum(acc[0][0]);
                if (lane == 0) part[done - flushed][wave] = t;
                ++done;
                if (done - flushed == KS_FLUSH) flush();
            }
            fill(buf[b], row + NB * stride);
        }
    }
    if (done > flushed) flush();
}

// LDS bytes one staged K-chunk of `itc` wave steps takes for batch B.
template <class U>
__host__ __device__ constexpr size_t gemv_lds_bytes(int B, int itc) {
    return (size_t)B * itc * 64 * ((U::UV / 4 + 1) * 16 + U::NS * 4);
}

// Batch 2..8 GEMV (and any batch-1 shape the register-resident kernels do not take):
// y[b, row] = sum_k W[row, k] x[b, k] (+ bias[row]) for b < rows <= B.
//   The activations of all batch rows are staged in LDS in unit order; a wave decodes the units of R weight rows
//   once per step and uses them for every batch row, reading the activations from LDS.  Work items (row group,
//   step) run through a ring of NBUF register buffers: with two, the next item's weights are in flight while one is
//   decoded; the big-batch variants keep one buffer (their accumulators need the registers) and rely on the other
//   resident waves to cover the latency.
//   grid: any number of workgroups of a multiple of 64 threads; waves take row groups of R rows round-robin.
//   itc : wave steps (64 units each) staged in LDS at a time; K beyond that is processed in further chunks,
//         each wave adding its partial sums to y (same wave, same order: deterministic).
template <class U, int B, int R, int CV, int NBUF>
__global__ void __launch_bounds__(512) gemv_lds_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                        const float *__restrict__ bias, float *__restrict__ y, int n, int k, int rows,
                                                        int itc, float nib) {
    constexpr int FMT = U::FMT, UQ = U::UV / 4, NS = U::NS, SG = U::SG;
    extern __shared__ float4 smem[];
    const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x, nwaves = nthreads >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int units = k / U::UV;
    const int steps = (units + 63) >> 6;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const int ngroups = (n + R - 1) / R;
    const int bs = itc * 64 * (UQ + 1);  // float4 stride between batch rows
    const int ss = itc * 64 * NS;        // float stride between batch rows of the partial sums
    float4 *xl = smem;
    float *sums = reinterpret_cast<float *>(xl + (size_t)B * bs);
    const int kq = k >> 2;  // quads per activation row
    const int first = blockIdx.x * nwaves + wave, gstride = gridDim.x * nwaves;

    for (int c0 = 0; c0 < steps; c0 += itc) {
        const int nit = min(itc, steps - c0);
        if (c0 > 0) __syncthreads();
        // ---- stage x[:, chunk] in unit order with the partial sums of each group of SG quads; eight loads per thread
        // are issued before the first LDS write so that their latencies overlap
        const int f0 = c0 * 64 * UQ, nq = nit * 64 * UQ;  // quads of the chunk per batch row (may run past kq: zero fill)
        for (int base = 0; base < B * nq; base += nthreads * 8) {
            float4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int idx = base + j * nthreads + tid;
                const int b = idx / nq, f = f0 + idx - b * nq;
                v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < B * nq && f < kq && b < rows) v[j] = reinterpret_cast<const float4 *>(x + (size_t)b * k)[f];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int idx = base + j * nthreads + tid;
                if (idx < B * nq) {  // whole waves: nq and nthreads are multiples of 64
                    const int b = idx / nq, f = f0 + idx - b * nq;
                    int u, g;
                    U::slot(f, u, g);
                    u -= c0 * 64;
                    xl[(size_t)b * bs + (size_t)u * (UQ + 1) + g] = v[j];
                    const float sm = group_sum<SG>((v[j].x + v[j].y) + (v[j].z + v[j].w));
                    if ((f & (SG - 1)) == 0) sums[(size_t)b * ss + u * NS + g / SG] = sm;
                }
            }
        }
        __syncthreads();
        // ---- work items (row group, step) through the ring
        typename U::Raw buf[NBUF][R];
        auto fill = [&](typename U::Raw(&dst)[R], int rg, int it) {
            const bool live = rg < ngroups;  // a dead item is "loaded" from the first bytes of the matrix: one cache line
            uint32_t off[U::NOFF];
            U::offsets(min((c0 + it) * 64 + lane, units - 1), off);
#pragma unroll
            for (int i = 0; i < U::NOFF; ++i) off[i] = live ? off[i] : 0u;
#pragma unroll
            for (int r = 0; r < R; ++r) U::load(dst[r], W + (live ? (size_t)min(rg * R + r, n - 1) * rowbytes : 0), off);
        };
        int rg_l = first, it_l = 0;  // next item to load
        int rg_c = first, it_c = 0;  // next item to decode
#pragma unroll
        for (int sl = 0; sl < NBUF; ++sl) {
            fill(buf[sl], rg_l, it_l);
            if (++it_l == nit) { it_l = 0; rg_l += gstride; }
        }
        float acc[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[r][b] = 0.f;
        while (rg_c < ngroups) {
#pragma unroll
            for (int sl = 0; sl < NBUF; ++sl) {
                if (rg_c < ngroups) {  // wave-uniform
                    const int uc = min((c0 + it_c) * 64 + lane, units - 1);  // lanes past the row end: last unit, zeroed x
                    const XLds xs{xl + (size_t)(it_c * 64 + lane) * (UQ + 1), sums + (it_c * 64 + lane) * NS, bs, ss};
                    U::template dot<B, R, CV>(buf[sl], uc, xs, acc, nib);
                    if (it_c == nit - 1) {
#pragma unroll
                        for (int r = 0; r < R; ++r) {
#pragma unroll
                            for (int b = 0; b < B; ++b) {
                                const float t = wave_sum(acc[r][b]);
                                acc[r][b] = 0.f;
                                const int row = rg_c * R + r;
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
                if (++it_c == nit) { it_c = 0; rg_c += gstride; }
                fill(buf[sl], rg_l, it_l);
                if (++it_l == nit) { it_l = 0; rg_l += gstride; }
            }
        }
    }
}

}  // namespace jitnn
