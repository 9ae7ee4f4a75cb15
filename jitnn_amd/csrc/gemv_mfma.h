// Batch 2..8 GEMV on raw GGUF blocks with the dot products on the matrix cores, at FP32-grade accuracy.
//
// With several activation rows the FP32 VALU path pays one multiply-add and one activation read per weight and
// per row; at eight rows that, not HBM, is the bound.  Here the weights of a tile meet all rows in one
// v_mfma_f32_16x16x32_f16:
//   * B operand: the quants of 16 weight rows x 32 values as FP16 integers - exact, they have at most 8 bits;
//   * A operand: 16 rows made of the (up to) 8 activation rows split in two FP16 parts, x * 2^e = hi + lo, rows
//     0..7 = hi, rows 8..15 = lo.  hi + lo carries 22 significant bits of x, the products with small integers are
//     exact in the FP32 accumulator, so the block sums are as good as FP32 arithmetic;
//   * the block scales (and the Q4_K / Q5_K / Q4_1 offsets) are applied in FP32 to the 4 x 16 block sums a wave
//     holds, never to individual weights.
// A workgroup of 8 waves (two per SIMD, 256 VGPRs each) owns groups of 16 weight rows and walks K in passes of
// 4096 values; wave w owns columns w and w + 8 of a pass (a column = 256 values: one K-quant super-block, eight
// 32-value blocks), so a tile is 16 weight rows x one column.
//   * Weights: the bytes of a tile are 16 contiguous runs (144 bytes each for Q4_K).  The wave copies them with
//     full 128-bit loads - consecutive lanes on consecutive 16-byte chunks of a run - through a two-deep ring of
//     registers into its own LDS region, and each lane then picks the bytes of its row in operand order from there.
//     No workgroup barrier is involved: the region belongs to the wave.
//   * Activations: a wave builds the A operands of its columns once per pass - one coalesced read of the 8 x 256
//     values, scale 2^e from the column's largest magnitude per row, FP16 split, transposition into operand order
//     through the same LDS region - and keeps them in 72 VGPRs for all row groups.  The loads of x go out before the
//     first weight loads (loads return in order) and the build runs while HBM works on the weights.
//   * A wave keeps the partial sums of up to four row groups; then the sums of the eight waves meet in LDS and are
//     added in wave order: a fixed summation order, no atomics.  Passes after the first add to y.
// The kernel is bound by the VALU work of turning quants into FP16 (about 170 instructions per tile) and of the
// operand build, not by HBM: it runs near 2.3 TB/s at every batch size from 2 to 8.
//
// Lane roles inside a wave: n = lane & 15 is the weight row of the group (B column, C column) and the A row it
// supplies; kq = lane >> 4 selects the eight K positions of a 32-value block the lane supplies to both operands.
// Which eight positions, and in which order, depends on how the format packs its quants (MTile<FMT>::quad_pos and
// the byte order 0, 2, 1, 3 of the dword decoders); a dot product only needs both operands to agree.
#pragma once
#include "common.h"

namespace jitnn {

constexpr int MF_WAVES = 8, MF_COLS = 2, MF_THREADS = MF_WAVES * 64;  // a workgroup covers MF_WAVES * MF_COLS = 16 columns = 4096 values of K per pass

typedef __fp16 h2raw __attribute__((ext_vector_type(2)));  // what v_cvt_pkrtz_f16_f32 returns

union H2 {
    uint32_t u;
    f16x2 h;
};
__device__ __forceinline__ f16x2 as_h2(uint32_t u) {
    H2 v;
    v.u = u;
    return v.h;
}
__device__ __forceinline__ f16x8 cat8(f16x2 a, f16x2 b, f16x2 c, f16x2 d) { return f16x8{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y}; }
__device__ __forceinline__ f16x2 splat2(float v) { return f16x2{(_Float16)v, (_Float16)v}; }

// 0x64006400: FP16 1024.0 twice.  Or-ing an integer below 1024 into the mantissa gives 1024 + it.  The constant is
// handed out through an empty asm so that it lives in a VGPR: only then can (w & mask) | magic be one v_and_or_b32
// (the instruction takes a single scalar or literal operand, and the mask is one already).
__device__ __forceinline__ uint32_t magic1024() {
    uint32_t m = 0x64006400u;
    asm("" : "+v"(m));
    return m;
}
// (1024 + q) pairs -> q - off, and (1024 + 16 q) pairs -> q - off, exact in FP16
__device__ __forceinline__ f16x2 magic_lo(uint32_t bits, float off) { return as_h2(bits) - splat2(1024.f + off); }
__device__ __forceinline__ f16x2 magic_hi(uint32_t bits, float off) {
    return __builtin_elementwise_fma(as_h2(bits), splat2(0.0625f), splat2(-64.f - off));
}
// dword of four 4-bit pairs -> low nibbles of bytes (0,2), (1,3) and high nibbles of bytes (0,2), (1,3), minus off
__device__ __forceinline__ void nibbles(uint32_t w, float off, f16x2 &l02, f16x2 &l13, f16x2 &h02, f16x2 &h13) {
    const uint32_t s = w >> 8, mg = magic1024();
    l02 = magic_lo((w & 0x000f000fu) | mg, off);
    l13 = magic_lo((s & 0x000f000fu) | mg, off);
    h02 = magic_hi((w & 0x00f000f0u) | mg, off);
    h13 = magic_hi((s & 0x00f000f0u) | mg, off);
}
// two bytes (lo, hi of a 16-bit field at `shift`) -> FP16 pair of their unsigned values
__device__ __forceinline__ f16x2 bytes2(uint32_t w, int shift) {
    const uint32_t v = w >> shift;
    return as_h2((v & 0xffu) | ((v << 8) & 0x00ff0000u) | 0x64006400u) - splat2(1024.f);
}

__device__ __forceinline__ f32x4 mfma16(const f16x8 a, const f16x8 b) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
}

// LDS reads of the staged weight bytes (p points into LDS; 16-bit pieces where a field is only 2-byte aligned)
__device__ __forceinline__ uint32_t sld16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }
__device__ __forceinline__ uint32_t sld32(const uint8_t *p) { return *reinterpret_cast<const uint32_t *>(p); }
__device__ __forceinline__ uint32_t sld32_a2(const uint8_t *p) { return sld16(p) | (sld16(p + 2) << 16); }
__device__ __forceinline__ u32x2 sld64(const uint8_t *p) { return *reinterpret_cast<const u32x2 *>(p); }
__device__ __forceinline__ u32x4 sld128(const uint8_t *p) { return *reinterpret_cast<const u32x4 *>(p); }

// A tile = 16 weight rows x 256 values.  Per format: the bytes of a tile row (BYTES, a multiple of 16), which lane
// group kq and which half h of its eight K slots the quad tq (values 4 tq .. 4 tq + 3 of a 32-value block) goes to
// (quad_pos), whether the per-block sums of x are needed (SUMS), and the tile product from the staged bytes p of
// this lane's weight row: acc[i] = sum over the tile of W[row n][k] * xt[A row 4 kq + i][k].
template <int FMT>
struct MTile;

// formats whose lane takes eight consecutive bytes of a 32-byte run: values 8 kq .. 8 kq + 7
__device__ __forceinline__ void quad_pos_bytes8(int tq, int &kq, int &h) {
    kq = tq >> 1;
    h = tq & 1;
}
// formats whose lane takes one dword of a 16-byte run of nibble pairs: values 4 kq .. and 16 + 4 kq ..
__device__ __forceinline__ void quad_pos_nib4(int tq, int &kq, int &h) {
    kq = tq & 3;
    h = tq >> 2;
}

struct K4Scales {
    float sc[8];
    uint32_t mnA, mnB;
    float d, dmin;
};
// the 6-bit scales and mins of a Q4_K / Q5_K super-block, bytewise (GgufKernels scaleMin: the first four in the low
// six bits of bytes 0..7, the last four split between the nibbles of bytes 8..11 and the top bits of bytes 0..7)
__device__ __forceinline__ K4Scales k4_scales(const u32x4 h) {
    K4Scales r;
    r.d = h2f(h.x);
    r.dmin = h2f(h.x >> 16);
    const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;
    const uint32_t scA = s0 & 0x3f3f3f3fu, scB = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    r.mnA = s1 & 0x3f3f3f3fu;
    r.mnB = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
    r.sc[0] = ub0(scA); r.sc[1] = ub1(scA); r.sc[2] = ub2(scA); r.sc[3] = ub3(scA);
    r.sc[4] = ub0(scB); r.sc[5] = ub1(scB); r.sc[6] = ub2(scB); r.sc[7] = ub3(scB);
    return r;
}
// offsets of a Q4_K / Q5_K tile: sum_j min_j * (sum of x over block j), the block sums arriving as A operand scaled by 1/64
__device__ __forceinline__ void k4_mins(const K4Scales &k, const f16x8 &xs, f32x4 &acc) {
    const f32x4 cm = mfma16(xs, cat8(bytes2(k.mnA, 0), bytes2(k.mnA, 16), bytes2(k.mnB, 0), bytes2(k.mnB, 16)));
    const float dm = k.dmin * 64.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(-dm, cm[i], acc[i]);
}

template <>
struct MTile<F_Q4_K> {
    static constexpr bool SUMS = true;
    static constexpr int BYTES = 144;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_bytes8(tq, kq, h); }
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &xs) {
        const K4Scales k = k4_scales(sld128(p));
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const u32x2 q = sld64(p + 16 + 32 * c + 8 * kq);
            f16x2 l0, l1, l2, l3, h0, h1, h2, h3;
            nibbles(q.x, 0.f, l0, l1, h0, h1);
            nibbles(q.y, 0.f, l2, l3, h2, h3);
            const f32x4 cl = mfma16(xa[2 * c], cat8(l0, l1, l2, l3));
            const f32x4 ch = mfma16(xa[2 * c + 1], cat8(h0, h1, h2, h3));
            const float dl = k.d * k.sc[2 * c], dh = k.d * k.sc[2 * c + 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(dh, ch[i], __builtin_fmaf(dl, cl[i], acc[i]));
        }
        k4_mins(k, xs, acc);
        return acc;
    }
};

template <>
struct MTile<F_Q5_K> {
    static constexpr bool SUMS = true;
    static constexpr int BYTES = 176;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_bytes8(tq, kq, h); }
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &xs) {
        const K4Scales k = k4_scales(sld128(p));
        const u32x2 qh2 = sld64(p + 16 + 8 * kq);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const u32x2 q = sld64(p + 48 + 32 * c + 8 * kq);
            f16x2 l[4], h[4];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t w = t ? q.y : q.x, qh = t ? qh2.y : qh2.x, s = w >> 8, qs = qh >> 8, mg = magic1024();
                // fifth bit of block 2c (2c + 1): bit 2c (2c + 1) of the qh byte at the same position
                l[2 * t] = magic_lo((w & 0x000f000fu) | (((qh >> (2 * c)) & 0x00010001u) << 4) | mg, 0.f);
                l[2 * t + 1] = magic_lo((s & 0x000f000fu) | (((qs >> (2 * c)) & 0x00010001u) << 4) | mg, 0.f);
                // high nibbles sit at 16 q: the fifth bit goes to bit 8 and the scale 1/16 brings both down
                h[2 * t] = magic_hi((w & 0x00f000f0u) | (((qh >> (2 * c + 1)) & 0x00010001u) << 8) | mg, 0.f);
                h[2 * t + 1] = magic_hi((s & 0x00f000f0u) | (((qs >> (2 * c + 1)) & 0x00010001u) << 8) | mg, 0.f);
            }
            const f32x4 cl = mfma16(xa[2 * c], cat8(l[0], l[1], l[2], l[3]));
            const f32x4 ch = mfma16(xa[2 * c + 1], cat8(h[0], h[1], h[2], h[3]));
            const float dl = k.d * k.sc[2 * c], dh = k.d * k.sc[2 * c + 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(dh, ch[i], __builtin_fmaf(dl, cl[i], acc[i]));
        }
        k4_mins(k, xs, acc);
        return acc;
    }
};

// Q4_0: eight 18-byte blocks per tile row; the dword a lane takes from a block holds values 4 kq .. 4 kq + 3 (low
// nibbles) and 16 + 4 kq .. (high nibbles)
template <>
struct MTile<F_Q4_0> {
    static constexpr bool SUMS = false;
    static constexpr int BYTES = 8 * 18;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_nib4(tq, kq, h); }
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float d = h2f(sld16(p + 18 * j));
            const uint32_t q = sld32_a2(p + 18 * j + 2 + 4 * kq);
            f16x2 l0, l1, h0, h1;
            nibbles(q, 8.f, l0, l1, h0, h1);
            const f32x4 c = mfma16(xa[j], cat8(l0, l1, h0, h1));
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(d, c[i], acc[i]);
        }
        return acc;
    }
};

// Q4_1: 20-byte blocks, w = d q + m; the offsets m_j are FP16 already and meet the block sums of x in one MFMA
template <>
struct MTile<F_Q4_1> {
    static constexpr bool SUMS = true;
    static constexpr int BYTES = 8 * 20;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_nib4(tq, kq, h); }
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &xs) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        f16x8 bm;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t dm = sld32(p + 20 * j);
            const uint32_t q = sld32(p + 20 * j + 4 + 4 * kq);
            f16x2 l0, l1, h0, h1;
            nibbles(q, 0.f, l0, l1, h0, h1);
            const f32x4 c = mfma16(xa[j], cat8(l0, l1, h0, h1));
            const float d = h2f(dm);
            bm[j] = as_h2(dm).y;
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(d, c[i], acc[i]);
        }
        const f32x4 cm = mfma16(xs, bm);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(64.f, cm[i], acc[i]);
        return acc;
    }
};

// Q8_0: 34-byte blocks of signed bytes; a lane takes bytes 8 kq .. 8 kq + 7 of each
template <>
struct MTile<F_Q8_0> {
    static constexpr bool SUMS = false;
    static constexpr int BYTES = 8 * 34;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_bytes8(tq, kq, h); }
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float d = h2f(sld16(p + 34 * j));
            // signed byte b -> (b + 128) unsigned -> 1024 + b + 128 -> b
            const uint32_t w0 = sld32_a2(p + 34 * j + 2 + 8 * kq) ^ 0x80808080u, w1 = sld32_a2(p + 34 * j + 6 + 8 * kq) ^ 0x80808080u;
            const uint32_t mg = magic1024();
            const f16x2 a0 = magic_lo((w0 & 0x00ff00ffu) | mg, 128.f), a1 = magic_lo(((w0 >> 8) & 0x00ff00ffu) | mg, 128.f);
            const f16x2 a2 = magic_lo((w1 & 0x00ff00ffu) | mg, 128.f), a3 = magic_lo(((w1 >> 8) & 0x00ff00ffu) | mg, 128.f);
            const f32x4 c = mfma16(xa[j], cat8(a0, a1, a2, a3));
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(d, c[i], acc[i]);
        }
        return acc;
    }
};

// Q6_K: 210-byte super-blocks (ql[128], qh[64], sixteen int8 scales, d); a scale covers 16 values, so the block sums
// come from v_mfma_f32_16x16x16_f16, two per 32-value block.  Block b = 4 nh + qt holds values l = 0..31 with low
// nibbles / high nibbles (qt >> 1) of ql[64 nh + 32 (qt & 1) + l] and bits 2 qt, 2 qt + 1 of qh[32 nh + l]
// (GgufKernels.java: Q6_K decode).  The run is copied as 13 chunks of 16 bytes plus the two bytes of d.
template <>
struct MTile<F_Q6_K> {
    static constexpr bool SUMS = false;
    static constexpr int BYTES = 210;
    __device__ static __forceinline__ void quad_pos(int tq, int &kq, int &h) { quad_pos_nib4(tq, kq, h); }  // half h = 16-value group
    __device__ static __forceinline__ f32x4 mma(const uint8_t *p, int kq, const f16x8 (&xa)[8], const f16x8 &) {
        const float d = h2f(sld16(p + 208));
        const u32x4 scw = sld128(p + 192);
        const uint32_t mg = magic1024();
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nh = 0; nh < 2; ++nh) {
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const uint32_t qh = sld32(p + 128 + 32 * nh + 16 * g + 4 * kq);
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) {
                    const uint32_t ql = sld32(p + 64 * nh + 32 * hb + 16 * g + 4 * kq);
#pragma unroll
                    for (int nib = 0; nib < 2; ++nib) {
                        const int qt = 2 * nib + hb, b = 4 * nh + qt;
                        const uint32_t q = ((ql >> (4 * nib)) & 0x0f0f0f0fu) | (((qh >> (2 * qt)) & 0x03030303u) << 4);  // four 6-bit quants
                        const f16x2 a02 = magic_lo((q & 0x00ff00ffu) | mg, 32.f), a13 = magic_lo(((q >> 8) & 0x00ff00ffu) | mg, 32.f);
                        const f16x4 bop = {a02.x, a02.y, a13.x, a13.y};
                        const f16x4 aop = g ? f16x4{xa[b][4], xa[b][5], xa[b][6], xa[b][7]} : f16x4{xa[b][0], xa[b][1], xa[b][2], xa[b][3]};
                        const f32x4 c = __builtin_amdgcn_mfma_f32_16x16x16f16(aop, bop, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        const int si = 8 * nh + 2 * qt + g;  // scale of values 16 g .. 16 g + 15 of block b
                        const float ds = d * (float)(int)(int8_t)((scw[si >> 2] >> (8 * (si & 3))) & 0xffu);
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(ds, c[i], acc[i]);
                    }
                }
            }
        }
        return acc;
    }
};

// Pitch of a tile row in a wave's LDS region: at least BYTES and an odd multiple of 16, so that the 16 rows of an
// operand read (two dwords per lane, 64 banks) start four banks apart and never collide.
template <int FMT>
__host__ __device__ constexpr int mf_row_pitch() {
    int p = (MTile<FMT>::BYTES + 15) / 16 * 16;
    return (p / 16) % 2 ? p : p + 16;
}
constexpr int MF_GROUPS = 4;            // row groups whose partial sums a wave keeps before the workgroup adds them
constexpr int MF_XBUILD = 4096 + 256;   // a region while a wave builds A operands in it: four 1 KiB operands + the block sums'
template <int FMT>
__host__ __device__ constexpr int mf_region_bytes() {  // one tile of weights, or the operand build
    return 16 * mf_row_pitch<FMT>() > MF_XBUILD ? 16 * mf_row_pitch<FMT>() : MF_XBUILD;
}
template <int FMT>
__host__ __device__ constexpr size_t gemv_mfma_lds_bytes() {
    return (size_t)MF_WAVES * MF_COLS * mf_region_bytes<FMT>() + (size_t)MF_WAVES * MF_GROUPS * 32 * 16;
}

// Orders this wave's LDS traffic where its lanes hand data to each other through the wave's own LDS region.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// max over aligned groups of 8 neighbouring lanes (DPP, same tree as group_sum<8>)
__device__ __forceinline__ float group_max8(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0xB1, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x4E, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x141, 0xF, 0xF, false)));
    return v;
}

// The A operands of one 256-value column from the quads v[t] = x[b, column + 32 t + 4 part .. + 3] a lane (row b = lane >> 3,
// part = lane & 7) holds: scale by 2^e -> hi / lo FP16 parts -> operand order through the LDS region `reg`.
template <class T>
__device__ __forceinline__ void mf_build_operands(const float4 (&v)[8], bool have, uint8_t *reg, int lane, f16x8 (&xa)[8], f16x8 &xs,
                                                  float (&inv)[4]) {
    const int b = lane >> 3, part = lane & 7, nq = lane & 15, kq = lane >> 4;
    float amax = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[t].x), fabsf(v[t].y)), fmaxf(fabsf(v[t].z), fabsf(v[t].w))));
    amax = group_max8(amax);
    float scale = 1.f;
    if (amax > 0.f && amax < 3.0e38f) {
        int e;
        frexpf(amax, &e);             // amax = f * 2^e, f in [0.5, 1)
        scale = ldexpf(1.f, 14 - e);  // largest scaled magnitude in [2^13, 2^14)
    }
    const float myinv = 1.f / scale;
#pragma unroll
    for (int i = 0; i < 4; ++i) inv[i] = __shfl(myinv, ((4 * kq + i) & 7) * 8);  // C rows 4 kq + i belong to activation row (4 kq + i) & 7
    if (!have) scale = 0.f;
    int pk, ph;
    T::quad_pos(part, pk, ph);
    float sm = 0.f;  // sum of block `part` of row b
    xs = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    // operand order: block, A row m (b: hi, b + 8: lo), lane group pk, half ph of the lane's eight slots; four blocks at a time
#pragma unroll
    for (int t0 = 0; t0 < 8; t0 += 4) {
#pragma unroll
        for (int t = t0; t < t0 + 4; ++t) {
            // byte order 0, 2, 1, 3 of the decoders; hi = x 2^e cut to FP16 (towards zero), lo = the exact rest
            const float a0 = v[t].x * scale, a1 = v[t].z * scale, a2 = v[t].y * scale, a3 = v[t].w * scale;
            if constexpr (T::SUMS) {
                const float bs = group_sum<8>((a0 + a1) + (a2 + a3));  // block t of row b: its eight quads sit in the eight lanes of b
                sm = part == t ? bs : sm;
            }
            const h2raw h01 = __builtin_amdgcn_cvt_pkrtz(a0, a1), h23 = __builtin_amdgcn_cvt_pkrtz(a2, a3);
            const h2raw l01 = __builtin_amdgcn_cvt_pkrtz(a0 - (float)h01.x, a1 - (float)h01.y);
            const h2raw l23 = __builtin_amdgcn_cvt_pkrtz(a2 - (float)h23.x, a3 - (float)h23.y);
            *reinterpret_cast<u32x2 *>(reg + (t & 3) * 1024 + (b + 16 * pk) * 16 + 8 * ph) =
                u32x2{__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23)};
            *reinterpret_cast<u32x2 *>(reg + (t & 3) * 1024 + (b + 8 + 16 * pk) * 16 + 8 * ph) =
                u32x2{__builtin_bit_cast(uint32_t, l01), __builtin_bit_cast(uint32_t, l23)};
        }
        if constexpr (T::SUMS) {
            if (t0 == 4) {
                // scaled by 1/64: a sum of 32 values below 2^14 stays below 2^13
                sm *= 0.015625f;
                const _Float16 shi = (_Float16)sm, slo = (_Float16)(sm - (float)shi);
                _Float16 *sreg = reinterpret_cast<_Float16 *>(reg + 4096);  // [A row m][block j]
                sreg[b * 8 + part] = shi;
                sreg[(b + 8) * 8 + part] = slo;
            }
        }
        wave_lds_sync();
#pragma unroll
        for (int j = 0; j < 4; ++j) xa[t0 + j] = *reinterpret_cast<const f16x8 *>(reg + j * 1024 + lane * 16);
        if constexpr (T::SUMS) {
            if (t0 == 4) {
                const f16x8 t8 = *reinterpret_cast<const f16x8 *>(reg + 4096 + nq * 16);
                if (kq == 0) xs = t8;  // only the first K slots of the operand carry the sums
            }
        }
        wave_lds_sync();
    }
}

// y[b, row] (+)= sum_k W[row, k] x[b, k] (+ bias[row]) for b < rows <= 8; k a multiple of 256, n >= 16.
//   grid: up to one workgroup per group of 16 weight rows (the host caps it at one per CU), MF_THREADS threads,
//   dynamic LDS gemv_mfma_lds_bytes<FMT>().
template <int FMT>
__global__ void __launch_bounds__(MF_THREADS) gemv_mfma_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x,
                                                                const float *__restrict__ bias, float *__restrict__ y, int n, int k, int rows,
                                                                int stride) {  // stride: the grid's workgroups (an argument, preloaded with the others: gridDim is fetched from a cold block)
    typedef MTile<FMT> T;
    constexpr int CH = T::BYTES / 16;           // whole 16-byte chunks of a tile row
    constexpr int TAIL = T::BYTES % 16;         // 0, or the 2 bytes of Q6_K's d after 13 chunks
    static_assert(TAIL == 0 || TAIL == 2, "a tile row is whole 16-byte chunks, or Q6_K's 13 chunks + d");
    constexpr int ALIGN = TAIL ? 2 : 16;        // Q6_K rows start on even addresses only
    constexpr int PITCH = mf_row_pitch<FMT>();
    constexpr int REGION = mf_region_bytes<FMT>();
    constexpr int NL = (16 * CH + 63) / 64;     // 128-bit loads per lane and tile
    constexpr int NC = MF_COLS, PASS = MF_WAVES * NC;
    extern __shared__ __attribute__((aligned(16))) uint8_t mf_smem[];
    const int tid = threadIdx.x, lane = tid & 63, nq = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t *const reg = mf_smem + wave * NC * REGION;                                            // this wave's own regions
    float4 *const red = reinterpret_cast<float4 *>(mf_smem + MF_WAVES * NC * REGION);             // [wave][group][32 lanes]
    const int tiles = k >> 8, ngroups = (n + 15) >> 4;
    const size_t rowbytes = (size_t)tiles * T::BYTES;

    // this lane's share of a tile's bytes: chunk c = lane + 64 i -> (row c / CH, 16-byte chunk c % CH of that row's run)
    int crow[NL], cidx[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int c = lane + 64 * i;
        crow[i] = c / CH;
        cidx[i] = c - crow[i] * CH;
    }

    for (int t0 = 0; t0 < tiles; t0 += PASS) {
        // wave w owns columns t0 + w and t0 + w + MF_WAVES of this pass
        bool live[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) live[c] = t0 + wave + c * MF_WAVES < tiles;  // wave-uniform
        // lane offsets of this wave's chunks inside a row group (a group of 16 rows x rowbytes stays far below 4 GiB)
        uint32_t loff[NC][NL];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int i = 0; i < NL; ++i)
                loff[c][i] = live[c] && crow[i] < 16 ? (uint32_t)(crow[i] * rowbytes + (size_t)(t0 + wave + c * MF_WAVES) * T::BYTES + (size_t)cidx[i] * 16) : 0u;
        }
        uint32_t toff[NC];  // TAIL: lanes 0..15 also fetch the last two bytes of their row's run
#pragma unroll
        for (int c = 0; c < NC; ++c)
            toff[c] = TAIL && live[c] && lane < 16 ? (uint32_t)(lane * rowbytes + (size_t)(t0 + wave + c * MF_WAVES) * T::BYTES + 16 * CH) : 0u;
        auto fetch = [&](u32x4(&dst)[NC][NL], uint32_t(&tl)[NC], int grp) {
            if (grp >= ngroups) return;  // workgroup-uniform
            // the last group of a ragged matrix is the last 16 rows: in bounds, its first rows computed twice, stored once
            const uint8_t *gb = W + (size_t)min(grp * 16, n - 16) * rowbytes;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
#pragma unroll
                for (int i = 0; i < NL; ++i) dst[c][i] = ld128<ALIGN>(gb + loff[c][i]);
                if constexpr (TAIL != 0) tl[c] = ld16(gb + toff[c]);
            }
        };
        auto stash = [&](const u32x4(&src)[NC][NL], const uint32_t(&tl)[NC]) {
#pragma unroll
            for (int c = 0; c < NC; ++c) {
#pragma unroll
                for (int i = 0; i < NL; ++i)
                    if (crow[i] < 16) *reinterpret_cast<u32x4 *>(reg + c * REGION + crow[i] * PITCH + cidx[i] * 16) = src[c][i];
                if constexpr (TAIL != 0)
                    if (lane < 16) *reinterpret_cast<uint16_t *>(reg + c * REGION + lane * PITCH + 16 * CH) = (uint16_t)tl[c];
            }
        };

        // ---- the activations of this wave's columns go out first, then the weights of its first two row groups:
        // loads return in order, and the A operands are built while HBM works on the weights.
        // lane = (activation row b, part): quad 8 t + part of a column for t = 0..7, i.e. quad `part` of every block
        float4 v[NC][8];
        bool have[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            have[c] = live[c] && (lane >> 3) < rows;
            const float *xp = x + (size_t)(have[c] ? lane >> 3 : 0) * k + (size_t)(live[c] ? t0 + wave + c * MF_WAVES : 0) * 256 + 4 * (lane & 7);
#pragma unroll
            for (int t = 0; t < 8; ++t) v[c][t] = *reinterpret_cast<const float4 *>(xp + 32 * t);
        }
        u32x4 st[2][NC][NL];
        uint32_t stt[2][NC];
        fetch(st[0], stt[0], blockIdx.x);
        fetch(st[1], stt[1], blockIdx.x + stride);

        f16x8 xa[NC][8], xs[NC];
        float inv[NC][4];
#pragma unroll
        for (int c = 0; c < NC; ++c) mf_build_operands<T>(v[c], have[c], reg + c * REGION, lane, xa[c], xs[c], inv[c]);

        // ---- row groups, MF_GROUPS at a time: registers -> the wave's LDS regions -> operands -> partial sums
        for (int base = blockIdx.x; base < ngroups; base += MF_GROUPS * stride) {
            f32x4 acc[MF_GROUPS];
#pragma unroll
            for (int gi = 0; gi < MF_GROUPS; ++gi) {
                const int grp = base + gi * stride;
                acc[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (grp < ngroups) {  // workgroup-uniform
                    stash(st[gi & 1], stt[gi & 1]);
                    fetch(st[gi & 1], stt[gi & 1], grp + 2 * stride);
                    wave_lds_sync();
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        if (!live[c]) continue;  // wave-uniform: nothing was staged for a column past the end of the row
                        const f32x4 a = T::mma(reg + c * REGION + nq * PITCH, kq, xa[c], xs[c]);
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc[gi][i] = __builtin_fmaf(a[i], inv[c][i], acc[gi][i]);
                    }
                    wave_lds_sync();
                }
            }
            // hi rows (kq 0, 1) + lo rows (kq 2, 3) of the same activation rows, then the waves' sums meet in LDS
#pragma unroll
            for (int gi = 0; gi < MF_GROUPS; ++gi) {
                float4 t;
                t.x = acc[gi][0] + __shfl_xor(acc[gi][0], 32);
                t.y = acc[gi][1] + __shfl_xor(acc[gi][1], 32);
                t.z = acc[gi][2] + __shfl_xor(acc[gi][2], 32);
                t.w = acc[gi][3] + __shfl_xor(acc[gi][3], 32);
                if (lane < 32) red[(wave * MF_GROUPS + gi) * 32 + lane] = t;
            }
            __syncthreads();
            {
                const int gi = tid >> 7, r = tid & 15, br = (tid >> 4) & 7, grp = base + gi * stride, row = min(grp * 16, n - 16) + r;
                const float *src = reinterpret_cast<const float *>(red + gi * 32 + r + 16 * (br >> 2)) + (br & 3);
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < MF_WAVES; ++w) sum += src[w * MF_GROUPS * 32 * 4];
                if (grp < ngroups && row >= grp * 16 && br < rows) {
                    float *o = y + (size_t)br * n + row;
                    if (t0 == 0) *o = bias ? sum + bias[row] : sum;
                    else *o += sum;
                }
            }
            __syncthreads();
        }
    }
}

}  // namespace jitnn
