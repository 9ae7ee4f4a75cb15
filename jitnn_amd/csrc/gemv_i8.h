// Batch-1 GEMV on raw K-quant blocks with the dot products on the matrix cores in INT8 (gfx950, wave64).
//
// The quants of a K-quant block are small integers (4, 5 or 6 bits) and sit in memory as nibbles and bit fields: two or
// three mask / shift instructions turn a dword of them into four INT8 values - an operand of v_mfma_i32_4x4x4_16b_i8 as
// it stands.  The activations are turned once per workgroup into 22-bit fixed point per 64-value chunk (a power-of-two
// step from the chunk's largest magnitude, rounding by one FMA with 1.5 * 2^23) and cut into three signed byte digits,
// v = d0 + 256 d1 + 65536 d2: three of the four operand rows of the 4x4x4 product.  The instruction multiplies sixteen
// independent 4x4 blocks, each with its own activations: lane 4 b + j feeds the quants of weight row j (of four rows) for
// chunk b (of sixteen) of the row, lane 4 b + i the digit plane i of chunk b's activations, and the three digit sums of
// (row j, chunk b) come back to lane 4 b + j - the lane that loaded that row's bytes and decodes its scales.  So the
// sums are exact integers, nothing crosses lanes between load and scale, and per 64 weights a lane issues 16 matrix
// instructions and about 24 mask / shift instructions where the FP32 kernel issues 32 conversions and 64 multiply-adds.
// Error against the FP64 reference: the rounding of x to 2^-22 of its chunk's largest magnitude (about 3e-7 of max|y|).
//
// Work decomposition: a workgroup has one wave per 1024 values of the row (four for K = 4096); a turn of the
// workgroup is a group of four consecutive weight rows, wave w multiplying its 1024-value slice of them.  The slice's
// partial sums of a turn leave the wave through a two-step DPP fold (16 floats to LDS); every i8_flush() turns the
// workgroup meets at a barrier and one thread per output adds the partial sums in a fixed order - no atomics, the
// result does not depend on the launch shape.  Weight bytes are prefetched PF turns ahead through a register ring with
// unconditional loads (turns past the end get a descriptor of extent zero: zeros, no traffic) so the hardware's
// in-order load counter is waited on exactly.  What a wave needs before its first loads arrives in scalar registers with
// the wave (leading kernel arguments, preloaded by the hardware: I8Lead); what the flush needs is fetched under the
// wait for the first weights - a cold argument block is a round trip to memory wherever it is first touched.
//
// A slice that holds an activation that is not finite takes a slow path (every weight decoded by the bit-exact
// expression of the dequantiser and multiplied in FP32) so that +-Inf and NaN come out as the reference's FP64 sum
// gives them (core/ops/Gguf.java:187-205).
#pragma once
#include "common.h"
#include "dequant.h"
#include "tu.h"

namespace jitnn {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int I8_MAX_WAVES = 16;
// turns between two joins of the waves' partial sums (a multiple of every ring length): 36 for one activation row - the 28 turns
// of a gate / up launch of an 8B layer fit one window: 14.1 against 14.5 us with 24 -, 24 for more (the 14 turns of a 14336-row
// matrix in one window: Q4_K 14336 x 4096 at two rows 9.2 against 10.2 us with 12)
__host__ __device__ constexpr int i8_flush(int rows) { return rows == 1 ? 36 : 24; }
// LDS of a wave: 16 chunks x 3 planes x 64 bytes while the activations are staged; afterwards the wave's partial sums,
// 2 windows x flush turns x rows x 16 floats
__host__ __device__ constexpr size_t gemv_i8_lds_per_wave(int rows) {
    const size_t stage = rows == 4 ? 4 * 3072 : 3072, sums = (size_t)2 * i8_flush(rows) * rows * 64;  // (four rows: all their planes at once)
    return sums > stage ? sums : stage;
}
__host__ __device__ constexpr size_t gemv_i8_lds_bytes(int waves, int rows = 1) { return (size_t)waves * gemv_i8_lds_per_wave(rows); }

// The three digit sums of a block as one number.  With quants of at most five bits the whole sum fits 32 bits
// (31 * 16 * 2^22 < 2^31); six-bit quants (63 * 16 * 2^22) need the last step in floating point.
__device__ __forceinline__ int i8_combine(const i32x4 &d) { return (((d[2] << 8) + d[1]) << 8) + d[0]; }
__device__ __forceinline__ float i8_combine_wide(const i32x4 &d) { return __builtin_fmaf((float)((d[2] << 8) + d[1]), 256.f, (float)d[0]); }

// Weight bytes come through buffer loads: the descriptor (base of the matrix, extent) and the byte offset of the turn's
// row group sit in scalar registers, the lane's own offsets in vector registers computed once - a load costs no vector
// arithmetic, and a descriptor of extent zero makes the loads of a turn past the end return zeros without touching memory.
__device__ __forceinline__ u32x4 i8_ld128(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, (int)soff, 0);
}

template <int FMT>
struct U8;

// scale and min of sub-blocks 2j and 2j+1 of a Q4_K / Q5_K super-block as packed byte pairs (h = the block's first 16
// bytes; reference: core/kernels/GgufKernels.java:74-83)
__device__ __forceinline__ void i8_scale_min(const u32x4 &h, int j, uint32_t &sc2, uint32_t &mn2) {
    const int sh = (j & 1) * 16;
    const uint32_t m1 = j < 2 ? 0x3f3fu : 0u, m2 = j < 2 ? 0u : 0x0f0fu, m3 = j < 2 ? 0u : 0x3030u;
    const uint32_t a = h.y >> sh, b = h.z >> sh, c = h.w >> sh;
    sc2 = (a & m1) | (c & m2) | ((a >> 2) & m3);
    mn2 = (b & m1) | ((c >> 4) & m2) | ((b >> 2) & m3);
}

// ---------------------------------------------------------------------------------------------- Q4_K
// Chunk c of a row = values [64 c, 64 c + 64): group c % 4 of super-block c / 4, 32 qs bytes whose low nibbles are the
// first 32 values (sub-block 2j) and whose high nibbles the last 32 (sub-block 2j + 1).
template <>
struct U8<F_Q4_K> {
    static constexpr int FMT = F_Q4_K, NSUM = 2;
    struct Raw { u32x4 h, q0, q1; };
    struct Off { uint32_t h, q; };  // byte offsets of the lane's fields from the first row of its row group
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) {
        Off o;
        o.h = row_off + (uint32_t)(c >> 2) * 144u;
        o.q = o.h + 16u + (uint32_t)(c & 3) * 32u;
        return o;
    }
    __device__ static __forceinline__ int x_first(int c, int j) { return c * 64 + j * 16; }  // the 16 values lane (c, j) stages
    __device__ static __forceinline__ int x_pos(int c, int e) { return c * 64 + e; }         // value e of the chunk in operand order
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.h = i8_ld128(rs, o.h, soff);
        r.q0 = i8_ld128(rs, o.q, soff);
        r.q1 = i8_ld128(rs, o.q + 16u, soff);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
        s[0] = s4[0] + s4[1];
        s[1] = s4[2] + s4[3];
    }
    // the operands of the turn: dwords 0..7 the low nibbles (values 0..31 of the chunk), 8..15 the high ones (values 32..63)
    static constexpr int CH = 2;  // chains of products: one per sub-block
    struct Scale { float d0, d1, m0, m1; };
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const uint32_t w = m < 4 ? r.q0[m & 3] : r.q1[m & 3];
            v[m] = w & 0x0f0f0f0fu;
            v[8 + m] = (w >> 4) & 0x0f0f0f0fu;
        }
    }
    __device__ static __forceinline__ void scales(const Raw &r, int c, Scale &sc) {
        uint32_t sc2, mn2;
        i8_scale_min(r.h, c & 3, sc2, mn2);
        const float d = h2f(r.h.x), dmin = h2f(r.h.x >> 16);
        sc.d0 = d * ub0(sc2);
        sc.d1 = d * ub1(sc2);
        sc.m0 = dmin * ub0(mn2);
        sc.m1 = dmin * ub1(mn2);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        const float t = __builtin_fmaf(sc.d0, (float)i8_combine(d[0]), sc.d1 * (float)i8_combine(d[1]));
        const float m = __builtin_fmaf(sc.m0, s[0], sc.m1 * s[1]);
        return __builtin_fmaf(t, sinv, -m);
    }
};

// ---------------------------------------------------------------------------------------------- Q5_K
// As Q4_K with a fifth bit: bit (2j + half) of qh[l] (core/kernels/GgufKernels.java:113-125); block 176 bytes:
// d, dmin, scales[12], qh[32], qs[128].
template <>
struct U8<F_Q5_K> {
    static constexpr int FMT = F_Q5_K, NSUM = 2;
    struct Raw { u32x4 h, h0, h1, q0, q1; };
    struct Off { uint32_t h, q; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) {
        Off o;
        o.h = row_off + (uint32_t)(c >> 2) * 176u;
        o.q = o.h + 48u + (uint32_t)(c & 3) * 32u;
        return o;
    }
    __device__ static __forceinline__ int x_first(int c, int j) { return c * 64 + j * 16; }
    __device__ static __forceinline__ int x_pos(int c, int e) { return c * 64 + e; }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.h = i8_ld128(rs, o.h, soff);
        r.h0 = i8_ld128(rs, o.h + 16u, soff);
        r.h1 = i8_ld128(rs, o.h + 32u, soff);
        r.q0 = i8_ld128(rs, o.q, soff);
        r.q1 = i8_ld128(rs, o.q + 16u, soff);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
        s[0] = s4[0] + s4[1];
        s[1] = s4[2] + s4[3];
    }
    static constexpr int CH = 2;
    typedef U8<F_Q4_K>::Scale Scale;
    __device__ static __forceinline__ void extract(const Raw &r, int c, uint32_t (&v)[16]) {
        const int sh = 2 * (c & 3);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const uint32_t w = m < 4 ? r.q0[m & 3] : r.q1[m & 3];
            const uint32_t hb = (m < 4 ? r.h0[m & 3] : r.h1[m & 3]) >> sh;  // bit 0 of every byte: sub-block 2j, bit 1: 2j + 1
            v[m] = (w & 0x0f0f0f0fu) | ((hb << 4) & 0x10101010u);
            v[8 + m] = ((w >> 4) & 0x0f0f0f0fu) | ((hb << 3) & 0x10101010u);
        }
    }
    __device__ static __forceinline__ void scales(const Raw &r, int c, Scale &sc) {
        uint32_t sc2, mn2;
        i8_scale_min(r.h, c & 3, sc2, mn2);
        const float d = h2f(r.h.x), dmin = h2f(r.h.x >> 16);
        sc.d0 = d * ub0(sc2);
        sc.d1 = d * ub1(sc2);
        sc.m0 = dmin * ub0(mn2);
        sc.m1 = dmin * ub1(mn2);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        return U8<F_Q4_K>::finish(sc, d, sinv, s);
    }
};

// ---------------------------------------------------------------------------------------------- Q6_K
// block_q6_K, 210 bytes: ql[128], qh[64], i8 scales[16], f16 d (core/kernels/GgufKernels.java:127-140).  Chunk
// c = 4 sb + 2 n + r covers l in [16 r, 16 r + 16) of half n of super-block sb for the four k: four runs of 16 values,
// run k at x[256 sb + 128 n + 32 k + 16 r ..], each with its own int8 scale (index 8 n + 2 k + r).  The quants come out
// as q in 0..63; the -32 of the format meets the sums of x over the runs.
//
// Blocks are 210 bytes long, so every other block of a row starts two bytes past a dword boundary - and a 16-byte load
// from such an address runs at 70 % of the rate of a dword-aligned one (4.6 against 6.5 TB/s streaming, measured; loads of
// 8 and 2 bytes cost more still).  U8Q6<true> (rows a multiple of 4 bytes long, i.e. K a multiple of 512, and matrices on
// dword boundaries) therefore fetches dword-aligned windows - the lane's field minus the block's two-byte shift - and
// shifts the fields into place with v_alignbit: the two bytes a window misses are the first two of the window that
// follows it in memory, which a neighbouring lane of the same block holds (the fields of the four chunks of a block tile
// ql and qh without gaps) and hands over with one DPP rotation.  U8Q6<false> loads the fields where they are.
template <bool ALIGNED>
struct U8Q6;

struct U8Q6Base {
    static constexpr int FMT = F_Q6_K, NSUM = 4;
    __device__ static __forceinline__ int x_first(int c, int j) { return (c >> 2) * 256 + ((c >> 1) & 1) * 128 + 32 * j + 16 * (c & 1); }
    __device__ static __forceinline__ int x_pos(int c, int e) { return x_first(c, e >> 4) + (e & 15); }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] = -32.f * s4[i];
    }
    static constexpr int CH = 4;  // one chain per run of 16 values
    struct Scale { float c[4]; };  // d * scale of run k
    // la, lb: the lane's 16 bytes of ql at 64 n + 16 r and 32 further on; qh: its 16 bytes of qh -> operands of run k in dwords 4k..4k+3
    __device__ static __forceinline__ void extract_fields(const u32x4 &la, const u32x4 &lb, const u32x4 &qh, uint32_t (&v)[16]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t a = la[i], b = lb[i], h = qh[i];
            v[i] = (a & 0x0f0f0f0fu) | ((h << 4) & 0x30303030u);
            v[4 + i] = (b & 0x0f0f0f0fu) | ((h << 2) & 0x30303030u);
            v[8 + i] = ((a >> 4) & 0x0f0f0f0fu) | (h & 0x30303030u);
            v[12 + i] = ((b >> 4) & 0x0f0f0f0fu) | ((h >> 2) & 0x30303030u);
        }
    }
    // sa, sb: dwords whose bytes 0 and 2 are the scales of runs 0, 1 | 2, 3; d: the block scale's bits
    __device__ static __forceinline__ void scale_fields(uint32_t sa, uint32_t sb, uint32_t d, Scale &sc) {
        const float df = h2f(d);
        sc.c[0] = df * (float)(int)(int8_t)sa;
        sc.c[1] = df * (float)(int)(int8_t)(sa >> 16);
        sc.c[2] = df * (float)(int)(int8_t)sb;
        sc.c[3] = df * (float)(int)(int8_t)(sb >> 16);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        float acc = sc.c[0] * __builtin_fmaf(i8_combine_wide(d[0]), sinv, s[0]);
#pragma unroll
        for (int k = 1; k < 4; ++k) acc = __builtin_fmaf(sc.c[k], __builtin_fmaf(i8_combine_wide(d[k]), sinv, s[k]), acc);
        return acc;
    }
};

template <>
struct U8Q6<false> : U8Q6Base {
    struct Raw { u32x4 la, lb, qh; u32x2 sc; uint32_t d; };
    struct Off { uint32_t la, qh, sc, d; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) {
        Off o;
        const uint32_t blk = row_off + (uint32_t)(c >> 2) * 210u, n = (uint32_t)(c >> 1) & 1u, r = (uint32_t)c & 1u;
        o.la = blk + 64u * n + 16u * r;
        o.qh = blk + 128u + 32u * n + 16u * r;
        o.sc = blk + 192u + 8u * n;
        o.d = blk + 208u;
        return o;
    }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.la = i8_ld128(rs, o.la, soff);   // (fields on 2-byte boundaries: buffer loads take them like the global ones)
        r.lb = i8_ld128(rs, o.la + 32u, soff);
        r.qh = i8_ld128(rs, o.qh, soff);
        r.sc = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)o.sc, (int)soff, 0);
        r.d = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rs, (int)o.d, (int)soff, 0);
    }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) { extract_fields(r.la, r.lb, r.qh, v); }
    __device__ static __forceinline__ void scales(const Raw &r, int c, Scale &sc) {
        const int sh = (c & 1) * 8;
        scale_fields(r.sc.x >> sh, r.sc.y >> sh, r.d, sc);
    }
};

typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));

template <>
struct U8Q6<true> : U8Q6Base {
    struct Raw { u32x4 la, lb, qh; u32x3 sc; uint32_t d; };  // dword-aligned windows: the fields start `shift` bytes into them
    struct Off { uint32_t la, qh, sc, d; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) {
        Off o;
        const uint32_t blk = row_off + (uint32_t)(c >> 2) * 210u, n = (uint32_t)(c >> 1) & 1u, r = (uint32_t)c & 1u;
        const uint32_t base = blk & ~3u;  // (row_off is a multiple of 4: the shift of a block is 2 for odd sb)
        o.la = base + 64u * n + 16u * r;
        o.qh = base + 128u + 32u * n + 16u * r;
        o.sc = base + 192u + 8u * n;
        o.d = base + 208u;
        return o;
    }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.la = i8_ld128(rs, o.la, soff);
        r.lb = i8_ld128(rs, o.la + 32u, soff);
        r.qh = i8_ld128(rs, o.qh, soff);
        r.sc = __builtin_amdgcn_raw_buffer_load_b96(rs, (int)o.sc, (int)soff, 0);
        r.d = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)o.d, (int)soff, 0);
    }
    // the first dword of the lane 4 further on / 4 back in its row of 16 lanes (the next / previous chunk of the block, same weight row)
    __device__ static __forceinline__ uint32_t next4(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x12C, 0xF, 0xF, false); }  // row_ror:12
    __device__ static __forceinline__ uint32_t prev4(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x124, 0xF, 0xF, false); }  // row_ror:4
    __device__ static __forceinline__ u32x4 shifted(const u32x4 &w, uint32_t after, uint32_t sh) {
        return u32x4{__builtin_amdgcn_alignbit(w.y, w.x, sh), __builtin_amdgcn_alignbit(w.z, w.y, sh), __builtin_amdgcn_alignbit(w.w, w.z, sh),
                     __builtin_amdgcn_alignbit(after, w.w, sh)};
    }
    __device__ static __forceinline__ void extract(const Raw &r, int c, uint32_t (&v)[16]) {
        const uint32_t sh = (uint32_t)((c >> 2) & 1) * 16u;  // bits the block's fields sit past their windows' starts
        const bool r0 = (c & 1) == 0, n0 = (c & 2) == 0, last = (c & 3) == 3;
        // In memory the windows of a block follow one another as la(b0) la(b1) lb(b0) lb(b1) la(b2) la(b3) lb(b2) lb(b3) qh(b0..b3)
        // scales (b = chunk of the block): the dword after a window is the first dword of the next one.
        const uint32_t nla = next4(r.la.x), nlb = next4(r.lb.x), nqh = next4(r.qh.x), nsc = next4(r.sc.x), plb = prev4(r.lb.x);
        extract_fields(shifted(r.la, r0 ? nla : plb, sh), shifted(r.lb, r0 ? nlb : n0 ? nla : nqh, sh), shifted(r.qh, last ? nsc : nqh, sh), v);
    }
    __device__ static __forceinline__ void scales(const Raw &r, int c, Scale &sc) {
        const uint32_t sh = (uint32_t)((c >> 2) & 1) * 16u;
        const uint32_t sx = __builtin_amdgcn_alignbit(r.sc.y, r.sc.x, sh), sy = __builtin_amdgcn_alignbit(r.sc.z, r.sc.y, sh);
        const int s8 = (c & 1) * 8;
        scale_fields(sx >> s8, sy >> s8, r.d >> sh, sc);
    }
};

template <>
struct U8<F_Q6_K> : U8Q6<false> {};

// ------------------------------------------------------------------------------------- the 32-value formats
// Q4_0 (18 bytes: f16 d, 16 bytes of nibbles), Q4_1 (20: d, m, nibbles) and Q8_0 (34: d, 32 int8) - core/kernels/GgufKernels.java:85-99,
// core/ops/Quant.java:137-144.  A chunk is two blocks (rows of a multiple of 64 values): a pair starts on a dword boundary
// (36, 40 and 68 bytes), the lane fetches it as whole dwords and shifts the first block's quants, which sit two bytes past
// one, into place with v_alignbit.  Value e of a 4-bit block is the low nibble of qs[e] for e < 16, the high nibble of
// qs[e - 16] otherwise, so the operands keep the order of the values; one chain of products per block, one scale each.
// Thirty-two products of up to 128 * 2^22 do not fit 32 bits: the digit sums are joined in floating point.
__device__ __forceinline__ u32x4 i8_shift2(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t w4) {
    return u32x4{__builtin_amdgcn_alignbit(w1, w0, 16), __builtin_amdgcn_alignbit(w2, w1, 16), __builtin_amdgcn_alignbit(w3, w2, 16),
                 __builtin_amdgcn_alignbit(w4, w3, 16)};
}

struct U8Pair32 {
    static constexpr int NSUM = 2, CH = 2;
    __device__ static __forceinline__ int x_first(int c, int j) { return c * 64 + j * 16; }
    __device__ static __forceinline__ int x_pos(int c, int e) { return c * 64 + e; }
    __device__ static __forceinline__ void nibbles(const u32x4 &q0, const u32x4 &q1, uint32_t (&v)[16]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = q0[i] & 0x0f0f0f0fu;
            v[4 + i] = (q0[i] >> 4) & 0x0f0f0f0fu;
            v[8 + i] = q1[i] & 0x0f0f0f0fu;
            v[12 + i] = (q1[i] >> 4) & 0x0f0f0f0fu;
        }
    }
};

template <>
struct U8<F_Q4_0> : U8Pair32 {
    static constexpr int FMT = F_Q4_0;
    struct Raw { u32x4 a, b; uint32_t c; };  // bytes 0-1 d0, 2-17 qs0, 18-19 d1, 20-35 qs1
    struct Off { uint32_t o; };
    struct Scale { float d0, d1; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) { return Off{row_off + (uint32_t)c * 36u}; }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.a = i8_ld128(rs, o.o, soff);
        r.b = i8_ld128(rs, o.o + 16u, soff);
        r.c = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)(o.o + 32u), (int)soff, 0);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {  // the -8 of the format meets the sums of x
        s[0] = -8.f * (s4[0] + s4[1]);
        s[1] = -8.f * (s4[2] + s4[3]);
    }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {
        nibbles(i8_shift2(r.a.x, r.a.y, r.a.z, r.a.w, r.b.x), u32x4{r.b.y, r.b.z, r.b.w, r.c}, v);
    }
    __device__ static __forceinline__ void scales(const Raw &r, int, Scale &sc) {
        sc.d0 = h2f(r.a.x);
        sc.d1 = h2f(r.b.x >> 16);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        return __builtin_fmaf(sc.d0, __builtin_fmaf(i8_combine_wide(d[0]), sinv, s[0]), sc.d1 * __builtin_fmaf(i8_combine_wide(d[1]), sinv, s[1]));
    }
};

template <>
struct U8<F_Q4_1> : U8Pair32 {
    static constexpr int FMT = F_Q4_1;
    struct Raw { u32x4 a, b; u32x2 c; };  // bytes 0-3 d0 m0, 4-19 qs0, 20-23 d1 m1, 24-39 qs1
    struct Off { uint32_t o; };
    struct Scale { float d0, m0, d1, m1; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) { return Off{row_off + (uint32_t)c * 40u}; }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.a = i8_ld128(rs, o.o, soff);
        r.b = i8_ld128(rs, o.o + 16u, soff);
        r.c = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)(o.o + 32u), (int)soff, 0);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
        s[0] = s4[0] + s4[1];
        s[1] = s4[2] + s4[3];
    }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {
        nibbles(u32x4{r.a.y, r.a.z, r.a.w, r.b.x}, u32x4{r.b.z, r.b.w, r.c.x, r.c.y}, v);
    }
    __device__ static __forceinline__ void scales(const Raw &r, int, Scale &sc) {
        sc.d0 = h2f(r.a.x);
        sc.m0 = h2f(r.a.x >> 16);
        sc.d1 = h2f(r.b.y);
        sc.m1 = h2f(r.b.y >> 16);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        const float t = __builtin_fmaf(sc.d0, i8_combine_wide(d[0]), sc.d1 * i8_combine_wide(d[1]));
        return __builtin_fmaf(t, sinv, __builtin_fmaf(sc.m0, s[0], sc.m1 * s[1]));
    }
};

template <>
struct U8<F_Q8_0> : U8Pair32 {
    static constexpr int FMT = F_Q8_0;
    struct Raw { u32x4 a, b, c, d; uint32_t e; };  // bytes 0-1 d0, 2-33 qs0, 34-35 d1, 36-67 qs1
    struct Off { uint32_t o; };
    struct Scale { float d0, d1; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) { return Off{row_off + (uint32_t)c * 68u}; }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.a = i8_ld128(rs, o.o, soff);
        r.b = i8_ld128(rs, o.o + 16u, soff);
        r.c = i8_ld128(rs, o.o + 32u, soff);
        r.d = i8_ld128(rs, o.o + 48u, soff);
        r.e = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)(o.o + 64u), (int)soff, 0);
    }
    __device__ static __forceinline__ void sums(const float (&)[4], float (&s)[NSUM]) { s[0] = s[1] = 0.f; }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {  // the quants are INT8 operands as they stand
        const u32x4 lo = i8_shift2(r.a.x, r.a.y, r.a.z, r.a.w, r.b.x), hi = i8_shift2(r.b.x, r.b.y, r.b.z, r.b.w, r.c.x);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = lo[i];
            v[4 + i] = hi[i];
        }
        v[8] = r.c.y; v[9] = r.c.z; v[10] = r.c.w; v[11] = r.d.x; v[12] = r.d.y; v[13] = r.d.z; v[14] = r.d.w; v[15] = r.e;
    }
    __device__ static __forceinline__ void scales(const Raw &r, int, Scale &sc) {
        sc.d0 = h2f(r.a.x);
        sc.d1 = h2f(r.c.x >> 16);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&)[NSUM]) {
        return __builtin_fmaf(sc.d0, i8_combine_wide(d[0]), sc.d1 * i8_combine_wide(d[1])) * sinv;
    }
};

// ------------------------------------------------------------------------------------- Q5_1
// block_q5_1, 24 bytes: f16 d, f16 m, 32 fifth bits qh, 16 bytes of nibbles; value e = (nibble e % 16 (low for e < 16) + 16 * bit e
// of qh) * d + m (core/kernels/GgufKernels.java:155-163).  A chunk is two blocks = 48 bytes = three 16-byte loads (matrices on
// dword boundaries: the caller checks).
template <>
struct U8<F_Q5_1> : U8Pair32 {
    static constexpr int FMT = F_Q5_1;
    struct Raw { u32x4 a, b, c; };  // a: d0 | m0, qh0, qs0[0..7]; b: qs0[8..15], d1 | m1, qh1; c: qs1
    struct Off { uint32_t o; };
    struct Scale { float d0, d1, m0, m1; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) { return Off{row_off + (uint32_t)c * 48u}; }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.a = i8_ld128(rs, o.o, soff);
        r.b = i8_ld128(rs, o.o + 16u, soff);
        r.c = i8_ld128(rs, o.o + 32u, soff);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
        s[0] = s4[0] + s4[1];
        s[1] = s4[2] + s4[3];
    }
    // the fifth bits of values 4i .. 4i + 3 (bits 4i .. of qh) as bit 4 of the four bytes of a dword: the four copies of the
    // nibble that the product makes (shifted by 0, 7, 14, 21) do not overlap, bit t of the nibble lands on bit 8t
    __device__ static __forceinline__ uint32_t fifth(uint32_t qh, int i) { return ((((qh >> (4 * i)) & 15u) * 0x00204081u) & 0x01010101u) << 4; }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {
        nibbles(u32x4{r.a.z, r.a.w, r.b.x, r.b.y}, r.c, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[i] |= fifth(r.a.y, i);
            v[8 + i] |= fifth(r.b.w, i);
        }
    }
    __device__ static __forceinline__ void scales(const Raw &r, int, Scale &sc) {
        sc.d0 = h2f(r.a.x);
        sc.m0 = h2f(r.a.x >> 16);
        sc.d1 = h2f(r.b.z);
        sc.m1 = h2f(r.b.z >> 16);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        const float t = __builtin_fmaf(sc.d0, i8_combine_wide(d[0]), sc.d1 * i8_combine_wide(d[1]));
        return __builtin_fmaf(t, sinv, __builtin_fmaf(sc.m0, s[0], sc.m1 * s[1]));
    }
};

// ------------------------------------------------------------------------------------- Q2_K
// block_q2_K, 84 bytes: 16 scale bytes (low nibble scale, high nibble min), 64 bytes of 2-bit quants, f16 d, f16 dmin; value
// 128 n + 32 j + l is bits 2j.. of qs[32 n + l], scaled by byte 8 n + 2 j + l / 16 (core/kernels/GgufKernels.java:166-175).
// Chunk c = 4 sb + 2 n + r takes the 16 bytes l in [16 r, 16 r + 16) of half n of super-block sb: four runs of 16 values
// (j = 0..3), each with its own scale byte - the element order of the Q6_K chunk.
template <>
struct U8<F_Q2_K> {
    static constexpr int FMT = F_Q2_K, NSUM = 4, CH = 4;
    struct Raw { u32x4 q; u32x2 sc; uint32_t dd; };
    struct Off { uint32_t q, sc, dd; };
    struct Scale { float c[4], m[4]; };
    __device__ static __forceinline__ Off offsets(int c, uint32_t row_off) {
        Off o;
        const uint32_t blk = row_off + (uint32_t)(c >> 2) * 84u, n = (uint32_t)(c >> 1) & 1u, r = (uint32_t)c & 1u;
        o.q = blk + 16u + 32u * n + 16u * r;
        o.sc = blk + 8u * n;
        o.dd = blk + 80u;
        return o;
    }
    __device__ static __forceinline__ int x_first(int c, int j) { return U8Q6Base::x_first(c, j); }
    __device__ static __forceinline__ int x_pos(int c, int e) { return U8Q6Base::x_pos(c, e); }
    __device__ static __forceinline__ void load(Raw &r, __amdgpu_buffer_rsrc_t rs, const Off &o, uint32_t soff) {
        r.q = i8_ld128(rs, o.q, soff);
        r.sc = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)o.sc, (int)soff, 0);
        r.dd = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, (int)o.dd, (int)soff, 0);
    }
    __device__ static __forceinline__ void sums(const float (&s4)[4], float (&s)[NSUM]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] = s4[i];
    }
    __device__ static __forceinline__ void extract(const Raw &r, int, uint32_t (&v)[16]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = r.q[i];
            v[i] = w & 0x03030303u;
            v[4 + i] = (w >> 2) & 0x03030303u;
            v[8 + i] = (w >> 4) & 0x03030303u;
            v[12 + i] = (w >> 6) & 0x03030303u;
        }
    }
    __device__ static __forceinline__ void scales(const Raw &r, int c, Scale &sc) {
        const int sh = (c & 1) * 8;
        const uint32_t sa = r.sc.x >> sh, sb = r.sc.y >> sh;  // bytes 0 and 2: the scale bytes of runs 0, 1 | 2, 3
        const float d = h2f(r.dd), dmin = h2f(r.dd >> 16);
        sc.c[0] = d * (float)(sa & 15u);
        sc.m[0] = dmin * (float)((sa >> 4) & 15u);
        sc.c[1] = d * (float)((sa >> 16) & 15u);
        sc.m[1] = dmin * (float)((sa >> 20) & 15u);
        sc.c[2] = d * (float)(sb & 15u);
        sc.m[2] = dmin * (float)((sb >> 4) & 15u);
        sc.c[3] = d * (float)((sb >> 16) & 15u);
        sc.m[3] = dmin * (float)((sb >> 20) & 15u);
    }
    __device__ static __forceinline__ float finish(const Scale &sc, const i32x4 (&d)[CH], float sinv, const float (&s)[NSUM]) {
        float acc = sc.c[0] * (float)i8_combine(d[0]), m = sc.m[0] * s[0];
#pragma unroll
        for (int k = 1; k < 4; ++k) {
            acc = __builtin_fmaf(sc.c[k], (float)i8_combine(d[k]), acc);
            m = __builtin_fmaf(sc.m[k], s[k], m);
        }
        return __builtin_fmaf(acc, sinv, -m);
    }
};

// The partial sums of a turn for B activation rows: the operands and scales of the weights are made once, every row runs its
// chains of products (the chains of a row interleaved, so that a product never waits for the one before it).
template <class U, int B>
__device__ __forceinline__ void i8_dot(const typename U::Raw &r, int c, const uint32_t (&xa)[B][16], const float (&sinv)[B], const float (&s)[B][U::NSUM],
                                       float (&out)[B]) {
    constexpr int CH = U::CH, L = 16 / CH;
    uint32_t v[16];
    U::extract(r, c, v);
    typename U::Scale sc;
    U::scales(r, c, sc);
    if constexpr (B == 4) {
        // Four rows have twelve digit planes, and a product has four operand rows: packed - operand set m = the plane vectors
        // 4 m .. 4 m + 3, vector 3 r + p being plane p of row r - they fill three products where a product per row leaves a quarter
        // of four empty.  The sums of (weight row j, chunk b) still all come back to lane 4 b + j: row r's three are picked out of
        // the three results by constant indices.
        i32x4 d[3][CH];
#pragma unroll
        for (int m = 0; m < 3; ++m)
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) d[m][ch] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < L; ++i)
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
#pragma unroll
                for (int m = 0; m < 3; ++m) d[m][ch] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)xa[m][ch * L + i], (int)v[ch * L + i], d[m][ch], 0, 0, 0);
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            i32x4 dd[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
                dd[ch] = i32x4{d[(3 * b) / 4][ch][(3 * b) % 4], d[(3 * b + 1) / 4][ch][(3 * b + 1) % 4], d[(3 * b + 2) / 4][ch][(3 * b + 2) % 4], 0};
            out[b] = U::finish(sc, dd, sinv[b], s[b]);
        }
    } else {
#pragma unroll
        for (int b = 0; b < B; ++b) {
            i32x4 d[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) d[ch] = i32x4{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < L; ++i)
#pragma unroll
                for (int ch = 0; ch < CH; ++ch) d[ch] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)xa[b][ch * L + i], (int)v[ch * L + i], d[ch], 0, 0, 0);
            out[b] = U::finish(sc, d, sinv[b], s[b]);
        }
    }
}

// The 16 activations xv of lane (chunk b, quarter j) of a wave's 1024-value slice -> fixed point, v = rint(x * s), |v| < 2^22, s a
// power of two from the chunk's largest magnitude, cut into three signed byte digits; the planes cross the wave's own LDS
// (`planes`, 3 KB) from staging order into operand order: xa = the sixteen operand dwords of this lane's plane, sinv = 1 / s,
// sums = the sums of x the unit's offset terms need.  Returns whether the slice holds an Inf or a NaN (xa is garbage then).
template <class U>
__device__ __forceinline__ bool i8_stage(const float4 (&xv)[4], u32x4 *planes, int b, int j, uint32_t (&xa)[16], float &sinv, float (&sums)[U::NSUM]) {
    uint32_t am = 0u;
    float sm = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        am = max(max(am, max(__float_as_uint(xv[i].x) & 0x7fffffffu, __float_as_uint(xv[i].y) & 0x7fffffffu)),
                 max(__float_as_uint(xv[i].z) & 0x7fffffffu, __float_as_uint(xv[i].w) & 0x7fffffffu));
        sm += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    }
    am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    am = max(am, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)am, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    const bool nonfinite = __builtin_amdgcn_ballot_w64(am >= 0x7f800000u) != 0;
    const uint32_t eb = min(max(am >> 23, 22u), 254u);
    const float s = __uint_as_float((275u - eb) << 23);
    sinv = __uint_as_float((eb - 21u) << 23);
    float s4[4];
    s4[0] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), 0x00, 0xF, 0xF, true));  // quad_perm [0,0,0,0]
    s4[1] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), 0x55, 0xF, 0xF, true));
    s4[2] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), 0xAA, 0xF, 0xF, true));
    s4[3] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(sm), 0xFF, 0xF, 0xF, true));
    U::sums(s4, sums);
    uint32_t pl[3][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float f[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
        uint32_t u[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) u[e] = __float_as_uint(__builtin_fmaf(f[e], s, 12582912.f)) + (0x00808080u - 0x4B400000u);
        // bytes 0..2 of u are the digits + 128; gather byte p of the four values into one dword, then flip the top bits
        const uint32_t t01 = __builtin_amdgcn_perm(u[1], u[0], 0x05010400u), t23 = __builtin_amdgcn_perm(u[3], u[2], 0x05010400u);
        pl[0][i] = __builtin_amdgcn_perm(t23, t01, 0x05040100u) ^ 0x80808080u;
        pl[1][i] = __builtin_amdgcn_perm(t23, t01, 0x07060302u) ^ 0x80808080u;
        const uint32_t w01 = __builtin_amdgcn_perm(u[1], u[0], 0x00000602u), w23 = __builtin_amdgcn_perm(u[3], u[2], 0x00000602u);
        pl[2][i] = __builtin_amdgcn_perm(w23, w01, 0x05040100u) ^ 0x80808080u;
    }
    // (a slice that is not finite leaves garbage here; the slow path does not read it)
#pragma unroll
    for (int p = 0; p < 3; ++p) planes[(b * 3 + p) * 4 + j] = u32x4{pl[p][0], pl[p][1], pl[p][2], pl[p][3]};
    // (the LDS accesses of a wave complete in order: its reads below see its writes above without a barrier)
    __builtin_amdgcn_wave_barrier();
    const int p = min(j, 2);  // operand row 3 of the product is not used: lane 4b + 3 feeds plane 2 again
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
        const u32x4 v = planes[(b * 3 + p) * 4 + qd];
        xa[qd * 4 + 0] = v.x; xa[qd * 4 + 1] = v.y; xa[qd * 4 + 2] = v.z; xa[qd * 4 + 3] = v.w;
    }
    __builtin_amdgcn_wave_barrier();
    return nonfinite;
}

// What a wave needs before its first loads, as the kernels take it in front of the argument block (fourteen dwords: as many as
// the hardware preloads into scalar registers): the first matrix, the activations, a second matrix (DUAL: the up projection;
// row segments: the second segment), the norm weight, the third segment's matrix, three packed numbers, the rows of all segments
// and of the first two.
struct I8Lead {
    const uint8_t *w0;
    const float *x;
    const uint8_t *wb;  // DUAL: w2; row segments: w[1]
    const float *nw;
    const uint8_t *wc;  // row segments: w[2]
    int k, nblocks, rows;
    int n, n0, n1;
};
// k / 64 (9 bits: rows of at most 16384 values) | workgroups (20 bits) | activation rows - 1 (3 bits)
__host__ __device__ constexpr uint32_t i8_pack(int k, int nblocks, int rows) { return (uint32_t)(k >> 6) | ((uint32_t)nblocks << 9) | ((uint32_t)(rows - 1) << 29); }

// -------------------------------------------------------------------------------------------------- the kernel body
// rb: the first activation row of this workgroup (launches of more than B rows put the row groups of B along blockIdx.y:
// their workgroups stream the same weight bytes at the same time, so one of them finds them in the cache)
template <class U, int B, int PF, bool BIAS, bool NORM, bool DUAL, int MAXW>
__device__ __forceinline__ void gemv_i8_body(const I8Lead &ld, const I8Args &a, const int bid, const int rb = 0) {
    constexpr int FMT = U::FMT, NB = PF + 1, FL = i8_flush(B);
    static_assert(FL % NB == 0 && FL % 2 == 0, "whole rings (and gate/up pairs) per flush window");
    static_assert(B == 1 || (!NORM && !DUAL), "the fused norm and the SwiGLU pair are batch-1 launches");
    extern __shared__ __align__(16) uint8_t i8_smem[];
    __shared__ float red[I8_MAX_WAVES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int k = ld.k, chunks = k >> 6, nblocks = ld.nblocks;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = (k + 1023) >> 10;  // (the launch has one wave per 1024 values of a row)
    constexpr size_t WAVE_LDS = gemv_i8_lds_per_wave(B);
    u32x4 *const planes = reinterpret_cast<u32x4 *>(i8_smem + (size_t)wave * WAVE_LDS);
    float *const mypart = reinterpret_cast<float *>(planes);  // after the staging: [2][FL][B][4 dpp rows][4 rows] partial sums of this wave
    const int b = lane >> 2, j = lane & 3;
    const int n = ld.n;
    const int groups = (n + 3) >> 2;
    const size_t rowbytes = (size_t)(k / block_values(FMT)) * block_bytes(FMT);
    const bool inrow = wave * 16 + b < chunks;      // lanes past the end of the row: zero activations
    const int c = inrow ? wave * 16 + b : chunks - 1;
    const typename U::Off off = U::offsets(c, (uint32_t)j * (uint32_t)rowbytes);
    const int turns = (groups + nblocks - 1) / nblocks;  // row groups this workgroup takes (the last may be missing)
    const int vturns = DUAL ? 2 * turns : turns;         // DUAL: a group's gate rows, then its up rows

    // ---- the activations this lane stages: 16 values of chunk c of every activation row
    const int xf = U::x_first(c, j);
    float4 xv[B][4], nv[4];
    // (unconditional loads from clamped addresses - chunk c and the activation row exist -, zeroed afterwards where the lane has
    // nothing to stage: a load behind a condition is a branch around it, eight of them stood in front of the first weight load)
#pragma unroll
    for (int r = 0; r < B; ++r) {
        const int xr = B == 1 ? rb + r : min(rb + r, ld.rows - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) xv[r][i] = reinterpret_cast<const float4 *>(ld.x + (size_t)xr * k + xf)[i];
    }
    if (NORM) {
#pragma unroll
        for (int i = 0; i < 4; ++i) nv[i] = reinterpret_cast<const float4 *>(ld.nw + xf)[i];
    }
    __builtin_amdgcn_sched_barrier(0);  // (the activations' loads first: loads return in order, and the wait for them must not be one for weight bytes)

    // ---- the ring of weight bytes
    typename U::Raw buf[NB];
    // A turn's row group g holds the rows min(4 g, n - 4) ... + 3 (the last group of a row count that is no multiple of four
    // overlaps its neighbour; the flush skips the rows it shares).  Group, segment and byte offset are wave-uniform: scalar
    // arithmetic, and no branch - with conditional loads the compiler cannot count the loads in flight.
    // (the segment's matrix by differences: a choice among three pointers by two conditions gets compiled into a table in
    // private memory)
    // Row segments (several matrices in one launch) exist only where the decode step uses them: with the fused norm.  Every other
    // launch has one matrix, and its per-turn scalar arithmetic - which a wave alone on its SIMD pays in full - stays short.
    constexpr bool SEGMENTS = NORM && !DUAL;
    const uint8_t *const w0 = ld.w0, *const wd = ld.wb;
    const ptrdiff_t d01 = SEGMENTS ? ld.wb - ld.w0 : 0, d12 = SEGMENTS ? ld.wc - ld.wb : 0;
    const int n0 = SEGMENTS ? ld.n0 : n, n01 = SEGMENTS ? ld.n0 + ld.n1 : n;
    auto fill = [&](typename U::Raw &dst, int t) {
        const int g = bid + (DUAL ? t >> 1 : t) * nblocks;
        // extent of the descriptor: everything for a group that exists, nothing past the last group (turns at or past
        // vturns are past it too) - by arithmetic, so that the descriptor stays in scalar registers
        // (read back through a scalar lane: as a plain select feeding the descriptor it is built in vector registers, and every
        // load then runs in a loop over the descriptor values the lanes hold)
        const int extent = __builtin_amdgcn_readfirstlane((g - groups) >> 31);
        const int r0 = min(4 * g, n - 4);
        const bool in1 = SEGMENTS && r0 >= n0, in2 = SEGMENTS && r0 >= n01;
        const uint8_t *base = w0 + (in1 ? d01 : 0) + (in2 ? d12 : 0);
        if (DUAL) base = (t & 1) ? wd : w0;
        const int local = r0 - (in1 ? n0 : 0) - (in2 ? n01 - n0 : 0);
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, extent, 0x00020000);
        U::load(dst, rs, off, (uint32_t)local * (uint32_t)rowbytes);
    };
#pragma unroll
    for (int i = 0; i < NB; ++i) fill(buf[i], i);
    __builtin_amdgcn_sched_barrier(0);  // the weight loads leave before anything waits for the activations
    {
        auto keep = [](float4 &v, uint32_t m) {  // (a mask, not a branch)
            v.x = __uint_as_float(__float_as_uint(v.x) & m); v.y = __uint_as_float(__float_as_uint(v.y) & m);
            v.z = __uint_as_float(__float_as_uint(v.z) & m); v.w = __uint_as_float(__float_as_uint(v.w) & m);
        };
#pragma unroll
        for (int r = 0; r < B; ++r) {
            const uint32_t m = inrow && (B == 1 || rb + r < ld.rows) ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < 4; ++i) keep(xv[r][i], m);
        }
        if (NORM) {
#pragma unroll
            for (int i = 0; i < 4; ++i) keep(nv[i], inrow ? 0xffffffffu : 0u);
        }
    }

    if (NORM) {
        // RMSNorm (ops/RowNorm.java:286-306): y = W (x * nw / sqrt(mean(x^2) + eps)).  The factor 1 / sqrt(...) is one number for the
        // whole vector, so it multiplies the outputs instead of the inputs: the activations go to fixed point as x * nw without
        // waiting for a workgroup-wide reduction, and the sum of squares (one partial per wave, in LDS) is only read after the
        // barrier that precedes the first outputs anyway.
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) ss += (xv[0][i].x * xv[0][i].x + xv[0][i].y * xv[0][i].y) + (xv[0][i].z * xv[0][i].z + xv[0][i].w * xv[0][i].w);
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            xv[0][i] = make_float4(xv[0][i].x * nv[i].x, xv[0][i].y * nv[i].y, xv[0][i].z * nv[i].z, xv[0][i].w * nv[i].w);
    }

    // ---- fixed point, row by row
    uint32_t xa[B][16];
    float sinv[B], sums[B][U::NSUM];
    bool slow = false;
    if constexpr (B == 4) {
        // (four rows: every row's planes into a region of its own, then the lane's three packed operand sets - see i8_dot)
        uint32_t unused[16];
#pragma unroll
        for (int r = 0; r < 4; ++r) slow = i8_stage<U>(xv[r], planes + r * 192, b, j, unused, sinv[r], sums[r]) || slow;
#pragma unroll
        for (int m = 0; m < 3; ++m) {
            const int vec = 4 * m + j, rr = vec / 3, p = vec - 3 * rr;
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const u32x4 v = planes[rr * 192 + (b * 3 + p) * 4 + qd];
                xa[m][qd * 4 + 0] = v.x; xa[m][qd * 4 + 1] = v.y; xa[m][qd * 4 + 2] = v.z; xa[m][qd * 4 + 3] = v.w;
            }
        }
        __builtin_amdgcn_wave_barrier();
    } else {
#pragma unroll
        for (int r = 0; r < B; ++r) slow = i8_stage<U>(xv[r], planes, b, j, xa[r], sinv[r], sums[r]) || slow;  // an Inf or NaN in this wave's slice
    }

    // What the flush needs of the argument block, asked for now: the round trip of the scalar cache runs while the wave would
    // wait for its first weight bytes anyway - fetched where they are first used, it sits between the last product and the
    // first store of every launch.
    asm volatile("" ::"s"(a.y[0]));
    if constexpr (BIAS) asm volatile("" ::"s"(a.bias[0]));
    if constexpr (NORM) asm volatile("" ::"s"(a.eps));
    if constexpr (SEGMENTS) asm volatile("" ::"s"(a.y[1]), "s"(a.y[2]));
    if constexpr (SEGMENTS && BIAS) asm volatile("" ::"s"(a.bias[1]), "s"(a.bias[2]));
    auto group_of = [&](int t) { return bid + (DUAL ? t >> 1 : t) * nblocks; };
    // one output of a window: the partial sums of all waves in wave order
    // (all reads issued before the first addition - a loop over the workgroup's actual number of waves waits for every wave's four
    // values in turn, 0.6 us at the end of a 14-wave workgroup; waves the workgroup does not have add zeros)
    auto joined = [&](int half, int tt, int r, int jj) {
        float part[MAXW];
#pragma unroll
        for (int w = 0; w < MAXW; ++w) {
            const float *p = reinterpret_cast<const float *>(i8_smem + (size_t)min(w, waves - 1) * WAVE_LDS) + ((half * FL + tt) * B + r) * 16 + jj;
            const float v = (p[0] + p[4]) + (p[8] + p[12]);
            part[w] = w < waves ? v : 0.f;
        }
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < MAXW; ++w) sum += part[w];
        return sum;
    };

    // a turn's partial sums of this wave: fold the sixteen chunks of every row (lanes 4b + j, b = 0..15) to four per row
    auto emit = [&](float acc, int half, int tt, int r) {
        if (!inrow) acc = 0.f;
        acc += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc), 0x114, 0xF, 0xF, true));  // row_shr:4
        acc += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc), 0x118, 0xF, 0xF, true));  // row_shr:8
        if ((lane & 15) >= 12) mypart[((half * FL + tt) * B + r) * 16 + (lane >> 4) * 4 + j] = acc;
    };

    for (int t0 = 0, half = 0; t0 < vturns; t0 += FL, half ^= 1) {
        const int tend = min(t0 + FL, vturns);
        if (!slow) {
#pragma unroll 1
            for (int tb = t0; tb < tend; tb += NB) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int t = tb + i;
                    if (t < tend && group_of(t) < groups) {  // wave-uniform
                        float acc[B];
                        i8_dot<U, B>(buf[i], c, xa, sinv, sums, acc);
#pragma unroll
                        for (int r = 0; r < B; ++r) emit(acc[r], half, t - t0, r);
                    }
                    fill(buf[i], t + NB);
                }
            }
        } else {
            // an activation of this slice is not finite: every weight by the dequantiser's own code, FP32 products, straight
            // from memory (four values at a time, in the order the operands have them)
#pragma unroll 1
            for (int t = t0; t < tend; ++t) {
                const int g = group_of(t);
                if (g >= groups) continue;
                const int row = min(4 * g, n - 4) + j;
                const bool in1 = SEGMENTS && row >= n0, in2 = SEGMENTS && row >= n01;
                const uint8_t *rp = (DUAL ? ((t & 1) ? wd : w0) : w0 + (in1 ? d01 : 0) + (in2 ? d12 : 0)) +
                                    (size_t)(row - (in1 ? n0 : 0) - (in2 ? n01 - n0 : 0)) * rowbytes;
#pragma unroll 1
                for (int r = 0; r < B; ++r) {
                    float acc = 0.f;
                    if (B == 1 || rb + r < ld.rows) {
#pragma unroll 1
                        for (int e = 0; e < 64; e += 4) {
                            const int p = U::x_pos(c, e);
                            const float4 w4 = dequant4<FMT>(rp, (size_t)p);
                            float4 x4 = *reinterpret_cast<const float4 *>(ld.x + (size_t)(rb + r) * k + p);
                            if (NORM) {
                                const float4 n4 = *reinterpret_cast<const float4 *>(ld.nw + p);
                                x4 = make_float4(x4.x * n4.x, x4.y * n4.y, x4.z * n4.z, x4.w * n4.w);
                            }
                            acc = __builtin_fmaf(w4.x, x4.x, acc);
                            acc = __builtin_fmaf(w4.y, x4.y, acc);
                            acc = __builtin_fmaf(w4.z, x4.z, acc);
                            acc = __builtin_fmaf(w4.w, x4.w, acc);
                        }
                    }
                    emit(acc, half, t - t0, r);
                }
            }
        }
        __syncthreads();  // (one barrier per window: the next window writes the other half of the partial-sum area)
        float nscale = 1.f;
        if (NORM) {
            float tot = 0.f;
            for (int w = 0; w < waves; ++w) tot += red[w];
            nscale = 1.f / sqrtf(tot / (float)k + a.eps);
        }
        const int outs = DUAL ? 2 * (tend - t0) : 4 * B * (tend - t0);
        for (int o = tid; o < outs; o += 64 * waves) {  // (a one-wave workgroup has fewer threads than a window has outputs)
            if (DUAL) {
                const int pr = o >> 2, jj = o & 3;
                const int g = group_of(t0 + 2 * pr), row = min(4 * g, n - 4) + jj;
                if (g < groups && row >= 4 * g) {
                    const float gate = joined(half, 2 * pr, 0, jj) * nscale, up = joined(half, 2 * pr + 1, 0, jj) * nscale;
                    a.y[0][row] = (gate / (1.f + __expf(-gate))) * up;
                }
            } else {
                const int jj = o & 3, r = (o >> 2) % B, tt = (o >> 2) / B;
                const int g = group_of(t0 + tt), row = min(4 * g, n - 4) + jj;
                if (g < groups && row >= 4 * g && (B == 1 || rb + r < ld.rows)) {
                    // (segment pointers by differences, as in fill: no dependent load from the argument block on the way out)
                    const bool in1 = SEGMENTS && row >= n0, in2 = SEGMENTS && row >= n01;
                    const int local = row - (in1 ? n0 : 0) - (in2 ? n01 - n0 : 0);
                    float *const yp = a.y[0] + (in1 ? a.y[1] - a.y[0] : 0) + (in2 ? a.y[2] - a.y[1] : 0);
                    float bias = 0.f;
                    if (BIAS) bias = (a.bias[0] + (in1 ? a.bias[1] - a.bias[0] : 0) + (in2 ? a.bias[2] - a.bias[1] : 0))[local];
                    const float sum = NORM ? joined(half, tt, r, jj) * nscale : joined(half, tt, r, jj);
                    yp[(size_t)(rb + r) * n + local] = BIAS ? sum + bias : sum;
                }
            }
        }
    }
}

// The leading arguments (I8Lead) are what a wave needs before its first loads can leave - the library is built with kernel-argument
// preloading, which hands them to the wave in scalar registers at its start; what the flush needs of `a` (outputs, biases) is
// fetched under the wait for the first weights.
// (the fused forms - norm, SwiGLU pair, row segments - take all fourteen dwords; a plain or biased launch the six it uses: every
// preloaded dword is written into every wave's registers at its start, and the headline launch ran 0.15 us longer with fourteen)
template <class U, int B, int PF, bool BIAS, bool NORM, bool DUAL, int MAXW>
__global__ void __launch_bounds__(64 * MAXW, (B > 1 ? 2 : 4)) gemv_i8_kernel(const uint8_t *w0, const float *x, const uint8_t *wb, const float *nw, const uint8_t *wc,
                                                                             const uint32_t packed, const int n, const int n0, const int n1, const I8Args a) {
    static_assert(NORM, "the fused forms");
    const I8Lead ld{w0, x, wb, nw, wc, (int)(packed & 511u) << 6, (int)((packed >> 9) & 0xfffffu), (int)(packed >> 29) + 1, n, n0, n1};
    gemv_i8_body<U, B, PF, BIAS, NORM, DUAL, MAXW>(ld, a, blockIdx.x, B * (int)blockIdx.y);
}
template <class U, int B, int PF, bool BIAS, int MAXW>
__global__ void __launch_bounds__(64 * MAXW, (B > 1 ? 2 : 4)) gemv_i8_plain_kernel(const uint8_t *w0, const float *x, const uint32_t packed, const int n, const I8Args a) {
    const I8Lead ld{w0, x, w0, nullptr, w0, (int)(packed & 511u) << 6, (int)((packed >> 9) & 0xfffffu), (int)(packed >> 29) + 1, n, n, 0};
    gemv_i8_body<U, B, PF, BIAS, false, false, MAXW>(ld, a, blockIdx.x, B * (int)blockIdx.y);
}

// Two sets of matrices in two formats over the same (normalised) activations in one launch - the q / k and the v
// projections of a Q4_K_M layer: workgroups below `split` run the first set (one or two row segments: wa, wa1 with na0 and
// na - na0 rows), the others the second (one matrix).  packed: k / 64 (9 bits) | split (11 bits) | workgroups (12 bits).
template <class UA, class UB, int PF, int MAXW>
__global__ void __launch_bounds__(64 * MAXW, 4) gemv_i8_pair_kernel(const uint8_t *wa, const uint8_t *wa1, const uint8_t *wb, const float *x, const float *nw,
                                                                    const uint32_t packed, const int na, const int na0, const int nb, const I8Args a, const I8Args b) {
    const int k = (int)(packed & 511u) << 6, split = (int)((packed >> 9) & 2047u), total = (int)(packed >> 20);
    if ((int)blockIdx.x < split) gemv_i8_body<UA, 1, PF, false, true, false, MAXW>(I8Lead{wa, x, wa1, nw, wa1, k, split, 1, na, na0, na - na0}, a, blockIdx.x);
    else gemv_i8_body<UB, 1, PF, false, true, false, MAXW>(I8Lead{wb, x, wb, nw, wb, k, total - split, 1, nb, nb, 0}, b, blockIdx.x - split);
}

}  // namespace jitnn
