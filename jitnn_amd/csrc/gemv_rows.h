// 2..64 activation rows against raw GGUF blocks in ONE pass over the weights, on the matrix cores, at FP32-grade accuracy.
//
// gemv_mfma_kernel (gemv_mfma.h) takes at most eight rows per pass and spends most of its instructions on things that
// do not depend on the weights' bytes: it rebuilds the activation operands in every workgroup and applies the block
// scales to every 4 x 16 block sum in FP32.  This kernel family moves both out of the way:
//   * rows_prepare_kernel builds the activation operands once per call: per group of eight rows and 256-value column of
//     K, the rows scaled by a power of two (from the column's largest magnitude per row) and split into two FP16 parts,
//     x 2^e = hi + lo, written in matrix-core operand order (hi and lo of a row in neighbouring operand rows, so that
//     their block sums meet in one lane) together with the column's block sums of x (per 32 values, or per 16 for Q6_K)
//     and the inverse scales - once per activation, for every weight that meets it.  The main kernel streams them from
//     L2: one 16-byte load per lane and operand.
//   * the block scales are folded into the weight operand where that is exact: a Q4_K / Q5_K quant times its 6-bit
//     scale is an integer below 2048, so sc * q is an FP16 value without rounding, and the matrix core accumulates the
//     eight sub-blocks of a super-block in one FP32 chain; only the super-block's d and dmin (and the activation scale)
//     meet the sums in FP32, once per 16 x 256 tile instead of once per block.  The conversion costs what the plain one
//     did: (1024 + q) * sc - 1024 * sc is one packed FMA on the pattern 0x6400 | q.  Q6_K's int8 scale times 6-bit quant
//     is not an FP16 integer, but its two parts are (RTile<F_Q6_K>): two operands per 32-value step.  The 32-value formats
//     have FP16 block scales, nothing folds: their operands are the quants, and each block's sum meets its d in FP32.
// A workgroup of eight waves owns tiles of 16 weight rows; wave w walks the 256-value columns w, w + 8, ... of K for the
// workgroup's tiles, T tiles at a time: it fetches the tiles' bytes of a column sixteen bytes a lane, parts them through
// a stage of its own in LDS (RStaged), turns them into operands once, and runs them against every group of eight
// activation rows.  Partial sums live in LDS per lane (the group index is a run-time value) and are added across the
// eight waves in wave order at the end of a tile batch: a fixed summation order, no atomics.  A launch with few tiles
// puts several workgroups on a batch, each with a share of the groups (gridDim.y).
#pragma once
#include "common.h"
#include "gemv_mfma.h"

namespace jitnn {

constexpr int GR_WAVES = 8, GR_THREADS = GR_WAVES * 64;
constexpr int GR_MAX_GROUPS = 8;            // groups of eight activation rows: up to 64 rows
constexpr int GR_OP_HALVES = 9 * 512;       // per (group, column): eight sub-block operands and the block-sum operand, 64 lanes x 8 halves each
constexpr int GR_T_MAX = 2;             // weight tiles a wave holds as operands at a time, at most (the kernel's parameter T)

__host__ __device__ constexpr size_t gemv_rows_ops_bytes(int groups, int k) { return (size_t)groups * (k / 256) * GR_OP_HALVES * 2; }
__host__ __device__ constexpr size_t gemv_rows_inv_bytes(int groups, int k) { return (size_t)groups * (k / 256) * 8 * sizeof(float); }
__host__ __device__ constexpr size_t gemv_rows_lds_bytes(int tiles_per_wave) { return (size_t)tiles_per_wave * GR_MAX_GROUPS * GR_THREADS * sizeof(float2); }

// One wave per (group g = blockIdx.y, column c = blockIdx.x): x [rows, k] -> operands.
// Operand s < 8 (sub-block s of the column): lane m + 16 kq holds, for operand row m = 2 b + part (b = activation row of
// the group, part 0 = hi, 1 = lo), the eight values 8 kq .. 8 kq + 7 of the sub-block in the order 0 2 1 3 4 6 5 7 - the
// order in which the weight decoders emit the bytes of a dword.  Operand 8, GS == 32: rows as above, slot j of the lanes
// kq = 0 = sum of sub-block j of the scaled row / 64, the other lanes zero.  GS == 16 (Q6_K, whose scales cover 16 values):
// slot j of the lanes kq = 0 and slot j - 8 of the lanes kq = 1 = sum of the 16-value group j / 64, sixteen groups.
// HALVES (the 4-bit 32-value formats, whose byte i holds values i and i + 16 of a block): lane group kq holds values
// 4 kq .. 4 kq + 3 and 16 + 4 kq .. + 3 of the sub-block instead of 8 kq .. 8 kq + 7, each four in the order 0 2 1 3.
// The work of one wave: column c of group g, the lane's eight quads v of its row already loaded (and normalised / gated).
template <int GS, bool HALVES>
__device__ __forceinline__ void rows_prepare_column(const float4 (&v)[8], _Float16 *__restrict__ ops, float *__restrict__ inv, int c, int g, int ncol,
                                                    bool have, int lane) {
    const int b = lane >> 3, part = lane & 7;
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
    if (!have) scale = 0.f;
    uint8_t *base = reinterpret_cast<uint8_t *>(ops + ((size_t)g * ncol + c) * GR_OP_HALVES);
    const int kq = HALVES ? part & 3 : part >> 1, h = HALVES ? part >> 2 : part & 1;  // the quad `part` of a sub-block: lane group and half of its eight slots
    float sm = 0.f, sm2 = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const float a0 = v[t].x * scale, a1 = v[t].z * scale, a2 = v[t].y * scale, a3 = v[t].w * scale;
        const float qs = (a0 + a1) + (a2 + a3);
        if constexpr (GS == 32) {
            const float bs = group_sum<8>(qs);  // sub-block t of row b: its eight quads sit in the eight lanes of b
            sm = part == t ? bs : sm;
        } else {
            // the two 16-value groups 2 t and 2 t + 1 of the sub-block: quads 0..3 and 4..7; lane `part` keeps groups
            // `part` and `part` + 8
            const float lo = group_sum<8>(part < 4 ? qs : 0.f), hi = group_sum<8>(part < 4 ? 0.f : qs);
            const float mine = (part & 1) ? hi : lo;
            sm = (part >> 1) == t ? mine : sm;
            sm2 = 4 + (part >> 1) == t ? mine : sm2;
        }
        const h2raw h01 = __builtin_amdgcn_cvt_pkrtz(a0, a1), h23 = __builtin_amdgcn_cvt_pkrtz(a2, a3);
        const h2raw l01 = __builtin_amdgcn_cvt_pkrtz(a0 - (float)h01.x, a1 - (float)h01.y);
        const h2raw l23 = __builtin_amdgcn_cvt_pkrtz(a2 - (float)h23.x, a3 - (float)h23.y);
        *reinterpret_cast<u32x2 *>(base + t * 1024 + (2 * b + 16 * kq) * 16 + 8 * h) = u32x2{__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23)};
        *reinterpret_cast<u32x2 *>(base + t * 1024 + (2 * b + 1 + 16 * kq) * 16 + 8 * h) = u32x2{__builtin_bit_cast(uint32_t, l01), __builtin_bit_cast(uint32_t, l23)};
    }
    // the block sums: scaled by 1/64 (a sum of 32 values below 2^14 stays below 2^13), hi / lo like the values
    sm *= 0.015625f;
    const _Float16 shi = (_Float16)sm, slo = (_Float16)(sm - (float)shi);
    _Float16 *sop = reinterpret_cast<_Float16 *>(base + 8 * 1024);
    if (lane >= (GS == 32 ? 16 : 32)) *reinterpret_cast<u32x4 *>(base + 8 * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
    sop[(2 * b) * 8 + part] = shi;
    sop[(2 * b + 1) * 8 + part] = slo;
    if constexpr (GS == 16) {
        sm2 *= 0.015625f;
        const _Float16 thi = (_Float16)sm2, tlo = (_Float16)(sm2 - (float)thi);
        sop[(16 + 2 * b) * 8 + part] = thi;
        sop[(16 + 2 * b + 1) * 8 + part] = tlo;
    }
    if (part == 0) inv[((size_t)g * ncol + c) * 8 + b] = myinv;
}

// One wave per (column c = blockIdx.x, group g = blockIdx.y): the lane's eight quads of its row, once, into every operand
// layout somebody asked for (weights of several kinds on one activation).  SWIGLU: the rows are silu(x) * up, up [rows, k]
// (F.swiglu, F.java:1159-1161) - the expression of swiglu_kernel.
struct RowsPrepareOut {
    _Float16 *ops[3];  // per layout (plain, sums per 16 values, halves): nullptr = not wanted
    float *inv[3];
};
template <bool SWIGLU>
__global__ void __launch_bounds__(64) rows_prepare_kernel(const float *__restrict__ x, const float *__restrict__ up, int rows, int k,
                                                           const RowsPrepareOut o) {  // (what the first loads need in front: preloaded with the wave)
    const int lane = threadIdx.x, b = lane >> 3, part = lane & 7;
    const int c = blockIdx.x, g = blockIdx.y, ncol = k >> 8;
    const int row = g * 8 + b;
    const bool have = row < rows;
    const size_t at = (size_t)(have ? row : 0) * k + (size_t)c * 256 + 4 * part;
    float4 v[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) v[t] = *reinterpret_cast<const float4 *>(x + at + 32 * t);
    if constexpr (SWIGLU) {
        auto sw = [](float gt, float u) { return (gt / (1.f + __expf(-gt))) * u; };
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float4 u = *reinterpret_cast<const float4 *>(up + at + 32 * t);
            v[t] = make_float4(sw(v[t].x, u.x), sw(v[t].y, u.y), sw(v[t].z, u.z), sw(v[t].w, u.w));
        }
    }
    if (o.ops[0]) rows_prepare_column<32, false>(v, o.ops[0], o.inv[0], c, g, ncol, have, lane);
    if (o.ops[1]) rows_prepare_column<16, false>(v, o.ops[1], o.inv[1], c, g, ncol, have, lane);
    if (o.ops[2]) rows_prepare_column<32, true>(v, o.ops[2], o.inv[2], c, g, ncol, have, lane);
}

// Per format: the bytes a lane (weight row n = lane & 15 of the tile, lane group kq = lane >> 4) fetches of a 256-value
// column of its row, and their operands with the block scales folded in.
template <int FMT>
struct RTile;

__device__ __forceinline__ f16x2 h2fma(uint32_t bits, f16x2 mul, f16x2 add) { return __builtin_elementwise_fma(as_h2(bits), mul, add); }

// How a wave gets a tile's bytes of a column (16 rows x BYTES).  A lane needs a few bytes of every field of its row's
// block; fetched like that - each load instruction touching sixteen lines for 4 or 8 bytes a lane - the launch is bound by
// the requests, not the bytes (14336 x 4096 Q4_0 at 9 rows: 46 us with sixteen narrow loads per tile and column, 27 us as
// below).  So the wave fetches the bytes once, sixteen a lane (four chunks of a row per lane quad and load, the odd chunks
// in a last load), parks them in LDS of its own and every lane picks its pieces there.
// CHUNKS * 16 <= BYTES bytes of a row go this way (a format fetches a tail of its own); STRIDE: of a row in LDS, a
// multiple of 16 and 4 * odd dwords where that is free (sixteen rows x four lane groups then hit 64 different banks).
template <int ROW_BYTES, int ROW_STRIDE, int ALIGN>
struct RStaged {
    static constexpr int BYTES = ROW_BYTES;
    static constexpr int CHUNKS = BYTES / 16, FULL = CHUNKS / 4, REST = CHUNKS % 4;
    static constexpr int STRIDE = ROW_STRIDE;
    static constexpr int STAGE_BYTES = 16 * STRIDE;
    static constexpr bool STAGED = true;
    static constexpr int RD = REST > 0 ? REST : 1;  // (a row of whole four-chunk loads has no load of odd chunks)
    static_assert(STRIDE >= 16 * CHUNKS && STRIDE % 16 == 0, "chunks of sixteen bytes");
    struct Raw {
        u32x4 c[FULL + (REST > 0 ? 1 : 0)];
        uint32_t tail;  // (formats with bytes past the chunks)
    };
    struct Ptr {
        const uint8_t *full;  // the lane's four-chunk loads
        int rest, row;        // from there to its load of the odd chunks, and to the row lane & 15 (rows of a tile are < 2 GiB apart)
    };
    // r0: first row of the tile
    __device__ static __forceinline__ Ptr ptr(const uint8_t *W, int r0, size_t rowbytes, int lane) {
        const int rb = (int)rowbytes, lr = lane >> 2;
        return {W + (size_t)(r0 + lr) * rowbytes + 16 * (lane & 3), (((lane / RD) & 15) - lr) * rb + 16 * (4 * FULL + lane % RD - (lane & 3)),
                ((lane & 15) - lr) * rb - 16 * (lane & 3)};
    }
    __device__ static __forceinline__ void load(Raw &r, const Ptr &p, int c) {
        const uint8_t *q = p.full + (size_t)c * BYTES;
#pragma unroll
        for (int i = 0; i < FULL; ++i) r.c[i] = ld128<ALIGN>(q + 64 * i);
        if constexpr (REST > 0) r.c[FULL] = ld128<ALIGN>(q + p.rest);  // (lanes past 16 REST repeat rows: the same lines)
    }
    // -> this lane's row (lane & 15 of the tile) in the wave's stage
    __device__ static __forceinline__ const uint8_t *park(const Raw &r, uint8_t *stage, int lane) {
#pragma unroll
        for (int i = 0; i < FULL; ++i) *reinterpret_cast<u32x4 *>(stage + (lane >> 2) * STRIDE + 16 * (lane & 3) + 64 * i) = r.c[i];
        if constexpr (REST > 0) {
            if (lane < 16 * REST) *reinterpret_cast<u32x4 *>(stage + (lane / RD) * STRIDE + 16 * (4 * FULL + lane % RD)) = r.c[FULL];
        }
        // the lanes of a wave run in step and LDS serves them in order: a fence for the compiler is all this needs
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        return stage + (lane & 15) * STRIDE;
    }
};

template <>
struct RTile<F_Q4_K> : RStaged<144, 144, 16> {
    static constexpr int NOPS = 8, SUMS = 32;  // weight operands per tile and column, values per block sum
    static constexpr bool BLOCK_SCALES = false, HALVES = false, MINS = true;
    __device__ static constexpr int aidx(int q) { return q; }  // the activation operand weight operand q meets
    struct Fields {
        u32x4 h;
        u32x2 q[4];
    };
    // B[s]: sc_s * q of sub-block s; Bm: the eight mins in the first eight K slots; d, dmin of the super-block
    __device__ static __forceinline__ void decode(const Raw &raw, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float &d, float &dmin) {
        const uint8_t *p = park(raw, stage, lane);
        const int kq = lane >> 4;
        Fields r;
        r.h = *reinterpret_cast<const u32x4 *>(p);
#pragma unroll
        for (int c = 0; c < 4; ++c) r.q[c] = *reinterpret_cast<const u32x2 *>(p + 16 + 32 * c + 8 * kq);
        const K4Scales k = k4_scales(r.h);
        d = k.d;
        dmin = k.dmin;
        const uint32_t mg = magic1024();
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const f16x2 ml = splat2(k.sc[2 * c]), al = splat2(-1024.f * k.sc[2 * c]);
            const f16x2 mh = splat2(0.0625f * k.sc[2 * c + 1]), ah = splat2(-64.f * k.sc[2 * c + 1]);
            const uint32_t w0 = r.q[c].x, w1 = r.q[c].y, s0 = w0 >> 8, s1 = w1 >> 8;
            B[2 * c] = cat8(h2fma((w0 & 0x000f000fu) | mg, ml, al), h2fma((s0 & 0x000f000fu) | mg, ml, al), h2fma((w1 & 0x000f000fu) | mg, ml, al),
                            h2fma((s1 & 0x000f000fu) | mg, ml, al));
            B[2 * c + 1] = cat8(h2fma((w0 & 0x00f000f0u) | mg, mh, ah), h2fma((s0 & 0x00f000f0u) | mg, mh, ah), h2fma((w1 & 0x00f000f0u) | mg, mh, ah),
                                h2fma((s1 & 0x00f000f0u) | mg, mh, ah));
        }
        Bm = cat8(bytes2(k.mnA, 0), bytes2(k.mnA, 16), bytes2(k.mnB, 0), bytes2(k.mnB, 16));
    }
};

template <>
struct RTile<F_Q5_K> : RStaged<176, 176, 16> {
    static constexpr int NOPS = 8, SUMS = 32;
    static constexpr bool BLOCK_SCALES = false, HALVES = false, MINS = true;
    __device__ static constexpr int aidx(int q) { return q; }
    struct Fields {
        u32x4 h;
        u32x2 qh;
        u32x2 q[4];
    };
    __device__ static __forceinline__ void decode(const Raw &raw, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float &d, float &dmin) {
        const uint8_t *p = park(raw, stage, lane);
        const int kq = lane >> 4;
        Fields r;
        r.h = *reinterpret_cast<const u32x4 *>(p);
        r.qh = *reinterpret_cast<const u32x2 *>(p + 16 + 8 * kq);
#pragma unroll
        for (int c = 0; c < 4; ++c) r.q[c] = *reinterpret_cast<const u32x2 *>(p + 48 + 32 * c + 8 * kq);
        const K4Scales k = k4_scales(r.h);
        d = k.d;
        dmin = k.dmin;
        const uint32_t mg = magic1024();
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const f16x2 ml = splat2(k.sc[2 * c]), al = splat2(-1024.f * k.sc[2 * c]);
            const f16x2 mh = splat2(0.0625f * k.sc[2 * c + 1]), ah = splat2(-64.f * k.sc[2 * c + 1]);
            f16x2 lo[4], hi[4];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t w = t ? r.q[c].y : r.q[c].x, qh = t ? r.qh.y : r.qh.x, s = w >> 8, qs = qh >> 8;
                // fifth bit of sub-block 2c (2c + 1): bit 2c (2c + 1) of the qh byte at the same position
                lo[2 * t] = h2fma((w & 0x000f000fu) | (((qh >> (2 * c)) & 0x00010001u) << 4) | mg, ml, al);
                lo[2 * t + 1] = h2fma((s & 0x000f000fu) | (((qs >> (2 * c)) & 0x00010001u) << 4) | mg, ml, al);
                hi[2 * t] = h2fma((w & 0x00f000f0u) | (((qh >> (2 * c + 1)) & 0x00010001u) << 8) | mg, mh, ah);
                hi[2 * t + 1] = h2fma((s & 0x00f000f0u) | (((qs >> (2 * c + 1)) & 0x00010001u) << 8) | mg, mh, ah);
            }
            B[2 * c] = cat8(lo[0], lo[1], lo[2], lo[3]);
            B[2 * c + 1] = cat8(hi[0], hi[1], hi[2], hi[3]);
        }
        Bm = cat8(bytes2(k.mnA, 0), bytes2(k.mnA, 16), bytes2(k.mnB, 0), bytes2(k.mnB, 16));
    }
};

// Q6_K: 210 bytes = ql[128] (low nibbles), qh[64] (two high bits), 16 int8 scales of 16 values each, d.  Value 128 n + 32 ty
// + l (n < 2, ty < 4, l < 32) is nibble ty / 2 of ql[64 n + 32 (ty & 1) + l] with bits 2 ty, 2 ty + 1 of qh[32 n + l] on top,
// minus 32; its scale is number 8 n + 2 ty + l / 16.  The 32-value step s = 4 n + ty of the matrix core takes l = 8 kq .. + 7
// from lane group kq - one scale per lane and step.  An int8 scale times a 6-bit quant (up to 8001) is not an FP16 integer,
// but the quant is 16 a + b with sc * b <= 1905 and sc * 16 a a multiple of 16 below 6100: two exact operands per step,
// both against the same activation operand; the -32 meets the sums of x per 16 values (operand 8 of
// rows_prepare_kernel<16>) as 32 * sc, a multiple of 32 below 4100.
template <>
struct RTile<F_Q6_K> : RStaged<210, 208, 2> {
    static constexpr int NOPS = 16, SUMS = 16;
    static constexpr bool BLOCK_SCALES = false, HALVES = false, MINS = true;
    __device__ static constexpr int aidx(int q) { return q >> 1; }  // operands 2 s (low nibble part) and 2 s + 1 (high bits) of step s
    struct Fields {
        u32x2 ql[4];  // [2 n + (ty & 1)]: bytes 64 n + 32 (ty & 1) + 8 kq .. + 7
        u32x2 qh[2];  // [n]: bytes 32 n + 8 kq .. + 7
        u32x4 sc;
    };
    // thirteen chunks and d, the last two bytes of the block, straight to the lanes of its row
    __device__ static __forceinline__ void load(Raw &r, const Ptr &p, int c) {
        RStaged<210, 208, 2>::load(r, p, c);
        r.tail = ld16(p.full + (size_t)c * BYTES + p.row + 208);
    }
    __device__ static __forceinline__ void decode(const Raw &raw, uint8_t *stage, int lane, f16x8 (&B)[16], f16x8 &Bm, float &d, float &dmin) {
        const uint8_t *p = park(raw, stage, lane);
        Fields r;
        {
            const int kq = lane >> 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) r.ql[i] = *reinterpret_cast<const u32x2 *>(p + 32 * i + 8 * kq);
#pragma unroll
            for (int n = 0; n < 2; ++n) r.qh[n] = *reinterpret_cast<const u32x2 *>(p + 128 + 32 * n + 8 * kq);
            r.sc = *reinterpret_cast<const u32x4 *>(p + 192);
        }
        d = h2f(raw.tail);
        dmin = d;  // the offset term is 32 * sc per group: y += d * (sum sc q x - 32 sum sc S)
        // FP16 64 + b with b in bits 4..7 of a half-word, 16 + a with a in bits 6, 7 (1024 + b, as the 6-bit scales of Q4_K
        // allow, would overflow: 1024 * 128)
        const uint32_t mgb = 0x54005400u, mga = 0x4c004c00u;
        const int kq = (int)(threadIdx.x >> 4) & 3;
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int ty = 0; ty < 4; ++ty) {
                // the scale of this lane's eight values of the step: number 8 n + 2 ty + kq / 2
                const int is0 = 8 * n + 2 * ty;  // even (a constant, the loops being unrolled): is0 and is0 + 1 share a dword of the scales
                const float scf = (float)(int)(int8_t)(r.sc[is0 >> 2] >> (8 * ((is0 & 3) + (kq >> 1))));
                const f16x2 mb = splat2(scf), ab = splat2(-64.f * scf);           // (64 + b) sc - 64 sc
                const f16x2 ma = splat2(16.f * scf), aa = splat2(-256.f * scf);   // (16 + a) 16 sc - 256 sc
                const u32x2 lw = r.ql[2 * n + (ty & 1)], hw = r.qh[n];
                f16x2 lo[4], hi[4];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t w = t ? lw.y : lw.x, h = t ? hw.y : hw.x;
                    // the nibble (low for ty < 2, high for the others) of bytes 0, 2 (1, 3) to bits 4..7 of the half-words
                    const uint32_t w02 = ty < 2 ? w << 4 : w, w13 = ty < 2 ? w >> 4 : w >> 8;
                    lo[2 * t] = h2fma((w02 & 0x00f000f0u) | mgb, mb, ab);
                    lo[2 * t + 1] = h2fma((w13 & 0x00f000f0u) | mgb, mb, ab);
                    // bits 2 ty, 2 ty + 1 of bytes 0, 2 (1, 3) to bits 6, 7 of the half-words
                    const uint32_t h02 = 2 * ty <= 6 ? h << (6 - 2 * ty) : h, h13 = h >> (2 + 2 * ty);
                    hi[2 * t] = h2fma((h02 & 0x00c000c0u) | mga, ma, aa);
                    hi[2 * t + 1] = h2fma((h13 & 0x00c000c0u) | mga, ma, aa);
                }
                B[2 * (4 * n + ty)] = cat8(lo[0], lo[1], lo[2], lo[3]);
                B[2 * (4 * n + ty) + 1] = cat8(hi[0], hi[1], hi[2], hi[3]);
            }
        // operand of the offsets: slot j of the lanes kq = 0 (1) = 32 * scale j (j + 8); the other lanes zero
        const uint32_t s0 = kq == 0 ? r.sc.x : r.sc.z, s1 = kq == 0 ? r.sc.y : r.sc.w;
        f16x2 m[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t sw = j < 2 ? s0 : s1;
            const float e0 = (float)(int)(int8_t)(sw >> (16 * (j & 1))), e1 = (float)(int)(int8_t)(sw >> (16 * (j & 1) + 8));
            m[j] = kq < 2 ? f16x2{(_Float16)(32.f * e0), (_Float16)(32.f * e1)} : f16x2{(_Float16)0.f, (_Float16)0.f};
        }
        Bm = cat8(m[0], m[1], m[2], m[3]);
    }
};

// The 32-value formats: a 256-value column of a row is eight blocks, each with an FP16 scale d of its own (and an FP16
// offset m for Q4_1).  d times a quant is not an FP16 value, so nothing is folded: the operands are the quants as small
// integers, the eight steps of a column keep eight separate sums, and each meets its block's d in FP32 (BLOCK_SCALES) -
// what gemv_mfma_kernel does too, but once for all groups of activation rows.
template <>
struct RTile<F_Q4_0> : RStaged<8 * 18, 144, 2> {
    static constexpr int NOPS = 8, SUMS = 32;
    static constexpr bool BLOCK_SCALES = true, HALVES = true, MINS = false;
    __device__ static __forceinline__ void decode(const Raw &r, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float (&dblk)[8]) {
        const uint8_t *row = park(r, stage, lane);
        const int kq = lane >> 4;
        const uint32_t mg = magic1024();
        const f16x2 off = splat2(-1032.f);  // -1024 of the exponent trick, -8 of the format
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t w = ld32<2>(row + 18 * s + 2 + 4 * kq);
            // bytes 4 kq .. + 3: low nibbles = values 4 kq + (0 2 | 1 3), high nibbles = values 16 + 4 kq + (0 2 | 1 3)
            B[s] = cat8(as_h2((w & 0x000f000fu) | mg) + off, as_h2(((w >> 8) & 0x000f000fu) | mg) + off,
                        as_h2(((w >> 4) & 0x000f000fu) | mg) + off, as_h2(((w >> 12) & 0x000f000fu) | mg) + off);
            dblk[s] = h2f(ld16(row + 18 * s));
        }
        Bm = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
};

template <>
struct RTile<F_Q4_1> : RStaged<8 * 20, 176, 4> {
    static constexpr int NOPS = 8, SUMS = 32;
    static constexpr bool BLOCK_SCALES = true, HALVES = true, MINS = true;
    __device__ static __forceinline__ void decode(const Raw &r, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float (&dblk)[8]) {
        const uint8_t *row = park(r, stage, lane);
        const int kq = lane >> 4;
        const uint32_t mg = magic1024();
        const f16x2 off = splat2(-1024.f);
        uint32_t dm[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint32_t w = ld32<4>(row + 20 * s + 4 + 4 * kq);
            B[s] = cat8(as_h2((w & 0x000f000fu) | mg) + off, as_h2(((w >> 8) & 0x000f000fu) | mg) + off,
                        as_h2(((w >> 4) & 0x000f000fu) | mg) + off, as_h2(((w >> 12) & 0x000f000fu) | mg) + off);
            dm[s] = ld32<4>(row + 20 * s);
            dblk[s] = h2f(dm[s]);
        }
        // the offsets m of the eight blocks against the block sums of x: slot s of the lanes kq = 0, FP16 as they are
        u32x4 mb;
#pragma unroll
        for (int j = 0; j < 4; ++j) mb[j] = kq == 0 ? (dm[2 * j] >> 16) | (dm[2 * j + 1] & 0xffff0000u) : 0u;
        Bm = __builtin_bit_cast(f16x8, mb);
    }
};

template <>
struct RTile<F_Q8_0> : RStaged<8 * 34, 272, 2> {
    static constexpr int NOPS = 8, SUMS = 32;
    static constexpr bool BLOCK_SCALES = true, HALVES = false, MINS = false;
    __device__ static __forceinline__ void decode(const Raw &r, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float (&dblk)[8]) {
        const uint8_t *row = park(r, stage, lane);
        const int kq = lane >> 4;
        const uint32_t mg = magic1024();
        const f16x2 off = splat2(-1152.f);  // -1024 of the exponent trick, -128 of the sign flip below
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const u32x2 q = ld64<2>(row + 34 * s + 2 + 8 * kq);
            const uint32_t w0 = q.x ^ 0x80808080u, w1 = q.y ^ 0x80808080u;  // int8 + 128: bytes 0 .. 255
            B[s] = cat8(as_h2((w0 & 0x00ff00ffu) | mg) + off, as_h2(((w0 >> 8) & 0x00ff00ffu) | mg) + off,
                        as_h2((w1 & 0x00ff00ffu) | mg) + off, as_h2(((w1 >> 8) & 0x00ff00ffu) | mg) + off);
            dblk[s] = h2f(ld16(row + 34 * s));
        }
        Bm = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
};

// Q5_1: blocks of 24 bytes - d, m, 32 fifth bits (bit i: value i), 16 bytes of nibbles (core/kernels/GgufKernels.java:155-163) -
// are Q4_1 blocks with a bit on top of every nibble: the four bits of a lane's low-nibble values and the four of its
// high-nibble values are spread to a byte each by one multiplication and OR-ed under the exponent with the nibbles.
// Eight blocks of a row are 192 bytes: three whole four-chunk loads.
template <>
struct RTile<F_Q5_1> : RStaged<8 * 24, 208, 16> {
    static constexpr int NOPS = 8, SUMS = 32;
    static constexpr bool BLOCK_SCALES = true, HALVES = true, MINS = true;
    __device__ static __forceinline__ void decode(const Raw &r, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float (&dblk)[8]) {
        const uint8_t *row = park(r, stage, lane);
        const int kq = lane >> 4;
        const uint32_t mg = magic1024();
        const f16x2 off = splat2(-1024.f);
        uint32_t dm[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const u32x2 hd = *reinterpret_cast<const u32x2 *>(row + 24 * s);  // d | m, the fifth bits
            const uint32_t w = *reinterpret_cast<const uint32_t *>(row + 24 * s + 8 + 4 * kq);
            dm[s] = hd.x;
            const uint32_t h = hd.y >> (4 * kq);
            // byte e = the fifth bit of value 4 kq + e (of value 16 + 4 kq + e): four disjoint shifted copies, no carries
            const uint32_t f0 = ((h & 15u) * 0x00204081u) & 0x01010101u, f1 = (((h >> 16) & 15u) * 0x00204081u) & 0x01010101u;
            B[s] = cat8(as_h2((w & 0x000f000fu) | ((f0 & 0x00010001u) << 4) | mg) + off, as_h2(((w >> 8) & 0x000f000fu) | (((f0 >> 8) & 0x00010001u) << 4) | mg) + off,
                        as_h2(((w >> 4) & 0x000f000fu) | ((f1 & 0x00010001u) << 4) | mg) + off,
                        as_h2(((w >> 12) & 0x000f000fu) | (((f1 >> 8) & 0x00010001u) << 4) | mg) + off);
            dblk[s] = h2f(dm[s]);
        }
        u32x4 mb;  // (the offsets m against the block sums of x, as for Q4_1)
#pragma unroll
        for (int j = 0; j < 4; ++j) mb[j] = kq == 0 ? (dm[2 * j] >> 16) | (dm[2 * j + 1] & 0xffff0000u) : 0u;
        Bm = __builtin_bit_cast(f16x8, mb);
    }
};

// Q2_K: 84 bytes = 16 scale bytes (low nibble: scale, high nibble: min, of 16 values each), qs[64] (2-bit quants), d, dmin.
// Value 128 n + 32 j + l is bits 2 j, 2 j + 1 of qs[32 n + l], its scale byte number 8 n + 2 j + l / 16
// (core/kernels/GgufKernels.java:166-175): Q6_K's element order and scale index, with a 4-bit scale (scale times quant at most
// 45: one exact operand per step) and, like Q4_K, minima - against the sums of x per 16 values - under a dmin of their own.
template <>
struct RTile<F_Q2_K> : RStaged<84, 80, 4> {
    static constexpr int NOPS = 8, SUMS = 16;
    static constexpr bool BLOCK_SCALES = false, HALVES = false, MINS = true;
    __device__ static constexpr int aidx(int q) { return q; }
    // five chunks and d | dmin, the last four bytes of the block, straight to the lanes of its row
    __device__ static __forceinline__ void load(Raw &r, const Ptr &p, int c) {
        RStaged<84, 80, 4>::load(r, p, c);
        r.tail = ld32<4>(p.full + (size_t)c * BYTES + p.row + 80);
    }
    __device__ static __forceinline__ void decode(const Raw &raw, uint8_t *stage, int lane, f16x8 (&B)[8], f16x8 &Bm, float &d, float &dmin) {
        const uint8_t *p = park(raw, stage, lane);
        const int kq = lane >> 4;
        const u32x4 sc = *reinterpret_cast<const u32x4 *>(p);
        u32x2 q[2];
#pragma unroll
        for (int n = 0; n < 2; ++n) q[n] = *reinterpret_cast<const u32x2 *>(p + 16 + 32 * n + 8 * kq);
        d = h2f(raw.tail);
        dmin = h2f(raw.tail >> 16);
        const uint32_t mg = magic1024();
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int ty = 0; ty < 4; ++ty) {
                const int is0 = 8 * n + 2 * ty;  // (even: the scale bytes is0 and is0 + 1 share a dword)
                const float scf = (float)((sc[is0 >> 2] >> (8 * ((is0 & 3) + (kq >> 1)))) & 15u);
                const f16x2 ml = splat2(scf), al = splat2(-1024.f * scf);  // (1024 + q) sc - 1024 sc
                f16x2 v[4];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t w = (t ? q[n].y : q[n].x) >> (2 * ty);
                    v[2 * t] = h2fma((w & 0x00030003u) | mg, ml, al);             // bytes 0, 2
                    v[2 * t + 1] = h2fma(((w >> 8) & 0x00030003u) | mg, ml, al);  // bytes 1, 3
                }
                B[4 * n + ty] = cat8(v[0], v[1], v[2], v[3]);
            }
        // operand of the minima: slot j of the lanes kq = 0 (1) = the min of scale byte j (j + 8); the other lanes zero
        const uint32_t s0 = kq == 0 ? sc.x : sc.z, s1 = kq == 0 ? sc.y : sc.w;
        f16x2 m[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t sw = (j < 2 ? s0 : s1) >> (16 * (j & 1));
            m[j] = kq < 2 ? f16x2{(_Float16)(float)((sw >> 4) & 15u), (_Float16)(float)((sw >> 12) & 15u)} : f16x2{(_Float16)0.f, (_Float16)0.f};
        }
        Bm = cat8(m[0], m[1], m[2], m[3]);
    }
};

template <int FMT>
__host__ __device__ constexpr size_t gemv_rows_stage_bytes(int tiles_per_wave) {
    return (size_t)GR_WAVES * tiles_per_wave * RTile<FMT>::STAGE_BYTES;
}

// y[b, row] = sum_k W[row, k] x[b, k] (+ bias[row]) (+ res[b, row]) for b < rows <= 8 * groups; k a multiple of 256, n >= 16.
//   ops / inv: the output of rows_prepare_kernel<RTile<FMT>::SUMS> for the same x.  grid: up to one workgroup per batch of T tiles of 16
//   weight rows (the host caps it at one per compute unit) x shares of the groups of activation rows; GR_THREADS threads;
//   gemv_rows_lds_bytes() + gemv_rows_stage_bytes() of dynamic LDS.
// T = 2 halves the activation-operand traffic per weight byte; T = 1 is for matrices with too few tiles to give every CU a
// workgroup otherwise.
template <int FMT, int T>
__global__ void __launch_bounds__(GR_THREADS) gemv_rows_kernel(const uint8_t *__restrict__ W, const _Float16 *__restrict__ ops,
                                                                const float *__restrict__ inv, int n, int k, int rows, int groups,
                                                                const uint32_t grid,  // gridDim.x | gridDim.y << 16 (an argument, preloaded: gridDim is fetched from a cold block)
                                                                const float *__restrict__ bias, const float *res, float *y) {  // (res may be y)
    // (argument order: the first fourteen dwords arrive in scalar registers with the wave - everything the first loads need; y,
    // which only the last lines use, is asked for here, not between the last product and the first store)
    asm volatile("" ::"s"(y), "s"(res));
    const int grid_x = (int)(grid & 0xffffu), grid_y = (int)(grid >> 16);
    typedef RTile<FMT> R;
    constexpr int NOPS = R::NOPS;
    extern __shared__ __attribute__((aligned(16))) uint8_t gr_smem[];
    float2 *accl = reinterpret_cast<float2 *>(gr_smem);  // [tile t][group g][thread]
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // (staged formats: behind accl, per wave and tile the sixteen rows of the column being decoded)
    uint8_t *stage = gr_smem + gemv_rows_lds_bytes(T) + gemv_rows_stage_bytes<FMT>(T) / GR_WAVES * wave;
    const int ncol = k >> 8, ntiles = (n + 15) >> 4, nbatch = (ntiles + T - 1) / T;
    const size_t rowbytes = (size_t)ncol * R::BYTES;
    // gridDim.y > 1 (matrices with few tiles): workgroup y takes the groups [gper y, gper y + gper) of activation rows - it
    // decodes the same weights as its neighbours and writes whole outputs of its own rows, nothing meets across workgroups
    if (grid_y > 1) {
        const int gper = (groups + grid_y - 1) / grid_y, g0 = (int)blockIdx.y * gper;
        if (g0 >= groups) return;
        ops += (size_t)g0 * ncol * GR_OP_HALVES;
        inv += (size_t)g0 * ncol * 8;
        y += (size_t)8 * g0 * n;
        if (res) res += (size_t)8 * g0 * n;
        rows -= 8 * g0;
        groups = min(gper, groups - g0);
    }

    // this lane's row of each tile of a batch (the last tile of a ragged matrix is the last 16 rows: in bounds, its first
    // rows computed twice, stored once)
    typename R::Ptr sp[T];
    typename R::Raw raw[T];
    auto point = [&](int tb) {
#pragma unroll
        for (int t = 0; t < T; ++t) sp[t] = R::ptr(W, min(min(tb * T + t, ntiles - 1) * 16, n - 16), rowbytes, lane);
    };
    auto fetch = [&](int col) {
#pragma unroll
        for (int t = 0; t < T; ++t) R::load(raw[t], sp[t], col);
    };
    // The bytes of a wave's next column are always on their way while it works on the current one - also across the end
    // of a batch, under the reduction of its sums (128256 x 4096 Q6_K at 9 rows: 215 -> 202 us; a few per cent on matrices
    // of two batches per workgroup).  Not for two tiles of Q6_K, whose 256 registers have no room for the second set of
    // row pointers (4096 x 14336 at 40 rows: 55.1 against 53.3 us with the spills).
    constexpr bool ACROSS = !(FMT == F_Q6_K && T == 2);
    if (ACROSS && (int)blockIdx.x < nbatch && wave < ncol) {
        point(blockIdx.x);
        fetch(wave);
    }
    for (int tb = blockIdx.x; tb < nbatch; tb += grid_x) {
        if (!ACROSS) {
            point(tb);
            if (wave < ncol) fetch(wave);
        }
        bool live[T];
#pragma unroll
        for (int t = 0; t < T; ++t) live[t] = tb * T + t < ntiles;  // workgroup-uniform
        for (int i = tid; i < T * groups * GR_THREADS; i += GR_THREADS) accl[i] = make_float2(0.f, 0.f);
        // (each thread only ever touches its own slots of accl until the final reduction: no barrier needed here)

        for (int c = wave; c < ncol; c += GR_WAVES) {
            f16x8 B[T][NOPS], Bm[T];
            float d[T], dmin64[T];
            float dblk[R::BLOCK_SCALES ? T : 1][8];
#pragma unroll
            for (int t = 0; t < T; ++t) {
                if constexpr (R::BLOCK_SCALES) {
                    R::decode(raw[t], stage + t * R::STAGE_BYTES, lane, B[t], Bm[t], dblk[t]);
                } else {
                    float dm;
                    R::decode(raw[t], stage + t * R::STAGE_BYTES, lane, B[t], Bm[t], d[t], dm);
                    dmin64[t] = dm * 64.f;
                }
            }
            if (c + GR_WAVES < ncol) {
                fetch(c + GR_WAVES);
            } else if (ACROSS && tb + grid_x < nbatch) {  // this batch's last column: the first of the next batch
                point(tb + grid_x);
                fetch(wave);
            }
            for (int g = 0; g < groups; ++g) {
                const _Float16 *op = ops + ((size_t)g * ncol + c) * GR_OP_HALVES + lane * 8;
                f16x8 A[9];
#pragma unroll
                for (int s = 0; s < 9; ++s) A[s] = *reinterpret_cast<const f16x8 *>(op + s * 512);
                const float2 iv = *reinterpret_cast<const float2 *>(inv + ((size_t)g * ncol + c) * 8 + 2 * kq);
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    if (!live[t]) continue;
                    // operand rows 4 kq + i: activation rows 2 kq (hi, lo) and 2 kq + 1 (hi, lo) of the group
                    float u0, u1;
                    if constexpr (R::BLOCK_SCALES) {
                        u0 = u1 = 0.f;
#pragma unroll
                        for (int s = 0; s < 8; ++s) {  // eight independent products, each block sum with its own d
                            const f32x4 cs = mfma16(A[s], B[t][s]);
                            u0 = __builtin_fmaf(dblk[t][s], cs[0] + cs[1], u0);
                            u1 = __builtin_fmaf(dblk[t][s], cs[2] + cs[3], u1);
                        }
                        if constexpr (R::MINS) {  // + m * (sum of x over the block): the sums were stored / 64
                            const f32x4 cm = mfma16(A[8], Bm[t]);
                            u0 = __builtin_fmaf(64.f, cm[0] + cm[1], u0);
                            u1 = __builtin_fmaf(64.f, cm[2] + cm[3], u1);
                        }
                    } else {
                        f32x4 cs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int s = 0; s < NOPS; ++s) cs = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[R::aidx(s)], B[t][s], cs, 0, 0, 0);
                        const f32x4 cm = mfma16(A[8], Bm[t]);
                        const float s0 = cs[0] + cs[1], s1 = cs[2] + cs[3], m0 = cm[0] + cm[1], m1 = cm[2] + cm[3];
                        u0 = __builtin_fmaf(d[t], s0, -dmin64[t] * m0);
                        u1 = __builtin_fmaf(d[t], s1, -dmin64[t] * m1);
                    }
                    float2 a = accl[(t * groups + g) * GR_THREADS + tid];
                    a.x = __builtin_fmaf(iv.x, u0, a.x);
                    a.y = __builtin_fmaf(iv.y, u1, a.y);
                    accl[(t * groups + g) * GR_THREADS + tid] = a;
                }
            }
        }
        __syncthreads();
        // the eight waves' partial sums, in wave order: item (t, g, lane position) -> two outputs
        for (int i = tid; i < T * groups * 64; i += GR_THREADS) {
            const int tg = i >> 6, l = i & 63, t = tg / groups, g = tg - t * groups;
            const int tile = tb * T + t;
            if (tile < ntiles) {
                float2 sum = make_float2(0.f, 0.f);
#pragma unroll
                for (int w = 0; w < GR_WAVES; ++w) {
                    const float2 p = accl[tg * GR_THREADS + w * 64 + l];
                    sum.x += p.x;
                    sum.y += p.y;
                }
                const int r = l & 15, row = min(tile * 16, n - 16) + r, b0 = g * 8 + 2 * (l >> 4);
                if (row >= tile * 16) {  // rows of a ragged last tile that an earlier tile already wrote are skipped
                    const float bv = bias ? bias[row] : 0.f;
                    // (res [rows, n]: a residual that rides along, y = res + x W^T - the layers of a model)
                    if (b0 < rows) y[(size_t)b0 * n + row] = sum.x + bv + (res ? res[(size_t)b0 * n + row] : 0.f);
                    if (b0 + 1 < rows) y[(size_t)(b0 + 1) * n + row] = sum.y + bv + (res ? res[(size_t)(b0 + 1) * n + row] : 0.f);
                }
            }
        }
        __syncthreads();
    }
}

}  // namespace jitnn
