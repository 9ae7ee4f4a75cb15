// gemv_i8_kernel: batch-1 (and two-row) GEMV on raw quantised blocks with INT8 matrix-core products.
#include "gemv_i8.h"
#include "tu.h"

namespace jitnn {

// K-quants with rows of whole super-blocks; the 32-value formats with rows of whole pairs of blocks (matrices of the formats
// fetched as dwords - the 32-value ones and Q2_K - on dword boundaries: the caller checks)
bool gemv_i8_supported(int fmt, int k) {
    if (fmt == F_Q4_0 || fmt == F_Q4_1 || fmt == F_Q8_0 || fmt == F_Q5_1) return k % 64 == 0 && k >= 64 && k <= 1024 * I8_MAX_WAVES;
    return (fmt == F_Q4_K || fmt == F_Q5_K || fmt == F_Q6_K || fmt == F_Q2_K) && k % 256 == 0 && k >= 256 && k <= 1024 * I8_MAX_WAVES;
}

typedef void (*i8_fused_fn)(const uint8_t *, const float *, const uint8_t *, const float *, const uint8_t *, uint32_t, int, int, int, const I8Args);
typedef void (*i8_plain_fn)(const uint8_t *, const float *, uint32_t, int, const I8Args);
struct i8_fn {  // one of the two is set
    i8_plain_fn plain = nullptr;
    i8_fused_fn fused = nullptr;
    explicit operator bool() const { return plain || fused; }
};
static i8_fn plain_fn(i8_plain_fn f) { i8_fn r; r.plain = f; return r; }
static i8_fn fused_fn(i8_fused_fn f) { i8_fn r; r.fused = f; return r; }

template <class U, int PF, int MAXW>
static i8_fn pick_mode(int mode) {
    switch (mode) {
    case I8_BIAS: return plain_fn(gemv_i8_plain_kernel<U, 1, PF, true, MAXW>);
    case I8_NORM: return fused_fn(gemv_i8_kernel<U, 1, PF, false, true, false, MAXW>);
    case I8_DUAL: return fused_fn(gemv_i8_kernel<U, 1, PF, false, true, true, MAXW>);
    default: return plain_fn(gemv_i8_plain_kernel<U, 1, PF, false, MAXW>);
    }
}

template <class U, int MAXW>
static i8_fn pick_pf(int mode, int pf) {
    if constexpr (U::FMT == F_Q5_K || U::FMT == F_Q8_0) return pf <= 1 ? pick_mode<U, 1, MAXW>(mode) : pick_mode<U, 2, MAXW>(mode);  // (five loads a turn: a fourth buffer does not fit 128 registers)
    else return pf <= 1 ? pick_mode<U, 1, MAXW>(mode) : pf == 2 ? pick_mode<U, 2, MAXW>(mode) : pick_mode<U, 3, MAXW>(mode);
}

// two or four activation rows (three run as four with one absent), rows of at most 4096 values; the body takes any number, but
// its products multiply one activation row each: from five rows on the 16-row tiles of gemv_mfma_kernel are faster
template <class U, int B>
static i8_fn pick_batch(int mode, int pf) {
    if (mode == I8_BIAS) return plain_fn(pf <= 1 ? gemv_i8_plain_kernel<U, B, 1, true, 4> : gemv_i8_plain_kernel<U, B, 2, true, 4>);
    return plain_fn(pf <= 1 ? gemv_i8_plain_kernel<U, B, 1, false, 4> : gemv_i8_plain_kernel<U, B, 2, false, 4>);
}

// Q5_1 and Q2_K: formats no fused launch of the decode step is built for - with or without a bias, nothing else
template <class U, int MAXW>
static i8_fn pick_plain(int mode, int pf) {
    if (mode != I8_BIAS && mode != I8_PLAIN) return i8_fn{};
    if constexpr (MAXW > 4) {  // (long rows: one turn in flight)
        return plain_fn(mode == I8_BIAS ? gemv_i8_plain_kernel<U, 1, 1, true, MAXW> : gemv_i8_plain_kernel<U, 1, 1, false, MAXW>);
    } else {
        if (mode == I8_BIAS) return plain_fn(pf <= 1 ? gemv_i8_plain_kernel<U, 1, 1, true, MAXW> : gemv_i8_plain_kernel<U, 1, 2, true, MAXW>);
        return plain_fn(pf <= 1 ? gemv_i8_plain_kernel<U, 1, 1, false, MAXW> : gemv_i8_plain_kernel<U, 1, 2, false, MAXW>);
    }
}

template <class U>
static i8_fn pick_rows(int rows, int waves, int mode, int pf) {
    if (rows == 1) return waves <= 4 ? pick_pf<U, 4>(mode, pf) : pick_plain<U, I8_MAX_WAVES>(mode, 1);  // (long rows: plain or biased, one turn in flight - the fused launches of the decode step have rows of at most 4096 values)
    if (waves > 4 || rows > 8 || (mode != I8_PLAIN && mode != I8_BIAS)) return i8_fn{};  // (five to eight rows: two groups of four)
    return rows > 2 ? pick_batch<U, 4>(mode, pf) : pick_batch<U, 2>(mode, pf);
}

template <class U>
static i8_fn pick_rows_plain(int rows, int waves, int mode, int pf) {
    if (rows == 1) return waves <= 4 ? pick_plain<U, 4>(mode, pf) : pick_plain<U, I8_MAX_WAVES>(mode, 1);
    if (waves > 4 || rows > 4 || (mode != I8_PLAIN && mode != I8_BIAS)) return i8_fn{};
    return rows > 2 ? pick_batch<U, 4>(mode, pf) : pick_batch<U, 2>(mode, pf);
}

static int batch_of(int rows) { return rows == 1 ? 1 : rows == 2 ? 2 : 4; }

// Q6_K rows a multiple of four bytes long in matrices on dword boundaries take the variant with dword-aligned loads
static bool q6_aligned(const I8Args &a) {
    bool ok = a.k % 512 == 0 && ((uintptr_t)a.w2 & 3) == 0;
    for (int i = 0; i < 3; ++i) ok = ok && ((uintptr_t)a.w[i] & 3) == 0;
    return ok;
}

bool gemv_i8_launch(int fmt, int mode, int pf, unsigned blocks, hipStream_t s, const I8Args &a) {
    const int waves = (a.k + 1023) / 1024, rows = a.rows < 1 ? 1 : a.rows;
    i8_fn fn;
    switch (fmt) {
    case F_Q4_K: fn = pick_rows<U8<F_Q4_K>>(rows, waves, mode, pf); break;
    case F_Q5_K: fn = pick_rows<U8<F_Q5_K>>(rows, waves, mode, pf); break;
    case F_Q4_0: fn = pick_rows<U8<F_Q4_0>>(rows, waves, mode, pf); break;
    case F_Q4_1: fn = pick_rows<U8<F_Q4_1>>(rows, waves, mode, pf); break;
    case F_Q8_0: fn = pick_rows<U8<F_Q8_0>>(rows, waves, mode, pf); break;
    case F_Q5_1: fn = pick_rows_plain<U8<F_Q5_1>>(rows, waves, mode, pf); break;
    case F_Q2_K: fn = pick_rows_plain<U8<F_Q2_K>>(rows, waves, mode, pf); break;
    case F_Q6_K: fn = q6_aligned(a) ? pick_rows<U8Q6<true>>(rows, waves, mode, pf) : pick_rows<U8Q6<false>>(rows, waves, mode, pf); break;
    default: break;
    }
    if (!fn) return false;
    const int bt = batch_of(rows);
    if (blocks >= (1u << 20) || rows > 8) return false;  // (what the packed argument holds)
    const dim3 grid(blocks, (rows + bt - 1) / bt), block(64 * waves);
    const size_t lds = gemv_i8_lds_bytes(waves, bt);
    const uint32_t packed = i8_pack(a.k, (int)blocks, rows);
    const int n = a.n[0] + a.n[1] + a.n[2];
    if (fn.plain) hipLaunchKernelGGL(fn.plain, grid, block, lds, s, a.w[0], a.x, packed, n, a);
    else hipLaunchKernelGGL(fn.fused, grid, block, lds, s, a.w[0], a.x, mode == I8_DUAL ? a.w2 : a.w[1], a.nw, a.w[2], packed, n, a.n[0], a.n[1], a);
    return true;
}

typedef void (*i8_pair_fn)(const uint8_t *, const uint8_t *, const uint8_t *, const float *, const float *, uint32_t, int, int, int, const I8Args, const I8Args);

template <int PF>
static i8_pair_fn pick_pair(int fa, int fb, bool al) {
    if (fa == F_Q4_K && fb == F_Q6_K) return al ? gemv_i8_pair_kernel<U8<F_Q4_K>, U8Q6<true>, PF, 4> : gemv_i8_pair_kernel<U8<F_Q4_K>, U8Q6<false>, PF, 4>;
    if (fa == F_Q4_K && fb == F_Q5_K) return gemv_i8_pair_kernel<U8<F_Q4_K>, U8<F_Q5_K>, PF, 4>;
    if (fa == F_Q5_K && fb == F_Q6_K) return al ? gemv_i8_pair_kernel<U8<F_Q5_K>, U8Q6<true>, PF, 4> : gemv_i8_pair_kernel<U8<F_Q5_K>, U8Q6<false>, PF, 4>;
    return nullptr;
}

bool gemv_i8_pair_supported(int fmt_a, int fmt_b) { return pick_pair<1>(fmt_a, fmt_b, false) != nullptr; }

bool gemv_i8_pair_launch(int fmt_a, int fmt_b, int pf, unsigned blocks_a, unsigned blocks_b, hipStream_t s, const I8Args &a, const I8Args &b) {
    const int waves = (a.k + 1023) / 1024;
    const bool al = fmt_b == F_Q6_K && q6_aligned(b);
    const i8_pair_fn fn = pf <= 1 ? pick_pair<1>(fmt_a, fmt_b, al) : pick_pair<2>(fmt_a, fmt_b, al);
    // (the first set: at most two row segments, the second one matrix; the split and the grid in 11 and 12 bits of the packed argument)
    if (!fn || waves > 4 || a.n[2] != 0 || b.n[1] != 0 || b.n[2] != 0 || blocks_a >= 2048 || blocks_a + blocks_b >= 4096) return false;
    const uint32_t packed = (uint32_t)(a.k >> 6) | (blocks_a << 9) | ((blocks_a + blocks_b) << 20);
    hipLaunchKernelGGL(fn, dim3(blocks_a + blocks_b), dim3(64 * waves), gemv_i8_lds_bytes(waves), s, a.w[0], a.w[1], b.w[0], a.x, a.nw, packed, a.n[0] + a.n[1], a.n[0], b.n[0], a,
                       b);
    return true;
}

}  // namespace jitnn
