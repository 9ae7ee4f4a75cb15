// gemv_i8_kernel: batch-1 GEMV of Q4_K, Q5_K and Q6_K weights with INT8 matrix-core products.
#include "gemv_i8.h"
#include "tu.h"

namespace jitnn {

bool gemv_i8_supported(int fmt, int k) {
    return (fmt == F_Q4_K || fmt == F_Q5_K || fmt == F_Q6_K) && k % 256 == 0 && k >= 256 && k <= 1024 * I8_MAX_WAVES;
}

typedef void (*i8_fn)(const I8Args);

template <class U, int PF, int MAXW>
static i8_fn pick_mode(int mode) {
    switch (mode) {
    case I8_BIAS: return gemv_i8_kernel<U, PF, true, false, false, MAXW>;
    case I8_NORM: return gemv_i8_kernel<U, PF, false, true, false, MAXW>;
    case I8_DUAL: return gemv_i8_kernel<U, PF, false, true, true, MAXW>;
    default: return gemv_i8_kernel<U, PF, false, false, false, MAXW>;
    }
}

template <class U, int MAXW>
static i8_fn pick_pf(int mode, int pf) {
    if constexpr (U::FMT == F_Q5_K) return pf <= 1 ? pick_mode<U, 1, MAXW>(mode) : pick_mode<U, 2, MAXW>(mode);
    else return pf <= 1 ? pick_mode<U, 1, MAXW>(mode) : pf == 2 ? pick_mode<U, 2, MAXW>(mode) : pick_mode<U, 3, MAXW>(mode);
}

template <int MAXW>
static i8_fn pick_fmt(int fmt, int mode, int pf, bool q6_aligned) {
    switch (fmt) {
    case F_Q4_K: return pick_pf<U8<F_Q4_K>, MAXW>(mode, pf);
    case F_Q5_K: return pick_pf<U8<F_Q5_K>, MAXW>(mode, pf < 2 ? pf : 2);  // (five loads a turn: a fourth buffer does not fit 128 registers)
    case F_Q6_K: return q6_aligned ? pick_pf<U8Q6<true>, MAXW>(mode, pf) : pick_pf<U8Q6<false>, MAXW>(mode, pf);
    default: return nullptr;
    }
}

// Q6_K rows a multiple of four bytes long in matrices on dword boundaries take the variant with dword-aligned loads
static bool q6_aligned(const I8Args &a) {
    bool ok = a.k % 512 == 0 && ((uintptr_t)a.w2 & 3) == 0;
    for (int i = 0; i < 3; ++i) ok = ok && ((uintptr_t)a.w[i] & 3) == 0;
    return ok;
}

void gemv_i8_launch(int fmt, int mode, int pf, unsigned blocks, hipStream_t s, const I8Args &a) {
    const int waves = (a.k + 1023) / 1024;
    const bool al = fmt == F_Q6_K && q6_aligned(a);
    const i8_fn fn = waves <= 4 ? pick_fmt<4>(fmt, mode, pf, al) : pick_fmt<I8_MAX_WAVES>(fmt, mode, pf, al);
    if (!fn) return;
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(64 * waves), gemv_i8_lds_bytes(waves), s, a);
}

typedef void (*i8_pair_fn)(const I8Args, const I8Args, int);

template <int PF>
static i8_pair_fn pick_pair(int fa, int fb, bool al) {
    if (fa == F_Q4_K && fb == F_Q6_K) return al ? gemv_i8_pair_kernel<U8<F_Q4_K>, U8Q6<true>, PF, 4> : gemv_i8_pair_kernel<U8<F_Q4_K>, U8Q6<false>, PF, 4>;
    if (fa == F_Q4_K && fb == F_Q5_K) return gemv_i8_pair_kernel<U8<F_Q4_K>, U8<F_Q5_K>, PF, 4>;
    if (fa == F_Q5_K && fb == F_Q6_K) return al ? gemv_i8_pair_kernel<U8<F_Q5_K>, U8Q6<true>, PF, 4> : gemv_i8_pair_kernel<U8<F_Q5_K>, U8Q6<false>, PF, 4>;
    return nullptr;
}

bool gemv_i8_pair_supported(int fmt_a, int fmt_b) { return pick_pair<1>(fmt_a, fmt_b, false) != nullptr; }

void gemv_i8_pair_launch(int fmt_a, int fmt_b, int pf, unsigned blocks_a, unsigned blocks_b, hipStream_t s, const I8Args &a, const I8Args &b) {
    const int waves = (a.k + 1023) / 1024;
    const bool al = fmt_b == F_Q6_K && q6_aligned(b);
    const i8_pair_fn fn = pf <= 1 ? pick_pair<1>(fmt_a, fmt_b, al) : pick_pair<2>(fmt_a, fmt_b, al);
    if (!fn || waves > 4) return;
    hipLaunchKernelGGL(fn, dim3(blocks_a + blocks_b), dim3(64 * waves), gemv_i8_lds_bytes(waves), s, a, b, (int)blocks_a);
}

}  // namespace jitnn
