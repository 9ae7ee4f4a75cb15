// gemv_rows_kernel: the formats it is built for.
#include "gemv_rows.h"
#include "tu.h"

namespace jitnn {

bool gemv_rows_supported(int fmt) { return gemv_rows_layout(fmt) >= 0; }

size_t gemv_rows_scratch_bytes(int rows, int k) {
    const int groups = (rows + 7) / 8;
    return gemv_rows_ops_bytes(groups, k) + gemv_rows_inv_bytes(groups, k);
}


// Two tiles per wave where that still gives every CU a workgroup - and, for many groups of activation rows, where it gives
// every other CU one: two tiles share the activation operands, which are what the launch waits for, and the idle half of the
// device takes a share of the groups (below).  4096 x 14336 at 40 rows, one tile against two: Q6_K 81.1 / 53.9 us, Q4_K 42.4 /
// 35.7, Q5_K 44.3 / 40.6, Q4_1 42.4 / 38.1; 4096 x 4096 Q4_K 18.9 / 17.3 - at 24 rows they are level or the single tile ahead
// (Q5_K 33.1 / 35.0), and Q4_0 and Q8_0 lose up to 40 rows (Q8_0 4096 x 4096 18.8 / 21.1) and gain little at 64: not for those.
// Without the sharing of groups only Q6_K, with its sixteen operands per tile, gains from two tiles on half the CUs (64.9;
// Q4_K 47.0, Q8_0 58.5 against 46.0).
static int tiles_per_wave(int fmt, int n, int k, int rows, unsigned max_blocks) {
    const unsigned pairs = (unsigned)(((n + 15) / 16 + 1) / 2);
    bool half = fmt == F_Q6_K && rows > 16 && k >= 8192;
    if (rows > 32 && k >= 4096 && (fmt == F_Q4_K || fmt == F_Q5_K || fmt == F_Q6_K || fmt == F_Q4_1)) half = true;
    return pairs >= max_blocks || (half && 2 * pairs >= max_blocks) ? 2 : 1;
}

template <int FMT>
static KernelRef kernel_ref(bool two) {
    return {two ? (const void *)gemv_rows_kernel<FMT, 2> : (const void *)gemv_rows_kernel<FMT, 1>,
            gemv_rows_lds_bytes(two ? 2 : 1) + gemv_rows_stage_bytes<FMT>(two ? 2 : 1)};
}

KernelRef gemv_rows_kernel_ref(int fmt, int n, int k, int rows, unsigned max_blocks) {
    const bool two = tiles_per_wave(fmt, n, k, rows, max_blocks) == 2;
    switch (fmt) {
    case F_Q4_K: return kernel_ref<F_Q4_K>(two);
    case F_Q5_K: return kernel_ref<F_Q5_K>(two);
    case F_Q6_K: return kernel_ref<F_Q6_K>(two);
    case F_Q4_0: return kernel_ref<F_Q4_0>(two);
    case F_Q4_1: return kernel_ref<F_Q4_1>(two);
    case F_Q8_0: return kernel_ref<F_Q8_0>(two);
    case F_Q5_1: return kernel_ref<F_Q5_1>(two);
    case F_Q2_K: return kernel_ref<F_Q2_K>(two);
    default: return {nullptr, 0};
    }
}

template <int FMT>
static constexpr int layout_of() {
    using R = RTile<FMT>;
    return R::SUMS == 16 ? GR_LAYOUT_SUMS16 : R::HALVES ? GR_LAYOUT_HALVES : GR_LAYOUT_PLAIN;
}

int gemv_rows_layout(int fmt) {
    switch (fmt) {
    case F_Q4_K: return layout_of<F_Q4_K>();
    case F_Q5_K: return layout_of<F_Q5_K>();
    case F_Q6_K: return layout_of<F_Q6_K>();
    case F_Q4_0: return layout_of<F_Q4_0>();
    case F_Q4_1: return layout_of<F_Q4_1>();
    case F_Q8_0: return layout_of<F_Q8_0>();
    case F_Q5_1: return layout_of<F_Q5_1>();
    case F_Q2_K: return layout_of<F_Q2_K>();
    default: return -1;
    }
}

static_assert(GR_LAYOUT_PLAIN == 0 && GR_LAYOUT_SUMS16 == 1 && GR_LAYOUT_HALVES == 2 && GR_LAYOUTS == 3, "RowsPrepareOut is indexed by layout");

void gemv_rows_prepare_launch(hipStream_t s, const float *x, const float *swiglu_up, void *const *scratch, int k, int rows) {
    const int groups = (rows + 7) / 8, ncol = k / 256;
    RowsPrepareOut o{};
    for (int l = 0; l < GR_LAYOUTS; ++l) {
        if (!scratch[l]) continue;
        o.ops[l] = reinterpret_cast<_Float16 *>(scratch[l]);
        o.inv[l] = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(scratch[l]) + gemv_rows_ops_bytes(groups, k));
    }
    const dim3 grid(ncol, groups);
    if (swiglu_up) hipLaunchKernelGGL(rows_prepare_kernel<true>, grid, dim3(64), 0, s, x, swiglu_up, rows, k, o);
    else hipLaunchKernelGGL(rows_prepare_kernel<false>, grid, dim3(64), 0, s, x, swiglu_up, rows, k, o);
}

template <int FMT>
static void launch(unsigned max_blocks, hipStream_t s, const uint8_t *W, const void *scratch, const float *bias, const float *res, float *y, int n, int k,
                   int rows) {
    const int groups = (rows + 7) / 8;
    const _Float16 *ops = reinterpret_cast<const _Float16 *>(scratch);
    const float *inv = reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(scratch) + gemv_rows_ops_bytes(groups, k));
    const int T = tiles_per_wave(FMT, n, k, rows, max_blocks), nbatch = ((n + 15) / 16 + T - 1) / T;
    const unsigned blocks = (unsigned)nbatch < max_blocks ? (unsigned)nbatch : max_blocks;
    // Few tiles: the groups of activation rows are shared out over as many workgroups per tile as the device has room for -
    // each decodes the tile's weights again (the device would idle otherwise) and writes whole outputs of its own rows.
    // 1024 x 4096 at 40 rows: Q6_K 30.0 -> 19.4 us, Q4_K 17.5 -> 13.5; twice as many workgroups as CUs: 23.4, 13.9.
    int gy = 1;
    if ((unsigned)nbatch * 2 <= max_blocks) {
        const int cap = (int)(max_blocks / (unsigned)nbatch), gper = (groups + cap - 1) / cap;
        gy = (groups + gper - 1) / gper;
    }
    if (T == 2) hipLaunchKernelGGL((gemv_rows_kernel<FMT, 2>), dim3(blocks, gy), dim3(GR_THREADS), gemv_rows_lds_bytes(2) + gemv_rows_stage_bytes<FMT>(2), s, W, ops, inv, n, k, rows, groups, blocks | ((unsigned)gy << 16), bias, res, y);
    else hipLaunchKernelGGL((gemv_rows_kernel<FMT, 1>), dim3(blocks, gy), dim3(GR_THREADS), gemv_rows_lds_bytes(1) + gemv_rows_stage_bytes<FMT>(1), s, W, ops, inv, n, k, rows, groups, blocks | ((unsigned)gy << 16), bias, res, y);
}

void gemv_rows_main_launch(int fmt, unsigned max_blocks, hipStream_t s, const uint8_t *W, const void *scratch, const float *bias, const float *res, float *y,
                           int n, int k, int rows) {
    switch (fmt) {
    case F_Q4_K: launch<F_Q4_K>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q5_K: launch<F_Q5_K>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q6_K: launch<F_Q6_K>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q4_0: launch<F_Q4_0>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q4_1: launch<F_Q4_1>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q8_0: launch<F_Q8_0>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q5_1: launch<F_Q5_1>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    case F_Q2_K: launch<F_Q2_K>(max_blocks, s, W, scratch, bias, res, y, n, k, rows); break;
    default: break;
    }
}

}  // namespace jitnn
