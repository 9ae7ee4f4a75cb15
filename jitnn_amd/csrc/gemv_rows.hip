// gemv_rows_kernel: the formats it is built for.
#include "gemv_rows.h"
#include "tu.h"

namespace jitnn {

bool gemv_rows_supported(int fmt) { return fmt == F_Q4_K || fmt == F_Q5_K; }

size_t gemv_rows_scratch_bytes(int rows, int k) {
    const int groups = (rows + 7) / 8;
    return gemv_rows_ops_bytes(groups, k) + gemv_rows_inv_bytes(groups, k);
}

KernelRef gemv_rows_kernel_ref(int fmt) {
    switch (fmt) {
    case F_Q4_K: return {(const void *)gemv_rows_kernel<F_Q4_K>, gemv_rows_lds_bytes()};
    case F_Q5_K: return {(const void *)gemv_rows_kernel<F_Q5_K>, gemv_rows_lds_bytes()};
    default: return {nullptr, 0};
    }
}

void gemv_rows_launch(int fmt, unsigned max_blocks, hipStream_t s, const uint8_t *W, const float *x, void *scratch, const float *bias, float *y, int n,
                      int k, int rows) {
    const int groups = (rows + 7) / 8, ncol = k / 256;
    _Float16 *ops = reinterpret_cast<_Float16 *>(scratch);
    float *inv = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(scratch) + gemv_rows_ops_bytes(groups, k));
    hipLaunchKernelGGL(rows_prepare_kernel, dim3(ncol, groups), dim3(64), 0, s, x, ops, inv, rows, k);
    const int nbatch = ((n + 15) / 16 + GR_T - 1) / GR_T;
    const unsigned blocks = (unsigned)nbatch < max_blocks ? (unsigned)nbatch : max_blocks;
    switch (fmt) {
    case F_Q4_K: hipLaunchKernelGGL(gemv_rows_kernel<F_Q4_K>, dim3(blocks), dim3(GR_THREADS), gemv_rows_lds_bytes(), s, W, ops, inv, bias, y, n, k, rows, groups); break;
    case F_Q5_K: hipLaunchKernelGGL(gemv_rows_kernel<F_Q5_K>, dim3(blocks), dim3(GR_THREADS), gemv_rows_lds_bytes(), s, W, ops, inv, bias, y, n, k, rows, groups); break;
    default: break;
    }
}

}  // namespace jitnn
