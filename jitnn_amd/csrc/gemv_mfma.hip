// gemv_mfma_kernel, all six formats.
#include "gemv_mfma.h"
#include "tu.h"

namespace jitnn {

KernelRef gemv_mfma_kernel_ref(int fmt) {
    switch (fmt) {
    case F_Q4_0: return {(const void *)gemv_mfma_kernel<F_Q4_0>, gemv_mfma_lds_bytes<F_Q4_0>()};
    case F_Q4_1: return {(const void *)gemv_mfma_kernel<F_Q4_1>, gemv_mfma_lds_bytes<F_Q4_1>()};
    case F_Q8_0: return {(const void *)gemv_mfma_kernel<F_Q8_0>, gemv_mfma_lds_bytes<F_Q8_0>()};
    case F_Q4_K: return {(const void *)gemv_mfma_kernel<F_Q4_K>, gemv_mfma_lds_bytes<F_Q4_K>()};
    case F_Q5_K: return {(const void *)gemv_mfma_kernel<F_Q5_K>, gemv_mfma_lds_bytes<F_Q5_K>()};
    case F_Q6_K: return {(const void *)gemv_mfma_kernel<F_Q6_K>, gemv_mfma_lds_bytes<F_Q6_K>()};
    default: return {nullptr, 0};
    }
}

void gemv_mfma_launch(int fmt, unsigned blocks, hipStream_t s, const uint8_t *W, const float *x, const float *bias, float *y, int n, int k, int rows) {
    switch (fmt) {
    case F_Q4_0: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q4_0>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q4_0>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    case F_Q4_1: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q4_1>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q4_1>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    case F_Q8_0: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q8_0>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q8_0>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    case F_Q4_K: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q4_K>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q4_K>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    case F_Q5_K: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q5_K>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q5_K>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    case F_Q6_K: hipLaunchKernelGGL(gemv_mfma_kernel<F_Q6_K>, dim3(blocks), dim3(MF_THREADS), gemv_mfma_lds_bytes<F_Q6_K>(), s, W, x, bias, y, n, k, rows, (int)blocks); break;
    default: break;
    }
}

}  // namespace jitnn
