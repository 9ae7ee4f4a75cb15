// prefill_mfma_dual_kernel (gate and up of a Llama FFN in one product, SwiGLU in the epilogue) for the 32-value formats.
#include "prefill.h"
#include "tu.h"

namespace jitnn {

KernelRef prefill_kernel_dual_q32(int fmt) {
    switch (fmt) {
    case F_Q4_0: return {(const void *)prefill_mfma_dual_kernel<F_Q4_0>, pf_lds_bytes<F_Q4_0>()};
    case F_Q4_1: return {(const void *)prefill_mfma_dual_kernel<F_Q4_1>, pf_lds_bytes<F_Q4_1>()};
    case F_Q8_0: return {(const void *)prefill_mfma_dual_kernel<F_Q8_0>, pf_lds_bytes<F_Q8_0>()};
    default: return {nullptr, 0};
    }
}

void prefill_launch_dual_q32(int fmt, dim3 grid, hipStream_t s, const uint8_t *W, const uint8_t *W2, const _Float16 *xo, const float *inv_scale, float *y,
                             int m, int n, int k) {
    switch (fmt) {
    case F_Q4_0: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q4_0>, grid, dim3(256), pf_lds_bytes<F_Q4_0>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    case F_Q4_1: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q4_1>, grid, dim3(256), pf_lds_bytes<F_Q4_1>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    case F_Q8_0: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q8_0>, grid, dim3(256), pf_lds_bytes<F_Q8_0>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    default: break;
    }
}

}  // namespace jitnn
