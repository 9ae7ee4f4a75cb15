// prefill_mfma_dual_kernel (gate and up of a Llama FFN in one product, SwiGLU in the epilogue) for the 256-value formats.
#include "prefill.h"
#include "tu.h"

namespace jitnn {

KernelRef prefill_kernel_dual_k(int fmt) {
    switch (fmt) {
    case F_Q4_K: return {(const void *)prefill_mfma_dual_kernel<F_Q4_K>, pf_lds_bytes<F_Q4_K>()};
    case F_Q5_K: return {(const void *)prefill_mfma_dual_kernel<F_Q5_K>, pf_lds_bytes<F_Q5_K>()};
    case F_Q6_K: return {(const void *)prefill_mfma_dual_kernel<F_Q6_K>, pf_lds_bytes<F_Q6_K>()};
    default: return {nullptr, 0};
    }
}

void prefill_launch_dual_k(int fmt, dim3 grid, hipStream_t s, const uint8_t *W, const uint8_t *W2, const _Float16 *xo, const float *inv_scale, float *y,
                           int m, int n, int k) {
    switch (fmt) {
    case F_Q4_K: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q4_K>, grid, dim3(256), pf_lds_bytes<F_Q4_K>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    case F_Q5_K: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q5_K>, grid, dim3(256), pf_lds_bytes<F_Q5_K>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    case F_Q6_K: hipLaunchKernelGGL(prefill_mfma_dual_kernel<F_Q6_K>, grid, dim3(256), pf_lds_bytes<F_Q6_K>(), s, W, W2, xo, inv_scale, y, m, n, k); break;
    default: break;
    }
}

}  // namespace jitnn
