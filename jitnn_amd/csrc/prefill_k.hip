// prefill_mfma_kernel for the 256-value formats (Q2_K among them).
#include "prefill.h"
#include "tu.h"

namespace jitnn {

KernelRef prefill_kernel_k(int fmt) {
    switch (fmt) {
    case F_Q4_K: return {(const void *)prefill_mfma_kernel<F_Q4_K>, pf_lds_bytes<F_Q4_K>()};
    case F_Q5_K: return {(const void *)prefill_mfma_kernel<F_Q5_K>, pf_lds_bytes<F_Q5_K>()};
    case F_Q6_K: return {(const void *)prefill_mfma_kernel<F_Q6_K>, pf_lds_bytes<F_Q6_K>()};
    case F_Q2_K: return {(const void *)prefill_mfma_kernel<F_Q2_K>, pf_lds_bytes<F_Q2_K>()};
    default: return {nullptr, 0};
    }
}

void prefill_launch_k(int fmt, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale, const float *bias, int m, int k) {
    switch (fmt) {
    case F_Q4_K: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q4_K>, grid, dim3(256), pf_lds_bytes<F_Q4_K>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q5_K: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q5_K>, grid, dim3(256), pf_lds_bytes<F_Q5_K>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q6_K: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q6_K>, grid, dim3(256), pf_lds_bytes<F_Q6_K>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q2_K: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q2_K>, grid, dim3(256), pf_lds_bytes<F_Q2_K>(), s, sg, xo, inv_scale, bias, m, k); break;
    default: break;
    }
}

}  // namespace jitnn
