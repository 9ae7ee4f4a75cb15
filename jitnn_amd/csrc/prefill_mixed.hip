// prefill_mfma_mixed_kernel: weights of two K-quant formats on one activation in one launch.
#include "prefill.h"
#include "tu.h"

namespace jitnn {

template <int FA, int FB>
constexpr size_t mixed_lds() { return pf_lds_bytes<FA>() > pf_lds_bytes<FB>() ? pf_lds_bytes<FA>() : pf_lds_bytes<FB>(); }

KernelRef prefill_kernel_mixed(int fmt_a, int fmt_b) {
    if (fmt_a == F_Q4_K && fmt_b == F_Q6_K) return {(const void *)prefill_mfma_mixed_kernel<F_Q4_K, F_Q6_K>, mixed_lds<F_Q4_K, F_Q6_K>()};
    if (fmt_a == F_Q5_K && fmt_b == F_Q6_K) return {(const void *)prefill_mfma_mixed_kernel<F_Q5_K, F_Q6_K>, mixed_lds<F_Q5_K, F_Q6_K>()};
    return {nullptr, 0};
}

void prefill_launch_mixed(int fmt_a, int fmt_b, int first_b, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale,
                          int m, int k) {
    if (fmt_a == F_Q4_K && fmt_b == F_Q6_K)
        hipLaunchKernelGGL((prefill_mfma_mixed_kernel<F_Q4_K, F_Q6_K>), grid, dim3(256), (mixed_lds<F_Q4_K, F_Q6_K>()), s, sg, first_b, xo, inv_scale, m, k);
    else if (fmt_a == F_Q5_K && fmt_b == F_Q6_K)
        hipLaunchKernelGGL((prefill_mfma_mixed_kernel<F_Q5_K, F_Q6_K>), grid, dim3(256), (mixed_lds<F_Q5_K, F_Q6_K>()), s, sg, first_b, xo, inv_scale, m, k);
}

}  // namespace jitnn
