// prefill_mfma_kernel for the 32-value formats (Q5_1 among them), the activation preparation and the join of K slices.
#include "prefill.h"
#include "tu.h"

namespace jitnn {

KernelRef prefill_kernel_q32(int fmt) {
    switch (fmt) {
    case F_Q4_0: return {(const void *)prefill_mfma_kernel<F_Q4_0>, pf_lds_bytes<F_Q4_0>()};
    case F_Q4_1: return {(const void *)prefill_mfma_kernel<F_Q4_1>, pf_lds_bytes<F_Q4_1>()};
    case F_Q8_0: return {(const void *)prefill_mfma_kernel<F_Q8_0>, pf_lds_bytes<F_Q8_0>()};
    case F_Q5_1: return {(const void *)prefill_mfma_kernel<F_Q5_1>, pf_lds_bytes<F_Q5_1>()};
    default: return {nullptr, 0};
    }
}

void prefill_launch_q32(int fmt, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale, const float *bias, int m, int k) {
    switch (fmt) {
    case F_Q4_0: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q4_0>, grid, dim3(256), pf_lds_bytes<F_Q4_0>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q4_1: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q4_1>, grid, dim3(256), pf_lds_bytes<F_Q4_1>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q8_0: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q8_0>, grid, dim3(256), pf_lds_bytes<F_Q8_0>(), s, sg, xo, inv_scale, bias, m, k); break;
    case F_Q5_1: hipLaunchKernelGGL(prefill_mfma_kernel<F_Q5_1>, grid, dim3(256), pf_lds_bytes<F_Q5_1>(), s, sg, xo, inv_scale, bias, m, k); break;
    default: break;
    }
}

template <int MODE>
static void prepare_one_launch(const float *x, float *inv_scale, _Float16 *xo, int rows, int k, int mblocks, const float *nw, float eps, hipStream_t s,
                               const float *part = nullptr, int splits = 0, float *xsum = nullptr) {
    const int pieces = pf_ksteps(k) * 2;  // per row; 256 threads take J each
    if (pieces <= 512) hipLaunchKernelGGL((x_prepare_kernel<2, MODE>), dim3(mblocks * 32), dim3(256), 0, s, x, inv_scale, xo, rows, k, nw, eps, part, splits, xsum);
    else if (pieces <= 1024) hipLaunchKernelGGL((x_prepare_kernel<4, MODE>), dim3(mblocks * 32), dim3(256), 0, s, x, inv_scale, xo, rows, k, nw, eps, part, splits, xsum);
    else hipLaunchKernelGGL((x_prepare_kernel<8, MODE>), dim3(mblocks * 32), dim3(256), 0, s, x, inv_scale, xo, rows, k, nw, eps, part, splits, xsum);
}

bool prefill_prepare_fuses_norm(int k) { return k <= XP_MAXK; }

void prefill_prepare_launch(const float *x, float *scale, float *inv_scale, _Float16 *xo, int rows, int k, int mblocks, const float *norm_w, float eps,
                            const float *swiglu_up, hipStream_t s, const PfPending *pend) {
    if (k <= XP_MAXK) {
        if (pend) prepare_one_launch<XP_NORM_JOIN>(pend->res, inv_scale, xo, rows, k, mblocks, norm_w, eps, s, pend->part, pend->splits, pend->out);
        else if (swiglu_up) prepare_one_launch<XP_SWIGLU>(x, inv_scale, xo, rows, k, mblocks, swiglu_up, 0.f, s);
        else if (norm_w) prepare_one_launch<XP_NORM>(x, inv_scale, xo, rows, k, mblocks, norm_w, eps, s);
        else prepare_one_launch<XP_PLAIN>(x, inv_scale, xo, rows, k, mblocks, nullptr, 0.f, s);
    } else {  // (callers ask prefill_prepare_fuses_norm first: rows this long take no norm or gate here)
        hipLaunchKernelGGL(x_row_scale_kernel, dim3(rows), dim3(256), 0, s, x, scale, inv_scale, k);
        hipLaunchKernelGGL(x_to_operand_kernel, dim3(mblocks, pf_ksteps(k) / 4), dim3(256), 0, s, x, scale, xo, rows, k);
    }
}

void prefill_join_launch(const float *part, const float *bias, const float *res, float *y, size_t count4, int n, int splits, unsigned blocks,
                         hipStream_t s) {
    hipLaunchKernelGGL(prefill_join_kernel, dim3(blocks), dim3(256), 0, s, part, bias, res, y, count4, n, splits);
}

void prefill_join_group_launch(const float *part, const PfSegments &sg, int m, unsigned blocks, hipStream_t s) {
    hipLaunchKernelGGL(prefill_join_group_kernel, dim3(blocks), dim3(256), 0, s, part, sg, m);
}

}  // namespace jitnn
