// Host entry points of the translation units that hold the matrix-core kernels.  The library is several .hip files so
// that it builds in parallel: every kernel template is instantiated in exactly one of them, the others reach it
// through the plain functions below (C++ linkage, hidden like everything that is not in include/jitnn_hip.h).
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace jitnn {

// a kernel and the dynamic LDS it needs (for hipFuncSetAttribute when that is more than 64 KiB); fn == nullptr: no such format
struct KernelRef {
    const void *fn;
    size_t lds;
};

// Up to three weights [n[i], k] of one activation in one launch of the many-row kernel: their row tiles (tiles[i] of
// them, 128 rows each) are numbered one after the other along blockIdx.x, slice after slice when the segment splits K:
// segment i takes tiles[i] * splits[i] workgroups, slice z of it the K steps [z * split_steps[i], (z + 1) * split_steps[i])
// and the array y[i] + z * m * n[i] (partial sums, to be joined).  Segments may split differently: the tiles of a format
// that takes longer per step get shorter slices.  Unused segments: n = tiles = 0, splits = 1.
struct PfSegments {
    const uint8_t *W[3];
    float *y[3];
    int n[3];
    int tiles[3];
    int splits[3];
    int split_steps[3];
};

// ---- prefill_k.hip (Q4_K, Q5_K, Q6_K), prefill_q32.hip (Q4_0, Q4_1, Q8_0): prefill_mfma_kernel<fmt>;
// prefill_mixed.hip: prefill_mfma_mixed_kernel for segments of two K-quant formats (first_b: the first segment of fmt_b)
KernelRef prefill_kernel_k(int fmt);
KernelRef prefill_kernel_q32(int fmt);
KernelRef prefill_kernel_mixed(int fmt_a, int fmt_b);  // fn == nullptr: this pair has no kernel
void prefill_launch_k(int fmt, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale, const float *bias, int m, int k);
void prefill_launch_q32(int fmt, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale, const float *bias, int m,
                        int k);
void prefill_launch_mixed(int fmt_a, int fmt_b, int first_b, dim3 grid, hipStream_t s, const PfSegments &sg, const _Float16 *xo, const float *inv_scale,
                          int m, int k);
// prefill_dual_k.hip, prefill_dual_q32.hip: prefill_mfma_dual_kernel<fmt>, y [m, n] = silu(x W^T) * (x W2^T) for two weights
// [n, k] of one format; grid (ceil(n / 64), token tiles)
KernelRef prefill_kernel_dual_k(int fmt);
KernelRef prefill_kernel_dual_q32(int fmt);
void prefill_launch_dual_k(int fmt, dim3 grid, hipStream_t s, const uint8_t *W, const uint8_t *W2, const _Float16 *xo, const float *inv_scale, float *y,
                           int m, int n, int k);
void prefill_launch_dual_q32(int fmt, dim3 grid, hipStream_t s, const uint8_t *W, const uint8_t *W2, const _Float16 *xo, const float *inv_scale, float *y,
                             int m, int n, int k);
// activation preparation and the join of K slices (prefill_q32.hip)
// (norm_w != nullptr: RMSNorm with that weight and eps fused into the preparation; swiglu_up != nullptr: the activations
// are silu(x) * swiglu_up, both [rows, k] - either only where prefill_prepare_fuses_norm(k))
bool prefill_prepare_fuses_norm(int k);
// The K slices of a linear whose join was left to the activation preparation that follows it: the row the preparation
// normalises is res + the slices in slice order, and is stored to out on the way.
struct PfPending {
    const float *part = nullptr;  // [splits][rows, n]
    const float *res = nullptr;   // [rows, n]
    float *out = nullptr;         // [rows, n]
    int splits = 0, n = 0;
};
// The K slices of a launch of several segments whose join was left to the kernel that reads the products next: part holds,
// segment after segment, sg.splits[i] arrays [rows, sg.n[i]].
struct PfGroupPending {
    const float *part = nullptr;
    PfSegments sg;
};
// (pend != nullptr: x is ignored, the rows come from *pend - with norm_w and rows the preparation normalises only)
void prefill_prepare_launch(const float *x, float *scale, float *inv_scale, _Float16 *xo, int rows, int k, int mblocks, const float *norm_w, float eps,
                            const float *swiglu_up, hipStream_t s, const PfPending *pend = nullptr);
void prefill_join_launch(const float *part, const float *bias, const float *res, float *y, size_t count4, int n, int splits, unsigned blocks,
                         hipStream_t s);
// the join of a launch of several segments: part = per segment splits[i] arrays [m, n[i]], one segment after the other
void prefill_join_group_launch(const float *part, const PfSegments &sg, int m, unsigned blocks, hipStream_t s);

// ---- gemv_mfma.hip: gemv_mfma_kernel<fmt>
KernelRef gemv_mfma_kernel_ref(int fmt);
void gemv_mfma_launch(int fmt, unsigned blocks, hipStream_t s, const uint8_t *W, const float *x, const float *bias, float *y, int n, int k, int rows);

// ---- gemv_rows.hip: rows_prepare_kernel + gemv_rows_kernel<fmt>: 2..64 rows in one pass over the weights.  The operands of
// the activations are prepared once per operand layout a format needs (gemv_rows_layout: block sums per 32 or per 16
// values, the values of a lane consecutive or in the two halves of a 4-bit block) into a scratch of
// gemv_rows_scratch_bytes and serve every weight of that layout that meets the same activations.
constexpr int GR_LAYOUT_PLAIN = 0, GR_LAYOUT_SUMS16 = 1, GR_LAYOUT_HALVES = 2, GR_LAYOUTS = 3;
bool gemv_rows_supported(int fmt);
int gemv_rows_layout(int fmt);                     // GR_LAYOUT_* of the format, -1: the kernel is not built for it
size_t gemv_rows_scratch_bytes(int rows, int k);   // operands + scales of `rows` activation rows of k values
KernelRef gemv_rows_kernel_ref(int fmt, int n, int k, int rows, unsigned max_blocks);  // the variant gemv_rows_main_launch picks for this shape
// every layout with a scratch (scratch[GR_LAYOUTS], nullptr: not wanted) in one launch; swiglu_up != nullptr: the rows are
// silu(x) * swiglu_up, both [rows, k]
void gemv_rows_prepare_launch(hipStream_t s, const float *x, const float *swiglu_up, void *const *scratch, int k, int rows);
// y = x W^T (+ bias [n]) (+ res [rows, n])
void gemv_rows_main_launch(int fmt, unsigned max_blocks, hipStream_t s, const uint8_t *W, const void *scratch, const float *bias, const float *res, float *y,
                           int n, int k, int rows);

// ---- gemv_i8.hip: gemv_i8_kernel / gemv_i8_plain_kernel<unit>: GEMV of one to four activation rows with INT8 matrix-core products on the
// raw quants.  The argument block of the kernels (the launchers put what a wave's first loads need in front of it, as scalar
// arguments the hardware preloads): up to three matrices of one format and row length share a launch and an activation vector (row segments
// numbered one after the other).  DUAL: w2 is a second matrix of the shape of w[0]; y[0] = silu(w[0] x) * (w2 x).
struct I8Args {
    const uint8_t *w[3];
    float *y[3];
    const float *bias[3];  // BIAS: added to the segment's rows (a residual rides here)
    int n[3];
    const uint8_t *w2;
    const float *x;   // [rows, k]
    const float *nw;  // NORM: RMSNorm weight [k]
    float eps;
    int k;
    int rows;  // activation rows (x [rows, k], y [rows, n]); more than one: a single matrix, no norm, no pair
};

constexpr int I8_PLAIN = 0, I8_BIAS = 1, I8_NORM = 2, I8_DUAL = 3;  // DUAL: norm + the SwiGLU pair
bool gemv_i8_supported(int fmt, int k);
// One wave per 1024 values of a row (the launchers set the workgroup size); pf = turns of weight bytes in flight per wave beyond the one being multiplied (1..3; 1..2 for
// two to four activation rows - a.rows in 2..4, rows of at most 4096 values, modes I8_PLAIN and I8_BIAS only)
bool gemv_i8_launch(int fmt, int mode, int pf, unsigned blocks, hipStream_t s, const I8Args &a);  // false: no kernel for this call, nothing launched
bool gemv_i8_pair_supported(int fmt_a, int fmt_b);
bool gemv_i8_pair_launch(int fmt_a, int fmt_b, int pf, unsigned blocks_a, unsigned blocks_b, hipStream_t s, const I8Args &a, const I8Args &b);

}  // namespace jitnn
