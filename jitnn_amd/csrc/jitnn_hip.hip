// C-ABI entry points of libjitnn_hip.so (declared in include/jitnn_hip.h): argument validation, weight
// handles, kernel selection and launch.  Host side of the path in C++; every kernel is in the headers
// included below.
#include "../../include/jitnn_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <utility>
#include <vector>

#include <sys/syscall.h>
#include <unistd.h>

#include "dequant.h"
#include "gemv.h"
#include "gemv_mfma.h"
#include "gguf_file.h"
#include "glue.h"
#include "prefill.h"
#include "tu.h"

using namespace jitnn;

struct jitnn_hip_weight {
    int fmt;  // of the blocks at dev: the caller's format, or the one an uploaded weight was rewritten into (below)
    int n, k;
    long long nbytes;
    uint8_t *dev;
    bool owned;
    int file_fmt = 0;  // != 0: what the caller uploaded, when that was another format of exactly the same values
    long long file_nbytes = 0;
};

// Scratch of the entry point that allocates nothing (jitnn_hip_linear_noalloc_dev): FP16 activations in operand order,
// their row scales and the partial sums of K slices of a many-row linear.  One copy per GPU, held until the process
// ends.  In host code this name is only a handle for hipGetSymbolAddress; the device address is kept in State.
#define JITNN_HIP_SCRATCH_BYTES (64ull << 20)
static __device__ __align__(256) unsigned char scratch[JITNN_HIP_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                                       \
    do {                                                                                                    \
        hipError_t e_ = (expr);                                                                             \
        if (e_ != hipSuccess) return fail(JITNN_HIP_EDEVICE, "%s: %s", #expr, hipGetErrorString(e_));       \
    } while (0)

struct State {
    bool ready = false;
    int device = -1;
    int cus = 0;
    long long hbm = 0;
    char name[256] = "";
    float nib = 0.f;  // 1 / (value of E4M3 byte 0x01): 512 for OCP, 1024 for FNUZ
    size_t max_lds = 0;      // LDS one workgroup may ask for
    size_t lds_per_cu = 0;   // LDS of a compute unit
    // JITNN_HIP_GEMV_MAX_ROWS: up to this many rows run the FP32 GEMV kernels (in batches of 8), more rows the FP16
    // MFMA kernel - the counterpart of jitnn.gguf.tiledRows (core/JitnnConfig.java:423-424).  64 keeps every row
    // count the reference's own tests use (1, 5, 40) on the FP32 path, whose error meets their 2e-4 / 1e-3 bars.
    int gemv_max_rows = 64;
    bool transcode = true;            // JITNN_HIP_TRANSCODE=0: uploaded Q5_0 / Q3_K blocks stay as they are (plain kernels)
    void *scratch_ptr = nullptr;    // device address of `scratch` on g.device (hipGetSymbolAddress at init)
    bool gemv_i8 = true;            // JITNN_HIP_GEMV_I8=0: batch-1 K-quant GEMV on the FP32 register kernels instead of the INT8 matrix-core one
};
State g;
std::mutex g_mu;


__global__ void fp8_probe_kernel(float *out) {
    f32x2 p = __builtin_amdgcn_cvt_pk_f32_fp8(0x00000f01, false);
    out[0] = p.x;
    out[1] = p.y;
}

// Pure streaming read: every thread xors the 16-byte words it loads; the store can never happen for real data
// but keeps the loads alive.  U loads in flight per lane (the workgroups stride the buffer together), NT: non-temporal loads.
template <int U, bool NT>
__global__ void __launch_bounds__(256) probe_read_kernel(const u32x4 *__restrict__ p, size_t n16, uint32_t *sink, uint32_t threads) {
    const size_t stride = threads;  // (the grid's threads as an argument: gridDim is fetched from a cold argument block by the wave's first instructions)
    u32x4 acc = {0, 0, 0, 0};
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = NT ? __builtin_nontemporal_load(p + i + u * stride) : p[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    for (; i < n16; i += stride) acc ^= p[i];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && sink) *sink = acc.x;
}

// ---- counters (jitnn_hip_stats): calls and tensor bytes per operator, the reference's telemetry convention
enum StatOp { ST_GEMV, ST_MFMA, ST_DEQUANT, ST_QUANT, ST_DECODE, ST_PREFILL, ST_COUNT };
const char *const kStatNames[ST_COUNT] = {"linear_gemv", "linear_mfma", "dequantize", "quantize_q8_0", "llama_decode", "llama_prefill"};
std::atomic<long long> g_stat_calls[ST_COUNT], g_stat_bytes[ST_COUNT];
thread_local int g_stat_nested = 0;  // inside a model step: its linears are the step's own traffic
void count_op(StatOp op, long long bytes) {
    if (g_stat_nested) return;
    g_stat_calls[op].fetch_add(1, std::memory_order_relaxed);
    g_stat_bytes[op].fetch_add(bytes, std::memory_order_relaxed);
}
struct StatNest {
    StatNest() { ++g_stat_nested; }
    ~StatNest() { --g_stat_nested; }
};

bool known(int fmt) { return block_values(fmt) != 0; }

bool calling_thread_is_main() { return (long)syscall(SYS_gettid) == (long)getpid(); }

// Kernels that want more than 64 KiB of dynamic LDS must be told so once; remembered per kernel so that steady-state
// launches (and launches under graph capture) make no attribute calls.
int allow_lds(const void *fn, size_t lds) {
    if (lds <= 65536) return JITNN_HIP_OK;
    static std::mutex mu;
    static std::vector<std::pair<const void *, size_t>> seen;
    std::lock_guard<std::mutex> lock(mu);
    for (auto &e : seen)
        if (e.first == fn && e.second >= lds) return JITNN_HIP_OK;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(JITNN_HIP_EDEVICE, "hipFuncSetAttribute(%zu bytes of LDS): %s", lds, hipGetErrorString(e));
    seen.emplace_back(fn, lds);
    return JITNN_HIP_OK;
}

int check_ready() {
    if (!g.ready) return fail(JITNN_HIP_ENODEVICE, "jitnn_hip_init has not succeeded in this process");
    return JITNN_HIP_OK;
}

// ------------------------------------------------------------------------------------------ launch tables

typedef void (*gemv_fn)(const uint8_t *, const float *, const float *, float *, int, int, int, int, float);

struct GemvVariant {
    gemv_fn fn;
    int B, R;
    size_t lds_per_step;  // LDS bytes per staged wave step
    int unit_values;      // values one lane decodes per step
};

template <class U, int B, int R, int NBUF>
GemvVariant variant() {
    // the fp8 nibble conversion only applies to the 4-bit formats; the others ignore CV
    constexpr int CV = (U::FMT == F_Q4_K || U::FMT == F_Q4_0 || U::FMT == F_Q4_1) ? 1 : 0;
    return GemvVariant{gemv_lds_kernel<U, B, R, CV, NBUF>, B, R, gemv_lds_bytes<U>(B, 1), U::UV};
}

// batch rows -> (rows decoded together, ring depth): chosen so that no variant spills registers
template <class U>
GemvVariant pick_unit(int rows) {
    if (rows <= 1) return variant<U, 1, 2, 2>();
    if (rows <= 2) return variant<U, 2, 2, 2>();
    if constexpr (U::FMT == F_Q8_0) {  // 17 dwords per block pair: one row at a time
        if (rows <= 4) return variant<U, 4, 1, 1>();
        return variant<U, 8, 1, 1>();
    } else {
        if (rows <= 4) return variant<U, 4, 2, 1>();
        return variant<U, 8, 2, 1>();
    }
}

GemvVariant pick(int fmt, int rows, bool pairs) {
    switch (fmt) {
    case F_Q4_0: return pairs ? pick_unit<UnitPair<F_Q4_0>>(rows) : pick_unit<Unit<F_Q4_0>>(rows);
    case F_Q4_1: return pairs ? pick_unit<UnitPair<F_Q4_1>>(rows) : pick_unit<Unit<F_Q4_1>>(rows);
    case F_Q8_0: return pairs ? pick_unit<UnitPair<F_Q8_0>>(rows) : pick_unit<Unit<F_Q8_0>>(rows);
    case F_Q4_K: return pick_unit<Unit<F_Q4_K>>(rows);
    case F_Q5_K: return pick_unit<Unit<F_Q5_K>>(rows);
    default: return pick_unit<Unit<F_Q6_K>>(rows);
    }
}

typedef void (*gemv1_fn)(const uint8_t *, const float *, const float *, float *, int, int, float);
typedef void (*xreg_fn)(const XregArgs);

// The 32-value formats decode pairs of blocks when the row holds an even number of them (aligned loads),
// single blocks otherwise.
template <int PF, bool BIAS, bool NORM, bool DUAL>
xreg_fn pick_xreg_fmt(int fmt, bool pairs) {
    switch (fmt) {
    case F_Q4_0:
        return pairs ? gemv_xreg_kernel<UnitPair<F_Q4_0>, 1, PF, BIAS, NORM, DUAL> : gemv_xreg_kernel<Unit<F_Q4_0>, 1, PF, BIAS, NORM, DUAL>;
    case F_Q4_1:
        return pairs ? gemv_xreg_kernel<UnitPair<F_Q4_1>, 1, PF, BIAS, NORM, DUAL> : gemv_xreg_kernel<Unit<F_Q4_1>, 1, PF, BIAS, NORM, DUAL>;
    case F_Q8_0:
        return pairs ? gemv_xreg_kernel<UnitPair<F_Q8_0>, 0, PF, BIAS, NORM, DUAL> : gemv_xreg_kernel<Unit<F_Q8_0>, 0, PF, BIAS, NORM, DUAL>;
    case F_Q4_K: return gemv_xreg_kernel<Unit<F_Q4_K>, 1, PF, BIAS, NORM, DUAL>;
    case F_Q5_K: return gemv_xreg_kernel<Unit<F_Q5_K>, 0, PF, BIAS, NORM, DUAL>;
    default: return gemv_xreg_kernel<Unit<F_Q6_K>, 0, PF, BIAS, NORM, DUAL>;
    }
}

// mode 0: plain; 1: with bias; 2: with fused RMSNorm; 3: fused RMSNorm + SwiGLU pair (PF 1 or 3)
xreg_fn pick_xreg(int fmt, bool pairs, int mode, int pf) {
    switch (mode) {
    case 1: return pf == 1 ? pick_xreg_fmt<1, true, false, false>(fmt, pairs) : pick_xreg_fmt<2, true, false, false>(fmt, pairs);
    case 2: return pf == 1 ? pick_xreg_fmt<1, false, true, false>(fmt, pairs) : pick_xreg_fmt<2, false, true, false>(fmt, pairs);
    case 3: return pf == 1 ? pick_xreg_fmt<1, false, true, true>(fmt, pairs) : pick_xreg_fmt<3, false, true, true>(fmt, pairs);
    default: return pf == 1 ? pick_xreg_fmt<1, false, false, false>(fmt, pairs) : pick_xreg_fmt<2, false, false, false>(fmt, pairs);
    }
}

// One launch of the register-resident batch-1 kernel (rows of at most 4096 values) over up to three matrices of one
// format and row length.  norm_w != NULL fuses the RMSNorm of x; w2 != NULL computes silu(w x) * (w2 x).
struct XregCall {
    const jitnn_hip_weight *w[3] = {nullptr, nullptr, nullptr};
    float *y[3] = {nullptr, nullptr, nullptr};
    const float *bias = nullptr;  // for w[0] only
    const jitnn_hip_weight *w2 = nullptr;
    const float *x = nullptr, *norm_w = nullptr;
    float eps = 0.f;
};

// kernel arguments of a call; returns the total number of rows
int xreg_args(const XregCall &c, XregArgs &a) {
    int n = 0;
    for (int i = 0; i < 3; ++i) {
        a.w[i] = c.w[i] ? c.w[i]->dev : c.w[0]->dev;
        a.y[i] = c.y[i] ? c.y[i] : c.y[0];
        a.bias[i] = c.bias;
        a.n[i] = c.w[i] ? c.w[i]->n : 0;
        n += a.n[i];
    }
    a.w2 = c.w2 ? c.w2->dev : nullptr;
    a.x = c.x;
    a.nw = c.norm_w;
    a.eps = c.eps;
    a.k = c.w[0]->k;
    a.nib = g.nib;
    return n;
}

// The INT8 matrix-core kernel (gemv_i8.h) takes what the register-resident kernels take of the K-quants, and rows of up
// to 16384 values.
constexpr int PREFILL_MIN_SLICE = 8;  // fewest K steps (of 64 values) a slice of a split many-row launch may have

// Its row groups are four rows: at least four rows in all, and the segments of a shared launch whole groups; its buffer
// loads address a matrix with 32 bits.
bool i8_ok(const XregCall &c) {
    if (!g.gemv_i8 || !gemv_i8_supported(c.w[0]->fmt, c.w[0]->k)) return false;
    int n = 0;
    for (int i = 0; i < 3; ++i) {
        if (!c.w[i]) continue;
        n += c.w[i]->n;
        if (c.w[i]->nbytes >= (1ll << 32) || (c.w[1] && c.w[i]->n % 4 != 0)) return false;
        if ((block_values(c.w[i]->fmt) == 32 || c.w[i]->fmt == F_Q2_K) && ((uintptr_t)c.w[i]->dev & 3) != 0) return false;  // (fetched as dwords)
        if (is_extra_format(c.w[i]->fmt) && (c.w[1] || c.w2 || c.norm_w)) return false;  // (Q5_1, Q2_K: no fused launches)
    }
    if (c.w2 && c.w2->nbytes >= (1ll << 32)) return false;
    if (c.w[1] && (!c.norm_w || c.w2)) return false;  // (several matrices in one launch: the kernel has that for the fused norm only)
    return n >= 4;
}

int i8_args(const XregCall &c, I8Args &a) {
    int n = 0;
    for (int i = 0; i < 3; ++i) {
        a.w[i] = c.w[i] ? c.w[i]->dev : c.w[0]->dev;
        a.y[i] = c.y[i] ? c.y[i] : c.y[0];
        a.bias[i] = c.bias;
        a.n[i] = c.w[i] ? c.w[i]->n : 0;
        n += a.n[i];
    }
    a.w2 = c.w2 ? c.w2->dev : nullptr;
    a.x = c.x;
    a.nw = c.norm_w;
    a.eps = c.eps;
    a.k = c.w[0]->k;
    a.rows = 1;
    return n;
}

// workgroups and turns in flight for a launch of `groups` row groups (four rows each) of `waves`-wave workgroups
void i8_shape(int fmt, int groups, int waves, bool dual, int &blocks, int &pf) {
    // Measured (us, pf / workgroups per CU): Q4_K 14336 x 4096 8.40 (1/2) 8.44 (2/1) 8.48 (3/1) 9.54 (1/4); Q4_K 4096 x 4096 4.75 (1/2)
    // 4.93 (1/1) 5.82 (1/4); Q6_K 128256 x 4096 71.9 (2/1) 72.9 (3/1) 73.6 (1/1) 74.5 (1/2); Q6_K 4096 x 14336 (14 waves) 12.9
    // (1/1) 14.3 (2/1) 16.2 (1/2).  Tall matrices: one workgroup per CU with two turns in flight behind the one being
    // multiplied; short ones: two workgroups with one; long rows: one with one.
    const int turns1 = (groups + g.cus - 1) / g.cus;
    // (Q8_0, twice the bytes of a 4-bit format per turn: one workgroup per CU on short matrices too - 4096 x 4096 5.50 us (1/1) against
    // 5.74 (1/2), 5.72 (2/1), 6.31 (2/2), 6.67 (1/3), 7.15 (1/4))
    const int per_cu = waves > 4 ? 1 : turns1 >= 8 ? 1 : (fmt == F_Q8_0 && turns1 >= 4) ? 1 : 2;
    pf = waves > 4 ? 1 : turns1 >= 8 ? (dual ? 3 : 2) : 1;  // (gate + up of an 8B layer: 14.4 us with three turns in flight, 15.1 with two)
    blocks = groups < g.cus * per_cu ? groups : g.cus * per_cu;
}

int launch_i8(const XregCall &c, hipStream_t stream) {
    I8Args a{};
    const int n = i8_args(c, a);
    const int mode = c.w2 ? I8_DUAL : c.norm_w ? I8_NORM : c.bias ? I8_BIAS : I8_PLAIN;
    int blocks, pf;
    i8_shape(c.w[0]->fmt, (n + 3) / 4, (a.k + 1023) / 1024, c.w2 != nullptr, blocks, pf);
    if (c.w[0]->fmt == F_Q5_K && pf > 2) pf = 2;  // (five loads per turn: a fourth buffer does not fit 128 registers)
    if (!gemv_i8_launch(c.w[0]->fmt, mode, pf, (unsigned)blocks, stream, a))
        return fail(JITNN_HIP_EDEVICE, "no INT8 GEMV kernel for format %d in mode %d, rows of %d values", c.w[0]->fmt, mode, a.k);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// Two to four activation rows, rows of at most 4096 values: the same kernel with the activations of all rows in registers - the
// operands and scales of the weights are made once, every row runs its own chains of products.  us per launch against the FP32
// two-row kernel / gemv_mfma_kernel - Q4_K 14336 x 4096: 8.9 (11.3) at two rows, 10.6 (13.9) at three, 11.3 (13.8) at four; Q4_0
// 11008 x 4096 at four: 9.6 (11.8); Q8_0 4096 x 4096: 6.7 (10.1); Q6_K 14336 x 4096: 14.3 (23.0).  The number of its 4x4x4 products
// grows with the rows (four rows: twelve digit planes in three products a step): eight rows (two groups of four along
// blockIdx.y) stay behind gemv_mfma_kernel, whose 16-row tiles take 14.5 us whatever the rows - from five rows on those stay
// ahead, except for Q6_K, whose tiles cost the most there (14336 x 4096 at eight rows: 22.6 against 28.4 us).
bool i8_batch_ok(const jitnn_hip_weight *w, int rows) {
    return g.gemv_i8 && rows >= 2 && rows <= (w->fmt == F_Q6_K ? 8 : 4) && gemv_i8_supported(w->fmt, w->k) && w->k <= 4096 && w->n >= 4 && w->nbytes < (1ll << 32) &&
           ((block_values(w->fmt) != 32 && w->fmt != F_Q2_K) || ((uintptr_t)w->dev & 3) == 0);
}

int launch_i8_batch(const jitnn_hip_weight *w, const float *x, int rows, const float *bias, float *y, hipStream_t stream) {
    I8Args a{};
    for (int i = 0; i < 3; ++i) {
        a.w[i] = w->dev;
        a.y[i] = y;
        a.bias[i] = bias;
    }
    a.n[0] = w->n;
    a.x = x;
    a.k = w->k;
    a.rows = rows;
    const int groups = (w->n + 3) / 4;
    // (us per launch by workgroups per CU / turns in flight, two rows - Q4_K 14336 x 4096: 10.4 (1 / 2) 10.3 (2 / 2) 10.6 (2 / 1) 11.6 (1 / 1)
    // 11.9 (3 / 1); Q4_0 11008 x 4096: 7.9 (1 / 2) 8.4 (2 / 1, 2 / 2) 8.6 (1 / 1); Q8_0 4096 x 4096: 6.4 (1 / 1) 6.7 (1 / 2) 6.9 (2 / 1) 7.7 (2 / 2);
    // four rows - Q4_K: 13.1 (1 / 2, 2 / 1) 14.0 (1 / 1); Q4_0: 10.6 (1 / 2) 10.9 (1 / 1) 11.0 (2 / 1); Q8_0: 7.1 (1 / 1) 7.7 (1 / 2) 9.1 (2 / 1))
    const int per_cu = 1, pf = (groups + g.cus - 1) / g.cus >= 8 ? 2 : 1;
    const int blocks = groups < g.cus * per_cu ? groups : g.cus * per_cu;
    if (!gemv_i8_launch(w->fmt, bias ? I8_BIAS : I8_PLAIN, pf, (unsigned)blocks, stream, a))
        return fail(JITNN_HIP_EDEVICE, "no INT8 GEMV kernel for format %d at %d rows of %d values", w->fmt, rows, a.k);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int launch_xreg(const XregCall &c, hipStream_t stream) {
    if (i8_ok(c) && !(c.norm_w && c.bias)) return launch_i8(c, stream);
    XregArgs a{};
    const int n = xreg_args(c, a);
    const int threads = XREG_THREADS, waves = threads / 64;
    int blocks = (n + waves - 1) / waves;
    // Two workgroups (eight waves) per CU measured best for streaming: fewer, longer row streams keep HBM pages
    // open.  A wave that sees many rows needs one row of prefetch; when it sees only a handful (a 14336-row
    // matrix gives a wave seven rows) a second row in flight covers the start-up latency.
    // Matrices of few rows (a wave sees two to four of them: attn_o, a 4096 x 4096 weight) do better with three
    // workgroups per CU and one row of prefetch: Q8_0 4096 x 4096 6.9 -> 6.5 us, attn_o of the 8B step 5.34 -> 5.25; from
    // 11008 rows on the two-workgroup shape is level or ahead (Q4_0 11008 x 4096 7.56 against 7.78 us).
    const bool few = n <= 8192 && !c.w2;
    const int cap = g.cus * (few ? 3 : 2);
    if (blocks > cap) blocks = cap;
    const int rows_per_wave = (n + blocks * waves - 1) / (blocks * waves);
    const int pf = few || rows_per_wave >= 16 ? 1 : 2;
    a.rpw = rows_per_wave;
    const int mode = c.w2 ? 3 : c.norm_w ? 2 : c.bias ? 1 : 0;
    xreg_fn fn = pick_xreg(c.w[0]->fmt, a.k % 64 == 0, mode, pf);
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(threads), 0, stream, a);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

typedef void (*xreg2_fn)(const XregArgs, const XregArgs, int);

// the pairs of K-quant formats a Q4_K_M / Q5_K_M layer mixes, first format < second
template <int PF>
xreg2_fn pick_xreg2_pf(int fa, int fb) {
    if (fa == F_Q4_K && fb == F_Q6_K) return gemv_xreg2_kernel<Unit<F_Q4_K>, 1, Unit<F_Q6_K>, 0, PF>;
    if (fa == F_Q4_K && fb == F_Q5_K) return gemv_xreg2_kernel<Unit<F_Q4_K>, 1, Unit<F_Q5_K>, 0, PF>;
    if (fa == F_Q5_K && fb == F_Q6_K) return gemv_xreg2_kernel<Unit<F_Q5_K>, 0, Unit<F_Q6_K>, 0, PF>;
    return nullptr;
}

bool xreg2_ok(int fa, int fb) { return pick_xreg2_pf<1>(fa < fb ? fa : fb, fa < fb ? fb : fa) != nullptr; }

// Two calls of different formats over the same normalised activations in one launch; the workgroups are shared out
// by the bytes each call streams.
int launch_xreg2(const XregCall &c0, const XregCall &c1, hipStream_t stream) {
    const bool swap = c0.w[0]->fmt > c1.w[0]->fmt;
    const XregCall &ca = swap ? c1 : c0, &cb = swap ? c0 : c1;
    if (i8_ok(ca) && i8_ok(cb) && ca.w[0]->k <= 4096 && gemv_i8_pair_supported(ca.w[0]->fmt, cb.w[0]->fmt)) {
        I8Args a{}, b{};
        const int ga = (i8_args(ca, a) + 3) / 4, gb = (i8_args(cb, b) + 3) / 4;
        const double ba = (double)ga * ca.w[0]->nbytes / ca.w[0]->n, bb = (double)gb * cb.w[0]->nbytes / cb.w[0]->n;
        int total, pf;
        i8_shape(ca.w[0]->fmt, ga + gb, (a.k + 1023) / 1024, false, total, pf);
        // (q, k | v of an 8B layer - 1536 row groups, six per CU -, us per launch by workgroups per CU / turns in flight: 6.7 (1 / 2)
        // 7.1 (1 / 1) 8.0 (2 / 1) 8.4 (2 / 2) 9.1 (3 / 1): the two formats' workgroups pace differently, one per CU keeps them apart)
        if (ga + gb >= 4 * g.cus) {
            total = g.cus;
            pf = 2;
        }
        if (total < 2) total = 2;
        int blocks_a = (int)(total * ba / (ba + bb) + 0.5);
        if (blocks_a < 1) blocks_a = 1;
        if (blocks_a > total - 1) blocks_a = total - 1;
        if (blocks_a > ga) blocks_a = ga;
        int blocks_b = total - blocks_a;
        if (blocks_b > gb) blocks_b = gb;
        if (!gemv_i8_pair_launch(ca.w[0]->fmt, cb.w[0]->fmt, pf > 2 ? 2 : pf, (unsigned)blocks_a, (unsigned)blocks_b, stream, a, b)) {
            // (a split the shared launch has no room for - three matrices of the first format, two of the second: a launch each)
            if (int rc = launch_i8(ca, stream)) return rc;
            return launch_i8(cb, stream);
        }
        HIP_TRY(hipGetLastError());
        return JITNN_HIP_OK;
    }
    XregArgs a{}, b{};
    const int na = xreg_args(ca, a), nb = xreg_args(cb, b);
    const int waves = XREG_THREADS / 64;
    const int cap = g.cus * 2;
    const double ba = (double)na * ca.w[0]->nbytes / ca.w[0]->n, bb = (double)nb * cb.w[0]->nbytes / cb.w[0]->n;
    int blocks_a = (int)(cap * ba / (ba + bb) + 0.5), blocks_b;
    if (blocks_a < 1) blocks_a = 1;
    if (blocks_a > cap - 1) blocks_a = cap - 1;
    blocks_b = cap - blocks_a;
    if (blocks_a > (na + waves - 1) / waves) blocks_a = (na + waves - 1) / waves;
    if (blocks_b > (nb + waves - 1) / waves) blocks_b = (nb + waves - 1) / waves;
    const int rpw_a = (na + blocks_a * waves - 1) / (blocks_a * waves), rpw_b = (nb + blocks_b * waves - 1) / (blocks_b * waves);
    // (one row of prefetch: the q, k | v launch of an 8B layer - 6144 rows, three per wave - 8.1 -> 7.7 us against two)
    const int pf = 1;
    a.rpw = rpw_a;
    b.rpw = rpw_b;
    xreg2_fn fn = pf == 1 ? pick_xreg2_pf<1>(ca.w[0]->fmt, cb.w[0]->fmt) : pick_xreg2_pf<2>(ca.w[0]->fmt, cb.w[0]->fmt);
    hipLaunchKernelGGL(fn, dim3(blocks_a + blocks_b), dim3(XREG_THREADS), 0, stream, a, b, blocks_a);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// Batch 1, rows of at most 4096 values: activations in registers, one row per wave iteration.
int launch_gemv_xreg(const jitnn_hip_weight *w, const float *x, const float *bias, float *y, hipStream_t stream) {
    XregCall c;
    c.w[0] = w;
    c.y[0] = y;
    c.bias = bias;
    c.x = x;
    return launch_xreg(c, stream);
}

template <int PF>
gemv1_fn pick_ksplit_pf(int fmt, bool pairs) {
    switch (fmt) {
    case F_Q4_0: return pairs ? gemv_ksplit_kernel<UnitPair<F_Q4_0>, 1, PF> : gemv_ksplit_kernel<Unit<F_Q4_0>, 1, PF>;
    case F_Q4_1: return pairs ? gemv_ksplit_kernel<UnitPair<F_Q4_1>, 1, PF> : gemv_ksplit_kernel<Unit<F_Q4_1>, 1, PF>;
    case F_Q8_0: return pairs ? gemv_ksplit_kernel<UnitPair<F_Q8_0>, 0, PF> : gemv_ksplit_kernel<Unit<F_Q8_0>, 0, PF>;
    case F_Q4_K: return gemv_ksplit_kernel<Unit<F_Q4_K>, 1, PF>;
    case F_Q5_K: return gemv_ksplit_kernel<Unit<F_Q5_K>, 0, PF>;
    default: return gemv_ksplit_kernel<Unit<F_Q6_K>, 0, PF>;
    }
}

size_t ksplit_lds(int fmt, int slices) {  // the single-block units need the most: 2 x 64 x (9 quads + 1 sum)
    if (block_values(fmt) == 32) return gemv_ksplit_lds_bytes<Unit<F_Q4_0>>(slices);
    return fmt == F_Q6_K ? gemv_ksplit_lds_bytes<Unit<F_Q6_K>>(slices) : gemv_ksplit_lds_bytes<Unit<F_Q4_K>>(slices);
}

// Batch 1, rows of 4097..32768 values: one wave per 4096-value slice of the row, partial sums joined in LDS.
int launch_gemv_ksplit(const jitnn_hip_weight *w, const float *x, const float *bias, float *y, hipStream_t stream) {
    {
        XregCall c;
        c.w[0] = w;
        c.y[0] = y;
        c.bias = bias;
        c.x = x;
        if (i8_ok(c)) return launch_i8(c, stream);
    }
    const int slices = (w->k + 4095) / 4096;
    const size_t lds = ksplit_lds(w->fmt, slices);
    int per_cu = (int)((g.lds_per_cu - 4096) / lds);  // workgroups of one CU by LDS
    if (per_cu < 1) per_cu = 1;
    const int waves_cap = 16 / slices > 0 ? 16 / slices : 1;  // at most 16 waves (4 per SIMD: the kernels use ~128 VGPRs)
    if (per_cu > waves_cap) per_cu = waves_cap;
    // One row of prefetch, and for matrices of few rows at most three workgroups per CU: the ffn_down of an 8B layer (Q6_K
    // 4096 x 14336, four waves per workgroup) 14.6 -> 14.2 us against four workgroups with two rows in flight each, Q5_K
    // 14.0 -> 13.0, Q4_K 4096 x 8192 8.45 -> 8.2; with many rows per workgroup more of them are better (Q4_K 14336 x 8192
    // 15.4 against 16.8 us with three).
    if (w->n <= 8192 && per_cu > 3) per_cu = 3;
    int blocks = w->n < g.cus * per_cu ? w->n : g.cus * per_cu;
    const int pf = 1;
    gemv1_fn fn = pf == 1 ? pick_ksplit_pf<1>(w->fmt, w->k % 64 == 0) : pick_ksplit_pf<2>(w->fmt, w->k % 64 == 0);
    if (int rc = allow_lds((const void *)fn, lds)) return rc;
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(64 * slices), lds, stream, w->dev, x, bias, y, w->n, w->k, g.nib);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

template <int PF, bool BIAS>
gemv1_fn pick_xreg_b2_fmt(int fmt, bool pairs) {
    switch (fmt) {
    case F_Q4_0: return pairs ? gemv_xreg_b2_kernel<UnitPair<F_Q4_0>, 1, PF, BIAS> : gemv_xreg_b2_kernel<Unit<F_Q4_0>, 1, PF, BIAS>;
    case F_Q4_1: return pairs ? gemv_xreg_b2_kernel<UnitPair<F_Q4_1>, 1, PF, BIAS> : gemv_xreg_b2_kernel<Unit<F_Q4_1>, 1, PF, BIAS>;
    case F_Q8_0: return pairs ? gemv_xreg_b2_kernel<UnitPair<F_Q8_0>, 0, PF, BIAS> : gemv_xreg_b2_kernel<Unit<F_Q8_0>, 0, PF, BIAS>;
    case F_Q4_K: return gemv_xreg_b2_kernel<Unit<F_Q4_K>, 1, PF, BIAS>;
    case F_Q5_K: return gemv_xreg_b2_kernel<Unit<F_Q5_K>, 0, PF, BIAS>;
    default: return gemv_xreg_b2_kernel<Unit<F_Q6_K>, 0, PF, BIAS>;
    }
}

// Batch 2, rows of at most 4096 values: both activation rows in registers.
int launch_gemv_xreg_b2(const jitnn_hip_weight *w, const float *x, const float *bias, float *y, hipStream_t stream) {
    const int waves = XREG_THREADS / 64;
    int blocks = (w->n + waves - 1) / waves;
    const int cap = g.cus * 2;
    if (blocks > cap) blocks = cap;
    const int rows_per_wave = (w->n + blocks * waves - 1) / (blocks * waves);
    const int pf = rows_per_wave >= 16 ? 1 : 2;
    const bool pairs = w->k % 64 == 0;
    gemv1_fn fn = bias ? (pf == 1 ? pick_xreg_b2_fmt<1, true>(w->fmt, pairs) : pick_xreg_b2_fmt<2, true>(w->fmt, pairs))
                       : (pf == 1 ? pick_xreg_b2_fmt<1, false>(w->fmt, pairs) : pick_xreg_b2_fmt<2, false>(w->fmt, pairs));
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(XREG_THREADS), 0, stream, w->dev, x, bias, y, w->n, w->k, g.nib);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// Batch 2..8, rows a multiple of 256 values long: block sums on the matrix cores, one workgroup of 8 waves per CU
// (the kernels live in gemv_mfma.hip).
int launch_gemv_mfma(const KernelRef &v, const jitnn_hip_weight *w, const float *x, int rows, const float *bias, float *y, hipStream_t stream) {
    if (int rc = allow_lds(v.fn, v.lds)) return rc;
    const int groups = (w->n + 15) / 16;
    const int blocks = groups < g.cus ? groups : g.cus;
    gemv_mfma_launch(w->fmt, (unsigned)blocks, stream, w->dev, x, bias, y, w->n, w->k, rows);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// Formats without a tuned kernel for this row count (Q5_0 and Q3_K left as they are, Q5_1 and Q2_K at more than one row or in
// shapes the INT8 kernel does not take): one wave per row on the bit-exact decoder.
int launch_gemv_plain(const jitnn_hip_weight *w, const float *x, int rows, const float *bias, float *y, hipStream_t stream) {
    int blocks = (w->n + 3) / 4;
    if (blocks > g.cus * 8) blocks = g.cus * 8;
    typedef void (*fn_t)(const uint8_t *, const float *, const float *, float *, int, int, int);
    fn_t fn = w->fmt == F_Q5_0 ? gemv_plain_kernel<F_Q5_0> : w->fmt == F_Q5_1 ? gemv_plain_kernel<F_Q5_1> : w->fmt == F_Q2_K ? gemv_plain_kernel<F_Q2_K>
                                                                                                                             : gemv_plain_kernel<F_Q3_K>;
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(256), 0, stream, w->dev, x, bias, y, w->n, w->k, rows);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int launch_gemv(const jitnn_hip_weight *w, const float *x, int rows, const float *bias, float *y, hipStream_t stream) {
    if (is_extra_format(w->fmt)) {
        if (rows == 1) {  // Q5_1 and Q2_K have units of the INT8 matrix-core kernel
            XregCall c;
            c.w[0] = w;
            c.y[0] = y;
            c.bias = bias;
            c.x = x;
            if (i8_ok(c)) return launch_i8(c, stream);
        } else if (i8_batch_ok(w, rows < 4 ? rows : 4)) {
            // up to four rows per launch; more rows - where the one-pass kernel of gemv_rows.h does not take the shape (it has tiles
            // for both formats: 14336 x 4096 at 5..8 rows Q5_1 23 us, Q2_K 19 us against 28, 29 as two launches here) - as a chain of
            // such launches, each streaming the weights again
            for (int r0 = 0; r0 < rows; r0 += 4)
                if (int rc = launch_i8_batch(w, x + (size_t)r0 * w->k, rows - r0 < 4 ? rows - r0 : 4, bias, y + (size_t)r0 * w->n, stream)) return rc;
            return JITNN_HIP_OK;
        }
        return launch_gemv_plain(w, x, rows, bias, y, stream);
    }
    if (i8_batch_ok(w, rows)) return launch_i8_batch(w, x, rows, bias, y, stream);
    if (rows == 2 && w->k <= 4096) return launch_gemv_xreg_b2(w, x, bias, y, stream);
    // Q6_K pays the most per weight on the matrix-core path (6-bit quants from two arrays, 16-value scale groups): up to
    // four rows its FP32 kernel is still ahead (measured: 33 vs 43 us at 2 rows, 151 vs 167 us at 4 rows on the output head)
    if (rows >= (w->fmt == F_Q6_K ? 5 : 2) && rows <= 8 && w->k % 256 == 0 && w->n >= 16) {
        const KernelRef v = gemv_mfma_kernel_ref(w->fmt);
        if (v.fn && v.lds <= g.max_lds) return launch_gemv_mfma(v, w, x, rows, bias, y, stream);
    }
    if (rows == 1) {
        if (w->k <= 4096) return launch_gemv_xreg(w, x, bias, y, stream);
        if (w->k <= 32768 && ksplit_lds(w->fmt, (w->k + 4095) / 4096) <= g.max_lds) return launch_gemv_ksplit(w, x, bias, y, stream);
    }
    GemvVariant v = pick(w->fmt, rows, w->k % 64 == 0);
    const int units = w->k / v.unit_values;
    const int steps = (units + 63) / 64;
    // stage as many steps as fit in 64 KiB (keeps several workgroups per CU); one step may need more
    int itc = (int)(65536 / v.lds_per_step);
    if (itc < 1) itc = 1;
    if (itc > steps) itc = steps;
    const size_t lds = v.lds_per_step * itc;
    if (lds > g.max_lds) return fail(JITNN_HIP_EINVAL, "GEMV needs %zu bytes of LDS, the device offers %zu", lds, g.max_lds);
    if (int rc = allow_lds((const void *)v.fn, lds)) return rc;
    // at least eight waves per CU: big LDS footprints leave room for one or two workgroups only, so those get 8 waves each
    int per_cu = (int)((g.lds_per_cu - 2048) / lds);
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 4) per_cu = 4;
    const int threads = per_cu >= 2 ? 256 : 512, waves = threads / 64;
    const int groups = (w->n + v.R - 1) / v.R;
    int blocks = (groups + waves - 1) / waves;
    const int cap = g.cus * per_cu;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(v.fn, dim3(blocks), dim3(threads), lds, stream, w->dev, x, bias, y, w->n, w->k, rows, itc, g.nib);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// Per-thread device scratch for the many-row path (FP16 activations and their row scales).  It only grows; a call
// on another stream than the last one first waits for the previous user, so concurrent streams of one thread
// cannot overwrite each other's activations.
struct Workspace {
    void *ptr = nullptr;
    size_t cap = 0;
    hipStream_t last = nullptr;
    hipEvent_t ev = nullptr;
    bool used = false;
};
thread_local Workspace g_ws;

// Where a many-row launch takes its scratch from: the calling thread's grow-only buffer (may allocate), or the
// library's static array (never allocates; the caller keeps calls on one GPU from overlapping).
enum ScratchSource { SCRATCH_THREAD, SCRATCH_STATIC };
void touch_thread_state();  // registers the calling thread's clean-up (defined below ThreadState)

int workspace(size_t bytes, hipStream_t stream, void **out, ScratchSource src = SCRATCH_THREAD) {
    if (src == SCRATCH_STATIC) {
        if (bytes > JITNN_HIP_SCRATCH_BYTES)
            return fail(JITNN_HIP_EINVAL, "this call needs %zu bytes of scratch; the entry point that allocates nothing has %llu", bytes,
                        (unsigned long long)JITNN_HIP_SCRATCH_BYTES);
        *out = g.scratch_ptr;
        return JITNN_HIP_OK;
    }
    Workspace &w = g_ws;
    touch_thread_state();  // a thread that only ever calls the device-pointer entry points must give its scratch back too
    if (!w.ev) HIP_TRY(hipEventCreateWithFlags(&w.ev, hipEventDisableTiming));
    if (bytes > w.cap) {
        if (w.ptr) HIP_TRY(hipFree(w.ptr));  // waits for the device: nobody is still reading the old block
        w.ptr = nullptr;
        w.cap = 0;
        const size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
        hipError_t e = hipMalloc(&w.ptr, want);
        if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipMalloc of %zu bytes of scratch: %s", want, hipGetErrorString(e));
        w.cap = want;
        w.used = false;
    }
    if (w.used && w.last != stream) HIP_TRY(hipStreamWaitEvent(stream, w.ev, 0));
    *out = w.ptr;
    return JITNN_HIP_OK;
}

int workspace_done(hipStream_t stream, ScratchSource src = SCRATCH_THREAD) {
    if (src == SCRATCH_STATIC) return JITNN_HIP_OK;
    Workspace &w = g_ws;
    HIP_TRY(hipEventRecord(w.ev, stream));
    w.last = stream;
    w.used = true;
    return JITNN_HIP_OK;
}

// Per-thread staging of the host-pointer entry points (jitnn_hip_linear, _dequantize, _quantize_q8_0, the model steps
// on host buffers): a pinned host buffer, a device buffer and a stream, all grow-only, so that a call costs copies and
// launches but no allocation.  Buffers beyond STAGE_KEEP_MAX are not kept (a dequantised matrix goes through in pieces).
constexpr size_t STAGE_KEEP_MAX = (size_t)128 << 20;
// 16-byte pieces from one buffer to another; one side is pinned host memory as the device sees it.  For the few KB of a
// GEMV call a launch costs less than a DMA transfer's set-up, and the bytes cross the bus in whole lines.
__global__ void __launch_bounds__(256) stage_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t count16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}
constexpr size_t STAGE_KERNEL_COPY_MAX = (size_t)1 << 20;  // above this a DMA transfer is as fast and leaves the compute units alone

struct HostStage {
    uint8_t *pinned = nullptr, *dev = nullptr;
    uint8_t *pinned_dev = nullptr;  // the pinned buffer's address on the device
    size_t pcap = 0, dcap = 0;
    hipStream_t stream = nullptr;
    void release() {
        if (pinned) (void)hipHostFree(pinned);
        if (dev) (void)hipFree(dev);
        if (stream) (void)hipStreamDestroy(stream);
        pinned = dev = pinned_dev = nullptr;
        pcap = dcap = 0;
        stream = nullptr;
    }
};
void release_workspace() {
    Workspace &w = g_ws;
    if (w.ptr) (void)hipFree(w.ptr);
    if (w.ev) (void)hipEventDestroy(w.ev);
    w = Workspace{};
}
struct ThreadState {
    HostStage stage;
    // A thread that ends gives its device memory back.  The process's first thread ends with the process, when the HIP
    // runtime may already be gone: its buffers are left to the process teardown.
    ~ThreadState() {
        if (is_main) return;
        stage.release();
        release_workspace();
    }
    bool is_main = false;
};
thread_local ThreadState g_thread;
bool calling_thread_is_main();
void touch_thread_state() { g_thread.is_main = calling_thread_is_main(); }

int stage_reserve(size_t pinned_bytes, size_t dev_bytes) {
    HostStage &st = g_thread.stage;
    g_thread.is_main = calling_thread_is_main();
    if (!st.stream) HIP_TRY(hipStreamCreateWithFlags(&st.stream, hipStreamNonBlocking));
    auto round = [](size_t b) { return (b + ((size_t)1 << 16) - 1) & ~(((size_t)1 << 16) - 1); };
    if (pinned_bytes > st.pcap) {
        if (st.pinned) HIP_TRY(hipHostFree(st.pinned));
        st.pinned = st.pinned_dev = nullptr;
        st.pcap = 0;
        const size_t want = round(pinned_bytes);
        hipError_t e = hipHostMalloc((void **)&st.pinned, want, hipHostMallocDefault);
        if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipHostMalloc of %zu bytes of staging: %s", want, hipGetErrorString(e));
        st.pcap = want;
        if (hipHostGetDevicePointer((void **)&st.pinned_dev, st.pinned, 0) != hipSuccess) {
            (void)hipGetLastError();
            st.pinned_dev = nullptr;  // not mapped: the DMA path is used
        }
    }
    if (dev_bytes > st.dcap) {
        if (st.dev) HIP_TRY(hipFree(st.dev));
        st.dev = nullptr;
        st.dcap = 0;
        const size_t want = round(dev_bytes);
        hipError_t e = hipMalloc((void **)&st.dev, want);
        if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipMalloc of %zu bytes of staging: %s", want, hipGetErrorString(e));
        st.dcap = want;
    }
    return JITNN_HIP_OK;
}

// More rows than the GEMV kernels take: FP16 activations in operand order + dequantise-to-LDS MFMA kernel.
// `count` weights of one row length share the activations x [rows, k] (prepared once): ys[i] = x ws[i]^T (+ bias, one
// weight only).  norm_w != nullptr: the RMSNorm in front of the linears is fused into the preparation (rows of at most
// XP_MAXK values; the caller checks with prefill_prepare_fuses_norm).
// residual != nullptr (one weight only): y = residual + x w^T, added by the join of the K slices, or, for a launch that
// does not split K, by a pass of its own over the product left in `tmp` [rows, n].
// part_ext / defer (one weight with a residual): the K slices go to part_ext ([8][rows, n] floats, the caller's) and, when the
// launch does split K, their join is left to the caller - *defer describes it, and the activation preparation of the next
// linears can do it on the way (pend: this call's activations are that pending row, not x).
int launch_prefill_group(const jitnn_hip_weight *const *ws, float *const *ys, int count, const float *x, int rows, const float *bias,
                         const float *norm_w, float eps, hipStream_t stream, const float *residual = nullptr, float *tmp = nullptr,
                         const float *swiglu_up = nullptr, ScratchSource src = SCRATCH_THREAD, float *part_ext = nullptr, PfPending *defer = nullptr,
                         const PfPending *pend = nullptr, PfGroupPending *gdefer = nullptr) {
    // (the kernels live in prefill_k.hip, prefill_q32.hip and prefill_mixed.hip)
    // Weights of one format - and a run of one K-quant format followed by a run of another for which a two-format kernel
    // exists - share a launch: their row tiles are numbered one after the other, so that the 1024-row k and v projections
    // fill the device together with q instead of splitting K eight ways each.
    struct Launch {
        int first, count, first_b;  // weights [first, first + count); first_b: where the second format starts (count: one format)
        int splits[3], split_steps[3];
        size_t part_bytes;
    } launch[4];
    int nlaunch = 0;
    if (count < 1 || count > 4) return fail(JITNN_HIP_EINVAL, "%d weights on one activation", count);
    if (residual && (count != 1 || !tmp || ws[0]->n % 4 != 0)) return fail(JITNN_HIP_EINVAL, "a residual needs one weight, rows of whole quads and a buffer");
    const int k = ws[0]->k;
    const int mtiles = (rows + PF_BM - 1) / PF_BM, mblocks = mtiles * (PF_BM / 32);  // operands padded to whole tiles of tokens
    const int nsteps = (k + PF_BK - 1) / PF_BK;
    auto kq = [](const jitnn_hip_weight *w) { return block_values(w->fmt) == 256; };
    auto tiles_of = [](const jitnn_hip_weight *w) { return (w->n + PF_BN - 1) / PF_BN; };
    for (int i = 0; i < count; ++i) {
        const jitnn_hip_weight *w = ws[i];
        if (w->k != k) return fail(JITNN_HIP_EINVAL, "weights of %d and %d values per row on one activation", k, w->k);
        const KernelRef kr = kq(w) ? prefill_kernel_k(w->fmt) : prefill_kernel_q32(w->fmt);
        if (!kr.fn) return fail(JITNN_HIP_EUNSUPPORTED, "no many-row kernel for format %d", w->fmt);
        if (int rc = allow_lds(kr.fn, kr.lds)) return rc;
    }
    for (int i = 0; i < count;) {
        Launch &l = launch[nlaunch++];
        l.first = i;
        int j = i + 1;
        const bool joinable = !bias && !residual;  // (several weights: partial sums of all of them are joined by one kernel)
        while (joinable && j < count && j - i < 3 && ws[j]->fmt == ws[i]->fmt && ws[j]->n % 4 == 0 && ws[i]->n % 4 == 0) ++j;
        l.first_b = j - i;
        if (joinable && j < count && j - i < 3 && ws[j]->fmt != ws[i]->fmt && ws[i]->n % 4 == 0 && ws[j]->n % 4 == 0) {
            const KernelRef kr = prefill_kernel_mixed(ws[i]->fmt, ws[j]->fmt);
            if (kr.fn) {
                if (int rc = allow_lds(kr.fn, kr.lds)) return rc;
                const int fb = ws[j]->fmt;
                while (j < count && j - i < 3 && ws[j]->fmt == fb && ws[j]->n % 4 == 0) ++j;
            }
        }
        l.count = j - i;
        int tiles = 0;
        size_t nsum = 0;
        for (int q = i; q < j; ++q) {
            tiles += tiles_of(ws[q]);
            nsum += (size_t)ws[q]->n;
        }
        // A launch that would leave most CUs idle (few, large tiles) splits K: every slice of at least 8 steps writes its
        // own partial y, a second kernel adds the slices in order.
        int splits = 1;
        if (nsum % 4 == 0 && ws[i]->n % 4 == 0) {
            while (splits < 8 && tiles * mtiles * splits * 2 <= g.cus && nsteps / (splits * 2) >= PREFILL_MIN_SLICE) splits *= 2;
        }
        int wgs = tiles * mtiles * splits;
        l.part_bytes = 0;
        for (int q = 0; q < l.count; ++q) {
            const jitnn_hip_weight *wq = ws[i + q];
            l.splits[q] = splits;
            // the second format of a two-format launch (Q6_K beside Q4_K or Q5_K) takes half as long again per step: its
            // tiles get slices half as long where the device has the room, so that the launch does not wait for them
            if (q >= l.first_b && splits > 1 && splits < 8 && wgs + tiles_of(wq) * mtiles * splits <= g.cus && nsteps / (splits * 2) >= PREFILL_MIN_SLICE) {
                l.splits[q] = splits * 2;
                wgs += tiles_of(wq) * mtiles * splits;
            }
            // slices of the 256-value formats start on whole blocks (four steps): the kernel stages their raw bytes by block
            l.split_steps[q] = (nsteps + l.splits[q] - 1) / l.splits[q];
            if (kq(wq)) l.split_steps[q] = (l.split_steps[q] + 3) & ~3;
            if (l.splits[q] > 1) l.part_bytes += (size_t)l.splits[q] * rows * wq->n * 4;
        }
        i = j;
    }
    size_t part_max = 0;
    for (int i = 0; i < nlaunch; ++i) part_max = std::max(part_max, launch[i].part_bytes);
    const size_t xo_bytes = (size_t)mblocks * pf_ksteps(k) * 1024;
    const size_t scale_bytes = ((size_t)rows * 8 + 255) & ~(size_t)255;
    void *wsp = nullptr;
    if (int rc = workspace(xo_bytes + scale_bytes + part_max, stream, &wsp, src)) return rc;
    _Float16 *xo = (_Float16 *)wsp;
    float *scale = (float *)((uint8_t *)wsp + xo_bytes), *inv = scale + rows;
    float *part = part_ext && count == 1 && residual ? part_ext : (float *)((uint8_t *)wsp + xo_bytes + scale_bytes);
    prefill_prepare_launch(x, scale, inv, xo, rows, k, mblocks, norm_w, eps, swiglu_up, stream, pend);
    for (int li = 0; li < nlaunch; ++li) {
        const Launch &l = launch[li];
        const jitnn_hip_weight *w = ws[l.first];
        const bool split = l.splits[0] > 1;  // (the segments of a launch split together or not at all)
        PfSegments sg{}, out{};
        for (int q = 0; q < 3; ++q) sg.splits[q] = out.splits[q] = 1;
        size_t before = 0;  // floats of partial sums of the segments before this one
        unsigned gx = 0;
        for (int q = 0; q < l.count; ++q) {
            const jitnn_hip_weight *wq = ws[l.first + q];
            sg.W[q] = wq->dev;
            sg.n[q] = wq->n;
            sg.tiles[q] = tiles_of(wq);
            sg.splits[q] = l.splits[q];
            sg.split_steps[q] = l.split_steps[q];
            sg.y[q] = split ? part + before : (residual ? tmp : ys[l.first + q]);
            before += (size_t)l.splits[q] * rows * wq->n;
            gx += (unsigned)(sg.tiles[q] * sg.splits[q]);
            out.y[q] = ys[l.first + q];
            out.n[q] = wq->n;
            out.splits[q] = l.splits[q];
        }
        const float *b1 = split ? nullptr : bias;
        const dim3 grid(gx, mtiles);
        if (l.first_b < l.count) prefill_launch_mixed(w->fmt, ws[l.first + l.first_b]->fmt, l.first_b, grid, stream, sg, xo, inv, rows, k);
        else if (kq(w)) prefill_launch_k(w->fmt, grid, stream, sg, xo, inv, b1, rows, k);
        else prefill_launch_q32(w->fmt, grid, stream, sg, xo, inv, b1, rows, k);
        if (split && l.count > 1 && gdefer && nlaunch == 1) {
            // the caller's next kernel adds the slices up as it reads them (they stay in this thread's scratch until its
            // next many-row call)
            gdefer->part = part;
            gdefer->sg = out;
        } else if (split && l.count > 1) {  // (the stream orders the next launch's partial sums after this join)
            size_t count4 = 0;
            for (int q = 0; q < l.count; ++q) count4 += (size_t)rows * sg.n[q] / 4;
            const unsigned blocks = (unsigned)std::min<size_t>((count4 + 255) / 256, (size_t)g.cus * 8);
            prefill_join_group_launch(part, out, rows, blocks, stream);
        } else if (split && defer && part == part_ext && !bias) {  // the join rides with the next activation preparation
            defer->part = part;
            defer->res = residual;
            defer->out = ys[l.first];
            defer->splits = l.splits[0];
            defer->n = w->n;
        } else if (split) {
            const size_t count4 = (size_t)rows * w->n / 4;
            const unsigned blocks = (unsigned)std::min<size_t>((count4 + 255) / 256, (size_t)g.cus * 8);
            prefill_join_launch(part, bias, residual, ys[l.first], count4, w->n, l.splits[0], blocks, stream);
        } else if (residual) {
            const size_t count4 = (size_t)rows * w->n / 4;
            const unsigned blocks = (unsigned)std::min<size_t>((count4 + 255) / 256, (size_t)g.cus * 8);
            hipLaunchKernelGGL(add_rows_kernel, dim3(blocks), dim3(256), 0, stream, reinterpret_cast<const float4 *>(tmp),
                               reinterpret_cast<const float4 *>(residual), reinterpret_cast<float4 *>(ys[l.first]), count4);
        }
    }
    HIP_TRY(hipGetLastError());
    return workspace_done(stream, src);
}

// h [rows, n] = silu(n(x) gate^T) * (n(x) up^T), n = RMSNorm with norm_w (which must fit the fused preparation): the gate
// and the up projection of a Llama FFN as one product whose epilogue forms the SwiGLU - the two [rows, n] products are
// neither stored nor read back.  pend: as in launch_prefill_group.
bool prefill_dual_ok(const jitnn_hip_weight *gate, const jitnn_hip_weight *up) {
    return gate->fmt == up->fmt && gate->n == up->n && gate->k == up->k && !is_extra_format(gate->fmt) &&
           prefill_prepare_fuses_norm(gate->k);
}

int launch_prefill_dual(const jitnn_hip_weight *gate, const jitnn_hip_weight *up, float *h, const float *x, int rows, const float *norm_w, float eps,
                        hipStream_t stream, const PfPending *pend) {
    const bool kq = block_values(gate->fmt) == 256;
    const KernelRef kr = kq ? prefill_kernel_dual_k(gate->fmt) : prefill_kernel_dual_q32(gate->fmt);
    if (!kr.fn) return fail(JITNN_HIP_EUNSUPPORTED, "no many-row kernel for format %d", gate->fmt);
    if (int rc = allow_lds(kr.fn, kr.lds)) return rc;
    const int k = gate->k, n = gate->n;
    const int mtiles = (rows + PF_BM - 1) / PF_BM, mblocks = mtiles * (PF_BM / 32);
    const size_t xo_bytes = (size_t)mblocks * pf_ksteps(k) * 1024;
    const size_t scale_bytes = ((size_t)rows * 8 + 255) & ~(size_t)255;
    void *wsp = nullptr;
    if (int rc = workspace(xo_bytes + scale_bytes, stream, &wsp, SCRATCH_THREAD)) return rc;
    _Float16 *xo = (_Float16 *)wsp;
    float *scale = (float *)((uint8_t *)wsp + xo_bytes), *inv = scale + rows;
    prefill_prepare_launch(x, scale, inv, xo, rows, k, mblocks, norm_w, eps, nullptr, stream, pend);
    const dim3 grid((unsigned)((n + PF_BN / 2 - 1) / (PF_BN / 2)), mtiles);
    if (kq) prefill_launch_dual_k(gate->fmt, grid, stream, gate->dev, up->dev, xo, inv, h, rows, n, k);
    else prefill_launch_dual_q32(gate->fmt, grid, stream, gate->dev, up->dev, xo, inv, h, rows, n, k);
    HIP_TRY(hipGetLastError());
    return workspace_done(stream, SCRATCH_THREAD);
}

int launch_prefill(const jitnn_hip_weight *w, const float *x, int rows, const float *bias, float *y, hipStream_t stream,
                   ScratchSource src = SCRATCH_THREAD) {
    return launch_prefill_group(&w, &y, 1, x, rows, bias, nullptr, 0.f, stream, nullptr, nullptr, nullptr, src);
}

template <int FMT>
void launch_dequant(const jitnn_hip_weight *w, float *y, hipStream_t stream) {
    const size_t quads = (size_t)w->n * w->k / 4;
    size_t blocks = (quads + 255) / 256;
    const size_t cap = (size_t)g.cus * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(dequant_kernel<FMT>, dim3((unsigned)blocks), dim3(256), 0, stream, w->dev, y, quads);
}

int check_weight_args(int fmt, long long nbytes, int n, int k, const void *blocks, jitnn_hip_weight **out) {
    if (!out) return fail(JITNN_HIP_EINVAL, "out is NULL");
    *out = nullptr;
    if (!blocks) return fail(JITNN_HIP_EINVAL, "blocks is NULL");
    long long need = jitnn_hip_weight_nbytes(fmt, n, k);
    if (need < 0) return (int)need;
    if (nbytes != need)
        return fail(JITNN_HIP_EINVAL, "format %d weight of shape [%d, %d] needs %lld bytes, got %lld", fmt, n, k, need, nbytes);
    return JITNN_HIP_OK;
}

}  // namespace

// ================================================================================================ C ABI

extern "C" {

const char *jitnn_hip_last_error(void) { return g_err; }

int jitnn_hip_block_values(int fmt) { return block_values(fmt); }
int jitnn_hip_block_bytes(int fmt) { return block_bytes(fmt); }

long long jitnn_hip_weight_nbytes(int fmt, long long n, long long k) {
    if (!known(fmt)) return fail(JITNN_HIP_EINVAL, "ggml type id %d is not one of Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K", fmt);
    if (n < 1 || k < 1) return fail(JITNN_HIP_EINVAL, "weight shape [%lld, %lld] is empty", n, k);
    if (k % block_values(fmt) != 0)
        return fail(JITNN_HIP_EINVAL, "format %d weight of shape [%lld, %lld]: last axis not a multiple of its block of %d", fmt, n, k,
                    block_values(fmt));
    if (n > 0x7fffffffLL || k > 0x7fffffffLL || n * k > 0x7fffffffLL)  // the reference's tensors hold at most Integer.MAX_VALUE values
        return fail(JITNN_HIP_EINVAL, "weight shape [%lld, %lld] holds more than 2^31-1 values", n, k);
    return n * (k / block_values(fmt)) * block_bytes(fmt);
}

int jitnn_hip_init(int device_ordinal) {
    std::lock_guard<std::mutex> lock(g_mu);
    if (g.ready) {
        if (device_ordinal != g.device) return fail(JITNN_HIP_EINVAL, "already initialised on device %d", g.device);
        return JITNN_HIP_OK;
    }
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) return fail(JITNN_HIP_ENODEVICE, "no HIP device: %s", hipGetErrorString(e));
    if (device_ordinal < 0 || device_ordinal >= count) return fail(JITNN_HIP_EINVAL, "device %d of %d", device_ordinal, count);
    HIP_TRY(hipSetDevice(device_ordinal));
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, device_ordinal));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return fail(JITNN_HIP_ENODEVICE, "device %d is %s; this library holds gfx950 code only", device_ordinal, p.gcnArchName);
    snprintf(g.name, sizeof g.name, "%s (%s)", p.name, p.gcnArchName);
    g.cus = p.multiProcessorCount;
    g.hbm = (long long)p.totalGlobalMem;
    int optin = 0;
    if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, device_ordinal) != hipSuccess || optin <= 0)
        optin = (int)p.sharedMemPerBlock;
    g.max_lds = (size_t)optin;
    g.lds_per_cu = p.maxSharedMemoryPerMultiProcessor > 0 ? (size_t)p.maxSharedMemoryPerMultiProcessor : g.max_lds;
    float *probe = nullptr;
    HIP_TRY(hipMalloc(&probe, 2 * sizeof(float)));
    hipLaunchKernelGGL(fp8_probe_kernel, dim3(1), dim3(1), 0, 0, probe);
    float h[2] = {0, 0};
    hipError_t ce = hipMemcpy(h, probe, sizeof h, hipMemcpyDeviceToHost);
    (void)hipFree(probe);
    if (ce != hipSuccess) return fail(JITNN_HIP_EDEVICE, "fp8 probe: %s", hipGetErrorString(ce));
    if (!(h[0] > 0.f) || h[1] != 15.f * h[0])
        return fail(JITNN_HIP_EDEVICE, "fp8 probe: E4M3 bytes 0x01, 0x0f decode to %g, %g; expected q * 2^-9 or q * 2^-10", h[0], h[1]);
    g.nib = 1.f / h[0];
    {   // the device address of the static scratch on this GPU (every GPU holds its own copy at its own address)
        void *sp = nullptr;
        hipError_t se = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));
        if (se != hipSuccess || !sp) return fail(JITNN_HIP_EDEVICE, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(se));
        g.scratch_ptr = sp;
    }
    if (const char *e = getenv("JITNN_HIP_GEMV_MAX_ROWS")) {
        int v = atoi(e);
        if (v >= 1) g.gemv_max_rows = v;
    }
    if (const char *e = getenv("JITNN_HIP_GEMV_I8")) g.gemv_i8 = atoi(e) != 0;
    if (const char *e = getenv("JITNN_HIP_TRANSCODE")) g.transcode = atoi(e) != 0;
    g.device = device_ordinal;
    g.ready = true;
    return JITNN_HIP_OK;
}

int jitnn_hip_device_info(char *name, int cap, int *compute_units, long long *hbm_bytes) {
    if (int rc = check_ready()) return rc;
    if (name && cap > 0) {
        strncpy(name, g.name, (size_t)cap - 1);
        name[cap - 1] = 0;
    }
    if (compute_units) *compute_units = g.cus;
    if (hbm_bytes) *hbm_bytes = g.hbm;
    return JITNN_HIP_OK;
}

int jitnn_hip_sync(void) {
    if (int rc = check_ready()) return rc;
    HIP_TRY(hipDeviceSynchronize());
    return JITNN_HIP_OK;
}

int jitnn_hip_stats(jitnn_hip_stat *out, int cap) {
    if (cap > 0 && !out) return fail(JITNN_HIP_EINVAL, "output is NULL");
    for (int i = 0; i < ST_COUNT && i < cap; ++i) {
        std::snprintf(out[i].name, sizeof(out[i].name), "%s", kStatNames[i]);
        out[i].calls = g_stat_calls[i].load(std::memory_order_relaxed);
        out[i].tensor_bytes = g_stat_bytes[i].load(std::memory_order_relaxed);
    }
    return ST_COUNT;
}

int jitnn_hip_stats_reset(void) {
    for (int i = 0; i < ST_COUNT; ++i) {
        g_stat_calls[i].store(0, std::memory_order_relaxed);
        g_stat_bytes[i].store(0, std::memory_order_relaxed);
    }
    return JITNN_HIP_OK;
}

int jitnn_hip_weight_upload(int fmt, const void *blocks_host, long long nbytes, int n, int k, jitnn_hip_weight **out) {
    if (int rc = check_weight_args(fmt, nbytes, n, k, blocks_host, out)) return rc;
    if (int rc = check_ready()) return rc;
    uint8_t *dev = nullptr;
    hipError_t e = hipMalloc(&dev, (size_t)nbytes);
    if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipMalloc of %lld bytes: %s", nbytes, hipGetErrorString(e));
    e = hipMemcpy(dev, blocks_host, (size_t)nbytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail(JITNN_HIP_EDEVICE, "hipMemcpy of %lld bytes: %s", nbytes, hipGetErrorString(e));
    }
    // Q5_0 and Q3_K have no kernels of their own but hold exactly the values of Q8_0 / Q6_K blocks (dequant.h): rewritten
    // once, here, they run on those formats' kernels with the same results, bit for bit where the dequantiser is concerned
    int dev_fmt = fmt;
    long long dev_nbytes = nbytes;
    if (g.transcode && (fmt == F_Q5_0 || fmt == F_Q3_K)) {
        dev_fmt = fmt == F_Q5_0 ? F_Q8_0 : F_Q6_K;
        dev_nbytes = jitnn_hip_weight_nbytes(dev_fmt, n, k);
        uint8_t *dev2 = nullptr;
        e = hipMalloc(&dev2, (size_t)dev_nbytes);
        if (e != hipSuccess) {
            (void)hipFree(dev);
            return fail(JITNN_HIP_ENOMEM, "hipMalloc of %lld bytes: %s", dev_nbytes, hipGetErrorString(e));
        }
        const size_t blocks = (size_t)n * k / block_values(fmt);
        const unsigned grid = (unsigned)std::min<size_t>((blocks + 255) / 256, (size_t)g.cus * 16);
        if (fmt == F_Q5_0) hipLaunchKernelGGL(transcode_q5_0_to_q8_0_kernel, dim3(grid), dim3(256), 0, nullptr, dev, dev2, blocks);
        else hipLaunchKernelGGL(transcode_q3_k_to_q6_k_kernel, dim3(grid), dim3(256), 0, nullptr, dev, dev2, blocks);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
        (void)hipFree(dev);
        dev = dev2;
        if (e != hipSuccess) {
            (void)hipFree(dev);
            return fail(JITNN_HIP_EDEVICE, "rewriting the blocks: %s", hipGetErrorString(e));
        }
    }
    jitnn_hip_weight *w = new (std::nothrow) jitnn_hip_weight{dev_fmt, n, k, dev_nbytes, dev, true};
    if (!w) {
        (void)hipFree(dev);
        return fail(JITNN_HIP_ENOMEM, "out of host memory");
    }
    if (dev_fmt != fmt) {
        w->file_fmt = fmt;
        w->file_nbytes = nbytes;
    }
    *out = w;
    return JITNN_HIP_OK;
}

int jitnn_hip_weight_wrap_dev(int fmt, const void *dev_blocks, long long nbytes, int n, int k, jitnn_hip_weight **out) {
    if (int rc = check_weight_args(fmt, nbytes, n, k, dev_blocks, out)) return rc;
    if (((uintptr_t)dev_blocks & 15) != 0) return fail(JITNN_HIP_EINVAL, "device blocks must be 16-byte aligned");
    jitnn_hip_weight *w = new (std::nothrow) jitnn_hip_weight{fmt, n, k, nbytes, (uint8_t *)dev_blocks, false};
    if (!w) return fail(JITNN_HIP_ENOMEM, "out of host memory");
    *out = w;
    return JITNN_HIP_OK;
}

int jitnn_hip_weight_free(jitnn_hip_weight *w) {
    if (!w) return JITNN_HIP_OK;
    int rc = JITNN_HIP_OK;
    if (w->owned && w->dev) {
        hipError_t e = hipFree(w->dev);
        if (e != hipSuccess) rc = fail(JITNN_HIP_EDEVICE, "hipFree: %s", hipGetErrorString(e));
    }
    delete w;
    return rc;
}

int jitnn_hip_weight_info(const jitnn_hip_weight *w, int *fmt, int *n, int *k, long long *nbytes) {
    if (!w) return fail(JITNN_HIP_EINVAL, "weight is NULL");
    if (fmt) *fmt = w->file_fmt ? w->file_fmt : w->fmt;  // (the caller's format and byte count, also where the device copy is another)
    if (n) *n = w->n;
    if (k) *k = w->k;
    if (nbytes) *nbytes = w->file_fmt ? w->file_nbytes : w->nbytes;
    return JITNN_HIP_OK;
}

int jitnn_hip_dequantize_dev(const jitnn_hip_weight *w, float *y_dev, void *stream) {
    if (!w || !y_dev) return fail(JITNN_HIP_EINVAL, "weight or output is NULL");
    if (int rc = check_ready()) return rc;
    hipStream_t s = (hipStream_t)stream;
    count_op(ST_DEQUANT, (long long)w->nbytes + 4ll * w->n * w->k);
    switch (w->fmt) {
    case F_Q4_0: launch_dequant<F_Q4_0>(w, y_dev, s); break;
    case F_Q4_1: launch_dequant<F_Q4_1>(w, y_dev, s); break;
    case F_Q8_0: launch_dequant<F_Q8_0>(w, y_dev, s); break;
    case F_Q4_K: launch_dequant<F_Q4_K>(w, y_dev, s); break;
    case F_Q5_K: launch_dequant<F_Q5_K>(w, y_dev, s); break;
    case F_Q5_0: launch_dequant<F_Q5_0>(w, y_dev, s); break;
    case F_Q5_1: launch_dequant<F_Q5_1>(w, y_dev, s); break;
    case F_Q2_K: launch_dequant<F_Q2_K>(w, y_dev, s); break;
    case F_Q3_K: launch_dequant<F_Q3_K>(w, y_dev, s); break;
    default: launch_dequant<F_Q6_K>(w, y_dev, s); break;
    }
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_dequantize(const jitnn_hip_weight *w, float *y_host) {
    if (!w || !y_host) return fail(JITNN_HIP_EINVAL, "weight or output is NULL");
    if (int rc = check_ready()) return rc;
    // in pieces of whole rows through the thread's device buffer: no allocation per call, bounded memory for any matrix
    const size_t row_out = (size_t)w->k * sizeof(float), row_in = (size_t)w->nbytes / w->n;
    size_t piece_rows = ((size_t)64 << 20) / row_out;
    if (piece_rows < 1) piece_rows = 1;
    if (piece_rows > (size_t)w->n) piece_rows = (size_t)w->n;
    if (int rc = stage_reserve(0, piece_rows * row_out)) return rc;
    HostStage &st = g_thread.stage;
    count_op(ST_DEQUANT, (long long)w->nbytes + 4ll * w->n * w->k);
    StatNest nest;
    for (size_t r0 = 0; r0 < (size_t)w->n; r0 += piece_rows) {
        const size_t nr = std::min(piece_rows, (size_t)w->n - r0);
        const jitnn_hip_weight part{w->fmt, (int)nr, w->k, (long long)(nr * row_in), w->dev + r0 * row_in, false};
        if (int rc = jitnn_hip_dequantize_dev(&part, (float *)st.dev, st.stream)) return rc;
        HIP_TRY(hipMemcpyAsync((uint8_t *)y_host + r0 * row_out, st.dev, nr * row_out, hipMemcpyDeviceToHost, st.stream));
        HIP_TRY(hipStreamSynchronize(st.stream));
    }
    return JITNN_HIP_OK;
}

}  // extern "C"

namespace {

// Does a linear of `rows` rows on this weight take the one-pass kernel of gemv_rows.h?  From 9 rows; rows of 12288 values and
// more - the ffn_down of an 8B layer, 4096 x 14336 - from 3: Q6_K 35.6 against 41.5-44.6 us, Q4_K 24.5 against 26.6-27.6,
// Q4_0 22.3 against 25.4, Q8_0 27.2 against 34.4, where the kernels for up to 8 rows pay their activation set-up per
// 4096-value slice (at 8192 values they are still ahead, 15.0 against 16.9).  Q4_0 and Q4_1 with shorter rows from 12: their
// kernels for up to 8 rows are the fastest of all, and 8 + 1..3 rows in two passes still beat the one pass (14336 x 4096
// Q4_0 at 9 rows 21.9 against 27.0 us, at 12 rows 26.2 against 27.0, at 20 rows 38.9 against 29.9).
bool rows_path(const jitnn_hip_weight *w, int rows) {
    int rows_min = 9;  // (up to 8 rows gemv_mfma_kernel is faster)
    if (w->k >= 12288) rows_min = 3;
    else if (w->fmt == F_Q4_0 || w->fmt == F_Q4_1) rows_min = 12;
    else if (is_extra_format(w->fmt)) rows_min = 5;  // (Q5_1, Q2_K: up to four rows are one launch of the INT8 kernel)
    return rows >= rows_min && rows <= 64 && rows <= g.gemv_max_rows && gemv_rows_supported(w->fmt) && w->k % 256 == 0 &&
           w->n >= 16;
}

// ys[i] = x ws[i]^T (+ bias) (+ residual [rows, n]; bias and residual with one weight only) for weights that all pass
// rows_path: the activation operands are prepared once per granularity of block sums and shared by the weights.
// swiglu_up: the activations are silu(x) * swiglu_up, formed by the preparation as it reads x.
int launch_rows_group(const jitnn_hip_weight *const *ws, float *const *ys, int count, const float *x, int rows, const float *bias, const float *residual,
                      hipStream_t s, ScratchSource src, const float *swiglu_up = nullptr) {
    const int k = ws[0]->k;
    bool need[GR_LAYOUTS] = {};  // the operand layouts the weights ask for
    for (int i = 0; i < count; ++i) {
        if (ws[i]->k != k) return fail(JITNN_HIP_EINVAL, "weights of %d and %d values per row on one activation", k, ws[i]->k);
        const KernelRef kr = gemv_rows_kernel_ref(ws[i]->fmt, ws[i]->n, k, rows, (unsigned)g.cus);
        if (int rc = allow_lds(kr.fn, kr.lds)) return rc;
        need[gemv_rows_layout(ws[i]->fmt)] = true;
    }
    const size_t one = (gemv_rows_scratch_bytes(rows, k) + 255) & ~(size_t)255;
    void *scratch = nullptr;
    int layouts = 0;
    for (int l = 0; l < GR_LAYOUTS; ++l) layouts += need[l];
    if (int rc = workspace(one * layouts, s, &scratch, src)) return rc;
    uint8_t *sc[GR_LAYOUTS] = {};
    for (int l = 0, used = 0; l < GR_LAYOUTS; ++l)
        if (need[l]) sc[l] = (uint8_t *)scratch + one * used++;
    gemv_rows_prepare_launch(s, x, swiglu_up, (void *const *)sc, k, rows);
    for (int i = 0; i < count; ++i)
        gemv_rows_main_launch(ws[i]->fmt, (unsigned)g.cus, s, ws[i]->dev, sc[gemv_rows_layout(ws[i]->fmt)], bias, residual, ys[i], ws[i]->n, k, rows);
    HIP_TRY(hipGetLastError());
    return workspace_done(s, src);
}

int linear_dev(const jitnn_hip_weight *w, const float *x_dev, int rows, const float *bias_dev, float *y_dev, hipStream_t s, ScratchSource src) {
    if (!w || !x_dev || !y_dev) return fail(JITNN_HIP_EINVAL, "weight, input or output is NULL");
    if (rows < 1) return fail(JITNN_HIP_EINVAL, "rows = %d", rows);
    if (int rc = check_ready()) return rc;
    const bool many = rows > g.gemv_max_rows && has_many_row_kernel(w->fmt);
    count_op(many ? ST_MFMA : ST_GEMV, (long long)w->nbytes + 4ll * rows * ((long long)w->k + w->n) + (bias_dev ? 4ll * w->n : 0));
    if (many) return launch_prefill(w, x_dev, rows, bias_dev, y_dev, s, src);
    // several rows, rows of whole 256-value columns: every row meets the weights in one pass over them (gemv_rows.h)
    if (rows_path(w, rows)) return launch_rows_group(&w, &y_dev, 1, x_dev, rows, bias_dev, nullptr, s, src);
    for (int r0 = 0; r0 < rows; r0 += 8) {
        const int nb = rows - r0 < 8 ? rows - r0 : 8;
        if (int rc = launch_gemv(w, x_dev + (size_t)r0 * w->k, nb, bias_dev, y_dev + (size_t)r0 * w->n, s)) return rc;
    }
    return JITNN_HIP_OK;
}

}  // namespace

extern "C" {

int jitnn_hip_linear_dev(const jitnn_hip_weight *w, const float *x_dev, int rows, const float *bias_dev, float *y_dev, void *stream) {
    return linear_dev(w, x_dev, rows, bias_dev, y_dev, (hipStream_t)stream, SCRATCH_THREAD);
}

int jitnn_hip_linear_noalloc_dev(const jitnn_hip_weight *w, const float *x_dev, int rows, const float *bias_dev, float *y_dev, void *stream) {
    return linear_dev(w, x_dev, rows, bias_dev, y_dev, (hipStream_t)stream, SCRATCH_STATIC);
}

long long jitnn_hip_noalloc_scratch_bytes(void) { return (long long)JITNN_HIP_SCRATCH_BYTES; }

int jitnn_hip_linear(const jitnn_hip_weight *w, const float *x_host, int rows, const float *bias_host, float *y_host) {
    if (!w || !x_host || !y_host) return fail(JITNN_HIP_EINVAL, "weight, input or output is NULL");
    if (rows < 1) return fail(JITNN_HIP_EINVAL, "rows = %d", rows);
    if (int rc = check_ready()) return rc;
    // layout of both staging buffers: [x | bias | y], x and bias going up in one copy, y coming back in one
    const size_t xb = (size_t)rows * w->k * 4, yb = (size_t)rows * w->n * 4, bb = bias_host ? (size_t)w->n * 4 : 0;
    const size_t bo = (xb + 255) & ~(size_t)255, yo = bo + ((bb + 255) & ~(size_t)255), total = yo + yb;
    const bool keep = total <= STAGE_KEEP_MAX;  // small calls go through pinned memory (one DMA each way, no page locking per call)
    if (int rc = stage_reserve(keep ? total : 0, total)) return rc;
    HostStage &st = g_thread.stage;
    // small calls: the device itself fetches the input from the pinned buffer and writes the result back into it
    const bool by_kernel = keep && st.pinned_dev && total <= STAGE_KERNEL_COPY_MAX;
    auto copy16 = [&](uint8_t *dst, const uint8_t *src, size_t bytes) {
        const size_t count16 = (bytes + 15) / 16;  // the sections of the layout are 256-byte aligned: rounding up stays inside
        const unsigned blocks = (unsigned)std::min<size_t>((count16 + 255) / 256, 64);
        hipLaunchKernelGGL(stage_copy_kernel, dim3(blocks), dim3(256), 0, st.stream, (uint4 *)dst, (const uint4 *)src, count16);
    };
    if (keep) {
        memcpy(st.pinned, x_host, xb);
        if (bias_host) memcpy(st.pinned + bo, bias_host, bb);
        const size_t up = bias_host ? bo + bb : xb;
        if (by_kernel) copy16(st.dev, st.pinned_dev, up);
        else HIP_TRY(hipMemcpyAsync(st.dev, st.pinned, up, hipMemcpyHostToDevice, st.stream));
    } else {
        HIP_TRY(hipMemcpyAsync(st.dev, x_host, xb, hipMemcpyHostToDevice, st.stream));
        if (bias_host) HIP_TRY(hipMemcpyAsync(st.dev + bo, bias_host, bb, hipMemcpyHostToDevice, st.stream));
    }
    int rc = jitnn_hip_linear_dev(w, (const float *)st.dev, rows, bias_host ? (const float *)(st.dev + bo) : nullptr, (float *)(st.dev + yo), st.stream);
    if (rc == JITNN_HIP_OK) {
        if (by_kernel) {
            copy16(st.pinned_dev + yo, st.dev + yo, yb);
            HIP_TRY(hipGetLastError());
        } else {
            HIP_TRY(hipMemcpyAsync(keep ? (void *)(st.pinned + yo) : (void *)y_host, st.dev + yo, yb, hipMemcpyDeviceToHost, st.stream));
        }
        HIP_TRY(hipStreamSynchronize(st.stream));
        if (keep) memcpy(y_host, st.pinned + yo, yb);
    }
    if (!keep) {  // a buffer this large is not held on to
        (void)hipStreamSynchronize(st.stream);
        (void)hipFree(st.dev);
        st.dev = nullptr;
        st.dcap = 0;
    }
    return rc;
}

int jitnn_hip_quantize_q8_0_dev(const float *x_dev, long long numel, void *blocks_dev, void *stream) {
    if (!x_dev || !blocks_dev) return fail(JITNN_HIP_EINVAL, "input or output is NULL");
    if (numel < 0 || numel % 32 != 0) return fail(JITNN_HIP_EINVAL, "Q8_0 needs a multiple of 32 values, got %lld", numel);
    if (int rc = check_ready()) return rc;
    if (numel == 0) return JITNN_HIP_OK;
    count_op(ST_QUANT, 4ll * numel + numel / 32 * 34);
    const size_t blocks = (size_t)numel / 32;
    size_t grid = (blocks + 4 * Q8Q_BLOCKS - 1) / (4 * Q8Q_BLOCKS);
    if (grid > (size_t)g.cus * 32) grid = (size_t)g.cus * 32;
    hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, x_dev, (uint8_t *)blocks_dev, blocks);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_quantize_q8_0(const float *x_host, long long numel, void *blocks_host) {
    if (!x_host || !blocks_host) return fail(JITNN_HIP_EINVAL, "input or output is NULL");
    if (numel < 0 || numel % 32 != 0) return fail(JITNN_HIP_EINVAL, "Q8_0 needs a multiple of 32 values, got %lld", numel);
    if (int rc = check_ready()) return rc;
    if (numel == 0) return JITNN_HIP_OK;
    // in pieces of whole blocks through the thread's device buffer
    const long long piece = (long long)16 << 20;  // values per piece: 64 MiB in, 17 MiB out
    const size_t xmax = (size_t)std::min(numel, piece) * 4, qo = (xmax + 255) & ~(size_t)255;
    if (int rc = stage_reserve(0, qo + (size_t)std::min(numel, piece) / 32 * 34)) return rc;
    HostStage &st = g_thread.stage;
    count_op(ST_QUANT, 4ll * numel + numel / 32 * 34);
    StatNest nest;
    for (long long v0 = 0; v0 < numel; v0 += piece) {
        const long long nv = std::min(piece, numel - v0);
        HIP_TRY(hipMemcpyAsync(st.dev, x_host + v0, (size_t)nv * 4, hipMemcpyHostToDevice, st.stream));
        if (int rc = jitnn_hip_quantize_q8_0_dev((const float *)st.dev, nv, st.dev + qo, st.stream)) return rc;
        HIP_TRY(hipMemcpyAsync((uint8_t *)blocks_host + v0 / 32 * 34, st.dev + qo, (size_t)nv / 32 * 34, hipMemcpyDeviceToHost, st.stream));
        HIP_TRY(hipStreamSynchronize(st.stream));
    }
    return JITNN_HIP_OK;
}

int jitnn_hip_thread_release(void) {
    if (!g.ready) return JITNN_HIP_OK;
    (void)hipDeviceSynchronize();
    g_thread.stage.release();
    release_workspace();
    return JITNN_HIP_OK;
}

int jitnn_hip_probe_read_shape_dev(const void *dev, long long nbytes, int workgroups_per_cu, int loads_in_flight, int nontemporal, void *stream) {
    if (!dev || nbytes < 16 || ((uintptr_t)dev & 15) != 0) return fail(JITNN_HIP_EINVAL, "need a 16-byte aligned buffer of at least 16 bytes");
    if (workgroups_per_cu < 1 || workgroups_per_cu > 16) return fail(JITNN_HIP_EINVAL, "%d workgroups per CU", workgroups_per_cu);
    if (int rc = check_ready()) return rc;
    typedef void (*fn_t)(const u32x4 *, size_t, uint32_t *, uint32_t);
    fn_t fn = nullptr;
    switch (loads_in_flight) {
    case 1: fn = nontemporal ? probe_read_kernel<1, true> : probe_read_kernel<1, false>; break;
    case 2: fn = nontemporal ? probe_read_kernel<2, true> : probe_read_kernel<2, false>; break;
    case 4: fn = nontemporal ? probe_read_kernel<4, true> : probe_read_kernel<4, false>; break;
    case 8: fn = nontemporal ? probe_read_kernel<8, true> : probe_read_kernel<8, false>; break;
    case 16: fn = nontemporal ? probe_read_kernel<16, true> : probe_read_kernel<16, false>; break;
    default: return fail(JITNN_HIP_EINVAL, "%d loads in flight (1, 2, 4, 8 or 16)", loads_in_flight);
    }
    hipLaunchKernelGGL(fn, dim3(g.cus * workgroups_per_cu), dim3(256), 0, (hipStream_t)stream, (const u32x4 *)dev, (size_t)nbytes / 16, (uint32_t *)nullptr,
                       (uint32_t)(g.cus * workgroups_per_cu * 256));
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_probe_read_dev(const void *dev, long long nbytes, void *stream) {
    return jitnn_hip_probe_read_shape_dev(dev, nbytes, 8, 1, 0, stream);  // the shape a sweep found fastest on 33 MB (6.4 us against 7.5 for 2 x 4)
}

int jitnn_hip_malloc(long long nbytes, void **dev) {
    if (!dev || nbytes < 0) return fail(JITNN_HIP_EINVAL, "bad arguments");
    *dev = nullptr;
    if (int rc = check_ready()) return rc;
    hipError_t e = hipMalloc(dev, (size_t)(nbytes > 0 ? nbytes : 1));
    if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipMalloc of %lld bytes: %s", nbytes, hipGetErrorString(e));
    return JITNN_HIP_OK;
}

int jitnn_hip_free(void *dev) {
    if (!dev) return JITNN_HIP_OK;
    HIP_TRY(hipFree(dev));
    return JITNN_HIP_OK;
}

int jitnn_hip_memcpy_h2d(void *dev, const void *host, long long nbytes) {
    if (!dev || !host || nbytes < 0) return fail(JITNN_HIP_EINVAL, "bad arguments");
    if (int rc = check_ready()) return rc;
    HIP_TRY(hipMemcpy(dev, host, (size_t)nbytes, hipMemcpyHostToDevice));
    return JITNN_HIP_OK;
}

int jitnn_hip_memcpy_d2h(void *host, const void *dev, long long nbytes) {
    if (!dev || !host || nbytes < 0) return fail(JITNN_HIP_EINVAL, "bad arguments");
    if (int rc = check_ready()) return rc;
    HIP_TRY(hipMemcpy(host, dev, (size_t)nbytes, hipMemcpyDeviceToHost));
    return JITNN_HIP_OK;
}

}  // extern "C"

// ================================================================================================ GGUF files

struct jitnn_hip_gguf {
    GgufFile *f;
};

extern "C" {

int jitnn_hip_gguf_open(const char *path, jitnn_hip_gguf **out) {
    if (!out) return fail(JITNN_HIP_EINVAL, "out is NULL");
    *out = nullptr;
    if (!path) return fail(JITNN_HIP_EINVAL, "path is NULL");
    std::string err;
    GgufFile *f = gguf_open(path, err);
    if (!f) return fail(JITNN_HIP_EIO, "%s", err.c_str());
    jitnn_hip_gguf *h = new (std::nothrow) jitnn_hip_gguf{f};
    if (!h) {
        delete f;
        return fail(JITNN_HIP_ENOMEM, "out of host memory");
    }
    *out = h;
    return JITNN_HIP_OK;
}

int jitnn_hip_gguf_close(jitnn_hip_gguf *h) {
    if (!h) return JITNN_HIP_OK;
    delete h->f;
    delete h;
    return JITNN_HIP_OK;
}

int jitnn_hip_gguf_header(const jitnn_hip_gguf *h, int *version, int *alignment, long long *data_offset, long long *tensor_count,
                          long long *kv_count) {
    if (!h) return fail(JITNN_HIP_EINVAL, "file is NULL");
    if (version) *version = h->f->version;
    if (alignment) *alignment = h->f->alignment;
    if (data_offset) *data_offset = h->f->data_offset;
    if (tensor_count) *tensor_count = (long long)h->f->tensors.size();
    if (kv_count) *kv_count = h->f->kv_count;
    return JITNN_HIP_OK;
}

long long jitnn_hip_gguf_metadata_json(const jitnn_hip_gguf *h, char *buf, long long cap) {
    if (!h) return fail(JITNN_HIP_EINVAL, "file is NULL");
    const std::string &j = h->f->metadata_json;
    if (buf && cap > 0) {
        const size_t n = j.size() < (size_t)cap - 1 ? j.size() : (size_t)cap - 1;
        memcpy(buf, j.data(), n);
        buf[n] = 0;
    }
    return (long long)j.size();
}

int jitnn_hip_gguf_tensor_name(const jitnn_hip_gguf *h, long long index, char *name, int cap) {
    if (!h || !name || cap < 1) return fail(JITNN_HIP_EINVAL, "bad arguments");
    if (index < 0 || index >= (long long)h->f->tensors.size()) return fail(JITNN_HIP_EINVAL, "tensor %lld of %zu", index, h->f->tensors.size());
    strncpy(name, h->f->tensors[(size_t)index].name.c_str(), (size_t)cap - 1);
    name[cap - 1] = 0;
    return JITNN_HIP_OK;
}

int jitnn_hip_gguf_tensor_info(const jitnn_hip_gguf *h, const char *name, int *type, int *ndims, long long *dims, long long *file_offset,
                               long long *nbytes) {
    if (!h || !name) return fail(JITNN_HIP_EINVAL, "file or name is NULL");
    const GgufTensor *t = h->f->find(name);
    if (!t) return fail(JITNN_HIP_EINVAL, "%s: no tensor %s", h->f->path.c_str(), name);
    if (type) *type = t->type_id;
    if (ndims) *ndims = (int)t->shape.size();
    if (dims)
        for (size_t i = 0; i < t->shape.size(); ++i) dims[i] = t->shape[i];
    if (file_offset) *file_offset = t->offset;
    if (nbytes) *nbytes = t->bytes;
    return JITNN_HIP_OK;
}

int jitnn_hip_gguf_tensor_read(const jitnn_hip_gguf *h, const char *name, void *dst_host, long long nbytes) {
    if (!h || !name || !dst_host) return fail(JITNN_HIP_EINVAL, "NULL argument");
    const GgufTensor *t = h->f->find(name);
    if (!t) return fail(JITNN_HIP_EINVAL, "%s: no tensor %s", h->f->path.c_str(), name);
    if (t->bytes < 0) return fail(JITNN_HIP_EUNSUPPORTED, "%s: ggml type %d is unknown, so its size is too", name, t->type_id);
    if (nbytes != t->bytes) return fail(JITNN_HIP_EINVAL, "%s holds %lld bytes, asked for %lld", name, t->bytes, nbytes);
    memcpy(dst_host, h->f->map + t->offset, (size_t)nbytes);
    return JITNN_HIP_OK;
}

int jitnn_hip_gguf_tensor_upload(const jitnn_hip_gguf *h, const char *name, jitnn_hip_weight **out) {
    if (!out) return fail(JITNN_HIP_EINVAL, "out is NULL");
    *out = nullptr;
    if (!h || !name) return fail(JITNN_HIP_EINVAL, "file or name is NULL");
    const GgufTensor *t = h->f->find(name);
    if (!t) return fail(JITNN_HIP_EINVAL, "%s: no tensor %s", h->f->path.c_str(), name);
    if (!known(t->type_id)) {
        const GgmlTypeInfo *ti = ggml_type(t->type_id);
        if (ti) return fail(JITNN_HIP_EUNSUPPORTED, "%s: ggml type %s has no block-quantised tensor type on this path", name, ti->name);
        return fail(JITNN_HIP_EUNSUPPORTED, "%s: ggml type id %d has no block-quantised tensor type on this path", name, t->type_id);
    }
    if (t->shape.empty() || t->numel > 0x7fffffffLL)
        return fail(JITNN_HIP_EUNSUPPORTED, "%s: %lld values; tensors hold at most 2^31-1", name, t->numel);
    const long long k = t->shape.back(), n = k > 0 ? t->numel / k : 0;
    return jitnn_hip_weight_upload(t->type_id, h->f->map + t->offset, t->bytes, (int)n, (int)k, out);
}

}  // extern "C"

// ================================================================================================ decode step

struct jitnn_hip_llama {
    int layers, d, heads, kv, hd, ffn, vocab, max_ctx;
    float eps, theta;
    const jitnn_hip_weight **w;  // [layers][7] then output
    const jitnn_hip_weight *w_out;
    float *norms;                // [layers][2][d] then output norm [d]
    float *kc, *vc;              // [layers][max_ctx][kv][hd]
    float *cosv, *sinv;          // [max_ctx][hd/2]
    float *xin, *xa, *xb, *xn, *q, *k, *v, *att, *gate, *up, *h, *part, *logits;  // (k and v: inside the buffer of q, behind it)
    int chunks_max;
    // many-token (prefill) buffers, [pf_cap, ...] each, allocated by the first prefill call and grown when a longer one comes
    int pf_cap;
    float *pf[11];  // xn, q, k, v, att, xa, xb, gate, up, h, the K slices of a linear whose join is deferred (8 x d per token)
    int rope_interleaved;  // 0: rotate-half pairs (i, i + D/2); 1: pairs (2i, 2i + 1)
    // token embedding table [vocab, d] in ggml type embd_fmt (F32 = 0, F16 = 1 or a block format), owned
    uint8_t *embd;
    int embd_fmt;
    int *tok_dev;   // [max_ctx] token ids of the generation loop (device)
    int *tok_pin;   // one token id in pinned host memory
};

namespace {

template <int D>
void launch_attention(const jitnn_hip_llama *m, int layer, int pos, hipStream_t st) {
    const int chunks = (pos + 1 + AttCfg<D>::CH - 1) / AttCfg<D>::CH;
    const size_t lo = (size_t)layer * m->max_ctx * m->kv * m->hd;
    // (q, k, v: one buffer, see jitnn_hip_llama_create)
    hipLaunchKernelGGL(attn_decode_kernel<D>, dim3(chunks, m->kv), dim3(256), 0, st, m->q, m->cosv, m->sinv, m->kc + lo, m->vc + lo, m->part,
                       (uint32_t)m->heads | ((uint32_t)m->kv << 16), (uint32_t)pos | (m->rope_interleaved ? 0x80000000u : 0u));
    constexpr int NPL = 1024 / D < 8 ? 1024 / D : 8;  // long contexts: more threads per value share the chunks
    if (chunks > 32) hipLaunchKernelGGL((attn_merge_kernel<D, NPL>), dim3(m->heads), dim3(NPL * D), 0, st, m->part, m->att, chunks);
    else hipLaunchKernelGGL((attn_merge_kernel<D, 2>), dim3(m->heads), dim3(2 * D), 0, st, m->part, m->att, chunks);
}

bool xreg_ok(const jitnn_hip_weight *w) { return w->k <= 4096 && !is_extra_format(w->fmt); }

// y_i = W_i RMSNorm(x; nw) for `count` (at most 3) weights over the same x.  Weights the register-resident kernel
// takes get the norm fused into their launch, neighbours of one format share the launch; anything else goes through
// a separate RMSNorm and the general GEMV.
int normed_linears(const jitnn_hip_llama *m, const jitnn_hip_weight *const *ws, float *const *ys, int count, const float *x, const float *nw,
                   hipStream_t st) {
    // runs of neighbours of one format and row length the register-resident kernel takes
    XregCall calls[3];
    int ncalls = 0;
    bool all = true;
    for (int i = 0; i < count;) {
        if (!xreg_ok(ws[i])) {
            all = false;
            break;
        }
        XregCall &c = calls[ncalls++];
        int j = 0;
        while (i + j < count && j < 3 && xreg_ok(ws[i + j]) && ws[i + j]->fmt == ws[i]->fmt && ws[i + j]->k == ws[i]->k) {
            c.w[j] = ws[i + j];
            c.y[j] = ys[i + j];
            ++j;
        }
        c.x = x;
        c.norm_w = nw;
        c.eps = m->eps;
        i += j;
    }
    if (all) {
        if (ncalls == 2 && calls[0].w[0]->k == calls[1].w[0]->k && calls[0].w[0]->k % 256 == 0 && xreg2_ok(calls[0].w[0]->fmt, calls[1].w[0]->fmt))
            return launch_xreg2(calls[0], calls[1], st);
        for (int c = 0; c < ncalls; ++c)
            if (int rc = launch_xreg(calls[c], st)) return rc;
        return JITNN_HIP_OK;
    }
    hipLaunchKernelGGL(rms_norm_kernel, dim3(1), dim3(256), 0, st, x, nw, m->xn, m->d, m->eps);
    for (int i = 0; i < count; ++i)
        if (int rc = launch_gemv(ws[i], m->xn, 1, nullptr, ys[i], st)) return rc;
    return JITNN_HIP_OK;
}

int check_model(const jitnn_hip_llama *m) {
    if (!m) return fail(JITNN_HIP_EINVAL, "model is NULL");
    for (int l = 0; l < m->layers; ++l)
        for (int i = 0; i < 7; ++i)
            if (!m->w[l * 7 + i]) return fail(JITNN_HIP_EINVAL, "layer %d has no weight %d", l, i);
    if (!m->w_out) return fail(JITNN_HIP_EINVAL, "no output weight");
    return JITNN_HIP_OK;
}

// bytes of every weight a step of the model reads (norm vectors included)
long long model_weight_bytes(const jitnn_hip_llama *m) {
    long long b = m->w_out->nbytes + 4ll * (2 * m->layers + 1) * m->d;
    for (int i = 0; i < m->layers * 7; ++i) b += m->w[i]->nbytes;
    return b;
}

// ys[i] = RMSNorm(x) ws[i]^T for `rows` rows.  With more rows than the GEMV kernels take (and formats the many-row
// kernels know) the norm is part of the one activation preparation the weights share; otherwise it is a kernel of its
// own into `xn` [rows, d] and the linears take their usual route.
// The join of a linear's K slices that a caller deferred and nobody could fuse: prefill_join_kernel after all.
void flush_pending(PfPending &p, int rows, hipStream_t st) {
    if (!p.part) return;
    const size_t count4 = (size_t)rows * p.n / 4;
    const unsigned blocks = (unsigned)std::min<size_t>((count4 + 255) / 256, (size_t)g.cus * 8);
    prefill_join_launch(p.part, nullptr, p.res, p.out, count4, p.n, p.splits, blocks, st);
    p = PfPending{};
}

// (pend: x - the output of the linear before - may still be in K slices; the shared preparation then adds them up)
int normed_linears_rows(const jitnn_hip_llama *m, const jitnn_hip_weight *const *ws, float *const *ys, int count, const float *x, int rows,
                        const float *nw, float *xn, hipStream_t st, PfPending *pend = nullptr, PfGroupPending *gdefer = nullptr) {
    bool group = rows > g.gemv_max_rows && prefill_prepare_fuses_norm(m->d);
    for (int i = 0; i < count; ++i) group = group && has_many_row_kernel(ws[i]->fmt);
    if (group) {
        const bool fused = pend && pend->part && pend->out == x && pend->n == m->d;
        const int rc = launch_prefill_group(ws, ys, count, x, rows, nullptr, nw, m->eps, st, nullptr, nullptr, nullptr, SCRATCH_THREAD, nullptr, nullptr,
                                            fused ? pend : nullptr, gdefer);
        if (fused) *pend = PfPending{};
        else if (pend) flush_pending(*pend, rows, st);  // (never both: a pending join is flushed before anybody reads its row)
        return rc;
    }
    if (pend) flush_pending(*pend, rows, st);
    hipLaunchKernelGGL(rms_norm_rows_kernel, dim3(rows), dim3(256), 0, st, x, nw, xn, m->d, m->eps);
    // the one-pass kernel for several rows prepares its activation operands once for all the weights that take it
    bool shared = count > 1;
    for (int i = 0; i < count; ++i) shared = shared && rows_path(ws[i], rows);
    if (shared) {
        for (int i = 0; i < count; ++i) count_op(ST_GEMV, (long long)ws[i]->nbytes + 4ll * rows * ((long long)ws[i]->k + ws[i]->n));
        return launch_rows_group(ws, ys, count, xn, rows, nullptr, nullptr, st, SCRATCH_THREAD);
    }
    for (int i = 0; i < count; ++i)
        if (int rc = jitnn_hip_linear_dev(ws[i], xn, rows, nullptr, ys[i], (void *)st)) return rc;
    return JITNN_HIP_OK;
}

// y = res + x w^T for `rows` rows (tmp [rows, n] is scratch).  up != nullptr: the activations are silu(x) * up (the FFN's
// gate and up projections); on the many-row path they are formed inside the activation preparation, otherwise by
// swiglu_kernel into `h` [rows, k].
// part / defer: see launch_prefill_group - the join of the K slices may be left to the caller.
int residual_linear_rows(const jitnn_hip_weight *w, const float *x, int rows, const float *res, float *tmp, float *y, hipStream_t st,
                         const float *up = nullptr, float *h = nullptr, float *part = nullptr, PfPending *defer = nullptr) {
    const bool many = rows > g.gemv_max_rows && has_many_row_kernel(w->fmt) && w->n % 4 == 0;
    if (many && (!up || prefill_prepare_fuses_norm(w->k))) {
        return launch_prefill_group(&w, &y, 1, x, rows, nullptr, nullptr, 0.f, st, res, tmp, up, SCRATCH_THREAD, part, defer);
    }
    if (up && rows_path(w, rows)) {  // silu(x) * up is formed by the preparation of the one-pass kernel
        count_op(ST_GEMV, (long long)w->nbytes + 4ll * rows * ((long long)w->k + w->n));
        return launch_rows_group(&w, &y, 1, x, rows, nullptr, res, st, SCRATCH_THREAD, up);
    }
    if (up) {
        const long long count = (long long)rows * w->k;
        const unsigned blocks = (unsigned)std::min<long long>((count + 1023) / 1024, (long long)g.cus * 16);
        hipLaunchKernelGGL(swiglu_kernel, dim3(blocks), dim3(256), 0, st, x, up, h, (int)count);
        x = h;
        if (many) return launch_prefill_group(&w, &y, 1, x, rows, nullptr, nullptr, 0.f, st, res, tmp);
    }
    if (rows_path(w, rows)) {  // the one-pass kernel adds the residual as it stores
        count_op(ST_GEMV, (long long)w->nbytes + 4ll * rows * ((long long)w->k + w->n));
        return launch_rows_group(&w, &y, 1, x, rows, nullptr, res, st, SCRATCH_THREAD);
    }
    if (int rc = jitnn_hip_linear_dev(w, x, rows, nullptr, tmp, (void *)st)) return rc;
    const size_t count4 = (size_t)rows * w->n / 4;
    const unsigned blocks = (unsigned)std::min<size_t>((count4 + 255) / 256, (size_t)g.cus * 8);
    hipLaunchKernelGGL(add_rows_kernel, dim3(blocks), dim3(256), 0, st, reinterpret_cast<const float4 *>(res), reinterpret_cast<const float4 *>(tmp),
                       reinterpret_cast<float4 *>(y), count4);
    return JITNN_HIP_OK;
}

// The many-token buffers of a model, for at least `tokens` rows.
int ensure_prefill(jitnn_hip_llama *m, int tokens) {
    if (tokens <= m->pf_cap) return JITNN_HIP_OK;
    HIP_TRY(hipDeviceSynchronize());  // earlier calls may still use the old buffers
    for (float *&b : m->pf) {
        if (b) (void)hipFree(b);
        b = nullptr;
    }
    m->pf_cap = 0;
    const size_t qd = (size_t)m->heads * m->hd, kd = (size_t)m->kv * m->hd;
    const size_t per[11] = {(size_t)m->d, qd, kd, kd, qd, (size_t)m->d, (size_t)m->d, (size_t)m->ffn, (size_t)m->ffn, (size_t)m->ffn, (size_t)8 * m->d};
    for (int i = 0; i < 11; ++i) {
        if (hipMalloc(&m->pf[i], per[i] * tokens * sizeof(float)) != hipSuccess) {
            (void)hipGetLastError();
            for (float *&b : m->pf) {
                if (b) (void)hipFree(b);
                b = nullptr;
            }
            return fail(JITNN_HIP_ENOMEM, "allocating the buffers of a %d-token prefill failed", tokens);
        }
    }
    m->pf_cap = tokens;
    return JITNN_HIP_OK;
}

template <int D>
int launch_attention_rows(const jitnn_hip_llama *m, int layer, int pos0, int tokens, const float *q, float *att, hipStream_t st) {
    const int group = m->heads / m->kv;
    const size_t lo = (size_t)layer * m->max_ctx * m->kv * m->hd;
    const float scale = 1.0f / sqrtf((float)D);
    // prompts beyond the GEMV range have FP16-operand linears on both sides of the attention: FP16 operands here too
    if (tokens > g.gemv_max_rows) {
        if constexpr (D == 64 || D == 128) {
            if (group <= AM_ROWS) {
                const int qt = AM_ROWS / group;
                const dim3 grid((tokens + qt - 1) / qt, m->kv);
                constexpr size_t lds = attn_prefill_mfma_lds_bytes<D>();
                if (int rc = allow_lds((const void *)attn_prefill_mfma_kernel<D>, lds)) return rc;
                hipLaunchKernelGGL(attn_prefill_mfma_kernel<D>, grid, dim3(AM_THREADS), lds, st, q, m->kc + lo, m->vc + lo, att, m->heads, m->kv, pos0, tokens,
                                   scale);
                return JITNN_HIP_OK;
            }
        }
    }
    const int qt = ATT_ROWS / group;
    const dim3 grid((tokens + qt - 1) / qt, m->kv);
    if (tokens > g.gemv_max_rows) {
        constexpr size_t lds = attn_prefill_h_lds_bytes<D>();
        if (int rc = allow_lds((const void *)attn_prefill_h_kernel<D>, lds)) return rc;
        hipLaunchKernelGGL(attn_prefill_h_kernel<D>, grid, dim3(256), lds, st, q, m->kc + lo, m->vc + lo, att, m->heads, m->kv, pos0, tokens, scale);
    } else {
        constexpr size_t lds = attn_prefill_lds_bytes<D>();
        if (int rc = allow_lds((const void *)attn_prefill_kernel<D>, lds)) return rc;
        hipLaunchKernelGGL(attn_prefill_kernel<D>, grid, dim3(256), lds, st, q, m->kc + lo, m->vc + lo, att, m->heads, m->kv, pos0, tokens, scale);
    }
    return JITNN_HIP_OK;
}

}  // namespace

extern "C" {

int jitnn_hip_llama_create(int layers, int d_model, int heads, int kv_heads, int head_dim, int ffn, int vocab, int max_ctx, float rms_eps,
                           float rope_theta, jitnn_hip_llama **out) {
    if (!out) return fail(JITNN_HIP_EINVAL, "out is NULL");
    *out = nullptr;
    if (layers < 1 || d_model < 1 || heads < 1 || kv_heads < 1 || ffn < 1 || vocab < 1 || max_ctx < 1)
        return fail(JITNN_HIP_EINVAL, "non-positive model dimension");
    if (heads % kv_heads != 0) return fail(JITNN_HIP_EINVAL, "grouped-query attention: %d query heads over %d key/value heads", heads, kv_heads);
    if (heads > 65535) return fail(JITNN_HIP_EINVAL, "%d query heads (the attention kernel's packed head counts hold 16 bits each)", heads);
    if (heads / kv_heads > ATT_GMAX) return fail(JITNN_HIP_EINVAL, "%d query heads per key/value head (at most %d are built)", heads / kv_heads, ATT_GMAX);
    if (head_dim != 64 && head_dim != 128 && head_dim != 192 && head_dim != 256)
        return fail(JITNN_HIP_EINVAL, "head_dim %d (64, 128, 192 and 256 are built)", head_dim);
    if (int rc = check_ready()) return rc;
    jitnn_hip_llama *m = new (std::nothrow) jitnn_hip_llama();
    if (!m) return fail(JITNN_HIP_ENOMEM, "out of host memory");
    *m = jitnn_hip_llama{};
    m->layers = layers; m->d = d_model; m->heads = heads; m->kv = kv_heads; m->hd = head_dim; m->ffn = ffn; m->vocab = vocab;
    m->max_ctx = max_ctx; m->eps = rms_eps; m->theta = rope_theta;
    m->w = new (std::nothrow) const jitnn_hip_weight *[(size_t)layers * 7]();
    m->chunks_max = (max_ctx + 15) / 16;  // the smallest key chunk any head size uses
    const size_t cache = (size_t)layers * max_ctx * kv_heads * head_dim;
    const int qd = heads * head_dim, kd = kv_heads * head_dim, half = head_dim / 2;
    struct { float **p; size_t n; } bufs[] = {
        {&m->norms, ((size_t)layers * 2 + 1) * d_model}, {&m->kc, cache}, {&m->vc, cache}, {&m->cosv, (size_t)max_ctx * half},
        {&m->sinv, (size_t)max_ctx * half}, {&m->xin, (size_t)d_model}, {&m->xa, (size_t)d_model}, {&m->xb, (size_t)d_model}, {&m->xn, (size_t)d_model},
        {&m->q, (size_t)qd + 2 * (size_t)kd}, {&m->att, (size_t)qd}, {&m->gate, (size_t)ffn}, {&m->up, (size_t)ffn},
        {&m->h, (size_t)ffn}, {&m->part, (size_t)heads * m->chunks_max * (head_dim + 2)}, {&m->logits, (size_t)vocab}};
    bool ok = m->w != nullptr;
    for (auto &b : bufs) {
        if (!ok) break;
        ok = hipMalloc(b.p, b.n * sizeof(float)) == hipSuccess;
    }
    if (ok) {  // the projections of a decode step: q [heads, D], k [kv_heads, D], v [kv_heads, D] in one buffer (one pointer for the attention kernel)
        m->k = m->q + qd;
        m->v = m->k + kd;
    }
    if (ok) {
        // cos/sin of t * base^(-2i/D) in double, stored FP32: Rope.tables (core/ops/Rope.java:86-102)
        float *c = new (std::nothrow) float[(size_t)max_ctx * half], *s = new (std::nothrow) float[(size_t)max_ctx * half];
        ok = c && s;
        if (ok) {
            for (int t = 0; t < max_ctx; ++t)
                for (int i = 0; i < half; ++i) {
                    const double frequency = pow((double)rope_theta, -2.0 * i / head_dim);
                    const double angle = t * frequency;
                    c[(size_t)t * half + i] = (float)cos(angle);
                    s[(size_t)t * half + i] = (float)sin(angle);
                }
            ok = hipMemcpy(m->cosv, c, (size_t)max_ctx * half * 4, hipMemcpyHostToDevice) == hipSuccess &&
                 hipMemcpy(m->sinv, s, (size_t)max_ctx * half * 4, hipMemcpyHostToDevice) == hipSuccess;
        }
        delete[] c;
        delete[] s;
    }
    if (!ok) {
        jitnn_hip_llama_free(m);
        return fail(JITNN_HIP_ENOMEM, "allocating the model buffers (%zu bytes of KV cache) failed", 2 * cache * sizeof(float));
    }
    *out = m;
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_free(jitnn_hip_llama *m) {
    if (!m) return JITNN_HIP_OK;
    float *bufs[] = {m->norms, m->kc, m->vc, m->cosv, m->sinv, m->xin, m->xa, m->xb, m->xn, m->q, m->att, m->gate, m->up, m->h, m->part, m->logits};
    for (float *b : bufs)
        if (b) (void)hipFree(b);
    for (float *b : m->pf)
        if (b) (void)hipFree(b);
    if (m->embd) (void)hipFree(m->embd);
    if (m->tok_dev) (void)hipFree(m->tok_dev);
    if (m->tok_pin) (void)hipHostFree(m->tok_pin);
    delete[] m->w;
    delete m;
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_set_weight(jitnn_hip_llama *m, int layer, int which, const jitnn_hip_weight *w) {
    if (!m || !w) return fail(JITNN_HIP_EINVAL, "model or weight is NULL");
    if (which < 0 || which > JITNN_HIP_W_OUTPUT) return fail(JITNN_HIP_EINVAL, "weight slot %d", which);
    const int qd = m->heads * m->hd, kd = m->kv * m->hd;
    const int en[] = {qd, kd, kd, m->d, m->ffn, m->ffn, m->d, m->vocab};
    const int ek[] = {m->d, m->d, m->d, qd, m->d, m->d, m->ffn, m->d};
    if (w->n != en[which] || w->k != ek[which])
        return fail(JITNN_HIP_EINVAL, "weight slot %d needs shape [%d, %d], got [%d, %d]", which, en[which], ek[which], w->n, w->k);
    if (which == JITNN_HIP_W_OUTPUT) {
        m->w_out = w;
        return JITNN_HIP_OK;
    }
    if (layer < 0 || layer >= m->layers) return fail(JITNN_HIP_EINVAL, "layer %d of %d", layer, m->layers);
    m->w[layer * 7 + which] = w;
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_set_norm(jitnn_hip_llama *m, int layer, int which, const float *w_host) {
    if (!m || !w_host) return fail(JITNN_HIP_EINVAL, "model or weights are NULL");
    size_t off;
    if (which == JITNN_HIP_NORM_OUTPUT) {
        off = (size_t)m->layers * 2 * m->d;
    } else if (which == JITNN_HIP_NORM_ATTN || which == JITNN_HIP_NORM_FFN) {
        if (layer < 0 || layer >= m->layers) return fail(JITNN_HIP_EINVAL, "layer %d of %d", layer, m->layers);
        off = ((size_t)layer * 2 + which) * m->d;
    } else {
        return fail(JITNN_HIP_EINVAL, "norm slot %d", which);
    }
    HIP_TRY(hipMemcpy(m->norms + off, w_host, (size_t)m->d * 4, hipMemcpyHostToDevice));
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_kv_write(jitnn_hip_llama *m, int layer, int pos0, int count, const float *k_host, const float *v_host) {
    if (!m || !k_host || !v_host) return fail(JITNN_HIP_EINVAL, "NULL argument");
    if (layer < 0 || layer >= m->layers || pos0 < 0 || count < 0 || pos0 + count > m->max_ctx)
        return fail(JITNN_HIP_EINVAL, "layer %d positions [%d, %d) of a cache of %d", layer, pos0, pos0 + count, m->max_ctx);
    const size_t row = (size_t)m->kv * m->hd, off = ((size_t)layer * m->max_ctx + pos0) * row;
    HIP_TRY(hipMemcpy(m->kc + off, k_host, count * row * 4, hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(m->vc + off, v_host, count * row * 4, hipMemcpyHostToDevice));
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_kv_read(const jitnn_hip_llama *m, int layer, int pos0, int count, float *k_host, float *v_host) {
    if (!m || !k_host || !v_host) return fail(JITNN_HIP_EINVAL, "NULL argument");
    if (layer < 0 || layer >= m->layers || pos0 < 0 || count < 0 || pos0 + count > m->max_ctx)
        return fail(JITNN_HIP_EINVAL, "layer %d positions [%d, %d) of a cache of %d", layer, pos0, pos0 + count, m->max_ctx);
    const size_t row = (size_t)m->kv * m->hd, off = ((size_t)layer * m->max_ctx + pos0) * row;
    HIP_TRY(hipMemcpy(k_host, m->kc + off, count * row * 4, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(v_host, m->vc + off, count * row * 4, hipMemcpyDeviceToHost));
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_decode_dev(jitnn_hip_llama *m, const float *x_dev, int pos, float *logits_dev, void *stream) {
    if (int rc = check_model(m)) return rc;
    if (!x_dev || !logits_dev) return fail(JITNN_HIP_EINVAL, "input or output is NULL");
    if (pos < 0 || pos >= m->max_ctx) return fail(JITNN_HIP_EINVAL, "position %d of a cache of %d", pos, m->max_ctx);
    hipStream_t st = (hipStream_t)stream;
    const int d = m->d;
    count_op(ST_DECODE, model_weight_bytes(m) + 4ll * m->layers * 2 * (pos + 1) * m->kv * m->hd + 4ll * (d + m->vocab));
    StatNest nest;
    // residual stream: layer input x (the caller's buffer for layer 0, xb afterwards) -> xa after attention -> xb after the FFN
    const float *x = x_dev;
    for (int l = 0; l < m->layers; ++l) {
        const jitnn_hip_weight *const *w = m->w + (size_t)l * 7;
        const float *nw = m->norms + (size_t)l * 2 * d;
        // q, k, v = W (RMSNorm x): the norm is fused into the linears; projections of one format share a launch
        {
            const jitnn_hip_weight *ws[3] = {w[JITNN_HIP_W_ATTN_Q], w[JITNN_HIP_W_ATTN_K], w[JITNN_HIP_W_ATTN_V]};
            float *ys[3] = {m->q, m->k, m->v};
            if (int rc = normed_linears(m, ws, ys, 3, x, nw, st)) return rc;
        }
        switch (m->hd) {  // RoPE, cache append and attention per key chunk, then the merge of the chunks
        case 64: launch_attention<64>(m, l, pos, st); break;
        case 128: launch_attention<128>(m, l, pos, st); break;
        case 192: launch_attention<192>(m, l, pos, st); break;
        default: launch_attention<256>(m, l, pos, st); break;
        }
        // xa = x + Wo att, xb = xa + W2 h: the residual rides in the linear's bias slot
        if (int rc = launch_gemv(w[JITNN_HIP_W_ATTN_O], m->att, 1, x, m->xa, st)) return rc;
        // h = silu(W1 n) * (W3 n), n = RMSNorm(xa): one launch when gate and up share a format
        const jitnn_hip_weight *wg = w[JITNN_HIP_W_FFN_GATE], *wu = w[JITNN_HIP_W_FFN_UP];
        if (xreg_ok(wg) && wg->fmt == wu->fmt) {
            XregCall c;
            c.w[0] = wg;
            c.w2 = wu;
            c.y[0] = m->h;
            c.x = m->xa;
            c.norm_w = nw + d;
            c.eps = m->eps;
            if (int rc = launch_xreg(c, st)) return rc;
        } else {
            const jitnn_hip_weight *ws[2] = {wg, wu};
            float *ys[2] = {m->gate, m->up};
            if (int rc = normed_linears(m, ws, ys, 2, m->xa, nw + d, st)) return rc;
            hipLaunchKernelGGL(swiglu_kernel, dim3((m->ffn + 1023) / 1024), dim3(256), 0, st, m->gate, m->up, m->h, m->ffn);
        }
        if (int rc = launch_gemv(w[JITNN_HIP_W_FFN_DOWN], m->h, 1, m->xa, m->xb, st)) return rc;
        x = m->xb;
    }
    {
        const jitnn_hip_weight *ws[1] = {m->w_out};
        float *ys[1] = {logits_dev};
        if (int rc = normed_linears(m, ws, ys, 1, x, m->norms + (size_t)m->layers * 2 * d, st)) return rc;
    }
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_prefill_dev(jitnn_hip_llama *m, const float *x_dev, int pos0, int tokens, float *logits_dev, void *stream) {
    if (int rc = check_model(m)) return rc;
    if (!x_dev) return fail(JITNN_HIP_EINVAL, "input is NULL");
    if (tokens < 1 || pos0 < 0 || pos0 > m->max_ctx - tokens)
        return fail(JITNN_HIP_EINVAL, "%d tokens from position %d in a cache of %d", tokens, pos0, m->max_ctx);
    if (m->d % 4 != 0) return fail(JITNN_HIP_EUNSUPPORTED, "d_model %d is not a multiple of 4", m->d);
    if (int rc = ensure_prefill(m, tokens)) return rc;
    hipStream_t st = (hipStream_t)stream;
    count_op(ST_PREFILL, model_weight_bytes(m) + 4ll * m->layers * 2 * (pos0 + tokens) * m->kv * m->hd + 4ll * ((long long)tokens * m->d + (logits_dev ? m->vocab : 0)));
    StatNest nest;
    const int d = m->d, T = tokens, qd = m->heads * m->hd;
    float *xn = m->pf[0], *q = m->pf[1], *k = m->pf[2], *v = m->pf[3], *att = m->pf[4], *xa = m->pf[5], *xb = m->pf[6], *gate = m->pf[7],
          *up = m->pf[8], *h = m->pf[9];
    const float *x = x_dev;
    PfPending pend;  // the K slices of the linear that wrote x, when their join is still to come
    PfGroupPending gp;  // the K slices of q, k and v between their launch and the rotation
    for (int l = 0; l < m->layers; ++l) {
        const jitnn_hip_weight *const *w = m->w + (size_t)l * 7;
        const float *nw = m->norms + (size_t)l * 2 * d;
        const size_t lo = (size_t)l * m->max_ctx * m->kv * m->hd;
        {
            const jitnn_hip_weight *ws[3] = {w[JITNN_HIP_W_ATTN_Q], w[JITNN_HIP_W_ATTN_K], w[JITNN_HIP_W_ATTN_V]};
            float *ys[3] = {q, k, v};
            if (int rc = normed_linears_rows(m, ws, ys, 3, x, T, nw, xn, st, &pend, &gp)) return rc;
        }
        if (gp.part) {  // q, k and v still lie in K slices: the rotation adds them up as it reads them
            hipLaunchKernelGGL(rope_append_rows_join_kernel, dim3(T), dim3(256), 0, st, gp.part, gp.sg.splits[0], gp.sg.splits[1], gp.sg.splits[2], T, q,
                               m->kc + lo, m->vc + lo, m->cosv, m->sinv, m->heads, m->kv, m->hd, pos0, m->rope_interleaved);
            gp.part = nullptr;
        } else {
            hipLaunchKernelGGL(rope_append_rows_kernel, dim3(T), dim3(256), 0, st, q, k, v, m->kc + lo, m->vc + lo, m->cosv, m->sinv, m->heads, m->kv,
                               m->hd, pos0, m->rope_interleaved);
        }
        int arc;
        switch (m->hd) {
        case 64: arc = launch_attention_rows<64>(m, l, pos0, T, q, att, st); break;
        case 128: arc = launch_attention_rows<128>(m, l, pos0, T, q, att, st); break;
        case 192: arc = launch_attention_rows<192>(m, l, pos0, T, q, att, st); break;
        default: arc = launch_attention_rows<256>(m, l, pos0, T, q, att, st); break;
        }
        if (arc) return arc;
        // xa = x + Wo att, xb = xa + W2 (silu(W1 n) * (W3 n)), n = RMSNorm(xa)
        if (int rc = residual_linear_rows(w[JITNN_HIP_W_ATTN_O], att, T, x, xn, xa, st, nullptr, nullptr, m->pf[10], &pend)) return rc;
        if (T > g.gemv_max_rows && prefill_dual_ok(w[JITNN_HIP_W_FFN_GATE], w[JITNN_HIP_W_FFN_UP])) {
            // gate and up as one product with the SwiGLU in its epilogue: h = silu(W1 n) * (W3 n) directly
            const bool fused = pend.part && pend.out == xa && pend.n == d;
            if (!fused) flush_pending(pend, T, st);
            const int rc = launch_prefill_dual(w[JITNN_HIP_W_FFN_GATE], w[JITNN_HIP_W_FFN_UP], h, xa, T, nw + d, m->eps, st, fused ? &pend : nullptr);
            if (fused) pend = PfPending{};
            if (rc) return rc;
            if (int rc2 = residual_linear_rows(w[JITNN_HIP_W_FFN_DOWN], h, T, xa, xn, xb, st, nullptr, nullptr, m->pf[10], &pend)) return rc2;
        } else {
            const jitnn_hip_weight *ws[2] = {w[JITNN_HIP_W_FFN_GATE], w[JITNN_HIP_W_FFN_UP]};
            float *ys[2] = {gate, up};
            if (int rc = normed_linears_rows(m, ws, ys, 2, xa, T, nw + d, xn, st, &pend)) return rc;
            if (int rc = residual_linear_rows(w[JITNN_HIP_W_FFN_DOWN], gate, T, xa, xn, xb, st, up, h, m->pf[10], &pend)) return rc;
        }
        x = xb;
    }
    (void)qd;
    flush_pending(pend, T, st);  // the last layer's output exists whole
    if (logits_dev) {  // the last token's logits
        const jitnn_hip_weight *ws[1] = {m->w_out};
        float *ys[1] = {logits_dev};
        if (int rc = normed_linears(m, ws, ys, 1, x + (size_t)(T - 1) * d, m->norms + (size_t)m->layers * 2 * d, st)) return rc;
    }
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

// ---- generation loop: embedding lookup, greedy choice, prompt + token-by-token decode --------------------------------

int jitnn_hip_llama_set_rope_interleaved(jitnn_hip_llama *m, int interleaved) {
    if (!m) return fail(JITNN_HIP_EINVAL, "model is NULL");
    m->rope_interleaved = interleaved != 0;
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_set_embedding(jitnn_hip_llama *m, int ggml_type, const void *table_host, long long nbytes) {
    if (!m || !table_host) return fail(JITNN_HIP_EINVAL, "model or table is NULL");
    long long need;
    if (ggml_type == 0 || ggml_type == 1) {
        need = (long long)m->vocab * m->d * (ggml_type == 0 ? 4 : 2);
    } else {
        need = jitnn_hip_weight_nbytes(ggml_type, m->vocab, m->d);
        if (need < 0) return (int)need;
    }
    if (nbytes != need) return fail(JITNN_HIP_EINVAL, "an embedding table [%d, %d] of ggml type %d holds %lld bytes, got %lld", m->vocab, m->d, ggml_type, need, nbytes);
    if (m->d % 4 != 0) return fail(JITNN_HIP_EUNSUPPORTED, "d_model %d is not a multiple of 4", m->d);
    if (int rc = check_ready()) return rc;
    if (m->embd) HIP_TRY(hipFree(m->embd));
    m->embd = nullptr;
    hipError_t e = hipMalloc(&m->embd, (size_t)nbytes);
    if (e != hipSuccess) return fail(JITNN_HIP_ENOMEM, "hipMalloc of %lld bytes: %s", nbytes, hipGetErrorString(e));
    HIP_TRY(hipMemcpy(m->embd, table_host, (size_t)nbytes, hipMemcpyHostToDevice));
    m->embd_fmt = ggml_type;
    if (!m->tok_dev) HIP_TRY(hipMalloc(&m->tok_dev, (size_t)m->max_ctx * sizeof(int)));
    if (!m->tok_pin) HIP_TRY(hipHostMalloc((void **)&m->tok_pin, sizeof(int), hipHostMallocDefault));
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_embed_dev(jitnn_hip_llama *m, const int *tokens_dev, int count, float *x_dev, void *stream) {
    if (!m || !tokens_dev || !x_dev) return fail(JITNN_HIP_EINVAL, "NULL argument");
    if (!m->embd) return fail(JITNN_HIP_EINVAL, "the model has no embedding table");
    if (count < 1) return fail(JITNN_HIP_EINVAL, "%d tokens", count);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)count), block(256);
    switch (m->embd_fmt) {
    case 0:
    case 1: hipLaunchKernelGGL(embed_plain_rows_kernel, grid, block, 0, st, (const void *)m->embd, m->embd_fmt, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q4_0: hipLaunchKernelGGL(dequant_rows_kernel<F_Q4_0>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q4_1: hipLaunchKernelGGL(dequant_rows_kernel<F_Q4_1>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q5_0: hipLaunchKernelGGL(dequant_rows_kernel<F_Q5_0>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q5_1: hipLaunchKernelGGL(dequant_rows_kernel<F_Q5_1>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q8_0: hipLaunchKernelGGL(dequant_rows_kernel<F_Q8_0>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q2_K: hipLaunchKernelGGL(dequant_rows_kernel<F_Q2_K>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q3_K: hipLaunchKernelGGL(dequant_rows_kernel<F_Q3_K>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q4_K: hipLaunchKernelGGL(dequant_rows_kernel<F_Q4_K>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    case F_Q5_K: hipLaunchKernelGGL(dequant_rows_kernel<F_Q5_K>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    default: hipLaunchKernelGGL(dequant_rows_kernel<F_Q6_K>, grid, block, 0, st, m->embd, tokens_dev, x_dev, m->d, m->vocab); break;
    }
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_argmax_dev(jitnn_hip_llama *m, const float *logits_dev, int *token_dev, void *stream) {
    if (!m || !logits_dev || !token_dev) return fail(JITNN_HIP_EINVAL, "NULL argument");
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits_dev, m->vocab, token_dev);
    HIP_TRY(hipGetLastError());
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_generate(jitnn_hip_llama *m, const int *prompt, int prompt_tokens, int pos0, int max_new_tokens, int eos_token, int *out_tokens,
                             void (*on_token)(int token, void *user), void *user) {
    if (int rc = check_model(m)) return rc;
    if (!prompt || (!out_tokens && max_new_tokens > 0)) return fail(JITNN_HIP_EINVAL, "prompt or output is NULL");
    if (!m->embd) return fail(JITNN_HIP_EINVAL, "the model has no embedding table");
    if (prompt_tokens < 1 || max_new_tokens < 0 || pos0 < 0) return fail(JITNN_HIP_EINVAL, "%d prompt tokens from position %d, %d new tokens", prompt_tokens, pos0, max_new_tokens);
    if ((long long)pos0 + prompt_tokens + max_new_tokens > (long long)m->max_ctx + 1)
        return fail(JITNN_HIP_EINVAL, "positions %d .. %d do not fit a cache of %d", pos0, pos0 + prompt_tokens + max_new_tokens - 2, m->max_ctx);
    for (int i = 0; i < prompt_tokens; ++i)
        if (prompt[i] < 0 || prompt[i] >= m->vocab) return fail(JITNN_HIP_EINVAL, "token %d of a vocabulary of %d", prompt[i], m->vocab);
    if (max_new_tokens == 0) return 0;
    if (int rc = stage_reserve(0, (size_t)prompt_tokens * m->d * 4)) return rc;
    HostStage &hs = g_thread.stage;
    hipStream_t st = hs.stream;
    // the prompt: embeddings of all tokens, one pass through the layers, logits of the last token
    HIP_TRY(hipMemcpyAsync(m->tok_dev, prompt, (size_t)prompt_tokens * sizeof(int), hipMemcpyHostToDevice, st));
    float *x = (float *)hs.dev;
    if (int rc = jitnn_hip_llama_embed_dev(m, m->tok_dev, prompt_tokens, x, st)) return rc;
    if (prompt_tokens == 1) {
        if (int rc = jitnn_hip_llama_decode_dev(m, x, pos0, m->logits, st)) return rc;
    } else {
        if (int rc = jitnn_hip_llama_prefill_dev(m, x, pos0, prompt_tokens, m->logits, st)) return rc;
    }
    int produced = 0;
    for (int pos = pos0 + prompt_tokens;; ++pos) {
        // greedy: the largest logit (Llm.generate runs at temperature 0, jitnn-llm/.../llm/Llm.java:74-76)
        if (int rc = jitnn_hip_llama_argmax_dev(m, m->logits, m->tok_dev, st)) return rc;
        HIP_TRY(hipMemcpyAsync(m->tok_pin, m->tok_dev, sizeof(int), hipMemcpyDeviceToHost, st));
        HIP_TRY(hipStreamSynchronize(st));
        const int tok = *m->tok_pin;
        if (tok == eos_token) break;
        out_tokens[produced++] = tok;
        if (on_token) on_token(tok, user);
        if (produced == max_new_tokens) break;
        if (int rc = jitnn_hip_llama_embed_dev(m, m->tok_dev, 1, m->xin, st)) return rc;
        if (int rc = jitnn_hip_llama_decode_dev(m, m->xin, pos, m->logits, st)) return rc;
    }
    HIP_TRY(hipStreamSynchronize(st));
    return produced;
}

int jitnn_hip_llama_prefill(jitnn_hip_llama *m, const float *x_host, int pos0, int tokens, float *logits_host) {
    if (int rc = check_model(m)) return rc;
    if (!x_host) return fail(JITNN_HIP_EINVAL, "input is NULL");
    if (tokens < 1) return fail(JITNN_HIP_EINVAL, "%d tokens", tokens);
    const size_t bytes = (size_t)tokens * m->d * 4;
    if (int rc = stage_reserve(0, bytes)) return rc;  // the embeddings go through the calling thread's device buffer
    HostStage &st = g_thread.stage;
    HIP_TRY(hipMemcpyAsync(st.dev, x_host, bytes, hipMemcpyHostToDevice, st.stream));
    if (int rc = jitnn_hip_llama_prefill_dev(m, (const float *)st.dev, pos0, tokens, logits_host ? m->logits : nullptr, st.stream)) return rc;
    if (logits_host) HIP_TRY(hipMemcpyAsync(logits_host, m->logits, (size_t)m->vocab * 4, hipMemcpyDeviceToHost, st.stream));
    hipError_t e = hipStreamSynchronize(st.stream);
    if (e != hipSuccess) return fail(JITNN_HIP_EDEVICE, "the prefill step failed: %s", hipGetErrorString(e));
    return JITNN_HIP_OK;
}

int jitnn_hip_llama_decode(jitnn_hip_llama *m, const float *x_host, int pos, float *logits_host) {
    if (int rc = check_model(m)) return rc;
    if (!x_host || !logits_host) return fail(JITNN_HIP_EINVAL, "input or output is NULL");
    HIP_TRY(hipMemcpy(m->xin, x_host, (size_t)m->d * 4, hipMemcpyHostToDevice));
    if (int rc = jitnn_hip_llama_decode_dev(m, m->xin, pos, m->logits, nullptr)) return rc;
    HIP_TRY(hipMemcpy(logits_host, m->logits, (size_t)m->vocab * 4, hipMemcpyDeviceToHost));
    return JITNN_HIP_OK;
}

}  // extern "C"
