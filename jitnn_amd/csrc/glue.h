// The small kernels between the quantised linears of a Llama-style decode step (batch 1): RMSNorm, rotary
// embedding + KV-cache append, grouped-query attention of one token over an FP32 cache, SwiGLU.  They are not the
// bandwidth story of the step (the weights are) and are written plainly in FP32; each follows the reference
// operator it stands for (paths below are under jitnn-core/src/main/java/ai/beestream/jitnn/).
#pragma once
#include "common.h"

namespace jitnn {

// y = x * (1 / sqrt(mean(x^2) + eps)) * w          (ops/RowNorm.java:286-306, RMS branch); one workgroup of 256.
__global__ void __launch_bounds__(256) rms_norm_kernel(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ y, int n,
                                                        float eps) {
    __shared__ float red[4];
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) s = __builtin_fmaf(x[i], x[i], s);
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    const float is = 1.f / sqrtf(s / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) y[i] = x[i] * is * w[i];
}

// Rotary embedding in the rotate-half form (pairs (i, i + D/2), interleaved = false) of the new token's query and
// key heads at position pos, then key and value appended to the cache   (ops/Rope.java:126-150, F.ropeHeads).
// cos/sin tables [positions, D/2] are computed on the host in double as Rope.tables does (ops/Rope.java:86-102).
//   q [heads, D] in place; k, v [kv_heads, D]; caches [max_ctx, kv_heads, D].
__global__ void __launch_bounds__(256) rope_append_kernel(float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                                                           float *__restrict__ kcache, float *__restrict__ vcache, const float *__restrict__ cosv,
                                                           const float *__restrict__ sinv, int heads, int kv_heads, int d, int pos) {
    const int half = d >> 1;
    const int total = (heads + kv_heads) * half;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
        const int h = i / half, p = i - h * half;
        const float c = cosv[(size_t)pos * half + p], s = sinv[(size_t)pos * half + p];
        if (h < heads) {
            float *r = q + (size_t)h * d;
            const float a = r[p], b = r[p + half];
            r[p] = a * c - b * s;
            r[p + half] = a * s + b * c;
        } else {
            const int g = h - heads;
            const float *r = k + (size_t)g * d;
            float *o = kcache + ((size_t)pos * kv_heads + g) * d;
            const float a = r[p], b = r[p + half];
            o[p] = a * c - b * s;
            o[p + half] = a * s + b * c;
        }
    }
    for (int i = blockIdx.x * 256 + threadIdx.x; i < kv_heads * d; i += gridDim.x * 256) vcache[(size_t)pos * kv_heads * d + i] = v[i];
}

// Attention of one query token over s cached positions, grouped heads   (F.scaledDotProductAttentionBTHD with
// F.repeatHeads, F.java:588-624; ops/FlashAttention.java:538-626): query head h reads key/value head h / group.
// Split over the keys: workgroup (chunk c, kv head g) handles keys [c*CH, c*CH + CH) for the `group` query heads
// of g (one wave per query head, so the cache chunk is read once per kv head) and leaves, per query head, the
// chunk's running maximum, its sum of exp and the unnormalised weighted value sum; attn_combine_kernel merges them.
constexpr int ATT_CH = 64;  // keys per workgroup

template <int D>  // head size, a multiple of 64 up to 256
__global__ void __launch_bounds__(256) attn_partial_kernel(const float *__restrict__ q, const float *__restrict__ kcache,
                                                            const float *__restrict__ vcache, float *__restrict__ part, int heads, int kv_heads,
                                                            int s, float scale) {
    constexpr int PER = D / 64;  // values of a head per lane
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int group = heads / kv_heads;
    const int g = blockIdx.y, c = blockIdx.x, chunks = gridDim.x;
    const int j0 = c * ATT_CH, j1 = min(s, j0 + ATT_CH);
    for (int hq = wave; hq < group; hq += 4) {
        const int h = g * group + hq;
        float qr[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) qr[i] = q[(size_t)h * D + lane + 64 * i];
        float m = -INFINITY, l = 0.f, acc[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) acc[i] = 0.f;
        for (int j = j0; j < j1; ++j) {
            const float *kj = kcache + ((size_t)j * kv_heads + g) * D;
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < PER; ++i) dot = __builtin_fmaf(qr[i], kj[lane + 64 * i], dot);
            dot = wave_sum(dot) * scale;
            const float mn = fmaxf(m, dot);
            const float corr = __expf(m - mn), p = __expf(dot - mn);
            const float *vj = vcache + ((size_t)j * kv_heads + g) * D;
            l = l * corr + p;
#pragma unroll
            for (int i = 0; i < PER; ++i) acc[i] = __builtin_fmaf(p, vj[lane + 64 * i], acc[i] * corr);
            m = mn;
        }
        float *o = part + ((size_t)h * chunks + c) * (D + 2);
#pragma unroll
        for (int i = 0; i < PER; ++i) o[lane + 64 * i] = acc[i];
        if (lane == 0) {
            o[D] = m;
            o[D + 1] = l;
        }
    }
}

template <int D>
__global__ void __launch_bounds__(64) attn_combine_kernel(const float *__restrict__ part, float *__restrict__ out, int chunks) {
    constexpr int PER = D / 64;
    const int h = blockIdx.x, lane = threadIdx.x;
    const float *p = part + (size_t)h * chunks * (D + 2);
    float m = -INFINITY;
    for (int c = 0; c < chunks; ++c) m = fmaxf(m, p[(size_t)c * (D + 2) + D]);
    float l = 0.f, acc[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) acc[i] = 0.f;
    for (int c = 0; c < chunks; ++c) {
        const float *pc = p + (size_t)c * (D + 2);
        const float w = __expf(pc[D] - m);
        l = __builtin_fmaf(pc[D + 1], w, l);
#pragma unroll
        for (int i = 0; i < PER; ++i) acc[i] = __builtin_fmaf(pc[lane + 64 * i], w, acc[i]);
    }
    const float il = 1.f / l;
#pragma unroll
    for (int i = 0; i < PER; ++i) out[(size_t)h * D + lane + 64 * i] = acc[i] * il;
}

// y = silu(gate) * up, silu(v) = v / (1 + exp(-v))   (F.swiglu, F.java:1159-1161; ops/RefMath.java:114)
__global__ void __launch_bounds__(256) swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, float *__restrict__ y, int n) {
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = gate[i];
        y[i] = (v / (1.f + __expf(-v))) * up[i];
    }
}

}  // namespace jitnn
