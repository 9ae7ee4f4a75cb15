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
    // (the decode step fuses this into its linears; this kernel serves rows longer than those kernels take)
    __shared__ float red[4];
    float s = 0.f;
#pragma unroll 8
    for (int i = threadIdx.x; i < n; i += 256) s = __builtin_fmaf(x[i], x[i], s);
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    const float is = 1.f / sqrtf(s / (float)n + eps);
#pragma unroll 8
    for (int i = threadIdx.x; i < n; i += 256) y[i] = x[i] * is * w[i];
}

// One token's attention: rotary embedding of the new query and key heads in the rotate-half
// form (pairs (i, i + D/2), interleaved = false; ops/Rope.java:126-150, F.ropeHeads), append of the rotated key and
// the value to the cache, grouped-query attention over the s = pos + 1 cached positions
// (F.scaledDotProductAttentionBTHD with F.repeatHeads, F.java:588-624; ops/FlashAttention.java:538-626: query head
// h reads key/value head h / group).
//   grid (chunks, kv_heads): a workgroup stages CH keys and values of one kv head in LDS (the cache chunk is read
//   once for the whole group of query heads), computes the group's scores from LDS, each chunk's softmax statistics
//   and unnormalised weighted value sum, and leaves them in `part` for attn_merge_kernel.
//   cos/sin tables [positions, D/2] come from the host in double (ops/Rope.java:86-102).
//   q_raw [heads, D], k_raw / v_raw [kv_heads, D] un-rotated; caches [max_ctx, kv_heads, D]; part [heads, chunks, D + 2].
constexpr int ATT_GMAX = 16;  // query heads per key/value head

template <int D>
struct AttCfg {
    static constexpr int CH = D <= 128 ? 32 : 16;  // keys per workgroup
};

template <int D>
__global__ void __launch_bounds__(256) attn_decode_kernel(const float *__restrict__ q_raw, const float *__restrict__ k_raw,
                                                           const float *__restrict__ v_raw, float *__restrict__ kcache,
                                                           float *__restrict__ vcache, const float *__restrict__ cosv,
                                                           const float *__restrict__ sinv, float *__restrict__ part, int heads, int kv_heads,
                                                           int pos, float scale) {
    constexpr int CH = AttCfg<D>::CH, HALF = D / 2, DQ = D / 4;
    __shared__ float Ks[CH][D + 1];
    __shared__ float Vs[CH][D];
    __shared__ float Qs[ATT_GMAX][D];
    __shared__ float Sc[ATT_GMAX][CH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int group = heads / kv_heads, g = blockIdx.y, c = blockIdx.x, chunks = gridDim.x;
    const int s = pos + 1, j0 = c * CH, nk = min(CH, s - j0);  // this chunk holds keys j0 .. j0 + nk - 1
    const float *cp = cosv + (size_t)pos * HALF, *sp = sinv + (size_t)pos * HALF;

    // ---- the group's query heads, rotated
    for (int i = tid; i < group * HALF; i += 256) {
        const int h = i / HALF, p = i - h * HALF;
        const float *r = q_raw + (size_t)(g * group + h) * D;
        const float a = r[p], b = r[p + HALF], cs = cp[p], sn = sp[p];
        Qs[h][p] = a * cs - b * sn;
        Qs[h][p + HALF] = a * sn + b * cs;
    }
    // ---- keys and values of the chunk: every load is issued before the first LDS write (one round trip to HBM);
    // the new token's row comes from k_raw / v_raw, rotated, and is appended to the cache on the way
    constexpr int NI = CH * DQ / 256;
    static_assert(CH * DQ % 256 == 0, "whole passes");
    float4 kreg[NI], vreg[NI];
#pragma unroll
    for (int it = 0; it < NI; ++it) {
        const int i = tid + it * 256, j = i / DQ, e = (i - j * DQ) * 4;
        kreg[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        vreg[it] = kreg[it];
        if (j < nk && j0 + j != pos) {
            const size_t row = ((size_t)(j0 + j) * kv_heads + g) * D;
            kreg[it] = *reinterpret_cast<const float4 *>(kcache + row + e);
            vreg[it] = *reinterpret_cast<const float4 *>(vcache + row + e);
        }
    }
#pragma unroll
    for (int it = 0; it < NI; ++it) {
        const int i = tid + it * 256, j = i / DQ, e = (i - j * DQ) * 4;
        if (j < nk && j0 + j == pos) {
            const size_t row = ((size_t)pos * kv_heads + g) * D;
            const float *r = k_raw + (size_t)g * D;
            const int p = e < HALF ? e : e - HALF;
            const float4 a = *reinterpret_cast<const float4 *>(r + p), b = *reinterpret_cast<const float4 *>(r + p + HALF);
            const float4 cs = *reinterpret_cast<const float4 *>(cp + p), sn = *reinterpret_cast<const float4 *>(sp + p);
            if (e < HALF) kreg[it] = make_float4(a.x * cs.x - b.x * sn.x, a.y * cs.y - b.y * sn.y, a.z * cs.z - b.z * sn.z, a.w * cs.w - b.w * sn.w);
            else kreg[it] = make_float4(a.x * sn.x + b.x * cs.x, a.y * sn.y + b.y * cs.y, a.z * sn.z + b.z * cs.z, a.w * sn.w + b.w * cs.w);
            vreg[it] = *reinterpret_cast<const float4 *>(v_raw + (size_t)g * D + e);
            *reinterpret_cast<float4 *>(kcache + row + e) = kreg[it];
            *reinterpret_cast<float4 *>(vcache + row + e) = vreg[it];
        }
        Ks[j][e] = kreg[it].x; Ks[j][e + 1] = kreg[it].y; Ks[j][e + 2] = kreg[it].z; Ks[j][e + 3] = kreg[it].w;
        *reinterpret_cast<float4 *>(&Vs[j][e]) = vreg[it];
    }
    __syncthreads();
    // ---- scores: one (query head, key) pair per thread
    for (int i = tid; i < group * CH; i += 256) {
        const int h = i / CH, j = i - h * CH;
        float dot = 0.f;
#pragma unroll 8
        for (int d = 0; d < D; ++d) dot = __builtin_fmaf(Qs[h][d], Ks[j][d], dot);
        Sc[h][j] = j < nk ? dot * scale : -INFINITY;
    }
    __syncthreads();
    // ---- softmax statistics of the chunk, one wave per query head
    for (int h = wave; h < group; h += 4) {
        const float sc = lane < CH ? Sc[h][lane] : -INFINITY;
        const float m = wave_max(sc);
        const float p = lane < CH && sc > -INFINITY ? __expf(sc - m) : 0.f;
        const float l = wave_sum(p);
        if (lane < CH) Sc[h][lane] = p;
        if (lane == 0) {
            float *o = part + ((size_t)(g * group + h) * chunks + c) * (D + 2);
            o[D] = m;
            o[D + 1] = l;
        }
    }
    __syncthreads();
    // ---- unnormalised weighted value sums
    for (int i = tid; i < group * D; i += 256) {
        const int h = i / D, d = i - h * D;
        float acc = 0.f;
#pragma unroll 8
        for (int j = 0; j < CH; ++j) acc = __builtin_fmaf(Sc[h][j], Vs[j][d], acc);
        part[((size_t)(g * group + h) * chunks + c) * (D + 2) + d] = acc;
    }
}

// Merge of the key chunks of attn_decode_kernel: one workgroup per query head, two threads per value - one takes the
// even chunks, one the odd ones, each with a running maximum over its chunks in order, then the two meet in LDS (a
// fixed summation order).  A thread issues the loads of 16 chunks before it uses the first, so a context of up to
// 1024 keys costs one round trip to memory.
// A separate launch on purpose: publishing the partial results to another workgroup inside one kernel needs
// device-scope fences, which cost several times this kernel on a part with one L2 per XCD.
template <int D>
__global__ void __launch_bounds__(2 * D) attn_merge_kernel(const float *__restrict__ part, float *__restrict__ out, int chunks) {
    constexpr int U = 16;
    __shared__ float sm[3][D];
    const int h = blockIdx.x, d = threadIdx.x % D, half = threadIdx.x / D;
    const float *p = part + (size_t)h * chunks * (D + 2);
    float m = -INFINITY, l = 0.f, acc = 0.f;
    for (int c0 = half; c0 < chunks; c0 += 2 * U) {
        float mm[U], ll[U], aa[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float *pc = p + (size_t)min(c0 + 2 * u, chunks - 1) * (D + 2);
            mm[u] = pc[D];
            ll[u] = pc[D + 1];
            aa[u] = pc[d];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c0 + 2 * u < chunks) {
                const float mn = fmaxf(m, mm[u]);
                const float a = __expf(m - mn), b = __expf(mm[u] - mn);
                l = l * a + ll[u] * b;
                acc = acc * a + aa[u] * b;
                m = mn;
            }
        }
    }
    if (half == 1) {
        sm[0][d] = m;
        sm[1][d] = l;
        sm[2][d] = acc;
    }
    __syncthreads();
    if (half == 0) {
        const float m1 = sm[0][d], l1 = sm[1][d], a1 = sm[2][d];
        if (m1 > -INFINITY) {  // the odd half saw at least one chunk
            const float mn = fmaxf(m, m1);
            const float a = __expf(m - mn), b = __expf(m1 - mn);
            l = l * a + l1 * b;
            acc = acc * a + a1 * b;
        }
        out[(size_t)h * D + d] = acc / l;
    }
}

// y = silu(gate) * up, silu(v) = v / (1 + exp(-v))   (F.swiglu, F.java:1159-1161; ops/RefMath.java:114)
__global__ void __launch_bounds__(256) swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, float *__restrict__ y, int n) {
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = gate[i];
        y[i] = (v / (1.f + __expf(-v))) * up[i];
    }
}

}  // namespace jitnn
