// The small kernels between the quantised linears of a Llama-style decode step (batch 1): RMSNorm, rotary
// embedding + KV-cache append, grouped-query attention of one token over an FP32 cache, SwiGLU.  They are not the
// bandwidth story of the step (the weights are) and are written plainly in FP32; each follows the reference
// operator it stands for (paths below are under jitnn-core/src/main/java/ai/beestream/jitnn/).
#pragma once
#include <type_traits>
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

// One token's attention: rotary embedding of the new query and key heads - pairs (i, i + D/2), the reference's default
// rotate-half form, or pairs (2i, 2i + 1) when `interleaved` (ops/Rope.java:126-150, F.ropeHeads) -, append of the rotated key and
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

// (Fourteen dwords of arguments, all preloaded into scalar registers with the wave: q, k and v of the new token are one buffer -
// q [heads, D], k [kv_heads, D], v [kv_heads, D] -, the head counts share a dword, the position carries the rotary pairing in its
// top bit, the scale is 1 / sqrt(D) and the number of chunks follows from the position.)
template <int D>
__global__ void __launch_bounds__(256) attn_decode_kernel(const float *__restrict__ qkv, const float *__restrict__ cosv, const float *__restrict__ sinv,
                                                           float *__restrict__ kcache, float *__restrict__ vcache, float *__restrict__ part,
                                                           const uint32_t head_counts, const uint32_t pos_pairing) {
    constexpr int CH = AttCfg<D>::CH, HALF = D / 2, DQ = D / 4;
    __shared__ float Ks[CH][D + 1];
    __shared__ float Vs[CH][D];
    __shared__ float Qs[ATT_GMAX][D];
    __shared__ float Sc[ATT_GMAX][CH];
    const int heads = (int)(head_counts & 0xffffu), kv_heads = (int)(head_counts >> 16), pos = (int)(pos_pairing & 0x7fffffffu);
    const bool interleaved = (pos_pairing >> 31) != 0;
    const float scale = 1.0f / sqrtf((float)D);
    const float *const q_raw = qkv, *const k_raw = qkv + (size_t)heads * D, *const v_raw = k_raw + (size_t)kv_heads * D;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int group = heads / kv_heads, g = blockIdx.y, c = blockIdx.x;
    const int s = pos + 1, j0 = c * CH, nk = min(CH, s - j0);  // this chunk holds keys j0 .. j0 + nk - 1
    const int chunks = (s + CH - 1) / CH;                      // (the grid's x extent)
    const float *cp = cosv + (size_t)pos * HALF, *sp = sinv + (size_t)pos * HALF;

    // ---- keys and values of the chunk: every load is issued before the first LDS write (one round trip to HBM) - and before
    // the query heads are fetched, whose wait would otherwise stand in front of these loads: two round trips in a row;
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
    // ---- the new token's key and value row (the last chunk only; row jp, the thread that also writes that row's slot below):
    // requested now, with everything else - fetched where the row is written, its round trip came after all the others, in
    // the workgroup the launch ends with
    const int jp = pos - j0, qp = (tid - jp * DQ) & 255;
    const bool mine = jp >= 0 && jp < CH && qp < DQ;
    const int ep = 4 * qp;
    float4 na = make_float4(0.f, 0.f, 0.f, 0.f), nb = na, nc = na, ns = na, nvv = na;
    if (mine) {
        const float *r = k_raw + (size_t)g * D;
        if (interleaved) {  // pairs (2i, 2i + 1): values e, e + 1 turn by angle e / 2, values e + 2, e + 3 by angle e / 2 + 1
            na = *reinterpret_cast<const float4 *>(r + ep);
            const float2 c2 = *reinterpret_cast<const float2 *>(cp + (ep >> 1)), s2 = *reinterpret_cast<const float2 *>(sp + (ep >> 1));
            nc = make_float4(c2.x, c2.y, 0.f, 0.f);
            ns = make_float4(s2.x, s2.y, 0.f, 0.f);
        } else {
            const int p = ep < HALF ? ep : ep - HALF;
            na = *reinterpret_cast<const float4 *>(r + p);
            nb = *reinterpret_cast<const float4 *>(r + p + HALF);
            nc = *reinterpret_cast<const float4 *>(cp + p);
            ns = *reinterpret_cast<const float4 *>(sp + p);
        }
        nvv = *reinterpret_cast<const float4 *>(v_raw + (size_t)g * D + ep);
    }
    // ---- the group's query heads, rotated
    for (int i = tid; i < group * HALF; i += 256) {
        const int h = i / HALF, p = i - h * HALF;
        const float *r = q_raw + (size_t)(g * group + h) * D;
        const int i0 = interleaved ? 2 * p : p, i1 = interleaved ? 2 * p + 1 : p + HALF;  // the pair rotated by angle p
        const float a = r[i0], b = r[i1], cs = cp[p], sn = sp[p];
        Qs[h][i0] = a * cs - b * sn;
        Qs[h][i1] = a * sn + b * cs;
    }
#pragma unroll
    for (int it = 0; it < NI; ++it) {
        const int i = tid + it * 256, j = i / DQ, e = (i - j * DQ) * 4;
        Ks[j][e] = kreg[it].x; Ks[j][e + 1] = kreg[it].y; Ks[j][e + 2] = kreg[it].z; Ks[j][e + 3] = kreg[it].w;
        *reinterpret_cast<float4 *>(&Vs[j][e]) = vreg[it];
    }
    if (mine) {  // (the slot of row jp was written - with zeros - by this same thread in the loop above)
        float4 kr;
        if (interleaved) kr = make_float4(na.x * nc.x - na.y * ns.x, na.x * ns.x + na.y * nc.x, na.z * nc.y - na.w * ns.y, na.z * ns.y + na.w * nc.y);
        else if (ep < HALF) kr = make_float4(na.x * nc.x - nb.x * ns.x, na.y * nc.y - nb.y * ns.y, na.z * nc.z - nb.z * ns.z, na.w * nc.w - nb.w * ns.w);
        else kr = make_float4(na.x * ns.x + nb.x * nc.x, na.y * ns.y + nb.y * nc.y, na.z * ns.z + nb.z * nc.z, na.w * ns.w + nb.w * nc.w);
        const size_t row = ((size_t)pos * kv_heads + g) * D;
        *reinterpret_cast<float4 *>(kcache + row + ep) = kr;
        *reinterpret_cast<float4 *>(vcache + row + ep) = nvv;
        Ks[jp][ep] = kr.x; Ks[jp][ep + 1] = kr.y; Ks[jp][ep + 2] = kr.z; Ks[jp][ep + 3] = kr.w;
        *reinterpret_cast<float4 *>(&Vs[jp][ep]) = nvv;
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

// Merge of the key chunks of attn_decode_kernel: one workgroup per query head, NP threads per value - thread p of a value
// takes the chunks p, p + NP, ..., each with a running maximum over its chunks in order, then the NP partial results meet
// in LDS and are combined in the order of p (a fixed summation order).  A thread issues the loads of 16 chunks before
// it uses the first: NP = 2 covers a context of 1024 keys in one round trip to memory; long contexts take NP = 8 (a
// context of 8192 keys: 256 chunks, two round trips instead of eight).
// A separate launch on purpose: publishing the partial results to another workgroup inside one kernel needs
// device-scope fences, which cost several times this kernel on a part with one L2 per XCD.
template <int D, int NP>
__device__ __forceinline__ void attn_merge_body(const float *__restrict__ p, float *__restrict__ out, int chunks) {
    constexpr int U = 16;
    __shared__ float sm[NP - 1][3][D];
    const int d = threadIdx.x % D, part = threadIdx.x / D;
    float m = -INFINITY, l = 0.f, acc = 0.f;
    for (int c0 = part; c0 < chunks; c0 += NP * U) {
        float mm[U], ll[U], aa[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float *pc = p + (size_t)min(c0 + NP * u, chunks - 1) * (D + 2);
            mm[u] = pc[D];
            ll[u] = pc[D + 1];
            aa[u] = pc[d];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c0 + NP * u < chunks) {
                const float mn = fmaxf(m, mm[u]);
                const float a = __expf(m - mn), b = __expf(mm[u] - mn);
                l = l * a + ll[u] * b;
                acc = acc * a + aa[u] * b;
                m = mn;
            }
        }
    }
    if (part > 0) {
        sm[part - 1][0][d] = m;
        sm[part - 1][1][d] = l;
        sm[part - 1][2][d] = acc;
    }
    __syncthreads();
    if (part == 0) {
#pragma unroll
        for (int q = 0; q < NP - 1; ++q) {
            const float m1 = sm[q][0][d], l1 = sm[q][1][d], a1 = sm[q][2][d];
            if (m1 > -INFINITY) {  // that part saw at least one chunk
                const float mn = fmaxf(m, m1);
                const float a = __expf(m - mn), b = __expf(m1 - mn);
                l = l * a + l1 * b;
                acc = acc * a + a1 * b;
                m = mn;
            }
        }
        out[d] = acc / l;
    }
}

template <int D, int NP>
__global__ void __launch_bounds__(NP * D) attn_merge_kernel(const float *__restrict__ part, float *__restrict__ out, int chunks) {
    const int h = blockIdx.x;
    attn_merge_body<D, NP>(part + (size_t)h * chunks * (D + 2), out + (size_t)h * D, chunks);
}

// ---------------------------------------------------------------------------------------------------------------
// Many tokens at once (prefill): the same operators row by row.  T tokens at positions pos0 .. pos0 + T - 1 attend
// causally to the cache (which must hold positions 0 .. pos0 - 1) and to one another.

// y[r] = RMSNorm(x[r]) for every row: one workgroup of 256 per row (ops/RowNorm.java:286-306, RMS branch).
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ y, int n,
                                                             float eps) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * n;
    float *yr = y + (size_t)blockIdx.x * n;
    float s = 0.f;
#pragma unroll 8
    for (int i = threadIdx.x; i < n; i += 256) s = __builtin_fmaf(xr[i], xr[i], s);
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    const float is = 1.f / sqrtf(s / (float)n + eps);
#pragma unroll 8
    for (int i = threadIdx.x; i < n; i += 256) yr[i] = xr[i] * is * w[i];
}

// Rotary embedding of the query heads in place (q [T, heads, D]) and of the key heads on their way into the cache,
// values copied into the cache: token t = blockIdx.x sits at position pos0 + t.  Same rotation as attn_decode_kernel.
__global__ void __launch_bounds__(256) rope_append_rows_kernel(float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                                                                float *__restrict__ kcache, float *__restrict__ vcache,
                                                                const float *__restrict__ cosv, const float *__restrict__ sinv, int heads, int kv_heads,
                                                                int D, int pos0, int interleaved) {
    const int t = blockIdx.x, pos = pos0 + t, half = D / 2;
    const float *cp = cosv + (size_t)pos * half, *sp = sinv + (size_t)pos * half;
    float *qt = q + (size_t)t * heads * D;
    for (int i = threadIdx.x; i < heads * half; i += 256) {
        const int h = i / half, p = i - h * half;
        const int i0 = h * D + (interleaved ? 2 * p : p), i1 = h * D + (interleaved ? 2 * p + 1 : p + half);
        const float a = qt[i0], b = qt[i1], cs = cp[p], sn = sp[p];
        qt[i0] = a * cs - b * sn;
        qt[i1] = a * sn + b * cs;
    }
    const float *kt = k + (size_t)t * kv_heads * D, *vt = v + (size_t)t * kv_heads * D;
    float *kc = kcache + (size_t)pos * kv_heads * D, *vc = vcache + (size_t)pos * kv_heads * D;
    for (int i = threadIdx.x; i < kv_heads * half; i += 256) {
        const int h = i / half, p = i - h * half;
        const int i0 = h * D + (interleaved ? 2 * p : p), i1 = h * D + (interleaved ? 2 * p + 1 : p + half);
        const float a = kt[i0], b = kt[i1], cs = cp[p], sn = sp[p];
        kc[i0] = a * cs - b * sn;
        kc[i1] = a * sn + b * cs;
    }
    for (int i = threadIdx.x; i < kv_heads * D; i += 256) vc[i] = vt[i];
}

// The same on projections that still lie in K slices (the many-row launch of q, k and v split K and left the join to this
// kernel): part holds splits[0] arrays [T, nq] of partial sums of q, then splits[1] arrays [T, nk] of k, then splits[2]
// arrays [T, nk] of v; an element is the sum of its slices in slice order, as the join kernel would have stored it.  The
// rotated queries go to q [T, heads, D].
__global__ void __launch_bounds__(256) rope_append_rows_join_kernel(const float *__restrict__ part, int s0, int s1, int s2, int T, float *__restrict__ q,
                                                                     float *__restrict__ kcache, float *__restrict__ vcache,
                                                                     const float *__restrict__ cosv, const float *__restrict__ sinv, int heads,
                                                                     int kv_heads, int D, int pos0, int interleaved) {
    const int t = blockIdx.x, pos = pos0 + t, half = D / 2;
    const int nq = heads * D, nk = kv_heads * D;
    const size_t zq = (size_t)T * nq, zk = (size_t)T * nk;  // floats per slice
    const float *pq = part + (size_t)t * nq, *pk = part + zq * s0 + (size_t)t * nk, *pv = part + zq * s0 + zk * s1 + (size_t)t * nk;
    const float *cp = cosv + (size_t)pos * half, *sp = sinv + (size_t)pos * half;
    // four values at a time, the loads of all Z >= splits slices issued before the first sum (slices past the last repeat
    // it and are not added; Z is the power of two at or above the launch's slices, at most the eight a many-row launch
    // makes): the sum runs in slice order
    auto joined = [&](auto zc, const float *p, size_t zs, int splits, int i) {
        constexpr int Z = decltype(zc)::value;
        float4 v[Z];
#pragma unroll
        for (int z = 0; z < Z; ++z) v[z] = *reinterpret_cast<const float4 *>(p + (size_t)min(z, splits - 1) * zs + i);
        float4 a = v[0];
#pragma unroll
        for (int z = 1; z < Z; ++z)
            if (z < splits) a = make_float4(a.x + v[z].x, a.y + v[z].y, a.z + v[z].z, a.w + v[z].w);
        return a;
    };
    // a rotation item: four angles p .. p + 3 of one head - values (p .. p + 3, p + half .. p + half + 3), or 2 p .. 2 p + 7 in pairs
    auto rotate = [&](auto zc, const float *src, size_t zs, int splits, float *dst, int nheads) {
        for (int i = threadIdx.x; i < nheads * (half / 4); i += 256) {
            const int h = i / (half / 4), p = 4 * (i - h * (half / 4));
            const float4 cs = *reinterpret_cast<const float4 *>(cp + p), sn = *reinterpret_cast<const float4 *>(sp + p);
            if (interleaved) {
                const int i0 = h * D + 2 * p;
                const float4 u = joined(zc, src, zs, splits, i0), w = joined(zc, src, zs, splits, i0 + 4);
                *reinterpret_cast<float4 *>(dst + i0) = make_float4(u.x * cs.x - u.y * sn.x, u.x * sn.x + u.y * cs.x, u.z * cs.y - u.w * sn.y, u.z * sn.y + u.w * cs.y);
                *reinterpret_cast<float4 *>(dst + i0 + 4) =
                    make_float4(w.x * cs.z - w.y * sn.z, w.x * sn.z + w.y * cs.z, w.z * cs.w - w.w * sn.w, w.z * sn.w + w.w * cs.w);
            } else {
                const int i0 = h * D + p, i1 = i0 + half;
                const float4 a = joined(zc, src, zs, splits, i0), b = joined(zc, src, zs, splits, i1);
                *reinterpret_cast<float4 *>(dst + i0) = make_float4(a.x * cs.x - b.x * sn.x, a.y * cs.y - b.y * sn.y, a.z * cs.z - b.z * sn.z, a.w * cs.w - b.w * sn.w);
                *reinterpret_cast<float4 *>(dst + i1) = make_float4(a.x * sn.x + b.x * cs.x, a.y * sn.y + b.y * cs.y, a.z * sn.z + b.z * cs.z, a.w * sn.w + b.w * cs.w);
            }
        }
    };
    auto with_slices = [&](int splits, auto &&f) {  // f(the power of two at or above splits, as a type)
        if (splits <= 1) f(std::integral_constant<int, 1>{});
        else if (splits <= 2) f(std::integral_constant<int, 2>{});
        else if (splits <= 4) f(std::integral_constant<int, 4>{});
        else f(std::integral_constant<int, 8>{});
    };
    with_slices(s0, [&](auto zc) { rotate(zc, pq, zq, s0, q + (size_t)t * nq, heads); });
    with_slices(s1, [&](auto zc) { rotate(zc, pk, zk, s1, kcache + (size_t)pos * nk, kv_heads); });
    float *vc = vcache + (size_t)pos * nk;
    with_slices(s2, [&](auto zc) {
        for (int i = 4 * threadIdx.x; i < nk; i += 1024) *reinterpret_cast<float4 *>(vc + i) = joined(zc, pv, zk, s2, i);
    });
}

// Causal attention of a block of consecutive tokens: the (token, query head) pairs of one key/value head - ATT_ROWS
// rows, i.e. ATT_ROWS / group tokens - walk the keys in chunks of CH, each chunk staged once in LDS for all of them; row
// r = tq * group + h sees key j when j <= pos0 + t0 + tq.  q is already rotated, every key comes from the cache.
// Register tiles instead of one LDS read per multiply-add: a thread owns ATT_RT rows x CH/16 keys of the scores and ATT_RT rows
// x D/16 values of the output.  The 16 threads of a DPP row hold all keys of their rows and all of these rows'
// output, so the running softmax (maximum, sum, rescaling of the output so far) stays inside the row of lanes: two DPP
// reductions per chunk, the probabilities handed from the score tile to the value tile through LDS without a
// workgroup barrier, no partial results in memory and no merge pass.
//   grid (token blocks, kv_heads), 256 threads, attn_prefill_lds_bytes<D>() of dynamic LDS; out [T, heads, D].
constexpr int ATT_ROWS = 32;  // 16 row groups of ATT_RT rows
constexpr int ATT_RT = ATT_ROWS / 16;
template <int D>
constexpr size_t attn_prefill_lds_bytes() {
    return sizeof(float) * ((size_t)ATT_ROWS * D + (size_t)AttCfg<D>::CH * (D + 4) + (size_t)AttCfg<D>::CH * D + (size_t)AttCfg<D>::CH * (ATT_ROWS + 4));
}
template <int D>
__global__ void __launch_bounds__(256) attn_prefill_kernel(const float *__restrict__ q, const float *__restrict__ kcache,
                                                            const float *__restrict__ vcache, float *__restrict__ out, int heads, int kv_heads, int pos0,
                                                            int T, float scale) {
    constexpr int CH = AttCfg<D>::CH, DQ = D / 4, KN = CH / 16, DV = D / 16, KP = D + 4, PP = ATT_ROWS + 4;
    static_assert(D % 64 == 0 && CH % 16 == 0, "tiles of 16 threads");
    extern __shared__ __align__(16) float att_smem[];
    float *Qs = att_smem;             // [ATT_ROWS][D]
    float *Ks = Qs + ATT_ROWS * D;    // [CH][D + 4]
    float *Vs = Ks + CH * KP;         // [CH][D]
    float *Pt = Vs + CH * D;          // [CH][ATT_ROWS + 4]: probabilities, key-major
    const int tid = threadIdx.x, rg = tid >> 4, kl = tid & 15;
    const int group = heads / kv_heads, QT = ATT_ROWS / group, rows = QT * group;
    const int g = blockIdx.y;
    // two workgroups share a CU and the early token blocks have few keys to walk: the upper half of the key/value heads
    // takes the blocks in reverse, so that the pair a CU is likely to hold has one long and one short walk
    const int tb = 2 * (int)blockIdx.y < kv_heads ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x;
    const int t0 = tb * QT;
    const int tl = min(t0 + QT, T) - 1;                // last token of the block
    const int nchunks = (pos0 + tl + CH) / CH;         // chunks that hold keys up to its position
    for (int i = tid; i < ATT_ROWS * DQ; i += 256) {
        const int r = i / DQ, e = (i - r * DQ) * 4, tq = r / group, h = r - tq * group;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < rows && t0 + tq < T) v = *reinterpret_cast<const float4 *>(q + ((size_t)(t0 + tq) * heads + g * group + h) * D + e);
        *reinterpret_cast<float4 *>(&Qs[r * D + e]) = v;
    }
    float mrun[ATT_RT], lrun[ATT_RT];
    float4 acc[ATT_RT][DV / 4];
#pragma unroll
    for (int i = 0; i < ATT_RT; ++i) {
        mrun[i] = -INFINITY;
        lrun[i] = 0.f;
#pragma unroll
        for (int e = 0; e < DV / 4; ++e) acc[i][e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int c = 0; c < nchunks; ++c) {
        const int j0 = c * CH, nk = min(CH, pos0 + tl + 1 - j0);
        __syncthreads();  // the chunk before has been read (first turn: the barrier below needs its twin)
        // (requesting the chunk one turn ahead into registers was tried: slower, it costs the second workgroup of the CU)
        for (int i = tid; i < CH * DQ; i += 256) {
            const int j = i / DQ, e = (i - j * DQ) * 4;
            float4 kk = make_float4(0.f, 0.f, 0.f, 0.f), vv = kk;
            if (j < nk) {
                const size_t row = ((size_t)(j0 + j) * kv_heads + g) * D;
                kk = *reinterpret_cast<const float4 *>(kcache + row + e);
                vv = *reinterpret_cast<const float4 *>(vcache + row + e);
            }
            *reinterpret_cast<float4 *>(&Ks[j * KP + e]) = kk;
            *reinterpret_cast<float4 *>(&Vs[j * D + e]) = vv;
        }
        __syncthreads();
        // ---- scores of rows ATT_RT rg .. against keys kl + 16 n
        float sc[ATT_RT][KN];
#pragma unroll
        for (int i = 0; i < ATT_RT; ++i)
#pragma unroll
            for (int n = 0; n < KN; ++n) sc[i][n] = 0.f;
#pragma unroll 4
        for (int d4 = 0; d4 < DQ; ++d4) {
            float4 qv[ATT_RT], kv[KN];
#pragma unroll
            for (int i = 0; i < ATT_RT; ++i) qv[i] = *reinterpret_cast<const float4 *>(&Qs[(ATT_RT * rg + i) * D + 4 * d4]);
#pragma unroll
            for (int n = 0; n < KN; ++n) kv[n] = *reinterpret_cast<const float4 *>(&Ks[(kl + 16 * n) * KP + 4 * d4]);
#pragma unroll
            for (int i = 0; i < ATT_RT; ++i)
#pragma unroll
                for (int n = 0; n < KN; ++n) {
                    sc[i][n] = __builtin_fmaf(qv[i].x, kv[n].x, sc[i][n]);
                    sc[i][n] = __builtin_fmaf(qv[i].y, kv[n].y, sc[i][n]);
                    sc[i][n] = __builtin_fmaf(qv[i].z, kv[n].z, sc[i][n]);
                    sc[i][n] = __builtin_fmaf(qv[i].w, kv[n].w, sc[i][n]);
                }
        }
        // ---- running softmax of each row (its keys sit in the 16 lanes of this DPP row, and so does its output)
#pragma unroll
        for (int i = 0; i < ATT_RT; ++i) {
            const int r = ATT_RT * rg + i, tq = r / group;
            const bool live = r < rows && t0 + tq < T;
            float mc = -INFINITY;
#pragma unroll
            for (int n = 0; n < KN; ++n) {
                const bool seen = live && j0 + kl + 16 * n <= pos0 + t0 + tq;
                sc[i][n] = seen ? sc[i][n] * scale : -INFINITY;
                mc = fmaxf(mc, sc[i][n]);
            }
            const float mn = fmaxf(mrun[i], row_max(mc));
            const float alpha = mrun[i] > -INFINITY ? __expf(mrun[i] - mn) : 0.f;  // (nothing seen so far: nothing to rescale)
            float ls = 0.f;
#pragma unroll
            for (int n = 0; n < KN; ++n) {
                const float p = sc[i][n] > -INFINITY ? __expf(sc[i][n] - mn) : 0.f;
                Pt[(kl + 16 * n) * PP + r] = p;
                ls += p;
            }
            lrun[i] = lrun[i] * alpha + row_sum(ls);
            mrun[i] = mn;
#pragma unroll
            for (int e = 0; e < DV / 4; ++e)
                acc[i][e] = make_float4(acc[i][e].x * alpha, acc[i][e].y * alpha, acc[i][e].z * alpha, acc[i][e].w * alpha);
        }
        // the probabilities of this row group were written by the 16 lanes that read them below: a wave-level hand-off
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ---- weighted value sums: rows ATT_RT rg .., values DV kl .. + DV - 1
#pragma unroll 4
        for (int j = 0; j < CH; ++j) {
            float pr[ATT_RT];
#pragma unroll
            for (int i = 0; i < ATT_RT; ++i) pr[i] = Pt[j * PP + ATT_RT * rg + i];
#pragma unroll
            for (int e = 0; e < DV / 4; ++e) {
                const float4 v = *reinterpret_cast<const float4 *>(&Vs[j * D + DV * kl + 4 * e]);
#pragma unroll
                for (int i = 0; i < ATT_RT; ++i) {
                    acc[i][e].x = __builtin_fmaf(pr[i], v.x, acc[i][e].x);
                    acc[i][e].y = __builtin_fmaf(pr[i], v.y, acc[i][e].y);
                    acc[i][e].z = __builtin_fmaf(pr[i], v.z, acc[i][e].z);
                    acc[i][e].w = __builtin_fmaf(pr[i], v.w, acc[i][e].w);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < ATT_RT; ++i) {
        const int r = ATT_RT * rg + i, tq = r / group, h = r - tq * group;
        if (r < rows && t0 + tq < T) {
            float *o = out + ((size_t)(t0 + tq) * heads + g * group + h) * D + DV * kl;
            const float il = 1.f / lrun[i];
#pragma unroll
            for (int e = 0; e < DV / 4; ++e)
                *reinterpret_cast<float4 *>(o + 4 * e) = make_float4(acc[i][e].x * il, acc[i][e].y * il, acc[i][e].z * il, acc[i][e].w * il);
        }
    }
}

// The same attention with FP16 operands for prompts beyond the GEMV range, where the linears around it run on FP16
// operands too: q, keys, values and probabilities go to LDS as binary16 (half the LDS traffic, twice the workgroups
// per CU), products are v_dot2_f32_f16 - two multiply-adds per instruction, FP32 accumulation - and the softmax
// statistics stay in FP32.  Values and probabilities are stored in pairs of consecutive keys so that a pair is one
// dot2 operand.  Same grid, same tiles and same causal rule as attn_prefill_kernel.
typedef _Float16 att_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 att_h4 __attribute__((ext_vector_type(4)));
typedef _Float16 att_h8 __attribute__((ext_vector_type(8)));
// (chunks of twice the keys of the FP32 kernels: the FP16 tiles leave room, and a chunk costs two barriers)
template <int D>
struct AttCfgH {
    static constexpr int CH = 2 * AttCfg<D>::CH;
};
template <int D>
constexpr size_t attn_prefill_h_lds_bytes() {
    return sizeof(_Float16) * ((size_t)ATT_ROWS * D + (size_t)AttCfgH<D>::CH * (D + 8) + (size_t)AttCfgH<D>::CH * D + (size_t)AttCfgH<D>::CH * ATT_ROWS);
}
template <int D>
__global__ void __launch_bounds__(256) attn_prefill_h_kernel(const float *__restrict__ q, const float *__restrict__ kcache,
                                                              const float *__restrict__ vcache, float *__restrict__ out, int heads, int kv_heads, int pos0,
                                                              int T, float scale) {
    constexpr int CH = AttCfgH<D>::CH, DQ = D / 4, KN = CH / 16, DV = D / 16, KP = D + 8;
    static_assert(D % 64 == 0 && CH % 16 == 0 && ATT_RT == 2, "tiles of 16 threads, two rows each");
    extern __shared__ __align__(16) float att_smem[];
    _Float16 *Qh = reinterpret_cast<_Float16 *>(att_smem);  // [ATT_ROWS][D]
    _Float16 *Kh = Qh + ATT_ROWS * D;                       // [CH][D + 8]
    _Float16 *Vh = Kh + CH * KP;                            // [CH / 2][D][2]: the values of two consecutive keys side by side
    _Float16 *Ph = Vh + CH * D;                             // [CH / 2][ATT_ROWS][2]: probabilities, likewise
    const int tid = threadIdx.x, rg = tid >> 4, kl = tid & 15;
    const int group = heads / kv_heads, QT = ATT_ROWS / group, rows = QT * group;
    const int g = blockIdx.y;
    const int tb = 2 * (int)blockIdx.y < kv_heads ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x;  // (as in attn_prefill_kernel)
    const int t0 = tb * QT;
    const int tl = min(t0 + QT, T) - 1;
    const int nchunks = (pos0 + tl + CH) / CH;
    for (int i = tid; i < ATT_ROWS * DQ; i += 256) {
        const int r = i / DQ, e = (i - r * DQ) * 4, tq = r / group, h = r - tq * group;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < rows && t0 + tq < T) v = *reinterpret_cast<const float4 *>(q + ((size_t)(t0 + tq) * heads + g * group + h) * D + e);
        *reinterpret_cast<att_h4 *>(&Qh[r * D + e]) = att_h4{(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
    }
    float mrun[ATT_RT], lrun[ATT_RT], acc[ATT_RT][DV];
#pragma unroll
    for (int i = 0; i < ATT_RT; ++i) {
        mrun[i] = -INFINITY;
        lrun[i] = 0.f;
#pragma unroll
        for (int e = 0; e < DV; ++e) acc[i][e] = 0.f;
    }
    // The keys and values of a chunk are requested one chunk ahead, into registers, so that the trip to L2 / HBM runs
    // under the arithmetic of the chunk before (with FP16 tiles the registers are there: 53 against 71 us per layer at
    // 512 tokens; the FP32 kernel loses its second workgroup per CU to them).  A thread takes pairs of keys, four
    // values of each; past the chunk's last key it re-reads that key, which the causal mask hides.
    constexpr int NIH = ((CH / 2) * DQ + 255) / 256;
    float4 rk0[NIH], rk1[NIH], rv0[NIH], rv1[NIH];
    auto fetch = [&](int c) {
        const int j0 = c * CH, nk = min(CH, pos0 + tl + 1 - j0);
#pragma unroll
        for (int it = 0; it < NIH; ++it) {
            const int i = min(tid + it * 256, (CH / 2) * DQ - 1), jp = i / DQ, e = (i - jp * DQ) * 4;
            const size_t r0 = ((size_t)(j0 + min(2 * jp, nk - 1)) * kv_heads + g) * D + e;
            const size_t r1 = ((size_t)(j0 + min(2 * jp + 1, nk - 1)) * kv_heads + g) * D + e;
            rk0[it] = *reinterpret_cast<const float4 *>(kcache + r0);
            rv0[it] = *reinterpret_cast<const float4 *>(vcache + r0);
            rk1[it] = *reinterpret_cast<const float4 *>(kcache + r1);
            rv1[it] = *reinterpret_cast<const float4 *>(vcache + r1);
        }
    };
    fetch(0);
    for (int c = 0; c < nchunks; ++c) {
        const int j0 = c * CH;
        __syncthreads();  // the chunk before has been read
#pragma unroll
        for (int it = 0; it < NIH; ++it) {
            const int i = tid + it * 256;
            if (i < (CH / 2) * DQ) {
                const int jp = i / DQ, e = (i - jp * DQ) * 4;
                const float4 k0 = rk0[it], k1 = rk1[it], v0 = rv0[it], v1 = rv1[it];
                *reinterpret_cast<att_h4 *>(&Kh[(2 * jp) * KP + e]) = att_h4{(_Float16)k0.x, (_Float16)k0.y, (_Float16)k0.z, (_Float16)k0.w};
                *reinterpret_cast<att_h4 *>(&Kh[(2 * jp + 1) * KP + e]) = att_h4{(_Float16)k1.x, (_Float16)k1.y, (_Float16)k1.z, (_Float16)k1.w};
                *reinterpret_cast<att_h8 *>(&Vh[(jp * D + e) * 2]) = att_h8{(_Float16)v0.x, (_Float16)v1.x, (_Float16)v0.y, (_Float16)v1.y,
                                                                         (_Float16)v0.z, (_Float16)v1.z, (_Float16)v0.w, (_Float16)v1.w};
            }
        }
        __syncthreads();
        if (c + 1 < nchunks) fetch(c + 1);
        // ---- scores of rows 2 rg, 2 rg + 1 against keys kl + 16 n: eight values of d per LDS read, four dot2 each
        float sc[ATT_RT][KN];
#pragma unroll
        for (int i = 0; i < ATT_RT; ++i)
#pragma unroll
            for (int n = 0; n < KN; ++n) sc[i][n] = 0.f;
#pragma unroll 4
        for (int d8 = 0; d8 < D / 8; ++d8) {
            att_h8 qv[ATT_RT], kv[KN];
#pragma unroll
            for (int i = 0; i < ATT_RT; ++i) qv[i] = *reinterpret_cast<const att_h8 *>(&Qh[(ATT_RT * rg + i) * D + 8 * d8]);
#pragma unroll
            for (int n = 0; n < KN; ++n) kv[n] = *reinterpret_cast<const att_h8 *>(&Kh[(kl + 16 * n) * KP + 8 * d8]);
#pragma unroll
            for (int i = 0; i < ATT_RT; ++i)
#pragma unroll
                for (int n = 0; n < KN; ++n)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        sc[i][n] = __builtin_amdgcn_fdot2(att_h2{qv[i][2 * t], qv[i][2 * t + 1]}, att_h2{kv[n][2 * t], kv[n][2 * t + 1]}, sc[i][n], false);
        }
        // ---- running softmax of each row, in FP32
#pragma unroll
        for (int i = 0; i < ATT_RT; ++i) {
            const int r = ATT_RT * rg + i, tq = r / group;
            const bool live = r < rows && t0 + tq < T;
            float mc = -INFINITY;
#pragma unroll
            for (int n = 0; n < KN; ++n) {
                const bool seen = live && j0 + kl + 16 * n <= pos0 + t0 + tq;
                sc[i][n] = seen ? sc[i][n] * scale : -INFINITY;
                mc = fmaxf(mc, sc[i][n]);
            }
            const float mn = fmaxf(mrun[i], row_max(mc));
            const float alpha = mrun[i] > -INFINITY ? __expf(mrun[i] - mn) : 0.f;
            float ls = 0.f;
#pragma unroll
            for (int n = 0; n < KN; ++n) {
                const float p = sc[i][n] > -INFINITY ? __expf(sc[i][n] - mn) : 0.f;
                const int j = kl + 16 * n;
                Ph[((j >> 1) * ATT_ROWS + r) * 2 + (j & 1)] = (_Float16)p;
                ls += p;
            }
            lrun[i] = lrun[i] * alpha + row_sum(ls);
            mrun[i] = mn;
#pragma unroll
            for (int e = 0; e < DV; ++e) acc[i][e] *= alpha;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ---- weighted value sums: rows 2 rg, 2 rg + 1, values DV kl .. + DV - 1, two keys per dot2
#pragma unroll 4
        for (int jp = 0; jp < CH / 2; ++jp) {
            const att_h4 pp = *reinterpret_cast<const att_h4 *>(&Ph[(jp * ATT_ROWS + ATT_RT * rg) * 2]);  // rows 2 rg and 2 rg + 1, keys 2 jp and 2 jp + 1
            const att_h2 pr[ATT_RT] = {att_h2{pp[0], pp[1]}, att_h2{pp[2], pp[3]}};
#pragma unroll
            for (int e8 = 0; e8 < DV / 4; ++e8) {
                const att_h8 v = *reinterpret_cast<const att_h8 *>(&Vh[(jp * D + DV * kl + 4 * e8) * 2]);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < ATT_RT; ++i) acc[i][4 * e8 + t] = __builtin_amdgcn_fdot2(pr[i], att_h2{v[2 * t], v[2 * t + 1]}, acc[i][4 * e8 + t], false);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < ATT_RT; ++i) {
        const int r = ATT_RT * rg + i, tq = r / group, h = r - tq * group;
        if (r < rows && t0 + tq < T) {
            float *o = out + ((size_t)(t0 + tq) * heads + g * group + h) * D + DV * kl;
            const float il = 1.f / lrun[i];
#pragma unroll
            for (int e = 0; e < DV / 4; ++e)
                *reinterpret_cast<float4 *>(o + 4 * e) = make_float4(acc[i][4 * e] * il, acc[i][4 * e + 1] * il, acc[i][4 * e + 2] * il, acc[i][4 * e + 3] * il);
        }
    }
}

// The same attention on the matrix cores (v_mfma_f32_16x16x32_f16, FP16 operands, FP32 accumulation and softmax), for
// heads of 64 or 128 values.  A workgroup of eight waves takes AM_ROWS = 64 (token, query head) rows of one key/value head
// and walks the keys in chunks of AM_CH = 64 staged once in LDS as binary16 for all of them; a wave takes 16 rows and ONE
// HALF of every chunk's keys (waves 0-3 the first 32, waves 4-7 the last 32), keeps its own running maximum, sum and
// output, and the two halves of a row meet once, at the end, through LDS.  What limits this kernel is the length of the
// dependent chain a wave walks per chunk (operand reads, MFMAs, softmax, MFMAs), not any unit's throughput: 16 rows x 64
// keys per wave took 20 us per layer at 512 tokens whether a workgroup held 64 or 128 rows.
//   * scores, transposed: S^T = K Q^T, so that a lane ends up with the scores of ONE query row (column lane % 16 of the
//     result) against the keys 4 (lane / 16) + i of every 16-key tile - the running softmax of a row needs its chunk
//     maximum from the three other lanes that hold the row's other keys (two shuffles), the row sum stays a per-lane
//     partial sum until the end;
//   * the contraction index of a matrix-core product may be numbered in any order as long as both operands use the
//     same one: the probabilities a lane holds after the softmax - keys 4 kq + i of two neighbouring 16-key tiles -
//     ARE its eight slots of the first operand of P V, when the values are laid out in LDS in that slot order
//     (transposed, [d][slot]).  No probability goes through LDS;
//   * the factor that rescales a row's output so far is handed from the lanes that know it (score layout: lane % 16 =
//     row) to the lanes that hold the output (rows 4 (lane / 16) + i) through 64 bytes of LDS per wave;
//   * keys and values of the chunk after next are requested into registers while the current one is multiplied; the LDS
//     tiles are double-buffered, one workgroup barrier per chunk; nothing about the loads is conditional (chunks past
//     the end repeat the last one, keys past the last visible one re-read it and are masked).
constexpr int AM_ROWS = 64, AM_CH = 64, AM_WAVES = 2 * (AM_ROWS / 16), AM_THREADS = 64 * AM_WAVES;
template <int D>
constexpr size_t attn_prefill_mfma_lds_bytes() {
    return (size_t)2 * ((size_t)AM_CH * (D + 8) + (size_t)D * (AM_CH + 8)) * sizeof(_Float16) + AM_WAVES * 16 * sizeof(float);  // (the
    // tiles also hold the second halves' outputs at the end: 4 waves x (16 x D + 32) floats fit for D >= 64)
}
template <int D>
__global__ void __launch_bounds__(AM_THREADS) attn_prefill_mfma_kernel(const float *__restrict__ q, const float *__restrict__ kcache,
                                                                 const float *__restrict__ vcache, float *__restrict__ out, int heads, int kv_heads,
                                                                 int pos0, int T, float scale) {
    constexpr int CH = AM_CH, KP = D + 8, VP = CH + 8, DB = D / 32, DT = D / 16, DQ = D / 4;
    constexpr int NIT = (CH / 2) * DQ / AM_THREADS;  // (key pair, four values of d) items per thread and chunk
    static_assert((CH / 2) * DQ % AM_THREADS == 0, "whole passes");
    static_assert(D == 64 || D == 128, "head sizes of this kernel");
    extern __shared__ __align__(16) float att_smem[];
    _Float16 *Kh = reinterpret_cast<_Float16 *>(att_smem);  // [2][CH][KP]
    _Float16 *Vt = Kh + 2 * CH * KP;                        // [2][D][VP]: values transposed, keys in slot order
    float *fx = reinterpret_cast<float *>(Vt + 2 * D * VP);  // [AM_WAVES][16]: a factor per row, from score layout to output layout
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, kq = lane >> 4;
    const int rt = wave & 3, half = wave >> 2;  // this wave's 16 rows of the block and its half of every chunk's keys
    const int group = heads / kv_heads, QT = AM_ROWS / group, rows = QT * group;
    const int g = blockIdx.y;
    // early token blocks walk few keys, late ones many: half of the key/value heads take the blocks in reverse
    const int tb = 2 * (int)blockIdx.y < kv_heads ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x;
    const int t0 = tb * QT;
    const int tl = min(t0 + QT, T) - 1;        // last token of the block
    const int jlast = pos0 + tl;               // last key any row of the block sees
    const int nchunks = jlast / CH + 1;
    // ---- this lane's query row (score layout): row r of the block, as the second operand of S^T = K Q^T
    const int r = 16 * rt + n, tq = r / group, hq = r - tq * group;
    const bool live = r < rows && t0 + tq < T;
    const int jmax = pos0 + t0 + tq;  // the last key the row sees
    const float scale2 = scale * 1.44269504088896341f;
    f16x8 qb[DB];
    {
        const float *qp = q + ((size_t)(t0 + (live ? tq : 0)) * heads + g * group + (live ? hq : 0)) * D + 8 * kq;
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            const float4 a = *reinterpret_cast<const float4 *>(qp + 32 * b), c = *reinterpret_cast<const float4 *>(qp + 32 * b + 4);
            qb[b] = live ? f16x8{(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w, (_Float16)c.x, (_Float16)c.y, (_Float16)c.z, (_Float16)c.w}
                         : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
    // ---- staging: an item is (key pair jp, values e .. e + 3).  Eight neighbouring lanes take the eight quads of a 128-byte
    // line of a key's row, the eight groups of eight lanes eight key pairs: a load touches whole lines, and the transposed
    // LDS stores of the values (a 4-byte word per d) spread over the banks instead of meeting in four of them.
    float4 rk0[NIT], rk1[NIT], rv0[NIT], rv1[NIT];
    auto item = [&](int it, int &jp, int &e) {
        const int wv = (tid >> 6) + it * AM_WAVES;  // wave-sized groups of items
        e = 4 * ((lane & 7) + 8 * (wv % (DQ / 8)));
        jp = (lane >> 3) + 8 * (wv / (DQ / 8));
    };
    auto fetch = [&](int c) {
        const int j0 = min(c, nchunks - 1) * CH;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            int jp, e;
            item(it, jp, e);
            const size_t r0 = ((size_t)min(j0 + 2 * jp, jlast) * kv_heads + g) * D + e;
            const size_t r1 = ((size_t)min(j0 + 2 * jp + 1, jlast) * kv_heads + g) * D + e;
            rk0[it] = *reinterpret_cast<const float4 *>(kcache + r0);
            rv0[it] = *reinterpret_cast<const float4 *>(vcache + r0);
            rk1[it] = *reinterpret_cast<const float4 *>(kcache + r1);
            rv1[it] = *reinterpret_cast<const float4 *>(vcache + r1);
        }
    };
    auto store = [&](int buf) {
        _Float16 *kh = Kh + buf * CH * KP, *vt = Vt + buf * D * VP;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            int jp, e;
            item(it, jp, e);
            const int j = 2 * jp;
            const float4 k0 = rk0[it], k1 = rk1[it], v0 = rv0[it], v1 = rv1[it];
            *reinterpret_cast<f16x4 *>(&kh[j * KP + e]) = f16x4{(_Float16)k0.x, (_Float16)k0.y, (_Float16)k0.z, (_Float16)k0.w};
            *reinterpret_cast<f16x4 *>(&kh[(j + 1) * KP + e]) = f16x4{(_Float16)k1.x, (_Float16)k1.y, (_Float16)k1.z, (_Float16)k1.w};
            // slot of key j within its 32-key step: lanes kq = (j % 16) / 4 hold keys 4 kq + i of the step's two 16-key tiles
            const int jj = j & 31, col = (j & ~31) + ((jj & 15) >> 2) * 8 + (jj & 3) + 4 * (jj >> 4);
            *reinterpret_cast<f16x2 *>(&vt[(e + 0) * VP + col]) = f16x2{(_Float16)v0.x, (_Float16)v1.x};
            *reinterpret_cast<f16x2 *>(&vt[(e + 1) * VP + col]) = f16x2{(_Float16)v0.y, (_Float16)v1.y};
            *reinterpret_cast<f16x2 *>(&vt[(e + 2) * VP + col]) = f16x2{(_Float16)v0.z, (_Float16)v1.z};
            *reinterpret_cast<f16x2 *>(&vt[(e + 3) * VP + col]) = f16x2{(_Float16)v0.w, (_Float16)v1.w};
        }
    };
    f32x4 o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrun = -INFINITY, lrun = 0.f;
    fetch(0);
    store(0);
    fetch(1);
    for (int c = 0; c < nchunks; ++c) {
        __syncthreads();  // chunk c is in its buffer; the other buffer has been read (chunk c - 1)
        store((c + 1) & 1);
        fetch(c + 2);
        const _Float16 *kh = Kh + (c & 1) * CH * KP, *vt = Vt + (c & 1) * D * VP;
        const int j0 = c * CH;
        // ---- S^T: this half's two tiles of 16 keys; the lane ends up with keys j0 + 32 half + 16 t + 4 kq + i of its row
        f32x4 st[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            st[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                const f16x8 a = *reinterpret_cast<const f16x8 *>(&kh[(32 * half + 16 * t + n) * KP + 32 * b + 8 * kq]);
                st[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qb[b], st[t], 0, 0, 0);
            }
        }
        // ---- running softmax of the row, in base 2: exp(scale s - m) = exp2(scale2 s - m2).  Only the chunks that reach
        // past the first row's last key (the diagonal of the block, and everything for rows that do not exist) need the
        // mask; in the others every score counts and no -inf can appear.
        float mc = -INFINITY;
        const bool masked = j0 + CH - 1 > pos0 + t0 || !(t0 + QT <= T && rows == AM_ROWS);  // workgroup-uniform
        if (masked) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool seen = live && j0 + 32 * half + 16 * t + 4 * kq + i <= jmax;
                    st[t][i] = seen ? st[t][i] * scale2 : -INFINITY;
                    mc = fmaxf(mc, st[t][i]);
                }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    st[t][i] *= scale2;
                    mc = fmaxf(mc, st[t][i]);
                }
        }
        mc = fmaxf(mc, __shfl_xor(mc, 16));
        mc = fmaxf(mc, __shfl_xor(mc, 32));
        const float mn = fmaxf(mrun, mc);  // (-inf while this half has not met a visible key of the row yet)
        const float alpha = mrun > -INFINITY ? __builtin_amdgcn_exp2f(mrun - mn) : 0.f;
        float ls = 0.f;
        if (masked) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float pv = st[t][i] > -INFINITY ? __builtin_amdgcn_exp2f(st[t][i] - mn) : 0.f;
                    st[t][i] = pv;
                    ls += pv;
                }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float pv = __builtin_amdgcn_exp2f(st[t][i] - mn);
                    st[t][i] = pv;
                    ls += pv;
                }
        }
        lrun = lrun * alpha + ls;
        mrun = mn;
        if (kq == 0) fx[16 * wave + n] = alpha;
        // (the LDS operations of one wave complete in order: the read below sees the write above)
        const f32x4 al = *reinterpret_cast<const f32x4 *>(&fx[16 * wave + 4 * kq]);
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            o[t][0] *= al[0];
            o[t][1] *= al[1];
            o[t][2] *= al[2];
            o[t][3] *= al[3];
        }
        // ---- O += P V over this half's 32 keys
        {
            const f16x8 pa = {(_Float16)st[0][0], (_Float16)st[0][1], (_Float16)st[0][2], (_Float16)st[0][3],
                              (_Float16)st[1][0], (_Float16)st[1][1], (_Float16)st[1][2], (_Float16)st[1][3]};
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                const f16x8 vb = *reinterpret_cast<const f16x8 *>(&vt[(16 * t + n) * VP + 32 * half + 8 * kq]);
                o[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vb, o[t], 0, 0, 0);
            }
        }
    }
    // ---- the two halves of a row meet: the waves of the second half leave maximum, sum and output in LDS (the tiles are
    // free after the last chunk), the waves of the first half combine, normalise and write.  The lane holds rows
    // 4 kq + i, values 16 t + n of the output, and - in score layout - the statistics of row n.
    lrun += __shfl_xor(lrun, 16);
    lrun += __shfl_xor(lrun, 32);
    __syncthreads();  // every wave is done with the tiles
    float *xo = att_smem + rt * (16 * D + 32);  // [DT][4][64] output, then 16 maxima, 16 sums
    if (half == 1) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) xo[(t * 4 + i) * 64 + lane] = o[t][i];
        if (kq == 0) {
            xo[16 * D + n] = mrun;
            xo[16 * D + 16 + n] = lrun;
        }
    }
    __syncthreads();
    if (half == 0) {
        const float m1 = xo[16 * D + n], l1 = xo[16 * D + 16 + n];
        const float mm = fmaxf(mrun, m1);
        const float a0 = mrun > -INFINITY ? __builtin_amdgcn_exp2f(mrun - mm) : 0.f, a1 = m1 > -INFINITY ? __builtin_amdgcn_exp2f(m1 - mm) : 0.f;
        const float il = live ? 1.f / (lrun * a0 + l1 * a1) : 0.f;
        if (kq == 0) {
            fx[16 * wave + n] = a0 * il;
            fx[16 * (wave + 4) + n] = a1 * il;
        }
        const f32x4 f0 = *reinterpret_cast<const f32x4 *>(&fx[16 * wave + 4 * kq]), f1 = *reinterpret_cast<const f32x4 *>(&fx[16 * (wave + 4) + 4 * kq]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ro = 16 * rt + 4 * kq + i, to = ro / group, ho = ro - to * group;
            if (ro < rows && t0 + to < T) {
                float *op = out + ((size_t)(t0 + to) * heads + g * group + ho) * D + n;
#pragma unroll
                for (int t = 0; t < DT; ++t) op[16 * t] = o[t][i] * f0[i] + xo[(t * 4 + i) * 64 + lane] * f1[i];
            }
        }
    }
}

// y = a + b, four values per thread (the residual connections of many rows)
__global__ void __launch_bounds__(256) add_rows_kernel(const float4 *__restrict__ a, const float4 *__restrict__ b, float4 *__restrict__ y, size_t count4) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count4; i += (size_t)gridDim.x * 256) {
        const float4 u = a[i], w = b[i];
        y[i] = make_float4(u.x + w.x, u.y + w.y, u.z + w.z, u.w + w.w);
    }
}

// y = silu(gate) * up, silu(v) = v / (1 + exp(-v))   (F.swiglu, F.java:1159-1161; ops/RefMath.java:114)
__global__ void __launch_bounds__(256) swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up, float *__restrict__ y, int n) {
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = gate[i];
        y[i] = (v / (1.f + __expf(-v))) * up[i];
    }
}

// Greedy choice of the next token: index of the largest logit, the lowest index among equals (NaN never wins).  One
// workgroup of 1024 threads: a strided scan per thread, then wave and workgroup reductions on (value, index) pairs.
__global__ void __launch_bounds__(1024) argmax_kernel(const float *__restrict__ x, int n, int *__restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 1024) {
        const float v = x[i];
        if (v > best || (v == best && i < idx)) {
            best = v;
            idx = i;
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(idx, off);
        if (ov > best || (ov == best && oi < idx)) {
            best = ov;
            idx = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
                best = bv[w];
                idx = bi[w];
            }
        *out = idx == 0x7fffffff ? 0 : idx;
    }
}

// x[t, :] = row token[t] of an unquantised embedding table [vocab, d] (F32: fmt 0, F16: fmt 1); block-quantised tables go
// through dequant_rows_kernel.  grid = tokens.  An id outside [0, vocab) reads nothing: its row is NaN.
__global__ void __launch_bounds__(256) embed_plain_rows_kernel(const void *__restrict__ table, int fmt, const int *__restrict__ tokens, float *__restrict__ x,
                                                                int d, int vocab) {
    const int t = blockIdx.x;
    const int id = tokens[t];
    if (id < 0 || id >= vocab) {
        for (int i = threadIdx.x; i < d; i += 256) x[(size_t)t * d + i] = __builtin_nanf("");
        return;
    }
    const size_t row = (size_t)id * d;
    for (int i = threadIdx.x; i < d; i += 256)
        x[(size_t)t * d + i] = fmt == 0 ? reinterpret_cast<const float *>(table)[row + i]
                                        : __half2float(reinterpret_cast<const __half *>(table)[row + i]);
}

}  // namespace jitnn
