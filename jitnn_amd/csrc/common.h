// Shared device helpers for the gfx950 kernels: block-format metadata, unaligned 128-bit loads,
// wave64 reductions.  Wavefronts are 64 lanes wide throughout; nothing here is written for 32.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace jitnn {

// ggml type ids as stored in GGUF files (reference: gguf/GgmlType.java:27-65)
// The first six are the formats of the quantised-linear path proper (tuned kernels); Q5_0, Q5_1, Q2_K and Q3_K are the
// other block formats the reference dequantises (core/kernels/GgufKernels.java:147-198): bit-exact dequantiser and a
// plain GEMV, so that every block tensor of a GGUF file is usable.
enum : int { F_Q4_0 = 2, F_Q4_1 = 3, F_Q8_0 = 8, F_Q4_K = 12, F_Q5_K = 13, F_Q6_K = 14, F_Q5_0 = 6, F_Q5_1 = 7, F_Q2_K = 10, F_Q3_K = 11 };

__host__ __device__ constexpr bool is_extra_format(int fmt) { return fmt == F_Q5_0 || fmt == F_Q5_1 || fmt == F_Q2_K || fmt == F_Q3_K; }
// (of these, Q5_1 and Q2_K have a decoder in the many-row kernel; Q5_0 and Q3_K reach it rewritten as Q8_0 and Q6_K)
__host__ __device__ constexpr bool has_many_row_kernel(int fmt) { return !is_extra_format(fmt) || fmt == F_Q5_1 || fmt == F_Q2_K; }

__host__ __device__ constexpr int block_values(int fmt) {
    return (fmt == F_Q4_0 || fmt == F_Q4_1 || fmt == F_Q8_0 || fmt == F_Q5_0 || fmt == F_Q5_1) ? 32
           : (fmt == F_Q4_K || fmt == F_Q5_K || fmt == F_Q6_K || fmt == F_Q2_K || fmt == F_Q3_K) ? 256 : 0;
}

__host__ __device__ constexpr int block_bytes(int fmt) {
    return fmt == F_Q4_0 ? 18 : fmt == F_Q4_1 ? 20 : fmt == F_Q8_0 ? 34 : fmt == F_Q4_K ? 144 : fmt == F_Q5_K ? 176 : fmt == F_Q6_K ? 210
           : fmt == F_Q5_0 ? 22 : fmt == F_Q5_1 ? 24 : fmt == F_Q2_K ? 84 : fmt == F_Q3_K ? 110 : 0;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// 128/64/32/16-bit global loads from addresses that are only A-byte aligned.  Q8_0, Q4_0 and Q6_K blocks
// are 34, 18 and 210 bytes long, so their fields sit on 2-byte boundaries; gfx950 global memory
// instructions accept that (the amdhsa target enables unaligned access mode), the C++ type system needs
// to be told.
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
typedef uint32_t u32_a2 __attribute__((aligned(2)));
template <int A>
__device__ __forceinline__ u32x4 ld128(const uint8_t *p) {
    if constexpr (A >= 16) return *reinterpret_cast<const u32x4 *>(p);
    else if constexpr (A >= 4) return *reinterpret_cast<const u32x4_a4 *>(p);
    else return *reinterpret_cast<const u32x4_a2 *>(p);
}
template <int A>
__device__ __forceinline__ u32x2 ld64(const uint8_t *p) {
    static_assert(A >= 2, "fields of GGUF blocks are at least 2-byte aligned");
    return *reinterpret_cast<const u32x2_a2 *>(p);
}
template <int A>
__device__ __forceinline__ uint32_t ld32(const uint8_t *p) {
    if constexpr (A >= 4) return *reinterpret_cast<const uint32_t *>(p);
    else return *reinterpret_cast<const u32_a2 *>(p);
}
__device__ __forceinline__ uint32_t ld16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// binary16 bits -> float (exact)
__device__ __forceinline__ float h2f(uint32_t bits) { return __half2float(__ushort_as_half((unsigned short)(bits & 0xffffu))); }

// Unsigned byte i of v as float: one v_cvt_f32_ubyte<i>.
__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

// Sum over aligned groups of G = 4 or 8 neighbouring lanes (every lane of a group receives the group's total):
// quad swaps, then for G = 8 the mirror within each half row - DPP moves inside the VALU, no LDS traffic.
template <int G>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(G == 4 || G == 8, "groups of 4 or 8 lanes");
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    if constexpr (G == 8) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    return v;
}

// Maximum / sum over each aligned row of 16 lanes (a DPP row); every lane of the row receives it.
__device__ __forceinline__ float row_max(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0xB1, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x4E, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x141, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x140, 0xF, 0xF, false)));
    return v;
}
__device__ __forceinline__ float row_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));
    return v;
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.  Four DPP steps fold each row of
// 16 lanes (quad swaps, then the two mirrors), then the four row totals are read through scalar lanes.
__device__ __forceinline__ float wave_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// Maximum over the 64 lanes of a wavefront; every lane receives it (same DPP tree as wave_sum).
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0xB1, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x4E, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x141, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x140, 0xF, 0xF, false)));
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

}  // namespace jitnn
