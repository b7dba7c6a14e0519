// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/et_amd.h"

namespace et {

// ---- error plumbing -------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define ET_HIP(call)                                                           \
    do {                                                                       \
        hipError_t e__ = (call);                                               \
        if (e__ != hipSuccess)                                                 \
            return ::et::hip_fail(e__, #call);                                 \
    } while (0)

#define ET_REQUIRE(cond, code, ...)                                            \
    do {                                                                       \
        if (!(cond)) {                                                         \
            ::et::set_error(__VA_ARGS__);                                      \
            return (code);                                                     \
        }                                                                      \
    } while (0)

static inline bool aligned16(const void *p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

static inline int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return hip_fail(e, what);
    return ET_OK;
}

// ---- vector types -----------------------------------------------------------
typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

// D(16x16,f32) += A(16x32,f16) * B(32x16,f16).
// Register layout (wave64), g = lane/16, c = lane%16:
//   a[j] = A[c][8g+j], b[j] = B[8g+j][c], d[r] = D[4g+r][c].
// Only the pairing of a[j] with b[j] inside the same lane group matters for
// the contraction, so any consistent assignment of k to (g,j) works.
__device__ __forceinline__ f32x4 mfma16x16x32(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 16 bytes per lane straight from global memory into LDS
// (global_load_lds_dwordx4): lane L of the wave writes at lds_base + 16*L;
// lds_base must be wave-uniform, the source address is free per lane.
// Completion is tracked by vmcnt.
__device__ __forceinline__ void load_lds16(const void *gsrc, void *lds_base) {
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void *)gsrc,
        (__attribute__((address_space(3))) void *)lds_base, 16, 0, 0);
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

// ---- wave64 reductions (all lanes receive the result) -----------------------
// Data-parallel-primitive moves inside a row of 16 lanes (no LDS round trip as
// with __shfl): quad_perm [1,0,3,2] and [2,3,0,1], row_half_mirror, row_mirror.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);  // pairs
    v += dpp_move<0x4E>(v);  // quads
    v += dpp_move<0x141>(v); // 8 lanes
    v += dpp_move<0x140>(v); // the row of 16: every lane holds its row's sum
    // the four rows through scalar registers
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

// GELU of four halves: x^3 in (packed) half, the sigmoid form of
// 0.5(1+tanh u) = 1/(1+exp(-2u)) in fp32, rounded to half, times x in half
// (kernels/linear.cu:36-48).
__device__ __forceinline__ f16x4 gelu4(f16x4 v) {
    const f16x4 x2 = v * v;
    const f16x4 x3 = v * x2;
    f32x4 t;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float s = __builtin_fmaf(0.044715f, (float)x3[r], (float)v[r]);
        const float e = __builtin_amdgcn_exp2f(s * (-1.5957691216057308f * 1.4426950408889634f));
        t[r] = __builtin_amdgcn_rcpf(1.0f + e);
    }
    return v * __builtin_convertvector(t, f16x4);
}

__device__ __forceinline__ float f16_bits_to_float(uint16_t b) {
    return (float)__builtin_bit_cast(f16, b);
}

} // namespace et
