// Shared device/host helpers of libhfrk_gfx950.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "hfrk_gfx950.h"

namespace hfrk {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kNumCU = 256;  // MI355X: 8 XCDs x 32 CUs
constexpr int kNumXCD = 8;

// Remember the last failing HIP call of this thread so that the C ABI can report it.
void set_last_hip_error(hipError_t e);

#define HFRK_HIP_TRY(expr)                      \
    do {                                        \
        hipError_t _e = (expr);                 \
        if (_e != hipSuccess) {                 \
            ::hfrk::set_last_hip_error(_e);     \
            return HFRK_HIP_ERROR;              \
        }                                       \
    } while (0)

// ---- 16-bit <-> fp32, by dtype tag -------------------------------------------------------------------------
// bf16: upper half of an fp32; conversion to bf16 rounds to nearest even (NaN kept quiet).
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_float(uint16_t b) {
    return __half2float(__ushort_as_half(b));
}

__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
    return __half_as_ushort(__float2half_rn(f));
}

template <int DT>
__device__ __forceinline__ float load16(uint16_t b) {
    if constexpr (DT == HFRK_BF16) return bf16_bits_to_float(b);
    else return f16_bits_to_float(b);
}

template <int DT>
__device__ __forceinline__ uint16_t store16(float f) {
    if constexpr (DT == HFRK_BF16) return float_to_bf16_bits(f);
    else return float_to_f16_bits(f);
}

// ---- fp32 -> OCP e4m3fn, saturating to +-448, round to nearest even ------------------------------------------
// v_cvt_pk_fp8_f32 on gfx950 produces OCP e4m3fn; the clamp makes the saturation explicit.  A NaN does not survive the
// clamp: v_med3_f32 with a NaN operand returns the minimum of the other two, so NaN is stored as -448 (0xFE), which is
// also what the reference's clamp-then-convert does with it.  The CPU oracle's encoder maps NaN to 0x7F instead; the two
// meet only on inputs that are already invalid.
__device__ __forceinline__ uint32_t cvt_pk_fp8(float a, float b, uint32_t old, bool high) {
    a = __builtin_amdgcn_fmed3f(a, 448.0f, -448.0f);
    b = __builtin_amdgcn_fmed3f(b, 448.0f, -448.0f);
    return high ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
}

__device__ __forceinline__ uint8_t cvt_fp8(float a) {
    a = __builtin_amdgcn_fmed3f(a, 448.0f, -448.0f);
    return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(a, a, 0u, false) & 0xffu);
}

// silu(g) * u * inv_scale in fp32, sigmoid as 1 / (1 + 2^(-g log2 e)) (the reference's form, swiglu_vectorized.cu:27-97)
__device__ __forceinline__ float silu_mul(float g, float u, float inv_scale) {
    const float e = __builtin_amdgcn_exp2f(-g * 1.44269504089f);
    return g * __builtin_amdgcn_rcpf(1.0f + e) * u * inv_scale;
}

// Raw buffer resource over [base, base+bytes): loads beyond `bytes` return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

}  // namespace hfrk
