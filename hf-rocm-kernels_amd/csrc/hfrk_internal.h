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

// Sum over the 64 lanes of a wave (xor butterfly): every lane returns the same bits.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// The two per-piece steps of the residual RMSNorm on 8 elements (16 bytes) of a row, shared by the stand-alone kernel
// (residual_rms.hip) and the GEMM's RMSNorm prologue (skinny_gemm_rows.hip) so that both produce the same bits:
//   z = round16(float(input) + float(residual)), ssq += float(z)^2 in element order;
//   fp8 = e4m3fn(clamp(float(z) * norm * float(weight) * inv_scale, +-448)).
template <int DT>
__device__ __forceinline__ uint4 rms_add_square(uint4 a, uint4 r, float& ssq) {
    const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, rw[4] = {r.x, r.y, r.z, r.w};
    uint32_t zw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint16_t lo = store16<DT>(load16<DT>((uint16_t)(aw[j] & 0xffff)) + load16<DT>((uint16_t)(rw[j] & 0xffff)));
        const uint16_t hi = store16<DT>(load16<DT>((uint16_t)(aw[j] >> 16)) + load16<DT>((uint16_t)(rw[j] >> 16)));
        const float fl = load16<DT>(lo), fh = load16<DT>(hi);
        ssq += fl * fl;
        ssq += fh * fh;
        zw[j] = (uint32_t)lo | ((uint32_t)hi << 16);
    }
    return make_uint4(zw[0], zw[1], zw[2], zw[3]);
}

template <int DT>
__device__ __forceinline__ uint2 rms_scale_to_fp8(uint4 z, uint4 w, float norm, float inv_scale) {
    const uint32_t zw[4] = {z.x, z.y, z.z, z.w}, ww[4] = {w.x, w.y, w.z, w.w};
    float y[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        y[2 * j] = load16<DT>((uint16_t)(zw[j] & 0xffff)) * norm * load16<DT>((uint16_t)(ww[j] & 0xffff)) * inv_scale;
        y[2 * j + 1] = load16<DT>((uint16_t)(zw[j] >> 16)) * norm * load16<DT>((uint16_t)(ww[j] >> 16)) * inv_scale;
    }
    uint32_t p0 = cvt_pk_fp8(y[0], y[1], 0u, false);
    p0 = cvt_pk_fp8(y[2], y[3], p0, true);
    uint32_t p1 = cvt_pk_fp8(y[4], y[5], 0u, false);
    p1 = cvt_pk_fp8(y[6], y[7], p1, true);
    return make_uint2(p0, p1);
}

// Raw buffer resource over [base, base+bytes): loads beyond `bytes` return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

}  // namespace hfrk
