// Per-token (per-row) dynamic FP8 quantisation fused into the two element-wise kernels of the decoder block, and on
// its own for activations that come from elsewhere (attention output -> o_proj):
//   residual_rms_dynamic:  residual <- input + residual;  y = rmsnorm(residual) * weight
//   swiglu_dynamic:        y = silu(gate) * up
//   quantize_fp8:          y = x   (also with one static scale: the reference's fp8_quantize, utils/fp8.py:6-29, on device)
// and in both:            scale[row] = max(amax_row |y| / 448, FLT_MIN);  output = e4m3fn(y / scale[row])
// The per-row scales feed the GEMM's per-token scale_a directly, so no activation scale has to be calibrated ahead
// of time.  The reference only has the static-scale forms (one scale_tensor for the whole tensor:
// operators/residual_rms/wrapped.py:94-95, operators/swiglu/wrapped.py:49-84); these kernels have no counterpart
// there and keep its arithmetic otherwise (16-bit residual add, fp32 normalisation and activation, one rounding).
//
// One workgroup per row; the row's y values stay in registers between the amax reduction and the quantisation, so
// the input is read once.  Needs 16-byte aligned rows (cols % 8 == 0) and cols <= 32768.
#include <cfloat>

#include "hfrk_internal.h"

namespace hfrk {

constexpr int kDynMaxThreads = 1024;
constexpr int kDynMaxIters = 4;

__device__ __forceinline__ float dyn_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float dyn_wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Sum / max over the workgroup; every thread returns the same bits.  `red` holds 16 floats and is not reused.
__device__ __forceinline__ float dyn_block_sum(float v, float* red) {
    v = dyn_wave_sum(v);
    const int wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += red[w];
    return total;
}

__device__ __forceinline__ float dyn_block_max(float v, float* red) {
    v = dyn_wave_max(v);
    const int wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float m = 0.f;
    for (int w = 0; w < nwaves; ++w) m = fmaxf(m, red[w]);
    return m;
}

__device__ __forceinline__ void dyn_zero_row(uint16_t* next_buffer, int buffer_cols) {
    if (buffer_cols <= 0) return;
    uint16_t* const row = next_buffer + (long)blockIdx.x * buffer_cols;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(row);
    int head = (int)(((16 - (addr & 15)) & 15) >> 1);
    if (head > buffer_cols) head = buffer_cols;
    const int body = (buffer_cols - head) >> 3;
    for (int i = threadIdx.x; i < head; i += blockDim.x) row[i] = 0;
    uint4* const vec = reinterpret_cast<uint4*>(row + head);
    for (int i = threadIdx.x; i < body; i += blockDim.x) vec[i] = make_uint4(0, 0, 0, 0);
    for (int i = head + body * 8 + threadIdx.x; i < buffer_cols; i += blockDim.x) row[i] = 0;
}

// Quantise the cached row: scale from the row maximum, 8 values per 8-byte store.
template <int ITERS>
__device__ __forceinline__ void dyn_quantise_row(const float (&y)[ITERS][8], float amax, uint8_t* out_row, float* scales,
                                                 int nvec) {
    const float scale = fmaxf(amax / 448.0f, FLT_MIN);
    const float inv = 1.0f / scale;
    if (threadIdx.x == 0) scales[blockIdx.x] = scale;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
        if (v < nvec) {
            uint32_t p0 = cvt_pk_fp8(y[it][0] * inv, y[it][1] * inv, 0u, false);
            p0 = cvt_pk_fp8(y[it][2] * inv, y[it][3] * inv, p0, true);
            uint32_t p1 = cvt_pk_fp8(y[it][4] * inv, y[it][5] * inv, 0u, false);
            p1 = cvt_pk_fp8(y[it][6] * inv, y[it][7] * inv, p1, true);
            reinterpret_cast<uint2*>(out_row)[v] = make_uint2(p0, p1);
        }
    }
}

template <int DT, int ITERS>
__global__ void __launch_bounds__(kDynMaxThreads) residual_rms_dynamic_kernel(
    const uint16_t* __restrict__ input, uint16_t* __restrict__ residual, const uint16_t* __restrict__ weight,
    uint8_t* __restrict__ output, float* __restrict__ scales, uint16_t* __restrict__ next_buffer, float epsilon, int cols,
    int buffer_cols) {
    __shared__ float red_sum[16], red_max[16];
    const long row_off = (long)blockIdx.x * cols;
    const int nvec = cols >> 3;
    uint4 wreg[ITERS];
    float y[ITERS][8];
    float ssq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
        wreg[it] = make_uint4(0, 0, 0, 0);
        if (v < nvec) wreg[it] = reinterpret_cast<const uint4*>(weight)[v];
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[it][j] = 0.f;
        if (v < nvec) {
            const uint4 a = reinterpret_cast<const uint4*>(input + row_off)[v];
            const uint4 r = reinterpret_cast<const uint4*>(residual + row_off)[v];
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, rw[4] = {r.x, r.y, r.z, r.w};
            uint32_t zw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint16_t lo = store16<DT>(load16<DT>((uint16_t)(aw[j] & 0xffff)) + load16<DT>((uint16_t)(rw[j] & 0xffff)));
                const uint16_t hi = store16<DT>(load16<DT>((uint16_t)(aw[j] >> 16)) + load16<DT>((uint16_t)(rw[j] >> 16)));
                y[it][2 * j] = load16<DT>(lo);
                y[it][2 * j + 1] = load16<DT>(hi);
                ssq += y[it][2 * j] * y[it][2 * j];
                ssq += y[it][2 * j + 1] * y[it][2 * j + 1];
                zw[j] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            reinterpret_cast<uint4*>(residual + row_off)[v] = make_uint4(zw[0], zw[1], zw[2], zw[3]);
        }
    }
    const float norm = rsqrtf(dyn_block_sum(ssq, red_sum) / (float)cols + epsilon);
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const uint32_t ww[4] = {wreg[it].x, wreg[it].y, wreg[it].z, wreg[it].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            y[it][2 * j] = y[it][2 * j] * norm * load16<DT>((uint16_t)(ww[j] & 0xffff));
            y[it][2 * j + 1] = y[it][2 * j + 1] * norm * load16<DT>((uint16_t)(ww[j] >> 16));
            amax = fmaxf(amax, fmaxf(fabsf(y[it][2 * j]), fabsf(y[it][2 * j + 1])));
        }
    }
    amax = dyn_block_max(amax, red_max);
    dyn_quantise_row<ITERS>(y, amax, output + row_off, scales, nvec);
    dyn_zero_row(next_buffer, buffer_cols);
}

template <int DT, int ITERS>
__global__ void __launch_bounds__(kDynMaxThreads) swiglu_dynamic_kernel(
    const uint16_t* __restrict__ gate_up, uint8_t* __restrict__ output, float* __restrict__ scales,
    uint16_t* __restrict__ next_buffer, int cols, int buffer_cols) {
    __shared__ float red_max[16];
    const uint16_t* const grow = gate_up + (long)blockIdx.x * 2 * cols;
    const int nvec = cols >> 3;
    float y[ITERS][8];
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[it][j] = 0.f;
        if (v < nvec) {
            const v4i g = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(grow) + v);
            const v4i u = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(grow + cols) + v);
            const uint32_t gw[4] = {(uint32_t)g[0], (uint32_t)g[1], (uint32_t)g[2], (uint32_t)g[3]};
            const uint32_t uw[4] = {(uint32_t)u[0], (uint32_t)u[1], (uint32_t)u[2], (uint32_t)u[3]};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                y[it][2 * j] = silu_mul(load16<DT>((uint16_t)(gw[j] & 0xffff)), load16<DT>((uint16_t)(uw[j] & 0xffff)), 1.0f);
                y[it][2 * j + 1] = silu_mul(load16<DT>((uint16_t)(gw[j] >> 16)), load16<DT>((uint16_t)(uw[j] >> 16)), 1.0f);
                amax = fmaxf(amax, fmaxf(fabsf(y[it][2 * j]), fabsf(y[it][2 * j + 1])));
            }
        }
    }
    amax = dyn_block_max(amax, red_max);
    dyn_quantise_row<ITERS>(y, amax, output + (long)blockIdx.x * cols, scales, nvec);
    dyn_zero_row(next_buffer, buffer_cols);
}

// Plain quantisation of a 16-bit activation block (what sits between an attention output and the o_proj GEMM):
// dynamic (static_scale == nullptr): scales[row] = max(amax_row |x| / 448, FLT_MIN), output = e4m3fn(x / scales[row]);
// static: output = e4m3fn(x / static_scale[0]), saturating, scales untouched.
template <int DT, int ITERS>
__global__ void __launch_bounds__(kDynMaxThreads) quantize_rows_kernel(
    const uint16_t* __restrict__ input, const float* __restrict__ static_scale, uint8_t* __restrict__ output,
    float* __restrict__ scales, int cols) {
    __shared__ float red_max[16];
    const uint16_t* const row = input + (long)blockIdx.x * cols;
    const int nvec = cols >> 3;
    float y[ITERS][8];
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[it][j] = 0.f;
        if (v < nvec) {
            const v4i x = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(row) + v);
            const uint32_t xw[4] = {(uint32_t)x[0], (uint32_t)x[1], (uint32_t)x[2], (uint32_t)x[3]};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                y[it][2 * j] = load16<DT>((uint16_t)(xw[j] & 0xffff));
                y[it][2 * j + 1] = load16<DT>((uint16_t)(xw[j] >> 16));
                amax = fmaxf(amax, fmaxf(fabsf(y[it][2 * j]), fabsf(y[it][2 * j + 1])));
            }
        }
    }
    if (static_scale) {
        const float inv = 1.0f / static_scale[0];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int v = threadIdx.x + it * blockDim.x;
            if (v < nvec) {
                uint32_t p0 = cvt_pk_fp8(y[it][0] * inv, y[it][1] * inv, 0u, false);
                p0 = cvt_pk_fp8(y[it][2] * inv, y[it][3] * inv, p0, true);
                uint32_t p1 = cvt_pk_fp8(y[it][4] * inv, y[it][5] * inv, 0u, false);
                p1 = cvt_pk_fp8(y[it][6] * inv, y[it][7] * inv, p1, true);
                reinterpret_cast<uint2*>(output + (long)blockIdx.x * cols)[v] = make_uint2(p0, p1);
            }
        }
        return;
    }
    amax = dyn_block_max(amax, red_max);
    dyn_quantise_row<ITERS>(y, amax, output + (long)blockIdx.x * cols, scales, nvec);
}

static bool dyn_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// threads and register-cache depth for a row of `nvec` 16-byte pieces; false when the row does not fit
static bool dyn_geometry(int nvec, int* threads, int* iters) {
    int t = ((nvec + 63) / 64) * 64;
    if (t > 512) t = ((nvec + 127) / 128) * 64;  // two pieces per thread before going to 1024 threads
    if (t > kDynMaxThreads) t = kDynMaxThreads;
    if (t < 64) t = 64;
    const int it = (nvec + t - 1) / t;
    if (it > kDynMaxIters) return false;
    *threads = t;
    *iters = it <= 1 ? 1 : it == 2 ? 2 : 4;
    return true;
}

}  // namespace hfrk

extern "C" int hfrk_residual_rms_dynamic(const void* input, void* residual, const void* weight, float epsilon, void* output,
                                         float* scales, void* next_buffer, int rows, int cols, int buffer_cols,
                                         int io_dtype, void* stream) {
    using namespace hfrk;
    if (rows < 0 || cols < 1 || buffer_cols < 0 || cols % 8 != 0) return HFRK_BAD_SHAPE;
    if (rows == 0) return HFRK_SUCCESS;
    if (!input || !residual || !weight || !output || !scales) return HFRK_BAD_SHAPE;
    if (buffer_cols > 0 && !next_buffer) return HFRK_BAD_SHAPE;
    if (io_dtype != HFRK_F16 && io_dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
    if (!dyn_aligned16(input) || !dyn_aligned16(residual) || !dyn_aligned16(weight) || (reinterpret_cast<uintptr_t>(output) & 7))
        return HFRK_BAD_ALIGNMENT;
    int threads = 0, iters = 0;
    if (!dyn_geometry(cols / 8, &threads, &iters)) return HFRK_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t* in = static_cast<const uint16_t*>(input);
    uint16_t* res = static_cast<uint16_t*>(residual);
    const uint16_t* w = static_cast<const uint16_t*>(weight);
    uint8_t* out = static_cast<uint8_t*>(output);
    uint16_t* nb = static_cast<uint16_t*>(next_buffer);
#define HFRK_DYN_RMS(DT_, IT_)                                                                                       \
    hipLaunchKernelGGL((residual_rms_dynamic_kernel<DT_, IT_>), dim3(rows), dim3(threads), 0, s, in, res, w, out,     \
                       scales, nb, epsilon, cols, buffer_cols)
    if (io_dtype == HFRK_F16) {
        if (iters == 1) HFRK_DYN_RMS(HFRK_F16, 1); else if (iters == 2) HFRK_DYN_RMS(HFRK_F16, 2); else HFRK_DYN_RMS(HFRK_F16, 4);
    } else {
        if (iters == 1) HFRK_DYN_RMS(HFRK_BF16, 1); else if (iters == 2) HFRK_DYN_RMS(HFRK_BF16, 2); else HFRK_DYN_RMS(HFRK_BF16, 4);
    }
#undef HFRK_DYN_RMS
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

extern "C" int hfrk_swiglu_dynamic(const void* gate_up, void* output, float* scales, void* next_buffer, int rows, int cols,
                                   int buffer_cols, int io_dtype, void* stream) {
    using namespace hfrk;
    if (rows < 0 || cols < 1 || buffer_cols < 0 || cols % 8 != 0) return HFRK_BAD_SHAPE;
    if (rows == 0) return HFRK_SUCCESS;
    if (!gate_up || !output || !scales) return HFRK_BAD_SHAPE;
    if (buffer_cols > 0 && !next_buffer) return HFRK_BAD_SHAPE;
    if (io_dtype != HFRK_F16 && io_dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
    if (!dyn_aligned16(gate_up) || (reinterpret_cast<uintptr_t>(output) & 7)) return HFRK_BAD_ALIGNMENT;
    int threads = 0, iters = 0;
    if (!dyn_geometry(cols / 8, &threads, &iters)) return HFRK_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t* in = static_cast<const uint16_t*>(gate_up);
    uint8_t* out = static_cast<uint8_t*>(output);
    uint16_t* nb = static_cast<uint16_t*>(next_buffer);
#define HFRK_DYN_SWIGLU(DT_, IT_)                                                                                    \
    hipLaunchKernelGGL((swiglu_dynamic_kernel<DT_, IT_>), dim3(rows), dim3(threads), 0, s, in, out, scales, nb, cols, \
                       buffer_cols)
    if (io_dtype == HFRK_F16) {
        if (iters == 1) HFRK_DYN_SWIGLU(HFRK_F16, 1); else if (iters == 2) HFRK_DYN_SWIGLU(HFRK_F16, 2); else HFRK_DYN_SWIGLU(HFRK_F16, 4);
    } else {
        if (iters == 1) HFRK_DYN_SWIGLU(HFRK_BF16, 1); else if (iters == 2) HFRK_DYN_SWIGLU(HFRK_BF16, 2); else HFRK_DYN_SWIGLU(HFRK_BF16, 4);
    }
#undef HFRK_DYN_SWIGLU
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

extern "C" int hfrk_quantize_fp8(const void* input, const float* static_scale, void* output, float* scales, int rows, int cols,
                                 int io_dtype, void* stream) {
    using namespace hfrk;
    if (rows < 0 || cols < 1 || cols % 8 != 0) return HFRK_BAD_SHAPE;
    if (rows == 0) return HFRK_SUCCESS;
    if (!input || !output || (!static_scale && !scales)) return HFRK_BAD_SHAPE;
    if (io_dtype != HFRK_F16 && io_dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
    if (!dyn_aligned16(input) || (reinterpret_cast<uintptr_t>(output) & 7)) return HFRK_BAD_ALIGNMENT;
    int threads = 0, iters = 0;
    if (!dyn_geometry(cols / 8, &threads, &iters)) return HFRK_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t* in = static_cast<const uint16_t*>(input);
    uint8_t* out = static_cast<uint8_t*>(output);
#define HFRK_QUANT(DT_, IT_) \
    hipLaunchKernelGGL((quantize_rows_kernel<DT_, IT_>), dim3(rows), dim3(threads), 0, s, in, static_scale, out, scales, cols)
    if (io_dtype == HFRK_F16) {
        if (iters == 1) HFRK_QUANT(HFRK_F16, 1); else if (iters == 2) HFRK_QUANT(HFRK_F16, 2); else HFRK_QUANT(HFRK_F16, 4);
    } else {
        if (iters == 1) HFRK_QUANT(HFRK_BF16, 1); else if (iters == 2) HFRK_QUANT(HFRK_BF16, 2); else HFRK_QUANT(HFRK_BF16, 4);
    }
#undef HFRK_QUANT
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}
