// residual <- input + residual;  output <- rmsnorm(residual) * weight [ / scale -> fp8 e4m3fn ];  next_buffer <- 0
//
// Replaces csrc/op_src/residual_rms/residual_rms_dispatch.cu:8-63 and its two kernels
// (residual_rms_scalar.cu:11-74, residual_rms_vectorized.cu:13-172).  One workgroup per row.  The summed row is
// kept in registers between the two passes (the reference parks it in a 32 KB LDS array), the sum of squares is
// reduced with cross-lane shuffles inside each wavefront and one LDS exchange of <= 16 floats between wavefronts,
// and every thread adds those partials in the same order, so the normaliser is identical for the whole row.
//
// Arithmetic (same points of rounding as the reference's torch functions, operators/residual_rms/reference.py:7-36):
//   z   = round16(float(input) + float(residual))            -> stored to residual, bit-exact with a torch add
//   r   = rsqrt(mean(float(z)^2) + eps)                      fp32
//   16-bit output:  round16( float(round16(float(z) * r)) * float(weight) )
//   fp8 output:     e4m3fn( clamp( float(z) * r * float(weight) * (1/scale), +-448 ) )   no 16-bit detour, as in
//                   the reference's vectorised kernel (residual_rms_vectorized.cu:124-135)
#include "hfrk_internal.h"

namespace hfrk {

constexpr int kRmsMaxThreads = 1024;

// Sum over the workgroup; every thread returns the same bits.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += red[w];
    return total;
}

__device__ __forceinline__ void zero_next_buffer_row(uint16_t* next_buffer, int buffer_cols) {
    if (buffer_cols <= 0) return;
    uint16_t* const row = next_buffer + (long)blockIdx.x * buffer_cols;
    // 16-byte stores where the row allows it, element stores for the ragged ends
    const uintptr_t addr = reinterpret_cast<uintptr_t>(row);
    int head = (int)(((16 - (addr & 15)) & 15) >> 1);
    if (head > buffer_cols) head = buffer_cols;
    const int body = (buffer_cols - head) >> 3;
    for (int i = threadIdx.x; i < head; i += blockDim.x) row[i] = 0;
    uint4* const vec = reinterpret_cast<uint4*>(row + head);
    for (int i = threadIdx.x; i < body; i += blockDim.x) vec[i] = make_uint4(0, 0, 0, 0);
    for (int i = head + body * 8 + threadIdx.x; i < buffer_cols; i += blockDim.x) row[i] = 0;
}

// 8 elements (16 bytes) per thread per iteration, ITERS iterations cached in registers: cols <= 8*blockDim*ITERS.
template <int DT, bool FP8_OUT, int ITERS>
__global__ void __launch_bounds__(kRmsMaxThreads) residual_rms_vec_kernel(
    const uint16_t* __restrict__ input, uint16_t* __restrict__ residual, const uint16_t* __restrict__ weight,
    const float* __restrict__ scale_tensor, void* __restrict__ output, uint16_t* __restrict__ next_buffer,
    float epsilon, int cols, int buffer_cols) {
    __shared__ float red[16];
    const long row_off = (long)blockIdx.x * cols;
    const int nvec = cols >> 3;
    uint4 z[ITERS], wreg[ITERS];
    float ssq = 0.f;
    // Everything the second pass needs is requested now, so that the kernel pays one memory latency, not two.
    float scale = 1.f;
    if constexpr (FP8_OUT) scale = scale_tensor[0];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
        wreg[it] = make_uint4(0, 0, 0, 0);
        if (v < nvec) wreg[it] = reinterpret_cast<const uint4*>(weight)[v];
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
        if (v < nvec) {
            const uint4 a = reinterpret_cast<const uint4*>(input + row_off)[v];
            const uint4 r = reinterpret_cast<const uint4*>(residual + row_off)[v];
            z[it] = rms_add_square<DT>(a, r, ssq);
            reinterpret_cast<uint4*>(residual + row_off)[v] = z[it];
        }
    }
    const float total = block_sum(ssq, red);
    const float norm = rsqrtf(total / (float)cols + epsilon);
    const float inv_scale = 1.f / scale;

#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = threadIdx.x + it * blockDim.x;
        if (v < nvec) {
            const uint4 w = wreg[it];
            const uint32_t zw[4] = {z[it].x, z[it].y, z[it].z, z[it].w}, ww[4] = {w.x, w.y, w.z, w.w};
            if constexpr (FP8_OUT) {
                reinterpret_cast<uint2*>(static_cast<uint8_t*>(output) + row_off)[v] = rms_scale_to_fp8<DT>(z[it], w, norm, inv_scale);
            } else {
                uint32_t ow[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint16_t nl = store16<DT>(load16<DT>((uint16_t)(zw[j] & 0xffff)) * norm);
                    const uint16_t nh = store16<DT>(load16<DT>((uint16_t)(zw[j] >> 16)) * norm);
                    const uint16_t ol = store16<DT>(load16<DT>(nl) * load16<DT>((uint16_t)(ww[j] & 0xffff)));
                    const uint16_t oh = store16<DT>(load16<DT>(nh) * load16<DT>((uint16_t)(ww[j] >> 16)));
                    ow[j] = (uint32_t)ol | ((uint32_t)oh << 16);
                }
                reinterpret_cast<uint4*>(static_cast<uint16_t*>(output) + row_off)[v] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
            }
        }
    }
    zero_next_buffer_row(next_buffer, buffer_cols);
}

// One element per thread per iteration; no alignment or divisibility requirement.  The second pass re-reads the
// residual this same thread wrote in the first.
template <int DT, bool FP8_OUT>
__global__ void __launch_bounds__(kRmsMaxThreads) residual_rms_scalar_kernel(
    const uint16_t* __restrict__ input, uint16_t* __restrict__ residual, const uint16_t* __restrict__ weight,
    const float* __restrict__ scale_tensor, void* __restrict__ output, uint16_t* __restrict__ next_buffer,
    float epsilon, int cols, int buffer_cols) {
    __shared__ float red[16];
    const long row_off = (long)blockIdx.x * cols;
    float ssq = 0.f;
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const uint16_t z = store16<DT>(load16<DT>(input[row_off + i]) + load16<DT>(residual[row_off + i]));
        const float f = load16<DT>(z);
        ssq += f * f;
        residual[row_off + i] = z;
    }
    const float total = block_sum(ssq, red);
    const float norm = rsqrtf(total / (float)cols + epsilon);
    float inv_scale = 1.f;
    if constexpr (FP8_OUT) inv_scale = 1.f / scale_tensor[0];
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const float zf = load16<DT>(residual[row_off + i]);
        const float wf = load16<DT>(weight[i]);
        if constexpr (FP8_OUT) {
            static_cast<uint8_t*>(output)[row_off + i] = cvt_fp8(zf * norm * wf * inv_scale);
        } else {
            const uint16_t n16 = store16<DT>(zf * norm);
            static_cast<uint16_t*>(output)[row_off + i] = store16<DT>(load16<DT>(n16) * wf);
        }
    }
    zero_next_buffer_row(next_buffer, buffer_cols);
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int DT, bool FP8_OUT>
static int launch_rms(const void* input, void* residual, const void* weight, const float* scale_tensor, float epsilon,
                      void* output, void* next_buffer, int rows, int cols, int buffer_cols, int num_threads,
                      bool force_scalar, hipStream_t stream) {
    const uint16_t* in = static_cast<const uint16_t*>(input);
    uint16_t* res = static_cast<uint16_t*>(residual);
    const uint16_t* w = static_cast<const uint16_t*>(weight);
    uint16_t* nb = static_cast<uint16_t*>(next_buffer);
    // 16-byte path: aligned rows (cols % 8 == 0 keeps every row aligned) and an aligned output row
    const bool out_ok = FP8_OUT ? ((reinterpret_cast<uintptr_t>(output) & 7) == 0) : aligned16(output);
    bool vec = !force_scalar && (cols % 8 == 0) && aligned16(input) && aligned16(residual) && aligned16(weight) && out_ok;
    int threads = num_threads;
    if (vec) {
        const int nvec = cols / 8;
        if (threads == 0) {
            // enough threads for one or two 16-byte pieces each, whole wavefronts, at most 1024
            threads = ((nvec + 63) / 64) * 64;
            if (threads > 512) threads = ((nvec + 127) / 128) * 64;
            if (threads > kRmsMaxThreads) threads = kRmsMaxThreads;
            if (threads < 64) threads = 64;
        }
        const int iters = (nvec + threads - 1) / threads;
        if (iters > 4) vec = false;  // would not fit the register cache: fall through to the strided kernel
        else {
#define HFRK_RMS_LAUNCH(IT)                                                                                          \
    hipLaunchKernelGGL((residual_rms_vec_kernel<DT, FP8_OUT, IT>), dim3(rows), dim3(threads), 0, stream, in, res, w, \
                       scale_tensor, output, nb, epsilon, cols, buffer_cols)
            if (iters <= 1) HFRK_RMS_LAUNCH(1);
            else if (iters == 2) HFRK_RMS_LAUNCH(2);
            else HFRK_RMS_LAUNCH(4);
#undef HFRK_RMS_LAUNCH
        }
    }
    if (!vec) {
        if (threads == 0) {
            threads = ((cols + 63) / 64) * 64;
            if (threads > kRmsMaxThreads) threads = kRmsMaxThreads;
        }
        hipLaunchKernelGGL((residual_rms_scalar_kernel<DT, FP8_OUT>), dim3(rows), dim3(threads), 0, stream, in, res, w,
                           scale_tensor, output, nb, epsilon, cols, buffer_cols);
    }
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

}  // namespace hfrk

extern "C" int hfrk_residual_rms(const void* input, void* residual, const void* weight, const float* scale_tensor,
                                 float epsilon, void* output, void* next_buffer, int rows, int cols, int buffer_cols,
                                 int io_dtype, int out_dtype, int num_threads, int force_scalar, void* stream) {
    using namespace hfrk;
    if (rows < 0 || cols < 1 || buffer_cols < 0) return HFRK_BAD_SHAPE;
    if (rows == 0) return HFRK_SUCCESS;
    if (!input || !residual || !weight || !output) return HFRK_BAD_SHAPE;
    if (buffer_cols > 0 && !next_buffer) return HFRK_BAD_SHAPE;
    if (io_dtype != HFRK_F16 && io_dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
    if (out_dtype != HFRK_FP8_E4M3FN && out_dtype != io_dtype) return HFRK_BAD_DTYPE;
    if (out_dtype == HFRK_FP8_E4M3FN && !scale_tensor) return HFRK_BAD_SHAPE;
    if (num_threads < 0 || num_threads > kRmsMaxThreads || (num_threads % 64) != 0) return HFRK_INVALID_CONFIG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fs = force_scalar != 0;
    const bool fp8 = out_dtype == HFRK_FP8_E4M3FN;
    if (io_dtype == HFRK_F16) {
        return fp8 ? launch_rms<HFRK_F16, true>(input, residual, weight, scale_tensor, epsilon, output, next_buffer, rows, cols, buffer_cols, num_threads, fs, s)
                   : launch_rms<HFRK_F16, false>(input, residual, weight, scale_tensor, epsilon, output, next_buffer, rows, cols, buffer_cols, num_threads, fs, s);
    }
    return fp8 ? launch_rms<HFRK_BF16, true>(input, residual, weight, scale_tensor, epsilon, output, next_buffer, rows, cols, buffer_cols, num_threads, fs, s)
               : launch_rms<HFRK_BF16, false>(input, residual, weight, scale_tensor, epsilon, output, next_buffer, rows, cols, buffer_cols, num_threads, fs, s);
}
