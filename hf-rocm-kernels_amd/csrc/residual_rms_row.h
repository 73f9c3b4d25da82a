// One row of the residual RMSNorm on 16-byte vectors, shared by the stand-alone kernel (residual_rms.hip) and by the
// single-launch MLP block (llama_mlp_block.hip): both run exactly this arithmetic in exactly this order, so a row
// normalised by either has the same bits.  The arithmetic is described at the top of residual_rms.hip.
#pragma once

#include "hfrk_internal.h"

namespace hfrk {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

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

// The workgroup normalises row `row`: 8 elements (16 bytes) per thread per iteration, ITERS iterations cached in
// registers (cols <= 8 * blockDim * ITERS, cols % 8 == 0, 16-byte aligned rows).  `red`: 16 floats of LDS.
// COHERENT: residual and output are stored write-through (sc0 sc1), for readers in other workgroups of the same launch.
template <int DT, bool FP8_OUT, int ITERS, bool COHERENT>
__device__ __forceinline__ void rms_row_vec(const uint16_t* __restrict__ input, uint16_t* __restrict__ residual,
                                            const uint16_t* __restrict__ weight, const float* __restrict__ scale_tensor,
                                            void* __restrict__ output, float epsilon, int cols, int row, float* red) {
    constexpr int kWriteThrough = 17;  // sc0 | sc1
    [[maybe_unused]] __amdgpu_buffer_rsrc_t res_rsrc, out_rsrc;
    if constexpr (COHERENT) {
        res_rsrc = make_rsrc(residual + (long)row * cols, (uint32_t)cols * 2u);
        out_rsrc = make_rsrc(static_cast<uint8_t*>(output) + (long)row * cols * (FP8_OUT ? 1 : 2), (uint32_t)cols * (FP8_OUT ? 1u : 2u));
    }
    const long row_off = (long)row * cols;
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
            z[it] = make_uint4(zw[0], zw[1], zw[2], zw[3]);
            if constexpr (COHERENT) __builtin_amdgcn_raw_buffer_store_b128(v4i{(int)zw[0], (int)zw[1], (int)zw[2], (int)zw[3]}, res_rsrc, (int)((uint32_t)v * 16u), 0, kWriteThrough);
            else reinterpret_cast<uint4*>(residual + row_off)[v] = z[it];
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
                if constexpr (COHERENT) __builtin_amdgcn_raw_buffer_store_b64(v2i{(int)p0, (int)p1}, out_rsrc, (int)((uint32_t)v * 8u), 0, kWriteThrough);
                else reinterpret_cast<uint2*>(static_cast<uint8_t*>(output) + row_off)[v] = make_uint2(p0, p1);
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
                if constexpr (COHERENT) __builtin_amdgcn_raw_buffer_store_b128(v4i{(int)ow[0], (int)ow[1], (int)ow[2], (int)ow[3]}, out_rsrc, (int)((uint32_t)v * 16u), 0, kWriteThrough);
                else reinterpret_cast<uint4*>(static_cast<uint16_t*>(output) + row_off)[v] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
            }
        }
    }
}

}  // namespace hfrk
