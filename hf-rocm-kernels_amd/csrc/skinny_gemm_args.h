// Launch arguments and device workspace shared by the two skinny-GEMM kernels.
#pragma once

#include "hfrk_internal.h"

namespace hfrk {

constexpr int kGemmWaves = 8;
constexpr int kGemmThreads = kGemmWaves * kWave;
constexpr int kTileBytes = 4096;       // 16 rows x 256 B: one K chunk of one 16-row tile
constexpr int kLdsLimit = 160 * 1024;  // LDS per CU on gfx950
constexpr int kMaxPanels = 1 << 20;    // arrival counters (one per row panel / row tile)
constexpr int kMaxGrid = 4 * kNumCU;   // persistent workgroups: up to 4 per CU when LDS and registers allow
constexpr size_t kWsFloats = (size_t)2 * kMaxGrid * kGemmWaves * 4 * 256;  // 2 slots x grid x up to 32 KB of fp32 partials

struct GemmArgs {
    const uint8_t* A;
    const uint8_t* B;
    void* D;
    const float* scale_a;
    const float* scale_b;
    int sa_stride, sb_stride;
    int m, n, k, b_stride;
    int d_dtype, accumulate;
    int panels, slabs, units, grid, nbuf;
    int chunks_q, chunks_r;  // wave-stream kernel: (panels * slabs) / grid and % grid
    float* ws;
    int* counters;
};

// wave-stream kernel (m <= 16), skinny_gemm_stream.hip
int launch_stream_kernel(const GemmArgs& args, int act_loads, int lds_bytes, hipStream_t stream);
constexpr int kStreamLdsBytes = kGemmWaves * 2 * kTileBytes;

}  // namespace hfrk
