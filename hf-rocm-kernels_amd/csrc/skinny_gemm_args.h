// Launch arguments and device workspace shared by the two skinny-GEMM kernels.
#pragma once

#include "hfrk_internal.h"

namespace hfrk {

constexpr int kGemmWaves = 8;
constexpr int kGemmThreads = kGemmWaves * kWave;
constexpr int kTileBytes = 4096;       // 16 rows x 256 B: one K chunk of one 16-row tile
constexpr int kLdsLimit = 160 * 1024;  // LDS per CU on gfx950
constexpr int kMaxPanels = 1 << 20;    // arrival counters (one per row panel / row tile)
constexpr int kMaxDevices = 64;     // devices this library keeps per-device state for
constexpr int kMaxGrid = 4 * kNumCU;   // what the workspace is sized for
// Largest grid a plan may ask for.  The row-split and wave-stream kernels take up to two workgroups per compute unit (the
// planner itself uses that for short bands at up to 4 rows, and forced plans of that size are part of the GPU tests); the
// K-split and workgroup kernels take one.  Larger grids were accepted once; a tuner sweep that forced them on 2048-row
// weights ended in a GPU fault whose cause was never found, no test covers them, and no measurement ever favoured them,
// so the launcher refuses them.
constexpr int kMaxStreamGrid = 2 * kNumCU;
constexpr size_t kWsFloats = (size_t)2 * kMaxGrid * kGemmWaves * 4 * 256;  // 2 slots x grid x up to 32 KB of fp32 partials

struct GemmArgs {
    const uint8_t* A;
    const uint8_t* B;
    void* D;
    const void* base;        // accumulate mode: the 16-bit [m,n] tensor added to the product (may be D itself); else null
    const float* out_scale;  // SwiGLU epilogue: the fp8 output is divided by out_scale[0]
    const float* scale_a;
    const float* scale_b;
    int sa_stride, sb_stride;
    int m, n, k, b_stride;
    int packed;              // B is in the pre-packed layout of pack_weight.hip (b_stride unused)
    int d_dtype;             // dtype of D; with the SwiGLU epilogue the 16-bit dtype the projections are rounded to
    int panels, slabs, units, grid;  // units = panels * slabs
    int chunks_q, chunks_r;  // stream kernel: (panels * slabs) / grid and % grid
    // row-split kernel: 4-row units per workgroup (rows_q, the first rows_r workgroups one more), and for both band
    // heights (a: rows_q + 1 units, b: rows_q) the tiles of a band, units per tile and how many tiles have one more.
    // On bands of whole 16-row tiles (skinny_gemm_rows_tiled.hip) rows_q / rows_r count those tiles, tiles_a / tiles_b the chunks
    // per 256 bytes of k (up to row_tiles 16-row tiles each), and base / extra are unused.
    int rows_q, rows_r;
    int tiles_a, base_a, extra_a, tiles_b, base_b, extra_b;
    uint32_t kc_magic;       // ceil(2^32 / slabs): i / slabs == umulhi(i, kc_magic) for the chunk indices of a band
    // row-split kernel: workgroup g walks k from chunk g mod slabs on (and wraps round).  Set for rows a multiple of 4 KB
    // apart when the 2048 waves of a launch would otherwise ask for the same offset within 4 KB at every moment: either
    // because every wave's run of chunks is a multiple of 16 long (13312 x 16384 at 8 rows: 41.7 us without, 33.7 with;
    // 16384 x 16384: 53.4 / 43.5), or because from 9 activation rows on all workgroups pull the same activation lines out
    // of L2 together (6144 x 4096 at 16 rows: 7.10 / 6.77; bands of at least 4 units).  Elsewhere the rotation costs 1-3 %.
    int k_rotate;
    // row-split kernel with the RMSNorm prologue (A is then unused): residual_out <- input + residual,
    // activations = e4m3fn(rmsnorm(residual_out) * weight / act_scale[0]), built in every workgroup's LDS
    const uint16_t* rms_input;
    const uint16_t* rms_residual;
    uint16_t* rms_residual_out;
    const uint16_t* rms_weight;
    const float* rms_act_scale;
    float rms_epsilon;
    int rms_dtype;           // HFRK_F16 / HFRK_BF16 of input, residual and weight
    float* ws;               // fp32 partial sums that cross workgroups
    uint32_t ws_bytes;       // size of ws: accesses beyond it are dropped by the buffer range check
    int* counters;           // arrival counters, zero between launches
};

// wave-stream kernel (m <= 32), skinny_gemm_stream.hip: act_loads = ceil(m/4) 16-byte activation loads per lane and
// chunk, row_tiles = 16-row weight tiles per chunk (1: act_loads 1..4; 2: act_loads 3..8)
// swiglu: the weight holds gate rows [0, n/2) and up rows [n/2, n); a chunk pairs gate tile t with up tile t
// (row_tiles must be 2) and the epilogue writes fp8(silu(gate) * up / out_scale) to D [m, n/2].
int launch_stream_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, int lds_bytes, hipStream_t stream);
constexpr int kStreamMaxM = 32;
constexpr int kStreamRt2MinChunksPerWave = 4;  // 9 <= m <= 16: two row tiles per chunk only if runs stay this long
constexpr int stream_lds_bytes(int act_loads, int row_tiles) {
    return kGemmWaves * (row_tiles + (act_loads + 3) / 4) * kTileBytes;
}
constexpr bool stream_variant_exists(int act_loads, int row_tiles, bool swiglu = false) {
    return swiglu ? (row_tiles == 2 && act_loads >= 1 && act_loads <= 4)
                  : (row_tiles == 1 && act_loads >= 1 && act_loads <= 4) || (row_tiles == 2 && act_loads >= 3 && act_loads <= 8);
}

// row-split wave-stream kernel (m <= 16), skinny_gemm_rows.hip: every workgroup owns a band of weight rows and all of k;
// act_loads = ceil(m/4), row_tiles = 16-row matrix tiles per chunk (1 or 2).  Needs k >= 512.
// swiglu: gate rows [0, n/2), up rows [n/2, n); row_tiles must be 2 (a gate and an up tile per chunk), bands and tiles count
// the n/2 output columns, D is fp8 [m, n/2]
// rms: the RMSNorm prologue (args.rms_*): up to 8 rows (act_loads <= 2), k = 4096 or 8192, row_tiles 1 (plain epilogue) or 2 (swiglu);
// lds_bytes is then rows_rms_lds_bytes(act_loads, row_tiles, k)
int launch_rows_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, bool rms, int lds_bytes, hipStream_t stream);
constexpr int kRowsRmsMaxM = 8;
constexpr int kRowsRmsRedBytes = 8 * kGemmWaves * 4;  // per-row, per-wave partial sums of squares
constexpr int rows_rms_lds_bytes(int act_loads, int row_tiles, int k) {
    return kGemmWaves * row_tiles * kTileBytes + kRowsRmsRedBytes + 4 * act_loads * k;  // weight tiles, partial sums, [4*act_loads, k] fp8
}
// the same kernel on bands of whole 16-row tiles (skinny_gemm_rows_tiled.hip): args.rows_q / rows_r count 16-row tiles (with swiglu:
// tiles of 16 output columns), args.packed selects the packed load format; no RMSNorm prologue
int launch_rows_tiled_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, int lds_bytes, hipStream_t stream);
constexpr int kRowsMaxM = 32;  // 17..32 rows: act_loads 6 (up to 24 rows) or 8, two matrix tiles per chunk
constexpr int rows_act_loads(int m) { return m <= 16 ? (m + 3) / 4 : m <= 24 ? 6 : 8; }
constexpr int rows_lds_bytes(int row_tiles, int act_loads) { return kGemmWaves * (row_tiles + (act_loads + 3) / 4) * kTileBytes; }
constexpr bool rows_variant_exists(int act_loads, int row_tiles) {
    return (act_loads >= 1 && act_loads <= 4 && (row_tiles == 1 || row_tiles == 2)) || ((act_loads == 6 || act_loads == 8) && row_tiles == 2);
}

// K-split kernel (skinny_gemm_ksplit.hip): the 8 waves of a workgroup split a K window of 8*wave_k bytes
// (wave_k = 256, 512, or 1024 with m_tiles <= 2), activations in registers.  Needs k % (8*wave_k) == 0.
// swiglu: gate rows [0, n/2), up rows [n/2, n); one window must cover K (wave_k = k / 8 = 256 or 512); panels counts the tiles of
// 16 output columns (n / 32), D is fp8 [m, n/2]
int launch_ksplit_kernel(const GemmArgs& args, int m_tiles, int wave_k, bool swiglu, int lds_bytes, hipStream_t stream);
constexpr bool ksplit_variant_exists(int m_tiles, int wave_k) {
    return m_tiles >= 1 && (((wave_k == 256 || wave_k == 512) && m_tiles <= 4) || (wave_k == 1024 && m_tiles <= 2));
}
constexpr int ksplit_lds_bytes(int m_tiles, int wave_k) {
    return kGemmWaves * (wave_k / 256) * kTileBytes + 2 * kGemmWaves * m_tiles * 1024;
}

}  // namespace hfrk
