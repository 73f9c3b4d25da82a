// Host-side planner of the FP8 skinny GEMM: which decomposition (hfrk_gemm_plan) a shape gets, and the check every plan
// passes before a launch, whether it comes from the planner, from a caller or from a plan table.  Counterpart of the
// reference's launcher-side shape checks and knob table (csrc/op_src/skinny_gemm/skinny_gemm_caller.cu:21-460,
// hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102).  Implemented in skinny_gemm_plan.hip; host code only.
#pragma once
#include "skinny_gemm_args.h"

namespace hfrk {

// LDS of the workgroup kernel: a 4 KB weight tile per wave and weight tile, two activation slabs of 16*mt rows
constexpr int lds_bytes_for(int mt, int wk, int ch, int rt = 1) {
    return kGemmWaves * rt * kTileBytes + 2 * 16 * mt * (256 * wk * ch);
}

// One decomposition, filled in for a shape (grid_hint 0: the decomposition's own choice of grid)
int fill_stream_plan(int m, int n, int k, int row_tiles, bool swiglu, int grid_hint, hfrk_gemm_plan* plan);
int fill_rows_plan(int m, int n, int k, int row_tiles, int grid_hint, hfrk_gemm_plan* plan);
int fill_rows_tiled_plan(int m, int n, int k, int row_tiles, int grid_hint, hfrk_gemm_plan* plan);
// The planner's rules per decomposition (HFRK_INVALID_CONFIG: not this decomposition for this shape)
int make_rows_plan(int m, int n, int k, hfrk_gemm_plan* plan);
int make_rows_tiled_plan(int m, int n, int k, hfrk_gemm_plan* plan);
int make_ksplit_plan(int m, int n, int k, hfrk_gemm_plan* plan);
// The planner: the plan of a plain GEMM call that brings none
int make_plan(int m, int n, int k, hfrk_gemm_plan* plan, bool packed = false);
// The plan of a launch with the RMSNorm prologue, or HFRK_BAD_SHAPE where the prologue does not exist
int make_rms_plan(int m, int n, int k, bool swiglu, hfrk_gemm_plan* p);
// Whether the kernels can run this plan on this shape (n: output columns with the SwiGLU epilogue)
int check_plan(int m, int n, int k, bool swiglu, const hfrk_gemm_plan* p, bool packed = false);
// Workspace bytes and arrival counters a plan's kernel may touch
size_t plan_ws_bytes(const hfrk_gemm_plan& p);
long plan_counters(const hfrk_gemm_plan& p);

}  // namespace hfrk
