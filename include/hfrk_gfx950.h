/*
 * hfrk_gfx950.h -- C ABI of libhfrk_gfx950.so: FP8 skinny GEMM, residual RMSNorm and SwiGLU for MI355X (gfx950).
 *
 * Plain pointers and sizes only; every pointer is a DEVICE pointer unless stated otherwise, every call is
 * asynchronous on `stream` (a hipStream_t passed as void*; NULL = the default stream) and launches on the
 * device that is current on the calling thread.  No call synchronises or reads back, and after hfrk_init for that
 * device none allocates (unless more than four streams launch GEMMs, see hfrk_init), so all of them can be recorded
 * into a HIP graph.
 *
 * FP8 is OCP e4m3fn (bias 7, max 448, no infinities) -- the format gfx950's matrix cores implement.  The
 * reference was written for gfx942's e4m3fnuz; on the same bits an fnuz value is half the fn value.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference tree).
 */
#ifndef HFRK_GFX950_H
#define HFRK_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  0..6 are the reference's SkinnyGemmReturnCode (csrc/op_src/skinny_gemm/skinny_gemm_caller.cu:9-17),
 * same numbers, same conditions; the rest are additions of this library. */
enum hfrk_status {
    HFRK_SUCCESS = 0,
    HFRK_M_ABOVE_WARPTILE_M = 1,            /* never returned (the reference has the check commented out) */
    HFRK_N_NOT_EVEN = 2,
    HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K = 3, /* k % ((512/op_m)*ops) != 0; k % 16 != 0; k % 256 != 0 with a packed weight
                                             * or with an explicit plan of another kernel than the wave-stream one
                                             * (a variant of it handles a row that ends inside a 256-byte chunk by
                                             * masking the missing 16-byte pieces; without a plan, calls of more
                                             * than 32 rows then run as two launches) */
    HFRK_TOO_MANY_WARPS = 4,                /* A_producers + B_producers + consumers > 16 */
    HFRK_QSIZE_TOO_SMALL = 5,
    HFRK_INVALID_CONFIG = 6,                /* knob tuple outside the accepted domain */
    HFRK_BAD_SHAPE = 7,                     /* m < 1, m > 64, n < 1, k < 1, extent over 2 GiB ... */
    HFRK_BAD_ALIGNMENT = 8,                 /* a pointer or stride that must be 16-byte aligned is not */
    HFRK_BAD_DTYPE = 9,
    HFRK_HIP_ERROR = 10,                    /* a HIP runtime call failed; hfrk_last_hip_error() has the code */
    HFRK_NOT_INITIALISED = 11,              /* workspace missing and the stream is capturing (call hfrk_init first) */
    HFRK_BAD_FILE = 12,                     /* a plan-table file that cannot be read or is not a plan table */
    HFRK_NO_WORKSPACE = 13,                 /* more streams hold a split-K workspace than the library allows (hfrk_release_stream) */
    HFRK_EXCEEDS_SCRATCH = 14               /* hfrk_skinny_gemm_noalloc: the plan needs more than the built-in scratch array holds */
};

/* Element types of 16-bit tensors. */
enum hfrk_dtype { HFRK_F16 = 0, HFRK_BF16 = 1, HFRK_FP8_E4M3FN = 2 };

/* What happens to the product before it is stored (hfrk_skinny_gemm_fused). */
enum hfrk_epilogue { HFRK_EPILOGUE_NONE = 0, HFRK_EPILOGUE_SWIGLU = 1 };

/* FP8 flavour of a weight handed to hfrk_pack_weight. */
enum hfrk_weight_format { HFRK_WEIGHT_E4M3FN = 0, HFRK_WEIGHT_E4M3FNUZ = 1 };

/* Largest m the skinny GEMM accepts. */
#define HFRK_GEMM_MAX_M 64

/* How one GEMM call is decomposed.  Filled by hfrk_skinny_gemm_plan(); may be edited and passed back to
 * hfrk_skinny_gemm_ex() by an autotuner (counterpart of the knob table in
 * hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102 and benchmarks/skinny_gemm/grid_search.py). */
typedef struct hfrk_gemm_plan {
    int m_tiles;   /* ceil(m/16): 16-row activation tiles (wave-stream: 1..2, others: 1..4; row-split: always 1, the kernel takes its tiles from ch) */
    int wn;        /* which decomposition:
                      -2          row-split (m <= 32, k >= 512): every workgroup owns a band of weight rows and all of k;
                                  bands of any number of 4-row units, row-major weights only
                      -3          the same on bands of whole 16-row tiles: row-major weights and the packed load format
                                  (same bits from both)
                       0          wave-stream (m <= 32): every wave streams its own run of chunks
                      -1          K-split (k % (2048*wk) == 0): the 8 waves of a workgroup split K, activations in registers
                       1..16      workgroup: a panel is wn 16-row weight tiles; the 8 waves are 8/wk row waves x wk K waves,
                                  each row wave takes wn*wk/8 tiles (1, or 2 with ch = 1) */
    int wk;        /* workgroup: waves spread over K (1, 2, 4, 8), wn*wk = 8 or 16.  wave-stream, row-split: 16-row weight tiles per chunk (1 or 2;
                      row-split above 16 rows: 2).
                      K-split: bytes of K per wave / 256 (1, 2, or 4 with m_tiles <= 2) */
    int ch;        /* workgroup: 256-byte K chunks each wave streams per slab (1 or 2).
                      wave-stream, row-split: 16-byte activation loads per lane and chunk, ceil(m/4) (row-split above 16 rows:
                      6 up to 24 rows, else 8).  K-split: 0 */
    int grid;      /* persistent workgroups launched */
    int panels;    /* workgroup: ceil(n / (16*wn)) row panels.  wave-stream: ceil(n / (16*wk)) row groups.
                      K-split: ceil(n/16) row tiles.  row-split: ceil(n/4) units of 4 rows (wn = -3: ceil(n/16) tiles) */
    int slabs;     /* workgroup: k / (256*wk*ch) K slabs per panel.  wave-stream: k/256 chunks per group.
                      K-split: k / (2048*wk) windows */
    int lds_bytes; /* dynamic LDS per workgroup */
} hfrk_gemm_plan;

/* Library version, for the binding to check.  110: plan kind wn = -3 (row-split on whole 16-row tiles, both weight layouts),
 * hfrk_skinny_gemm_rms_plan; the bench-only probe entry points are no longer part of this library (100 had them). */
int hfrk_version(void);

/* Split-K workspaces.  A GEMM whose row tiles are shared between workgroups parks fp32 partial sums in a workspace
 * (64 MB + 4 MB of arrival counters) and the last workgroup to arrive adds them.  Two GEMMs that run at the same time
 * must not share a workspace, so each stream that launches a GEMM owns one, taken from a per-device pool on the
 * stream's first launch and kept from then on; launches on different streams are therefore independent of each other,
 * as the reference's are (it needs no workspace: it adds fp16 atomics into the caller's zeroed output,
 * csrc/op_src/skinny_gemm/consumers/mfma_16x16x32_consumer.cu:155-163).
 *   hfrk_init             allocates the first 4 workspaces of the current device.  Idempotent, thread-safe.  The pool
 *                         grows by itself (up to 64) when a fifth stream appears, except while that stream is being
 *                         captured into a graph (no allocation inside a capture): then the call returns
 *                         HFRK_NOT_INITIALISED, so run hfrk_init, and one launch per further stream, before capturing.
 *   hfrk_release_stream   returns the stream's workspace to the pool (before destroying a stream that has launched
 *                         GEMMs; the stream must have finished them).  HFRK_SUCCESS also when it owned none.
 *   hfrk_reset_workspace  zeroes the arrival counters of every workspace of the current device, asynchronously on
 *                         `stream`: for after a launch that did not run to its end (a device fault, a killed process
 *                         sharing the context).  No GEMM may be running on the device meanwhile.
 *   hfrk_workspace_id     index of the workspace `stream` owns on the current device, or -1 (diagnostics and tests).
 * A graph records the workspace of the stream it was captured on: replay it ordered with that stream's other GEMM work,
 * or capture on a stream of its own, as torch.cuda.graph does. */
int hfrk_init(void);
int hfrk_release_stream(void* stream);
int hfrk_reset_workspace(void* stream);
int hfrk_workspace_id(void* stream);

/* hipError_t of the last failed HIP call on this thread (0 if none). */
int hfrk_last_hip_error(void);

/* Human-readable text for a status code (static storage). */
const char* hfrk_status_string(int status);

/* Pure host function: the reference launcher's argument checks, same order, same codes
 * (csrc/op_src/skinny_gemm/skinny_gemm_caller.cu:33-72,455-457), plus this library's own shape limits.
 * Touches no device. */
int hfrk_skinny_gemm_validate(int m, int n, int k, int b_stride, int split_k, int A_producers, int B_producers,
                              int consumers, int a_lanes, int b_lanes, int qsize, int op_m, int ops);

/* Pure host function: choose the decomposition for a shape (counterpart of infer_skinny_gemm_params,
 * hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102).  Returns HFRK_SUCCESS or a shape error. */
int hfrk_skinny_gemm_plan(int m, int n, int k, hfrk_gemm_plan* plan);

/* Plan table (host only, thread-safe): tuned decompositions, keyed (m, n, k, packed), that take the planner's place
 * whenever a GEMM entry point is called without a plan (the SwiGLU epilogue keeps its own plan).  An entry also serves
 * the smaller m that run the same kernel on the same work: m' <= 16 serves m > m' - 4 rounded to fours (8 serves 5..8),
 * m' > 16 serves down to the previous multiple of 16 (32 serves 17..32); the nearest entry at or above m wins.
 * Counterpart of the reference's tuned table, hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102, filled from
 * sweeps like its benchmarks/skinny_gemm/grid_search.py.
 *   hfrk_plan_table_set    validates the plan for the shape like hfrk_skinny_gemm_ex does and stores it; plan == NULL
 *                          removes the entry.  Returns HFRK_SUCCESS or the validation status.
 *   hfrk_plan_table_get    the plan a call without one would use: the entry, or the planner's choice.
 *   hfrk_plan_table_clear  drops every entry, returns how many there were. */
int hfrk_plan_table_set(int m, int n, int k, int packed, const hfrk_gemm_plan* plan);
int hfrk_plan_table_get(int m, int n, int k, int packed, hfrk_gemm_plan* plan);
int hfrk_plan_table_clear(void);

/* Install every entry of a plan-table file through hfrk_plan_table_set (host only; `path` is a host string).  The
 * file is the JSON that this package's grid-search tool writes: {"format": "hfrk-plan-table-1", "entries": [{"m", "n",
 * "k", "packed", "plan": {"m_tiles", "wn", "wk", "ch", "grid", "panels", "slabs", "lds_bytes"}, ...}]}; other members
 * are ignored.  strict != 0: the first malformed entry (HFRK_BAD_FILE) or rejected plan (its validation status) ends the
 * load; strict == 0: such entries are skipped.  *installed (may be NULL) receives the number of entries installed.
 * Counterpart, for hosts without Python, of shipping the tuned table inside the wrapper
 * (hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102). */
int hfrk_plan_table_load(const char* path, int strict, int* installed);

/* D[m,n] += scale_tensor[0] * A[m,k] . B[k,n]
 * Replaces `int skinny_gemm(...)` at csrc/op_src/skinny_gemm/skinny_gemm_caller.cu:21-32, the function behind
 * torch.ops._HFRK_C.skinny_gemm_tb (csrc/op_src/skinny_gemm/skinny_gemm_binding.cu:16-42), same argument order.
 *   A   fp8 e4m3fn [m,k] row-major            B   fp8 e4m3fn [k,n] with unit stride along k: row n of the
 *   D   16-bit [m,n] row-major, d_dtype           weight starts at B + n*b_stride (b_stride in elements)
 *   scale_tensor  one fp32 (the product of the activation and weight scales)
 * D is accumulated into, once, in fp32 (D = round(float(D) + scale*acc)): callers pre-zero it or preload a
 * bias, as with the reference, but the result is deterministic and rounded a single time.
 * split_k and the eight knob integers are validated exactly like the reference's and are otherwise advisory:
 * the decomposition comes from hfrk_skinny_gemm_plan(). */
int hfrk_skinny_gemm(const void* A, const void* B, void* D, const float* scale_tensor, int m, int n, int k,
                     int b_stride, int split_k, int A_producers, int B_producers, int consumers, int a_lanes,
                     int b_lanes, int qsize, int op_m, int ops, int d_dtype, void* stream);

/* General form: D[i,j] = (accumulate ? D[i,j] : 0) + scale_a[i*sa_stride] * scale_b[j*sb_stride] * sum_k A[i,k] B[k,j]
 * sa_stride / sb_stride are 0 (one scalar) or 1 (per token / per output channel).  scale_b may be NULL (= 1).
 * plan may be NULL (the library plans).  No reference counterpart for the per-row/per-channel scales: the
 * reference asserts scale_tensor.numel()==1 (hf_rocm_kernels/operators/skinny_gemm/wrapped.py:18). */
int hfrk_skinny_gemm_ex(const void* A, const void* B, void* D, const float* scale_a, int sa_stride,
                        const float* scale_b, int sb_stride, int m, int n, int k, int b_stride, int d_dtype,
                        int accumulate, const hfrk_gemm_plan* plan, void* stream);

/* hfrk_skinny_gemm_ex for callers that cannot allocate and cannot let the library allocate on their behalf: code under
 * HIP graph capture that has not run hfrk_init, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference.  Same arguments and bit-identical results; the partial sums and arrival counters go to an array that is
 * part of the library's code object (16 MB + 65536 counters, 16.25 MB on every device the library runs on, held until
 * the process ends) instead of a workspace from the pool, so the call performs no hipMalloc / hipFree and nothing that
 * allocates.
 * Limits: the plan (the caller's, or the library's choice for the shape) may need at most 16 MB of partial sums
 * (1 KB per 16x16 tile a workgroup may have to hand over: 2 x grid x row tiles x activation tiles for the streaming
 * kernels) and 65536 counters (n <= 262144).  Everything the planner and the shipped plan tables choose fits (their
 * largest: 8 row waves x 4 activation tiles on 256 workgroups); explicit plans with 16 row tiles per panel at m > 32 or
 * grids above 256 may not, and return HFRK_EXCEEDS_SCRATCH before anything is launched.
 * All calls on one device share the array: calls that overlap on a device (two streams, two threads) race; order them
 * on one stream.  Each call first clears the counters its plan uses (a small kernel on `stream`), so a launch that
 * never finished leaves nothing behind. */
int hfrk_skinny_gemm_noalloc(const void* A, const void* B, void* D, const float* scale_a, int sa_stride,
                             const float* scale_b, int sb_stride, int m, int n, int k, int b_stride, int d_dtype,
                             int accumulate, const hfrk_gemm_plan* plan, void* stream);

/* The GEMM with what the decoder block does around it folded in (no reference counterpart as one call; it stands
 * for skinny_gemm followed by swiglu in hf_rocm_kernels/combined_ops/llama_mlp.py:43-56, and for the residual add
 * after the down projection).
 *   epilogue HFRK_EPILOGUE_NONE:   D[i,j] = (base ? base[i,j] : 0) + scale_a[i] * scale_b[j] * sum_k A[i,k] B[k,j]
 *       base: 16-bit [m,n] like D, may be D itself (= accumulate) or another tensor (e.g. the residual), or NULL.
 *   epilogue HFRK_EPILOGUE_SWIGLU: B is a gate_up weight, gate rows [0, n/2), up rows [n/2, n);
 *       D[i,j] = e4m3fn( silu(g) * u / out_scale[0] ),  g, u = the two projections of column j, each rounded to
 *       d_dtype first (what the unfused chain stores between its two kernels);  D is fp8 [m, n/2], 4-byte aligned.
 *       Needs n % 32 == 0, base == NULL and m <= 16; or m <= 64 with k = 2048 or 4096 (the K-split kernel, whose one
 *       window then covers k); or m <= 32 on a row-major weight whose n/2 output columns deal out over the workgroups
 *       (the row-split kernel with two activation tiles: k % 256 == 0, at least 1024 columns).  Otherwise HFRK_BAD_SHAPE
 *       (callers then run the two kernels).
 * Scales and plan as in hfrk_skinny_gemm_ex; a plan passed with the SwiGLU epilogue describes n/2 output columns
 * with wk = 2. */
int hfrk_skinny_gemm_fused(const void* A, const void* B, void* D, const void* base, const float* scale_a, int sa_stride,
                           const float* scale_b, int sb_stride, const float* out_scale, int m, int n, int k,
                           int b_stride, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream);

/* hfrk_skinny_gemm_fused with the residual RMSNorm that feeds it as the kernel's prologue: one launch for what the
 * reference's chain runs as `residual_rms` followed by `skinny_gemm` (hf_rocm_kernels/combined_ops/llama_mlp.py:23-41;
 * csrc/op_src/residual_rms/residual_rms_dispatch.cu:8-63 for the norm).
 *   residual_out <- input + residual (one 16-bit add; a buffer of its own: every workgroup reads the old residual);
 *   A = e4m3fn(rmsnorm(residual_out) * rms_weight / act_scale[0]) is built in every workgroup's LDS, bit-identical to what
 *   hfrk_residual_rms writes; then the GEMM and its epilogue as in hfrk_skinny_gemm_fused, with scale_a one float
 *   (activation scale x weight scale).  input, residual, residual_out [m,k] and rms_weight [k] are io_dtype (f16/bf16),
 *   16-byte aligned.
 * Exists in the row-split kernel: row-major weights, m <= 8, k = 4096 or 8192, a shape whose rows deal out evenly over the
 * workgroups (HFRK_BAD_SHAPE otherwise: callers then run the two launches); an explicit plan must be a row-split plan with
 * wk = 1 (2 with the SwiGLU epilogue). */
int hfrk_skinny_gemm_rms_fused(const void* input, const void* residual, void* residual_out, const void* rms_weight,
                               float epsilon, const float* act_scale, int io_dtype, const void* B, void* D, const void* base,
                               const float* scale_a, const float* scale_b, int sb_stride, const float* out_scale, int m, int n,
                               int k, int b_stride, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream);

/* Whether hfrk_skinny_gemm_rms_fused has a prologue for a row-major weight of n rows (gate and up rows together with the
 * SwiGLU epilogue) and, if so, the plan it launches with when none is passed: HFRK_SUCCESS and *plan, or HFRK_BAD_SHAPE.
 * Host only.  Same decision as the entry point's (one function behind both); the plan table is not consulted. */
int hfrk_skinny_gemm_rms_plan(int m, int n, int k, int epilogue, hfrk_gemm_plan* plan);

/* Weight load format (no reference counterpart: the reference streams row-major weights through an LDS ring,
 * csrc/op_src/skinny_gemm/producers/n_full_tiles.cu:4-127, and stores fn bits viewed as fnuz,
 * hf_rocm_kernels/utils/fp8.py:27-29).  A weight packed once when the model is loaded is read by the GEMM as one
 * contiguous run per wave, already in matrix-core operand order.
 *   packed layout: 16-row x 256-byte chunks, rows padded with zeros to a multiple of 16; chunk (tile, kc) at
 *   (tile * k/256 + kc) * 4096; inside a chunk, 16-byte piece j (0..3) of lane l (0..63) at j*1024 + l*16 holds
 *   row l%16, bytes (j/2)*128 + (l/16)*32 + (j%2)*16 .. +16.
 * hfrk_packed_weight_bytes: size of the packed buffer (0 if k % 256 != 0 or a size is not positive).  Host only.
 * hfrk_pack_weight: src [n,k] fp8 row-major with row stride src_stride -> dst packed.  src_format
 *   HFRK_WEIGHT_E4M3FNUZ re-encodes on the way (see hfrk_reencode_fnuz).  src and dst must not overlap.
 * hfrk_unpack_weight: the inverse (padding rows dropped); pack then unpack returns the source bytes.
 * hfrk_reencode_fnuz: count bytes of e4m3fnuz -> e4m3fn with the same values (dst may be src).  Exact for every
 *   code except magnitudes below 2^-6, which land on fn's subnormal grid of 2^-9 (round to nearest even); the
 *   fnuz NaN 0x80 becomes the fn NaN 0x7f.  Scales stay as they are.
 * A layer's per-output-channel scales can live in the same allocation, behind the packed bytes:
 * hfrk_packed_weight_bytes_scaled: hfrk_packed_weight_bytes + 4 bytes per padded row (16 * ceil(n/16) float32).
 * hfrk_pack_weight_scaled: hfrk_pack_weight, then scales[0..n) copied behind the bytes (zeros for the padding rows).
 * hfrk_packed_weight_scales: where they are, packed + hfrk_packed_weight_bytes(n, k) (NULL if that is 0).  Host only.
 *   The unscaled functions work on the front part of such a buffer unchanged. */
size_t hfrk_packed_weight_bytes(int n, int k);
int hfrk_pack_weight(const void* src, int src_stride, int src_format, void* dst, int n, int k, void* stream);
int hfrk_unpack_weight(const void* src, void* dst, int dst_stride, int n, int k, void* stream);
int hfrk_reencode_fnuz(const void* src, void* dst, size_t count, void* stream);
size_t hfrk_packed_weight_bytes_scaled(int n, int k);
int hfrk_pack_weight_scaled(const void* src, int src_stride, int src_format, const float* scales, void* dst, int n, int k,
                            void* stream);
const float* hfrk_packed_weight_scales(const void* packed, int n, int k);

/* hfrk_skinny_gemm_fused on a packed weight: same results bit for bit (same operands, same order of sums), B is
 * the buffer hfrk_pack_weight wrote for this n and k.  With the SwiGLU epilogue n % 32 == 0 as before.
 * sb_stride HFRK_SCALES_IN_PACKED_BUFFER: B is a buffer of hfrk_pack_weight_scaled and its per-channel scales are
 * used; scale_b is ignored. */
#define HFRK_SCALES_IN_PACKED_BUFFER (-1)
int hfrk_skinny_gemm_packed(const void* A, const void* B_packed, void* D, const void* base, const float* scale_a,
                            int sa_stride, const float* scale_b, int sb_stride, const float* out_scale, int m, int n,
                            int k, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream);

/* residual <- input + residual (one 16-bit add); output <- rmsnorm(residual) * weight, optionally / scale -> fp8.
 * Replaces `void residual_rms(...)` at csrc/op_src/residual_rms/residual_rms_dispatch.cu:8-63.
 *   input, residual [rows,cols] io_dtype (f16/bf16) row-major; weight [cols] io_dtype
 *   scale_tensor: one fp32, used (and required) only when out_dtype is fp8
 *   output [rows,cols] out_dtype: HFRK_FP8_E4M3FN, or io_dtype
 *   next_buffer: rows*buffer_cols 16-bit elements set to zero (may be NULL when buffer_cols==0)
 *   num_threads: 0 = choose; else threads per row (multiple of 64, <= 1024).  force_scalar: use the
 *   one-element-per-thread kernel even when the 16-byte path applies. */
int hfrk_residual_rms(const void* input, void* residual, const void* weight, const float* scale_tensor,
                      float epsilon, void* output, void* next_buffer, int rows, int cols, int buffer_cols,
                      int io_dtype, int out_dtype, int num_threads, int force_scalar, void* stream);

/* output[r,c] = fp8( silu(gate_up[r,c]) * gate_up[r,cols+c] / scale ), gate_up [rows, 2*cols] io_dtype.
 * Replaces `void swiglu(...)` at csrc/op_src/swiglu/swiglu_dispatch.cu:8-42.  next_buffer as above. */
int hfrk_swiglu(const void* gate_up, const float* scale_tensor, void* output, void* next_buffer, int rows,
                int cols, int buffer_cols, int io_dtype, int num_threads, int force_scalar, void* stream);

/* Per-token dynamic quantisation (no reference counterpart: the reference's kernels take one static scale_tensor,
 * hf_rocm_kernels/operators/residual_rms/wrapped.py:94-95, operators/swiglu/wrapped.py:49-84).
 *   residual <- input + residual;  y = rmsnorm(residual) * weight       (hfrk_residual_rms_dynamic)
 *   y = silu(gate_up[:, :cols]) * gate_up[:, cols:]                     (hfrk_swiglu_dynamic)
 *   scales[r] = max(amax_c |y[r,c]| / 448, FLT_MIN);  output[r,c] = e4m3fn(y[r,c] / scales[r])
 * scales: rows fp32 values, ready to be the GEMM's per-token scale_a.  Rows must be 16-byte aligned (cols % 8 == 0)
 * and cols <= 32768, else HFRK_BAD_SHAPE / HFRK_BAD_ALIGNMENT.  next_buffer as in hfrk_residual_rms. */
int hfrk_residual_rms_dynamic(const void* input, void* residual, const void* weight, float epsilon, void* output,
                              float* scales, void* next_buffer, int rows, int cols, int buffer_cols, int io_dtype,
                              void* stream);
int hfrk_swiglu_dynamic(const void* gate_up, void* output, float* scales, void* next_buffer, int rows, int cols,
                        int buffer_cols, int io_dtype, void* stream);

/* FP8 quantisation of a 16-bit activation block [rows, cols] (the device form of fp8_quantize,
 * hf_rocm_kernels/utils/fp8.py:6-29, which the reference runs as torch ops on the caller's side; here also per token).
 *   static_scale != NULL:  output = e4m3fn(clamp(input / static_scale[0], +-448)); scales is not touched (may be NULL)
 *   static_scale == NULL:  scales[r] = max(amax_c |input[r,c]| / 448, FLT_MIN); output[r,c] = e4m3fn(input[r,c] / scales[r])
 * Same limits as the dynamic kernels above: cols % 8 == 0, cols <= 32768, 16-byte aligned input, 8-byte aligned output. */
int hfrk_quantize_fp8(const void* input, const float* static_scale, void* output, float* scales, int rows, int cols,
                      int io_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HFRK_GFX950_H */
