// torch.ops._HFRK_C.* -- the operator surface of the reference (csrc/torch_bindings.cpp:20-44, csrc/ops.h:8-19),
// same schemas, implemented by forwarding plain pointers to the C ABI of libhfrk_gfx950.so.
// No kernel lives here: this file only unpacks tensors, checks them, selects device and stream.
#include <Python.h>

#include <ATen/ATen.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include "hfrk_gfx950.h"

namespace {

// Make the tensor's device current for the duration of a call (the launchers use the current device).
struct DeviceScope {
    c10::DeviceIndex prev;
    bool changed;
    explicit DeviceScope(const at::Tensor& t) : prev(c10::hip::current_device()), changed(false) {
        const c10::DeviceIndex want = t.device().index();
        if (want >= 0 && want != prev) {
            c10::hip::set_device(want);
            changed = true;
        }
    }
    ~DeviceScope() {
        if (changed) c10::hip::set_device(prev);
    }
};

void* current_stream(const at::Tensor& t) {
    return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

int dtype16(const at::Tensor& t, const char* name) {
    if (t.scalar_type() == at::kBFloat16) return HFRK_BF16;
    if (t.scalar_type() == at::kHalf) return HFRK_F16;
    TORCH_CHECK(false, name, " must be float16 or bfloat16, got ", t.scalar_type());
}

void check_fp8(const at::Tensor& t, const char* name) {
    TORCH_CHECK(t.scalar_type() != at::kFloat8_e4m3fnuz, name,
                " is float8_e4m3fnuz: gfx950 computes in OCP float8_e4m3fn (same bits read as twice the fnuz value); "
                "re-encode the tensor or pass a float8_e4m3fn view and double its scale");
    TORCH_CHECK(t.scalar_type() == at::kFloat8_e4m3fn, name, " must be float8_e4m3fn, got ", t.scalar_type());
}

void check_same_device(const at::Tensor& ref, const at::Tensor& t, const char* name) {
    TORCH_CHECK(t.device() == ref.device(), name, " is on ", t.device(), " but expected ", ref.device());
}

void raise_on(int status, const char* op) {
    TORCH_CHECK(status == HFRK_SUCCESS, op, " failed: ", hfrk_status_string(status), " (status ", status,
                ", hip error ", hfrk_last_hip_error(), ")");
}

// reference: csrc/op_src/increment/increment_op.cu:3
void increment(at::Tensor& x) { x += 1; }

// reference: csrc/op_src/residual_rms/residual_rms_dispatch.cu:8-63
void residual_rms(at::Tensor& input, at::Tensor& residual, at::Tensor& weight, at::Tensor& scale_tensor, double epsilon,
                  at::Tensor& output, at::Tensor& next_buffer, int64_t num_threads, bool force_scalar) {
    TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous [rows, cols] tensor");
    TORCH_CHECK(residual.sizes() == input.sizes() && residual.is_contiguous(), "residual must match input and be contiguous");
    TORCH_CHECK(weight.dim() == 1 && weight.size(0) == input.size(1) && weight.is_contiguous(), "weight must be [cols]");
    TORCH_CHECK(output.sizes() == input.sizes() && output.is_contiguous(), "output must match input and be contiguous");
    const int io = dtype16(input, "input");
    TORCH_CHECK(residual.scalar_type() == input.scalar_type() && weight.scalar_type() == input.scalar_type(),
                "input, residual and weight must share one 16-bit dtype");
    int out = io;
    if (output.scalar_type() != input.scalar_type()) {
        check_fp8(output, "output");
        out = HFRK_FP8_E4M3FN;
        TORCH_CHECK(scale_tensor.numel() == 1 && scale_tensor.scalar_type() == at::kFloat, "fp8 output needs a one-element float32 scale_tensor");
        check_same_device(input, scale_tensor, "scale_tensor");
    }
    check_same_device(input, residual, "residual");
    check_same_device(input, weight, "weight");
    check_same_device(input, output, "output");
    int64_t buffer_cols = 0;
    void* nb = nullptr;
    if (next_buffer.numel() > 0) {
        TORCH_CHECK(next_buffer.dim() == 2 && next_buffer.size(0) == input.size(0) && next_buffer.is_contiguous(),
                    "next_buffer must be a contiguous [rows, buffer_cols] tensor");
        TORCH_CHECK(next_buffer.element_size() == 2, "next_buffer must hold 16-bit elements");
        check_same_device(input, next_buffer, "next_buffer");
        buffer_cols = next_buffer.size(1);
        nb = next_buffer.data_ptr();
    }
    DeviceScope scope(input);
    raise_on(hfrk_residual_rms(input.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                               out == HFRK_FP8_E4M3FN ? scale_tensor.data_ptr<float>() : nullptr, (float)epsilon,
                               output.data_ptr(), nb, (int)input.size(0), (int)input.size(1), (int)buffer_cols, io, out,
                               (int)num_threads, force_scalar ? 1 : 0, current_stream(input)),
             "residual_rms");
}

// reference: csrc/op_src/swiglu/swiglu_dispatch.cu:8-42
void swiglu(at::Tensor& gate_up, at::Tensor& scale_tensor, at::Tensor& output, at::Tensor& next_buffer, int64_t num_threads,
            bool force_scalar) {
    TORCH_CHECK(gate_up.dim() == 2 && gate_up.is_contiguous() && gate_up.size(1) % 2 == 0,
                "gate_up must be a contiguous [rows, 2*cols] tensor");
    const int io = dtype16(gate_up, "gate_up");
    const int64_t rows = gate_up.size(0), cols = gate_up.size(1) / 2;
    check_fp8(output, "output");
    TORCH_CHECK(output.dim() == 2 && output.size(0) == rows && output.size(1) == cols && output.is_contiguous(),
                "output must be a contiguous [rows, cols] tensor");
    TORCH_CHECK(scale_tensor.numel() == 1 && scale_tensor.scalar_type() == at::kFloat, "scale_tensor must be one float32");
    check_same_device(gate_up, scale_tensor, "scale_tensor");
    check_same_device(gate_up, output, "output");
    int64_t buffer_cols = 0;
    void* nb = nullptr;
    if (next_buffer.numel() > 0) {
        TORCH_CHECK(next_buffer.dim() == 2 && next_buffer.size(0) == rows && next_buffer.is_contiguous(),
                    "next_buffer must be a contiguous [rows, buffer_cols] tensor");
        TORCH_CHECK(next_buffer.element_size() == 2, "next_buffer must hold 16-bit elements");
        check_same_device(gate_up, next_buffer, "next_buffer");
        buffer_cols = next_buffer.size(1);
        nb = next_buffer.data_ptr();
    }
    DeviceScope scope(gate_up);
    raise_on(hfrk_swiglu(gate_up.data_ptr(), scale_tensor.data_ptr<float>(), output.data_ptr(), nb, (int)rows, (int)cols,
                         (int)buffer_cols, io, (int)(num_threads < 0 ? 0 : num_threads), force_scalar ? 1 : 0,
                         current_stream(gate_up)),
             "swiglu");
}

void check_gemm_operands(const at::Tensor& A, const at::Tensor& B, const at::Tensor& D) {
    TORCH_CHECK(A.dim() == 2 && A.is_contiguous(), "A must be a contiguous [m, k] tensor");
    TORCH_CHECK(B.dim() == 2 && B.size(0) == A.size(1) && B.stride(0) == 1, "B must be [k, n] with unit stride along k");
    TORCH_CHECK(D.dim() == 2 && D.size(0) == A.size(0) && D.size(1) == B.size(1) && D.is_contiguous(),
                "D must be a contiguous [m, n] tensor");
    check_fp8(A, "A");
    check_fp8(B, "B");
    check_same_device(A, B, "B");
    check_same_device(A, D, "D");
}

// reference: csrc/op_src/skinny_gemm/skinny_gemm_binding.cu:16-42.  Returns the status code like the reference;
// misuse of dtypes/devices raises instead of reading garbage.
int64_t skinny_gemm_tb(at::Tensor& A, at::Tensor& B, at::Tensor& D, at::Tensor& scale_tensor, int64_t split_k,
                       int64_t A_producers, int64_t B_producers, int64_t consumers, int64_t a_lanes, int64_t b_lanes,
                       int64_t qsize, int64_t op_m, int64_t ops) {
    check_gemm_operands(A, B, D);
    TORCH_CHECK(scale_tensor.numel() == 1 && scale_tensor.scalar_type() == at::kFloat, "scale_tensor must be one float32");
    check_same_device(A, scale_tensor, "scale_tensor");
    const int d_dtype = dtype16(D, "D");
    DeviceScope scope(A);  // before the stream is looked up
    return hfrk_skinny_gemm(A.data_ptr(), B.data_ptr(), D.data_ptr(), scale_tensor.data_ptr<float>(), (int)A.size(0),
                            (int)B.size(1), (int)A.size(1), (int)B.stride(1), (int)split_k, (int)A_producers,
                            (int)B_producers, (int)consumers, (int)a_lanes, (int)b_lanes, (int)qsize, (int)op_m, (int)ops,
                            d_dtype, current_stream(A));
}

// Per-token (scale_a: 1 or m values) x per-output-channel (scale_b: 1 or n values) scaling.  No reference counterpart.
int64_t skinny_gemm_scaled(at::Tensor& A, at::Tensor& B, at::Tensor& D, at::Tensor& scale_a, at::Tensor& scale_b,
                           bool accumulate) {
    check_gemm_operands(A, B, D);
    const int64_t m = A.size(0), n = B.size(1);
    TORCH_CHECK(scale_a.scalar_type() == at::kFloat && scale_a.is_contiguous() && (scale_a.numel() == 1 || scale_a.numel() == m),
                "scale_a must be float32 with 1 or m elements");
    TORCH_CHECK(scale_b.scalar_type() == at::kFloat && scale_b.is_contiguous() && (scale_b.numel() == 1 || scale_b.numel() == n),
                "scale_b must be float32 with 1 or n elements");
    check_same_device(A, scale_a, "scale_a");
    check_same_device(A, scale_b, "scale_b");
    const int d_dtype = dtype16(D, "D");
    DeviceScope scope(A);
    return hfrk_skinny_gemm_ex(A.data_ptr(), B.data_ptr(), D.data_ptr(), scale_a.data_ptr<float>(),
                               scale_a.numel() == 1 ? 0 : 1, scale_b.data_ptr<float>(), scale_b.numel() == 1 ? 0 : 1, (int)m,
                               (int)n, (int)A.size(1), (int)B.stride(1), d_dtype, accumulate ? 1 : 0, nullptr,
                               current_stream(A));
}

static void next_buffer_args(const at::Tensor& like, const at::Tensor& next_buffer, int64_t rows, void** nb, int64_t* buffer_cols) {
    *nb = nullptr;
    *buffer_cols = 0;
    if (next_buffer.numel() > 0) {
        TORCH_CHECK(next_buffer.dim() == 2 && next_buffer.size(0) == rows && next_buffer.is_contiguous(),
                    "next_buffer must be a contiguous [rows, buffer_cols] tensor");
        TORCH_CHECK(next_buffer.element_size() == 2, "next_buffer must hold 16-bit elements");
        check_same_device(like, next_buffer, "next_buffer");
        *buffer_cols = next_buffer.size(1);
        *nb = next_buffer.data_ptr();
    }
}

// residual RMSNorm with per-row dynamic fp8 quantisation: output fp8 [rows, cols], scales fp32 [rows].  No reference counterpart.
void residual_rms_dynamic(at::Tensor& input, at::Tensor& residual, at::Tensor& weight, double epsilon, at::Tensor& output,
                          at::Tensor& scales, at::Tensor& next_buffer) {
    TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous [rows, cols] tensor");
    TORCH_CHECK(residual.sizes() == input.sizes() && residual.is_contiguous(), "residual must match input and be contiguous");
    TORCH_CHECK(weight.dim() == 1 && weight.size(0) == input.size(1) && weight.is_contiguous(), "weight must be [cols]");
    TORCH_CHECK(output.sizes() == input.sizes() && output.is_contiguous(), "output must match input and be contiguous");
    const int io = dtype16(input, "input");
    TORCH_CHECK(residual.scalar_type() == input.scalar_type() && weight.scalar_type() == input.scalar_type(),
                "input, residual and weight must share one 16-bit dtype");
    check_fp8(output, "output");
    TORCH_CHECK(scales.scalar_type() == at::kFloat && scales.is_contiguous() && scales.numel() == input.size(0),
                "scales must be a contiguous float32 tensor with one element per row");
    check_same_device(input, residual, "residual");
    check_same_device(input, weight, "weight");
    check_same_device(input, output, "output");
    check_same_device(input, scales, "scales");
    void* nb;
    int64_t buffer_cols;
    next_buffer_args(input, next_buffer, input.size(0), &nb, &buffer_cols);
    DeviceScope scope(input);
    raise_on(hfrk_residual_rms_dynamic(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), (float)epsilon, output.data_ptr(),
                                       scales.data_ptr<float>(), nb, (int)input.size(0), (int)input.size(1), (int)buffer_cols, io,
                                       current_stream(input)),
             "residual_rms_dynamic");
}

// SwiGLU with per-row dynamic fp8 quantisation.  No reference counterpart.
void swiglu_dynamic(at::Tensor& gate_up, at::Tensor& output, at::Tensor& scales, at::Tensor& next_buffer) {
    TORCH_CHECK(gate_up.dim() == 2 && gate_up.is_contiguous() && gate_up.size(1) % 2 == 0,
                "gate_up must be a contiguous [rows, 2*cols] tensor");
    const int io = dtype16(gate_up, "gate_up");
    const int64_t rows = gate_up.size(0), cols = gate_up.size(1) / 2;
    check_fp8(output, "output");
    TORCH_CHECK(output.dim() == 2 && output.size(0) == rows && output.size(1) == cols && output.is_contiguous(),
                "output must be a contiguous [rows, cols] tensor");
    TORCH_CHECK(scales.scalar_type() == at::kFloat && scales.is_contiguous() && scales.numel() == rows,
                "scales must be a contiguous float32 tensor with one element per row");
    check_same_device(gate_up, output, "output");
    check_same_device(gate_up, scales, "scales");
    void* nb;
    int64_t buffer_cols;
    next_buffer_args(gate_up, next_buffer, rows, &nb, &buffer_cols);
    DeviceScope scope(gate_up);
    raise_on(hfrk_swiglu_dynamic(gate_up.data_ptr(), output.data_ptr(), scales.data_ptr<float>(), nb, (int)rows, (int)cols,
                                 (int)buffer_cols, io, current_stream(gate_up)),
             "swiglu_dynamic");
}

// 16-bit [rows, cols] -> float8_e4m3fn: with one static scale (the reference's fp8_quantize, hf_rocm_kernels/utils/fp8.py:6-29,
// as one kernel) or, scale_tensor None, one dynamic scale per row written to `scales`.
void quantize_fp8(at::Tensor& input, const std::optional<at::Tensor>& scale_tensor, at::Tensor& output, at::Tensor& scales) {
    TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous [rows, cols] tensor");
    const int io = dtype16(input, "input");
    check_fp8(output, "output");
    TORCH_CHECK(output.sizes() == input.sizes() && output.is_contiguous(), "output must match input and be contiguous");
    check_same_device(input, output, "output");
    const float* static_scale = nullptr;
    float* scales_ptr = nullptr;
    if (scale_tensor.has_value()) {
        TORCH_CHECK(scale_tensor->numel() == 1 && scale_tensor->scalar_type() == at::kFloat, "scale_tensor must be one float32");
        check_same_device(input, *scale_tensor, "scale_tensor");
        static_scale = scale_tensor->data_ptr<float>();
    } else {
        TORCH_CHECK(scales.scalar_type() == at::kFloat && scales.is_contiguous() && scales.numel() == input.size(0),
                    "scales must be a contiguous float32 tensor with one element per row");
        check_same_device(input, scales, "scales");
        scales_ptr = scales.data_ptr<float>();
    }
    DeviceScope scope(input);
    raise_on(hfrk_quantize_fp8(input.data_ptr(), static_scale, output.data_ptr(), scales_ptr, (int)input.size(0), (int)input.size(1), io,
                               current_stream(input)),
             "quantize_fp8");
}

// The GEMM with the surrounding element-wise work folded in.  No reference counterpart as one op.
//   epilogue 0: D = (base ? base : 0) + scale_a x scale_b x A.B, base a 16-bit [m,n] tensor (D itself, a residual) or None
//   epilogue 1: B is a gate_up weight [k, 2*inter]; D fp8 [m, inter] = e4m3fn(silu(gate) * up / out_scale), the two
//               projections rounded to `intermediate_dtype` (0 = float16, 1 = bfloat16) first
// Shared by skinny_gemm_fused (B = the [k, n] view of a row-major weight) and skinny_gemm_packed (B = the buffer
// pack_weight wrote, n given by the caller).
int64_t gemm_fused_common(at::Tensor& A, at::Tensor& B, bool packed, int64_t n, at::Tensor& D,
                          const std::optional<at::Tensor>& base, at::Tensor& scale_a,
                          const std::optional<at::Tensor>& scale_b, const std::optional<at::Tensor>& out_scale,
                          int64_t epilogue, int64_t intermediate_dtype) {
    TORCH_CHECK(A.dim() == 2 && A.is_contiguous(), "A must be a contiguous [m, k] tensor");
    check_fp8(A, "A");
    check_fp8(B, "B");
    if (packed) {
        TORCH_CHECK(n >= 1 && n < (int64_t(1) << 30) && A.size(1) < (int64_t(1) << 30), "n and k must fit 30 bits");
        const size_t plain = hfrk_packed_weight_bytes((int)n, (int)A.size(1)), scaled = hfrk_packed_weight_bytes_scaled((int)n, (int)A.size(1));
        TORCH_CHECK(B.is_contiguous() && B.numel() > 0 && ((size_t)B.numel() == plain || (size_t)B.numel() == scaled),
                    "B must be the packed buffer of a [n, k] weight (pack_weight, pack_weight_scaled) with k = A.size(1)");
    } else {
        TORCH_CHECK(B.dim() == 2 && B.size(0) == A.size(1) && B.stride(0) == 1, "B must be [k, n] with unit stride along k");
    }
    check_same_device(A, B, "B");
    check_same_device(A, D, "D");
    const int64_t m = A.size(0);
    TORCH_CHECK(scale_a.scalar_type() == at::kFloat && scale_a.is_contiguous() && (scale_a.numel() == 1 || scale_a.numel() == m),
                "scale_a must be float32 with 1 or m elements");
    check_same_device(A, scale_a, "scale_a");
    // None = 1, in either weight layout: the scales a pack_weight_scaled buffer carries apply only when the caller passes
    // them (PackedWeight.scales is a view of that part of the buffer), so one call means one thing whatever the layout.
    const float* scale_b_ptr = nullptr;
    int sb_stride = 0;
    if (scale_b.has_value()) {
        TORCH_CHECK(scale_b->scalar_type() == at::kFloat && scale_b->is_contiguous() && (scale_b->numel() == 1 || scale_b->numel() == n),
                    "scale_b must be float32 with 1 or n elements");
        check_same_device(A, *scale_b, "scale_b");
        scale_b_ptr = scale_b->data_ptr<float>();
        sb_stride = scale_b->numel() == 1 ? 0 : 1;
    }
    int d_dtype;
    const void* base_ptr = nullptr;
    const float* out_scale_ptr = nullptr;
    if (epilogue == HFRK_EPILOGUE_SWIGLU) {
        TORCH_CHECK(n % 2 == 0 && D.dim() == 2 && D.size(0) == m && D.size(1) == n / 2 && D.is_contiguous(),
                    "D must be a contiguous [m, n/2] tensor");
        check_fp8(D, "D");
        TORCH_CHECK(out_scale.has_value() && out_scale->numel() == 1 && out_scale->scalar_type() == at::kFloat,
                    "out_scale must be one float32");
        check_same_device(A, *out_scale, "out_scale");
        TORCH_CHECK(!base.has_value(), "base cannot be combined with the SwiGLU epilogue");
        TORCH_CHECK(intermediate_dtype == HFRK_F16 || intermediate_dtype == HFRK_BF16, "intermediate_dtype must be 0 (float16) or 1 (bfloat16)");
        d_dtype = (int)intermediate_dtype;
        out_scale_ptr = out_scale->data_ptr<float>();
    } else {
        TORCH_CHECK(D.dim() == 2 && D.size(0) == m && D.size(1) == n && D.is_contiguous(), "D must be a contiguous [m, n] tensor");
        d_dtype = dtype16(D, "D");
        if (base.has_value()) {
            TORCH_CHECK(base->sizes() == D.sizes() && base->is_contiguous() && base->scalar_type() == D.scalar_type(),
                        "base must be a contiguous tensor with D's shape and dtype");
            check_same_device(A, *base, "base");
            base_ptr = base->data_ptr();
        }
    }
    DeviceScope scope(A);
    if (packed)
        return hfrk_skinny_gemm_packed(A.data_ptr(), B.data_ptr(), D.data_ptr(), base_ptr, scale_a.data_ptr<float>(),
                                       scale_a.numel() == 1 ? 0 : 1, scale_b_ptr, sb_stride, out_scale_ptr, (int)m, (int)n,
                                       (int)A.size(1), d_dtype, (int)epilogue, nullptr, current_stream(A));
    return hfrk_skinny_gemm_fused(A.data_ptr(), B.data_ptr(), D.data_ptr(), base_ptr, scale_a.data_ptr<float>(),
                                  scale_a.numel() == 1 ? 0 : 1, scale_b_ptr, sb_stride, out_scale_ptr, (int)m, (int)n, (int)A.size(1), (int)B.stride(1), d_dtype, (int)epilogue,
                                  nullptr, current_stream(A));
}

int64_t skinny_gemm_fused(at::Tensor& A, at::Tensor& B, at::Tensor& D, const std::optional<at::Tensor>& base,
                          at::Tensor& scale_a, const std::optional<at::Tensor>& scale_b, const std::optional<at::Tensor>& out_scale,
                          int64_t epilogue, int64_t intermediate_dtype) {
    TORCH_CHECK(B.dim() == 2, "B must be [k, n] with unit stride along k");
    return gemm_fused_common(A, B, false, B.size(1), D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype);
}

// skinny_gemm_fused with the residual RMSNorm of its activations as the kernel's prologue (no reference counterpart as one
// op: the reference launches residual_rms, then skinny_gemm).  residual_out <- input + residual; the GEMM multiplies
// e4m3fn(rmsnorm(residual_out) * rms_weight / act_scale) by B.  Returns the launcher's status: 7 (HFRK_BAD_SHAPE) where the
// prologue does not exist (more than 8 rows, k other than 4096 / 8192, rows that do not deal out evenly).
int64_t skinny_gemm_rms_fused(at::Tensor& input, at::Tensor& residual, at::Tensor& residual_out, at::Tensor& rms_weight,
                              double epsilon, at::Tensor& act_scale, at::Tensor& B, at::Tensor& D,
                              const std::optional<at::Tensor>& base, at::Tensor& scale_a, const std::optional<at::Tensor>& scale_b,
                              const std::optional<at::Tensor>& out_scale, int64_t epilogue, int64_t intermediate_dtype) {
    TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous [m, k] tensor");
    const int io = dtype16(input, "input");
    const int64_t m = input.size(0), k = input.size(1);
    TORCH_CHECK(residual.sizes() == input.sizes() && residual.is_contiguous() && residual.scalar_type() == input.scalar_type(),
                "residual must be a contiguous tensor with input's shape and dtype");
    TORCH_CHECK(residual_out.sizes() == input.sizes() && residual_out.is_contiguous() && residual_out.scalar_type() == input.scalar_type(),
                "residual_out must be a contiguous tensor with input's shape and dtype");
    TORCH_CHECK(rms_weight.dim() == 1 && rms_weight.size(0) == k && rms_weight.is_contiguous() && rms_weight.scalar_type() == input.scalar_type(),
                "rms_weight must be a contiguous [k] tensor of input's dtype");
    TORCH_CHECK(act_scale.numel() == 1 && act_scale.scalar_type() == at::kFloat, "act_scale must be one float32");
    TORCH_CHECK(scale_a.numel() == 1 && scale_a.scalar_type() == at::kFloat, "scale_a must be one float32");
    check_fp8(B, "B");
    TORCH_CHECK(B.dim() == 2 && B.size(0) == k && B.stride(0) == 1, "B must be [k, n] with unit stride along k");
    const int64_t n = B.size(1);
    for (const at::Tensor* t : {&residual, &residual_out, &rms_weight, &act_scale, &B, &D, &scale_a}) check_same_device(input, *t, "every tensor");
    const float* scale_b_ptr = nullptr;
    int sb_stride = 0;
    if (scale_b.has_value()) {
        TORCH_CHECK(scale_b->scalar_type() == at::kFloat && scale_b->is_contiguous() && (scale_b->numel() == 1 || scale_b->numel() == n),
                    "scale_b must be float32 with 1 or n elements");
        check_same_device(input, *scale_b, "scale_b");
        scale_b_ptr = scale_b->data_ptr<float>();
        sb_stride = scale_b->numel() == 1 ? 0 : 1;
    }
    int d_dtype;
    const void* base_ptr = nullptr;
    const float* out_scale_ptr = nullptr;
    if (epilogue == HFRK_EPILOGUE_SWIGLU) {
        TORCH_CHECK(n % 2 == 0 && D.dim() == 2 && D.size(0) == m && D.size(1) == n / 2 && D.is_contiguous(), "D must be a contiguous [m, n/2] tensor");
        check_fp8(D, "D");
        TORCH_CHECK(out_scale.has_value() && out_scale->numel() == 1 && out_scale->scalar_type() == at::kFloat, "out_scale must be one float32");
        check_same_device(input, *out_scale, "out_scale");
        TORCH_CHECK(!base.has_value(), "base cannot be combined with the SwiGLU epilogue");
        TORCH_CHECK(intermediate_dtype == HFRK_F16 || intermediate_dtype == HFRK_BF16, "intermediate_dtype must be 0 (float16) or 1 (bfloat16)");
        d_dtype = (int)intermediate_dtype;
        out_scale_ptr = out_scale->data_ptr<float>();
    } else {
        TORCH_CHECK(D.dim() == 2 && D.size(0) == m && D.size(1) == n && D.is_contiguous(), "D must be a contiguous [m, n] tensor");
        d_dtype = dtype16(D, "D");
        if (base.has_value()) {
            TORCH_CHECK(base->sizes() == D.sizes() && base->is_contiguous() && base->scalar_type() == D.scalar_type(),
                        "base must be a contiguous tensor with D's shape and dtype");
            check_same_device(input, *base, "base");
            base_ptr = base->data_ptr();
        }
    }
    DeviceScope scope(input);
    return hfrk_skinny_gemm_rms_fused(input.data_ptr(), residual.data_ptr(), residual_out.data_ptr(), rms_weight.data_ptr(), (float)epsilon,
                                      act_scale.data_ptr<float>(), io, B.data_ptr(), D.data_ptr(), base_ptr, scale_a.data_ptr<float>(),
                                      scale_b_ptr, sb_stride, out_scale_ptr, (int)m, (int)n, (int)k, (int)B.stride(1), d_dtype,
                                      (int)epilogue, nullptr, current_stream(input));
}

// The same on a weight in the load format of hfrk_pack_weight (no reference counterpart).
int64_t skinny_gemm_packed(at::Tensor& A, at::Tensor& B_packed, int64_t n, at::Tensor& D, const std::optional<at::Tensor>& base,
                           at::Tensor& scale_a, const std::optional<at::Tensor>& scale_b, const std::optional<at::Tensor>& out_scale,
                           int64_t epilogue, int64_t intermediate_dtype) {
    return gemm_fused_common(A, B_packed, true, n, D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype);
}

bool is_byte_tensor(const at::Tensor& t) {
    return t.scalar_type() == at::kByte || t.scalar_type() == at::kFloat8_e4m3fn || t.scalar_type() == at::kFloat8_e4m3fnuz;
}

// The fused GEMM for tracers: same call as skinny_gemm_fused / skinny_gemm_packed, but a status other than 0 raises
// instead of being returned.  An operator that returns an integer cannot be part of a traced graph; one that returns
// nothing can.
void skinny_gemm_checked(at::Tensor& A, at::Tensor& B, bool packed, int64_t n, at::Tensor& D, const std::optional<at::Tensor>& base,
                         at::Tensor& scale_a, const std::optional<at::Tensor>& scale_b, const std::optional<at::Tensor>& out_scale,
                         int64_t epilogue, int64_t intermediate_dtype) {
    TORCH_CHECK(packed || B.dim() == 2, "B must be [k, n] with unit stride along k");
    raise_on((int)gemm_fused_common(A, B, packed, packed ? n : B.size(1), D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype),
             "skinny_gemm_checked");
}

// Row-major [n, k] fp8 weight -> packed load format; src_format 1 re-encodes e4m3fnuz values as e4m3fn on the way.
void pack_weight(at::Tensor& src, at::Tensor& dst, int64_t src_format) {
    TORCH_CHECK(src.dim() == 2 && src.stride(1) == 1 && is_byte_tensor(src), "src must be a [n, k] one-byte tensor with unit stride along k");
    TORCH_CHECK(src.size(0) < (int64_t(1) << 30) && src.size(1) < (int64_t(1) << 30), "n and k must fit 30 bits");
    const int n = (int)src.size(0), k = (int)src.size(1);
    TORCH_CHECK(is_byte_tensor(dst) && dst.is_contiguous() && (size_t)dst.numel() == hfrk_packed_weight_bytes(n, k) && dst.numel() > 0,
                "dst must be a contiguous one-byte tensor of hfrk_packed_weight_bytes(n, k) elements (k % 256 == 0)");
    check_same_device(src, dst, "dst");
    DeviceScope scope(src);
    raise_on(hfrk_pack_weight(src.data_ptr(), (int)src.stride(0), (int)src_format, dst.data_ptr(), n, k, current_stream(src)), "pack_weight");
}

// The same with the weight's per-output-channel scales stored behind the packed bytes (one allocation per layer).
void pack_weight_scaled(at::Tensor& src, at::Tensor& scales, at::Tensor& dst, int64_t src_format) {
    TORCH_CHECK(src.dim() == 2 && src.stride(1) == 1 && is_byte_tensor(src), "src must be a [n, k] one-byte tensor with unit stride along k");
    TORCH_CHECK(src.size(0) < (int64_t(1) << 30) && src.size(1) < (int64_t(1) << 30), "n and k must fit 30 bits");
    const int n = (int)src.size(0), k = (int)src.size(1);
    TORCH_CHECK(scales.scalar_type() == at::kFloat && scales.is_contiguous() && scales.numel() == n, "scales must be n contiguous float32 values");
    TORCH_CHECK(is_byte_tensor(dst) && dst.is_contiguous() && (size_t)dst.numel() == hfrk_packed_weight_bytes_scaled(n, k) && dst.numel() > 0,
                "dst must be a contiguous one-byte tensor of hfrk_packed_weight_bytes_scaled(n, k) elements (k % 256 == 0)");
    check_same_device(src, dst, "dst");
    check_same_device(src, scales, "scales");
    DeviceScope scope(src);
    raise_on(hfrk_pack_weight_scaled(src.data_ptr(), (int)src.stride(0), (int)src_format, scales.data_ptr<float>(), dst.data_ptr(), n, k,
                                     current_stream(src)), "pack_weight_scaled");
}

void unpack_weight(at::Tensor& src, at::Tensor& dst) {
    TORCH_CHECK(dst.dim() == 2 && dst.stride(1) == 1 && is_byte_tensor(dst), "dst must be a [n, k] one-byte tensor with unit stride along k");
    TORCH_CHECK(dst.size(0) < (int64_t(1) << 30) && dst.size(1) < (int64_t(1) << 30), "n and k must fit 30 bits");
    const int n = (int)dst.size(0), k = (int)dst.size(1);
    TORCH_CHECK(is_byte_tensor(src) && src.is_contiguous() && src.numel() > 0 &&
                    ((size_t)src.numel() == hfrk_packed_weight_bytes(n, k) || (size_t)src.numel() == hfrk_packed_weight_bytes_scaled(n, k)),
                "src must be a contiguous one-byte tensor of hfrk_packed_weight_bytes(n, k) elements (k % 256 == 0), or that plus its scales");
    check_same_device(src, dst, "dst");
    DeviceScope scope(src);
    raise_on(hfrk_unpack_weight(src.data_ptr(), dst.data_ptr(), (int)dst.stride(0), n, k, current_stream(src)), "unpack_weight");
}

// e4m3fnuz bytes -> e4m3fn bytes with the same values (dst may be src).
void reencode_fnuz(at::Tensor& src, at::Tensor& dst) {
    TORCH_CHECK(is_byte_tensor(src) && is_byte_tensor(dst) && src.is_contiguous() && dst.is_contiguous() && src.numel() == dst.numel(),
                "src and dst must be contiguous one-byte tensors of the same size");
    check_same_device(src, dst, "dst");
    DeviceScope scope(src);
    raise_on(hfrk_reencode_fnuz(src.data_ptr(), dst.data_ptr(), (size_t)src.numel(), current_stream(src)), "reencode_fnuz");
}

}  // namespace

TORCH_LIBRARY(_HFRK_C, ops) {
    ops.def("increment(Tensor! x) -> ()");
    ops.impl("increment", c10::kCUDA, &increment);

    ops.def(
        "residual_rms(Tensor input, Tensor! residual, Tensor weight, Tensor scale_tensor, float epsilon, Tensor! "
        "output, Tensor! next_buffer, int num_threads, bool force_scalar) -> ()");
    ops.impl("residual_rms", c10::kCUDA, &residual_rms);

    ops.def(
        "swiglu(Tensor gate_up, Tensor scale_tensor, Tensor! output, Tensor! next_buffer, int num_threads, "
        "bool force_scalar) -> ()");
    ops.impl("swiglu", c10::kCUDA, &swiglu);

    ops.def(
        "skinny_gemm_tb(Tensor A, Tensor B, Tensor! D, Tensor scale_tensor, int split_k, int A_producers, "
        "int B_producers, int consumers, int a_lanes, int b_lanes, int qsize, int op_m, int ops) -> int");
    ops.impl("skinny_gemm_tb", c10::kCUDA, &skinny_gemm_tb);

    ops.def("skinny_gemm_scaled(Tensor A, Tensor B, Tensor! D, Tensor scale_a, Tensor scale_b, bool accumulate) -> int");
    ops.impl("skinny_gemm_scaled", c10::kCUDA, &skinny_gemm_scaled);

    ops.def(
        "skinny_gemm_fused(Tensor A, Tensor B, Tensor! D, Tensor? base, Tensor scale_a, Tensor? scale_b, "
        "Tensor? out_scale, int epilogue, int intermediate_dtype) -> int");
    ops.impl("skinny_gemm_fused", c10::kCUDA, &skinny_gemm_fused);
    ops.def(
        "skinny_gemm_rms_fused(Tensor input, Tensor residual, Tensor! residual_out, Tensor rms_weight, float epsilon, "
        "Tensor act_scale, Tensor B, Tensor! D, Tensor? base, Tensor scale_a, Tensor? scale_b, Tensor? out_scale, "
        "int epilogue, int intermediate_dtype) -> int");
    ops.impl("skinny_gemm_rms_fused", c10::kCUDA, &skinny_gemm_rms_fused);

    ops.def(
        "skinny_gemm_packed(Tensor A, Tensor B_packed, int n, Tensor! D, Tensor? base, Tensor scale_a, Tensor? scale_b, "
        "Tensor? out_scale, int epilogue, int intermediate_dtype) -> int");
    ops.impl("skinny_gemm_packed", c10::kCUDA, &skinny_gemm_packed);

    ops.def(
        "skinny_gemm_checked(Tensor A, Tensor B, bool packed, int n, Tensor! D, Tensor? base, Tensor scale_a, Tensor? scale_b, "
        "Tensor? out_scale, int epilogue, int intermediate_dtype) -> ()");
    ops.impl("skinny_gemm_checked", c10::kCUDA, &skinny_gemm_checked);

    ops.def("pack_weight(Tensor src, Tensor! dst, int src_format) -> ()");
    ops.impl("pack_weight", c10::kCUDA, &pack_weight);
    ops.def("pack_weight_scaled(Tensor src, Tensor scales, Tensor! dst, int src_format) -> ()");
    ops.impl("pack_weight_scaled", c10::kCUDA, &pack_weight_scaled);
    ops.def("unpack_weight(Tensor src, Tensor! dst) -> ()");
    ops.impl("unpack_weight", c10::kCUDA, &unpack_weight);
    ops.def("reencode_fnuz(Tensor src, Tensor! dst) -> ()");
    ops.impl("reencode_fnuz", c10::kCUDA, &reencode_fnuz);

    ops.def(
        "residual_rms_dynamic(Tensor input, Tensor! residual, Tensor weight, float epsilon, Tensor! output, "
        "Tensor! scales, Tensor! next_buffer) -> ()");
    ops.impl("residual_rms_dynamic", c10::kCUDA, &residual_rms_dynamic);

    ops.def("swiglu_dynamic(Tensor gate_up, Tensor! output, Tensor! scales, Tensor! next_buffer) -> ()");
    ops.impl("swiglu_dynamic", c10::kCUDA, &swiglu_dynamic);

    ops.def("quantize_fp8(Tensor input, Tensor? scale_tensor, Tensor! output, Tensor! scales) -> ()");
    ops.impl("quantize_fp8", c10::kCUDA, &quantize_fp8);
}

// `import hf_rocm_kernels._HFRK_C` loads this library and thereby runs the registration above.
PyMODINIT_FUNC PyInit__HFRK_C(void) {
    static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_HFRK_C", nullptr, 0, nullptr};
    return PyModule_Create(&module);
}
