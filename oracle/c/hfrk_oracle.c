/*
 * Plain-C restatement of the arithmetic of the FP8 skinny-GEMM path.  TEST INFRASTRUCTURE ONLY: it is loaded by
 * tests/ (to pin the torch-based oracle next to it) and never by the shipped package.
 *
 * What each function follows in the reference tree:
 *   decode / encode      the e4m3 format the reference quantises to (hf_rocm_kernels/utils/fp8.py:6-29), taken as
 *                        OCP e4m3fn: bias 7, max 448, S.1111.111 = NaN
 *   gemm_int / gemm_f32  D = scale * A . B of csrc/op_src/skinny_gemm/skinny_gemm_kernel.cu:6-79 with the epilogue
 *                        of consumers/mfma_16x16x32_consumer.cu:129-163, i.e. what torch._scaled_mm computes in
 *                        operators/skinny_gemm/reference.py:18-25
 *   rms_row              operators/residual_rms/reference.py:69-72 and residual_rms_scalar.cu:24-40
 *   swiglu               operators/swiglu/reference.py:19-23 and swiglu_scalar.cu:52-61
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

double hfrk_oracle_decode_e4m3fn(uint8_t code) {
    const int sign = code >> 7, exp = (code >> 3) & 0xF, man = code & 0x7;
    double v;
    if (exp == 0xF && man == 0x7) return NAN;
    if (exp == 0) v = ldexp((double)man, -9);
    else v = ldexp(1.0 + man / 8.0, exp - 7);
    return sign ? -v : v;
}

/* value * 2^9 as an integer (every finite e4m3fn value is a multiple of 2^-9); 0 for NaN codes */
static int32_t fixed9(uint8_t code) {
    const int sign = code >> 7, exp = (code >> 3) & 0xF, man = code & 0x7;
    int32_t v;
    if (exp == 0xF && man == 0x7) return 0;
    if (exp == 0) v = man;
    else v = (8 + man) << (exp - 1); /* (1 + man/8) * 2^(exp-7) * 2^9 = (8+man) * 2^(exp-1) */
    return sign ? -v : v;
}

/* round to nearest, ties to even, saturating at +-448; NaN -> 0x7F */
uint8_t hfrk_oracle_encode_e4m3fn(double x) {
    if (isnan(x)) return 0x7F;
    const uint8_t sign = signbit(x) ? 0x80 : 0;
    double mag = fabs(x);
    if (mag >= 448.0) return sign | 0x7E;
    int best = 0;
    double best_d = INFINITY;
    for (int code = 0; code <= 0x7E; ++code) {
        const double d = fabs(hfrk_oracle_decode_e4m3fn((uint8_t)code) - mag);
        if (d < best_d || (d == best_d && (code & 1) == 0)) {
            best_d = d;
            best = code;
        }
    }
    return sign | (uint8_t)best;
}

/* out[i*n+j] = sum_k A[i,k] * W[j,k] in units of 2^-18, exact.  A [m,k], W [n,k] row-major with row stride ldw. */
void hfrk_oracle_gemm_int(const uint8_t* A, const uint8_t* W, int m, int n, int k, int ldw, int64_t* out) {
#pragma omp parallel for schedule(static)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            int64_t acc = 0;
            for (int t = 0; t < k; ++t) acc += (int64_t)fixed9(A[(size_t)i * k + t]) * fixed9(W[(size_t)j * ldw + t]);
            out[(size_t)i * n + j] = acc;
        }
    }
}

/* The fp32 path named by the parity statement: dequantise each operand with its scale, multiply-accumulate in
 * fp32 in k order, add the bias.  sa has m entries (sa_stride 1) or one (0); sw likewise over n. */
void hfrk_oracle_gemm_f32(const uint8_t* A, const uint8_t* W, const float* sa, int sa_stride, const float* sw,
                          int sw_stride, const float* bias, int m, int n, int k, int ldw, float* out) {
#pragma omp parallel for schedule(static)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            float acc = 0.f;
            const float a_s = sa[(size_t)i * sa_stride], w_s = sw[(size_t)j * sw_stride];
            for (int t = 0; t < k; ++t) {
                const float av = (float)hfrk_oracle_decode_e4m3fn(A[(size_t)i * k + t]) * a_s;
                const float wv = (float)hfrk_oracle_decode_e4m3fn(W[(size_t)j * ldw + t]) * w_s;
                acc += av * wv;
            }
            out[(size_t)i * n + j] = acc + (bias ? bias[(size_t)i * n + j] : 0.f);
        }
    }
}

/* y[c] = z[c] * rsqrt(mean(z^2) + eps) * w[c] for one row, in double: the textbook formula */
void hfrk_oracle_rms_row(const double* z, const double* w, double eps, int cols, double* y) {
    double ss = 0.0;
    for (int c = 0; c < cols; ++c) ss += z[c] * z[c];
    const double r = 1.0 / sqrt(ss / cols + eps);
    for (int c = 0; c < cols; ++c) y[c] = z[c] * r * w[c];
}

/* out[r,c] = gate[r,c] / (1 + exp(-gate[r,c])) * up[r,c], gate = cols [0,n), up = cols [n,2n) of each row */
void hfrk_oracle_swiglu(const double* gate_up, int rows, int n, double* out) {
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < n; ++c) {
            const double g = gate_up[(size_t)r * 2 * n + c], u = gate_up[(size_t)r * 2 * n + n + c];
            out[(size_t)r * n + c] = g / (1.0 + exp(-g)) * u;
        }
}
