// Weight load format: row-major [n, k] e4m3 weights <-> the packed layout the GEMM kernels can stream without an
// LDS pass, and e4m3fnuz (gfx942 checkpoints) -> OCP e4m3fn re-encoding.  The step before the GEMM path: it runs
// once per weight when a model is loaded, not per token.
//
// Packed layout.  The weight is cut into chunks of 16 rows x 256 K-bytes (the GEMM kernels' unit of work), rows
// padded with zeros to a multiple of 16.  Chunk (tile, kc) -- rows [16 tile, 16 tile + 16), bytes [256 kc, 256 kc + 256)
// of each -- occupies the 4096 bytes at (tile * k/256 + kc) * 4096, so chunks that a wave streams one after the
// other (K fastest) are contiguous in memory.  Inside a chunk the bytes are in v_mfma_f32_16x16x128_f8f6f4 operand
// order: 16-byte piece j (0..3) of lane l (0..63) is at j * 1024 + l * 16 and holds row l % 16, bytes
// (j / 2) * 128 + (l / 16) * 32 + (j % 2) * 16 .. +16 of the chunk.  Pieces 2h and 2h+1 of a lane are its operand of
// MFMA step h; one `buffer_load_dwordx4` per piece reads 1 KB contiguous per wave.
//
// The reference has no load format: its kernel reads row-major weights through an LDS ring
// (csrc/op_src/skinny_gemm/producers/n_full_tiles.cu:4-127), and its fp8 tensors are fn bits viewed as fnuz with a
// doubled scale (hf_rocm_kernels/utils/fp8.py:27-29).
#include "hfrk_internal.h"

namespace hfrk {

constexpr int kPackWaves = 4;
constexpr int kChunkBytes = 4096;

// fnuz -> fn on four packed bytes, value preserving.  On the same bits an fnuz value is half the fn value, so a
// code with exponent field >= 2 just loses one from the exponent (code - 8).  Codes with magnitude bits below 16 are
// mag * 2^-10, half a unit of fn's subnormal grid: mag / 2 rounded to nearest even, which as an fn code is that
// number itself (8 = the smallest normal).  0x80 is fnuz's NaN and becomes fn's (0x7f).
__device__ __forceinline__ uint32_t fnuz_to_fn4(uint32_t x) {
    const uint32_t mag = x & 0x7f7f7f7fu, sign = x & 0x80808080u;
    const uint32_t big = ((mag + 0x70707070u) & 0x80808080u) >> 7;  // 1 in bytes with mag >= 16
    const uint32_t big_mask = big * 0xffu;
    const uint32_t r_big = ((mag | 0x80808080u) - 0x08080808u) & 0x7f7f7f7fu;  // no borrow leaves a byte
    const uint32_t half = (mag >> 1) & 0x3f3f3f3fu;
    const uint32_t r_small = half + (mag & half & 0x01010101u);  // + 1 when the dropped bit is set and the result is odd
    uint32_t out = sign | (big_mask & r_big) | (~big_mask & r_small);
    const uint32_t y = x ^ 0x80808080u;  // zero bytes here were 0x80
    const uint32_t is_nan = ~(((y & 0x7f7f7f7fu) + 0x7f7f7f7fu) | y | 0x7f7f7f7fu) >> 7;  // 1 in those bytes
    return (out & ~(is_nan * 0xffu)) | (is_nan * 0x7fu);
}

__device__ __forceinline__ v4i fnuz_to_fn16(v4i q) {
    return v4i{(int)fnuz_to_fn4((uint32_t)q[0]), (int)fnuz_to_fn4((uint32_t)q[1]), (int)fnuz_to_fn4((uint32_t)q[2]),
               (int)fnuz_to_fn4((uint32_t)q[3])};
}

// One wave per chunk.  Row-major side: load/store t moves rows 4t + l/16, bytes (l%16)*16 .. +16 (4 rows x 256
// contiguous bytes per instruction).  Packed side: piece j at j*1024 + l*16.  In between, the wave's private 4 KB
// LDS tile, XOR-swizzled so that neither side has bank conflicts -- the same pass the GEMM kernels make per chunk
// when they read a row-major weight.
template <bool UNPACK, bool FNUZ>
__global__ void __launch_bounds__(kPackWaves* kWave) pack_weight_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                                       int n, int k, int row_stride, uint32_t chunks) {
    constexpr uint32_t kOutOfRange = 0x80000000u;
    __shared__ __align__(16) uint8_t lds[kPackWaves * kChunkBytes];
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    uint8_t* const tile_mem = lds + wv * kChunkBytes;
    const uint32_t KC = (uint32_t)k >> 8;
    const uint32_t tiles = (uint32_t)(n + 15) >> 4;
    const uint8_t* const rows = UNPACK ? dst : src;  // the row-major side
    const __amdgpu_buffer_rsrc_t row_rsrc = make_rsrc(rows, (uint32_t)(n - 1) * (uint32_t)row_stride + (uint32_t)k);
    const __amdgpu_buffer_rsrc_t pk_rsrc = make_rsrc(UNPACK ? src : dst, tiles * KC * (uint32_t)kChunkBytes);
    int row_off[4], op_off[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int row = 4 * t + lg;
        row_off[t] = row * 256 + ((li ^ row) << 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) op_off[j] = li * 256 + ((((8 * (j >> 1) + 2 * lg + (j & 1)) ^ li) & 15) << 4);

    for (uint32_t c = blockIdx.x * kPackWaves + wv; c < chunks; c += gridDim.x * kPackWaves) {
        const uint32_t tile = c / KC, kc = c - tile * KC;
        const uint32_t pk_base = c * (uint32_t)kChunkBytes + (uint32_t)lane * 16u;
        v4i q[4];
        if constexpr (!UNPACK) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t row = tile * 16u + 4u * t + (uint32_t)lg;  // rows >= n: padding, read as zero
                q[t] = __builtin_amdgcn_raw_buffer_load_b128(row_rsrc, row < (uint32_t)n ? (int)(row * (uint32_t)row_stride + kc * 256u + (uint32_t)li * 16u) : (int)kOutOfRange, 0, 2 /* nt */);
                if constexpr (FNUZ) q[t] = fnuz_to_fn16(q[t]);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) *reinterpret_cast<v4i*>(tile_mem + row_off[t]) = q[t];
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) q[j] = __builtin_amdgcn_raw_buffer_load_b128(pk_rsrc, (int)(pk_base + (uint32_t)j * 1024u), 0, 2 /* nt */);
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<v4i*>(tile_mem + op_off[j]) = q[j];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if constexpr (!UNPACK) {
#pragma unroll
            for (int j = 0; j < 4; ++j) q[j] = *reinterpret_cast<const v4i*>(tile_mem + op_off[j]);
#pragma unroll
            for (int j = 0; j < 4; ++j) __builtin_amdgcn_raw_buffer_store_b128(q[j], pk_rsrc, (int)(pk_base + (uint32_t)j * 1024u), 0, 0);
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) q[t] = *reinterpret_cast<const v4i*>(tile_mem + row_off[t]);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t row = tile * 16u + 4u * t + (uint32_t)lg;  // padding rows are dropped
                __builtin_amdgcn_raw_buffer_store_b128(q[t], row_rsrc, row < (uint32_t)n ? (int)(row * (uint32_t)row_stride + kc * 256u + (uint32_t)li * 16u) : (int)kOutOfRange, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

// Elementwise fnuz -> fn over `count` bytes: 16 bytes per lane and step, the tail byte by byte through the same
// word function.
__global__ void __launch_bounds__(256) reencode_fnuz_kernel(const uint8_t* src, uint8_t* dst, size_t count) {
    const size_t vecs = count / 16;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs; i += stride)
        reinterpret_cast<v4i*>(dst)[i] = fnuz_to_fn16(__builtin_nontemporal_load(reinterpret_cast<const v4i*>(src) + i));
    for (size_t i = vecs * 16 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride)
        dst[i] = (uint8_t)fnuz_to_fn4(src[i]);
}

static int check_weight(const void* rows, const void* packed, int n, int k, int row_stride) {
    if (!rows || !packed || n < 1 || k < 1 || row_stride < k) return HFRK_BAD_SHAPE;
    if (k % 256 != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (((long)n + 16) * row_stride + k >= (1L << 31) || ((long)n + 16) * k >= (1L << 31)) return HFRK_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(rows) | reinterpret_cast<uintptr_t>(packed)) & 15 || (row_stride & 15)) return HFRK_BAD_ALIGNMENT;
    return HFRK_SUCCESS;
}

template <bool UNPACK, bool FNUZ>
static int launch_pack(const void* src, void* dst, int n, int k, int row_stride, hipStream_t stream) {
    const uint32_t chunks = (uint32_t)((n + 15) / 16) * (uint32_t)(k / 256);
    const uint32_t blocks = (chunks + kPackWaves - 1) / kPackWaves;
    const uint32_t grid = blocks < 16u * kNumCU ? blocks : 16u * kNumCU;
    hipLaunchKernelGGL((pack_weight_kernel<UNPACK, FNUZ>), dim3(grid), dim3(kPackWaves * kWave), 0, stream,
                       static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), n, k, row_stride, chunks);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

// the per-output-channel scales behind the packed bytes: n values, then zeros up to the padded row count
__global__ void pack_scales_kernel(const float* __restrict__ src, float* __restrict__ dst, int n, int n_padded) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_padded) dst[i] = i < n ? src[i] : 0.0f;
}

}  // namespace hfrk

extern "C" {

size_t hfrk_packed_weight_bytes(int n, int k) {
    if (n < 1 || k < 1 || k % 256 != 0) return 0;
    return (size_t)((n + 15) / 16) * 16 * (size_t)k;
}

size_t hfrk_packed_weight_bytes_scaled(int n, int k) {
    const size_t bytes = hfrk_packed_weight_bytes(n, k);
    return bytes ? bytes + (size_t)((n + 15) / 16) * 16 * sizeof(float) : 0;
}

const float* hfrk_packed_weight_scales(const void* packed, int n, int k) {
    const size_t bytes = hfrk_packed_weight_bytes(n, k);
    return (bytes && packed) ? reinterpret_cast<const float*>(static_cast<const uint8_t*>(packed) + bytes) : nullptr;
}

int hfrk_pack_weight_scaled(const void* src, int src_stride, int src_format, const float* scales, void* dst, int n, int k,
                            void* stream) {
    if (!scales) return HFRK_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(scales) & 3) return HFRK_BAD_ALIGNMENT;
    const int rc = hfrk_pack_weight(src, src_stride, src_format, dst, n, k, stream);
    if (rc != HFRK_SUCCESS) return rc;
    const int n_padded = (n + 15) / 16 * 16;
    float* tail = const_cast<float*>(hfrk_packed_weight_scales(dst, n, k));
    hipLaunchKernelGGL(hfrk::pack_scales_kernel, dim3((n_padded + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       scales, tail, n, n_padded);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

int hfrk_pack_weight(const void* src, int src_stride, int src_format, void* dst, int n, int k, void* stream) {
    const int rc = hfrk::check_weight(src, dst, n, k, src_stride);
    if (rc != HFRK_SUCCESS) return rc;
    if (src_format == HFRK_WEIGHT_E4M3FN) return hfrk::launch_pack<false, false>(src, dst, n, k, src_stride, static_cast<hipStream_t>(stream));
    if (src_format == HFRK_WEIGHT_E4M3FNUZ) return hfrk::launch_pack<false, true>(src, dst, n, k, src_stride, static_cast<hipStream_t>(stream));
    return HFRK_BAD_DTYPE;
}

int hfrk_unpack_weight(const void* src, void* dst, int dst_stride, int n, int k, void* stream) {
    const int rc = hfrk::check_weight(dst, src, n, k, dst_stride);
    if (rc != HFRK_SUCCESS) return rc;
    return hfrk::launch_pack<true, false>(src, dst, n, k, dst_stride, static_cast<hipStream_t>(stream));
}

int hfrk_reencode_fnuz(const void* src, void* dst, size_t count, void* stream) {
    if (count == 0) return HFRK_SUCCESS;
    if (!src || !dst) return HFRK_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) return HFRK_BAD_ALIGNMENT;
    const size_t blocks = (count / 16 + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 1 ? 1 : blocks > 8u * hfrk::kNumCU ? 8u * hfrk::kNumCU : blocks);
    hipLaunchKernelGGL(hfrk::reencode_fnuz_kernel, dim3(grid), dim3(256), 0, stream ? static_cast<hipStream_t>(stream) : nullptr,
                       static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), count);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

}  // extern "C"
