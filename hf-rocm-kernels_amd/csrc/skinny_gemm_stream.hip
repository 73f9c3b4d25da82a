// FP8 skinny GEMM, m <= 32: every wavefront streams its own run of weight chunks, nothing is shared in the loop.
//
// The weight matrix is cut into chunks of 16*RT rows x 256 K-bytes (RT = 1 or 2 row tiles of 16 rows: 4 or 8 KB),
// numbered row group by row group, K fastest.  ("Row tile" below means such a group of RT tiles.)
// The chunk sequence is split evenly over the workgroups (the first `C % G` of them get one chunk more) and, inside
// a workgroup, evenly over its 8 waves, so a wave owns one contiguous run: part of a row tile, then whole row
// tiles, then part of another.  For each chunk the wave loads the weights (4*RT 16-byte `nt` loads per lane, 4 rows
// x 256 contiguous bytes per instruction) and the matching m x 256 bytes of activations (L1/L2 hits; rows >= m are
// out of the buffer's range and cost no traffic), turns both into MFMA operand layout through private,
// XOR-swizzled LDS tiles, and issues 2*RT*MT v_mfma_f32_16x16x128_f8f6f4 (MT = 16-row activation tiles).  RT = 2
// halves the activation bytes read from L2 per weight byte, which is what limits m >= 16; for small m a 4 KB
// chunk gives the short runs of the decode shapes more requests to overlap.  The next chunk's loads are issued
// as soon as the registers have been copied to LDS.  There is no barrier, no shared staging and no cross-wave
// dependency in the loop: measured, this loop sustains the same bandwidth as a kernel that only reads the weights.
//
// What the decode shapes leave to optimise is serial instruction count: a launch lives 5-20 us, one wave retires
// a few hundred instructions per microsecond, and both the code before the first load and the code after the last
// MFMA sit on the critical path.  Hence the division-free chunk partition (quotient and remainder come from the
// host), the early first request, and the closed-form reduction below that needs no exchanged descriptors.
//
// Sums that a wave cannot finish alone (a row tile split between waves) are combined once, after the loop:
// a wave whose run starts inside a row tile leaves that partial 16x16 fp32 tile in LDS, one barrier, and the wave
// that holds the tile's first chunk in this workgroup adds the partials of the waves after it whose runs start
// before the tile (or the workgroup's range) ends -- wave runs are consecutive, so that is a comparison per wave.
// A row tile split between workgroups goes through the workspace with a per-tile arrival counter; the last
// workgroup to arrive adds the partials in workgroup order.  Both orders are fixed, so results are
// bit-reproducible.  Scales, the optional accumulate-into-D and the single rounding to 16 bits happen there.
//
// Replaces, for m <= 32, the reference's csrc/op_src/skinny_gemm/skinny_gemm_kernel.cu:6-79 with its producers and
// consumers (producers/n_full_tiles.cu:4-127, consumers/mfma_16x16x32_consumer.cu:1-168,
// consumers/smfma_16x16x64_consumer.cu:1-158).
#include "skinny_gemm_stream_body.h"

namespace hfrk {

// Template parameters as in skinny_gemm_stream_body.h.
template <int MA, int RT, bool SWIGLU, bool PACKED>
__global__ void __launch_bounds__(kGemmThreads) skinny_gemm_stream_kernel(const GemmArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    stream_gemm_body<MA, RT, SWIGLU, PACKED, false>(a, lds, NoGate{});
}

template <int MA, int RT, bool SWIGLU, bool PACKED>
static int launch_stream_packing(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = skinny_gemm_stream_kernel<MA, RT, SWIGLU, PACKED>;
    static bool attr_done[64] = {};
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev >= 0 && dev < 64 && !attr_done[dev]) {
        HFRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
        attr_done[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3(args.grid), dim3(kGemmThreads), lds_bytes, stream, args);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

template <int MA, int RT, bool SWIGLU>
static int launch_stream_one(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    return args.packed ? launch_stream_packing<MA, RT, SWIGLU, true>(args, lds_bytes, stream)
                       : launch_stream_packing<MA, RT, SWIGLU, false>(args, lds_bytes, stream);
}

int launch_stream_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, int lds_bytes, hipStream_t stream) {
    if (lds_bytes != stream_lds_bytes(act_loads, row_tiles)) return HFRK_INVALID_CONFIG;
    if (swiglu) {
        if (row_tiles != 2) return HFRK_INVALID_CONFIG;
        switch (act_loads) {
            case 1: return launch_stream_one<1, 2, true>(args, lds_bytes, stream);
            case 2: return launch_stream_one<2, 2, true>(args, lds_bytes, stream);
            case 3: return launch_stream_one<3, 2, true>(args, lds_bytes, stream);
            case 4: return launch_stream_one<4, 2, true>(args, lds_bytes, stream);
        }
        return HFRK_INVALID_CONFIG;
    }
    if (row_tiles == 1) {
        switch (act_loads) {
            case 1: return launch_stream_one<1, 1, false>(args, lds_bytes, stream);
            case 2: return launch_stream_one<2, 1, false>(args, lds_bytes, stream);
            case 3: return launch_stream_one<3, 1, false>(args, lds_bytes, stream);
            case 4: return launch_stream_one<4, 1, false>(args, lds_bytes, stream);
        }
    } else if (row_tiles == 2) {
        switch (act_loads) {
            case 3: return launch_stream_one<3, 2, false>(args, lds_bytes, stream);
            case 4: return launch_stream_one<4, 2, false>(args, lds_bytes, stream);
            case 5: return launch_stream_one<5, 2, false>(args, lds_bytes, stream);
            case 6: return launch_stream_one<6, 2, false>(args, lds_bytes, stream);
            case 7: return launch_stream_one<7, 2, false>(args, lds_bytes, stream);
            case 8: return launch_stream_one<8, 2, false>(args, lds_bytes, stream);
        }
    }
    return HFRK_INVALID_CONFIG;
}

}  // namespace hfrk
