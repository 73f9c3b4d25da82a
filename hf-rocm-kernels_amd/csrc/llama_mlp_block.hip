// The decoder MLP sub-block in one launch: residual RMSNorm -> fp8, gate_up GEMM with the SwiGLU epilogue -> fp8,
// down GEMM + residual.  Same arithmetic, same roundings and same summation orders as the three launches it replaces
// (residual_rms_row.h, skinny_gemm_stream_body.h run twice), so the results have the same bits; what it removes is
// two kernel boundaries: each costs a drained machine, a launch, and the latency of the first weight bytes.
//
// 256 persistent workgroups, one per CU, all resident at once.  Phases are separated by a grid-wide gate (an arrival
// counter in device memory); a wave requests the first weight chunk of the next phase BEFORE it waits at the gate,
// since weights depend on nothing, so the weight stream restarts without a cold start:
//   gate 1: workgroups 0 .. m-1 normalise one row each (write-through stores), everyone arrives
//   phase 1: gate_up GEMM + SwiGLU, activations = the normalised rows, output fp8 [m, inter] (write-through stores)
//   gate 2: everyone arrives once its part of phase 1 is stored
//   phase 2: down GEMM, activations = phase 1's output, epilogue adds the updated residual
// Data that crosses workgroups inside the launch is stored write-through to memory and read after the reading CU's
// L1 and the XCD's L2 have dropped what they held (an acquire fence behind each gate).
//
// The wait at a gate is bounded: a workgroup that has polled `spin_limit` times without seeing all arrivals counts
// a time-out in bar[1] and goes on (its results are then wrong, and hfrk_llama_mlp_block_timeouts reports it).
// That can only happen if the workgroups are not all resident, i.e. if something else occupies CUs for as long.
//
// Replaces the launch sequence of the reference's combined_ops/llama_mlp.py:7-60.
#include "residual_rms_row.h"
#include "skinny_gemm_stream_body.h"

namespace hfrk {

// Every wave calls this once per gate.  `bar[0]` only ever grows: ticket t belongs to gate number t / nwg of the
// counter's lifetime, and that gate opens when the counter reaches the next multiple of nwg (a power of two, so the
// arithmetic survives the counter wrapping around).
__device__ __forceinline__ void grid_gate(unsigned* bar, unsigned nwg, int spin_limit) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's stores are in memory
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned ticket = __hip_atomic_fetch_add(&bar[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned target = (ticket | (nwg - 1u)) + 1u;
        int spins = 0;
        while ((int)(__hip_atomic_load(&bar[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
            if (++spins > spin_limit) {
                __hip_atomic_fetch_add(&bar[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
    }
    __syncthreads();
    // what this CU's L1 and this XCD's L2 hold of the other workgroups' outputs is dropped before anything is read
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

template <int DT, int MA, bool PACKED>
__global__ void __launch_bounds__(kGemmThreads) llama_mlp_block_kernel(const MlpBlockArgs p) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ float red[16];
    const unsigned nwg = gridDim.x;
    auto gate1 = [&]() __attribute__((always_inline)) {
        if ((int)blockIdx.x < p.gate_up.m) {
            const int row = (int)blockIdx.x;
            if (p.hidden <= 8 * kGemmThreads)
                rms_row_vec<DT, true, 1, true>(p.input, p.residual, p.rms_weight, p.rms_scale, p.normalized, p.epsilon, p.hidden, row, red);
            else
                rms_row_vec<DT, true, 2, true>(p.input, p.residual, p.rms_weight, p.rms_scale, p.normalized, p.epsilon, p.hidden, row, red);
        }
        grid_gate(p.bar, nwg, p.spin_limit);
    };
    stream_gemm_body<MA, 2, true, PACKED, true>(p.gate_up, lds, gate1);
    auto gate2 = [&]() __attribute__((always_inline)) { grid_gate(p.bar, nwg, p.spin_limit); };
    stream_gemm_body<MA, 1, false, PACKED, true>(p.down, lds, gate2);
}

template <int DT, int MA, bool PACKED>
static int launch_block_variant(const MlpBlockArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = llama_mlp_block_kernel<DT, MA, PACKED>;
    static bool attr_done[64] = {};
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev >= 0 && dev < 64 && !attr_done[dev]) {
        HFRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, stream_lds_bytes(4, 2)));  // the kernel also has static LDS
        attr_done[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3(args.gate_up.grid), dim3(kGemmThreads), lds_bytes, stream, args);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

template <int DT, int MA>
static int launch_block_packing(const MlpBlockArgs& args, int lds_bytes, hipStream_t stream) {
    return args.gate_up.packed ? launch_block_variant<DT, MA, true>(args, lds_bytes, stream)
                               : launch_block_variant<DT, MA, false>(args, lds_bytes, stream);
}

template <int DT>
static int launch_block_dtype(const MlpBlockArgs& args, int act_loads, int lds_bytes, hipStream_t stream) {
    switch (act_loads) {
        case 1: return launch_block_packing<DT, 1>(args, lds_bytes, stream);
        case 2: return launch_block_packing<DT, 2>(args, lds_bytes, stream);
        case 3: return launch_block_packing<DT, 3>(args, lds_bytes, stream);
        case 4: return launch_block_packing<DT, 4>(args, lds_bytes, stream);
    }
    return HFRK_INVALID_CONFIG;
}

int launch_mlp_block_kernel(const MlpBlockArgs& args, int act_loads, hipStream_t stream) {
    // every gate needs all workgroups resident: one per CU, and the two GEMM phases share the grid
    if (args.gate_up.grid != kNumCU || args.down.grid != kNumCU) return HFRK_INVALID_CONFIG;
    if (args.gate_up.packed != args.down.packed) return HFRK_INVALID_CONFIG;
    const int lds_bytes = stream_lds_bytes(act_loads, 2);  // the larger of the two phases
    return args.io_dtype == HFRK_BF16 ? launch_block_dtype<HFRK_BF16>(args, act_loads, lds_bytes, stream)
                                      : launch_block_dtype<HFRK_F16>(args, act_loads, lds_bytes, stream);
}

}  // namespace hfrk
