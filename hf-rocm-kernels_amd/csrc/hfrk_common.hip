// Status text, version and per-thread HIP error slot of libhfrk_gfx950.so.
#include "hfrk_internal.h"

namespace hfrk {

static thread_local int g_last_hip_error = 0;

void set_last_hip_error(hipError_t e) { g_last_hip_error = static_cast<int>(e); }

}  // namespace hfrk

extern "C" {

int hfrk_version(void) { return 110; }

int hfrk_last_hip_error(void) { return hfrk::g_last_hip_error; }

const char* hfrk_status_string(int status) {
    switch (status) {
        case HFRK_SUCCESS: return "success";
        case HFRK_M_ABOVE_WARPTILE_M: return "m is greater than the warp tile";
        case HFRK_N_NOT_EVEN: return "n is not even";
        case HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K: return "k is not divisible by the K tile (256, or (512/op_m)*ops)";
        case HFRK_TOO_MANY_WARPS: return "A_producers + B_producers + consumers is greater than 16";
        case HFRK_QSIZE_TOO_SMALL: return "qsize is less than A_producers/a_lanes, B_producers/b_lanes or consumers";
        case HFRK_INVALID_CONFIG: return "invalid configuration";
        case HFRK_BAD_SHAPE: return "unsupported shape or null pointer";
        case HFRK_BAD_ALIGNMENT: return "pointer or stride is not aligned as required";
        case HFRK_BAD_DTYPE: return "unsupported element type";
        case HFRK_HIP_ERROR: return "HIP runtime error (see hfrk_last_hip_error)";
        case HFRK_NOT_INITIALISED: return "no free split-K workspace and the stream is capturing: call hfrk_init(), and launch once on further streams, first";
        case HFRK_BAD_FILE: return "plan-table file cannot be read or is not a plan table";
        case HFRK_EXCEEDS_SCRATCH: return "the plan needs more partial sums or counters than the allocation-free entry point's scratch array holds";
        case HFRK_NO_WORKSPACE: return "too many streams hold a split-K workspace (hfrk_release_stream frees one)";
        default: return "unknown status";
    }
}

}  // extern "C"
