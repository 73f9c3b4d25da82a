// Row-split kernel for row-major weights dealt out in 4-row units (the planner's choice up to 16 rows, and 17..32 rows by
// rule), with its SwiGLU-epilogue and RMSNorm-prologue variants: instantiations of skinny_gemm_rows_impl.h.
#include "skinny_gemm_rows_impl.h"

namespace hfrk {

int launch_rows_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, bool rms, int lds_bytes, hipStream_t stream) {
    if (!rows_variant_exists(act_loads, row_tiles)) return HFRK_INVALID_CONFIG;
    if (swiglu && row_tiles != 2) return HFRK_INVALID_CONFIG;
    if (rms) {  // variants: up to 8 rows; one tile per chunk with the plain epilogue, gate + up tile with SwiGLU
        if (act_loads > 2 || row_tiles != (swiglu ? 2 : 1) || (args.k != 4096 && args.k != 8192)) return HFRK_INVALID_CONFIG;
        if (lds_bytes != rows_rms_lds_bytes(act_loads, row_tiles, args.k)) return HFRK_INVALID_CONFIG;
        if (act_loads == 1) return swiglu ? launch_rows_one<1, 2, true, true>(args, lds_bytes, stream) : launch_rows_one<1, 1, false, true>(args, lds_bytes, stream);
        return swiglu ? launch_rows_one<2, 2, true, true>(args, lds_bytes, stream) : launch_rows_one<2, 1, false, true>(args, lds_bytes, stream);
    }
    if (lds_bytes != rows_lds_bytes(row_tiles, act_loads)) return HFRK_INVALID_CONFIG;
    if (act_loads > 4) {  // 17..32 rows: two activation tiles, two weight tiles per chunk
        if (row_tiles != 2) return HFRK_INVALID_CONFIG;
        if (swiglu) return act_loads == 6 ? launch_rows_one<6, 2, true, false>(args, lds_bytes, stream) : launch_rows_one<8, 2, true, false>(args, lds_bytes, stream);
        return act_loads == 6 ? launch_rows_one<6, 2, false, false>(args, lds_bytes, stream) : launch_rows_one<8, 2, false, false>(args, lds_bytes, stream);
    }
#define HFRK_ROWS_CASE(MA_)                                                                     \
    case MA_:                                                                                   \
        if (swiglu) return launch_rows_one<MA_, 2, true, false>(args, lds_bytes, stream);       \
        return row_tiles == 1 ? launch_rows_one<MA_, 1, false, false>(args, lds_bytes, stream)  \
                              : launch_rows_one<MA_, 2, false, false>(args, lds_bytes, stream);
    switch (act_loads) {
        HFRK_ROWS_CASE(1)
        HFRK_ROWS_CASE(2)
        HFRK_ROWS_CASE(3)
        HFRK_ROWS_CASE(4)
    }
#undef HFRK_ROWS_CASE
    return HFRK_INVALID_CONFIG;
}

}  // namespace hfrk
