// Row-split kernel on bands of whole 16-row tiles, for row-major weights and for weights in the packed load format
// (pack_weight.hip): instantiations of skinny_gemm_rows_impl.h.  The packed variant is what replaces, for a weight packed
// at load time, the reference's LDS ring between its weight producers and its consumers
// (csrc/op_src/skinny_gemm/producers/n_full_tiles.cu:4-127): the registers a load fills are the matrix-core operands.
#include "skinny_gemm_rows_impl.h"

namespace hfrk {

template <int LAYOUT>
static int launch_rows_tiled_layout(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, int lds_bytes, hipStream_t stream) {
    if (act_loads > 4) {  // 17..32 rows: two activation tiles, two weight tiles per chunk
        if (row_tiles != 2) return HFRK_INVALID_CONFIG;
        if (swiglu) return act_loads == 6 ? launch_rows_one<6, 2, true, false, LAYOUT>(args, lds_bytes, stream)
                                          : launch_rows_one<8, 2, true, false, LAYOUT>(args, lds_bytes, stream);
        return act_loads == 6 ? launch_rows_one<6, 2, false, false, LAYOUT>(args, lds_bytes, stream)
                              : launch_rows_one<8, 2, false, false, LAYOUT>(args, lds_bytes, stream);
    }
#define HFRK_ROWS_CASE(MA_)                                                                             \
    case MA_:                                                                                           \
        if (swiglu) return launch_rows_one<MA_, 2, true, false, LAYOUT>(args, lds_bytes, stream);       \
        return row_tiles == 1 ? launch_rows_one<MA_, 1, false, false, LAYOUT>(args, lds_bytes, stream)  \
                              : launch_rows_one<MA_, 2, false, false, LAYOUT>(args, lds_bytes, stream);
    switch (act_loads) {
        HFRK_ROWS_CASE(1)
        HFRK_ROWS_CASE(2)
        HFRK_ROWS_CASE(3)
        HFRK_ROWS_CASE(4)
    }
#undef HFRK_ROWS_CASE
    return HFRK_INVALID_CONFIG;
}

int launch_rows_tiled_kernel(const GemmArgs& args, int act_loads, int row_tiles, bool swiglu, int lds_bytes, hipStream_t stream) {
    if (!rows_variant_exists(act_loads, row_tiles)) return HFRK_INVALID_CONFIG;
    if (swiglu && row_tiles != 2) return HFRK_INVALID_CONFIG;
    if (lds_bytes != rows_lds_bytes(row_tiles, act_loads)) return HFRK_INVALID_CONFIG;
    return args.packed ? launch_rows_tiled_layout<kRowsPacked>(args, act_loads, row_tiles, swiglu, lds_bytes, stream)
                       : launch_rows_tiled_layout<kRowsTiles>(args, act_loads, row_tiles, swiglu, lds_bytes, stream);
}

}  // namespace hfrk
