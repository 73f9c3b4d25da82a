// What the row-split kernels (skinny_gemm_rows.hip, skinny_gemm_rows_tiled.hip) do with a finished 16x16 sum: scale, add the
// old D values (accumulate mode), round once, store -- or, with the SwiGLU epilogue, round gate and up to the 16-bit
// intermediate dtype, apply silu(gate) * up / out_scale and store four fp8 values
// (the reference's csrc/op_src/swiglu/swiglu_vectorized.cu:27-97 as the GEMM's epilogue).
// A lane (li = lane % 16, lg = lane / 16) holds D[16*mt + li][n0 + v], v = 0..3, n0 = row0 + 16*rt + 4*lg, of every
// (activation tile mt, weight tile rt) of a chunk.
#pragma once
#include "skinny_gemm_args.h"

namespace hfrk {

typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// two fp32 -> two 16-bit values in one register, round to nearest even (v_cvt_pk_bf16_f32 / v_cvt_f16_f32)
__device__ __forceinline__ uint32_t pack16(float lo, float hi, bool bf16) {
    const v2f v = {lo, hi};
    return bf16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf))
                : __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2h));
}

// MT = 16-row activation tiles, RT = 16-row weight tiles per chunk.
template <int MT, int RT, bool SWIGLU>
struct RowsEpilogue {
    static constexpr uint32_t kOutOfRange = 0x80000000u;
    // Old D values (accumulate mode) and per-channel scales of one tile, requested ahead of the epilogue that uses them
    struct Pre { v2i d[MT * RT]; v4i sb[RT]; };

    const GemmArgs& a;
    __amdgpu_buffer_rsrc_t d_rsrc, base_rsrc, sb_rsrc;
    int n_out;            // columns of D
    bool accumulate, vec, per_channel, bf16, want_pre;
    float sa_mt[MT];      // lane li holds the accumulator column of activation row 16 mt + li
    float inv_out_scale;
    int li, lg;

    __device__ __forceinline__ RowsEpilogue(const GemmArgs& args, int lane) : a(args), li(lane & 15), lg(lane >> 4) {
        n_out = SWIGLU ? (a.n >> 1) : a.n;
        d_rsrc = make_rsrc(a.D, (uint32_t)a.m * (uint32_t)n_out * (SWIGLU ? 1u : 2u));
        base_rsrc = make_rsrc(a.base, a.base ? (uint32_t)a.m * (uint32_t)a.n * 2u : 0u);
        sb_rsrc = make_rsrc(a.scale_b, a.scale_b ? (uint32_t)a.n * 4u : 0u);
        accumulate = !SWIGLU && a.base != nullptr;
        vec = SWIGLU || (a.n & 3) == 0;  // then a lane's four outputs are all inside n and aligned
        per_channel = a.scale_b && a.sb_stride;
        bf16 = a.d_dtype == HFRK_BF16;
        want_pre = vec && (accumulate || per_channel);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            sa_mt[mt] = a.scale_a[(long)min(16 * mt + li, a.m - 1) * a.sa_stride] * ((a.scale_b && !a.sb_stride) ? a.scale_b[0] : 1.0f);
        inv_out_scale = 1.0f;
        if constexpr (SWIGLU) {
            const float os = a.out_scale[0];
            inv_out_scale = os != 0.f ? 1.0f / os : 1.0f;
        }
    }

    // Old D values and per-channel scales of a tile whose first row is `row0` and that holds `units` 4-row units (aligned n
    // only; ragged n fetches in the epilogue).  Nothing is requested when nothing is wanted.
    __device__ __forceinline__ Pre prefetch(int row0, int units, bool wanted) const {
        Pre p;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) p.sb[rt] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < MT * RT; ++u) p.d[u] = v2i{0, 0};
        if (wanted && want_pre) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const int ul = SWIGLU ? lg : 4 * rt + lg;                        // this lane's unit of the tile
                const int n0 = row0 + 4 * ul + (SWIGLU ? rt * (a.n >> 1) : 0);  // its first weight row (= scale channel)
                const bool ok = ul < units && n0 < a.n;
                p.sb[rt] = __builtin_amdgcn_raw_buffer_load_b128(sb_rsrc, (per_channel && ok) ? n0 * 4 : (int)kOutOfRange, 0, 0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    p.d[mt * RT + rt] = __builtin_amdgcn_raw_buffer_load_b64(base_rsrc, (accumulate && ok && 16 * mt + li < a.m) ? (int)(((uint32_t)(16 * mt + li) * (uint32_t)a.n + (uint32_t)n0) * 2u) : (int)kOutOfRange, 0, 0);
            }
        }
        return p;
    }

    // scale, add D (accumulate mode), round once, store: acc[mt * RT + rt]
    __device__ __forceinline__ void store(int row0, int units, const v4f (&acc)[MT * RT], const Pre& pre) const {
        if constexpr (SWIGLU) {
            // acc[mt * RT] = gate, acc[mt * RT + 1] = up of output columns n0 .. n0+3 of activation tile mt.  The unfused chain stores
            // both projections in the 16-bit dtype between its two kernels: round them the same way before the activation.
            const int n0 = row0 + 4 * lg;
            const v4f sbg = __builtin_bit_cast(v4f, pre.sb[0]), sbu = __builtin_bit_cast(v4f, pre.sb[RT - 1]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const float sa = sa_mt[mt];
                const int arow = 16 * mt + li;
                float y[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float g = acc[mt * RT][v] * (sa * (per_channel ? sbg[v] : 1.0f));
                    float u = acc[mt * RT + RT - 1][v] * (sa * (per_channel ? sbu[v] : 1.0f));
                    g = bf16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(g)) : load16<HFRK_F16>(store16<HFRK_F16>(g));
                    u = bf16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(u)) : load16<HFRK_F16>(store16<HFRK_F16>(u));
                    y[v] = silu_mul(g, u, inv_out_scale);
                }
                uint32_t packed = cvt_pk_fp8(y[0], y[1], 0u, false);
                packed = cvt_pk_fp8(y[2], y[3], packed, true);
                const bool live = arow < a.m && lg < units && n0 < n_out;
                __builtin_amdgcn_raw_buffer_store_b32((int)packed, d_rsrc, live ? (int)((uint32_t)arow * (uint32_t)n_out + (uint32_t)n0) : (int)kOutOfRange, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < MT * RT; ++u) {
            const int mt = u / RT, rt = u % RT;
            const int arow = 16 * mt + li;  // activation row = row of D
            const float sa = sa_mt[mt];
            const int ul = 4 * rt + lg;
            const int n0 = row0 + 4 * ul;
            const bool live = arow < a.m && ul < units && n0 < a.n;
            const uint32_t d_off = ((uint32_t)arow * (uint32_t)a.n + (uint32_t)n0) * 2u;
            if (vec) {
                const v4f sb = __builtin_bit_cast(v4f, pre.sb[rt]);
                const uint32_t d0 = (uint32_t)pre.d[u][0], d1 = (uint32_t)pre.d[u][1];
                float r[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) r[v] = acc[u][v] * (per_channel ? sa * sb[v] : sa);
                if (accumulate) {
                    if (bf16) {
                        r[0] += __uint_as_float(d0 << 16); r[1] += __uint_as_float(d0 & 0xffff0000u);
                        r[2] += __uint_as_float(d1 << 16); r[3] += __uint_as_float(d1 & 0xffff0000u);
                    } else {
                        r[0] += f16_bits_to_float((uint16_t)d0); r[1] += f16_bits_to_float((uint16_t)(d0 >> 16));
                        r[2] += f16_bits_to_float((uint16_t)d1); r[3] += f16_bits_to_float((uint16_t)(d1 >> 16));
                    }
                }
                const v2i packed = {(int)pack16(r[0], r[1], bf16), (int)pack16(r[2], r[3], bf16)};
                __builtin_amdgcn_raw_buffer_store_b64(packed, d_rsrc, live ? (int)d_off : (int)kOutOfRange, 0, 0);
            } else {
                // ragged n: 2-byte accesses whose out-of-range offsets mask the columns beyond n
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint32_t off = (live && n0 + v < a.n) ? d_off + 2u * v : kOutOfRange;
                    const uint32_t old = accumulate ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(base_rsrc, (int)off, 0, 0) : 0u;
                    const float sbv = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sb_rsrc, (live && per_channel && n0 + v < a.n) ? (n0 + v) * 4 : (int)kOutOfRange, 0, 0));
                    float r = acc[u][v] * (per_channel ? sa * sbv : sa);
                    if (accumulate) r += bf16 ? bf16_bits_to_float((uint16_t)old) : f16_bits_to_float((uint16_t)old);
                    __builtin_amdgcn_raw_buffer_store_b16((short)(pack16(r, 0.f, bf16) & 0xffffu), d_rsrc, (int)off, 0, 0);
                }
            }
        }
    }
};

}  // namespace hfrk
