// FP8 skinny GEMM, m <= 16 (up to 32 with a second activation tile), weights of at least a few rows per workgroup: the
// row-split wave-stream kernel.
//
// Every workgroup owns a contiguous band of weight rows and all of K for them, so no sum ever crosses workgroups: there
// is no workspace, no arrival counter and no memory round trip after the weight stream ends.  The weight rows are dealt
// out in units of 4 rows (what one 16-byte load instruction of a wave covers: 4 rows x 256 bytes), `rows_q` units per
// workgroup and one more for the first `rows_r`; a band is cut into tiles of at most 4*RT units of nearly equal height
// (RT = 1 or 2 matrix-core tiles of 16 rows), e.g. 40 rows = 16 + 12 + 12.  Loads of a short tile's missing units are
// out of the buffer's range and cost no traffic.  Inside the workgroup the sequence of chunks (tile-major, K fastest;
// a chunk is one tile x 256 K-bytes) is split evenly over the 8 waves, each wave streams its run exactly like the
// wave-stream kernel of skinny_gemm_stream.hip (private swizzled LDS tiles, v_mfma_f32_16x16x128_f8f6f4, the next
// chunk requested as soon as the registers are free).
//
// A launch of this kind lives 5-70 us and a lone wave retires one instruction every 2-4 ns, so what is not streaming is
// instruction count on the critical path.  Two places matter and are kept short:
//  * before the first request: the partition is a handful of scalar multiplies (the tile geometry of both band heights
//    and the reciprocal of the chunk count come from the host), and everything the end of the kernel will need -- which
//    wave finishes which tile, whose partial sums it adds, where the results go, the old D values and channel scales --
//    is worked out after the first request, while it is in flight;
//  * after the last matrix instruction: a wave whose run starts inside a tile leaves its partial 16x16 tile in LDS, one
//    barrier, and the wave whose run holds the tile's first chunk adds the partials of the waves after it (a
//    precomputed bit mask says which), scales, rounds once and stores.  Each wave finishes at most one tile there.
// Sums are added in wave order: results are bit-reproducible.
//
// Two things the host decides per launch: where in k a workgroup starts (rotated by its index when all waves of the launch
// would otherwise read the same offset within 4 KB at every moment, GemmArgs::k_rotate), and how many workgroups there are
// (the planner in skinny_gemm_plan.hip: whole 16-row tiles where a grid of 224..256 gives them, twice the workgroups for short
// bands at up to 4 rows, no bands of exactly 512 KB).
//
// Replaces, for these shapes, the reference's csrc/op_src/skinny_gemm/skinny_gemm_kernel.cu:6-79 with its producers and
// consumers (producers/n_full_tiles.cu:4-127, consumers/mfma_16x16x32_consumer.cu:1-168,
// consumers/smfma_16x16x64_consumer.cu:1-158).
//
// This header holds the kernel template and its launcher; skinny_gemm_rows.hip instantiates it for row-major weights dealt
// out in 4-row units, skinny_gemm_rows_tiled.hip for bands of whole 16-row tiles in either weight layout.
#pragma once
#include "skinny_gemm_rows_epilogue.h"

namespace hfrk {

// MA = ceil(m/4): 16-byte activation loads per lane and chunk (rows 4t .. 4t+3), RT = 16-row matrix tiles per chunk.
// MA = 6 or 8 (17..32 rows, RT = 2): the activation rows fill two 16-row tiles, and every weight operand read from LDS
// feeds one matrix instruction per activation tile.
// SWIGLU: the weight is a gate_up projection (gate rows [0, n/2), up rows [n/2, n)).  Bands, units and tiles then count
// output columns (n/2 of them); a chunk pairs up to 16 gate rows with the up rows of the same columns (RT = 2: the gate
// tile and the up tile), and the epilogue stores e4m3fn(silu(gate) * up / out_scale) into D [m, n/2] instead of the two
// 16-bit projections -- the SwiGLU kernel of csrc/op_src/swiglu/swiglu_vectorized.cu:27-97 as the GEMM's epilogue.
// RMS: the residual RMSNorm that feeds the projection runs as the kernel's prologue (the reference launches it as a
// kernel of its own, hf_rocm_kernels/combined_ops/llama_mlp.py:23-33, csrc/op_src/residual_rms/residual_rms_vectorized.cu:13-172).
// Every workgroup adds input and residual, reduces the sums of squares of all rows and writes the normalised, quantised
// rows [4*MA, k] into its own LDS, in the order the matrix cores read them; the loop then takes the activation operands
// from there and loads nothing but weights.  Thread t owns the 16-byte pieces t and t + 512 of every row, the partial
// sums are added in the stand-alone kernel's order, and both use the same per-piece functions: the activations are
// bit-identical to residual_rms's.  Workgroup r stores row r of the summed residual (to a buffer of its own: every
// workgroup reads the old residual, so it cannot be updated in place).  k = 4096 or 8192, up to 8 rows.
// LAYOUT: how the weight rows are dealt out and read.
//   kRowsUnits   row-major weights, bands of any number of 4-row units, cut into tiles of nearly equal height (above).
//   kRowsTiles   row-major weights, bands of whole 16-row tiles: `rows_q` / `rows_r` count tiles, and a band is cut into
//                chunks of RT tiles each, a last one of fewer when the count is odd.
//   kRowsPacked  the same bands read from the packed load format (pack_weight.hip: chunk (tile, kc) is 4 KB at
//                (tile * k/256 + kc) * 4096, already in matrix-core operand order): four 1 KB-contiguous loads per tile
//                whose registers are the operands, no pass through LDS for the weights.  Chunk sequence, runs per wave,
//                operands and order of every sum are those of kRowsTiles: the two give the same bits.
enum { kRowsUnits = 0, kRowsTiles = 1, kRowsPacked = 2 };
template <int MA, int RT, bool SWIGLU, bool RMS, int LAYOUT = kRowsUnits>
__global__ void __launch_bounds__(kGemmThreads) skinny_gemm_rows_kernel(const GemmArgs a) {
    constexpr bool TILED = LAYOUT != kRowsUnits, PACKED = LAYOUT == kRowsPacked;
    static_assert(!(TILED && RMS), "the RMSNorm prologue exists for row-major weights dealt out in 4-row units");
    constexpr int PT = SWIGLU ? 4 : 4 * RT;  // 4-row units a chunk can hold (SwiGLU: 16 output columns, their gate and their up rows)
    static_assert(!SWIGLU || RT == 2, "the SwiGLU epilogue pairs one gate tile with one up tile");
    static_assert(!RMS || MA <= 2, "the RMSNorm prologue keeps every row in registers: up to 8 rows");
    constexpr int MT = (MA + 3) / 4;  // 16-row activation tiles: 2 from 17 rows on (two matrix tiles per chunk, either epilogue)
    static_assert(MT == 1 || (MT == 2 && RT == 2 && !RMS), "above 16 rows: two weight tiles per chunk, no RMSNorm prologue");
    constexpr uint32_t kOutOfRange = 0x80000000u;
    constexpr int kWaveLds = (RMS ? RT : RT + MT) * kTileBytes;  // RT weight tiles, MT activation tiles (RMS: rows staged once instead)
    constexpr int R = 4 * MA;                                  // activation rows the MA loads (or the staged block) hold
    constexpr int kSlotStride = kWaveLds / 16;       // in v4f

    extern __shared__ __align__(16) uint8_t lds[];
    // A wave's partial sums (MT x RT x 64 lanes x 16 bytes) go to the start of its own weight tiles, which are dead by then.
    v4f* const slots = reinterpret_cast<v4f*>(lds);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;

    // ---- this workgroup's band of rows and this wave's run of chunks -----------------------------------------------
    const int G = a.grid;
    const int b = blockIdx.x;
    const int g = ((G & 7) == 0) ? (b & 7) * (G >> 3) + (b >> 3) : b;  // XCD x owns logical ids [x*G/8, (x+1)*G/8)
    const bool tall = g < a.rows_r;                                    // one unit (TILED: one 16-row tile) more than the others
    const int u0 = (g * a.rows_q + min(g, a.rows_r)) * (TILED ? 4 : 1);  // first 4-row unit of the band
    const int T = tall ? a.tiles_a : a.tiles_b;                        // tiles (chunks per 256 bytes of k) of the band
    const int ubase = tall ? a.base_a : a.base_b;                      // units per tile, the first `uextra` tiles one more
    const int uextra = tall ? a.extra_a : a.extra_b;
    const int band_units = 4 * (a.rows_q + (tall ? 1 : 0));            // TILED: the band's height in units
    // height in units and first row of tile t of the band
    auto units_of = [&](int t) __attribute__((always_inline)) { return TILED ? min(PT, band_units - PT * t) : ubase + (t < uextra ? 1 : 0); };
    auto row0_of = [&](int t) __attribute__((always_inline)) { return TILED ? 4 * (u0 + PT * t) : 4 * (u0 + t * ubase + min(t, uextra)); };
    const int KC = a.slabs;                                            // 256-byte chunks per tile
    const int TC = T * KC;
    const int i0 = (wv * TC) >> 3, i1 = ((wv + 1) * TC) >> 3;          // chunks [i0, i1) of the band, tile-major
    const int count = i1 - i0;
    int tile = (int)__umulhi((uint32_t)i0, a.kc_magic);               // i0 / KC
    int kc = i0 - tile * KC;

    // ---- first request, as early as possible ---------------------------------------------------------------------
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.B, PACKED ? (uint32_t)((a.n + 15) >> 4) * (uint32_t)KC * (uint32_t)kTileBytes
                                                                : (uint32_t)(a.n - 1) * (uint32_t)a.b_stride + (uint32_t)a.k);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a.A, (uint32_t)a.m * (uint32_t)a.k);
    const uint32_t w_lane_off = (uint32_t)lg * (uint32_t)a.b_stride + (uint32_t)li * 16u;
    const uint32_t a_lane_off = (uint32_t)lg * (uint32_t)a.k + (uint32_t)li * 16u;
    v4i wq[4 * RT], aq[MA];
    int itile = tile, ikc = kc;                                        // chunk being requested
    // Where the host asks for it, the point in k at which a workgroup starts is rotated by its index: chunk kc of a tile
    // reads K bytes ((kc + g) mod KC) * 256.  Every tile still sums all of k once, but the 2048 waves of a launch, which
    // advance in step, no longer ask for the same offset within their rows at the same moment (see k_rotate).
    const int rot = a.k_rotate ? g - (int)__umulhi((uint32_t)g, a.kc_magic) * KC : 0;  // g mod KC
    int ikr = kc + rot - (kc + rot >= KC ? KC : 0);                    // its rotated position in k
    int iunits = units_of(itile);                                      // its tile's height in units
    int irow0 = row0_of(itile);                                        // its tile's first row
    uint32_t irow_off = (uint32_t)irow0 * (uint32_t)a.b_stride;
    // The offsets of a chunk's loads are worked out one chunk ahead (while the loads before them are in flight): between the
    // arrival of a chunk and the request for the next one a wave has nothing in flight, so only the copy to LDS and the load
    // instructions themselves stand there (about 30 instructions fewer per chunk; 0.2-0.4 us on a 10-20 us launch).
    uint32_t a_voff[MA], w_voff[4 * RT];
    auto chunk_offsets = [&]() __attribute__((always_inline)) {
        const uint32_t kbyte = (uint32_t)ikr * 256u;
#pragma unroll
        for (int t = 0; t < MA; ++t) a_voff[t] = a_lane_off + kbyte + (uint32_t)(4 * t) * (uint32_t)a.k;
        if constexpr (PACKED) {
            // load t = 16-byte piece t % 4 of every lane's operand of 16-row tile t / 4 of the chunk (SWIGLU: 0 = the gate tile,
            // 1 = the up tile of the same columns, n/32 tiles further down); a tile the chunk does not have reads as zero
#pragma unroll
            for (int t = 0; t < 4 * RT; ++t) {
                const uint32_t tile16 = (uint32_t)(irow0 >> 4) + (SWIGLU ? (uint32_t)(t / 4) * (uint32_t)(a.n >> 5) : (uint32_t)(t / 4));
                const bool have = SWIGLU || 4 * (t / 4) < iunits;
                w_voff[t] = have ? (tile16 * (uint32_t)KC + (uint32_t)ikr) * (uint32_t)kTileBytes + (uint32_t)(t % 4) * 1024u + (uint32_t)lane * 16u
                                 : kOutOfRange;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4 * RT; ++t) {  // unit t of the tile; a unit the tile does not have reads as zero, without traffic
                // SWIGLU: loads 0..3 fetch the tile's gate rows, loads 4..7 the up rows of the same columns, n/2 rows further down
                const int unit = SWIGLU ? t % 4 : t;
                const uint32_t row = SWIGLU ? (uint32_t)(4 * unit + (t / 4) * (a.n >> 1)) : (uint32_t)(4 * t);
                const uint32_t off = unit < iunits ? irow_off + kbyte + row * (uint32_t)a.b_stride : kOutOfRange;
                w_voff[t] = w_lane_off + off;
            }
        }
    };
    auto issue_chunk = [&]() __attribute__((always_inline)) {
        if constexpr (!RMS) {
#pragma unroll
            for (int t = 0; t < MA; ++t) aq[t] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)a_voff[t], 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 4 * RT; ++t) wq[t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)w_voff[t], 0, 2 /* nt */);
    };
    auto next_chunk = [&]() __attribute__((always_inline)) {
        if (++ikr == KC) ikr = 0;
        if (++ikc == KC) {
            ikc = 0;
            irow0 += 4 * iunits;
            irow_off = (uint32_t)irow0 * (uint32_t)a.b_stride;
            ++itile;
            iunits = units_of(itile);
        }
    };
    chunk_offsets();
    if (count > 0) issue_chunk();
    __builtin_amdgcn_sched_barrier(0);  // keep the set-up below behind the first request

    // ---- the rest of the set-up, while the first chunk is on its way -------------------------------------------------
    // everything the end of the kernel needs to turn a sum into output: buffer resources, scales, dtype (skinny_gemm_rows_epilogue.h)
    const RowsEpilogue<MT, RT, SWIGLU> epi(a, lane);
    using Pre = typename RowsEpilogue<MT, RT, SWIGLU>::Pre;

    uint8_t* const tw = lds + wv * kWaveLds;  // this wave's RT weight tiles, then its activation tile(s)
    uint8_t* const ta = tw + RT * kTileBytes;
    // RMS: behind all weight tiles the partial sums of squares [R][8 waves], then the staged rows.  16-byte piece p of row r
    // (p = kc*16 + h*8 + lg*2 + half: K chunk, 128-byte half, lane group, low / high 16 bytes of the lane's 32) lies at
    // ((((kc*2 + h)*2 + half)*4 + lg)*R + r)*16: what the lanes (lg, li < R) of one operand read fetch is contiguous.
    // Rows from m on are neither computed nor staged: what the matrix cores read there feeds output rows nobody stores.
    float* const red = reinterpret_cast<float*>(lds + kGemmWaves * kWaveLds);
    uint8_t* const stage = lds + kGemmWaves * kWaveLds + kRowsRmsRedBytes;
    if constexpr (RMS) {
        const bool rbf16 = a.rms_dtype == HFRK_BF16;
        const uint32_t row_bytes = (uint32_t)a.k * 2u;
        const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(a.rms_input, (uint32_t)a.m * row_bytes);
        const __amdgpu_buffer_rsrc_t res_rsrc = make_rsrc(a.rms_residual, (uint32_t)a.m * row_bytes);
        const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(a.rms_residual_out, (uint32_t)a.m * row_bytes);
        const __amdgpu_buffer_rsrc_t nw_rsrc = make_rsrc(a.rms_weight, row_bytes);
        const bool two = a.k > 4096;  // pieces t and t + 512 of a row (k = 8192), else piece t only
        uint4 z[R][2], wreg[2];
        float ssq[R];
#pragma unroll
        for (int it = 0; it < 2; ++it)
            wreg[it] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(nw_rsrc, (it == 0 || two) ? (tid + it * kGemmThreads) * 16 : (int)kOutOfRange, 0, 0));
        // every row is requested before the first is used: one memory latency for the block, not one per row (the stores
        // of the summed residual below would otherwise keep the next row's loads behind them)
        uint4 xin[R][2], xres[R][2];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= a.m) continue;  // uniform
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const int off = (it == 0 || two) ? (int)((uint32_t)r * row_bytes + (uint32_t)(tid + it * kGemmThreads) * 16u) : (int)kOutOfRange;
                xin[r][it] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, off, 0, 0));
                xres[r][it] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(res_rsrc, off, 0, 0));
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            ssq[r] = 0.f;
            if (r >= a.m) continue;
#pragma unroll
            for (int it = 0; it < 2; ++it)
                z[r][it] = rbf16 ? rms_add_square<HFRK_BF16>(xin[r][it], xres[r][it], ssq[r]) : rms_add_square<HFRK_F16>(xin[r][it], xres[r][it], ssq[r]);
        }
        if (g < a.m) {  // workgroup g stores row g of the summed residual
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r != g) continue;
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int off = (it == 0 || two) ? (int)((uint32_t)r * row_bytes + (uint32_t)(tid + it * kGemmThreads) * 16u) : (int)kOutOfRange;
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, z[r][it]), out_rsrc, off, 0, 0);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= a.m) continue;
            const float s = wave_sum(ssq[r]);
            if (lane == 0) red[r * kGemmWaves + wv] = s;
        }
        __syncthreads();
        const float inv_scale = 1.f / a.rms_act_scale[0];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= a.m) continue;
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < kGemmWaves; ++w) total += red[r * kGemmWaves + w];
            const float norm = rsqrtf(total / (float)a.k + a.rms_epsilon);
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                if (it == 1 && !two) break;
                const uint2 q = rbf16 ? rms_scale_to_fp8<HFRK_BF16>(z[r][it], wreg[it], norm, inv_scale)
                                      : rms_scale_to_fp8<HFRK_F16>(z[r][it], wreg[it], norm, inv_scale);
                const int v = tid + it * kGemmThreads;  // 8 K-bytes v*8 .. v*8+8: half of 16-byte piece p = v / 2
                const int p = v >> 1;
                const int chunk = p >> 4, h = (p >> 3) & 1, grp = (p >> 1) & 3, half = p & 1;
                *reinterpret_cast<uint2*>(stage + ((((chunk * 2 + h) * 2 + half) * 4 + grp) * R + r) * 16 + (v & 1) * 8) = q;
            }
        }
        __syncthreads();
    }
    int wr_off[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int row = 4 * t + lg;
        wr_off[t] = row * 256 + ((li ^ row) << 4);
    }
    int rd_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) rd_off[h] = li * 256 + ((((8 * h + 2 * lg) ^ li) & 15) << 4);

    auto prefetch = [&](int row0, int units, bool wanted) __attribute__((always_inline)) { return epi.prefetch(row0, units, wanted); };
    auto epilogue = [&](int row0, int units, const v4f (&acc)[MT * RT], const Pre& pre) __attribute__((always_inline)) { epi.store(row0, units, acc, pre); };

    // ---- what the end of the kernel will do, decided now ----------------------------------------------------------------
    // A run that starts inside a tile (kb0 != 0) hands the partial sum of that tile over; a wave without chunks hands over
    // zeros, so that the finishing wave can add by position alone.  The wave whose run holds a tile's first chunk finishes
    // it: in the loop when the tile also ends inside the run, after the barrier when it ends in a later wave's run.
    const int tile_h = tile, kb0 = kc;
    const bool hand_over = count == 0 || kb0 != 0;
    const int jl = (int)__umulhi((uint32_t)i1, a.kc_magic);  // the tile the run ends in
    const int ke = i1 - jl * KC;                             // its chunks before the end of the run
    const bool finisher = count > 0 && ke != 0 && jl * KC >= i0;
    const int units_l = units_of(jl);
    const int row0_l = row0_of(jl);
    uint32_t addmask = 0;  // bit j: wave j's run starts before that tile ends, its partial belongs to it
    {
        const int e = (jl + 1) * KC;
#pragma unroll
        for (int j = 1; j < kGemmWaves; ++j)
            if (j > wv && ((j * TC) >> 3) < e) addmask |= 1u << j;
    }
    // The D values and scales of that tile are asked for behind the wave's last weight request, not here: the wait for a
    // chunk also waits for every load issued since, so a request placed here stands in front of the first chunk's use
    // (accumulate mode, M = 1 / 8: 4096 x 4096 5.11 / 5.38 -> 4.98 / 5.19 us, 28672 x 4096 20.1 / 20.4 -> 19.6 / 20.0,
    // 4096 x 14336 11.0 -> 10.85).  With two workgroups per CU it is the other way round (6144 x 4096 on 512 workgroups:
    // 6.04 -> 6.19), so there the request stays here.
    const bool late_pre = G <= kNumCU && count > 1;
    Pre pre_l = prefetch(row0_l, units_l, finisher && !late_pre);

    // ---- streaming loop ---------------------------------------------------------------------------------------------
    int kr = ikr;                                            // rotated k position of the chunk being multiplied
    int units = iunits;                                      // geometry of the tile being multiplied
    int row0 = row0_of(tile);
    Pre pre_next = prefetch(row0, units, count > 0 && kc == KC - 1 && !(kb0 != 0)), pre_cur;
    v4f acc[MT * RT], part_h[MT * RT];  // [activation tile][weight tile]
#pragma unroll
    for (int u = 0; u < MT * RT; ++u) acc[u] = part_h[u] = v4f{0.f, 0.f, 0.f, 0.f};
    if (count > 1) {  // the second chunk's offsets
        next_chunk();
        chunk_offsets();
    }
    for (int i = 0; i < count; ++i) {
        if constexpr (!RMS) {
#pragma unroll
            for (int t = 0; t < MA; ++t) *reinterpret_cast<v4i*>(ta + (t / 4) * kTileBytes + wr_off[t % 4]) = aq[t];
        }
        v4i wcur[4 * RT];  // PACKED: the chunk's operands, out of the way of the next request
#pragma unroll
        for (int t = 0; t < 4 * RT; ++t) {
            if constexpr (PACKED) wcur[t] = wq[t];
            else *reinterpret_cast<v4i*>(tw + (t / 4) * kTileBytes + wr_off[t % 4]) = wq[t];
        }
        pre_cur = pre_next;
        if (i + 1 < count) {  // registers are free again: request the next chunk before the LDS reads and MFMAs
            issue_chunk();
            // the chunk that ends a tile this wave finishes in the loop brings the tile's D along
            pre_next = prefetch(irow0, iunits, ikc == KC - 1 && !(itile == tile_h && kb0 != 0));
            if (i + 2 == count && finisher && late_pre) pre_l = prefetch(row0_l, units_l, true);
            if (i + 2 < count) {  // and the offsets of the one after it, for the next turn
                next_chunk();
                chunk_offsets();
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // every operand of the chunk is requested from LDS before the first MFMA
        v8i wop[2][RT], aop[2][MT];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                v4i lo, hi;
                if constexpr (PACKED) {
                    lo = wcur[4 * rt + 2 * h];
                    hi = wcur[4 * rt + 2 * h + 1];
                } else {
                    lo = *reinterpret_cast<const v4i*>(tw + rt * kTileBytes + rd_off[h]);
                    hi = *reinterpret_cast<const v4i*>(tw + rt * kTileBytes + (rd_off[h] ^ 16));
                }
                wop[h][rt] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
            v4i lo, hi;
            if constexpr (RMS) {
                // lanes li >= R read row R - 1 again: they feed output rows that are never stored
                const uint8_t* const piece = stage + ((((kr * 2 + h) * 2) * 4 + lg) * R + min(li, R - 1)) * 16;
                lo = *reinterpret_cast<const v4i*>(piece);
                hi = *reinterpret_cast<const v4i*>(piece + 4 * R * 16);
            } else {
                lo = *reinterpret_cast<const v4i*>(ta + mt * kTileBytes + rd_off[h]);
                hi = *reinterpret_cast<const v4i*>(ta + mt * kTileBytes + (rd_off[h] ^ 16));
            }
            aop[h][mt] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the requests above ahead of the MFMAs below
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int u = 0; u < MT * RT; ++u)
                acc[u] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wop[h][u % RT], aop[h][u / RT], acc[u], 0, 0, 0, 0, 0, 0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if constexpr (RMS) {
            if (++kr == KC) kr = 0;
        }
        if (++kc == KC) {  // a tile ends inside this wave's run
            if (tile == tile_h && kb0 != 0) {  // its first chunks belong to an earlier wave
#pragma unroll
                for (int u = 0; u < MT * RT; ++u) part_h[u] = acc[u];
            } else {
                epilogue(row0, units, acc, pre_cur);  // all of it was ours
            }
#pragma unroll
            for (int u = 0; u < MT * RT; ++u) acc[u] = v4f{0.f, 0.f, 0.f, 0.f};
            kc = 0;
            row0 += 4 * units;
            ++tile;
            units = units_of(tile);
        }
    }
    // a run that lies inside one tile that began in an earlier wave: everything it has is that tile's partial sum
    if (count > 0 && kc != 0 && tile == tile_h && kb0 != 0) {
#pragma unroll
        for (int u = 0; u < MT * RT; ++u) part_h[u] = acc[u];
    }

    // ---- combine the partial tiles of this workgroup ----------------------------------------------------------------
    // Every wave leaves a partial sum (zeros when it has none to hand over), so that the finishing wave can read all seven
    // slots at once and add each with a factor of one or zero: no select, no branch, exact.
#pragma unroll
    for (int u = 0; u < MT * RT; ++u) slots[wv * kSlotStride + u * 64 + lane] = hand_over ? part_h[u] : v4f{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    if (!finisher) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {  // one activation tile at a time: seven waves' partials of it in registers
        v4f other[kGemmWaves][RT];
#pragma unroll
        for (int j = 1; j < kGemmWaves; ++j)
#pragma unroll
            for (int u = 0; u < RT; ++u) other[j][u] = slots[j * kSlotStride + (mt * RT + u) * 64 + lane];
#pragma unroll
        for (int j = 1; j < kGemmWaves; ++j) {
            const float f = (addmask >> j) & 1u ? 1.0f : 0.0f;
#pragma unroll
            for (int u = 0; u < RT; ++u)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[mt * RT + u][v] = __builtin_fmaf(other[j][u][v], f, acc[mt * RT + u][v]);
        }
    }
    epilogue(row0_l, units_l, acc, pre_l);
}

template <int MA, int RT, bool SWIGLU, bool RMS, int LAYOUT = kRowsUnits>
static int launch_rows_one(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = skinny_gemm_rows_kernel<MA, RT, SWIGLU, RMS, LAYOUT>;
    static bool attr_done[kMaxDevices] = {};
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev >= 0 && dev < kMaxDevices && !attr_done[dev]) {
        HFRK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
        attr_done[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3(args.grid), dim3(kGemmThreads), lds_bytes, stream, args);
    HFRK_HIP_TRY(hipGetLastError());
    return HFRK_SUCCESS;
}

}  // namespace hfrk
