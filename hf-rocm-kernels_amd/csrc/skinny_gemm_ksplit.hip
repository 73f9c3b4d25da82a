// FP8 skinny GEMM, 17 <= m <= 64 (usable from 1): the 8 waves of a workgroup split K, the activations live in
// registers, the weights stream past them.
//
// K is cut into windows of 8*KW bytes (KW = 256, 512 or -- up to 32 rows -- 1024 per wave).  A workgroup works inside one window at a time:
// wave w holds the activation rows for its KW bytes of the window as MFMA operands in VGPRs (16*MT rows x KW bytes,
// loaded once per window) and, for every 16-row weight tile the workgroup owns, streams that tile's 16 x KW bytes
// (16-byte `nt` loads, 4 rows x 256 contiguous bytes per instruction), turns them into operand layout through a
// private swizzled LDS tile and issues MT * KW/128 v_mfma_f32_16x16x128_f8f6f4.  No activation byte is read in the
// loop, from L2 or from LDS: what the workgroup kernel spends on re-reading activation tiles from LDS (4 bytes per
// weight byte at 64 rows) is gone, which is what this decomposition is for.
//
// The 8 partial 16x(16*MT) tiles of a unit are summed through LDS: everyone writes, one barrier, waves 0..MT-1 each
// add the eight partials of one 16x16 tile in wave order and finish it (double-buffered, so the others are already
// streaming the next tile).  With more than one window per row tile the finished window-partials go through the
// workspace with a per-tile arrival counter, and the last arriver adds them in window order: sums are
// bit-reproducible.  Units are numbered window-major, so a workgroup's contiguous range stays inside one window
// (the activations are reloaded at most once or twice per launch).
//
// Replaces, for these m, the reference's csrc/op_src/skinny_gemm/skinny_gemm_kernel.cu:6-79 with its producers and
// consumers (producers/n_full_tiles.cu:4-127, producers/4_half_tiles.cu:5-113,
// consumers/mfma_16x16x32_consumer.cu:1-168).
#include "skinny_gemm_args.h"

namespace hfrk {

// PACKED: the weight is in the pre-packed layout (pack_weight.hip), chunk (tile, kc) at (tile * k/256 + kc) * 4096 in
// MFMA operand order: a wave's piece of a unit is KW/256 contiguous chunks, the loaded registers are the operands,
// and each chunk of the next unit is requested as soon as the MFMAs of the current one have taken its registers.
// SWIGLU: the weight is a gate_up projection (gate rows [0, n/2), up rows [n/2, n)) and one window covers K.  A unit
// is then a tile of 16 output columns, worked as two passes of the loop body: the gate tile t, whose finished sums the
// waves 0..MT-1 keep in registers, then the up tile t + n/32, after which they store
// e4m3fn(silu(gate) * up / out_scale) into D [m, n/2] instead of the two 16-bit projections -- the SwiGLU kernel of
// csrc/op_src/swiglu/swiglu_vectorized.cu:27-97 as the GEMM's epilogue, here for 17..64 rows.
template <int MT, int KW, bool PACKED, bool SWIGLU>
__global__ void __launch_bounds__(kGemmThreads) skinny_gemm_ksplit_kernel(const GemmArgs a) {
    constexpr uint32_t kOutOfRange = 0x80000000u;
    constexpr int PASSES = SWIGLU ? 2 : 1;
    constexpr int kCoherent = 17;     // sc0 | sc1
    constexpr int KCH = KW / 256;     // 256-byte column chunks of a wave's weight piece
    constexpr int KST = KW / 128;     // MFMA K steps per unit
    constexpr int kTileLds = kGemmWaves * KCH * kTileBytes;  // private transposition tiles
    constexpr int kRedBuf = kGemmWaves * MT * 64;            // v4f per reduction buffer

    extern __shared__ __align__(16) uint8_t lds[];
    v4f* const red = reinterpret_cast<v4f*>(lds + kTileLds);  // [2][wave][mt][lane]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;

    // ---- this workgroup's units (u = window * T + tile; 32-bit, the host checks (grid + 1) * units < 2^31) ---------
    const int G = a.grid;
    const int T = a.panels;  // 16-row tiles (SWIGLU: tiles of 16 output columns, T = n / 32)
    const int S = a.slabs;   // windows (SWIGLU: 1)
    const int b = blockIdx.x;
    const int g = ((G & 7) == 0) ? (b & 7) * (G >> 3) + (b >> 3) : b;  // XCD x owns logical ids [x*G/8, (x+1)*G/8)
    const uint32_t uq = (uint32_t)a.chunks_q, ur = (uint32_t)a.chunks_r;  // units / G, units % G
    const uint32_t u0 = (uint32_t)g * uq + min((uint32_t)g, ur);
    const int count = (int)(uq + ((uint32_t)g < ur ? 1u : 0u));
    int win = (int)(u0 / (uint32_t)T);
    int tile = (int)(u0 - (uint32_t)win * (uint32_t)T);

    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.B, PACKED ? (uint32_t)(PASSES * T) * (uint32_t)a.k * 16u
                                                                : (uint32_t)(a.n - 1) * (uint32_t)a.b_stride + (uint32_t)a.k);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a.A, (uint32_t)a.m * (uint32_t)a.k);
    const __amdgpu_buffer_rsrc_t ws_rsrc = make_rsrc(a.ws, a.ws_bytes);
    const int n_out = SWIGLU ? (a.n >> 1) : a.n;  // columns of D
    const __amdgpu_buffer_rsrc_t d_rsrc = make_rsrc(a.D, (uint32_t)a.m * (uint32_t)n_out * (SWIGLU ? 1u : 2u));
    const __amdgpu_buffer_rsrc_t base_rsrc = make_rsrc(a.base, a.base ? (uint32_t)a.m * (uint32_t)a.n * 2u : 0u);
    const __amdgpu_buffer_rsrc_t sb_rsrc = make_rsrc(a.scale_b, a.scale_b ? (uint32_t)a.n * 4u : 0u);
    const bool accumulate = !SWIGLU && a.base != nullptr;
    const bool per_channel = a.scale_b && a.sb_stride;
    const bool vec = SWIGLU || (a.n & 3) == 0;

    // ---- weight stream: load t of column chunk c brings rows 4t + lg, bytes c*256 + li*16 .. +16 of the wave's piece --
    const uint32_t w_lane_off = (uint32_t)lg * (uint32_t)a.b_stride + (uint32_t)wv * KW + (uint32_t)li * 16u;
    v4i wq[KCH][4];
    int itile = tile, iwin = win;  // unit being requested
    int ipass = 0;                 // SWIGLU: 0 = its gate tile, 1 = its up tile
    // column chunk c of the wave's piece of unit (itile, iwin); `base` is the unit's row-major offset
    auto issue_chunk = [&](int c, uint32_t base) __attribute__((always_inline)) {
        if constexpr (PACKED) {
            const uint32_t chunk = (uint32_t)(itile + ipass * T) * ((uint32_t)a.k >> 8) + ((uint32_t)iwin * 8u + (uint32_t)wv) * KCH + (uint32_t)c;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                wq[c][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)(chunk * (uint32_t)kTileBytes + (uint32_t)t * 1024u + (uint32_t)lane * 16u), 0, 2 /* nt */);
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                wq[c][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)(w_lane_off + base + (uint32_t)(4 * t) * (uint32_t)a.b_stride + (uint32_t)c * 256u), 0, 2 /* nt */);
        }
    };
    auto issue_unit = [&]() __attribute__((always_inline)) {
        const uint32_t base = (uint32_t)(itile + ipass * T) * 16u * (uint32_t)a.b_stride + (uint32_t)iwin * (8u * KW);
#pragma unroll
        for (int c = 0; c < KCH; ++c) issue_chunk(c, base);
    };
    if (count > 0) issue_unit();
    __builtin_amdgcn_sched_barrier(0);  // the first weight request goes out before anything else is set up

    uint8_t* const tw = lds + wv * KCH * kTileBytes;  // this wave's transposition tiles
    int wr_off[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int row = 4 * t + lg;
        wr_off[t] = row * 256 + ((li ^ row) << 4);
    }
    int rd_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) rd_off[h] = li * 256 + ((((8 * h + 2 * lg) ^ li) & 15) << 4);

    // ---- activations of one window, as MFMA B operands: lane (li, lg) ends up with row mt*16 + li, bytes
    // ks*128 + lg*32 .. +32 of the wave's K piece.  Loaded like the weights (4 rows x 256 contiguous bytes per
    // instruction, 16 cache lines instead of the 64 a load in operand order touches) and turned through the wave's
    // first transposition tile, which is idle whenever this runs.
    v8i areg[MT][KST];
    auto load_window = [&](int w) __attribute__((always_inline)) {
        const uint32_t kbase = (uint32_t)w * (8u * KW) + (uint32_t)wv * KW + (uint32_t)li * 16u;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int c = 0; c < KCH; ++c) {
                v4i q[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int row = mt * 16 + 4 * t + lg;  // rows >= m read as zero
                    q[t] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, row < a.m ? (int)((uint32_t)row * (uint32_t)a.k + kbase + (uint32_t)c * 256u) : (int)kOutOfRange, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) *reinterpret_cast<v4i*>(tw + wr_off[t]) = q[t];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const v4i lo = *reinterpret_cast<const v4i*>(tw + rd_off[h]);
                    const v4i hi = *reinterpret_cast<const v4i*>(tw + (rd_off[h] ^ 16));
                    areg[mt][2 * c + h] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
    };
    if (count > 0) load_window(win);

    float sa[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        sa[mt] = a.scale_a[(long)min(mt * 16 + li, a.m - 1) * a.sa_stride] * ((a.scale_b && !a.sb_stride) ? a.scale_b[0] : 1.0f);

    // scale, add base (accumulate mode), round once, store one 16x16 tile: lane holds D^T[n0 + v][mrow], v = 0..3
    auto epilogue = [&](int t, int mt, v4f acc) __attribute__((always_inline)) {
        const int n0 = t * 16 + 4 * lg;
        const int mrow = mt * 16 + li;
        const bool live = mrow < a.m && n0 < a.n;
        const uint32_t d_off = ((uint32_t)mrow * (uint32_t)a.n + (uint32_t)n0) * 2u;
        uint32_t old[4], off[4];
        v4f sb;
        if (vec) {
            sb = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(sb_rsrc, (live && per_channel) ? n0 * 4 : (int)kOutOfRange, 0, 0));
            const v2i d = __builtin_amdgcn_raw_buffer_load_b64(base_rsrc, (live && accumulate) ? (int)d_off : (int)kOutOfRange, 0, 0);
            old[0] = (uint32_t)d[0] & 0xffffu; old[1] = (uint32_t)d[0] >> 16;
            old[2] = (uint32_t)d[1] & 0xffffu; old[3] = (uint32_t)d[1] >> 16;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                off[v] = (live && n0 + v < a.n) ? d_off + 2u * v : kOutOfRange;
                old[v] = accumulate ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(base_rsrc, (int)off[v], 0, 0) : 0u;
                sb[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sb_rsrc, (live && per_channel && n0 + v < a.n) ? (n0 + v) * 4 : (int)kOutOfRange, 0, 0));
            }
        }
        const float sam = mt == 0 ? sa[0] : mt == 1 ? sa[MT > 1 ? 1 : 0] : mt == 2 ? sa[MT > 2 ? 2 : 0] : sa[MT > 3 ? 3 : 0];
        uint32_t o[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float r = acc[v] * (sam * (per_channel ? sb[v] : 1.0f));
            const float bs = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>((uint16_t)old[v]) : load16<HFRK_F16>((uint16_t)old[v]);
            const float sum = accumulate ? bs + r : r;
            o[v] = a.d_dtype == HFRK_BF16 ? store16<HFRK_BF16>(sum) : store16<HFRK_F16>(sum);
        }
        if (vec) {
            const v2i packed = {(int)(o[0] | (o[1] << 16)), (int)(o[2] | (o[3] << 16))};
            __builtin_amdgcn_raw_buffer_store_b64(packed, d_rsrc, live ? (int)d_off : (int)kOutOfRange, 0, 0);
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) __builtin_amdgcn_raw_buffer_store_b16((short)o[v], d_rsrc, (int)off[v], 0, 0);
        }
    };

    // SWIGLU: gate and up sums of output columns n0 .. n0+3 (n0 = t*16 + 4*lg) of row mt*16 + li, each rounded to the
    // 16-bit dtype the unfused chain stores between its two kernels, then silu(gate) * up / out_scale as four fp8
    float inv_out_scale = 1.0f;
    if constexpr (SWIGLU) {
        const float os = a.out_scale[0];
        inv_out_scale = os != 0.f ? 1.0f / os : 1.0f;
    }
    auto epilogue_swiglu = [&](int t, int mt, v4f gate, v4f up) __attribute__((always_inline)) {
        const int n0 = t * 16 + 4 * lg;
        const int mrow = mt * 16 + li;
        const bool live = mrow < a.m && n0 < n_out;
        const v4f sbg = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(sb_rsrc, (live && per_channel) ? n0 * 4 : (int)kOutOfRange, 0, 0));
        const v4f sbu = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(sb_rsrc, (live && per_channel) ? (n_out + n0) * 4 : (int)kOutOfRange, 0, 0));
        const float sam = mt == 0 ? sa[0] : mt == 1 ? sa[MT > 1 ? 1 : 0] : mt == 2 ? sa[MT > 2 ? 2 : 0] : sa[MT > 3 ? 3 : 0];
        float y[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float g = gate[v] * (sam * (per_channel ? sbg[v] : 1.0f));
            float u = up[v] * (sam * (per_channel ? sbu[v] : 1.0f));
            g = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(g)) : load16<HFRK_F16>(store16<HFRK_F16>(g));
            u = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(u)) : load16<HFRK_F16>(store16<HFRK_F16>(u));
            y[v] = silu_mul(g, u, inv_out_scale);
        }
        uint32_t packed = cvt_pk_fp8(y[0], y[1], 0u, false);
        packed = cvt_pk_fp8(y[2], y[3], packed, true);
        __builtin_amdgcn_raw_buffer_store_b32((int)packed, d_rsrc, live ? (int)((uint32_t)mrow * (uint32_t)n_out + (uint32_t)n0) : (int)kOutOfRange, 0, 0);
    };

    // Several windows (S > 1): a unit's share of its tile goes to the workspace and an arrival counter decides who adds
    // the shares.  Store, acknowledgement, counter round trip and the verdict are spread over two units so that none of
    // them is waited for where it was issued: the share is stored at the end of unit i, acknowledged and counted at the
    // top of unit i+1 (when nothing else of this wave is in flight), and the counter's answer is looked at after unit
    // i+1's MFMAs; only then does the last arriver add the shares and store the tile.
    // (The 1 KB-per-wave variants have no register to carry this state across units: they count and settle on the spot.)
    constexpr bool kDeferred = KW < 1024;
    int stored_tile = -1;   // share in flight, arrival not yet counted
    int counted_tile = -1;  // arrival counted, answer not yet looked at
    int ticket = 0;         // lane 0: what the counter held before this wave's arrival
    auto count_arrival = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): every lane's share acknowledged before the arrival is counted
        if (lane == 0) ticket = atomicAdd(a.counters + stored_tile * MT + wv, 1);
        counted_tile = stored_tile;
        stored_tile = -1;
    };
    auto settle = [&]() __attribute__((always_inline)) {
        const int t = counted_tile;
        counted_tile = -1;
        int last = 0;
        if (lane == 0) {
            last = ticket == S - 1;
            if (last) a.counters[t * MT + wv] = 0;  // ready for the next launch
        }
        if (__builtin_amdgcn_readfirstlane(last) == 0) return;
        v4f total = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
        for (int j0 = 0; j0 < S; j0 += 4) {
            v4i q[4];
#pragma unroll
            for (int x = 0; x < 4; ++x)  // four shares in flight; past the last window the load is out of range: zeros
                q[x] = __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, j0 + x < S ? ((((j0 + x) * T + t) * MT + wv) * 64 + lane) * 16 : (int)kOutOfRange, 0, kCoherent);
#pragma unroll
            for (int x = 0; x < 4; ++x) total += __builtin_bit_cast(v4f, q[x]);
        }
        epilogue(t, wv, total);
    };

    // ---- unit loop ----------------------------------------------------------------------------------------------------
    v4f gate_sum = v4f{0.f, 0.f, 0.f, 0.f};  // SWIGLU, waves 0..MT-1: the gate tile's sums, kept over the up tile's pass
#pragma unroll 1
    for (int i = 0; i < PASSES * count; ++i) {
        if constexpr (!PACKED) {
#pragma unroll
            for (int c = 0; c < KCH; ++c)
#pragma unroll
                for (int t = 0; t < 4; ++t) *reinterpret_cast<v4i*>(tw + c * kTileBytes + wr_off[t]) = wq[c][t];
        }
        if constexpr (kDeferred) {
            if (S > 1 && wv < MT && stored_tile >= 0) count_arrival();
        }
        const bool more = i + 1 < PASSES * count;
        bool new_window = false;
        if (more) {  // row-major: registers are free again, request the next unit before the LDS reads and MFMAs
            if (SWIGLU && ipass == 0) {
                ipass = 1;  // the same columns' up tile
            } else {
                ipass = 0;
                if (++itile == T) { itile = 0; ++iwin; new_window = true; }
            }
            if constexpr (!PACKED) issue_unit();
        }
        if constexpr (!PACKED) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        v4f acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
            // both weight operands of the column chunk are requested from LDS before its first MFMA
            v8i wop[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                v4i lo, hi;
                if constexpr (PACKED) {
                    lo = wq[c][2 * h];
                    hi = wq[c][2 * h + 1];
                } else {
                    lo = *reinterpret_cast<const v4i*>(tw + c * kTileBytes + rd_off[h]);
                    hi = *reinterpret_cast<const v4i*>(tw + c * kTileBytes + (rd_off[h] ^ 16));
                }
                wop[h] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wop[h], areg[mt][2 * c + h], acc[mt], 0, 0, 0, 0, 0, 0);
            if constexpr (PACKED) {
                if (more) issue_chunk(c, 0u);
            }
        }
        if constexpr (!PACKED) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }

        // sum the eight K pieces: buffer i & 1 (the barrier of the next unit separates its reuse from these reads)
        v4f* const rb = red + (i & 1) * kRedBuf;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) rb[(wv * MT + mt) * 64 + lane] = acc[mt];
        __syncthreads();
        if (wv < MT) {
            v4f part[kGemmWaves];
#pragma unroll
            for (int w = 0; w < kGemmWaves; ++w) part[w] = rb[(w * MT + wv) * 64 + lane];
            v4f sum = part[0];
#pragma unroll
            for (int w = 1; w < kGemmWaves; ++w) sum += part[w];
            if (S > 1) {
                if constexpr (kDeferred) {
                    if (counted_tile >= 0) settle();  // the unit before this one
                }
                // this window's share of tile (tile, wv) goes to the workspace; whoever completes the tile adds the shares
                const int slot = (win * T + tile) * MT + wv;
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, sum), ws_rsrc, (slot * 64 + lane) * 16, 0, kCoherent);
                stored_tile = tile;
                if constexpr (!kDeferred) {
                    count_arrival();
                    settle();
                }
            } else if constexpr (SWIGLU) {
                if ((i & 1) == 0) gate_sum = sum;
                else epilogue_swiglu(tile, wv, gate_sum, sum);
            } else {
                epilogue(tile, wv, sum);
            }
        }
        // advance to the unit whose weights are already on their way
        if (more) {
            tile = itile;
            if (new_window) {
                win = iwin;
                load_window(win);
            }
        }
    }
    if constexpr (kDeferred) {
        if (S > 1 && wv < MT) {  // the last unit's share
            if (stored_tile >= 0) count_arrival();
            if (counted_tile >= 0) settle();
        }
    }
}

template <int MT, int KW, bool PACKED, bool SWIGLU>
static int launch_ksplit_packing(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = skinny_gemm_ksplit_kernel<MT, KW, PACKED, SWIGLU>;
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

template <int MT, int KW>
static int launch_ksplit_one(const GemmArgs& args, bool swiglu, int lds_bytes, hipStream_t stream) {
    if constexpr (KW <= 512) {  // the SwiGLU epilogue: one window of 2048 or 4096 bytes covers K
        if (swiglu)
            return args.packed ? launch_ksplit_packing<MT, KW, true, true>(args, lds_bytes, stream)
                               : launch_ksplit_packing<MT, KW, false, true>(args, lds_bytes, stream);
    }
    if (swiglu) return HFRK_INVALID_CONFIG;
    return args.packed ? launch_ksplit_packing<MT, KW, true, false>(args, lds_bytes, stream)
                       : launch_ksplit_packing<MT, KW, false, false>(args, lds_bytes, stream);
}

int launch_ksplit_kernel(const GemmArgs& args, int m_tiles, int wave_k, bool swiglu, int lds_bytes, hipStream_t stream) {
    if (lds_bytes != ksplit_lds_bytes(m_tiles, wave_k)) return HFRK_INVALID_CONFIG;
    if (!ksplit_variant_exists(m_tiles, wave_k)) return HFRK_INVALID_CONFIG;
    if (swiglu && args.slabs != 1) return HFRK_INVALID_CONFIG;
#define HFRK_KSPLIT_CASE(MT_)                                                                          \
    case MT_:                                                                                          \
        return wave_k == 256 ? launch_ksplit_one<MT_, 256>(args, swiglu, lds_bytes, stream)            \
                             : launch_ksplit_one<MT_, 512>(args, swiglu, lds_bytes, stream);
    if (wave_k == 1024) {  // 16*MT rows x 1 KB of activations per wave: registers allow two tiles
        return m_tiles == 1 ? launch_ksplit_one<1, 1024>(args, swiglu, lds_bytes, stream)
                            : launch_ksplit_one<2, 1024>(args, swiglu, lds_bytes, stream);
    }
    switch (m_tiles) {
        HFRK_KSPLIT_CASE(1)
        HFRK_KSPLIT_CASE(2)
        HFRK_KSPLIT_CASE(3)
        HFRK_KSPLIT_CASE(4)
    }
#undef HFRK_KSPLIT_CASE
    return HFRK_INVALID_CONFIG;
}

}  // namespace hfrk
