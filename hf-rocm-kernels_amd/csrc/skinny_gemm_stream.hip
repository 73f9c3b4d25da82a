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
#include "skinny_gemm_args.h"

namespace hfrk {

// MA = 16-byte activation loads per lane and chunk: load t brings rows 4t .. 4t+3, so 4*MA >= m.
// RT = 16-row weight tiles per chunk.
// SWIGLU: the weight is a gate_up projection (gate rows [0, n/2), up rows [n/2, n)); a chunk pairs gate tile t with
// up tile t (RT = 2) and the epilogue stores fp8(silu(gate) * up / out_scale) into D [m, n/2] instead of the two
// 16-bit projections -- the SwiGLU kernel of csrc/op_src/swiglu/swiglu_vectorized.cu:27-97 as a GEMM epilogue.
// PACKED: the weight is in the pre-packed layout (pack_weight.hip): chunk (tile, kc) is 4 KB at
// (tile * KC + kc) * 4096, already in MFMA operand order, so a chunk is one contiguous read and needs no LDS pass.
// RAGGED_K: row-major weights whose k is a multiple of 16 but not of 256: the last chunk of a row is cut short by whole
// 16-byte pieces, and the lanes whose piece lies beyond k read zeros in both operands (the reference accepts such k
// with its narrow tiles, csrc/op_src/skinny_gemm/skinny_gemm_caller.cu:33-48).  A variant of its own, so that the
// common case keeps its instruction count before the first request.
enum { kLayoutRowMajor = 0, kLayoutPacked = 1, kLayoutRaggedK = 2 };
template <int MA, int RT, bool SWIGLU, int LAYOUT>
__global__ void __launch_bounds__(kGemmThreads) skinny_gemm_stream_kernel(const GemmArgs a) {
    constexpr bool PACKED = LAYOUT == kLayoutPacked, RAGGED_K = LAYOUT == kLayoutRaggedK;
    constexpr uint32_t kOutOfRange = 0x80000000u;
    constexpr int kCoherent = 17;  // sc0 | sc1
    constexpr int MT = (MA + 3) / 4;  // 16-row activation tiles
    constexpr int SUB = RT * MT;      // 16x16 output tiles per row group
    constexpr int kWaveLds = (RT + MT) * kTileBytes;
    static_assert(!SWIGLU || RT == 2, "the SwiGLU epilogue pairs one gate tile with one up tile");

    extern __shared__ __align__(16) uint8_t lds[];
    // After its loop a wave's tiles are dead; its partial-sum slots (SUB x 64 lanes x 16 bytes <= RT x 4 KB) reuse
    // the start of its own weight tiles, so no other wave's data is touched before the barrier.
    v4f* const slots = reinterpret_cast<v4f*>(lds);  // slot `sub` of wave w at v4f index w * kSlotStride + sub * 64
    constexpr int kSlotStride = kWaveLds / 16;       // in v4f

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;

    // ---- this wave's run of chunks (all 32-bit: the host checks (grid + 1) * chunks < 2^31) ------------------------
    const int G = a.grid;
    const int KC = a.slabs;  // 256-byte chunks per row tile
    const int b = blockIdx.x;
    const int g = ((G & 7) == 0) ? (b & 7) * (G >> 3) + (b >> 3) : b;  // XCD x owns logical ids [x*G/8, (x+1)*G/8)
    const uint32_t cq = (uint32_t)a.chunks_q, cr = (uint32_t)a.chunks_r;  // chunks / G, chunks % G
    const uint32_t c0 = (uint32_t)g * cq + min((uint32_t)g, cr);
    const uint32_t nwg = cq + ((uint32_t)g < cr ? 1u : 0u);
    const uint32_t c1 = c0 + nwg;
    const uint32_t w0 = c0 + (uint32_t)wv * nwg / kGemmWaves, w1 = c0 + (uint32_t)(wv + 1) * nwg / kGemmWaves;
    const int count = (int)(w1 - w0);
    int tile = (int)(w0 / (uint32_t)KC);  // chunk being multiplied
    int kc = (int)(w0 - (uint32_t)tile * (uint32_t)KC);

    // ---- first request, as early as possible ---------------------------------------------------------------------
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.B, PACKED ? (uint32_t)((a.n + 15) >> 4) * (uint32_t)KC * (uint32_t)kTileBytes
                                                                : (uint32_t)(a.n - 1) * (uint32_t)a.b_stride + (uint32_t)a.k);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a.A, (uint32_t)a.m * (uint32_t)a.k);
    const uint32_t w_lane_off = (uint32_t)lg * (uint32_t)a.b_stride + (uint32_t)li * 16u;
    const uint32_t a_lane_off = (uint32_t)lg * (uint32_t)a.k + (uint32_t)li * 16u;
    // RAGGED_K: in a row's last chunk the lanes whose piece lies beyond k start from an out-of-range offset
    const bool beyond_k = RAGGED_K && (KC - 1) * 256 + li * 16 >= a.k;
    const uint32_t w_tail_off = beyond_k ? kOutOfRange : w_lane_off, a_tail_off = beyond_k ? kOutOfRange : a_lane_off;
    v4i wq[4 * RT], aq[MA];
    int itile = tile, ikc = kc;  // chunk being requested
    auto issue_chunk = [&]() __attribute__((always_inline)) {
        const uint32_t abase = (uint32_t)ikc * 256u;
        // row group t: weight rows [16*RT*t, 16*RT*(t+1)), or with SWIGLU rows [16t, 16t+16) and n/2 + the same
        const uint32_t wbase = (uint32_t)itile * (SWIGLU ? 16u : 16u * RT) * (uint32_t)a.b_stride + (uint32_t)ikc * 256u;
        const bool last = RAGGED_K && ikc == KC - 1;  // uniform
        const uint32_t a_off = last ? a_tail_off : a_lane_off, w_off = last ? w_tail_off : w_lane_off;
#pragma unroll
        for (int t = 0; t < MA; ++t)
            aq[t] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(a_off + abase + (uint32_t)(4 * t) * (uint32_t)a.k), 0, 0);
        if constexpr (PACKED) {
            // 16-row tile of row group t: RT*t + rt, or with SWIGLU t (gate) and n/32 + t (up); a tile past the last
            // one (odd tile count, RT = 2) is out of the buffer's range and reads as zero
#pragma unroll
            for (int t = 0; t < 4 * RT; ++t) {
                const uint32_t tl = SWIGLU ? (uint32_t)itile + (uint32_t)(t / 4) * (uint32_t)(a.n >> 5) : (uint32_t)itile * RT + (uint32_t)(t / 4);
                wq[t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)((tl * (uint32_t)KC + (uint32_t)ikc) * (uint32_t)kTileBytes + (uint32_t)(t % 4) * 1024u + (uint32_t)lane * 16u), 0, 2 /* nt */);
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4 * RT; ++t)
                wq[t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)(w_off + wbase + (uint32_t)(SWIGLU ? (t / 4) * (a.n >> 1) + 4 * (t % 4) : 4 * t) * (uint32_t)a.b_stride), 0, 2 /* nt */);
        }
    };
    if (count > 0) issue_chunk();
    __builtin_amdgcn_sched_barrier(0);  // keep the set-up below behind the first request

    // ---- the rest of the set-up -----------------------------------------------------------------------------------
    const __amdgpu_buffer_rsrc_t ws_rsrc = make_rsrc(a.ws, a.ws_bytes);
    const int n_out = SWIGLU ? (a.n >> 1) : a.n;  // columns of D
    const __amdgpu_buffer_rsrc_t d_rsrc = make_rsrc(a.D, (uint32_t)a.m * (uint32_t)n_out * (SWIGLU ? 1u : 2u));
    const __amdgpu_buffer_rsrc_t base_rsrc = make_rsrc(a.base, a.base ? (uint32_t)a.m * (uint32_t)a.n * 2u : 0u);
    const bool accumulate = !SWIGLU && a.base != nullptr;
    const __amdgpu_buffer_rsrc_t sb_rsrc = make_rsrc(a.scale_b, a.scale_b ? (uint32_t)a.n * 4u : 0u);
    const bool vec = SWIGLU || ((a.n & 3) == 0);  // then a lane's four outputs n0 .. n0+3 are all inside n and aligned
    const bool per_channel = a.scale_b && a.sb_stride;
    // Lane li holds the accumulator column of activation row (= output row) mt*16 + li of activation tile mt.
    // The scales are fetched behind the first chunk's requests: a wait for them up front would hold back the whole
    // stream by one memory latency.
    float sa[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        sa[mt] = a.scale_a[(long)min(mt * 16 + li, a.m - 1) * a.sa_stride] * ((a.scale_b && !a.sb_stride) ? a.scale_b[0] : 1.0f);
    float inv_out_scale = 1.0f;
    if (SWIGLU) {
        const float os = a.out_scale[0];
        inv_out_scale = os != 0.f ? 1.0f / os : 1.0f;
    }

    uint8_t* const tw = lds + wv * kWaveLds;  // this wave's RT weight tiles, then its MT activation tiles
    uint8_t* const ta = tw + RT * kTileBytes;
    int wr_off[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int row = 4 * t + lg;
        wr_off[t] = row * 256 + ((li ^ row) << 4);
    }
    int rd_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) rd_off[h] = li * 256 + ((((8 * h + 2 * lg) ^ li) & 15) << 4);

    // Old D values (accumulate mode) and per-channel scales of one row tile, requested ahead of the epilogue that
    // uses them (aligned n only).  Nothing is requested when nothing is wanted: even a load that is out of range
    // and touches no memory returns in order, behind the CU's queue of real requests, and would be waited for.
    struct Pre { v2i d[SUB]; v4i sb[RT]; };
    const bool want_pre = vec && (accumulate || per_channel);
    auto prefetch = [&](int t, bool wanted) __attribute__((always_inline)) {
        Pre p;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            p.sb[rt] = v4i{0, 0, 0, 0};
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) p.d[rt * MT + mt] = v2i{0, 0};
        }
        if (wanted && want_pre) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const int n0 = SWIGLU ? rt * (a.n >> 1) + t * 16 + 4 * lg : (t * RT + rt) * 16 + 4 * lg;  // weight row
                p.sb[rt] = __builtin_amdgcn_raw_buffer_load_b128(sb_rsrc, (per_channel && n0 < a.n) ? n0 * 4 : (int)kOutOfRange, 0, 0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const int mrow = mt * 16 + li;
                    const bool ok = accumulate && mrow < a.m && n0 < a.n;
                    p.d[rt * MT + mt] = __builtin_amdgcn_raw_buffer_load_b64(base_rsrc, ok ? (int)(((uint32_t)mrow * (uint32_t)a.n + (uint32_t)n0) * 2u) : (int)kOutOfRange, 0, 0);
                }
            }
        }
        return p;
    };

    // scale, add D (accumulate mode), round once, store: lane holds D^T[n0 + v][mrow], v = 0..3, of every 16x16 tile.
    // Aligned n: D and the channel scales were prefetched (pre), one 8-byte store.  Ragged n (n % 4 != 0): 2-byte
    // buffer accesses whose out-of-range offsets mask the columns beyond n, fetched here.
    auto epilogue = [&](int t, const v4f (&acc)[SUB], const Pre& pre) __attribute__((always_inline)) {
        if constexpr (SWIGLU) {
            // acc[0*MT+mt] = gate tile, acc[1*MT+mt] = up tile of the same output columns n0 .. n0+3
            const int n0 = t * 16 + 4 * lg;
            const v4f sbg = __builtin_bit_cast(v4f, pre.sb[0]), sbu = __builtin_bit_cast(v4f, pre.sb[1]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int mrow = mt * 16 + li;
                float y[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float g = acc[mt][v] * (sa[mt] * (per_channel ? sbg[v] : 1.0f));
                    float u = acc[MT + mt][v] * (sa[mt] * (per_channel ? sbu[v] : 1.0f));
                    // the unfused chain rounds both projections to 16 bits before the activation: do the same
                    g = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(g)) : load16<HFRK_F16>(store16<HFRK_F16>(g));
                    u = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>(store16<HFRK_BF16>(u)) : load16<HFRK_F16>(store16<HFRK_F16>(u));
                    y[v] = silu_mul(g, u, inv_out_scale);
                }
                uint32_t packed = cvt_pk_fp8(y[0], y[1], 0u, false);
                packed = cvt_pk_fp8(y[2], y[3], packed, true);
                const bool live = mrow < a.m && n0 < n_out;
                __builtin_amdgcn_raw_buffer_store_b32((int)packed, d_rsrc, live ? (int)((uint32_t)mrow * (uint32_t)n_out + (uint32_t)n0) : (int)kOutOfRange, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int n0 = (t * RT + rt) * 16 + 4 * lg;
                const int mrow = mt * 16 + li;
                const bool live = mrow < a.m && n0 < a.n;
                const uint32_t d_off = ((uint32_t)mrow * (uint32_t)a.n + (uint32_t)n0) * 2u;
                uint32_t old[4];
                v4f sb;
                uint32_t off[4];
                if (vec) {
                    sb = __builtin_bit_cast(v4f, pre.sb[rt]);  // (a bit_cast of a single vector element would read element 0)
                    const v2i d = pre.d[rt * MT + mt];
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
                uint32_t o[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float r = acc[rt * MT + mt][v] * (sa[mt] * (per_channel ? sb[v] : 1.0f));
                    const float base = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>((uint16_t)old[v]) : load16<HFRK_F16>((uint16_t)old[v]);
                    const float sum = accumulate ? base + r : r;
                    o[v] = a.d_dtype == HFRK_BF16 ? store16<HFRK_BF16>(sum) : store16<HFRK_F16>(sum);
                }
                if (vec) {
                    const v2i packed = {(int)(o[0] | (o[1] << 16)), (int)(o[2] | (o[3] << 16))};
                    __builtin_amdgcn_raw_buffer_store_b64(packed, d_rsrc, live ? (int)d_off : (int)kOutOfRange, 0, 0);
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v) __builtin_amdgcn_raw_buffer_store_b16((short)o[v], d_rsrc, (int)off[v], 0, 0);
                }
            }
        }
    };

    // A wave's run is: [head segment] [whole row tiles ...] [last segment]; head/last may be partial tiles.
    const int tile_h = tile, kb_h = kc;
    const int ke_h = min(KC, kb_h + count);
    const bool head_partial = count > 0 && !(kb_h == 0 && ke_h == KC);

    // ---- streaming loop ---------------------------------------------------------------------------------------
    Pre pre_next = prefetch(tile, count > 0 && kc == KC - 1), pre_cur;
    v4f acc[SUB], part_h[SUB];
#pragma unroll
    for (int u = 0; u < SUB; ++u) acc[u] = part_h[u] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < count; ++i) {
#pragma unroll
        for (int t = 0; t < MA; ++t) *reinterpret_cast<v4i*>(ta + (t / 4) * kTileBytes + wr_off[t % 4]) = aq[t];
        v4i wcur[4 * RT];  // PACKED: the chunk's operands, out of the way of the next request
#pragma unroll
        for (int t = 0; t < 4 * RT; ++t) {
            if constexpr (PACKED) wcur[t] = wq[t];
            else *reinterpret_cast<v4i*>(tw + (t / 4) * kTileBytes + wr_off[t % 4]) = wq[t];
        }
        pre_cur = pre_next;
        if (i + 1 < count) {  // registers are free again: request the next chunk before the LDS reads and MFMAs
            if (++ikc == KC) { ikc = 0; ++itile; }
            issue_chunk();
            pre_next = prefetch(itile, ikc == KC - 1);  // the chunk that ends a row tile brings the tile's D along
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // every operand of the chunk is requested from LDS before the first MFMA: one LDS latency per chunk, and the
        // MFMAs start as their operands arrive (the LDS answers in order)
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
                const v4i lo = *reinterpret_cast<const v4i*>(ta + mt * kTileBytes + rd_off[h]);
                const v4i hi = *reinterpret_cast<const v4i*>(ta + mt * kTileBytes + (rd_off[h] ^ 16));
                aop[h][mt] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the requests above ahead of the MFMAs below
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[rt * MT + mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wop[h][rt], aop[h][mt], acc[rt * MT + mt], 0, 0, 0, 0, 0, 0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (++kc == KC) {  // a row tile ends inside this wave's run
            if (tile == tile_h && head_partial) {  // its first chunks belong to an earlier wave
#pragma unroll
                for (int u = 0; u < SUB; ++u) part_h[u] = acc[u];
            } else {
                epilogue(tile, acc, pre_cur);  // all of it was ours
            }
#pragma unroll
            for (int u = 0; u < SUB; ++u) acc[u] = v4f{0.f, 0.f, 0.f, 0.f};
            kc = 0;
            ++tile;
        }
    }
    // Here (tile, kc) is the position behind the run.  kc != 0: the run ends inside row tile `tile`, whose first kc
    // chunks are in acc -- unless the whole run lies inside that one tile, then they are the head segment.
    const bool last_partial = count > 0 && kc != 0 && tile != tile_h;
    const int tile_l = tile;
    if (count > 0 && kc != 0 && tile == tile_h) {
#pragma unroll
        for (int u = 0; u < SUB; ++u) part_h[u] = acc[u];
    }

    // ---- combine the partial tiles of this workgroup ------------------------------------------------------------
    // A segment that starts its tile inside this workgroup (first K chunk of the tile, or first chunk of the
    // workgroup's range) makes this wave the one that finishes the tile.  Its D values are requested now, so that
    // they arrive while the partial sums are exchanged.  Every other head segment goes to the wave's slot; a wave
    // without chunks leaves zeros there, so that the finishing wave can add by position alone.
    const bool fin_h = head_partial && (kb_h == 0 || w0 == c0);
    const Pre pre_h = prefetch(tile_h, fin_h);
    const Pre pre_l = prefetch(tile_l, last_partial);
    if (!fin_h && (head_partial || count == 0)) {
#pragma unroll
        for (int u = 0; u < SUB; ++u) slots[wv * kSlotStride + u * 64 + lane] = part_h[u];
    }
    __syncthreads();
    if (!fin_h && !last_partial) return;

    // This part runs on one wave per row tile, after everything else: it is kept short, and the two possible
    // segments (head, last) share one copy of the code.
#pragma unroll 1
    for (int seg = 0; seg < 2; ++seg) {
        if (!(seg == 0 ? fin_h : last_partial)) continue;
        const int t = seg == 0 ? tile_h : tile_l;
        const int kb = seg == 0 ? kb_h : 0;
        // the waves after this one whose runs start before the tile (or the workgroup's range) ends hold the rest
        const uint32_t t_lo = (uint32_t)t * (uint32_t)KC;
        const uint32_t t_end = min(t_lo + (uint32_t)KC, c1);
        v4f sum[SUB];
        Pre pre;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) pre.sb[rt] = seg == 0 ? pre_h.sb[rt] : pre_l.sb[rt];
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            pre.d[u] = seg == 0 ? pre_h.d[u] : pre_l.d[u];
            sum[u] = seg == 0 ? part_h[u] : acc[u];
            v4f other[kGemmWaves];
#pragma unroll
            for (int j = 1; j < kGemmWaves; ++j) other[j] = slots[j * kSlotStride + u * 64 + lane];  // garbage where unused: never added
#pragma unroll
            for (int j = 1; j < kGemmWaves; ++j)
                if (j > wv && c0 + (uint32_t)j * nwg / kGemmWaves < t_end) sum[u] += other[j];
        }
        const int ke = (int)(t_end - t_lo);
        if (!(kb == 0 && ke == KC)) {
            // the tile continues in a neighbouring workgroup: park this workgroup's share, count the arrival
            const int slot = (c0 >= t_lo) ? 0 : 1;  // slot 0: the tile holds this workgroup's first chunk
#pragma unroll
            for (int u = 0; u < SUB; ++u)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, sum[u]), ws_rsrc, (((g * 2 + slot) * SUB + u) * 64 + lane) * 16, 0, kCoherent);
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): every lane's store acknowledged before the arrival is counted
            int last = 0;
            if (lane == 0) {
                const int mine = ke - kb;
                const int seen = atomicAdd(&a.counters[t], mine);
                last = (seen + mine == KC);
                if (last) a.counters[t] = 0;  // ready for the next launch
            }
            last = __builtin_amdgcn_readfirstlane(last);
            if (!last) continue;
            // contributors are the workgroups whose chunk range meets [t_lo, t_lo + KC), in id order; only the first
            // of them can have the tile as its second (slot 1).  owner(c) = the workgroup whose range holds chunk c.
            auto owner = [&](uint32_t c) __attribute__((always_inline)) {
                const uint32_t big = cr * (cq + 1u);  // chunks held by the first cr workgroups
                return c < big ? (int)(c / (cq + 1u)) : (int)(cr + (c - big) / cq);
            };
            const int g_first = owner(t_lo), g_last = owner(t_lo + (uint32_t)KC - 1u);
            const int sl_first = ((uint32_t)g_first * cq + min((uint32_t)g_first, cr) == t_lo) ? 0 : 1;
#pragma unroll
            for (int u = 0; u < SUB; ++u) sum[u] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
            for (int base = g_first; base <= g_last; base += 4) {
#pragma unroll
                for (int u = 0; u < SUB; ++u) {
                    v4i q[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {  // four partials in flight; past the last one the load is out of range: zeros
                        const int gg = base + w;
                        const int sl = gg == g_first ? sl_first : 0;
                        q[w] = __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, gg <= g_last ? (((gg * 2 + sl) * SUB + u) * 64 + lane) * 16 : (int)kOutOfRange, 0, kCoherent);
                    }
#pragma unroll
                    for (int w = 0; w < 4; ++w) sum[u] += __builtin_bit_cast(v4f, q[w]);
                }
            }
        }
        epilogue(t, sum, pre);
    }
}

template <int MA, int RT, bool SWIGLU, int LAYOUT>
static int launch_stream_packing(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = skinny_gemm_stream_kernel<MA, RT, SWIGLU, LAYOUT>;
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
    if (args.packed) return launch_stream_packing<MA, RT, SWIGLU, kLayoutPacked>(args, lds_bytes, stream);
    if (args.k % 256 != 0) return launch_stream_packing<MA, RT, SWIGLU, kLayoutRaggedK>(args, lds_bytes, stream);
    return launch_stream_packing<MA, RT, SWIGLU, kLayoutRowMajor>(args, lds_bytes, stream);
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
