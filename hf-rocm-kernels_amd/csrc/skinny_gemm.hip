// FP8 (OCP e4m3fn) skinny GEMM for MI355X / gfx950:  D[m,n] = base[m,n] + sa[m] * sb[n] * sum_k A[m,k] * W[n,k],  m <= 64.
//
// This file holds the host side of the GEMM (workspaces, plan table, launcher, the extern "C" entry points) and the
// workgroup-cooperative kernel the planner uses above 16 rows; the planner is in skinny_gemm_plan.hip, the kernels for
// fewer rows in skinny_gemm_rows_impl.h, skinny_gemm_stream.hip and skinny_gemm_ksplit.hip.
//
// Replaces the reference's persistent producer/consumer kernel and its consumers
// (csrc/op_src/skinny_gemm/skinny_gemm_kernel.cu:6-79, producers/n_full_tiles.cu:4-127,
// consumers/mfma_16x16x32_consumer.cu:1-168, consumers/smfma_16x16x64_consumer.cu:1-158) with a different
// design: the op is a pure weight stream (2*m flop per weight byte against ~625 flop/byte of machine balance),
// so everything is organised around keeping 16-byte, fully coalesced, non-temporal weight loads in flight.
//
//  * Work unit = (panel of 16*WN weight rows) x (K slab of 256*WK*CH bytes).  Units are ordered slab-fastest and
//    cut into `grid` equal contiguous ranges, one per persistent workgroup (stream-K): every CU streams the same
//    number of bytes whatever the shape.  Logical workgroup ids are laid out so that one XCD owns one contiguous
//    range of units (neighbouring workgroups, which may share a panel, share an L2).
//  * A workgroup is 8 waves = WN (rows) x WK (K).  Per 256-byte K chunk a wave issues four 16-byte buffer loads
//    per lane, each instruction covering 4 weight rows x 256 contiguous bytes (two full cache lines per row),
//    `nt` so the stream does not displace the activations in L2.  Two units are always in flight per wave.
//  * The chunk is turned into MFMA operand layout (lane = row + 16*kgroup, 32 contiguous K bytes per lane)
//    through a wave-private, XOR-swizzled 4 KB LDS tile: no barrier, the wave only waits on its own LDS ops.
//  * The activation slab [16*MT, KS] is staged in LDS once per unit for all 8 waves (double buffered, same
//    swizzle), so the only global traffic in the loop is the weight stream.
//  * Contraction: v_mfma_f32_16x16x128_f8f6f4, weights as the A operand (rows = n), activations as the
//    B operand (cols = m), fp32 accumulators held across all the slabs a workgroup owns of a panel.
//  * When a panel ends: waves that split K inside the workgroup are summed through LDS; if the workgroup owned
//    every slab of the panel it writes D directly, otherwise it parks its fp32 partial in the workspace and the
//    workgroup that arrives last (per-panel counter) adds the partials in workgroup order -- a fixed order, so
//    results are bit-reproducible -- applies the scales once, adds D (accumulate mode) and rounds once.
#include <functional>
#include <mutex>
#include <thread>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "skinny_gemm_args.h"
#include "skinny_gemm_plan.h"

namespace hfrk {

// first unit of logical workgroup g
// 32-bit on purpose (64-bit division is a long instruction sequence); the host checks units * (grid + 1) < 2^31.
__device__ __forceinline__ int unit_begin(int g, int units, int grid) { return (int)(((uint32_t)g * (uint32_t)units) / (uint32_t)grid); }

// PACKED: the weight is in the pre-packed layout (pack_weight.hip), chunk (tile, kc) at (tile * k/256 + kc) * 4096 in
// MFMA operand order: the loads are 1 KB contiguous per instruction and the chunk skips the transposition tile.
// RT = 16-row weight tiles per wave and chunk (1 or 2).  With 2 a wave's activation operands, read from LDS once per
// 128 K-bytes, multiply two weight tiles: half the activation bytes through the LDS pipe per weight byte, which is what
// bounds this kernel from 32 rows up.
template <int MT, int WN, int WK, int CH, int RT, bool PACKED>
__global__ void __launch_bounds__(kGemmThreads) skinny_gemm_kernel(const GemmArgs a) {
    static_assert(WN * WK == kGemmWaves, "a workgroup is 8 waves");
    static_assert(RT == 1 || RT == 2, "one or two weight tiles per wave");
    constexpr int KS = 256 * WK * CH;        // bytes of K per slab
    constexpr int BN = 16 * WN * RT;         // weight rows per panel
    constexpr int ST = RT * MT;              // 16x16 output tiles per wave: index rt * MT + mt
    constexpr int ACT_BYTES = 16 * MT * KS;  // one staged activation slab
    constexpr int KP = KS / 16;              // 16-byte pieces per activation row of a slab
    constexpr int PIECES = 16 * MT * KP;
    constexpr int APT = (PIECES + kGemmThreads - 1) / kGemmThreads;  // activation pieces per thread

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* const tbuf_all = lds;
    uint8_t* const act_all = lds + kGemmWaves * RT * kTileBytes;
    // One word for the "last arriver" verdict of a panel flush.  It lives at the start of wave 0's transposition tile:
    // during a flush no tile holds weights (the unit's MFMAs are done, the next unit's tiles are written after the flush's
    // last barrier), and the K-wave reduction that borrows the tiles as scratch writes only those of waves with wk != 0.
    int* const flag = reinterpret_cast<int*>(tbuf_all);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave / WK, wk = wave % WK;
    const int li = lane & 15, lg = lane >> 4;

    const int G = a.grid, S = a.slabs, U = a.units;
    const int b = blockIdx.x;
    const int g = ((G & 7) == 0) ? (b & 7) * (G >> 3) + (b >> 3) : b;  // XCD x owns logical ids [x*G/8, (x+1)*G/8)
    const int u0 = unit_begin(g, U, G), u1 = unit_begin(g + 1, U, G);
    if (u0 >= u1) return;  // cannot happen when grid <= units; uniform for the whole workgroup

    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(a.B, PACKED ? (uint32_t)((a.n + 15) >> 4) * (uint32_t)a.k * 16u
                                                                : (uint32_t)(a.n - 1) * (uint32_t)a.b_stride + (uint32_t)a.k);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a.A, (uint32_t)a.m * (uint32_t)a.k);
    uint16_t* const D = reinterpret_cast<uint16_t*>(a.D);
    const uint16_t* const Dbase = reinterpret_cast<const uint16_t*>(a.base);  // added to the product when not null
    const bool accumulate = a.base != nullptr;

    // ---- per-panel epilogue inputs, fetched when the panel's first weight loads are issued -------------------
    // The vector-memory counter retires in issue order, so a load issued at the end of a panel would wait for
    // every prefetched weight chunk; issued up front, D and the channel scales are long home when needed.
    // A lane owns D[mt*16 + li][n0 .. n0+3], n0 = panel*BN + (wn*RT + rt)*16 + 4*lg.  At most two panels are open at once.
    // With 8 output tiles per wave (64 rows x two weight tiles) there are no registers for that: the epilogue fetches.
    constexpr bool kPrefetchEpilogue = ST < 8;
    constexpr int kCtx = kPrefetchEpilogue ? 2 : 1;
    uint2 dq[kCtx][ST];
    float sbq[kCtx][RT][4];
    float saq[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int mrow = min(mt * 16 + li, a.m - 1);
        saq[mt] = a.scale_a[(long)mrow * a.sa_stride];
    }
    const bool n_vec = (a.n & 3) == 0;
    auto panel_fetch = [&](int panel, uint2 (&dd)[ST], float (&sb)[RT][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int n0 = panel * BN + (wn * RT + rt) * 16 + 4 * lg;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = min(n0 + v, a.n - 1);
                sb[rt][v] = a.scale_b ? a.scale_b[(long)n * a.sb_stride] : 1.0f;
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                dd[rt * MT + mt] = make_uint2(0u, 0u);
                const int mrow = mt * 16 + li;
                if (accumulate && mrow < a.m) {
                    const uint16_t* const drow = Dbase + (long)mrow * a.n;
                    if (n_vec && n0 + 3 < a.n) {
                        dd[rt * MT + mt] = *reinterpret_cast<const uint2*>(drow + n0);
                    } else {
                        uint32_t e[4];
#pragma unroll
                        for (int v = 0; v < 4; ++v) e[v] = (n0 + v < a.n) ? drow[n0 + v] : 0u;
                        dd[rt * MT + mt] = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
                    }
                }
            }
        }
    };
    int fetch_par = 0;  // which of the two contexts the next panel_fetch fills

    // ---- weight stream -------------------------------------------------------------------------------------
    // load t of a chunk: lane -> weight row 4t + lane/16, bytes (lane%16)*16 .. +16 of the 256-byte chunk
    const uint32_t w_lane_off = (uint32_t)lg * (uint32_t)a.b_stride + (uint32_t)li * 16u;
    v4i wq[2][CH][RT][4];
    int ip = u0 / S, is = u0 % S;  // (panel, slab) of the next unit to issue
    // Panel p walks its K slabs starting from slab p % S (sums do not care about the order): workgroups that move
    // through their panels in step then read different activation slabs at any moment instead of all hitting
    // the same few L2 lines.
    auto phys_slab = [&](int panel, int slab) __attribute__((always_inline)) {
        const int r = slab + panel % S;
        return r >= S ? r - S : r;
    };
    bool issue_first = true;       // next unit to issue opens a panel for this workgroup
    // Every step issues the same number of loads, in range or not: a unit past the end of this workgroup's range
    // is requested at an offset beyond the buffer, which returns zeros without touching memory.  That keeps the
    // count of loads in flight a compile-time constant, so each wait leaves exactly the prefetched unit pending.
    // Weight chunk c of unit (ip, is) into register set X.
    auto issue_chunk = [&](auto sel, int c, bool in_range) __attribute__((always_inline)) {
        constexpr int X = decltype(sel)::value;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int tile = ip * (WN * RT) + wn * RT + rt;  // 16-row weight tile
            if constexpr (PACKED) {
                // a tile past the last one (n not a multiple of the panel height) lies beyond the buffer and reads as zero
                const uint32_t chunk = (uint32_t)tile * ((uint32_t)a.k >> 8) + (uint32_t)phys_slab(ip, is) * (WK * CH) + (uint32_t)(c * WK + wk);
                const uint32_t base = in_range ? chunk * (uint32_t)kTileBytes + (uint32_t)lane * 16u : 0x80000000u;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    wq[X][c][rt][t] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)(base + (uint32_t)t * 1024u), 0, 2 /* nt */);
            } else {
                const uint32_t base = in_range ? (uint32_t)(tile * 16) * (uint32_t)a.b_stride + (uint32_t)phys_slab(ip, is) * KS +
                                                     (uint32_t)(c * WK + wk) * 256u
                                               : 0x80000000u;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    wq[X][c][rt][t] = __builtin_amdgcn_raw_buffer_load_b128(
                        w_rsrc, (int)(w_lane_off + base + (uint32_t)(4 * t) * (uint32_t)a.b_stride), 0, 2 /* nt */);
            }
        }
    };
    // Epilogue inputs of unit (ip, is) if it opens a panel, then move on to the next unit.
    auto issue_done = [&](bool in_range) __attribute__((always_inline)) {
        if (in_range && issue_first) {
            if constexpr (kPrefetchEpilogue) {
                if (wk == 0) {
                    if (fetch_par) panel_fetch(ip, dq[kCtx - 1], sbq[kCtx - 1]);
                    else panel_fetch(ip, dq[0], sbq[0]);
                }
            }
            fetch_par ^= 1;
        }
        issue_first = false;
        if (++is == S) { is = 0; ++ip; issue_first = true; }
    };
    auto issue_unit = [&](auto sel, bool in_range) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < CH; ++c) issue_chunk(sel, c, in_range);
        issue_done(in_range);
    };

    // ---- activation slab staging ---------------------------------------------------------------------------
    v4i aq[APT];
    // always called just before issue_unit for the same unit, so (ip, is) name that unit
    auto act_load = [&](bool in_range) __attribute__((always_inline)) {
        const uint32_t base = in_range ? (uint32_t)phys_slab(ip, is) * KS : 0x80000000u;
#pragma unroll
        for (int q = 0; q < APT; ++q) {
            const int idx = tid + q * kGemmThreads;
            if (PIECES % kGemmThreads == 0 || idx < PIECES) {
                const int row = idx / KP, kp = idx % KP;
                aq[q] = __builtin_amdgcn_raw_buffer_load_b128(
                    a_rsrc, (int)((uint32_t)row * (uint32_t)a.k + base + (uint32_t)kp * 16u), 0, 0);
            }
        }
    };
    auto act_store = [&](int buf) __attribute__((always_inline)) {
        uint8_t* const dst = act_all + buf * ACT_BYTES;
#pragma unroll
        for (int q = 0; q < APT; ++q) {
            const int idx = tid + q * kGemmThreads;
            if (PIECES % kGemmThreads == 0 || idx < PIECES) {
                const int row = idx / KP, kp = idx % KP;
                *reinterpret_cast<v4i*>(dst + row * KS + (kp >> 4) * 256 + (((kp & 15) ^ (row & 15)) << 4)) = aq[q];
            }
        }
    };

    v4f acc[ST];
#pragma unroll
    for (int st = 0; st < ST; ++st) acc[st] = v4f{0.f, 0.f, 0.f, 0.f};

    uint8_t* const tb = tbuf_all + wave * RT * kTileBytes;  // this wave's RT transposition tiles
    // swizzled offsets of this lane inside a 16 x 256 B tile: as writer (row 4t+lg, piece li) and as reader (row li)
    int wr_off[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int row = 4 * t + lg;
        wr_off[t] = row * 256 + ((li ^ row) << 4);
    }
    int rd_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) rd_off[h] = ((((8 * h + 2 * lg) ^ li) & 15) << 4);  // piece 8h+2g; its pair is ^16

    // Multiply unit u (register set X, activation buffer `buf`).  The registers of a chunk are free once its tile
    // is written, so the same chunk of unit u+2 is requested right there, ahead of the LDS reads and the MFMAs.
    auto consume_unit = [&](auto sel, int buf, bool next_in_range) __attribute__((always_inline)) {
        constexpr int X = decltype(sel)::value;
        const uint8_t* const act = act_all + buf * ACT_BYTES;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            v4i wcur[RT][4];  // PACKED: the chunk's operands, out of the way of the next request
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if constexpr (PACKED) wcur[rt][t] = wq[X][c][rt][t];
                    else *reinterpret_cast<v4i*>(tb + rt * kTileBytes + wr_off[t]) = wq[X][c][rt][t];
                }
            issue_chunk(sel, c, next_in_range);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int kblk = c * WK + wk;
            // Every operand of the chunk is requested from LDS before the first MFMA: one LDS latency per chunk instead
            // of one per pair of MFMAs (the LDS answers in order, so the MFMAs start as their operands arrive).  The
            // variants with the most accumulators and prefetch registers do it per 128-byte K step: two latencies.
            constexpr int HB = (MT >= 3 && (CH == 2 || RT == 2)) ? 1 : 2;  // K steps requested together
            v8i wop[2][RT], aop[2][MT];
#pragma unroll
            for (int h0 = 0; h0 < 2; h0 += HB) {
#pragma unroll
            for (int h = h0; h < h0 + HB; ++h) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    v4i wlo, whi;
                    if constexpr (PACKED) {
                        wlo = wcur[rt][2 * h];
                        whi = wcur[rt][2 * h + 1];
                    } else {
                        wlo = *reinterpret_cast<const v4i*>(tb + rt * kTileBytes + li * 256 + rd_off[h]);
                        whi = *reinterpret_cast<const v4i*>(tb + rt * kTileBytes + li * 256 + (rd_off[h] ^ 16));
                    }
                    wop[h][rt] = v8i{wlo[0], wlo[1], wlo[2], wlo[3], whi[0], whi[1], whi[2], whi[3]};
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const uint8_t* const arow = act + (mt * 16 + li) * KS + kblk * 256;
                    const v4i alo = *reinterpret_cast<const v4i*>(arow + rd_off[h]);
                    const v4i ahi = *reinterpret_cast<const v4i*>(arow + (rd_off[h] ^ 16));
                    aop[h][mt] = v8i{alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the requests above ahead of the MFMAs below
#pragma unroll
            for (int h = h0; h < h0 + HB; ++h)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        acc[rt * MT + mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wop[h][rt], aop[h][mt], acc[rt * MT + mt], 0, 0, 0, 0, 0, 0);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    };

    // ---- epilogue ------------------------------------------------------------------------------------------
    // lane holds, per m-tile, D^T[n0 + v][mt*16 + li], v = 0..3: scale, add the fetched D, round once, store
    auto store_panel = [&](int panel, int par) __attribute__((always_inline)) {
        if constexpr (!kPrefetchEpilogue) {
            panel_fetch(panel, dq[0], sbq[0]);
            par = 0;
        }
#pragma unroll
        for (int st = 0; st < ST; ++st) {
            const int rt = st / MT, mt = st % MT;
            const int n0 = panel * BN + (wn * RT + rt) * 16 + 4 * lg;
            const bool vec_ok = n_vec && (n0 + 3 < a.n);
            const int mrow = mt * 16 + li;
            if (mrow >= a.m) continue;
            const uint2 old = par ? dq[kCtx - 1][st] : dq[0][st];
            const uint32_t oe[4] = {old.x & 0xffffu, old.x >> 16, old.y & 0xffffu, old.y >> 16};
            uint32_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float r = acc[st][v] * (saq[mt] * (par ? sbq[kCtx - 1][rt][v] : sbq[0][rt][v]));
                const float base = a.d_dtype == HFRK_BF16 ? load16<HFRK_BF16>((uint16_t)oe[v]) : load16<HFRK_F16>((uint16_t)oe[v]);
                const float sum = accumulate ? base + r : r;
                o[v] = a.d_dtype == HFRK_BF16 ? store16<HFRK_BF16>(sum) : store16<HFRK_F16>(sum);
            }
            uint16_t* const drow = D + (long)mrow * a.n;
            if (vec_ok) {
                *reinterpret_cast<uint2*>(drow + n0) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n0 + v < a.n) drow[n0 + v] = (uint16_t)o[v];
            }
        }
    };

    // fp32 partial of (workgroup gg, slot): [wn][rt * MT + mt][lane] float4.  Partials cross XCDs, whose L2s are not coherent
    // with each other: they are written through to memory and read past the caches (sc0 sc1 on both sides), which
    // keeps them coherent per location without the L2 write-back / invalidate a device-scope fence would cost.
    const __amdgpu_buffer_rsrc_t ws_rsrc = make_rsrc(a.ws, a.ws_bytes);
    auto ws_off = [&](int gg, int slot, int st) __attribute__((always_inline)) -> int {
        return (((gg * 2 + slot) * (WN * ST) + wn * ST + st) * 64 + lane) * 16;
    };
    constexpr int kCoherent = 17;  // sc0 | sc1

    int flush_par = 0;  // context of the panel that closes next
    // close panel `panel`, of which this workgroup covered slabs [s_first, s_end)
    auto flush_panel = [&](int panel, int s_first, int s_end) __attribute__((always_inline)) {
        if constexpr (WK > 1) {
            // sum the WK waves that share rows; their transposition tiles are idle here and serve as scratch
            v4f* const mine = reinterpret_cast<v4f*>(tb);
            if (wk != 0) {
#pragma unroll
                for (int st = 0; st < ST; ++st) mine[st * 64 + lane] = acc[st];
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int w = 1; w < WK; ++w) {
                    const v4f* const other = reinterpret_cast<const v4f*>(tbuf_all + (wn * WK + w) * RT * kTileBytes);
#pragma unroll
                    for (int st = 0; st < ST; ++st) acc[st] += other[st * 64 + lane];
                }
            }
            __syncthreads();
        }
        const bool full = (s_first == 0) && (s_end == S);
        if (full) {
            if (wk == 0) store_panel(panel, flush_par);
        } else {
            const int slot = (panel == u0 / S) ? 0 : 1;
            if (wk == 0) {
#pragma unroll
                for (int st = 0; st < ST; ++st)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, acc[st]), ws_rsrc, ws_off(g, slot, st), 0, kCoherent);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stores acknowledged before the arrival is counted
            }
            __syncthreads();
            if (tid == 0) {
                const int mine = s_end - s_first;
                const int seen = atomicAdd(&a.counters[panel], mine);
                const int last = (seen + mine == S);
                if (last) a.counters[panel] = 0;  // ready for the next launch
                *flag = last;
            }
            __syncthreads();
            const int last = *flag;
            if (last && wk == 0) {
                // contributors are the workgroups whose unit range meets [panel*S, (panel+1)*S), in id order
                const uint32_t lo = (uint32_t)panel * (uint32_t)S, hi = lo + (uint32_t)S;
                const int g_first = (int)(((lo + 1) * (uint32_t)G + (uint32_t)U - 1) / (uint32_t)U) - 1;
                const int g_last = (int)((hi * (uint32_t)G + (uint32_t)U - 1) / (uint32_t)U) - 1;
#pragma unroll
                for (int st = 0; st < ST; ++st) acc[st] = v4f{0.f, 0.f, 0.f, 0.f};
                // kInFlight contributors' shares are requested together (each round trip to memory is paid once per
                // batch, not once per contributor) and added in id order; past the last one the offset is out of the
                // buffer's range and the load returns zeros
                constexpr int kInFlight = ST == 6 ? 1 : ST >= 8 ? 2 : 4;  // what the registers of each variant allow without spilling
#pragma unroll 1
                for (int first = g_first; first <= g_last; first += kInFlight) {
                    v4i share[kInFlight][ST];
#pragma unroll
                    for (int w = 0; w < kInFlight; ++w) {
                        const int gg = first + w;
                        const int sl = (unit_begin(gg, U, G) / S == panel) ? 0 : 1;
#pragma unroll
                        for (int st = 0; st < ST; ++st)
                            share[w][st] = __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, gg <= g_last ? ws_off(gg, sl, st) : (int)0x80000000u, 0, kCoherent);
                    }
#pragma unroll
                    for (int w = 0; w < kInFlight; ++w)
#pragma unroll
                        for (int st = 0; st < ST; ++st) acc[st] += __builtin_bit_cast(v4f, share[w][st]);
                }
                store_panel(panel, flush_par);
            }
            __syncthreads();  // `flag` may be rewritten by the next flush
        }
        flush_par ^= 1;
#pragma unroll
        for (int st = 0; st < ST; ++st) acc[st] = v4f{0.f, 0.f, 0.f, 0.f};
    };

    // ---- main loop -----------------------------------------------------------------------------------------
    // Issue order matters because loads retire in order: the activation slab of unit u+2 is requested before the
    // weights of unit u+2, so storing it to LDS at the top of step u+1 never waits on weights still in flight.
    using Sel0 = std::integral_constant<int, 0>;
    using Sel1 = std::integral_constant<int, 1>;
    int cp = u0 / S, cs = u0 % S;  // (panel, slab) of the unit being consumed
    int s_first = cs;              // first slab this workgroup covers of the current panel
    auto next_slab = [&](int s) __attribute__((always_inline)) { return (s + 1 == S) ? 0 : s + 1; };

    act_load(true);
    issue_unit(Sel0{}, true);
    act_store(0);
    act_load(u0 + 1 < u1);
    issue_unit(Sel1{}, u0 + 1 < u1);
    __syncthreads();

    // One step = one unit.  A step whose unit lies past u1 (odd range length) multiplies zeros and changes nothing.
    auto step = [&](auto sel, int u) __attribute__((always_inline)) {
        constexpr int X = decltype(sel)::value;
        const int ns = next_slab(cs);
        if (u + 1 < u1) act_store(X ^ 1);  // slab of unit u+1, requested one step ago
        act_load(u + 2 < u1);
        consume_unit(sel, X, u + 2 < u1);
        if (u < u1 && (u + 1 == u1 || ns == 0)) {
            flush_panel(cp, s_first, cs + 1);
            s_first = 0;
        }
        issue_done(u + 2 < u1);
        if (u + 1 < u1) __syncthreads();
        cs = ns;
        if (ns == 0) ++cp;
    };
    for (int u = u0; u < u1; u += 2) {
        step(Sel0{}, u);
        step(Sel1{}, u + 1);
    }
}

// ------------------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------------------
// Split-K workspaces.  Partial sums that cross workgroups and the arrival counters that decide who adds them live in a
// workspace; two GEMMs that run at the same time must not share one, so every stream gets its own from a small per-device
// pool (launches on one stream are ordered, so they can share).  The reference needs none of this: it adds fp16 atomics
// into the caller's output (consumers/mfma_16x16x32_consumer.cu:155-163), which makes its calls independent of each other.
struct Workspace {
    float* ws = nullptr;
    int* counters = nullptr;
};
struct DeviceState {
    std::vector<Workspace> pool;                 // allocated workspaces
    std::vector<int> unassigned;                 // indices into pool that no stream owns
    std::unordered_map<uint64_t, int> by_stream; // stream key -> index into pool
};
static DeviceState g_dev[kMaxDevices];
static std::mutex g_mutex;

constexpr int kInitialWorkspaces = 4;  // allocated by hfrk_init: the streams a capture may meet for the first time
constexpr int kMaxWorkspaces = 64;     // 68 MB each; a 65th concurrent stream gets HFRK_NO_WORKSPACE

__global__ void zero_ints_kernel(int* p, int count) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = 0;
}

// The per-thread default stream is one handle for as many streams as there are threads.
static uint64_t stream_key(hipStream_t stream) {
    uint64_t key = reinterpret_cast<uintptr_t>(stream);
    if (stream == hipStreamPerThread) key ^= (uint64_t)std::hash<std::thread::id>()(std::this_thread::get_id()) << 8;
    return key;
}

// caller holds g_mutex
static int grow_pool(DeviceState& d) {
    Workspace w;
    HFRK_HIP_TRY(hipMalloc(&w.ws, kWsFloats * sizeof(float)));
    hipError_t e = hipMalloc(&w.counters, kMaxPanels * sizeof(int));
    if (e == hipSuccess) e = hipMemset(w.counters, 0, kMaxPanels * sizeof(int));
    if (e != hipSuccess) {
        (void)hipFree(w.ws);
        if (w.counters) (void)hipFree(w.counters);
        set_last_hip_error(e);
        return HFRK_HIP_ERROR;
    }
    d.pool.push_back(w);
    d.unassigned.push_back((int)d.pool.size() - 1);
    return HFRK_SUCCESS;
}

static bool is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

// The workspace of `stream` on device `dev`: the one it already owns, else an unassigned one, else (outside a capture)
// a newly allocated one.
static int workspace_for(int dev, hipStream_t stream, Workspace* out) {
    if (dev < 0 || dev >= kMaxDevices) return HFRK_BAD_SHAPE;
    DeviceState& d = g_dev[dev];
    const uint64_t key = stream_key(stream);
    std::lock_guard<std::mutex> lock(g_mutex);
    const auto it = d.by_stream.find(key);
    if (it != d.by_stream.end()) {
        *out = d.pool[it->second];
        return HFRK_SUCCESS;
    }
    if (d.unassigned.empty()) {
        if (is_capturing(stream)) return HFRK_NOT_INITIALISED;
        if ((int)d.pool.size() >= kMaxWorkspaces) return HFRK_NO_WORKSPACE;
        do {  // the first launch on a device does what hfrk_init does
            const int rc = grow_pool(d);
            if (rc != HFRK_SUCCESS) return rc;
        } while ((int)d.pool.size() < kInitialWorkspaces);
    }
    const int idx = d.unassigned.back();
    d.unassigned.pop_back();
    d.by_stream.emplace(key, idx);
    *out = d.pool[idx];
    return HFRK_SUCCESS;
}

// ---- the allocation-free entry point's scratch: one array per device, part of the code object -----------------------------
// First kStaticWsBytes: fp32 partial sums; then kStaticCounters arrival counters.
constexpr size_t kStaticWsBytes = (size_t)16 << 20;
constexpr int kStaticCounters = 1 << 16;
static __device__ __align__(256) unsigned char scratch[kStaticWsBytes + (size_t)kStaticCounters * sizeof(int)];
static unsigned char* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, from hipGetSymbolAddress

// `scratch` names the array on the host side only; kernels and HIP calls take the address looked up here.
static int static_scratch(int dev, unsigned char** out) {
    if (dev < 0 || dev >= kMaxDevices) return HFRK_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        HFRK_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return HFRK_HIP_ERROR;
        g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return HFRK_SUCCESS;
}

template <int MT, int WN, int WK, int CH, int RT, bool PACKED>
static int launch_packing(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    auto kern = skinny_gemm_kernel<MT, WN, WK, CH, RT, PACKED>;
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

template <int MT, int WN, int WK, int CH, int RT>
static int launch_one(const GemmArgs& args, int lds_bytes, hipStream_t stream) {
    return args.packed ? launch_packing<MT, WN, WK, CH, RT, true>(args, lds_bytes, stream)
                       : launch_packing<MT, WN, WK, CH, RT, false>(args, lds_bytes, stream);
}

template <int MT>
static int launch_mt(const GemmArgs& args, const hfrk_gemm_plan& p, hipStream_t stream) {
    // decompositions whose activation slabs cannot fit in LDS are never planned and are not compiled
    // WN_ = row waves; the plan's wn = WN_ * RT_ tiles per panel
#define HFRK_CASE(WN_, WK_, CH_, RT_)                                                        \
    if constexpr (lds_bytes_for(MT, WK_, CH_, RT_) <= kLdsLimit) {                           \
        if (p.wn == WN_ * RT_ && p.wk == WK_ && p.ch == CH_) return launch_one<MT, WN_, WK_, CH_, RT_>(args, p.lds_bytes, stream); \
    }
    HFRK_CASE(1, 8, 1, 1) HFRK_CASE(1, 8, 2, 1) HFRK_CASE(2, 4, 1, 1) HFRK_CASE(2, 4, 2, 1)
    HFRK_CASE(4, 2, 1, 1) HFRK_CASE(4, 2, 2, 1) HFRK_CASE(8, 1, 1, 1) HFRK_CASE(8, 1, 2, 1)
    HFRK_CASE(1, 8, 1, 2) HFRK_CASE(2, 4, 1, 2) HFRK_CASE(4, 2, 1, 2) HFRK_CASE(8, 1, 1, 2)
#undef HFRK_CASE
    return HFRK_INVALID_CONFIG;
}

// ---- plan table: tuned decompositions that replace the planner's rule for exact (m, n, k, weight layout) keys ----------
// Filled by an autotuner (hfrk_plan_table_set) from on-device sweeps; consulted whenever a caller leaves the plan to
// the library.  Counterpart of the reference's tuned knob table (hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102).
static std::unordered_map<uint64_t, hfrk_gemm_plan> g_plan_table;
static std::mutex g_plan_mutex;

static bool plan_key(int m, int n, int k, int packed, uint64_t* key) {
    if (m < 1 || m > HFRK_GEMM_MAX_M || n < 1 || n >= (1 << 24) || k < 1 || (k >> 8) >= (1 << 16) || k % 256 != 0) return false;
    *key = ((uint64_t)(packed ? 1 : 0) << 47) | ((uint64_t)m << 40) | ((uint64_t)n << 16) | (uint64_t)(k >> 8);
    return true;
}

// The tuned plan if there is one, else the planner's.  An entry tuned for m' also serves every m below it that runs the
// same kernel instance on the same work: for m <= 16 the same number of 4-row activation loads (m' = 8 serves 5..8),
// above that the same number of 16-row tiles (m' = 32 serves 17..32); rows past m are out of the buffer's range and
// cost no traffic.  The nearest such entry wins.
static int choose_plan(int m, int n, int k, bool packed, hfrk_gemm_plan* plan) {
    uint64_t key;
    if (plan_key(m, n, k, packed, &key)) {
        const int top = m <= 16 ? (m + 3) / 4 * 4 : (m + 15) / 16 * 16;
        std::lock_guard<std::mutex> lock(g_plan_mutex);
        for (int mm = m; mm <= top && !g_plan_table.empty(); ++mm) {
            if (!plan_key(mm, n, k, packed, &key)) break;
            const auto it = g_plan_table.find(key);
            if (it != g_plan_table.end() && check_plan(m, n, k, false, &it->second, packed) == HFRK_SUCCESS) {
                *plan = it->second;
                return HFRK_SUCCESS;
            }
        }
    }
    return make_plan(m, n, k, plan, packed);
}

// D = (base ? base : 0) + scale_a x scale_b x A.B   (epilogue 0), or the fused SwiGLU form (epilogue 1).
// use_static: partial sums and counters go to this device's `scratch` array instead of the stream's workspace.
// rms: the activations are not read from A but built by the kernel's RMSNorm prologue from these 16-bit tensors.
struct RmsPrologue {
    const void* input;
    const void* residual;
    void* residual_out;
    const void* weight;
    const float* act_scale;
    float epsilon;
    int dtype;
};
static int gemm_launch(const void* A, const void* B, void* D, const void* base, const float* scale_a, int sa_stride,
                       const float* scale_b, int sb_stride, const float* out_scale, int m, int n, int k, int b_stride,
                       int d_dtype, int epilogue, const hfrk_gemm_plan* user_plan, hipStream_t stream, bool packed = false,
                       bool use_static = false, const RmsPrologue* rms = nullptr) {
    if (packed) b_stride = k;
    if (m < 1 || m > HFRK_GEMM_MAX_M || n < 1 || k < 1 || b_stride < k) return HFRK_BAD_SHAPE;
    if (k % 16 != 0 || (packed && k % 256 != 0)) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (d_dtype != HFRK_F16 && d_dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
    if (rms) {
        // the prologue exists in the row-split kernel: row-major weights, up to 8 rows, k = 4096 or 8192 (every thread of a
        // workgroup owns one or two 16-byte pieces of each row)
        if (packed || m > kRowsRmsMaxM || (k != 4096 && k != 8192) || sa_stride != 0) return HFRK_BAD_SHAPE;
        if (!rms->input || !rms->residual || !rms->residual_out || !rms->weight || !rms->act_scale) return HFRK_BAD_SHAPE;
        if (rms->residual_out == rms->residual || rms->residual_out == rms->input) return HFRK_BAD_SHAPE;  // every workgroup reads both
        if (rms->dtype != HFRK_F16 && rms->dtype != HFRK_BF16) return HFRK_BAD_DTYPE;
        if ((reinterpret_cast<uintptr_t>(rms->input) | reinterpret_cast<uintptr_t>(rms->residual) |
             reinterpret_cast<uintptr_t>(rms->residual_out) | reinterpret_cast<uintptr_t>(rms->weight)) & 15)
            return HFRK_BAD_ALIGNMENT;
        A = B;  // not read; keeps the checks below on one path
    }
    if (!A || !B || !D || !scale_a) return HFRK_BAD_SHAPE;
    if ((sa_stride != 0 && sa_stride != 1) || (sb_stride != 0 && sb_stride != 1)) return HFRK_BAD_SHAPE;
    if (epilogue != HFRK_EPILOGUE_NONE && epilogue != HFRK_EPILOGUE_SWIGLU) return HFRK_INVALID_CONFIG;
    const bool swiglu = epilogue == HFRK_EPILOGUE_SWIGLU;
    // SwiGLU epilogue: up to 16 rows in the wave-stream / row-split kernels; above, in the K-split kernel when one window covers K,
    // and up to 32 rows in the row-split kernel (two activation tiles) on any k it takes
    if (swiglu && (!out_scale || base || n % 32 != 0 || (m > kRowsMaxM && k != 2048 && k != 4096))) return HFRK_BAD_SHAPE;
    // every offset the kernel forms, including rows of the last (padded) panel, must stay below 2^31
    if (((long)n + 128) * b_stride + k >= (1L << 31) || (long)m * k >= (1L << 31)) return HFRK_BAD_SHAPE;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15 || (b_stride & 15)) return HFRK_BAD_ALIGNMENT;
    if (swiglu) {
        if (reinterpret_cast<uintptr_t>(D) & 3) return HFRK_BAD_ALIGNMENT;  // 4 fp8 outputs per store
    } else {
        // the vector path needs 8-byte aligned rows: report rather than take a slow path silently
        const uintptr_t both = reinterpret_cast<uintptr_t>(D) | reinterpret_cast<uintptr_t>(base);
        if ((both & 1) || ((n & 3) == 0 && (both & 7))) return HFRK_BAD_ALIGNMENT;
    }

    if (!user_plan && k % 256 != 0 && m > kStreamMaxM) {
        // A cut-short last chunk is handled by the kernels for up to 32 rows: more rows run as two launches over the
        // same weight (the reference accepts such k only with its narrowest tiles, skinny_gemm_caller.cu:33-48; the
        // shapes it is tuned for are all multiples of 256).
        const int first = kStreamMaxM;
        const size_t row_bytes = (size_t)n * 2;
        int rc = gemm_launch(A, B, D, base, scale_a, sa_stride, scale_b, sb_stride, out_scale, first, n, k, b_stride, d_dtype,
                             epilogue, nullptr, stream, packed, use_static);
        if (rc != HFRK_SUCCESS) return rc;
        return gemm_launch(static_cast<const uint8_t*>(A) + (size_t)first * k, B, static_cast<uint8_t*>(D) + first * row_bytes,
                           base ? static_cast<const uint8_t*>(base) + first * row_bytes : nullptr, scale_a + (size_t)first * sa_stride,
                           sa_stride, scale_b, sb_stride, out_scale, m - first, n, k, b_stride, d_dtype, epilogue, nullptr, stream,
                           packed, use_static);
    }
    hfrk_gemm_plan p;
    if (user_plan) {
        p = *user_plan;
        const int rc = check_plan(m, swiglu ? n / 2 : n, k, swiglu, &p, packed);
        if (rc != HFRK_SUCCESS) return rc;
        if (rms && (p.wn != -2 || p.wk != (swiglu ? 2 : 1) || p.grid <= m)) return HFRK_INVALID_CONFIG;
    } else if (rms) {
        const int rc = make_rms_plan(m, n, k, swiglu, &p);
        if (rc != HFRK_SUCCESS) return rc;
    } else {
        int rc;
        if (swiglu && m > 16 && (k == 2048 || k == 4096)) {
            rc = make_ksplit_plan(m, n / 2, k, &p);  // tiles of 16 output columns; a gate and an up pass per tile
        } else if (swiglu && m > 16) {
            // 17..32 rows on other k: bands of output columns in the row-split kernel, two activation tiles (row-major weights whose
            // columns deal out over the workgroups; callers run the two kernels where this returns HFRK_BAD_SHAPE)
            rc = (!packed && m <= kRowsMaxM && make_rows_plan(m, n / 2, k, &p) == HFRK_SUCCESS) ? fill_rows_plan(m, n / 2, k, 2, p.grid, &p) : HFRK_BAD_SHAPE;
        } else if (swiglu && !packed && make_rows_plan(m, n / 2, k, &p) == HFRK_SUCCESS) {
            // bands of output columns; every chunk holds the gate rows and the up rows of up to 16 of them
            rc = fill_rows_plan(m, n / 2, k, 2, p.grid, &p);
        } else if (swiglu && packed && make_rows_tiled_plan(m, n / 2, k, &p) == HFRK_SUCCESS) {
            rc = fill_rows_tiled_plan(m, n / 2, k, 2, p.grid, &p);  // the same on bands of whole tiles of 16 output columns
        } else if (swiglu) {
            rc = fill_stream_plan(m, n / 2, k, 1, false, 0, &p);
            if (rc == HFRK_SUCCESS) {  // the chunk count of a one-tile plan over n/2 rows, but every chunk holds a gate and an up tile
                p.wk = 2;
                p.lds_bytes = stream_lds_bytes(p.ch, 2);
            }
        } else {
            rc = choose_plan(m, n, k, packed, &p);
        }
        if (rc != HFRK_SUCCESS) return rc;
    }

    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    Workspace st;
    size_t ws_bytes = kWsFloats * sizeof(float);
    long counters = kMaxPanels;
    if (plan_ws_bytes(p) == 0 && plan_counters(p) == 0) {
        ws_bytes = 0;  // nothing crosses workgroups under this plan: no workspace is taken
        counters = 0;
        use_static = false;
    } else if (use_static) {
        unsigned char* ptr = nullptr;
        const int rc = static_scratch(dev, &ptr);
        if (rc != HFRK_SUCCESS) return rc;
        st.ws = reinterpret_cast<float*>(ptr);
        st.counters = reinterpret_cast<int*>(ptr + kStaticWsBytes);
        ws_bytes = kStaticWsBytes;
        counters = kStaticCounters;
    } else {
        const int rc = workspace_for(dev, stream, &st);
        if (rc != HFRK_SUCCESS) return rc;
    }
    if (plan_ws_bytes(p) > ws_bytes || plan_counters(p) > counters) return use_static ? HFRK_EXCEEDS_SCRATCH : HFRK_BAD_SHAPE;
    if (use_static) {
        // The array keeps whatever the last call (or a launch that never finished) left: the counters of this plan start at zero.
        const int count = (int)plan_counters(p);
        hipLaunchKernelGGL(zero_ints_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, st.counters, count);
        HFRK_HIP_TRY(hipGetLastError());
    }

    GemmArgs args{};
    args.A = static_cast<const uint8_t*>(A);
    args.B = static_cast<const uint8_t*>(B);
    args.D = D;
    args.base = base;
    args.out_scale = out_scale;
    args.scale_a = scale_a;
    args.scale_b = scale_b;
    args.sa_stride = sa_stride;
    args.sb_stride = sb_stride;
    args.m = m;
    args.n = n;
    args.k = k;
    args.b_stride = b_stride;
    args.packed = packed ? 1 : 0;
    args.d_dtype = d_dtype;
    args.panels = p.panels;
    args.slabs = p.slabs;
    args.units = p.panels * p.slabs;
    args.grid = p.grid;
    args.chunks_q = args.units / p.grid;
    args.chunks_r = args.units % p.grid;
    args.ws = st.ws;
    args.ws_bytes = (uint32_t)ws_bytes;
    args.counters = st.counters;
    if (p.wn == -2) {
        const int per_tile = swiglu ? 4 : 4 * p.wk;  // units a tile can hold (SwiGLU: 16 output columns, their gate and their up rows)
        args.rows_q = p.panels / p.grid;
        args.rows_r = p.panels % p.grid;
        auto geometry = [&](int units, int* tiles, int* base, int* extra) {
            *tiles = (units + per_tile - 1) / per_tile;
            *base = *tiles ? units / *tiles : 0;
            *extra = *tiles ? units % *tiles : 0;
        };
        geometry(args.rows_q + 1, &args.tiles_a, &args.base_a, &args.extra_a);
        geometry(args.rows_q, &args.tiles_b, &args.base_b, &args.extra_b);
        args.kc_magic = (uint32_t)(((1ULL << 32) + (uint64_t)p.slabs - 1) / (uint64_t)p.slabs);
        {
            // chunks per wave in the band height most workgroups have
            const int tiles = 2 * args.rows_r > p.grid ? args.tiles_a : args.tiles_b;
            const long run8 = (long)tiles * p.slabs;  // eight waves' worth
            const bool same_offset = run8 % 8 == 0 && (run8 / 8) % 16 == 0;
            const bool shared_lines = p.ch >= 3 && p.panels >= 4 * p.grid;  // (bands of 2-3 units lose 3 %: 2304 x 16384)
            args.k_rotate = (b_stride % 4096 == 0 && (same_offset || shared_lines)) ? 1 : 0;
        }
        if (rms) {
            args.rms_input = static_cast<const uint16_t*>(rms->input);
            args.rms_residual = static_cast<const uint16_t*>(rms->residual);
            args.rms_residual_out = static_cast<uint16_t*>(rms->residual_out);
            args.rms_weight = static_cast<const uint16_t*>(rms->weight);
            args.rms_act_scale = rms->act_scale;
            args.rms_epsilon = rms->epsilon;
            args.rms_dtype = rms->dtype;
            return launch_rows_kernel(args, p.ch, p.wk, swiglu, true, rows_rms_lds_bytes(p.ch, p.wk, k), stream);
        }
        return launch_rows_kernel(args, p.ch, p.wk, swiglu, false, p.lds_bytes, stream);
    }
    if (p.wn == -3) {
        const int per_tile = swiglu ? 4 : 4 * p.wk;  // units a chunk can hold
        args.rows_q = p.panels / p.grid;            // 16-row tiles per workgroup, the first rows_r workgroups one more
        args.rows_r = p.panels % p.grid;
        args.tiles_a = (4 * (args.rows_q + 1) + per_tile - 1) / per_tile;
        args.tiles_b = (4 * args.rows_q + per_tile - 1) / per_tile;
        args.base_a = args.base_b = per_tile;
        args.extra_a = args.extra_b = 0;
        args.kc_magic = (uint32_t)(((1ULL << 32) + (uint64_t)p.slabs - 1) / (uint64_t)p.slabs);
        {
            // as for the 4-row dealing below; a packed weight is contiguous, so its bands are always a whole number of 4 KB apart
            const int tiles = 2 * args.rows_r > p.grid ? args.tiles_a : args.tiles_b;
            const long run8 = (long)tiles * p.slabs;
            const bool same_offset = run8 % 8 == 0 && (run8 / 8) % 16 == 0;
            const bool shared_lines = p.ch >= 3 && p.panels >= p.grid;
            args.k_rotate = ((packed || b_stride % 4096 == 0) && (same_offset || shared_lines)) ? 1 : 0;
        }
        return launch_rows_tiled_kernel(args, p.ch, p.wk, swiglu, p.lds_bytes, stream);
    }
    if (p.wn == 0) return launch_stream_kernel(args, p.ch, p.wk, swiglu, p.lds_bytes, stream);
    if (p.wn == -1) return launch_ksplit_kernel(args, p.m_tiles, p.wk * 256, swiglu, p.lds_bytes, stream);
    switch (p.m_tiles) {
        case 1: return launch_mt<1>(args, p, stream);
        case 2: return launch_mt<2>(args, p, stream);
        case 3: return launch_mt<3>(args, p, stream);
        case 4: return launch_mt<4>(args, p, stream);
    }
    return HFRK_INVALID_CONFIG;
}

}  // namespace hfrk

extern "C" {

int hfrk_init(void) {
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= hfrk::kMaxDevices) return HFRK_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(hfrk::g_mutex);
    hfrk::DeviceState& d = hfrk::g_dev[dev];
    while ((int)d.pool.size() < hfrk::kInitialWorkspaces) {
        const int rc = hfrk::grow_pool(d);
        if (rc != HFRK_SUCCESS) return rc;
    }
    if (hfrk::g_scratch_ptr[dev] == nullptr) {  // this device's copy of the allocation-free entry point's array
        void* ptr = nullptr;
        HFRK_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(hfrk::scratch)));
        if (ptr == nullptr) return HFRK_HIP_ERROR;
        hfrk::g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
    }
    return HFRK_SUCCESS;
}

int hfrk_release_stream(void* stream) {
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= hfrk::kMaxDevices) return HFRK_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(hfrk::g_mutex);
    hfrk::DeviceState& d = hfrk::g_dev[dev];
    const auto it = d.by_stream.find(hfrk::stream_key(static_cast<hipStream_t>(stream)));
    if (it == d.by_stream.end()) return HFRK_SUCCESS;
    d.unassigned.push_back(it->second);
    d.by_stream.erase(it);
    return HFRK_SUCCESS;
}

int hfrk_reset_workspace(void* stream) {
    int dev = 0;
    HFRK_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= hfrk::kMaxDevices) return HFRK_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(hfrk::g_mutex);
    for (const hfrk::Workspace& w : hfrk::g_dev[dev].pool) {
        hipLaunchKernelGGL(hfrk::zero_ints_kernel, dim3(hfrk::kMaxPanels / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                           w.counters, hfrk::kMaxPanels);
        HFRK_HIP_TRY(hipGetLastError());
    }
    return HFRK_SUCCESS;
}

int hfrk_workspace_id(void* stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= hfrk::kMaxDevices) return -1;
    std::lock_guard<std::mutex> lock(hfrk::g_mutex);
    const hfrk::DeviceState& d = hfrk::g_dev[dev];
    const auto it = d.by_stream.find(hfrk::stream_key(static_cast<hipStream_t>(stream)));
    return it == d.by_stream.end() ? -1 : it->second;
}

int hfrk_skinny_gemm_validate(int m, int n, int k, int b_stride, int split_k, int A_producers, int B_producers,
                              int consumers, int a_lanes, int b_lanes, int qsize, int op_m, int ops) {
    (void)split_k;
    // the reference derives its K tile from the MFMA shape it would use: (512/op_m) * ops
    if (op_m != 8 && op_m != 16 && op_m != 32) return HFRK_INVALID_CONFIG;
    const int warptile_k = (512 / op_m) * ops;
    if (n % 2 != 0) return HFRK_N_NOT_EVEN;
    if (warptile_k <= 0 || k % warptile_k != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (A_producers + B_producers + consumers > 16) return HFRK_TOO_MANY_WARPS;
    if (a_lanes <= 0 || b_lanes <= 0) return HFRK_INVALID_CONFIG;
    if (qsize < A_producers / a_lanes || qsize < B_producers / b_lanes || qsize < consumers) return HFRK_QSIZE_TOO_SMALL;
    if (a_lanes > 4 || b_lanes > 6 || qsize < 1 || qsize > 6 || (ops != 4 && ops != 8)) return HFRK_INVALID_CONFIG;
    // limits of this implementation
    if (m < 1 || m > HFRK_GEMM_MAX_M || n < 1 || k < 1 || b_stride < k) return HFRK_BAD_SHAPE;
    if (k % 16 != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;  // (never after the check above: the reference's tiles are 64+ wide)
    if (b_stride % 16 != 0) return HFRK_BAD_ALIGNMENT;
    return HFRK_SUCCESS;
}

int hfrk_skinny_gemm_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    if (!plan) return HFRK_BAD_SHAPE;
    return hfrk::make_plan(m, n, k, plan);
}

int hfrk_plan_table_set(int m, int n, int k, int packed, const hfrk_gemm_plan* plan) {
    uint64_t key;
    if (!hfrk::plan_key(m, n, k, packed, &key)) return HFRK_BAD_SHAPE;
    if (plan) {
        const int rc = hfrk::check_plan(m, n, k, false, plan, packed != 0);
        if (rc != HFRK_SUCCESS) return rc;
    }
    std::lock_guard<std::mutex> lock(hfrk::g_plan_mutex);
    if (plan) hfrk::g_plan_table[key] = *plan;
    else hfrk::g_plan_table.erase(key);
    return HFRK_SUCCESS;
}

int hfrk_plan_table_get(int m, int n, int k, int packed, hfrk_gemm_plan* plan) {
    if (!plan) return HFRK_BAD_SHAPE;
    return hfrk::choose_plan(m, n, k, packed != 0, plan);
}

int hfrk_plan_table_clear(void) {
    std::lock_guard<std::mutex> lock(hfrk::g_plan_mutex);
    const int size = (int)hfrk::g_plan_table.size();
    hfrk::g_plan_table.clear();
    return size;
}

int hfrk_skinny_gemm(const void* A, const void* B, void* D, const float* scale_tensor, int m, int n, int k,
                     int b_stride, int split_k, int A_producers, int B_producers, int consumers, int a_lanes,
                     int b_lanes, int qsize, int op_m, int ops, int d_dtype, void* stream) {
    const int rc = hfrk_skinny_gemm_validate(m, n, k, b_stride, split_k, A_producers, B_producers, consumers, a_lanes,
                                             b_lanes, qsize, op_m, ops);
    if (rc != HFRK_SUCCESS) return rc;
    return hfrk::gemm_launch(A, B, D, D, scale_tensor, 0, nullptr, 0, nullptr, m, n, k, b_stride, d_dtype,
                             HFRK_EPILOGUE_NONE, nullptr, static_cast<hipStream_t>(stream));
}

int hfrk_skinny_gemm_ex(const void* A, const void* B, void* D, const float* scale_a, int sa_stride,
                        const float* scale_b, int sb_stride, int m, int n, int k, int b_stride, int d_dtype,
                        int accumulate, const hfrk_gemm_plan* plan, void* stream) {
    return hfrk::gemm_launch(A, B, D, accumulate ? D : nullptr, scale_a, sa_stride, scale_b, sb_stride, nullptr, m, n, k,
                             b_stride, d_dtype, HFRK_EPILOGUE_NONE, plan, static_cast<hipStream_t>(stream));
}

int hfrk_skinny_gemm_noalloc(const void* A, const void* B, void* D, const float* scale_a, int sa_stride,
                             const float* scale_b, int sb_stride, int m, int n, int k, int b_stride, int d_dtype,
                             int accumulate, const hfrk_gemm_plan* plan, void* stream) {
    return hfrk::gemm_launch(A, B, D, accumulate ? D : nullptr, scale_a, sa_stride, scale_b, sb_stride, nullptr, m, n, k,
                             b_stride, d_dtype, HFRK_EPILOGUE_NONE, plan, static_cast<hipStream_t>(stream), false, true);
}

int hfrk_skinny_gemm_fused(const void* A, const void* B, void* D, const void* base, const float* scale_a, int sa_stride,
                           const float* scale_b, int sb_stride, const float* out_scale, int m, int n, int k,
                           int b_stride, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream) {
    return hfrk::gemm_launch(A, B, D, base, scale_a, sa_stride, scale_b, sb_stride, out_scale, m, n, k, b_stride, d_dtype,
                             epilogue, plan, static_cast<hipStream_t>(stream));
}

int hfrk_skinny_gemm_rms_plan(int m, int n, int k, int epilogue, hfrk_gemm_plan* plan) {
    if (!plan || (epilogue != HFRK_EPILOGUE_NONE && epilogue != HFRK_EPILOGUE_SWIGLU)) return HFRK_INVALID_CONFIG;
    return hfrk::make_rms_plan(m, n, k, epilogue == HFRK_EPILOGUE_SWIGLU, plan);
}

int hfrk_skinny_gemm_rms_fused(const void* input, const void* residual, void* residual_out, const void* rms_weight,
                               float epsilon, const float* act_scale, int io_dtype, const void* B, void* D, const void* base,
                               const float* scale_a, const float* scale_b, int sb_stride, const float* out_scale, int m, int n,
                               int k, int b_stride, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream) {
    const hfrk::RmsPrologue rms{input, residual, residual_out, rms_weight, act_scale, epsilon, io_dtype};
    return hfrk::gemm_launch(nullptr, B, D, base, scale_a, 0, scale_b, sb_stride, out_scale, m, n, k, b_stride, d_dtype, epilogue,
                             plan, static_cast<hipStream_t>(stream), false, false, &rms);
}

int hfrk_skinny_gemm_packed(const void* A, const void* B_packed, void* D, const void* base, const float* scale_a,
                            int sa_stride, const float* scale_b, int sb_stride, const float* out_scale, int m, int n,
                            int k, int d_dtype, int epilogue, const hfrk_gemm_plan* plan, void* stream) {
    if (sb_stride == HFRK_SCALES_IN_PACKED_BUFFER) {  // the per-channel scales hfrk_pack_weight_scaled stored behind the bytes
        scale_b = hfrk_packed_weight_scales(B_packed, n, k);
        if (!scale_b) return k % 256 != 0 ? HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K : HFRK_BAD_SHAPE;
        sb_stride = 1;
    }
    return hfrk::gemm_launch(A, B_packed, D, base, scale_a, sa_stride, scale_b, sb_stride, out_scale, m, n, k, k, d_dtype,
                             epilogue, plan, static_cast<hipStream_t>(stream), true);
}

}  // extern "C"
