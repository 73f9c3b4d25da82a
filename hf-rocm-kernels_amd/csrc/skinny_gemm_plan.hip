// Host-side planner of the FP8 skinny GEMM (declarations and what each function is for: skinny_gemm_plan.h).  The rules are
// measurements on MI355X, quoted where they are applied, not a model.
#include "skinny_gemm_plan.h"

namespace hfrk {


// m <= 32: every wave streams its own run of (16*RT-row group, 256-byte K chunk) chunks (skinny_gemm_stream.hip).
int fill_stream_plan(int m, int n, int k, int row_tiles, bool swiglu, int grid_hint, hfrk_gemm_plan* plan) {
    const int act_loads = (m + 3) / 4;
    if (!stream_variant_exists(act_loads, row_tiles, swiglu)) return HFRK_INVALID_CONFIG;
    const long tiles = (n + 16 * row_tiles - 1) / (16 * row_tiles);  // swiglu: n/2 output columns in tiles of 16
    if (tiles > kMaxPanels) return HFRK_BAD_SHAPE;
    const int kc = (k + 255) / 256;  // the last chunk of a row may be cut short (row-major weights, k % 16 == 0)
    const long chunks = tiles * kc;
    long grid = grid_hint > 0 ? grid_hint : kNumCU;
    if (grid > chunks) grid = chunks;
    if (grid >= 8) grid -= grid % 8;  // whole XCD groups
    // A grid that divides the row tiles keeps every tile inside one workgroup (no workspace round trip).  Worth the idle
    // CUs in two cases, both measured: at least three quarters of the CUs and short runs (under 64 chunks per workgroup
    // on the full grid; 6144 x 4096 on 192), or one or two tiles per workgroup with runs of at most 80 chunks, down to
    // 160 workgroups (3584 x 18944 on 224: 13.7 against 16.4 us; 5120 x 5120 on 160: 8.0 against 9.0).  On longer runs
    // the round trip is small against the CUs left idle (13312 x 16384: 43.6 us on 208 against 39.7 on 256).
    if (grid_hint <= 0 && grid == kNumCU && tiles % kNumCU != 0)
        for (long g = kNumCU - 8; g >= 5 * kNumCU / 8; g -= 8) {
            if (tiles % g != 0) continue;
            const bool short_runs = g >= 3 * kNumCU / 4 && chunks < 64L * kNumCU;
            const bool few_tiles = tiles / g <= 2 && chunks / g <= 80;
            if (short_runs || few_tiles) { grid = g; break; }
        }
    // When every workgroup's share of the weight is a multiple of 512 KB, all workgroups walk addresses that agree in
    // their low 19 bits at the same time and crowd onto a few memory channels (16384 x 8192: 30.5 us on 256 workgroups,
    // 24.8 on 248; 16384 x 16384: 54.3 against 45.8; rows padded by 256 bytes have the same effect).  A grid of 248 breaks
    // the alignment.
    if (grid_hint <= 0 && grid == kNumCU && (chunks * row_tiles * kTileBytes) % ((long)kNumCU << 19) == 0) grid = kNumCU - 8;
    plan->m_tiles = (act_loads + 3) / 4;
    plan->wn = 0;
    plan->wk = row_tiles;
    plan->ch = act_loads;
    plan->grid = (int)grid;
    plan->panels = (int)tiles;
    plan->slabs = kc;
    plan->lds_bytes = stream_lds_bytes(act_loads, row_tiles);
    return HFRK_SUCCESS;
}

static int make_stream_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    const int act_loads = (m + 3) / 4;
    // Two row tiles per chunk halve the activation bytes pulled from L2 per weight byte: needed above 16 rows,
    // worth it from 9 rows on once a wave's run still has a few 8 KB chunks and a row group has at least 16 of them
    // (k >= 4096; on 32768 x 2048 at 16 rows one tile per chunk takes 12.9 us, two take 14.5).
    int row_tiles = 1;
    if (act_loads > 4) {
        row_tiles = 2;
    } else if (act_loads >= 3 && k >= 4096) {
        const long chunks2 = (long)((n + 31) / 32) * ((k + 255) / 256);
        if (chunks2 >= (long)kStreamRt2MinChunksPerWave * kNumCU * kGemmWaves) row_tiles = 2;
    }
    return fill_stream_plan(m, n, k, row_tiles, false, 0, plan);
}

// m <= 16: every workgroup owns a band of weight rows (4-row units dealt out evenly) and all of k (skinny_gemm_rows.hip).
// plan: wn = -2, wk = matrix tiles per chunk, ch = activation loads, panels = 4-row units, slabs = k / 256.
int fill_rows_plan(int m, int n, int k, int row_tiles, int grid_hint, hfrk_gemm_plan* plan) {
    const int act_loads = rows_act_loads(m);
    if (m > kRowsMaxM || !rows_variant_exists(act_loads, row_tiles) || k < 512 || k % 256 != 0) return HFRK_INVALID_CONFIG;
    const long units = (n + 3) / 4;
    long grid = grid_hint > 0 ? grid_hint : kNumCU;
    if (grid > units) grid = units;
    if (grid >= 8 && grid_hint <= 0) grid -= grid % 8;
    plan->m_tiles = 1;
    plan->wn = -2;
    plan->wk = row_tiles;
    plan->ch = act_loads;
    plan->grid = (int)grid;
    plan->panels = (int)units;
    plan->slabs = k / 256;
    plan->lds_bytes = rows_lds_bytes(row_tiles, act_loads);
    return HFRK_SUCCESS;
}

// The planner takes the row-split decomposition when there is at least one 4-row unit per workgroup and the busiest
// workgroup is at most 40 % above the mean (2304 x 16384, 2.25 units per workgroup: 9.5 us against 10.3 for the wave-stream
// split).  Sweeps over 23 weight shapes say what else matters:
//  * tiles that are not full (a band height that is no multiple of 16 rows) cost 3-11 %, because a wave keeps one chunk
//    in flight and a 12-row chunk is 3 KB instead of 4.  So a grid between 224 and 256 that gives every workgroup whole
//    16-row tiles is taken when there is one (3584 rows: 224 workgroups, 4.6 against 5.2 us); otherwise, up to 4
//    activation rows and bands of at most 48 rows, twice the workgroups with half the band each put more bytes in flight
//    (6144 x 4096: 6.05 against 6.5 us; 10240 x 8192: 14.9 against 15.6; no gain from 5 rows on, where the activation
//    loads of 16 waves per CU weigh in);
//  * two matrix tiles per chunk from 9 rows on, once a band has 24 rows to fill them (57344 x 8192 at 16 rows: 72.3
//    against 79.5 us; 4096 x 4096, 16 rows per band: 5.7 against 6.3 the other way).
int make_rows_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    if (m > kRowsMaxM || k < 512 || k % 256 != 0) return HFRK_INVALID_CONFIG;
    const long units = (n + 3) / 4;
    if (units < kNumCU) return HFRK_INVALID_CONFIG;
    long grid = kNumCU;
    const long busiest = (units + grid - 1) / grid;
    if (units * 10 < busiest * grid * 7) return HFRK_INVALID_CONFIG;
    // A band of exactly 512 KB (every workgroup's weight bytes, rows a power of two apart) is the one size at which the
    // workgroups, walking their bands in step, keep landing on the same memory channels even with the start in k rotated:
    // 0.65 of peak where the neighbouring sizes reach 0.75-0.78 (16384 x 8192, 8192 x 16384, 32768 x 4096: 25.5-25.7 us;
    // 256 KB, 1 MB and 1.5 MB bands are fine).  Two matrix tiles per chunk walk it differently (22.0-22.7 us), and a grid
    // that would create such bands is not taken for the sake of whole tiles (14336 x 8192: 22.4 us on 224 workgroups,
    // 19.4 on 256).
    auto half_mb_bands = [&](long g) { return units % g == 0 && 4 * (units / g) * (long)k == (1L << 19); };
    // Bands of 20..44 rows that are no multiple of 16 cut into one or two chunks per 256 bytes of k with two matrix tiles per
    // chunk instead of two or three (20 rows: one 5 KB chunk instead of 3 + 2 KB), which pays from 5 rows on once k is long
    // enough: 5120 x 8192 9.3 against 9.7 us at 8 rows and 9.8 against 11.1 at 16, 5120 x 16384 15.9 / 16.6 against 16.9 / 19.3,
    // 10240 x 8192 15.8 against 16.3 at 8, 11264 x 16384 31.0 against 32.4; at k = 5120 from 9 rows on (5120 x 5120 at 16: 7.9
    // against 8.5) and below on bands of 36+ rows (10240 x 5120 at 8: 11.1 against 11.6; 6144 x 5120 8.0 against 7.8 the other
    // way); level at k = 3072 and on bands of 52 rows (13312 x 16384).
    // On long k such bands also beat a smaller grid of whole tiles (7168 x 14336 at 8 rows: 18.1 us on 256 against 19.2 on 224).
    auto ragged = [&](long band) {
        if (m < 5) return band == 20 && k >= 8192;  // (5120 x 8192 / 14336 / 16384 at 1 row: 9.0 / 13.7 / 15.6 us against 9.4 / 14.3 / 16.3 on 512 workgroups)
        return band > 16 && band <= 48 && band % 16 != 0 && (k >= 8192 || (k >= 5120 && (band >= 36 || m >= 9)));
    };
    if (units % (4 * grid) != 0 && !(k >= 8192 && ragged(4 * busiest))) {
        long whole = 0;
        for (long g = kNumCU - 8; g >= 7 * kNumCU / 8; g -= 8)
            if (units % (4 * g) == 0 && !half_mb_bands(g)) { whole = g; break; }
        if (whole) grid = whole;
        else if (m <= 4 && 4 * busiest <= 48 && units >= 4 * kNumCU) grid = 2 * kNumCU;  // bands of at least 8 rows
    }
    const long rows_per_band = 4 * ((units + grid - 1) / grid);
    const bool ragged_band = ragged(rows_per_band) && (m >= 5 || grid == kNumCU);
    const int row_tiles = (m > 16 || (m >= 9 && rows_per_band >= 24) || (half_mb_bands(grid) && rows_per_band >= 24) || ragged_band) ? 2 : 1;
    return fill_rows_plan(m, n, k, row_tiles, (int)grid, plan);
}

// The row-split decomposition on bands of whole 16-row tiles (skinny_gemm_rows_tiled.hip), the form a weight in the packed
// load format can take: plan wn = -3, wk = 16-row tiles per chunk, ch = activation loads, panels = 16-row tiles, slabs = k / 256.
int fill_rows_tiled_plan(int m, int n, int k, int row_tiles, int grid_hint, hfrk_gemm_plan* plan) {
    const int act_loads = rows_act_loads(m);
    if (m > kRowsMaxM || !rows_variant_exists(act_loads, row_tiles) || k < 512 || k % 256 != 0) return HFRK_INVALID_CONFIG;
    const long tiles = (n + 15) / 16;
    long grid = grid_hint > 0 ? grid_hint : kNumCU;
    if (grid > tiles) grid = tiles;
    plan->m_tiles = 1;
    plan->wn = -3;
    plan->wk = row_tiles;
    plan->ch = act_loads;
    plan->grid = (int)grid;
    plan->panels = (int)tiles;
    plan->slabs = k / 256;
    plan->lds_bytes = rows_lds_bytes(row_tiles, act_loads);
    return HFRK_SUCCESS;
}

// Packed weights up to 16 activation rows.  Rules read off a sweep of every decomposition over the Llama-3 8B / 70B weights:
//  * the busiest workgroup's tile count is what it is on 256 workgroups, ceil(tiles / 256); the grid is the smallest
//    multiple of 8 from 192 on that keeps it (6144 x 4096: 384 tiles, 2 each on 192 workgroups, 6.5 us against 6.9 on 256;
//    10240 x 8192: 640 tiles, up to 3 each on 216..240 workgroups, 15.9 us against 16.5 on 256);
//  * two tiles per chunk from 9 rows on when a band has two, and at any row count on k above 16384 (8192 x 28672: 37.7 us
//    against 39.4 at 8 rows);
//  * not on the largest weights (57344 x 8192: 73.6-76.5 us against 72.8 for the workgroup kernel and 68.5 for the row-major
//    weight -- a run of 56 contiguous chunks per wave is the slowest way to read that much memory).
//  * from 144 tiles (2304 rows, the smallest weight measured) on, one tile per workgroup: 2304..3040 rows x k = 2048..14336 at 1 /
//    8 / 16 rows are 4-49 % faster than the wave-stream split and, at k = 2048, 0-37 % faster than the K-split kernel (2304 x
//    4096: 4.3 / 4.6 / 5.0 us against 6.3 / 6.5 / 6.7; 3040 x 2048: 3.6 / 4.0 / 4.2 against 4.9 / 5.0 / 5.0; 2304 x 14336 at 16 rows,
//    10.9 against 10.3, is the one case behind), so the rule comes before the K-split rule for small weights.
int make_rows_tiled_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    if (m > 16 || k < 512 || k % 256 != 0) return HFRK_INVALID_CONFIG;
    const long tiles = (n + 15) / 16;
    if (tiles < 9 * kNumCU / 16 || (long)n * k > (256L << 20)) return HFRK_INVALID_CONFIG;
    const long busiest = (tiles + kNumCU - 1) / kNumCU;
    long grid = (tiles + busiest - 1) / busiest;
    grid = (grid + 7) / 8 * 8;
    if (grid < 3 * kNumCU / 4) grid = 3 * kNumCU / 4;
    if (grid > kNumCU) grid = kNumCU;
    if (grid > tiles) grid = tiles;
    if (tiles * 10 < ((tiles + grid - 1) / grid) * grid * 7) return HFRK_INVALID_CONFIG;  // busiest at most 40 % above the mean
    const long band_tiles = (tiles + grid - 1) / grid;
    const int row_tiles = (band_tiles >= 2 && (m >= 9 || k > 16384)) ? 2 : 1;
    return fill_rows_tiled_plan(m, n, k, row_tiles, (int)grid, plan);
}

// Packed weights at 17..32 rows (two activation tiles, two weight tiles per chunk): the grid.  One tile each while there are
// at most 256 tiles; one pair of tiles each from 160 pairs on (5120 rows on 160 workgroups, 6144 on 192); more pairs only
// where they deal out evenly over 192..256 workgroups (13312 rows: 2 pairs each on 208).  Uneven deals of more than 256
// pairs are left to the other kernels (10240 rows, 320 pairs: 3-9 % behind them on 192 workgroups at k = 3072, 5120, 14336).
static int make_rows_tiled_pairs_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    if (m <= 16 || m > kRowsMaxM || k < 512 || k % 256 != 0) return HFRK_INVALID_CONFIG;
    const long tiles = (n + 15) / 16, pairs = (tiles + 1) / 2;
    long grid = 0;
    if (tiles <= kNumCU) {
        grid = tiles;
    } else if (pairs <= kNumCU) {
        grid = pairs >= 5 * kNumCU / 8 ? pairs : kNumCU;
    } else {
        for (long g = kNumCU; g >= 3 * kNumCU / 4 && !grid; g -= 8)
            if (tiles % 2 == 0 && pairs % g == 0) grid = g;
        if (!grid) return HFRK_INVALID_CONFIG;
    }
    return fill_rows_tiled_plan(m, n, k, 2, (int)grid, plan);
}

// 17 <= m <= 64 (valid from 1): the waves of a workgroup split K windows of 8*wave_k bytes, activations in registers
// (skinny_gemm_ksplit.hip).  wave_k 512 keeps twice the bytes in flight and halves the window count, 256 makes
// twice the units: take the one whose busiest workgroup streams fewer bytes.
static int fill_ksplit_plan(int m, int n, int k, int wave_k, int grid_hint, hfrk_gemm_plan* plan) {
    const int mt = (m + 15) / 16;
    if (!ksplit_variant_exists(mt, wave_k)) return HFRK_INVALID_CONFIG;
    if (k % (8 * wave_k) != 0) return HFRK_INVALID_CONFIG;
    const long tiles = (n + 15) / 16, windows = k / (8 * wave_k);
    const long units = tiles * windows;
    if (tiles * mt > kMaxPanels) return HFRK_BAD_SHAPE;                          // one arrival counter per 16x16 tile
    if (windows > 1 && (size_t)units * mt * 256 > kWsFloats) return HFRK_BAD_SHAPE;  // a 16x16 fp32 share per unit and tile
    long grid = grid_hint > 0 ? grid_hint : kNumCU;
    if (grid > units) grid = units;
    if (grid >= 8) grid -= grid % 8;
    plan->m_tiles = mt;
    plan->wn = -1;
    plan->wk = wave_k / 256;
    plan->ch = 0;
    plan->grid = (int)grid;
    plan->panels = (int)tiles;
    plan->slabs = (int)windows;
    plan->lds_bytes = ksplit_lds_bytes(mt, wave_k);
    return HFRK_SUCCESS;
}

// The planner uses this decomposition only when one window of 256 or 512 bytes per wave covers K (k = 2048 or 4096):
// then a unit is finished inside its workgroup.  With several windows every unit makes a workspace round trip
// (store, acknowledge, counter) on the critical path of its workgroup, and with 1 KB per wave (k = 8192, up to 32
// rows) the kernel sits at 254 registers; measured, the workgroup kernel is faster in both cases.
int make_ksplit_plan(int m, int n, int k, hfrk_gemm_plan* plan) {
    if (k != 2048 && k != 4096) return HFRK_INVALID_CONFIG;
    return fill_ksplit_plan(m, n, k, k / 8, 0, plan);
}

// Which decomposition for which shape.  The rules are measurements on MI355X over the Llama-3 8B/70B linears
// (sweeps of every decomposition at m = 1..64), not a model:
//   m <= 16          row-split kernel (a band of weight rows and all of k per workgroup) when the rows deal out evenly,
//                    else the wave-stream kernel (chunk runs that may split a tile's k between workgroups); K-split kernel
//                    for weights of at most 2048 chunks (8 MB) when one window of it covers k
//   17 <= m <= 32    row-split kernel with two activation tiles on bands of 12-64 rows and moderate k (rule below), behind
//                    whole 64-row panels of the workgroup kernel from 12288 weight rows on
//   m  > 16          workgroup kernel on whole row panels per workgroup where they deal out evenly (make_whole_panel_plan);
//                    K-split kernel (activations in registers) when one window of it covers k; otherwise the
//                    workgroup kernel, which stages the activation slab once per workgroup in LDS:
//                    4 row waves x 2 K waves almost everywhere; 2 x 4 on k = 16384 (n >= 8192, up to 48 rows) and
//                    for narrow weights (n <= 2048: more K parallelism
//                    where there are few row panels; from 2304 rows on 4 x 2 is 6-15 % faster, measured on 2304..5120 x
//                    8192..16384 at m = 32, 48); 8 x 1 for 49+ rows on the largest weights (fewest reductions)
// workgroup decomposition with wn row waves x (8 / wn) K waves and ch chunks per slab, on min(256, units) workgroups
static int fill_workgroup_plan(int m, int n, int k, int wn, int ch, hfrk_gemm_plan* plan) {
    const int mt = (m + 15) / 16, wk = kGemmWaves / wn, ks = 256 * wk * ch;
    if (k % ks != 0 || lds_bytes_for(mt, wk, ch) > kLdsLimit) return HFRK_INVALID_CONFIG;
    const long panels = (n + 16 * wn - 1) / (16 * wn);
    if (panels > kMaxPanels) return HFRK_BAD_SHAPE;
    const long slabs = k / ks, units = panels * slabs;
    // Small weights (a workgroup's run of units shorter than a panel): a grid under which every run is a whole fraction of
    // a panel.  Runs that straddle panel boundaries add contributors to both panels' exchanges (3072 x 8192 at 32 / 64
    // rows: 768 units are 3 per workgroup on 256, cutting the 16-slab panels unevenly, 12.1 / 15.0 us; 4 per workgroup on
    // 192, 9.8 / 12.4 us; 6144 x 5120 at 64 rows: 17.8 on 256, 15.0 on 192).  Down to 192 workgroups; longer runs keep the
    // full grid (20480 x 8192: 36.0 us on 160 workgroups with whole panels against 34.6 on 256).
    long grid = units < kNumCU ? units : kNumCU;
    if (units > kNumCU)
        for (long g = kNumCU; g >= 3 * kNumCU / 4; g -= 8) {
            if (units % g != 0) continue;
            const long per = units / g;
            if (per < slabs && slabs % per == 0) { grid = g; break; }
        }
    plan->m_tiles = mt;
    plan->wn = wn;
    plan->wk = wk;
    plan->ch = ch;
    plan->grid = (int)grid;
    plan->panels = (int)panels;
    plan->slabs = k / ks;
    plan->lds_bytes = lds_bytes_for(mt, wk, ch);
    return HFRK_SUCCESS;
}

// 17+ rows: when the row panels of the workgroup kernel deal out evenly over 224..256 workgroups, every workgroup owns whole
// panels and all of k for them -- no split of k between workgroups, no exchange at the end of the launch -- and the
// activation slab is staged once for 8 waves.  The tallest panel that divides wins: 256 rows (8 row waves, two weight
// tiles each), 128 (8 row waves) or 64 (4 row waves x 2 K waves).  Against the planner's other choice at 32 / 48 / 64 rows:
// 57344 x 8192 (224 panels of 256 rows) 75.8 / 77.0 / 79.0 us against 79.8 / 84.3 / 91.1; 28672 x 8192 (224 of 128) 38.9 /
// 40.8 / 42.5 against 43.9 / 46.2 / 55.8; 28672 x 4096 22.4 / 23.9 / 25.4 against 24.4 / 25.0 / 27.0 (K-split kernel);
// 32768 x 4096 24.7 / 26.4 / 28.3 against 27.6 / 28.2 / 30.2; 16384 x 4096 (256 panels of 64) 14.3 / 15.7 / 17.4 against
// 16.0 / 16.7 / 18.2; 14336 x 4096 (224 of 64) 13.5 / 14.9 / 16.5 against 15.3 / 15.9 / 17.1.  Up to k = 8192: on 16384 x
// 16384 (a megabyte of weights per 64-row panel) the rules below are 6-7 % ahead.
// One panel per workgroup also on 160..216 workgroups: idle compute units cost in proportion to the bytes, the exchange
// they save does not, and the other rules' deal over 256 is uneven for such row counts.  At 32 / 48 / 64 rows, against the
// rules below:
//   64-row panels, the shorter k the fewer workgroups: 10240 rows on 160 workgroups 10.0 / 11.5 / 12.9 us against 13.7 / 16.4 /
//   17.7 at k = 3072 and 14.9 / 16.9 / 18.5 against 16.4 / 18.7 / 20.1 at 5120, level at 8192, 4-11 % behind at 14336; 12288
//   rows on 192: 26-30 % ahead at 3072, 5-10 % at 8192 (level at 64 rows), level at 14336; 13312 rows on 208: 28-36 % ahead
//   at 3072, 22-29 % at 8192, 13-17 % at 14336, level at 16384.  At k = 4096 the K-split kernel is 4-8 % ahead of 160 / 192
//   such workgroups from 33 rows on;
//   128-row panels (taken first): 24576 rows on 192 workgroups 16.0 / 17.7 / 18.8 against 18.8 / 21.7 / 23.9 at k = 3072, 35.0
//   / 37.8 / 39.9 against 36.3 / 39.9 / 43.1 at 8192, 64.2 / 68.1 / 71.5 against 70.5 / 78.3 / 82.4 at 16384 (level at 14336);
//   20480 rows on 160: 15.0 / 16.7 / 17.8 against 17.3 / 19.7 / 21.3 at 3072, 32.4 / 35.4 / 37.4 against 34.4 / 36.7 / 38.3
//   at 8192, behind from 14336 on and behind the K-split kernel at 4096;
//   k = 16384 up to 48 rows: 64-row panels with two chunks per slab, 14336 rows on 224 workgroups 41.9 / 43.7 us against 44.9
//   / 49.8, 16384 rows on 256 46.8 / 48.5 against 47.4 / 52.2 (with one chunk per slab it is 6-7 % behind there).
static int make_whole_panel_plan(int m, int n, int k, hfrk_gemm_plan* plan, bool packed = false) {
    const int mt = (m + 15) / 16;
    const int heights[4] = {256, 128, 64, 32};
    for (int hi = 0; hi < 4; ++hi) {
        const int h = heights[hi];
        if (n % h != 0) continue;
        const long panels = n / h;
        // 32-row panels (2 row waves x 4 K waves), one each on 160..256 workgroups: short k that no K-split window covers, up to
        // 48 rows (8192 x 3072 9.7 / 10.1 us at 33 / 48 rows against 11.2 / 11.4, 7168 x 5120 12.5 / 13.1 against 13.5 / 14.0,
        // 6144 x 3072 on 192 workgroups 9.2 / 9.6 against 10.6 / 10.9, 5120 x 5120 on 160 11.8 / 12.4 against 12.9 / 13.1; at
        // 64 rows level or 9 % behind, at k = 8192 18-27 % behind, at k = 2048 / 4096 7-24 % behind the K-split kernel)
        if (h == 32 && (panels > kNumCU || k > 5120 || k == 2048 || k == 4096 || m > 48)) continue;
        // (a packed 128-row panel at k = 8192 is 1 MB of contiguous bytes per workgroup: 28672 x 8192 at 20 / 32 rows 48.9 / 48.0 us
        // against 41.0 / 41.8 on 64-row panels, two per workgroup; 24576 x 8192 42.0 against 36.4 for the rules below)
        if (h == 128 && packed && k == 8192) continue;
        long g_try[2] = {0, 0};  // several panels each on 224..256 workgroups; one panel each on fewer
        if (k <= 8192)
            for (long g = kNumCU; g >= 7 * kNumCU / 8 && !g_try[0]; g -= 8)
                if (panels % g == 0) g_try[0] = g;
        // (what the rules below choose from 25 rows on; at 64 rows 8 row waves are 3 % ahead on 16384 x 14336)
        if (h == 64 && k > 8192 && k <= 14336 && panels == kNumCU && m <= 48) g_try[0] = panels;
        if (h == 64 && k == 16384 && m <= 48 && panels == kNumCU) g_try[0] = panels;
        if (panels % 8 == 0 && panels < kNumCU) {
            bool one_each = false;
            if (h == 64) one_each = panels >= (k <= 5120 ? 160 : k <= 8192 ? 192 : 208) && k <= 14336 && !(k == 4096 && m > 32 && panels < 208);
            if (h == 64 && k == 16384 && m <= 48) one_each = panels >= 208;
            if (h == 128) one_each = panels >= 192 || (panels >= 160 && k <= 8192 && k != 4096 && k != 2048);
            if (h == 32) one_each = panels >= 160;
            if (one_each) g_try[1] = panels;
        }
        for (int gi = 0; gi < 2; ++gi) {
            const long g = g_try[gi];
            if (g == 0) continue;
            const int wn = h == 32 ? 2 : h == 64 ? 4 : 8, wk = kGemmWaves / wn, rt = h == 256 ? 2 : 1;
            // two chunks per slab on short k with 8 row waves (28672 x 4096 at 64 rows: 25.4 against 26.5 us), else one
            int ch = ((wn == 8 && rt == 1 && k <= 5120 && k % 512 == 0) || (wn == 4 && k > 14336)) ? 2 : 1;
            if (lds_bytes_for(mt, wk, ch, rt) > kLdsLimit) ch = 1;
            const int ks = 256 * wk * ch;
            if (k % ks != 0 || lds_bytes_for(mt, wk, ch, rt) > kLdsLimit || panels > kMaxPanels) continue;
            plan->m_tiles = mt;
            plan->wn = wn * rt;
            plan->wk = wk;
            plan->ch = ch;
            plan->grid = (int)g;
            plan->panels = (int)panels;
            plan->slabs = k / ks;
            plan->lds_bytes = lds_bytes_for(mt, wk, ch, rt);
            return HFRK_SUCCESS;
        }
    }
    return HFRK_INVALID_CONFIG;
}

// Long k (14336, 16384): 128-row panels, 8 row waves, each panel's k cut between 2 or 4 workgroups, on the 192..256
// workgroups that makes.  Against the other rules at 32 / 48 / 64 rows: 6144 x 16384 (4 x 48 panels) 21.5 / 24.3 / 25.8 us
// against 25.3 / 28.4 / 30.4 and 5-7 % ahead at k = 14336; 13312 x 16384 (2 x 104) 39.7 / 42.0 / 45.0 against 42.8 / 48.1 /
// 50.1; 12288 x 16384 (2 x 96) 3-5 % ahead; 8192 x 16384 (4 x 64) 29.8 against 35.9 at 64 rows, but 3-4 % behind 2 row
// waves x 4 K waves up to 48 rows, so all 256 workgroups only from 49 rows on.
static int make_split_panel_plan(int m, int n, int k, hfrk_gemm_plan* plan, bool packed) {
    if (k < 14336 || k > 16384 || n % 128 != 0) return HFRK_INVALID_CONFIG;
    const long panels = n / 128, slabs = k / 256;
    for (int f = 2; f <= 4; f += 2) {
        const long g = panels * f;
        if (g < 3 * kNumCU / 4 || g > kNumCU || g % 8 != 0 || slabs % f != 0 || (g == kNumCU && (m <= 48 || packed))) continue;  // (packed 8192 x 16384 at 64 rows: 30.6 us against 29.6)
        if (fill_workgroup_plan(m, n, k, 8, 1, plan) != HFRK_SUCCESS) return HFRK_INVALID_CONFIG;
        plan->grid = (int)g;
        return HFRK_SUCCESS;
    }
    return HFRK_INVALID_CONFIG;
}

int make_plan(int m, int n, int k, hfrk_gemm_plan* plan, bool packed) {
    if (m < 1 || m > HFRK_GEMM_MAX_M || n < 1 || k < 1) return HFRK_BAD_SHAPE;
    if (k % 16 != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
    if (k % 256 != 0) {
        // A row that ends inside a 256-byte chunk: a variant of the wave-stream kernel masks the missing pieces (row-major
        // weights, up to 32 activation rows; a call with more rows runs as two launches, see gemm_launch).
        if (packed || m > kStreamMaxM) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
        return make_stream_plan(m, n, k, plan);
    }
    // k = 1024 is four chunks per row tile: too few for the wave-stream split and half a K-split window.  Four K waves
    // cover it in one slab, so nothing is exchanged between workgroups (1024 x 1024: 4.2 against 5.2 us at 1 row,
    // 5120 x 1024: 5.7 against 7.3 at 32 rows); on weights wider than 12288 rows the other kernels catch up.
    if (k == 1024 && n <= 12288 && fill_workgroup_plan(m, n, k, 2, 1, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;
    if (m <= 16) {
        // Small weights: with at most one 4 KB chunk per wave the wave-stream split leaves waves idle and sends every row
        // tile through the workspace; one workgroup per tile, its 8 waves splitting K, finishes inside the workgroup
        // (2048 x 2048: 3.8 against 5.2 us; 2048 x 4096: 5.0 against 5.8).
        const long chunks = (long)((n + 15) / 16) * (k / 256);
        if (packed && make_rows_tiled_plan(m, n, k, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;  // bands of whole 16-row tiles
        // (from 2304 rows on, the smallest weight measured against it, the row-split kernel is ahead of that rule as well: 2304..4096
        // x 2048 at 1 / 8 / 16 rows 3.4-3.95 / 3.7-4.2 / 3.9-4.3 us against 3.8-4.3 / 4.0-4.5 / 4.1-4.6)
        if (!packed && n >= 2304 && make_rows_plan(m, n, k, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;
        if (chunks <= (long)kNumCU * kGemmWaves && make_ksplit_plan(m, n, k, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;
        // Bands of rows per workgroup: nothing crosses workgroups and the end of the launch is short (0.3-1.3 us less than
        // the wave-stream split on every Llama-3 8B / 70B projection at 1..16 rows).
        if (!packed && make_rows_plan(m, n, k, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;  // (bands of any multiple of 4 rows: row-major weights only)
        return make_stream_plan(m, n, k, plan);
    }
    // 17..32 rows in the row-split kernel (two activation tiles): every workgroup then pulls all m x k activation bytes out
    // of L2 itself, which pays while a band's chunks stay large against them and k is moderate.  Measured against the
    // kernels below at 24 / 32 rows: 6144 x 4096 7.96 / 8.70 us against 9.54 / 9.55 (K-split, 1.5 tiles per workgroup),
    // 8192 x 8192 13.5 / 14.3 against 15.2 / 15.2, 10240 x 8192 18.5 against 19.4 at 24, 13312 x 16384 38.2 against 41.0 at
    // 24, 16384 x 2048 8.9 against 10.3; slower on bands of 16 rows (4096 x 14336 +2 / +12 %), on k = 28672 (+3 / +7 %), at
    // 32 rows with k = 16384 (8192 x 16384: 27.0 us against 25.3 for 2 row waves x 4 K waves below; bands of 40 rows and more
    // +6 to +8 %) and on the largest weights (57344 x 8192 +9 %, 32768 x 8192 +16 %).
    // Bands of 12-20 rows (3072..5120 weight rows) on k up to 8192 as well, where the kernels below deal their units
    // unevenly: 5120 x 5120 8.95 / 9.2 / 9.9 / 10.1 us at 20 / 24 / 28 / 32 rows against 11.3-11.6, 3072 x 3072 6.7 / 6.8 /
    // 7.3 / 7.35 against 8.5, 4096 x 5120 8.4 / 8.5 / 9.2 / 9.35 against 9.8-9.9, 5120 x 8192 11.0 / 11.3 / 12.1 / 12.4 against
    // 13.7-13.8.  Not where one K-split window covers k and its tiles deal out evenly (3072 and 4096 rows at k = 2048 and
    // 4096: level or 0.3-0.9 us behind), nor above 24 rows at k = 8192 on bands under 20 rows or at k = 2048.
    // Packed weights first take the kernel where pairs of tiles deal out evenly over 256 workgroups on a weight of at most 64 MiB
    // (at 20-24 / 32 rows: 8192 x 8192 13.9 / 14.8 us against 16.4 / 16.1 for the kernels below, 16384 x 4096 13.7 / 14.5 against
    // 17.4 / 17.4, 8192 x 4096 9.0 / 9.4 against 9.5 / 9.5), and otherwise follow the same rule on bands of whole tiles
    // (make_rows_tiled_pairs_plan).  A sweep of 11 row counts x 5 k at 20 and 32 rows: where the rule takes the kernel the
    // packed weight gains 2-35 % over the kernels below (3072 x 3072 6.3 / 6.8 us against 8.5, 4096 x 5120 8.1 / 8.9 against 9.7,
    // 5120 x 8192 11.5 / 12.9 against 14.0, 6144 x 8192 11.9 against 13.5 at 20 rows, 13312 x 4096 12.2 against 13.9) or is level;
    // where it does not, the kernel is 3-14 % behind.  On a packed weight whole 64-row
    // panels do not come first at k = 4096 (13312 / 14336 x 4096 at 20 rows: 12.1 / 12.5 us against 13.9 / 14.4).
    if (m <= kRowsMaxM && packed && n % 16 == 0 && (n / 16) % (2 * kNumCU) == 0 && k >= 4096 && (long)n * k <= (64L << 20) &&
        fill_rows_tiled_plan(m, n, k, 2, kNumCU, plan) == HFRK_SUCCESS)
        return HFRK_SUCCESS;
    if (m <= kRowsMaxM) {
        const long band_rows = 4 * (((long)(n + 3) / 4 + kNumCU - 1) / kNumCU);
        // (k = 2048 above 24 rows: the K-split kernel is 3-4 % ahead, 6144 x 2048 6.5 against 6.7 us)
        bool fits = band_rows >= 24 && (m <= 24 ? (band_rows <= 64 && k <= 16384) : (band_rows <= 32 && k >= 3072 && k <= 8192));
        if (band_rows >= 12 && band_rows < 24 && k >= (m <= 24 ? 2048 : 3072) && k <= 8192)
            fits = ((k != 2048 && k != 4096) || band_rows >= 20) && (m <= 24 || k < 8192 || band_rows >= 20);
        // From 12288 weight rows on, whole 64-row panels per workgroup come first where they exist: at 20 / 24 rows 12288 x
        // 8192 19.8 / 20.0 us against 20.5 / 21.2, 13312 x 8192 20.6 / 20.8 against 21.7 / 22.2, 14336 x 5120 15.7 / 15.8 against
        // 17.2 / 17.7, 16384 x 14336 39.4 / 39.2 against 42.1 / 43.3; level at k = 4096 and 16384 and on 10240 rows.
        if (fits && band_rows >= 48 && k != 2048 && k < 16384 && !(packed && k == 4096) &&
            make_whole_panel_plan(m, n, k, plan, packed) == HFRK_SUCCESS)
            return HFRK_SUCCESS;
        if (fits && (packed ? make_rows_tiled_pairs_plan(m, n, k, plan) : make_rows_plan(m, n, k, plan)) == HFRK_SUCCESS) return HFRK_SUCCESS;
    }
    if (k >= 16384 && make_split_panel_plan(m, n, k, plan, packed) == HFRK_SUCCESS) return HFRK_SUCCESS;
    if (make_whole_panel_plan(m, n, k, plan, packed) == HFRK_SUCCESS) return HFRK_SUCCESS;
    if (make_split_panel_plan(m, n, k, plan, packed) == HFRK_SUCCESS) return HFRK_SUCCESS;
    if (make_ksplit_plan(m, n, k, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;
    const double weight_mb = (double)n * k / 1.0e6;
    // 2 x 4 also on k = 16384 from 8192 rows on (up to 48 activation rows: 8192 x 16384 25.3 against 27+ us at 32 and 27.8
    // against 34.5 at 48; 10240 / 12288 / 16384 / 20480 / 24576 x 16384 at 32: 5-9 % faster; 13312 x 16384 equal; not on
    // k = 28672, where 8192 x 28672 takes 43.1 us with it against 39.9).
    // 8 x 1 from 220 MB on: 12288 x 16384 and 24576 x 8192 (201 MB) take 44.6 / 42.6 us with 4 x 2 against 50.3 / 47.0,
    // 8192 x 28672 (235 MB) and 16384 x 16384 (268 MB) are 1-6 % faster with 8 x 1.
    int first = 4;
    if (m <= 48 && (n <= 2048 || (k >= 16384 && k < 24576 && n >= 8192))) first = 2;
    else if (weight_mb >= 220.0 && m > 48) first = 8;
    const int prefs[3][4] = {{2, 4, 1, 8}, {4, 2, 8, 1}, {8, 4, 2, 1}};
    const int* pref = first == 2 ? prefs[0] : first == 4 ? prefs[1] : prefs[2];
    for (int pi = 0; pi < 4; ++pi)
        for (int ch = 1; ch <= 2; ++ch)
            if (fill_workgroup_plan(m, n, k, pref[pi], ch, plan) == HFRK_SUCCESS) return HFRK_SUCCESS;
    return HFRK_BAD_SHAPE;
}

int check_plan(int m, int n, int k, bool swiglu, const hfrk_gemm_plan* p, bool packed) {
    if (swiglu && p->wn != 0 && p->wn != -2 && p->wn != -1 && p->wn != -3) return HFRK_INVALID_CONFIG;  // the workgroup kernel has no fused epilogue
    if (p->wn == -3) {  // row-split on bands of whole 16-row tiles, either weight layout: wk = tiles per chunk, ch = activation loads
        if (swiglu && p->wk != 2) return HFRK_INVALID_CONFIG;
        if (m > kRowsMaxM || !rows_variant_exists(p->ch, p->wk) || 4 * p->ch < m || k < 512) return HFRK_INVALID_CONFIG;
        if (k % 256 != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
        if (p->m_tiles != 1 || p->panels != (n + 15) / 16 || p->slabs != k / 256) return HFRK_INVALID_CONFIG;
        if (p->grid < 1 || p->grid > kMaxStreamGrid || p->grid > p->panels) return HFRK_INVALID_CONFIG;
        if (p->lds_bytes != rows_lds_bytes(p->wk, p->ch)) return HFRK_INVALID_CONFIG;
        if (((long)p->panels / p->grid + 2) * p->slabs * p->slabs >= (1L << 31)) return HFRK_BAD_SHAPE;  // as below
        return HFRK_SUCCESS;
    }
    if (p->wn == -2) {  // row-split decomposition: wk = matrix tiles per chunk, ch = activation loads
        if (packed) return HFRK_INVALID_CONFIG;  // bands of any 4-row height do not fit the packed format's 16-row tiles
        if (swiglu && p->wk != 2) return HFRK_INVALID_CONFIG;  // n counts output columns; a chunk holds their gate and their up rows
        if (m > kRowsMaxM || !rows_variant_exists(p->ch, p->wk) || 4 * p->ch < m || k < 512) return HFRK_INVALID_CONFIG;
        if (k % 256 != 0) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;
        if (p->m_tiles != 1 || p->panels != (n + 3) / 4 || p->slabs != k / 256) return HFRK_INVALID_CONFIG;
        if (p->grid < 1 || p->grid > kMaxStreamGrid || p->grid > p->panels) return HFRK_INVALID_CONFIG;
        if (p->lds_bytes != rows_lds_bytes(p->wk, p->ch)) return HFRK_INVALID_CONFIG;
        // a band's chunk indices stay far below 2^32 / slabs (the kernel divides by multiplying with a reciprocal)
        if (((long)p->panels / p->grid / 4 + 2) * p->slabs * p->slabs >= (1L << 31)) return HFRK_BAD_SHAPE;
        return HFRK_SUCCESS;
    }
    if (k % 256 != 0 && (packed || p->wn != 0)) return HFRK_K_NOT_DIVISIBLE_BY_WARPTILE_K;  // only the wave-stream kernel cuts a chunk short
    if (p->wn == -1) {  // K-split decomposition: wk = wave_k / 256
        hfrk_gemm_plan want;
        const int rc = fill_ksplit_plan(m, n, k, p->wk * 256, p->grid, &want);
        if (rc != HFRK_SUCCESS) return rc;
        if (p->grid < 1 || p->grid > kNumCU || p->grid > (long)want.panels * want.slabs) return HFRK_INVALID_CONFIG;
        if (p->m_tiles != want.m_tiles || p->ch != 0 || p->panels != want.panels || p->slabs != want.slabs ||
            p->lds_bytes != want.lds_bytes)
            return HFRK_INVALID_CONFIG;
        if (swiglu && (want.slabs != 1 || p->wk > 2)) return HFRK_INVALID_CONFIG;  // gate and up sums meet inside one workgroup
        if ((long)want.panels * want.slabs * (p->grid + 1) >= (1L << 31)) return HFRK_BAD_SHAPE;
        return HFRK_SUCCESS;
    }
    if (p->wn == 0) {  // wave-stream decomposition: wk = row tiles per chunk, ch = activation loads
        if (m > kStreamMaxM || !stream_variant_exists(p->ch, p->wk, swiglu) || 4 * p->ch < m) return HFRK_INVALID_CONFIG;
        if (p->m_tiles != (p->ch + 3) / 4) return HFRK_INVALID_CONFIG;
        const int rows = swiglu ? 16 : 16 * p->wk;  // with the SwiGLU epilogue n counts output columns: one gate + one up tile
        if (p->panels != (n + rows - 1) / rows || p->slabs != (k + 255) / 256 || p->panels > kMaxPanels) return HFRK_INVALID_CONFIG;
        const long chunks = (long)p->panels * p->slabs;
        if (p->grid < 1 || p->grid > kMaxStreamGrid || p->grid > chunks) return HFRK_INVALID_CONFIG;
        if (chunks * (p->grid + 1) >= (1L << 31)) return HFRK_BAD_SHAPE;  // the kernel's chunk arithmetic is 32-bit
        if (p->lds_bytes != stream_lds_bytes(p->ch, p->wk)) return HFRK_INVALID_CONFIG;
        return HFRK_SUCCESS;
    }
    if (p->m_tiles < 1 || p->m_tiles > 4 || p->m_tiles * 16 < m) return HFRK_INVALID_CONFIG;
    // wn counts the 16-row tiles of a panel: one per row wave (wn * wk = 8) or, with one chunk per slab, two (wn * wk = 16)
    if (!(p->wk == 1 || p->wk == 2 || p->wk == 4 || p->wk == 8)) return HFRK_INVALID_CONFIG;
    const int rt = p->wn * p->wk / kGemmWaves;
    if (p->wn < 1 || p->wn * p->wk != rt * kGemmWaves || (rt != 1 && rt != 2)) return HFRK_INVALID_CONFIG;
    if (p->ch != 1 && p->ch != 2) return HFRK_INVALID_CONFIG;
    if (rt == 2 && p->ch != 1) return HFRK_INVALID_CONFIG;  // registers
    const int ks = 256 * p->wk * p->ch, bn = 16 * p->wn;
    if (k % ks != 0 || p->slabs != k / ks || p->panels != (n + bn - 1) / bn) return HFRK_INVALID_CONFIG;
    if (p->panels > kMaxPanels) return HFRK_INVALID_CONFIG;
    const long units = (long)p->panels * p->slabs;
    // One workgroup per compute unit at most: with more, workgroups of up to 160 KB of LDS run in two rounds over shared
    // partial-sum slots and arrival counters, a regime no test of this kernel covers (see kMaxStreamGrid).
    if (p->grid < 1 || p->grid > kNumCU || p->grid > units) return HFRK_INVALID_CONFIG;
    if (units * (p->grid + 1) >= (1L << 31)) return HFRK_BAD_SHAPE;  // the kernel's unit arithmetic is 32-bit
    if (p->lds_bytes != lds_bytes_for(p->m_tiles, p->wk, p->ch, rt) || p->lds_bytes > kLdsLimit) return HFRK_INVALID_CONFIG;
    return HFRK_SUCCESS;
}


// Workspace bytes and arrival counters a plan's kernel may touch (the kernels' own slot arithmetic, 1 KB per 16x16 fp32 tile).
size_t plan_ws_bytes(const hfrk_gemm_plan& p) {
    if (p.wn <= -2) return 0;  // row-split: nothing crosses workgroups
    if (p.wn == 0) return (size_t)p.grid * 2 * (p.wk * ((p.ch + 3) / 4)) * 1024;  // two slots per workgroup, row tiles x activation tiles
    if (p.wn == -1) return p.slabs > 1 ? (size_t)p.panels * p.slabs * p.m_tiles * 1024 : 0;  // one share per unit and activation tile
    return (size_t)p.grid * 2 * (p.wn * p.m_tiles) * 1024;  // two slots per workgroup, a panel's tiles x activation tiles
}
long plan_counters(const hfrk_gemm_plan& p) { return p.wn <= -2 ? 0 : p.wn == -1 ? (long)p.panels * p.m_tiles : p.panels; }


// The plan of a launch with the RMSNorm prologue: the row-split plan of the shape with one matrix tile per chunk (SwiGLU:
// the gate and the up tile), whatever the planner or the plan table would take for the plain GEMM.  HFRK_BAD_SHAPE where the
// prologue does not exist: more than 8 rows, k other than 4096 or 8192 (every thread of a workgroup owns one or two 16-byte
// pieces of each row), rows that do not deal out over the workgroups.
int make_rms_plan(int m, int n, int k, bool swiglu, hfrk_gemm_plan* p) {
    if (m < 1 || m > kRowsRmsMaxM || (k != 4096 && k != 8192) || n < 1 || (swiglu && n % 32 != 0)) return HFRK_BAD_SHAPE;
    const int n_eff = swiglu ? n / 2 : n;
    if (make_rows_plan(m, n_eff, k, p) != HFRK_SUCCESS || p->grid <= m) return HFRK_BAD_SHAPE;
    return fill_rows_plan(m, n_eff, k, swiglu ? 2 : 1, p->grid, p);
}

}  // namespace hfrk
