"""Address audit of the four GEMM kernels on the host, no GPU.

Every address a kernel forms is restated here from the kernel sources (csrc/skinny_gemm*.hip) and checked against the
object it points into, for every workgroup, wave and extreme lane of a launch:

  * buffer-resource offsets (weights, activations, outputs, workspace): an access the kernel means to make lies inside
    [0, num_records); an access it means to suppress (a row past n, a unit past the workgroup's range, an activation
    row past m) lies at or beyond num_records as an unsigned 32-bit number, where the hardware returns zeros / drops the
    store -- in particular no such offset wraps round 2^32 back into the buffer;
  * raw-pointer accesses (arrival counters, the workgroup kernel's output stores): the index is inside the array;
  * LDS: every region a kernel carves out of its dynamic LDS ends at or below the plan's lds_bytes;
  * workspace slots: every share written lies below plan_ws_bytes, and the shares the last arriver reads are exactly
    the shares the contributors wrote (same workgroup, same slot), whose arrival counts add up to the number that makes
    somebody last -- also when the grid is larger than the number of compute units and workgroups run in two rounds.

The plans audited include the ones a tuner sweep once forced on 2048-row weights with 4 activation rows (every
decomposition, grids 192..512, per-tensor scale with a null channel-scale pointer) before that run ended in a GPU fault:
the enumeration of that sweep is restated below as it was then, although the library now refuses part of it.
"""
import ctypes
import itertools

import pytest

from hf_rocm_kernels import _capi

U32 = 1 << 32
OOR = 0x80000000          # the kernels' "out of range" base offset
TILE = 4096
WS_BYTES = 2 * 1024 * 8 * 4 * 256 * 4   # kWsFloats * 4
MAX_PANELS = 1 << 20
LANES = [(li, lg) for li in (0, 15) for lg in (0, 3)]   # extreme lanes: offsets are monotone in li and lg


class Buf:
    """A buffer resource of `records` bytes: check an access the kernel intends (live) or suppresses (not live)."""

    def __init__(self, name, records):
        self.name, self.records, self.hits = name, records, 0
        assert 0 <= records < (1 << 31), (name, records)

    def access(self, off, size, live, what=None):
        off %= U32
        inside = off + size <= self.records
        if live:
            assert inside, (self.name, "live access out of range", off, size, self.records, what)
            self.hits += 1
        else:
            assert not inside, (self.name, "suppressed access lands inside the buffer", off, size, self.records, what)


def plan_ws_bytes(p):
    if p.wn == -2:
        return 0
    if p.wn == 0:
        return p.grid * 2 * (p.wk * ((p.ch + 3) // 4)) * 1024
    if p.wn == -1:
        return p.panels * p.slabs * p.m_tiles * 1024 if p.slabs > 1 else 0
    return p.grid * 2 * (p.wn * p.m_tiles) * 1024


def plan_counters(p):
    return 0 if p.wn == -2 else p.panels * p.m_tiles if p.wn == -1 else p.panels


def xcd_ids(G):
    """blockIdx -> logical workgroup id: a bijection for every grid."""
    ids = [((b & 7) * (G >> 3) + (b >> 3)) if G % 8 == 0 else b for b in range(G)]
    assert sorted(ids) == list(range(G))
    return ids


# ---------------------------------------------------------------------------------------------------------------------
# workgroup kernel (skinny_gemm.hip, skinny_gemm_kernel)
def audit_workgroup(m, n, k, b_stride, p, packed=False):
    rt = p.wn * p.wk // 8
    WN, WK, CH, MT = p.wn // rt, p.wk, p.ch, p.m_tiles
    assert WN * WK == 8 and rt in (1, 2)
    KS, BN, ST = 256 * WK * CH, 16 * WN * rt, rt * MT
    S, P, G = p.slabs, p.panels, p.grid
    U = S * P
    assert U * (G + 1) < (1 << 31) and G <= U
    # LDS: 8 waves x rt transposition tiles, then two activation slabs
    ACT = 16 * MT * KS
    assert 8 * rt * TILE + 2 * ACT == p.lds_bytes <= 160 * 1024
    KP = KS // 16
    for row in (0, 16 * MT - 1):      # act_store: dst + row*KS + (kp>>4)*256 + ((kp&15)^(row&15))<<4, 16 bytes
        for kp in (0, KP - 1):
            assert row * KS + (kp >> 4) * 256 + (((kp & 15) ^ (row & 15)) << 4) + 16 <= ACT
    assert ST * 64 * 16 <= rt * TILE  # K-wave reduction borrows a wave's own tiles
    w = Buf("weights", ((n + 15) // 16) * k * 16 if packed else (n - 1) * b_stride + k)
    a = Buf("activations", m * k)
    ws = Buf("workspace", WS_BYTES)
    need_ws, need_ctr = plan_ws_bytes(p), plan_counters(p)
    assert need_ws <= WS_BYTES and need_ctr <= MAX_PANELS
    ub = lambda g: (g * U) // G
    written = {}    # (panel) -> list of (g, slot, slabs)
    stored = set()  # panels stored directly
    xcd_ids(G)
    for g in range(G):
        u0, u1 = ub(g), ub(g + 1)
        assert u0 < u1
        assert (g * U) % U32 == g * U  # unit_begin is 32-bit
        for u in range(u0, u1):
            ip, is_ = divmod(u, S)
            phys = (is_ + ip % S) % S
            assert 0 <= phys < S
            for wave in range(8):
                wn, wk = divmod(wave, WK)
                for r in range(rt):
                    tile = ip * (WN * rt) + wn * rt + r
                    for c in (0, CH - 1):
                        if packed:
                            chunk = tile * (k >> 8) + phys * (WK * CH) + c * WK + wk
                            for t in (0, 3):
                                for lane in (0, 63):
                                    w.access(chunk * TILE + lane * 16 + t * 1024, 16, tile * 16 < ((n + 15) // 16) * 16)
                        else:
                            base = tile * 16 * b_stride + phys * KS + (c * WK + wk) * 256
                            for t in (0, 3):
                                for li, lg in LANES:
                                    row = tile * 16 + 4 * t + lg
                                    w.access(lg * b_stride + li * 16 + base + 4 * t * b_stride, 16, row < n, (g, u, wave))
            # activation slab of the unit: pieces idx = tid + q*512 < 16*MT*KP
            for idx in (0, 16 * MT * KP - 1):
                row, kp = divmod(idx, KP)
                a.access(row * k + phys * KS + kp * 16, 16, row < m)
        # the unit past the end of the range (prefetch depth 2): out of range by construction
        for lane_off in (0, 3 * b_stride + 240 + 12 * b_stride):
            w.access(OOR + lane_off, 16, False)
        a.access(OOR + (16 * MT - 1) * k + (KP - 1) * 16, 16, False)
        # panels this workgroup closes
        first_panel = u0 // S
        for panel in range(u0 // S, (u1 - 1) // S + 1):
            lo, hi = max(u0, panel * S), min(u1, (panel + 1) * S)
            assert panel < need_ctr or (lo == panel * S and hi == (panel + 1) * S)
            if lo == panel * S and hi == (panel + 1) * S:
                stored.add(panel)
                continue
            slot = 0 if panel == first_panel else 1
            for wn in range(WN):
                for st in (0, ST - 1):
                    off = (((g * 2 + slot) * (WN * ST) + wn * ST + st) * 64 + 63) * 16
                    assert off + 16 <= need_ws
                    ws.access(off, 16, True)
            written.setdefault(panel, []).append((g, slot, hi - lo))
    # the last arriver's view of every split panel
    for panel, shares in written.items():
        assert panel not in stored
        assert sum(s for _, _, s in shares) == S          # somebody sees seen + mine == S, exactly once
        lo, hi = panel * S, (panel + 1) * S
        assert ((lo + 1) * G + U - 1) < U32 and (hi * G + U - 1) < U32
        g_first = ((lo + 1) * G + U - 1) // U - 1
        g_last = (hi * G + U - 1) // U - 1
        read = [(gg, 0 if ub(gg) // S == panel else 1) for gg in range(g_first, g_last + 1)]
        assert read == [(g, s) for g, s, _ in shares], (panel, read, shares)
    assert stored | set(written) == set(range(P))
    # output: raw pointers guarded by mrow < m and n0 + v < n; the largest index a live lane forms
    n0_max = (P - 1) * BN + (WN * rt - 1) * 16 + 12 + 3
    assert min(n0_max, n - 1) + (m - 1) * n < m * n
    return w.hits


# ---------------------------------------------------------------------------------------------------------------------
# wave-stream kernel (skinny_gemm_stream.hip)
def audit_stream(m, n, k, b_stride, p, packed=False):
    RT, MA = p.wk, p.ch
    MT = (MA + 3) // 4
    SUB = RT * MT
    KC, T, G = p.slabs, p.panels, p.grid
    C = KC * T
    assert C * (G + 1) < (1 << 31) and G <= C and 4 * MA >= m
    wave_lds = (RT + MT) * TILE
    assert 8 * wave_lds == p.lds_bytes <= 160 * 1024
    assert SUB * 64 * 16 <= RT * TILE or SUB * 64 * 16 <= wave_lds   # partial-sum slots inside the wave's own tiles
    w = Buf("weights", ((n + 15) >> 4) * KC * TILE if packed else (n - 1) * b_stride + k)
    a = Buf("activations", m * k)
    need_ws = plan_ws_bytes(p)
    assert need_ws <= WS_BYTES and T <= MAX_PANELS
    cq, cr = divmod(C, G)
    ragged_k = k % 256 != 0
    written = {}
    finished = [0] * T
    xcd_ids(G)
    for g in range(G):
        c0 = g * cq + min(g, cr)
        nwg = cq + (1 if g < cr else 0)
        c1 = c0 + nwg
        assert nwg >= 1
        segs = {}   # tile -> [first chunk, end) this workgroup holds
        for wv in range(8):
            w0, w1 = c0 + wv * nwg // 8, c0 + (wv + 1) * nwg // 8
            for c in {w0, w1 - 1} if w1 > w0 else ():
                tile, kc = divmod(c, KC)
                last = ragged_k and kc == KC - 1
                for li, lg in LANES:
                    beyond = last and (KC - 1) * 256 + li * 16 >= k
                    for t in (0, MA - 1):
                        row = 4 * t + lg
                        a.access((OOR if beyond else 0) + lg * k + li * 16 + kc * 256 + 4 * t * k, 16, row < m and not beyond)
                    for t in (0, 4 * RT - 1):
                        if packed:
                            tl = tile * RT + t // 4
                            w.access((tl * KC + kc) * TILE + (t % 4) * 1024 + (lg * 16 + li) * 16, 16, tl < (n + 15) >> 4)
                        else:
                            row = tile * 16 * RT + 4 * t + lg
                            w.access((OOR if beyond else 0) + lg * b_stride + li * 16 + tile * 16 * RT * b_stride + kc * 256 + 4 * t * b_stride,
                                     16, row < n and not beyond)
        for t in range(c0 // KC, (c1 - 1) // KC + 1):
            lo, hi = max(c0, t * KC), min(c1, (t + 1) * KC)
            if lo == t * KC and hi == (t + 1) * KC:
                finished[t] += 1
                continue
            slot = 0 if c0 >= t * KC else 1
            off = (((g * 2 + slot) * SUB + SUB - 1) * 64 + 63) * 16
            assert off + 16 <= need_ws
            written.setdefault(t, []).append((g, slot, hi - lo))
    owner = lambda c: c // (cq + 1) if c < cr * (cq + 1) else cr + (c - cr * (cq + 1)) // cq
    for t, shares in written.items():
        assert finished[t] == 0 and sum(s for _, _, s in shares) == KC
        g_first, g_last = owner(t * KC), owner(t * KC + KC - 1)
        sl_first = 0 if g_first * cq + min(g_first, cr) == t * KC else 1
        read = [(gg, sl_first if gg == g_first else 0) for gg in range(g_first, g_last + 1)]
        assert read == [(g, s) for g, s, _ in shares], (t, read, shares)
    assert all(finished[t] == 1 or t in written for t in range(T))
    return w.hits


# ---------------------------------------------------------------------------------------------------------------------
# K-split kernel (skinny_gemm_ksplit.hip)
def audit_ksplit(m, n, k, b_stride, p, packed=False):
    MT, KW = p.m_tiles, 256 * p.wk
    KCH = KW // 256
    T, S, G = p.panels, p.slabs, p.grid
    U = T * S
    assert k == S * 8 * KW and T == (n + 15) // 16 and G <= U and G <= 256 and U * (G + 1) < (1 << 31)
    assert 8 * KCH * TILE + 2 * 8 * MT * 64 * 16 == p.lds_bytes <= 160 * 1024
    w = Buf("weights", T * k * 16 if packed else (n - 1) * b_stride + k)
    a = Buf("activations", m * k)
    need_ws, need_ctr = plan_ws_bytes(p), plan_counters(p)
    assert need_ws <= WS_BYTES and need_ctr <= MAX_PANELS
    uq, ur = divmod(U, G)
    arrivals = {}
    xcd_ids(G)
    for g in range(G):
        u0 = g * uq + min(g, ur)
        count = uq + (1 if g < ur else 0)
        assert count >= 1
        for u in range(u0, u0 + count):
            win, tile = divmod(u, T)
            assert win < S
            for wv in (0, 7):
                for c in (0, KCH - 1):
                    if packed:
                        chunk = tile * (k >> 8) + (win * 8 + wv) * KCH + c
                        w.access(chunk * TILE + 3 * 1024 + 63 * 16, 16, True)
                    else:
                        base = tile * 16 * b_stride + win * 8 * KW
                        for t in (0, 3):
                            for li, lg in LANES:
                                row = tile * 16 + 4 * t + lg
                                w.access(lg * b_stride + wv * KW + li * 16 + base + 4 * t * b_stride + c * 256, 16, row < n)
                    for mt in (0, MT - 1):   # the window's activations
                        for t in (0, 3):
                            for li, lg in LANES:
                                row = mt * 16 + 4 * t + lg
                                off = row * k + win * 8 * KW + wv * KW + li * 16 + c * 256 if row < m else OOR
                                a.access(off, 16, row < m)
            if S > 1:
                for wv in range(MT):
                    slot = (win * T + tile) * MT + wv
                    assert (slot * 64 + 63) * 16 + 16 <= need_ws
                    assert tile * MT + wv < need_ctr
                    arrivals.setdefault((tile, wv), []).append(win)
    for (tile, wv), wins in arrivals.items():
        assert sorted(wins) == list(range(S))   # ticket S-1 is drawn exactly once; the reader walks windows 0..S-1
    return w.hits


# ---------------------------------------------------------------------------------------------------------------------
# row-split kernel (skinny_gemm_rows.hip)
def audit_rows(m, n, k, b_stride, p, swiglu=False):
    RT, MA = p.wk, p.ch
    MT = (MA + 3) // 4
    G, units, KC = p.grid, p.panels, p.slabs
    per_tile = 4 if swiglu else 4 * RT
    assert units == (n + 3) // 4 and KC == k // 256 and k % 256 == 0 and G <= units and 4 * MA >= m
    wave_lds = (RT + MT) * TILE
    assert 8 * wave_lds == p.lds_bytes <= 160 * 1024
    assert MT * RT * 64 * 16 <= RT * TILE   # a wave's partial sums fit the start of its own weight tiles
    # (SwiGLU: n counts the output columns; the weight has 2n rows, gate rows first)
    n_rows = 2 * n if swiglu else n
    w = Buf("weights", (n_rows - 1) * b_stride + k)
    a = Buf("activations", m * k)
    q, r = divmod(units, G)
    xcd_ids(G)
    for g in range(G):
        nu, u0 = q + (1 if g < r else 0), g * q + min(g, r)
        T = -(-nu // per_tile)
        base, extra = nu // T, nu % T
        TC = T * KC
        rot_cases = (0, g % KC)
        for wv in range(8):
            i0, i1 = (wv * TC) >> 3, ((wv + 1) * TC) >> 3
            for i in {i0, i1 - 1} if i1 > i0 else ():
                j, kc = divmod(i, KC)
                height = base + (1 if j < extra else 0)
                row0 = 4 * (u0 + j * base + min(j, extra))
                for rot in rot_cases:
                    kr = (kc + rot) % KC
                    for li, lg in LANES:
                        for t in (0, MA - 1):
                            a.access(lg * k + li * 16 + kr * 256 + 4 * t * k, 16, 4 * t + lg < m)
                        for t in range(4 * RT):
                            unit = t % 4 if swiglu else t
                            rowoff = 4 * unit + (t // 4) * n if swiglu else 4 * t
                            row = row0 + rowoff + lg
                            if unit < height:
                                w.access(lg * b_stride + li * 16 + row0 * b_stride + kr * 256 + rowoff * b_stride, 16, row - (t // 4) * n < n if swiglu else row < n)
                            else:
                                w.access(lg * b_stride + li * 16 + OOR, 16, False)
    return w.hits


# ---------------------------------------------------------------------------------------------------------------------
# row-split kernel on bands of whole 16-row tiles (skinny_gemm_rows_tiled.hip), row-major and packed weights
def audit_tiles(m, n, k, b_stride, p, swiglu=False, packed=False):
    RT, MA = p.wk, p.ch
    MT = (MA + 3) // 4
    G, tiles, KC = p.grid, p.panels, p.slabs
    PT = 4 if swiglu else 4 * RT       # 4-row units per chunk
    assert tiles == (n + 15) // 16 and KC == k // 256 and k % 256 == 0 and k >= 512 and G <= min(tiles, 512) and 4 * MA >= m
    wave_lds = (RT + MT) * TILE
    assert 8 * wave_lds == p.lds_bytes <= 160 * 1024
    assert MT * RT * 64 * 16 <= RT * TILE   # a wave's partial sums fit the start of its own weight tiles
    n_rows = 2 * n if swiglu else n
    w = Buf("weights", ((n_rows + 15) >> 4) * KC * TILE if packed else (n_rows - 1) * b_stride + k)
    a = Buf("activations", m * k)
    q, r = divmod(tiles, G)
    xcd_ids(G)
    for g in range(G):
        nt, t0 = q + (1 if g < r else 0), g * q + min(g, r)
        band_units, u0 = 4 * nt, 4 * t0
        T = -(-band_units // PT)
        TC = T * KC
        for wv in range(8):
            i0, i1 = (wv * TC) >> 3, ((wv + 1) * TC) >> 3
            for i in {i0, i1 - 1} if i1 > i0 else ():
                j, kc = divmod(i, KC)
                units, row0 = min(PT, band_units - PT * j), 4 * (u0 + PT * j)
                assert units >= 4 and units % 4 == 0 and row0 % 16 == 0
                for rot in (0, g % KC):
                    kr = (kc + rot) % KC
                    for li, lg in LANES:
                        for t in (0, MA - 1):
                            a.access(lg * k + li * 16 + kr * 256 + 4 * t * k, 16, 4 * t + lg < m)
                        for t in range(4 * RT):
                            if packed:   # piece t % 4 of 16-row tile t // 4 of the chunk
                                tile16 = (row0 >> 4) + (t // 4) * ((2 * n) >> 5 if swiglu else 1)
                                if swiglu or 4 * (t // 4) < units:
                                    w.access((tile16 * KC + kr) * TILE + (t % 4) * 1024 + (lg * 16 + li) * 16, 16, True)
                                else:
                                    w.access(OOR, 16, False)
                            else:
                                unit = t % 4 if swiglu else t
                                rowoff = 4 * unit + (t // 4) * n if swiglu else 4 * t
                                row = row0 + rowoff + lg
                                if unit < units:
                                    w.access(lg * b_stride + li * 16 + (row0 + rowoff) * b_stride + kr * 256, 16,
                                             row - (t // 4) * n < n if swiglu else row < n)
                                else:
                                    w.access(lg * b_stride + li * 16 + OOR, 16, False)
    return w.hits


def audit(m, n, k, p, packed=False):
    if p.wn == -2:
        return audit_rows(m, n, k, k, p)
    if p.wn == -3:
        return audit_tiles(m, n, k, k, p, packed=packed)
    if p.wn == 0:
        return audit_stream(m, n, k, k, p, packed)
    if p.wn == -1:
        return audit_ksplit(m, n, k, k, p, packed)
    return audit_workgroup(m, n, k, k, p, packed)


# ---------------------------------------------------------------------------------------------------------------------
def sweep_plans_as_the_tuner_once_made_them(m, n, k, grids):
    """The enumeration of the tuner at the time of the faulting sweep: grids up to 512 (two-tile workgroup plans) and 1024."""
    mt = (m + 15) // 16
    plans = []
    if m <= 32:
        ma, kc = (m + 3) // 4, k // 256
        for rt in (1, 2):
            if (rt == 1 and ma <= 4) or (rt == 2 and 3 <= ma <= 8):
                groups = -(-n // (16 * rt))
                for g in grids:
                    plans.append(_capi.GemmPlan((ma + 3) // 4, 0, rt, ma, min(g, groups * kc), groups, kc, 8 * (rt + (ma + 3) // 4) * 4096))
    if m <= 32 and k >= 512:
        units = -(-n // 4)
        ma = (m + 3) // 4 if m <= 16 else (6 if m <= 24 else 8)
        for rt in ((1, 2) if m <= 16 else (2,)):
            for g in grids:
                plans.append(_capi.GemmPlan(1, -2, rt, ma, min(g, units), units, k // 256, 8 * (rt + (ma + 3) // 4) * 4096))
    for wave_k in (256, 512, 1024):
        if k % (8 * wave_k) == 0 and (wave_k < 1024 or mt <= 2):
            tiles, windows = -(-n // 16), k // (8 * wave_k)
            if windows > 1 and tiles * windows * mt * 256 > 2 * 1024 * 8 * 4 * 256:
                continue
            for g in grids:
                plans.append(_capi.GemmPlan(mt, -1, wave_k // 256, 0, min(g, 256, tiles * windows), tiles, windows,
                                            8 * (wave_k // 256) * 4096 + 16 * mt * 1024))
    for wn, ch, rt in itertools.product((1, 2, 4, 8), (1, 2), (1, 2)):
        wk = 8 // wn
        ks = 256 * wk * ch
        lds = 8 * rt * 4096 + 2 * 16 * mt * ks
        if k % ks or lds > 160 * 1024 or (rt == 2 and ch != 1):
            continue
        panels, slabs = -(-n // (16 * wn * rt)), k // ks
        for g in grids:
            plans.append(_capi.GemmPlan(mt, wn * rt, wk, ch, min(g, panels * slabs, 512 if rt == 2 else 1024), panels, slabs, lds))
    return plans


@pytest.mark.parametrize("k", [2048, 4096, 28672])
def test_every_plan_of_the_sweep_that_faulted_stays_inside_its_buffers(k):
    m, n = 4, 2048
    plans = sweep_plans_as_the_tuner_once_made_them(m, n, k, [192, 224, 256, 512])
    kinds = set()
    for p in plans:
        assert audit(m, n, k, p) > 0, p.as_dict()
        kinds.add(p.wn if p.wn <= 0 else 1)
    assert kinds == {-2, -1, 0, 1}
    if k == 28672:  # (the two smaller weights have at most 256 units of work for that kernel)
        assert any(p.grid > 256 and p.wn > 0 for p in plans)   # including workgroup plans that run in two rounds per compute unit


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (8, 6144, 4096), (16, 28672, 4096), (32, 4096, 14336), (64, 8192, 8192),
                                   (40, 1000, 2048), (17, 50, 256), (8, 1027, 768), (33, 4100, 1024), (64, 57344, 8192),
                                   (5, 130, 512), (24, 8192, 8192), (48, 8192, 28672)])
def test_planner_and_forced_plans_stay_inside_their_buffers(m, n, k):
    """The planner's own plan and every plan the sweep tool proposes today, in both weight layouts where they exist."""
    from hf_rocm_kernels.benchmarks.skinny_gemm import grid_search
    plans = [_capi.plan(m, n, k)] + grid_search.candidate_plans(m, n, k, [7, 200, 256, 512])
    for p in plans:
        if p.panels * p.slabs > 300000:
            continue   # (a Python loop over units)
        assert audit(m, n, k, p) > 0, p.as_dict()
        if p.wn != -2 and k % 256 == 0:
            assert audit(m, n, k, p, packed=True) > 0, p.as_dict()
    if k % 256 == 0 and m <= 16:
        lib = _capi.load()
        p = _capi.GemmPlan()
        assert lib.hfrk_plan_table_get(m, n, k, 1, ctypes.byref(p)) == _capi.SUCCESS   # the planner's answer for a packed weight
        assert audit(m, n, k, p, packed=True) > 0, p.as_dict()


def test_k_that_ends_inside_a_chunk_and_padded_row_strides():
    p = _capi.plan(8, 4096, 4096 + 128)
    assert p.wn == 0 and audit(8, 4096, 4096 + 128, p) > 0
    p = _capi.plan(3, 130, 144)
    assert audit(3, 130, 144, p) > 0
    for m, n, k, stride in [(8, 1000, 1024, 1024 + 256), (32, 512, 2048, 4096), (64, 777, 4096, 4096 + 16)]:
        p = _capi.plan(m, n, k)
        fn = {-2: audit_rows, -3: audit_tiles, 0: audit_stream, -1: audit_ksplit}.get(p.wn, audit_workgroup)
        assert fn(m, n, k, stride, p) > 0


def test_swiglu_bands_of_the_row_split_kernel():
    """SwiGLU epilogue: bands count the n/2 output columns, a chunk holds their gate rows and, n/2 rows further down, their up rows."""
    for m, n_out, k in [(8, 14336, 4096), (16, 2080, 512), (1, 28672, 8192)]:
        units = -(-n_out // 4)
        p = _capi.GemmPlan(1, -2, 2, (m + 3) // 4, min(256, units), units, k // 256, 8 * 3 * 4096)
        assert audit_rows(m, n_out, k, k, p, swiglu=True) > 0
        tiles = -(-n_out // 16)
        p = _capi.GemmPlan(1, -3, 2, (m + 3) // 4, min(200, tiles), tiles, k // 256, 8 * 3 * 4096)
        assert audit_tiles(m, n_out, k, k, p, swiglu=True) > 0
        assert audit_tiles(m, n_out, k, k, p, swiglu=True, packed=True) > 0


def test_library_refuses_grids_no_test_covers():
    """More than one workgroup per compute unit: accepted for the row-split and wave-stream kernels up to 512 (the planner uses
    it, forced plans of that size are GPU-tested), refused for the K-split and workgroup kernels and beyond 512 everywhere."""
    lib = _capi.load()
    m, n, k = 4, 2048, 28672
    try_plan = lambda p: lib.hfrk_plan_table_set(m, n, k, 0, ctypes.byref(p))
    try:
        wg = lambda grid: _capi.GemmPlan(1, 8, 1, 1, grid, n // 128, k // 256, 8 * 4096 + 2 * 16 * 256)
        assert try_plan(wg(256)) == _capi.SUCCESS
        assert try_plan(wg(257)) == _capi.INVALID_CONFIG and try_plan(wg(512)) == _capi.INVALID_CONFIG
        two_tiles = lambda grid: _capi.GemmPlan(1, 16, 1, 1, grid, n // 256, k // 256, 2 * 8 * 4096 + 2 * 16 * 256)
        assert try_plan(two_tiles(256)) == _capi.SUCCESS and try_plan(two_tiles(512)) == _capi.INVALID_CONFIG
        ks = lambda grid: _capi.GemmPlan(1, -1, 1, 0, grid, n // 16, k // 2048, 8 * 4096 + 16 * 1024)
        assert try_plan(ks(256)) == _capi.SUCCESS and try_plan(ks(264)) == _capi.INVALID_CONFIG
        rows = lambda grid: _capi.GemmPlan(1, -2, 1, 1, grid, n // 4, k // 256, 8 * 2 * 4096)
        assert try_plan(rows(512)) == _capi.SUCCESS and try_plan(rows(513)) == _capi.INVALID_CONFIG
        stream = lambda grid: _capi.GemmPlan(1, 0, 1, 1, grid, n // 16, k // 256, 8 * 2 * 4096)
        assert try_plan(stream(512)) == _capi.SUCCESS and try_plan(stream(1024)) == _capi.INVALID_CONFIG
    finally:
        lib.hfrk_plan_table_clear()
    from hf_rocm_kernels.benchmarks.skinny_gemm import grid_search
    assert not hasattr(grid_search, "small_weights")
    import inspect
    assert "small-weights" not in inspect.getsource(grid_search)
    for p in grid_search.candidate_plans(m, 4096, k, [192, 512, 1024]):
        assert p.grid <= (512 if p.wn in (0, -2, -3) else 256)


def test_whatever_the_plan_check_accepts_stays_inside_its_buffers():
    """Seeded random plans of every kind on random small shapes, offered to the library the way a plan table or a caller would
    (hfrk_plan_table_set runs the launcher's check): every plan it accepts is audited, in the weight layout it was accepted
    for.  The point is the converse of the hand-made cases above -- not "these plans are fine" but "the check lets nothing
    through that is not"."""
    import random
    rng = random.Random(20250)
    lib = _capi.load()
    accepted = {-3: 0, -2: 0, -1: 0, 0: 0, 1: 0}
    offered = 0
    while min(accepted.values()) < 40 and offered < 60000:
        m = rng.choice([1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 25, 32, 33, 48, 64])
        n = rng.choice([16 * rng.randrange(1, 160), 4 * rng.randrange(1, 640), rng.randrange(1, 2600)])
        k = 256 * rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 32]) if rng.random() < 0.9 else 16 * rng.randrange(1, 200)
        packed = rng.random() < 0.4
        kind = rng.choice([-3, -2, -1, 0, 1])
        mt = (m + 15) // 16
        ma = (m + 3) // 4 if m <= 16 else rng.choice([6, 8])
        grid = rng.choice([1, 2, 7, 8, 64, 100, 192, 200, 256, 264, 320, 512, 513, 1024])
        if kind in (-3, -2):
            rt = rng.choice([1, 2])
            panels = -(-n // 16) if kind == -3 else -(-n // 4)
            p = _capi.GemmPlan(1, kind, rt, rng.choice([ma, ma, ma + 1, 4]), min(grid, panels) if rng.random() < 0.9 else grid, panels,
                               k // 256, 8 * (rt + (max(ma, 1) + 3) // 4) * 4096)
        elif kind == -1:
            wave_k = rng.choice([256, 512, 1024])
            tiles, windows = -(-n // 16), max(1, k // (8 * wave_k))
            p = _capi.GemmPlan(mt, -1, wave_k // 256, 0, min(grid, tiles * windows), tiles, windows, 8 * (wave_k // 256) * 4096 + 16 * mt * 1024)
        elif kind == 0:
            rt = rng.choice([1, 2])
            groups, kc = -(-n // (16 * rt)), -(-k // 256)
            p = _capi.GemmPlan((ma + 3) // 4, 0, rt, ma, min(grid, groups * kc), groups, kc, 8 * (rt + (ma + 3) // 4) * 4096)
        else:
            wn, ch, rt = rng.choice([1, 2, 4, 8]), rng.choice([1, 2]), rng.choice([1, 1, 2])
            wk = 8 // wn
            ks = 256 * wk * ch
            panels, slabs = -(-n // (16 * wn * rt)), max(1, k // ks)
            p = _capi.GemmPlan(mt, wn * rt, wk, ch, min(grid, panels * slabs), panels, slabs, 8 * rt * 4096 + 2 * 16 * mt * ks)
        offered += 1
        status = lib.hfrk_plan_table_set(m, n, k, int(packed), ctypes.byref(p))
        if status != _capi.SUCCESS:
            continue
        lib.hfrk_plan_table_set(m, n, k, int(packed), None)   # (take it out again)
        if accepted[min(p.wn, 1)] >= 60:
            continue
        accepted[min(p.wn, 1)] += 1
        assert p.grid <= (512 if p.wn in (-3, -2, 0) else 256)
        assert audit(m, n, k, p, packed=packed) > 0, (m, n, k, packed, p.as_dict())
    assert min(accepted.values()) >= 40, (accepted, offered)
