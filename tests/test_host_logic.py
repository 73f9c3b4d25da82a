"""Host-side logic, no GPU: the C ABI loads and exports what the header declares, the launcher's validation
returns the reference's codes, the planner's decomposition covers every (panel, slab) exactly once and the index
arithmetic the kernel uses to find a panel's contributors matches brute force, the torch op schemas are the
reference's, and the Python wrappers reject what the reference's wrappers reject."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from hf_rocm_kernels import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "hfrk_gfx950.h")).read()
    declared = set(re.findall(r"\b(hfrk_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_capi.SIGNATURES), declared ^ set(_capi.SIGNATURES)
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _capi.load().hfrk_version() >= 100
    assert _capi.status_string(0) == "success" and "even" in _capi.status_string(2)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", "/nonexistent/libhfrk_gfx950.so")
    with pytest.raises(ImportError):
        _capi.load()


def _validate(m=8, n=4096, k=4096, b_stride=None, split_k=1, A=3, B=4, C=3, al=1, bl=4, q=3, op_m=8, ops=4):
    return _capi.load().hfrk_skinny_gemm_validate(m, n, k, k if b_stride is None else b_stride, split_k, A, B, C, al, bl, q, op_m, ops)


def test_validation_codes_match_the_reference_launcher():
    assert _validate() == _capi.SUCCESS
    assert _validate(n=4097) == _capi.N_NOT_EVEN
    assert _validate(k=4096 + 128) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K      # (512/8)*4 = 256
    # k that is no multiple of 256 passes wherever the reference's tile (512/op_m)*ops divides it (skinny_gemm_caller.cu:33-48)
    assert _validate(k=128, op_m=16, ops=4) == _capi.SUCCESS
    assert _validate(k=4096 + 128, op_m=16, ops=4) == _capi.SUCCESS
    assert _validate(k=4096 + 64, op_m=32, ops=4) == _capi.SUCCESS
    assert _validate(k=4096 + 64, op_m=16, ops=4) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    assert _validate(A=6, B=6, C=5) == _capi.TOO_MANY_WARPS
    assert _validate(A=3, B=4, C=3, q=2) == _capi.QSIZE_TOO_SMALL              # consumers > qsize
    assert _validate(B=8, bl=1, q=3, A=2, C=2) == _capi.QSIZE_TOO_SMALL        # B_producers / b_lanes > qsize
    assert _validate(op_m=12) == _capi.INVALID_CONFIG
    assert _validate(ops=2, k=4096) == _capi.INVALID_CONFIG
    assert _validate(bl=0) == _capi.INVALID_CONFIG
    # order of the reference's checks: n parity is reported before K divisibility, K before the warp count
    assert _validate(n=4097, k=100) == _capi.N_NOT_EVEN
    assert _validate(k=100, A=9, B=9, C=9) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    # limits of this implementation
    assert _validate(m=65) == _capi.BAD_SHAPE
    assert _validate(b_stride=4096 + 8) == _capi.BAD_ALIGNMENT
    # every knob set the reference's own table returns is accepted (wrapped.py:45-102 of the reference)
    for (A, B, C, al, bl, q, om, ops) in [(3, 5, 2, 1, 4, 3, 8, 4), (2, 3, 2, 1, 4, 2, 16, 8), (2, 4, 2, 2, 4, 3, 16, 4),
                                          (3, 6, 2, 1, 4, 3, 8, 4), (3, 6, 3, 2, 3, 3, 16, 8), (2, 7, 2, 1, 4, 2, 8, 4)]:
        assert _validate(m=8 if om == 8 else 16, n=16384, k=2048, A=A, B=B, C=C, al=al, bl=bl, q=q, op_m=om, ops=ops) == 0


SHAPES = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336), (10240, 8192), (8192, 8192), (57344, 8192),
          (8192, 28672), (128, 256), (1000, 512), (50, 256), (13312, 16384), (2304, 16384)]


def _stream_ranges(plan):
    """Wave-stream decomposition: the first C % G workgroups hold C // G + 1 consecutive chunks, the others C // G."""
    C, G = plan.panels * plan.slabs, plan.grid
    q, r = divmod(C, G)
    return [(g * q + min(g, r), g * q + min(g, r) + q + (1 if g < r else 0)) for g in range(G)]


def _emulate_stream(plan):
    """Chunks (row tile, K chunk) split over workgroups, then over their 8 waves; who touches which row tile."""
    KC, T = plan.slabs, plan.panels
    cover = [0] * (T * KC)
    wg_of_tile = [[] for _ in range(T)]
    for g, (c0, c1) in enumerate(_stream_ranges(plan)):
        assert c0 < c1
        n = c1 - c0
        for w in range(8):
            for c in range(c0 + w * n // 8, c0 + (w + 1) * n // 8):
                cover[c] += 1
        for t in range(c0 // KC, (c1 - 1) // KC + 1):
            wg_of_tile[t].append(g)
    return cover, wg_of_tile


def _stream_owner(plan, c):
    """The kernel's closed form for the workgroup whose range holds chunk c."""
    q, r = divmod(plan.panels * plan.slabs, plan.grid)
    big = r * (q + 1)
    return c // (q + 1) if c < big else r + (c - big) // q


def _emulate(plan, n, k):
    """Replays the kernel's decomposition arithmetic on the host and returns per-panel coverage."""
    S, P, G = plan.slabs, plan.panels, plan.grid
    U = S * P
    ub = lambda g: (g * U) // G
    cover = [[0] * S for _ in range(P)]
    contributors = [[] for _ in range(P)]
    for g in range(G):
        u0, u1 = ub(g), ub(g + 1)
        assert u0 < u1, "empty workgroup"
        for u in range(u0, u1):
            p, s = divmod(u, S)
            phys = (s + p % S) % S      # slab rotation: must stay a bijection per panel
            cover[p][phys] += 1
            if not contributors[p] or contributors[p][-1] != g:
                contributors[p].append(g)
    return cover, contributors, ub


def _emulate_rows(plan):
    """Replays the row-split kernel's arithmetic on the host: bands of 4-row units per workgroup, tiles of nearly equal
    height per band, chunk runs per wave, and the end-of-kernel roles (who hands a partial over, who finishes which tile,
    whose partials it adds).  Returns nothing; asserts that every (unit, K chunk) is multiplied exactly once and every
    tile is finished exactly once from exactly the partials that exist."""
    G, units, KC, per_tile = plan.grid, plan.panels, plan.slabs, 4 * plan.wk
    tiled = plan.wn == -3   # bands of whole 16-row tiles (plan.panels counts them): chunks of per_tile units, a last one of fewer
    if tiled:
        units *= 4
    q, r = divmod(plan.panels, G)
    magic = ((1 << 32) + KC - 1) // KC
    assert magic < (1 << 32)
    cover = [[0] * KC for _ in range(units)]
    for g in range(G):
        nu, u0 = q + (1 if g < r else 0), g * q + min(g, r)
        assert nu >= 1, "empty workgroup"
        if tiled:
            nu, u0 = 4 * nu, 4 * u0
        T = -(-nu // per_tile)
        base, extra = nu // T, nu % T
        TC = T * KC
        runs = [((w * TC) >> 3, ((w + 1) * TC) >> 3) for w in range(8)]
        assert runs[0][0] == 0 and runs[-1][1] == TC and all(a[1] == b[0] for a, b in zip(runs, runs[1:]))
        pieces = [[] for _ in range(T)]  # waves that multiply chunks of tile j, in order
        for w, (i0, i1) in enumerate(runs):
            for i in (i0, i1):
                assert (i * magic) >> 32 == i // KC  # the kernel divides by multiplying with the reciprocal
            for i in range(i0, i1):
                j, kc = divmod(i, KC)
                first, height = j * base + min(j, extra), base + (1 if j < extra else 0)
                if tiled:
                    first, height = per_tile * j, min(per_tile, nu - per_tile * j)
                assert 1 <= height <= per_tile
                for t in range(height):
                    cover[u0 + first + t][kc] += 1
                if not pieces[j] or pieces[j][-1] != w:
                    pieces[j].append(w)
        assert tiled or sum(base + (1 if j < extra else 0) for j in range(T)) == nu
        finished = [0] * T
        for w, (i0, i1) in enumerate(runs):
            count, kb0 = i1 - i0, i0 % KC
            for j in range(T):  # tiles that begin and end inside the run: finished in the loop, by this wave alone
                if count > 0 and j * KC >= i0 and (j + 1) * KC <= i1:
                    finished[j] += 1
                    assert pieces[j] == [w]
            jl = i1 // KC
            ke = i1 - jl * KC
            if count > 0 and ke != 0 and jl * KC >= i0:  # finishes tile jl after the barrier
                finished[jl] += 1
                added = [x for x in range(1, 8) if x > w and ((x * TC) >> 3) < (jl + 1) * KC]
                for x in added:  # each hands over: an empty run (zeros), or a run that starts inside tile jl
                    x0, x1 = runs[x]
                    assert x1 == x0 or (x0 % KC != 0 and x0 // KC == jl), (g, w, x)
                assert [x for x in added if runs[x][1] > runs[x][0]] == [x for x in pieces[jl] if x != w], (g, w, jl)
            if count > 0 and kb0 != 0:  # hands the partial of its first tile over: somebody before it must finish that tile
                assert pieces[i0 // KC][0] < w
        assert finished == [1] * T, (g, finished)
    assert all(c == 1 for row in cover for c in row)


@pytest.mark.parametrize("rt", [1, 2])
@pytest.mark.parametrize("n,k,grid", [(4096, 4096, 256), (6144, 4096, 256), (10240, 8192, 256), (10240, 8192, 512), (57344, 8192, 256),
                                      (4096, 14336, 256), (1000, 512, 77), (1000, 512, 250), (50, 512, 13), (130, 1024, 7),
                                      (2304, 16384, 256), (1024, 512, 256), (28672, 4096, 1), (8192, 28672, 512), (8200, 768, 200)])
def test_row_split_decomposition_on_the_host(n, k, grid, rt):
    units = -(-n // 4)
    plan = _capi.GemmPlan(1, -2, rt, 2, min(grid, units), units, k // 256, 8 * (rt + 1) * 4096)
    assert _capi.load().hfrk_plan_table_set(8, n, k, 0, ctypes.byref(plan)) == _capi.SUCCESS   # the library accepts it
    assert _capi.load().hfrk_plan_table_set(8, n, k, 0, None) == _capi.SUCCESS
    assert _capi.load().hfrk_plan_table_set(8, n, k, 1, ctypes.byref(plan)) == _capi.INVALID_CONFIG   # not for the packed load format
    _emulate_rows(plan)
    # the same on bands of whole 16-row tiles, the form both weight layouts take
    tiles = -(-n // 16)
    plan = _capi.GemmPlan(1, -3, rt, 2, min(grid, tiles), tiles, k // 256, 8 * (rt + 1) * 4096)
    for packed in (0, 1):
        assert _capi.load().hfrk_plan_table_set(8, n, k, packed, ctypes.byref(plan)) == _capi.SUCCESS
        assert _capi.load().hfrk_plan_table_set(8, n, k, packed, None) == _capi.SUCCESS
    _emulate_rows(plan)


@pytest.mark.parametrize("m", [1, 8, 16, 33, 64])
@pytest.mark.parametrize("n,k", SHAPES)
def test_plan_covers_every_unit_once_and_contributor_formula(m, n, k):
    plan = _capi.plan(m, n, k)
    if plan.wn == -2:  # m <= 16, rows that deal out evenly: row-split decomposition
        assert m <= 16 and plan.ch == (m + 3) // 4 and plan.m_tiles == 1 and plan.slabs == k // 256 and plan.panels == -(-n // 4)
        assert plan.wk in (1, 2) and plan.lds_bytes == 8 * (plan.wk + 1) * 4096 and 1 <= plan.grid <= min(512, plan.panels)
        _emulate_rows(plan)
        return
    if plan.wn == 0:  # m <= 16: wave-stream decomposition
        assert m <= 16 and plan.ch == (m + 3) // 4 and plan.m_tiles == (plan.ch + 3) // 4 and plan.slabs == k // 256
        assert plan.wk in (1, 2) and (plan.wk == 2 or m <= 16) and plan.panels == -(-n // (16 * plan.wk))
        assert plan.lds_bytes == 8 * (plan.wk + plan.m_tiles) * 4096
        assert 1 <= plan.grid <= min(256, plan.panels * plan.slabs) and plan.lds_bytes <= 160 * 1024
        cover, wg_of_tile = _emulate_stream(plan)
        assert all(c == 1 for c in cover)
        KC = plan.slabs
        for t, who in enumerate(wg_of_tile):
            lo, hi = t * KC, (t + 1) * KC
            assert who == list(range(_stream_owner(plan, lo), _stream_owner(plan, hi - 1) + 1)), (t, who)
        return
    assert m > 16
    if plan.wn == -1:  # K-split decomposition: units = (window, row tile), window-major, split like the stream chunks
        wave_k = 256 * plan.wk
        assert wave_k in (256, 512) and k == 8 * wave_k and plan.ch == 0 and plan.m_tiles == (m + 15) // 16
        assert plan.panels == -(-n // 16) and plan.slabs == k // (8 * wave_k)
        assert 1 <= plan.grid <= min(256, plan.panels * plan.slabs)
        assert plan.lds_bytes == 8 * plan.wk * 4096 + 16 * plan.m_tiles * 1024 <= 160 * 1024
        ranges = _stream_ranges(plan)
        assert ranges[0][0] == 0 and ranges[-1][1] == plan.panels * plan.slabs
        assert all(a[1] == b[0] and a[0] < a[1] for a, b in zip(ranges, ranges[1:]))
        return
    # (wn * wk = 16: two weight tiles per row wave, taken where 256-row panels deal out evenly over the workgroups)
    assert plan.m_tiles == (m + 15) // 16 and plan.wn * plan.wk in (8, 16) and plan.ch in (1, 2)
    ks = 256 * plan.wk * plan.ch
    assert k % ks == 0 and plan.slabs == k // ks and plan.panels == -(-n // (16 * plan.wn))
    assert 1 <= plan.grid <= min(256, plan.panels * plan.slabs)
    assert plan.lds_bytes <= 160 * 1024
    cover, contributors, ub = _emulate(plan, n, k)
    assert all(c == 1 for row in cover for c in row)
    S, G, U = plan.slabs, plan.grid, plan.slabs * plan.panels
    for p, who in enumerate(contributors):
        lo, hi = p * S, (p + 1) * S
        g_first = ((lo + 1) * G + U - 1) // U - 1      # the kernel's closed form
        g_last = (hi * G + U - 1) // U - 1
        assert who == list(range(g_first, g_last + 1)), (p, who, g_first, g_last)
        # slot rule: a workgroup's partial for its first panel goes to slot 0, for its last to slot 1; never both the same
        for g in who:
            first_panel, last_panel = ub(g) // S, (ub(g + 1) - 1) // S
            assert p in (first_panel, last_panel) or (ub(g) <= lo and hi <= ub(g + 1))


def test_planner_on_random_shapes_gives_plans_the_launcher_accepts_and_that_cover_the_work():
    """The planner's rules are many and were read off sweeps of particular shapes: on 400 seeded random shapes (row counts
    1..64, weights of 16..60000 rows including ragged ones, k up to 32768 in steps of 256, a third of them in the packed
    load format) whatever it answers must pass the
    launcher's own check (hfrk_plan_table_set runs it) and, replayed on the host, multiply every unit of work exactly once."""
    import random
    from hf_rocm_kernels import plan_table
    rng = random.Random(20250)
    lib = _capi.load()
    kinds = set()
    plan_table.clear()
    try:
        for _ in range(400):
            m = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 20, 24, 25, 28, 32, 33, 40, 48, 49, 64])
            n = rng.choice([rng.randrange(16, 60000), 64 * rng.randrange(1, 900), 128 * rng.randrange(1, 450), 4 * rng.randrange(4, 15000)])
            k = 256 * rng.choice([rng.randrange(1, 129), rng.choice([4, 8, 12, 16, 20, 32, 56, 64, 112])])
            p = _capi.GemmPlan()
            packed = rng.randrange(3) == 0  # the planner's answer for weights in the packed load format (empty table: its rules)
            status = lib.hfrk_plan_table_get(m, n, k, int(packed), ctypes.byref(p))
            assert status == _capi.SUCCESS, (m, n, k, packed, _capi.status_string(status))
            assert lib.hfrk_plan_table_set(m, n, k, int(packed), ctypes.byref(p)) == _capi.SUCCESS, (m, n, k, packed, p.as_dict())
            plan_table.clear()
            assert not packed or p.wn != -2  # bands of any 4-row height do not exist in 16-row packed tiles
            assert packed or p.wn != -3      # (the planner deals row-major weights in 4-row units)
            kinds.add(p.wn if p.wn <= 0 else 1)
            if p.panels * p.slabs > 200000:
                continue  # (the replay is a Python loop over units)
            if p.wn in (-2, -3):
                _emulate_rows(p)
            elif p.wn == 0:
                assert all(c == 1 for c in _emulate_stream(p)[0]), (m, n, k)
            elif p.wn == -1:
                r = _stream_ranges(p)
                assert r[0][0] == 0 and r[-1][1] == p.panels * p.slabs and all(a[1] == b[0] and a[0] < a[1] for a, b in zip(r, r[1:]))
            else:
                assert all(c == 1 for row in _emulate(p, n, k)[0] for c in row), (m, n, k)
    finally:
        plan_table.clear()
    assert kinds == {-3, -2, -1, 0, 1}


def test_plan_rejects_what_the_kernel_cannot_take():
    p = _capi.GemmPlan()
    lib = _capi.load()
    assert lib.hfrk_skinny_gemm_plan(65, 128, 256, ctypes.byref(p)) == _capi.BAD_SHAPE
    assert lib.hfrk_skinny_gemm_plan(0, 128, 256, ctypes.byref(p)) == _capi.BAD_SHAPE
    assert lib.hfrk_skinny_gemm_plan(8, 128, 300, ctypes.byref(p)) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    assert lib.hfrk_skinny_gemm_plan(8, 128, 256, None) == _capi.BAD_SHAPE


def test_rms_prologue_predicate_is_the_plan_the_fused_entry_launches_with():
    """`hfrk_skinny_gemm_rms_plan` is the one decision behind `rms_prologue_available` and `hfrk_skinny_gemm_rms_fused`: a
    row-split plan (wn = -2) with one weight tile per chunk (two with SwiGLU: gate and up) on more workgroups than rows, or
    HFRK_BAD_SHAPE -- never another decomposition, whatever the plan table holds for the plain GEMM."""
    rng = np.random.default_rng(11)
    lib = _capi.load()
    seen = {True: 0, False: 0}
    for _ in range(400):
        m = int(rng.integers(1, 12))
        n = int(rng.choice([256, 512, 1000, 2048, 3584, 4096, 4098, 6144, 10240, 14336, 28672])) + 32 * int(rng.integers(0, 3))
        k = int(rng.choice([2048, 4096, 8192, 4352, 16384]))
        for epilogue in (_capi.EPILOGUE_NONE, _capi.EPILOGUE_SWIGLU):
            p = _capi.rms_plan(m, n, k, epilogue)
            seen[p is not None] += 1
            if p is None:
                continue
            swiglu = epilogue == _capi.EPILOGUE_SWIGLU
            assert m <= 8 and k in (4096, 8192) and (not swiglu or n % 32 == 0)
            assert p.wn == -2 and p.wk == (2 if swiglu else 1) and p.grid > m and p.slabs == k // 256
            n_eff = n // 2 if swiglu else n
            assert p.panels == (n_eff + 3) // 4
            _emulate_rows(p)
    assert seen[True] > 100 and seen[False] > 100
    assert _capi.rms_plan(9, 4096, 4096) is None and _capi.rms_plan(4, 4096, 2048) is None and _capi.rms_plan(4, 512, 4096) is None
    assert _capi.rms_plan(4, 4096 + 16, 4096, _capi.EPILOGUE_SWIGLU) is None
    p = _capi.GemmPlan()
    assert lib.hfrk_skinny_gemm_rms_plan(4, 4096, 4096, 7, ctypes.byref(p)) == _capi.INVALID_CONFIG
    assert lib.hfrk_skinny_gemm_rms_plan(4, 4096, 4096, 0, None) == _capi.INVALID_CONFIG
    # a table entry for the plain GEMM does not change it
    stream = _capi.GemmPlan(1, 0, 1, 1, 256, 256, 16, 8 * 2 * 4096)
    before = _capi.rms_plan(4, 4096, 4096)
    from hf_rocm_kernels import plan_table
    try:
        assert lib.hfrk_plan_table_set(4, 4096, 4096, 0, ctypes.byref(stream)) == 0
        assert plan_table.get_plan(4, 4096, 4096).wn == 0
        after = _capi.rms_plan(4, 4096, 4096)
        assert after is not None and (after.wn, after.wk, after.grid) == (before.wn, before.wk, before.grid)
    finally:
        plan_table.remove_plan(4, 4096, 4096)


def test_plans_for_k_that_ends_inside_a_chunk():
    """k % 16 == 0 is enough for row-major weights up to 32 rows: wave-stream plans count the cut-short last chunk
    (slabs = ceil(k / 256)); packed weights, the other kernels and single plans above 32 rows need k % 256 == 0."""
    p = _capi.GemmPlan()
    lib = _capi.load()
    assert lib.hfrk_skinny_gemm_plan(8, 4096, 4096 + 128, ctypes.byref(p)) == 0
    assert p.wn == 0 and p.slabs == 17 and p.panels == 256
    assert lib.hfrk_skinny_gemm_plan(32, 1000, 640, ctypes.byref(p)) == 0
    assert p.wn == 0 and p.slabs == 3
    assert lib.hfrk_skinny_gemm_plan(8, 256, 144, ctypes.byref(p)) == 0
    assert p.wn == 0 and p.slabs == 1
    assert lib.hfrk_skinny_gemm_plan(33, 1000, 640, ctypes.byref(p)) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    assert lib.hfrk_skinny_gemm_plan(8, 1000, 648, ctypes.byref(p)) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K


def test_row_split_plans_for_17_to_32_rows_and_for_half_megabyte_bands():
    """The planner's row-split rules beyond 16 rows and around 512 KB bands: 17..32 rows run the row-split kernel with a
    second activation tile (ch = 6 up to 24 rows, else 8; two weight tiles per chunk) on bands of 24..64 rows with
    moderate k; a weight whose bands would come to exactly 512 KB gets two weight tiles per chunk at any row count, and
    a grid chosen for whole tiles is not taken when it creates such bands."""
    p = _capi.GemmPlan()
    lib = _capi.load()
    plan = lambda m, n, k: (lib.hfrk_skinny_gemm_plan(m, n, k, ctypes.byref(p)), p.wn, p.wk, p.ch, p.grid, p.lds_bytes)
    assert plan(24, 8192, 8192) == (0, -2, 2, 6, 256, 8 * 4 * 4096)
    assert plan(32, 8192, 8192) == (0, -2, 2, 8, 256, 8 * 4 * 4096)
    assert plan(20, 6144, 4096)[1:4] == (-2, 2, 6) and plan(32, 6144, 4096)[1:4] == (-2, 2, 8)
    assert plan(32, 8192, 16384)[1:3] == (2, 4)  # 2 row waves x 4 K waves on long k
    assert plan(32, 10240, 8192)[1] != -2      # bands of 40 rows: up to 24 rows only
    assert plan(24, 4096, 14336)[1] != -2      # bands of 16 rows
    assert plan(24, 8192, 28672)[1] != -2      # k above 16384
    assert plan(33, 8192, 8192)[1] != -2
    # 512 KB bands
    assert plan(1, 16384, 8192)[1:5] == (-2, 2, 1, 256)
    assert plan(8, 8192, 16384)[1:5] == (-2, 2, 2, 256)
    assert plan(4, 32768, 4096)[1:5] == (-2, 2, 1, 256)
    assert plan(1, 14336, 8192)[1:5] == (-2, 1, 1, 256)       # 224 workgroups would make 64-row bands of 512 KB
    assert plan(1, 14336, 4096)[1:5] == (-2, 1, 1, 224)       # 256 KB bands: the whole-tile grid stands
    assert plan(1, 16384, 16384)[1:5] == (-2, 1, 1, 256)      # 1 MB bands are fine with one tile per chunk
    # ragged bands of 20..44 rows: two matrix tiles per chunk from 5 rows on, on long enough k; 256 workgroups rather than
    # fewer with whole tiles
    assert plan(8, 5120, 8192)[1:5] == (-2, 2, 2, 256) and plan(4, 5120, 8192)[1:5] == (-2, 2, 1, 256) and plan(4, 5120, 4096)[1:5] == (-2, 1, 1, 512)
    assert plan(4, 10240, 8192)[2] == 1 and plan(8, 5120, 5120)[2] == 1
    assert plan(16, 5120, 5120)[1:5] == (-2, 2, 4, 256) and plan(8, 10240, 5120)[2] == 2 and plan(8, 13312, 16384)[2] == 1
    assert plan(8, 7168, 14336)[1:5] == (-2, 2, 2, 256) and plan(8, 7168, 4096)[1:5] == (-2, 1, 2, 224)
    assert plan(8, 6144, 4096)[1:5] == (-2, 1, 2, 256)
    # bands of 12-20 rows on k up to 8192, except where one K-split window covers k and its tiles deal out evenly
    assert plan(20, 5120, 5120)[1:4] == (-2, 2, 6) and plan(32, 3072, 3072)[1:4] == (-2, 2, 8)
    assert plan(24, 5120, 4096)[1] == -2 and plan(24, 4096, 4096)[1] == -1
    assert plan(32, 4096, 8192)[1] > 0 and plan(24, 4096, 8192)[1] == -2


def test_workgroup_plans_on_whole_and_split_panels():
    """From 17 rows on the planner deals whole row panels to workgroups where the row count allows: several each on
    224..256 workgroups, one each on 160..216 (64-row panels on short k, 128-row panels), and on long k 128-row panels
    whose k is cut between 2 or 4 workgroups."""
    p = _capi.GemmPlan()
    lib = _capi.load()
    plan = lambda m, n, k: (lib.hfrk_skinny_gemm_plan(m, n, k, ctypes.byref(p)), p.wn, p.wk, p.ch, p.grid, p.panels)
    assert plan(64, 57344, 8192)[1:6] == (16, 1, 1, 224, 224)
    assert plan(48, 28672, 4096)[1:6] == (8, 1, 2, 224, 224)
    assert plan(40, 16384, 4096)[1:6] == (4, 2, 1, 256, 256)
    # one panel per workgroup on fewer workgroups
    assert plan(64, 10240, 3072)[1:6] == (4, 2, 1, 160, 160)
    assert plan(64, 10240, 8192)[4] == 256                      # too much k for 160 workgroups
    assert plan(48, 12288, 8192)[1:6] == (4, 2, 1, 192, 192)
    assert plan(33, 13312, 14336)[1:6] == (4, 2, 1, 208, 208)
    assert plan(48, 12288, 4096)[1] == -1 and plan(32, 12288, 4096)[1:6] == (4, 2, 1, 192, 192)
    assert plan(48, 24576, 16384)[1:6] == (8, 1, 1, 192, 192)
    assert plan(64, 20480, 3072)[1:6] == (8, 1, 2, 160, 160)
    assert plan(64, 20480, 4096)[1] == -1 and plan(64, 20480, 14336)[4] == 256
    # k = 16384: 64-row panels with two chunks per slab up to 48 rows; 128-row panels cut in k
    assert plan(40, 16384, 16384)[1:6] == (4, 2, 2, 256, 256)
    assert plan(64, 16384, 16384)[1:3] == (8, 1)
    assert plan(48, 13312, 16384)[1:6] == (8, 1, 1, 208, 104)
    assert plan(32, 6144, 16384)[1:6] == (8, 1, 1, 192, 48)
    assert plan(32, 6144, 14336)[1:6] == (8, 1, 1, 192, 48)
    assert plan(48, 8192, 16384)[1:3] == (2, 4) and plan(64, 8192, 16384)[1:6] == (8, 1, 1, 256, 64)
    # 32-row panels (2 row waves x 4 K waves), one each, on short k that no K-split window covers, up to 48 rows
    assert plan(48, 8192, 3072)[1:6] == (2, 4, 1, 256, 256) and plan(33, 7168, 5120)[1:6] == (2, 4, 1, 224, 224)
    assert plan(48, 6144, 3072)[1:6] == (2, 4, 1, 192, 192) and plan(40, 5120, 5120)[1:6] == (2, 4, 1, 160, 160)
    assert plan(64, 8192, 3072)[1:3] == (4, 2) and plan(48, 8192, 8192)[1:3] == (4, 2) and plan(48, 8192, 4096)[1] == -1
    # 17..24 rows: whole 64-row panels come before the row-split kernel from 12288 weight rows on
    assert plan(24, 13312, 8192)[1:6] == (4, 2, 1, 208, 208) and plan(20, 16384, 14336)[1:6] == (4, 2, 1, 256, 256)
    assert plan(24, 10240, 8192)[1] == -2 and plan(19, 16384, 2048)[1] == -2 and plan(24, 16384, 16384)[1] == -2


def test_op_schemas_are_the_reference_schemas():
    import hf_rocm_kernels  # noqa: F401  (loads _HFRK_C)
    # the definition strings of the reference's csrc/torch_bindings.cpp:22,26-28,32-34,38-40, verbatim
    expect = {
        "increment": "increment(Tensor! x) -> ()",
        "residual_rms": "residual_rms(Tensor input, Tensor! residual, Tensor weight, Tensor scale_tensor, float epsilon, Tensor! "
                        "output, Tensor! next_buffer, int num_threads, bool force_scalar) -> ()",
        "swiglu": "swiglu(Tensor gate_up, Tensor scale_tensor, Tensor! output, Tensor! next_buffer, int num_threads, "
                  "bool force_scalar) -> ()",
        "skinny_gemm_tb": "skinny_gemm_tb(Tensor A, Tensor B, Tensor! D, Tensor scale_tensor, int split_k, int A_producers, "
                          "int B_producers, int consumers, int a_lanes, int b_lanes, int qsize, int op_m, int ops) -> int",
    }
    for name, schema in expect.items():
        got = getattr(torch.ops._HFRK_C, name).default._schema
        want = torch._C.parse_schema("_HFRK_C::" + schema)
        assert str(got) == str(want), (str(got), str(want))
        assert [(a.name, str(a.type), a.alias_info is not None and a.alias_info.is_write) for a in got.arguments] == \
               [(a.name, str(a.type), a.alias_info is not None and a.alias_info.is_write) for a in want.arguments]


def test_ops_have_no_cpu_path():
    import hf_rocm_kernels  # noqa: F401
    a = torch.zeros(8, 256).to(torch.float8_e4m3fn)
    b = torch.zeros(128, 256).to(torch.float8_e4m3fn).t()
    d = torch.zeros(8, 128, dtype=torch.bfloat16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops._HFRK_C.skinny_gemm_tb(a, b, d, torch.ones(1), 1, 3, 4, 3, 1, 4, 3, 8, 4)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops._HFRK_C.swiglu(torch.zeros(2, 16, dtype=torch.float16), torch.ones(1), torch.zeros(2, 8).to(torch.float8_e4m3fn),
                                 torch.zeros(2, 0, dtype=torch.float16), 64, False)


def test_wrapper_assertions_mirror_the_reference():
    from hf_rocm_kernels import residual_rms, skinny_gemm, swiglu
    from hf_rocm_kernels.operators.residual_rms.wrapped import infer_num_threads as rms_threads
    from hf_rocm_kernels.operators.skinny_gemm.wrapped import infer_skinny_gemm_m_params, skinny_gemm_checks
    from hf_rocm_kernels.operators.swiglu.wrapped import infer_num_threads as swiglu_threads

    a = torch.zeros(8, 256).to(torch.float8_e4m3fn)
    b = torch.zeros(128, 256).to(torch.float8_e4m3fn).t()
    d = torch.zeros(8, 128, dtype=torch.bfloat16)
    one = torch.ones(1)
    with pytest.raises(AssertionError, match="cuda"):     # device check comes last, as in the reference
        skinny_gemm(a, b, one, d)
    with pytest.raises(AssertionError, match="2 dimensions"):
        skinny_gemm_checks(a[0], b, one, d)
    with pytest.raises(AssertionError, match="to be the same"):
        skinny_gemm_checks(a[:, :128].contiguous(), b, one, d)
    with pytest.raises(AssertionError, match="to be 1"):
        skinny_gemm_checks(a, b, torch.ones(2), d)
    with pytest.raises(AssertionError, match="column-major"):
        skinny_gemm_checks(a, b.t().contiguous().t().contiguous(), one, d)
    with pytest.raises(AssertionError, match="float8_e4m3fn"):
        skinny_gemm_checks(a.view(torch.uint8).view(torch.float8_e4m3fnuz), b, one, d)
    with pytest.raises(AssertionError, match="bfloat16 or torch.float16"):
        skinny_gemm_checks(a, b, one, d.float())
    assert infer_skinny_gemm_m_params(8) == (1, 8) and infer_skinny_gemm_m_params(16) == (1, 16)
    assert infer_skinny_gemm_m_params(17) == (2, 16)
    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(AssertionError, match="cuda"):
        residual_rms(x, x.clone(), torch.ones(64, dtype=torch.float16), 1e-5)
    with pytest.raises(AssertionError, match="same shape"):
        residual_rms(x, x[:2].clone(), torch.ones(64, dtype=torch.float16), 1e-5)
    with pytest.raises(ValueError):
        rms_threads(4, 2048)
    assert rms_threads(4, 0) == 0 and rms_threads(4, 100) == 128 and rms_threads(4, 1024) == 1024
    with pytest.raises(AssertionError, match="even number of columns"):
        swiglu(torch.zeros(4, 63, dtype=torch.float16), one)
    with pytest.raises(AssertionError, match="cuda"):
        swiglu(torch.zeros(4, 64, dtype=torch.float16), one)
    assert swiglu_threads(8, False, 128) == 128 and swiglu_threads(8, False, -1) == 256


def test_data_generators_are_seeded_and_follow_the_recipes():
    from hf_rocm_kernels.operators.residual_rms import generate_residual_rms_data
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data, generate_skinny_gemm_data
    from hf_rocm_kernels.operators.swiglu import generate_swiglu_data
    from oracle import skinny_gemm as og

    a, b, s, out = generate_skinny_gemm_data(4, 32, 256, seed=0, device="cpu")
    a2, b2, s2, _ = generate_skinny_gemm_data(4, 32, 256, seed=0, device="cpu")
    oa, ob, os_, _ = og.generate_skinny_gemm_data(4, 32, 256, seed=0)   # the oracle's twin draws the same bits
    for x, y, z in ((a, a2, oa), (b, b2, ob)):
        assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)) and torch.equal(x.view(torch.uint8), z.view(torch.uint8))
    assert torch.equal(s, s2) and torch.equal(s, os_) and 1 <= float(s) < 3
    assert a.shape == (4, 256) and b.shape == (256, 32) and b.stride(0) == 1 and out.shape == (4, 32) and out.abs().sum() == 0
    a, w, sa, sw = generate_llama_gemm_data(16, 64, 512, seed=1, device="cpu", per_token=True, per_channel=True, outlier_rows=(3,))
    assert sa.shape == (16,) and sw.shape == (64,) and w.stride(0) == 1
    assert float(sa[3]) > 5 * float(sa.median())          # the x20 outlier row gets its own, larger scale
    assert (a.float().abs().amax(dim=1) == 448).all()
    x, r, wt, eps, sc, nb = generate_residual_rms_data(3, 64, 16, dtype=torch.float8_e4m3fn, seed=2, device="cpu", io_dtype=torch.bfloat16)
    assert x.dtype == torch.bfloat16 and sc is not None and nb.shape == (3, 16) and 1e-5 <= eps < 2e-5
    gu, sc, nb = generate_swiglu_data(3, 32, 0, seed=3, device="cpu")
    assert gu.shape == (3, 64) and nb is None


def test_package_reference_functions_agree_with_the_oracle():
    """The torch references the package exports for its users (as the reference package does) are a second,
    independently written statement of the same arithmetic as the oracle: bit-equal on the CPU."""
    from hf_rocm_kernels.operators.residual_rms import precise_residual_rms, reference_residual_rms
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data, reference_skinny_gemm
    from hf_rocm_kernels.operators.swiglu import reference_swiglu
    from oracle import residual_rms as orms
    from oracle import skinny_gemm as og
    from oracle import swiglu as osw
    a, b, sa, sw = generate_llama_gemm_data(5, 96, 512, seed=2, device="cpu", per_token=True, per_channel=True)
    base = torch.randn(5, 96, generator=torch.Generator().manual_seed(1)).to(torch.float16)
    assert torch.equal(reference_skinny_gemm(a, b, sa, sw), og.reference_skinny_gemm(a, b, sa, sw))
    assert torch.equal(reference_skinny_gemm(a, b, sa, sw, output=base), og.reference_skinny_gemm(a, b, sa, sw, output=base))
    g = torch.Generator().manual_seed(4)
    for dtype in (torch.float16, torch.bfloat16):
        x, r = torch.randn(3, 64, generator=g).to(dtype), torch.randn(3, 64, generator=g).to(dtype)
        w = torch.randn(64, generator=g).to(dtype)
        scale = torch.tensor([1.7])
        for s in (scale, None):
            mine, ref = reference_residual_rms(x, r, w, 1e-5, s), orms.reference_residual_rms(x, r, w, 1e-5, s)
            assert torch.equal(mine[0].float(), ref[0].float()) and torch.equal(mine[1], ref[1])
            pm, pr = precise_residual_rms(x, r, w, 1e-5, s), orms.precise_residual_rms(x, r, w, 1e-5, s)
            # float64 with the factors multiplied in another order: equal to the last bits, and equal once quantised
            assert torch.allclose(pm[0].double(), pr[0].double(), rtol=1e-14, atol=0) and torch.equal(pm[1], pr[1])
            assert s is None or torch.equal(pm[0].float(), pr[0].float())
        gu = torch.randn(3, 128, generator=g).mul(3).to(dtype)
        assert torch.equal(reference_swiglu(gu, scale).float(), osw.reference_swiglu(gu, scale).float())


def test_bench_table_bookkeeping():
    from hf_rocm_kernels.utils.benchmarking import Bench, randomize_tensors
    b = Bench.__new__(Bench)  # the constructor queries the GPU
    b._measures = {}
    b.add_raw_measure("torch", 8, 10.0)
    b.add_raw_measure("ours", 8, 4.0)
    b.add_raw_measure("ours", 16, 5.0)
    b.add_speedup_column("torch", "ours")
    t = b.table("M")
    assert t["M"] == [8, 16] and t["Speedup"] == [2.5, "-"] and t["torch"] == [10.0, "-"]
    with pytest.raises(ValueError):
        b.add_speedup_column("missing", "ours")
    x = torch.zeros(4, 4, dtype=torch.float16)
    y = randomize_tensors(x)
    assert y.shape == x.shape and y.dtype == x.dtype and not torch.equal(x, y) and randomize_tensors(3) == 3


def test_plan_table_overrides_the_planner_and_round_trips_through_a_file(tmp_path, monkeypatch):
    """hfrk_plan_table_* are host functions: entries replace the planner's choice for their key (and the smaller m of the same bucket), invalid plans
    are refused with the launcher's status, and a table survives save -> clear -> load (also via HFRK_PLAN_TABLE)."""
    from hf_rocm_kernels import plan_table
    plan_table.clear()
    m, n, k = 8, 6144, 4096
    planner = _capi.plan(m, n, k)
    assert plan_table.get_plan(m, n, k).as_dict() == planner.as_dict()
    tuned = _capi.GemmPlan(1, 0, 1, 2, 128, n // 16, k // 256, 8 * 2 * 4096)  # the wave-stream kernel on 128 workgroups
    assert tuned.as_dict() != planner.as_dict()
    plan_table.set_plan(m, n, k, tuned)
    assert plan_table.get_plan(m, n, k).as_dict() == tuned.as_dict()
    assert _capi.plan(m, n, k).as_dict() == planner.as_dict()          # hfrk_skinny_gemm_plan stays the planner's rule
    assert plan_table.get_plan(m, n, k, packed=True).as_dict() != tuned.as_dict()     # another key: the planner's choice for packed weights
    # the entry also serves the smaller m with the same activation loads (5..8), and no other
    for mm in (5, 6, 7):
        assert plan_table.get_plan(mm, n, k).as_dict() == tuned.as_dict(), mm
    for mm in (4, 9):
        assert plan_table.get_plan(mm, n, k).as_dict() == _capi.plan(mm, n, k).as_dict(), mm
    nearer = _capi.GemmPlan(1, 0, 1, 2, 64, n // 16, k // 256, 8 * 2 * 4096)
    plan_table.set_plan(6, n, k, nearer)
    assert plan_table.get_plan(5, n, k).as_dict() == nearer.as_dict()      # the nearest entry at or above m
    assert plan_table.get_plan(7, n, k).as_dict() == tuned.as_dict()
    plan_table.remove_plan(6, n, k)
    # above 16 rows the bucket is a 16-row tile: an entry for 32 serves 17..32
    big = _capi.plan(32, n, k)
    big32 = _capi.GemmPlan(big.m_tiles, big.wn, big.wk, big.ch, max(8, big.grid // 2), big.panels, big.slabs, big.lds_bytes)
    plan_table.set_plan(32, n, k, big32)
    assert plan_table.get_plan(17, n, k).as_dict() == big32.as_dict()
    assert plan_table.get_plan(16, n, k).as_dict() == _capi.plan(16, n, k).as_dict()
    assert plan_table.get_plan(33, n, k).as_dict() == _capi.plan(33, n, k).as_dict()
    plan_table.remove_plan(32, n, k)
    # a plan that does not fit the shape is refused and changes nothing
    bad = _capi.GemmPlan(1, 0, 1, 1, 128, n // 16, k // 256, 8 * 2 * 4096)  # 4 rows of activations for m = 8
    with pytest.raises(RuntimeError):
        plan_table.set_plan(m, n, k, bad)
    assert _capi.load().hfrk_plan_table_set(m, n, 100, 0, ctypes.byref(tuned)) == _capi.BAD_SHAPE
    assert plan_table.get_plan(m, n, k).as_dict() == tuned.as_dict()
    # a workgroup-kernel entry for a shape the planner gives to the wave-stream kernel
    wg = _capi.GemmPlan(1, 4, 2, 1, 200, n // 64, k // 512, 8 * 4096 + 2 * 16 * 512)
    plan_table.set_plan(16, n, k, wg, packed=True)
    path = tmp_path / "table.json"
    plan_table.save([{"m": m, "n": n, "k": k, "packed": False, "plan": tuned.as_dict(), "us": 7.5},
                     {"m": 16, "n": n, "k": k, "packed": True, "plan": wg.as_dict()}], str(path))
    assert plan_table.clear() == 2
    assert plan_table.get_plan(m, n, k).as_dict() == planner.as_dict()
    assert plan_table.load(str(path)) == 2
    assert plan_table.get_plan(m, n, k).as_dict() == tuned.as_dict()
    assert plan_table.get_plan(16, n, k, packed=True).as_dict() == wg.as_dict()
    plan_table.remove_plan(m, n, k)
    assert plan_table.get_plan(m, n, k).as_dict() == planner.as_dict()
    assert plan_table.clear() == 1
    monkeypatch.setenv(plan_table.ENV_VAR, str(path))
    assert plan_table.load_from_environment() == 2
    assert plan_table.clear() == 2
    monkeypatch.setenv(plan_table.ENV_VAR, "none")
    assert plan_table.load_from_environment() is None
    monkeypatch.delenv(plan_table.ENV_VAR)
    shipped = plan_table.load_from_environment()   # the table shipped with the package: every entry must be accepted
    import json
    tables = plan_table.shipped_tables()
    assert plan_table.DEFAULT_TABLE in tables and len(tables) >= 2
    assert shipped == sum(len(json.load(open(t))["entries"]) for t in tables) and shipped > 0
    assert plan_table.clear() == shipped
    other = tmp_path / "other.json"
    other.write_text('{"format": "something else", "entries": []}')
    with pytest.raises(ValueError):
        plan_table.load(str(other))
    # an entry the library rejects: strict raises, non-strict skips it
    plan_table.save([{"m": m, "n": n, "k": k, "plan": bad.as_dict()}, {"m": m, "n": n, "k": k, "plan": tuned.as_dict()}], str(other))
    with pytest.raises(RuntimeError):
        plan_table.load(str(other))
    plan_table.clear()
    assert plan_table.load(str(other), strict=False) == 1
    plan_table.clear()


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (8, 6144, 4096), (16, 28672, 4096), (32, 4096, 14336), (64, 8192, 8192),
                                   (40, 1000, 2048), (17, 50, 256), (4, 2048, 2048), (4, 2048, 4096), (4, 2048, 28672)])
def test_every_plan_the_sweep_tool_proposes_is_one_the_library_accepts(m, n, k):
    """benchmarks/skinny_gemm/grid_search.py enumerates hfrk_gemm_plan structs by its own arithmetic; the library
    validates plans with its own (hfrk_plan_table_set runs the launcher's check, no device needed).  They must agree,
    for every decomposition family, and describe() must name each one.  Every accepted plan also goes through the host-side
    restatement of its kernel's index arithmetic: every unit of work covered exactly once, ranges contiguous."""
    from hf_rocm_kernels import plan_table
    from hf_rocm_kernels.benchmarks.skinny_gemm import grid_search
    plans = grid_search.candidate_plans(m, n, k, [7, 160, 224, 256, 512])
    assert plans
    families = set()
    plan_table.clear()
    try:
        for p in plans:
            status = _capi.load().hfrk_plan_table_set(m, n, k, 0, ctypes.byref(p))
            assert status == _capi.SUCCESS, (grid_search.describe(p), p.as_dict(), _capi.status_string(status))
            families.add(grid_search.describe(p).split()[0])
            if p.wn in (-2, -3):
                _emulate_rows(p)
            elif p.wn == 0:
                assert all(c == 1 for c in _emulate_stream(p)[0]), grid_search.describe(p)
            elif p.wn == -1:
                r = _stream_ranges(p)
                assert r[0][0] == 0 and r[-1][1] == p.panels * p.slabs and all(a[1] == b[0] for a, b in zip(r, r[1:]))
            else:
                assert all(c == 1 for row in _emulate(p, n, k)[0] for c in row), grid_search.describe(p)
    finally:
        plan_table.clear()
    assert "workgroup" in families
    assert ("wave-stream" in families) == (m <= 32)


def _c_load(path, strict=True):
    count = ctypes.c_int(-1)
    status = _capi.load().hfrk_plan_table_load(str(path).encode(), int(strict), ctypes.byref(count))
    return status, count.value


def test_c_loader_installs_the_shipped_table_like_the_python_loader():
    """hfrk_plan_table_load (for hosts without Python) and plan_table.load read the same file to the same table."""
    import json
    from hf_rocm_kernels import plan_table
    entries = json.load(open(plan_table.DEFAULT_TABLE))["entries"]
    try:
        plan_table.clear()
        assert plan_table.load(plan_table.DEFAULT_TABLE) == len(entries)
        by_python = [plan_table.get_plan(e["m"], e["n"], e["k"], e["packed"]).as_dict() for e in entries]
        assert plan_table.clear() == len(entries)
        assert _c_load(plan_table.DEFAULT_TABLE) == (_capi.SUCCESS, len(entries))
        by_c = [plan_table.get_plan(e["m"], e["n"], e["k"], e["packed"]).as_dict() for e in entries]
        assert by_c == by_python == [e["plan"] for e in entries]
        assert plan_table.clear() == len(entries)
    finally:
        plan_table.clear()
        plan_table.load_from_environment()


def test_c_loader_rejects_what_is_not_a_plan_table(tmp_path):
    import json
    from hf_rocm_kernels import plan_table
    good = {"m": 8, "n": 6144, "k": 4096, "packed": False, "plan": _capi.GemmPlan(1, 0, 1, 2, 192, 384, 16, 65536).as_dict(),   # valid for both weight layouts
            "us": 7.25, "note": "caf\u00e9 \"x\""}
    wrong_shape = dict(good, n=100, plan=dict(good["plan"]))        # the plan does not fit n = 100
    no_grid = dict(good, m=4, plan={k: v for k, v in good["plan"].items() if k != "grid"})
    fractional = dict(good, m=2, plan=dict(good["plan"], grid=12.5))

    def write(name, text):
        path = tmp_path / name
        path.write_text(text)
        return path

    def table(entries, fmt=plan_table.FORMAT):
        return json.dumps({"format": fmt, "device": "test", "entries": entries, "extra": [1, {"a": None}, True]}, indent=1)

    try:
        plan_table.clear()
        assert _c_load(tmp_path / "missing.json") == (_capi.BAD_FILE, 0)
        assert _capi.load().hfrk_plan_table_load(None, 1, None) == _capi.BAD_SHAPE
        for name, text in [("empty.json", ""), ("array.json", "[]"), ("cut.json", table([good])[:-20]), ("trailing.json", table([good]) + "x"),
                           ("format.json", table([good], fmt="other")), ("noentries.json", json.dumps({"format": plan_table.FORMAT})),
                           ("deep.json", "[" * 100 + "]" * 100), ("badnum.json", table([good]).replace("6144", "6144."))]:
            assert _c_load(write(name, text)) == (_capi.BAD_FILE, 0), name
        assert plan_table.clear() == 0
        # members the loader does not know are skipped, escapes are read, installed counts entries
        assert _c_load(write("good.json", table([good]))) == (_capi.SUCCESS, 1)
        assert plan_table.get_plan(8, 6144, 4096).as_dict() == good["plan"]
        assert _capi.load().hfrk_plan_table_load(str(tmp_path / "good.json").encode(), 1, None) == _capi.SUCCESS
        assert plan_table.clear() == 1
        # strict: the first bad entry ends the load with its status, entries before it stay; lenient: bad entries are skipped
        mixed = write("mixed.json", table([good, wrong_shape, no_grid, fractional, dict(good, m=7)]))
        status, count = _c_load(mixed, strict=True)
        assert status != _capi.SUCCESS and status != _capi.BAD_FILE and count == 1
        assert plan_table.clear() == 1
        assert _c_load(write("nogrid.json", table([no_grid])), strict=True) == (_capi.BAD_FILE, 0)
        assert _c_load(write("frac.json", table([fractional])), strict=True) == (_capi.BAD_FILE, 0)
        assert _c_load(mixed, strict=False) == (_capi.SUCCESS, 2)
        assert plan_table.clear() == 2
        # the file a Python save writes is what the C loader reads
        saved = tmp_path / "saved.json"
        plan_table.save([good, dict(good, packed=True)], str(saved))
        assert _c_load(saved) == (_capi.SUCCESS, 2)
        assert plan_table.clear() == 2
    finally:
        plan_table.clear()
        plan_table.load_from_environment()


def test_fp8_linear_keeps_its_quantised_buffers_through_dtype_casts():
    """`.half()` / `.to(torch.bfloat16)` on a converted model cast the bias only; the fp8 weight and its float32 scales stay
    what the GEMM takes, through `state_dict` round trips too.  Layers the activation quantiser cannot take are left alone."""
    from hf_rocm_kernels.layers.fp8_linear import Fp8Linear, convert_linear_layers
    torch.manual_seed(5)
    model = torch.nn.Sequential(torch.nn.Linear(512, 64, bias=True), torch.nn.Linear(256, 32, bias=False),
                                torch.nn.Linear(100, 8), torch.nn.Linear(33024, 2, bias=False)).to(torch.bfloat16)
    assert convert_linear_layers(model) == 2
    assert isinstance(model[0], Fp8Linear) and isinstance(model[1], Fp8Linear)
    assert isinstance(model[2], torch.nn.Linear) and isinstance(model[3], torch.nn.Linear)  # k % 256 != 0; k > 32768
    layer = model[0]
    layer.register_buffer("input_scale", torch.tensor([0.02]))
    weight_bits = layer.weight_data.view(torch.uint8).clone()
    scale = layer.weight_scale.clone()
    for cast in (lambda mod: mod.half(), lambda mod: mod.to(torch.bfloat16), lambda mod: mod.float(), lambda mod: mod.to("cpu")):
        cast(model)
        assert layer.weight_data.dtype == torch.float8_e4m3fn and layer.weight_scale.dtype == torch.float32
        assert layer.input_scale.dtype == torch.float32
        assert torch.equal(layer.weight_data.view(torch.uint8), weight_bits) and torch.equal(layer.weight_scale, scale)
        assert layer.weight is layer.weight_data  # the operand follows the buffer
    model.half()
    assert layer.bias.dtype == torch.float16
    state = {name: t.clone() for name, t in model.state_dict().items()}
    assert state["0.weight_data"].dtype == torch.float8_e4m3fn
    twin = torch.nn.Sequential(torch.nn.Linear(512, 64, bias=True), torch.nn.Linear(256, 32, bias=False),
                               torch.nn.Linear(100, 8), torch.nn.Linear(33024, 2, bias=False)).to(torch.bfloat16)
    convert_linear_layers(twin)
    twin[0].register_buffer("input_scale", torch.zeros(1))
    twin.half().load_state_dict(state)
    assert torch.equal(twin[0].weight_data.view(torch.uint8), weight_bits) and torch.equal(twin[0].weight_scale, scale)
    assert twin[0].weight is twin[0].weight_data
