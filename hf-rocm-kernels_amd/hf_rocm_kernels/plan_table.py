"""Tuned GEMM decompositions, persisted: a JSON file of (m, n, k, weight layout) -> plan entries that the library
consults in place of its planner's rules.

Counterpart of the reference's hand-maintained knob table (hf_rocm_kernels/operators/skinny_gemm/wrapped.py:42-102),
but produced on the box: `benchmarks/skinny_gemm/grid_search.py --save table.json` times every decomposition and
keeps the winners that beat the planner; `load(path)` installs them through `hfrk_plan_table_set`, which validates
each plan for its shape.  At import the package installs the tables it ships (plan_tables/gfx950_*.json) or the
one HFRK_PLAN_TABLE names (`none`: no table).
"""
import ctypes
import glob
import json
import os
from typing import Dict, Iterable, List, Optional

from . import _capi

FORMAT = "hfrk-plan-table-1"
ENV_VAR = "HFRK_PLAN_TABLE"
_PLAN_FIELDS = [name for name, _ in _capi.GemmPlan._fields_]


def _to_struct(plan: Dict[str, int]) -> _capi.GemmPlan:
    return _capi.GemmPlan(*[int(plan[name]) for name in _PLAN_FIELDS])


def set_plan(m: int, n: int, k: int, plan, packed: bool = False) -> None:
    """Install one entry (a GemmPlan or a dict of its fields); raises if the plan does not fit the shape."""
    struct = plan if isinstance(plan, _capi.GemmPlan) else _to_struct(plan)
    _capi.check(_capi.load().hfrk_plan_table_set(int(m), int(n), int(k), int(bool(packed)), ctypes.byref(struct)),
                f"hfrk_plan_table_set({m}, {n}, {k})")


def remove_plan(m: int, n: int, k: int, packed: bool = False) -> None:
    _capi.check(_capi.load().hfrk_plan_table_set(int(m), int(n), int(k), int(bool(packed)), None), "hfrk_plan_table_set")


def get_plan(m: int, n: int, k: int, packed: bool = False) -> _capi.GemmPlan:
    """The plan a call without an explicit one uses: the table's entry, else the planner's choice."""
    p = _capi.GemmPlan()
    _capi.check(_capi.load().hfrk_plan_table_get(int(m), int(n), int(k), int(bool(packed)), ctypes.byref(p)), "hfrk_plan_table_get")
    return p


def clear() -> int:
    """Drop every entry; returns how many there were."""
    return _capi.load().hfrk_plan_table_clear()


def save(entries: Iterable[dict], path: str, device: str = "gfx950") -> None:
    """entries: dicts with m, n, k, packed, plan (dict of the plan's fields) and any measurement fields."""
    with open(path, "w") as f:
        json.dump({"format": FORMAT, "device": device, "entries": list(entries)}, f, indent=1)


def load(path: str, strict: bool = True) -> int:
    """Install every entry of a table file; returns how many.  strict=False skips entries the library rejects
    (a table tuned with another library version) instead of raising."""
    with open(path) as f:
        table = json.load(f)
    if table.get("format") != FORMAT:
        raise ValueError(f"{path}: not a plan table ({table.get('format')!r})")
    count = 0
    for e in table["entries"]:
        try:
            set_plan(e["m"], e["n"], e["k"], e["plan"], bool(e.get("packed", False)))
            count += 1
        except RuntimeError:
            if strict:
                raise
    return count


_TABLE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plan_tables")
DEFAULT_TABLE = os.path.join(_TABLE_DIR, "gfx950_llama3.json")   # Llama-3 8B/70B and Llama-3.1-405B TP8 shard shapes


def shipped_tables() -> List[str]:
    """Every table the package ships for this device (plan_tables/gfx950_*.json), in name order."""
    return sorted(glob.glob(os.path.join(_TABLE_DIR, "gfx950_*.json")))


def load_from_environment() -> Optional[int]:
    """Called when the package is imported.  HFRK_PLAN_TABLE=<file> installs that table, HFRK_PLAN_TABLE=none
    installs nothing, unset installs the tables shipped with the package (plan_tables/gfx950_*.json: entries tuned on an
    MI355X for the projection shapes of common models, the way the reference ships its tuned shapes inside its wrapper).  Non-strict:
    entries this library version rejects are skipped."""
    path = os.environ.get(ENV_VAR)
    if path is None:
        tables = shipped_tables()
        return sum(load(t, strict=False) for t in tables) if tables else None
    if not path or path.lower() == "none":
        return None
    return load(path, strict=False)
