"""TEST INFRASTRUCTURE -- ctypes door onto oracle/_ref/libref_memory.so, the reference's own
memory planner (src/structure/memory/*.cpp) compiled by oracle/Makefile from /root/reference."""
from __future__ import annotations

import ctypes
import os
from typing import List, Sequence, Tuple

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "libref_memory.so")


def available() -> bool:
    return os.path.exists(LIB_PATH)


_lib = None


def plan(kind: int, requests: Sequence[Tuple[int, int, int]]) -> Tuple[List[int], int]:
    """kind 0 = PlainInfos + LinearPlan, 1 = GreedyInfos + GreedyPlan."""
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(LIB_PATH)
    n = len(requests)
    arr = ctypes.c_uint64 * max(n, 1)
    starts = arr(*[r[0] for r in requests])
    ends = arr(*[r[1] for r in requests])
    sizes = arr(*[r[2] for r in requests])
    offsets = arr()
    maximum = ctypes.c_uint64(0)
    rc = _lib.ref_memory_plan(ctypes.c_int(kind), ctypes.c_int(n), starts, ends, sizes, offsets, ctypes.byref(maximum))
    if rc != 0:
        raise RuntimeError(f"ref_memory_plan returned {rc}")
    return [int(offsets[i]) for i in range(n)], int(maximum.value)
