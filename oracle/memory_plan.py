"""TEST INFRASTRUCTURE -- Python restatement of FluidML's arena planners.

Follows reference src/structure/memory/{info,linear,greedy}.cpp: requests are (start, end, size)
triples pushed in a given order; `linear_plan` bump-allocates in push order, `greedy_plan` pops the
largest request first (std::priority_queue over size only -> heapq-free restatement of libstdc++'s
push_heap/pop_heap below) and best-fits it between the address ranges of already placed requests
whose widened lifetimes meet its own.

Pinned by tests/test_memory_plan.py against oracle/_ref/libref_memory.so (the reference's own sources,
compiled) on thousands of seeded request sets, and by closed forms.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

SIZE_MAX = (1 << 64) - 1


# --- libstdc++ binary max-heap (bits/stl_heap.h: __push_heap / __adjust_heap), comparator = size only
def _push_heap(heap: list, less) -> None:
    hole = len(heap) - 1
    value = heap[hole]
    parent = (hole - 1) // 2
    while hole > 0 and less(heap[parent], value):
        heap[hole] = heap[parent]
        hole = parent
        parent = (hole - 1) // 2
    heap[hole] = value


def _pop_heap(heap: list, less):
    """Moves the top to the back and restores the heap on the rest, as std::pop_heap does."""
    last = len(heap) - 1
    value = heap[last]
    heap[last] = heap[0]
    length = last
    hole = 0
    child = 0
    while child < (length - 1) // 2:
        child = 2 * (child + 1)
        if less(heap[child], heap[child - 1]):
            child -= 1
        heap[hole] = heap[child]
        hole = child
    if (length & 1) == 0 and child == (length - 2) // 2:
        child = 2 * (child + 1)
        heap[hole] = heap[child - 1]
        hole = child - 1
    # __push_heap(first, hole, top=0, value)
    parent = (hole - 1) // 2
    while hole > 0 and less(heap[parent], value):
        heap[hole] = heap[parent]
        hole = parent
        parent = (hole - 1) // 2
    heap[hole] = value
    return heap.pop()


def greedy_pop_order(sizes: Sequence[int]) -> List[int]:
    """Indices in the order GreedyInfos pops them (reference info.cpp:36-52)."""
    less = lambda a, b: a[0] < b[0]  # noqa: E731  (InfoCompare: size only)
    heap: list = []
    for i, s in enumerate(sizes):
        heap.append((s, i))
        _push_heap(heap, less)
    order = []
    while heap:
        order.append(_pop_heap(heap, less)[1])
    return order


def _take(runs: List[List[int]], lo: int, hi: int) -> None:
    """Memory::Busy (reference greedy.cpp:97-174) on an ascending list of [lo, hi) runs."""
    if lo >= hi:
        return
    if not runs:
        runs.append([lo, hi])
        return
    first = runs[0]
    if hi < first[0]:
        runs.insert(0, [lo, hi])
        return
    if lo <= first[1] and hi >= first[0]:
        first[0] = min(first[0], lo)
        first[1] = max(first[1], hi)
        if len(runs) > 1 and runs[1][0] <= hi:  # at most one successor, its end taken as is
            first[1] = runs[1][1]
            del runs[1]
        return
    cur = 0
    while cur + 1 < len(runs) and runs[cur + 1][1] < lo:
        cur += 1
    nxt = cur + 1
    while nxt < len(runs) and runs[nxt][0] < hi:
        lo = min(lo, runs[nxt][0])
        hi = max(hi, runs[nxt][1])
        nxt += 1
    has_next = nxt < len(runs)
    apart = (not has_next) or runs[nxt][0] > hi
    if apart and runs[cur][1] >= lo:
        runs[cur][1] = hi
        del runs[cur + 1:nxt]
    elif has_next and runs[nxt][0] <= hi and runs[cur][1] < lo:
        runs[nxt][0] = lo
        del runs[cur + 1:nxt]
    elif apart and runs[cur][1] < lo:
        del runs[cur + 1:nxt]
        runs.insert(cur + 1, [lo, hi])
    elif has_next and runs[cur][1] >= lo and runs[nxt][0] <= hi:
        runs[cur][1] = runs[nxt][1]
        del runs[cur + 1:nxt + 1]
    else:
        raise AssertionError("unreachable branch of Memory::Busy")


def _fit(runs: List[List[int]], size: int) -> int:
    """Memory::Alloc (reference greedy.cpp:176-207): smallest interior gap, else after the tail."""
    if not runs:
        return 0
    where, best = SIZE_MAX, SIZE_MAX
    for i in range(len(runs)):
        if i + 1 < len(runs):
            gap = (runs[i + 1][0] - runs[i][1]) & SIZE_MAX  # size_t arithmetic
            if gap >= size and gap < best:
                where, best = runs[i][1], gap
        elif best == SIZE_MAX:
            where = runs[i][1]
    return where


def greedy_plan(requests: Sequence[Tuple[int, int, int]]) -> Tuple[List[int], int]:
    """requests[i] = (start, end, size) in push order -> (offset per request, arena bytes)."""
    offsets = [0] * len(requests)
    placed = []  # (lo, hi, life_lo, life_hi)
    for i in greedy_pop_order([r[2] for r in requests]):
        start, end, size = requests[i]
        life_lo, life_hi = start, end + 1
        runs: List[List[int]] = []
        for lo, hi, plo, phi in placed:
            if plo <= life_hi and phi >= life_lo:
                _take(runs, lo, hi)
        at = _fit(runs, size)
        placed.append((at, at + size, life_lo, life_hi))
        offsets[i] = at
    maximum = max((o + r[2] for o, r in zip(offsets, requests)), default=0)
    return offsets, maximum


def linear_plan(requests: Sequence[Tuple[int, int, int]]) -> Tuple[List[int], int]:
    """reference linear.cpp:5-15: every request at the current maximum, in push order."""
    offsets, top = [], 0
    for _, _, size in requests:
        offsets.append(top)
        top = max(top, top + size)
    return offsets, top
