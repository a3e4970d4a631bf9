"""The arena planner must produce the reference's offsets bit for bit.

Three implementations are compared on the same seeded request sets:
  * the reference's own src/structure/memory/*.cpp, compiled into oracle/_ref/libref_memory.so,
  * the Python restatement oracle/memory_plan.py,
  * the product planner (fluidml_amd/csrc/host/structure/memory/memory.cpp) through `fluidml._plan_memory`.
plus closed forms and the no-overlap invariant the reference only asserts in DEBUG builds
(reference greedy.cpp:72-93 Manager::Check).
"""
import numpy as np
import pytest

from oracle import memory_plan, ref_memory


def product_plan(kind, requests):
    from fluidml_amd import fluidml

    offsets, maximum = fluidml._plan_memory(kind, [r[0] for r in requests], [r[1] for r in requests], [r[2] for r in requests])
    return list(offsets), maximum


def random_requests(rng, n, steps, sizes):
    reqs = []
    for _ in range(n):
        a, b = sorted(rng.integers(0, steps, size=2).tolist())
        reqs.append((a, b, int(rng.choice(sizes))))
    return reqs


CASES = [
    # (count, time steps, size menu): few distinct sizes force heap ties, as BERT's equal tensors do
    (5, 4, [4, 8]),
    (12, 6, [64, 64, 128]),
    (30, 12, [393216, 393216, 786432, 1572864, 6144, 512]),
    (60, 40, [16, 32, 48, 64, 100, 4096]),
    (120, 30, [393216]),
    (200, 416, [393216, 393216, 393216, 786432, 1572864, 6144, 512, 128]),
]

needs_ref = pytest.mark.skipif(not ref_memory.available(), reason="oracle/_ref/libref_memory.so not built")


@needs_ref
@pytest.mark.parametrize("count,steps,sizes", CASES)
def test_greedy_matches_reference_sources(count, steps, sizes):
    rng = np.random.default_rng(count * 1000 + steps)
    for trial in range(150 if count <= 60 else 25):
        reqs = random_requests(rng, count, steps, sizes)
        want = ref_memory.plan(1, reqs)
        assert memory_plan.greedy_plan(reqs) == want, f"python restatement, trial {trial}"
        assert product_plan(1, reqs) == want, f"product planner, trial {trial}"


@needs_ref
def test_greedy_matches_reference_on_degenerate_requests():
    rng = np.random.default_rng(7)
    for trial in range(300):
        n = int(rng.integers(1, 25))
        reqs = random_requests(rng, n, 5, [0, 0, 1, 3, 3, 8])  # zero sizes: Busy ignores empty ranges
        want = ref_memory.plan(1, reqs)
        assert memory_plan.greedy_plan(reqs) == want
        assert product_plan(1, reqs) == want


@needs_ref
def test_linear_matches_reference_sources():
    rng = np.random.default_rng(3)
    for _ in range(50):
        reqs = random_requests(rng, int(rng.integers(1, 40)), 20, [4, 64, 100, 4096])
        want = ref_memory.plan(0, reqs)
        assert memory_plan.linear_plan(reqs) == want
        assert product_plan(0, reqs) == want


@needs_ref
def test_empty_lifetime_request_like_an_unused_value():
    """(SIZE_MAX, 0) is what the reference's planner builds for a value without users
    (reference planner.cpp:262-279 in a release build): it co-lives with nothing and lands at 0."""
    size_max = (1 << 64) - 1
    reqs = [(0, 3, 100), (size_max, 0, 40), (1, 2, 100)]
    want = ref_memory.plan(1, reqs)
    assert want[0][1] == 0
    assert memory_plan.greedy_plan([(0, 3, 100), (size_max, 0, 40), (1, 2, 100)])[0][1] == 0
    assert product_plan(1, reqs) == want


@pytest.mark.parametrize("impl", ["product", "python"])
def test_closed_forms(impl):
    plan = (lambda r: product_plan(1, r)) if impl == "product" else memory_plan.greedy_plan
    # lifetimes more than one step apart never meet: everything at offset 0
    apart = [(0, 0, 100), (2, 2, 60), (4, 4, 100), (6, 6, 30)]
    assert plan(apart) == ([0, 0, 0, 0], 100)
    # all alive together: stacked from 0 in descending size order
    together = [(0, 5, 30), (0, 5, 100), (0, 5, 60)]
    offsets, maximum = plan(together)
    assert maximum == 190 and offsets == [160, 0, 100]
    # adjacent steps count as overlapping (lifetimes are widened by one, reference greedy.cpp:248)
    adjacent = [(0, 0, 100), (1, 1, 100)]
    assert plan(adjacent) == ([0, 100], 200)
    # a hole below the first busy run is never reused (reference greedy.cpp:180-207)
    reqs = [(0, 0, 100), (0, 4, 50), (4, 4, 10)]
    offsets, _ = plan(reqs)
    assert offsets[0] == 0 and offsets[1] == 100 and offsets[2] == 150


@pytest.mark.parametrize("impl", ["product", "python"])
def test_no_two_live_tensors_overlap(impl):
    plan = (lambda r: product_plan(1, r)) if impl == "product" else memory_plan.greedy_plan
    rng = np.random.default_rng(11)
    for _ in range(40):
        reqs = random_requests(rng, 80, 50, [393216, 786432, 1572864, 6144, 512, 128, 24])
        offsets, maximum = plan(reqs)
        assert maximum == max(o + r[2] for o, r in zip(offsets, reqs))
        for i, (si, ei, zi) in enumerate(reqs):
            for j in range(i + 1, len(reqs)):
                sj, ej, zj = reqs[j]
                if si <= ej and sj <= ei and zi and zj:  # alive at a common step
                    assert offsets[i] + zi <= offsets[j] or offsets[j] + zj <= offsets[i], (i, j)
        # the arena is at least as big as the busiest step needs
        busiest = max(sum(z for s, e, z in reqs if s <= t <= e) for t in range(50))
        assert maximum >= busiest


def test_pop_order_is_libstdcxx_heap_order():
    """GreedyInfos' tie order among equal sizes: checked against std::priority_queue through the product
    (which uses the same container as the reference) by planning requests that never co-live, so the
    placement order is invisible, and requests that always co-live, so offsets reveal the pop order."""
    sizes = [8, 8, 8, 16, 8, 16, 8, 8, 4, 8]
    reqs = [(0, 9, s) for s in sizes]
    offsets, _ = product_plan(1, reqs)
    order = sorted(range(len(sizes)), key=lambda i: offsets[i])
    assert order == memory_plan.greedy_pop_order(sizes)
