"""Whole-graph parity on the GPU: Executor.compile + invoke (the reference's entry points,
include/worker/executor.h:18-36) against the oracle's graph runner on the same seeded weights
and inputs, for the three executor flavours, with and without launch-plan capture, and with
DP-chosen (non-identity) layouts -- which the reference itself never tests numerically
(test/python/node/node_test.py only drives make_plain_greedy)."""
import os
import sys

import numpy as np
import pytest

from oracle import graph_runner
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _mods():
    from fluidml_amd import fluidml, models

    return fluidml, models


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def tiny_bert(tmp_path_factory):
    fluidml, models = _mods()
    net = models.bert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32, seed=5)
    path = str(tmp_path_factory.mktemp("onnx") / "tiny_bert.onnx")
    net.save(path)
    feeds = models.bert_inputs(16, 100, seed=6)
    feeds["attention_mask"][0, 12:] = 0.0  # exercise the additive mask
    want = graph_runner.run_graph(net, feeds)
    return net, path, feeds, want


def _invoke(ex, net, feeds):
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    ns = ex.invoke(args)
    assert ns > 0
    return outs


@pytest.mark.parametrize("flavour", ["plain_linear", "plain_greedy", "dp_greedy"])
@pytest.mark.parametrize("graph", [False, True], ids=["launches", "captured"])
@pytest.mark.parametrize("fuse", [True, False], ids=["fused", "unfused"])
def test_tiny_bert_matches_oracle(device, tiny_bert, flavour, graph, fuse, monkeypatch):
    fluidml, _ = _mods()
    net, path, feeds, want = tiny_bert
    monkeypatch.setenv("FLUIDML_HIP_GRAPH", "1" if graph else "0")
    monkeypatch.setenv("FLUIDML_FUSE", "1" if fuse else "0")
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")  # every tensor gets the reversed layout
    announce("tiny bert", flavour, "graph" if graph else "launches", "fused" if fuse else "unfused")
    ex = getattr(fluidml.Executor, "make_" + flavour)("tiny_" + flavour, 3)
    ex.compile(path)
    plan = ex.plan()
    if fuse:
        assert len(plan["launches"]) < len(plan["steps"])
    else:
        assert len(plan["launches"]) == len(plan["steps"])
    if flavour == "dp_greedy":
        layouts = {s["output"]: s["output_layout"] for s in ex.plan()["steps"]}
        assert any(l != sorted(l) for l in layouts.values()), "DP plan should use non-identity layouts"
    for _ in range(2):  # second call replays the captured plan
        got = _invoke(ex, net, feeds)
        for name, ref in want.items():
            assert_close(got[name], ref, what=f"{flavour} {name}")


def test_dp_measured_layouts_match_oracle(device, tiny_bert, monkeypatch, tmp_path):
    """Layouts picked from hipEvent-measured costs, then replayed from the saved cost table."""
    fluidml, _ = _mods()
    net, path, feeds, want = tiny_bert
    monkeypatch.setenv("FLUIDML_DP_COST", "measure")
    announce("tiny bert dp measured")
    ex = fluidml.Executor.make_dp_greedy("tiny_dp_measured")
    json_path = str(tmp_path / "dp.json")
    ex.compile(path, None, None, json_path)
    got = _invoke(ex, net, feeds)
    for name, ref in want.items():
        assert_close(got[name], ref, what=f"dp measured {name}")
    first = {s["output"]: s["output_layout"] for s in ex.plan()["steps"]}
    # the proposal was timed as a whole against the default layouts and the faster plan kept; "plan" lists what runs
    import json

    doc = json.load(open(json_path))
    assert {"dp_table", "plan", "whole_graph_ns"} <= set(doc)
    timing = doc["whole_graph_ns"]
    assert timing["kept"] == ("dp" if timing["dp"] <= timing["default_layouts"] else "default_layouts")
    assert ("dp_plan" in doc) == (timing["kept"] == "default_layouts")
    for name, layout in first.items():
        if name in doc["plan"] and name not in {v.name for v in net.outputs}:
            assert doc["plan"][name] == layout, name
    # same cost table -> same decision, same layouts
    monkeypatch.setenv("FLUIDML_DP_COST", json_path)
    announce("tiny bert dp replay from table")
    ex2 = fluidml.Executor.make_dp_greedy("tiny_dp_replay")
    ex2.compile(path)
    second = {s["output"]: s["output_layout"] for s in ex2.plan()["steps"]}
    assert first == second
    got = _invoke(ex2, net, feeds)
    for name, ref in want.items():
        assert_close(got[name], ref, what=f"dp replay {name}")


@pytest.mark.parametrize("fuse", [True, False], ids=["fused", "unfused"])
def test_graph_passes_match_oracle(device, tiny_bert, fuse, monkeypatch):
    """With FLUIDML_GRAPH_PASSES=1 the GELU chain and the mask preparation run as the reference's fused nodes
    (AddDivErfAddMulMul, UnsqueezeSubLhsScalarMulRhsScalar); the oracle runs the original, unfused graph."""
    fluidml, _ = _mods()
    net, path, feeds, want = tiny_bert
    monkeypatch.setenv("FLUIDML_GRAPH_PASSES", "1")
    monkeypatch.setenv("FLUIDML_FUSE", "1" if fuse else "0")
    announce("tiny bert graph passes", fuse)
    ex = fluidml.Executor.make_plain_greedy("tiny_passes")
    ex.compile(path)
    kernels = [s["kernel"] for s in ex.plan()["steps"]]
    assert kernels.count("AddDivErfAddMulMulKernel") == 2 and kernels.count("UnsqueezeSubLhsScalarMulRhsScalarKernel") == 1
    assert len(kernels) < len(net.nodes)
    got = _invoke(ex, net, feeds)
    for name, ref in want.items():
        assert_close(got[name], ref, what=f"graph passes {name}")


def test_bf16_opt_in(device, tiny_bert, monkeypatch):
    """FLUIDML_BF16=1 moves every MatMul to the bf16 path; the result stays close to the fp32 oracle but is not
    held to the fp32 tolerance (its error is reported separately by bench.py --bf16)."""
    fluidml, _ = _mods()
    net, path, feeds, want = tiny_bert
    monkeypatch.setenv("FLUIDML_BF16", "1")
    announce("tiny bert bf16")
    ex = fluidml.Executor.make_plain_greedy("tiny_bf16")
    ex.compile(path)
    got = _invoke(ex, net, feeds)
    monkeypatch.setenv("FLUIDML_BF16", "0")
    ex32 = fluidml.Executor.make_plain_greedy("tiny_fp32")
    ex32.compile(path)
    got32 = _invoke(ex32, net, feeds)
    for name, ref in want.items():
        err = np.abs(got[name] - ref).max()
        assert 0 < err < 0.1, f"bf16 path: max abs err {err}"
        assert np.abs(got32[name] - ref).max() < err  # and the default path is the more exact one


def test_invoke_errors(device, tiny_bert):
    fluidml, _ = _mods()
    net, path, feeds, _ = tiny_bert
    ex = fluidml.Executor.make_plain_greedy("tiny_err")
    ex.compile(path)
    args = {k: v for k, v in feeds.items()}
    with pytest.raises((KeyError, IndexError)):  # missing output name: std::out_of_range (reference runner.cpp:70)
        ex.invoke(args)
    args[net.outputs[0].name] = np.zeros((3,), np.float32)
    with pytest.raises(ValueError):
        ex.invoke(args)


def test_profile_and_accounting(device, tiny_bert):
    fluidml, _ = _mods()
    net, path, feeds, _ = tiny_bert
    ex = fluidml.Executor.make_plain_greedy("tiny_prof")
    ex.compile(path)
    plan = ex.plan()
    assert plan["peak_device_bytes"] == plan["arena_bytes"] + plan["constant_bytes"] + plan["interface_bytes"] + plan["private_bytes"]
    _invoke(ex, net, feeds)
    times = ex.profile(2, 5)
    run = [l for l in plan["launches"] if l["kind"] != "View"]  # a view step is not run: its readers use strides
    assert len(times) == len(run)  # one entry per launch of the schedule
    assert sum(len(t["node"].split("+")) for t in times) == len(net.nodes) - (len(plan["launches"]) - len(run))
    assert all(t["ns"] > 0 for t in times)
    mm = [t for t in times if t["kernel"].startswith("MatMulKernel")]
    assert mm and all(t["flops"] > 0 for t in mm)
    assert ex.time_replay_ns(2, 5) > 0


def test_compiler_cli_invoke(device, tiny_bert, tmp_path, capsys):
    """The command-line compiler with the benchmark executables' protocol (reference benchmark/bert.cpp:11-38):
    compile once, Invoke on zero-filled inputs, report the nanoseconds Invoke returns."""
    import json

    from fluidml_amd import compiler

    _, path, _, _ = tiny_bert
    announce("compiler cli", "dp_greedy", "--invoke 3")
    rc = compiler.main(["-n", "cli_bert", "-i", path, "-m", "dp_greedy", "-e", "2", "--json", str(tmp_path / "dp.json"),
                        "--invoke", "3"])
    assert rc == 0
    summary = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert summary["mode"] == "dp_greedy" and len(summary["invoke_ns"]) == 3
    assert all(ns > 0 for ns in summary["invoke_ns"])
    assert (tmp_path / "dp.json").stat().st_size > 0


def test_reference_constant_relayout_switch(device, tmp_path, monkeypatch):
    """FL_REF_CONSTANT_GATHERED (bit 6 of FLUIDML_REF_QUIRKS): under the DP executor a constant stored with a layout
    other than the default is written the reference's way (src/worker/builder.cpp:290-297) and so reads back permuted
    unless the layout's numbering is its own inverse.  The graph's MatMul weight [6, 10] ends up stored transposed
    under constant costs: with the switch the result is the oracle's on the permuted weight, without it the oracle's
    on the weight itself."""
    from oracle import kernels as ok

    fluidml, models = _mods()
    rng = np.random.default_rng(31)
    weight = rng.uniform(-1, 1, size=(6, 10)).astype(np.float32)
    feeds = {"x": rng.uniform(-1, 1, size=(1, 4, 6)).astype(np.float32)}

    def net_with(w):
        g = models.Net("constant_relayout", 1)
        x = g.input("x", np.float32, (1, 4, 6))
        g.output(g.unary("Tanh", g.matmul(g.relu(x), g.const(w))))
        return g

    net = net_with(weight)
    path = net.save(str(tmp_path / "net.onnx"))
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    results = {}
    for quirks in ("0", "64"):
        monkeypatch.setenv("FLUIDML_REF_QUIRKS", quirks)
        announce("constant re-layout, FLUIDML_REF_QUIRKS =", quirks)
        ex = fluidml.Executor.make_dp_greedy("relayout" + quirks)
        ex.compile(path)
        layouts = [op["layout"] for s in ex.plan()["steps"] for op in s["inputs"] if op["space"] == "constant" and list(op["shape"]) == [6, 10]]
        assert layouts == [[1, 0]], layouts
        (results[quirks],) = _invoke(ex, net, feeds).values()
    (name,) = [v.name for v in net.outputs]
    assert_close(results["0"], graph_runner.run_graph(net, feeds)[name], what="constant stored with a layout, ONNX semantics")
    permuted = ok.reference_constant(weight, [1, 0])[1]
    assert not np.array_equal(permuted, weight)
    want = graph_runner.run_graph(net_with(permuted), feeds)[name]
    assert_close(results["64"], want, what="constant stored the reference's way")
    assert not np.allclose(results["64"], results["0"], rtol=1e-3, atol=1e-4)
