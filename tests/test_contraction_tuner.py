"""The tile-configuration pick of the contraction launches (the counterpart of the autotune inside the reference's
MatMul / Gemm generators, src/structure/kernel/generator/matmul.cpp:88-131, gemm.cpp:106-151): selection rule, table
round trip and replay on the CPU; measured picks, replay from the emitted JSON and parity per fixed pick on the GPU."""
import json
import os

import numpy as np
import pytest

FL_ERR_UNSUPPORTED = -8


def _fluidml():
    """fluidml_amd is imported on first use, never while pytest collects: on a GPU box torch has to load its HIP
    runtime before this package's library is loaded (the device fixture does that), or the process ends up with two
    HIP runtimes and the second one to start finds no device."""
    from fluidml_amd import fluidml

    return fluidml


def _models():
    from fluidml_amd import models

    return models


def _fake_device(times, refused=()):
    """launch / elapsed functions over a table {(tile, splits): ns}; configurations in `refused` return the C ABI's
    'unsupported' code."""
    state = {"last": None, "launches": []}

    def launch(bits):
        key = ((bits >> 4) & 0xF, (bits >> 8) & 0x3F)
        state["launches"].append(key)
        if key in refused:
            return FL_ERR_UNSUPPORTED
        state["last"] = key
        return 0

    def elapsed():
        return float(times[state["last"]])

    return launch, elapsed, state


def test_candidates_cover_every_tile_and_the_usual_splits():
    full = _fluidml()._contraction_candidates(True)
    assert len(full) == len(set(full)) == 8 * 9
    assert {t for t, _ in full} == set(range(1, 9))
    assert {s for _, s in full} == {0, 1, 2, 3, 4, 6, 8, 12, 16}
    short = _fluidml()._contraction_candidates(False)
    assert (0, 0) not in short and set(short) == {(t, 0) for t in range(1, 9)} | {(0, s) for s in (1, 2, 4, 8)}


def test_selection_takes_the_fastest_admissible_configuration():
    cands = [(1, 0), (3, 0), (3, 2), (5, 4)]
    times = {(0, 0): 1000, (1, 0): 990, (3, 0): 900, (3, 2): 800, (5, 4): 700}
    launch, elapsed, state = _fake_device(times, refused={(5, 4)})
    tile, splits, ns, rule_ns = _fluidml()._contraction_measure(cands, launch, elapsed, 2, 0.015)
    assert (tile, splits, ns, rule_ns) == (3, 2, 800.0, 1000.0)
    # a refused configuration is tried once and never timed; the others run one warm-up round plus `rounds`
    assert state["launches"].count((5, 4)) == 1 and state["launches"].count((3, 2)) == 3


def test_selection_keeps_the_rule_inside_the_margin():
    # 1 % faster does not replace the rule (two compiles of one graph would flip between equals), 2 % does
    for gain, want in ((0.99, (0, 0)), (0.98, (3, 0))):
        launch, elapsed, _ = _fake_device({(0, 0): 1000, (3, 0): 1000 * gain})
        tile, splits, _, _ = _fluidml()._contraction_measure([(3, 0)], launch, elapsed, 1, 0.015)
        assert (tile, splits) == want


def test_selection_fails_when_the_rule_itself_is_refused():
    launch, elapsed, _ = _fake_device({(0, 0): 1}, refused={(0, 0)})
    with pytest.raises(RuntimeError):
        _fluidml()._contraction_measure([(1, 0)], launch, elapsed, 1, 0.015)


def _small_bert(tmp_path):
    net = _models().bert_base(seq=32, layers=2, hidden=128, heads=4, ffn=256, vocab=500, max_pos=64, seed=3)
    return net, net.save(os.path.join(tmp_path, "bert.onnx"))


def test_saved_table_is_replayed_without_a_device(tmp_path):
    """A table written by one compile fixes the configuration of the next one's launches: nothing is timed (there is
    no device here), signatures the table lacks keep the library's rule."""
    net, path = _small_bert(tmp_path)
    ex = _fluidml().Executor.make_plain_greedy("first")
    ex.compile(path)
    choices = ex.contraction_choices()
    assert len(choices) >= 6 and all(tile == 0 and splits == 0 for _, tile, splits in choices)
    signatures = sorted({sig for sig, _, _ in choices})
    table = {sig: {"tile": 1 + i % 7, "splits": [0, 1, 2][i % 3], "ns": 1000 + i, "rule_ns": 2000} for i, sig in enumerate(signatures[:-1])}
    saved = os.path.join(tmp_path, "saved.json")
    with open(saved, "w") as f:
        json.dump({"contraction_table": table, "side_branches": {"kept": False}}, f)
    ex2 = _fluidml().Executor.make_plain_greedy("second")
    ex2.context().set_tune(saved)
    ex2.compile(path)
    # (without a device the picks are applied when the plan is materialised; the table itself is what compile holds)
    assert json.loads(ex2.context().contraction_table_json()) == table
    # and the table survives a round trip through its own JSON, keys in order
    ctx = _fluidml().Context()
    ctx.load_contraction_table(ex2.context().contraction_table_json())
    assert ctx.contraction_table_json() == ex2.context().contraction_table_json()
    assert list(json.loads(ctx.contraction_table_json())) == sorted(table)


def test_table_rejects_entries_that_name_no_configuration():
    ctx = _fluidml().Context()
    with pytest.raises(RuntimeError):
        ctx.load_contraction_table(json.dumps({"x": {"tile": 9, "splits": 0}}))
    with pytest.raises(RuntimeError):
        ctx.load_contraction_table(json.dumps({"x": {"tile": 1, "splits": 64}}))


def test_generator_signature_follows_the_layouts(tmp_path):
    """Yield keys its kernels by the layout triple (reference generator/matmul.cpp:94-98); the table's key carries
    the strides the layouts give the operands."""
    net, path = _small_bert(tmp_path)
    name = next(n.name for n in net.nodes if n.op_type == "MatMul")
    plain = _fluidml()._contraction_signature(path, name, [0, 1, 2], [0, 1], [0, 1, 2])
    moved = _fluidml()._contraction_signature(path, name, [0, 2, 1], [1, 0], [0, 1, 2])
    assert plain != moved
    assert "(4096,128,1)" in plain and "(128,1)" in plain
    assert "(4096,1,32)" in moved and "(1,128)" in moved
    not_a_contraction = next(n.name for n in net.nodes if n.op_type == "Softmax")
    assert _fluidml()._contraction_signature(path, not_a_contraction, [0, 1, 2, 3], [], [0, 1, 2, 3]) == ""


# ------------------------------------------------------------------------------------------------ on the GPU

def _announce(*what):
    import sys

    print("[case]", *what, flush=True)
    sys.stdout.flush()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(128, 256, 192, 0), (40, 128, 72, 0), (197, 384, 100, 0), (64, 1024, 64, 0), (96, 256, 96, 3)],
                         ids=lambda s: "x".join(map(str, s)))
def test_every_tile_configuration_matches_the_oracle(device, shape):
    """MatMul + bias through fluidml_hip_matmul_chain with every (tile, splits) the flags can name: a configuration
    either refuses the operands (FL_ERR_UNSUPPORTED, output untouched) or gives the oracle's result within the
    tolerance; the same configuration twice gives the same bits (K splits included: partial tiles are added in split
    order).  Shapes: tile multiples, ragged edges in M and N, a long K with few tiles, a base that is not 16-byte
    aligned (which takes the direct-to-LDS tiles away)."""
    import ctypes

    from fluidml_amd import cabi
    from oracle import kernels as ok
    from tests.util import DeviceView, assert_close

    M, K, N, misalign = shape
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    a = rng.uniform(-1, 1, size=(1, M, K)).astype(np.float32)
    w = rng.uniform(-0.5, 0.5, size=(K, N)).astype(np.float32)
    b = rng.uniform(-1, 1, size=(N,)).astype(np.float32)
    t0, want = ok.View.empty((1, M, N)), ok.View.empty((1, M, N))
    ok.matmul(ok.View(a), ok.View(w), t0)
    ok.binary_f32(ok.BOP_ADD, ok.View(b), t0, want)
    da, dw, db = DeviceView(ok.View(a), device, misalign), DeviceView(ok.View(w), device), DeviceView(ok.View(b), device)
    ran, refused = [], []
    for tile in range(0, 9):  # (8: bf16 operands only, refused here like every configuration that does not fit)
        for splits in (0, 1, 2, 3, 4, 8):
            flags = (tile << 4) | (splits << 8)
            outs = []
            for rep in range(2):
                dout = DeviceView(ok.View.empty((1, M, N), np.float32, None, fill=7), device)
                _announce("matmul_chain", shape, "tile", tile, "splits", splits, "run", rep)
                rc = cabi.lib.fluidml_hip_matmul_chain(da.ref(), dw.ref(), db.ref(), dout.ref(), None, ctypes.c_uint32(flags), None)
                got = dout.logical()
                if rc == FL_ERR_UNSUPPORTED:
                    assert (got == 7).all(), "a refused configuration must not launch anything"
                    break
                assert rc == 0, cabi.error_string(rc)
                assert_close(got, want.logical(), what=f"tile {tile} splits {splits}")
                outs.append(got)
            if len(outs) == 2:
                assert np.array_equal(outs[0], outs[1]), f"tile {tile} splits {splits}: two runs differ"
                ran.append((tile, splits))
            else:
                refused.append((tile, splits))
    assert (0, 0) in ran and (1, 0) in ran and (2, 0) in ran  # the rule and the register-staged tiles take anything
    if misalign == 0 and K % 128 == 0:
        assert {(t, 0) for t in range(3, 8)} <= set(ran)  # every direct-to-LDS tile exists for aligned operands
    if misalign != 0:
        assert not any(t >= 3 for t, _ in ran)
    assert all((t, 1) in ran for t, s in ran if s == 0)  # one workgroup per tile is always possible


def _mlp_graph():
    """Two projections at shapes where the library's rule is not the fastest configuration by a wide margin
    ([1024,256]x[256,1024] and [197,768]x[768,768]: 13 % and 18 % in a sweep over all configurations)."""
    g = _models().Net("mlp", 11)
    x = g.input("x", np.float32, (1, 1024, 256))
    y = g.input("y", np.float32, (1, 197, 768))
    h = g.unary("Relu", g.linear(x, g.normal((256, 1024), 0.05), g.normal((1024,), 0.5)))
    g.output(g.linear(h, g.normal((1024, 256), 0.05), g.normal((256,), 0.5)))
    g.output(g.unary("Tanh", g.linear(y, g.normal((768, 768), 0.05), g.normal((768,), 0.5))))
    rng = np.random.default_rng(5)
    feeds = {"x": rng.standard_normal((1, 1024, 256), dtype=np.float32), "y": rng.standard_normal((1, 197, 768), dtype=np.float32)}
    return g, feeds


@pytest.mark.gpu
def test_compile_picks_by_measurement_and_replays_the_pick(device, tmp_path):
    """Compile times the tile configurations of every contraction inside the schedule, keeps the fastest per
    signature and writes the table into its JSON; at least one of this graph's launches ends up off the library's
    rule.  A second compile that is given the JSON times nothing, launches the same configurations and produces the
    same bits; both match the oracle, as does the schedule with tuning switched off."""
    from oracle import graph_runner
    from tests.util import assert_close

    net, feeds = _mlp_graph()
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / "mlp.onnx"))

    def run(tune, name):
        ex = _fluidml().Executor.make_plain_greedy(name)
        ex.context().set_tune(tune)
        out_json = str(tmp_path / (name + ".json"))
        _announce("compile", name, "tune", tune)
        ex.compile(path, json=out_json)
        args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
        outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
        args.update(outs)
        for _ in range(2):
            assert ex.invoke(args) > 0
            for k, ref in want.items():
                assert_close(outs[k], ref, what=f"{name} {k}")
        return ex, out_json, outs

    tuned, tuned_json, tuned_outs = run("measure", "tuned")
    doc = json.load(open(tuned_json))
    table = doc["contraction_table"]
    choices = tuned.contraction_choices()
    print("[picks]", [(t, s) for _, t, s in choices], flush=True)
    assert len(choices) == 3 and {sig for sig, _, _ in choices} == set(table)
    for sig, tile, splits in choices:
        entry = table[sig]
        assert (entry["tile"], entry["splits"]) == (tile, splits)
        assert entry["ns"] > 0 and entry["ns"] <= entry["rule_ns"]
        if (tile, splits) != (0, 0):
            assert entry["ns"] < entry["rule_ns"] * (1 - 0.015)  # the rule is only replaced by a clear win
    assert any((tile, splits) != (0, 0) for _, tile, splits in choices), "the sweep's two clear wins were not picked"

    replayed, _, replayed_outs = run(tuned_json, "replayed")
    assert replayed.contraction_choices() == choices
    for k in tuned_outs:
        assert np.array_equal(tuned_outs[k], replayed_outs[k]), "a fixed pick gives the same bits"

    plain, plain_json, _ = run("off", "rule")
    assert all((t, s) == (0, 0) for _, t, s in plain.contraction_choices())
    assert "contraction_table" not in (json.load(open(plain_json)) or {})  # (the plain planners' JSON is `null`)


@pytest.mark.gpu
def test_generator_yields_a_tuned_kernel_per_layout_triple(device, tmp_path):
    """The DP executor goes through the generators: Yield(lhs, rhs, out layouts) times the standalone kernel's
    configurations for exactly those layouts and records the pick under the layouts' signature (reference
    generator/matmul.cpp:88-131)."""
    net, feeds = _mlp_graph()
    path = net.save(str(tmp_path / "mlp.onnx"))
    ex = _fluidml().Executor.make_dp_greedy("dp")
    ex.context().set_cost_mode("constant")
    ex.context().set_tune("measure")
    _announce("compile dp_greedy, constant costs, tune measure")
    ex.compile(path)
    table = json.loads(ex.context().contraction_table_json())
    standalone = [s for s in table if s.startswith("MatMulKernel") and s.endswith("standalone")]
    assert len(standalone) == 3
    for sig in standalone:
        assert table[sig]["rule_ns"] > 0 and table[sig]["ns"] <= table[sig]["rule_ns"]
