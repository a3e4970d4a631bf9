"""Whole-graph GPU parity for the other benchmark configurations (ConvBERT, GPT-NeoX prefill,
EfficientNet-B0, VGG-16) at reduced width/depth: Executor.compile + invoke against the oracle's
graph runner on the same seeded weights and inputs, with the reference's plain layouts and with
DP-chosen (reversed) layouts.  The full-size graphs only differ in extents; their plans are frozen
by the CPU suite and their throughput is reported by bench.py --config."""
import sys

import numpy as np
import pytest

from oracle import graph_runner
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _cases():
    from fluidml_amd import models

    return {
        "convbert": (lambda: models.convbert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32),
                     lambda: models.bert_inputs(16, 100, seed=7)),
        "gpt_neox": (lambda: models.gpt_neox(seq=24, layers=2, hidden=64, heads=2, ffn=128, vocab=120),
                     lambda: models.gpt_neox_inputs(24, 120, seed=8)),
        # other extents: other memory plans under the same fusion passes
        "convbert_wide": (lambda: models.convbert_base(seq=40, layers=3, hidden=96, heads=6, ffn=192, vocab=64, max_pos=64),
                          lambda: models.bert_inputs(40, 64, seed=17)),
        "gpt_neox_deep": (lambda: models.gpt_neox(seq=48, layers=3, hidden=128, heads=4, ffn=256, vocab=90),
                          lambda: models.gpt_neox_inputs(48, 90, seed=18)),
        "efficientnet_b0": (lambda: models.efficientnet_b0(image=64, classes=10, width_div=4),
                            lambda: models.image_input((1, 3, 64, 64), seed=9)),
        "vgg16": (lambda: models.vgg16(batch=2, image=32, classes=10, width_div=8, fc=512),
                  lambda: models.image_input((2, 3, 32, 32), seed=10)),
    }


@pytest.mark.parametrize("flavour", ["plain_greedy", "dp_greedy"])
@pytest.mark.parametrize("config", ["convbert", "gpt_neox", "efficientnet_b0", "vgg16", "convbert_wide", "gpt_neox_deep"])
def test_config_matches_oracle(device, config, flavour, tmp_path, monkeypatch):
    from fluidml_amd import fluidml

    make_net, make_feeds = _cases()[config]
    net, feeds = make_net(), make_feeds()
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / f"{config}.onnx"))
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    print("[case]", config, flavour, len(net.nodes), "nodes", flush=True)
    sys.stdout.flush()
    ex = getattr(fluidml.Executor, "make_" + flavour)(config, 2)
    ex.compile(path)
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    for _ in range(2):
        assert ex.invoke(args) > 0
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"{config} {flavour} {name}")


@pytest.mark.parametrize("config", ["convbert", "gpt_neox", "convbert_wide", "efficientnet_b0"])
def test_without_tensors_moved_out_of_the_arena(device, config, tmp_path, monkeypatch):
    """FLUIDML_MOVE_OUT_OFF=1: every tensor stays where the memory plan put it, so the fusions that need a buffer
    of their own do not happen and the launches they replaced run instead (the Pad -> Gather -> Transpose copy of
    ConvBERT's convolution branch among them); fewer tensors live outside the arena, the results are the same."""
    from fluidml_amd import fluidml

    make_net, make_feeds = _cases()[config]
    net, feeds = make_net(), make_feeds()
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / f"{config}.onnx"))
    plans = {}
    for off in ("", "1"):
        if off:
            monkeypatch.setenv("FLUIDML_MOVE_OUT_OFF", off)
        print("[case]", config, "FLUIDML_MOVE_OUT_OFF =", off or "(unset)", flush=True)
        ex = fluidml.Executor.make_plain_greedy(config + off, 1)
        ex.compile(path)
        plans[off] = ex.plan()
        args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
        outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
        args.update(outs)
        assert ex.invoke(args) > 0
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"{config} FLUIDML_MOVE_OUT_OFF={off} {name}")
    kept = plans["1"]
    assert all(not l["moved_out"] and not l["writes_inside"] for l in kept["launches"])
    runs = lambda plan: len([l for l in plan["launches"] if l["kind"] not in ("View", "Placed")])
    assert runs(kept) >= runs(plans[""])
    if config.startswith("convbert"):
        assert any(l["kind"] == "PadViewCopy" for l in kept["launches"])
        assert any(l["writes_inside"] for l in plans[""]["launches"])


@pytest.mark.parametrize("use_graph", [True, False], ids=["captured", "eager"])
@pytest.mark.parametrize("config", ["convbert", "gpt_neox", "efficientnet_b0", "convbert_wide", "gpt_neox_deep"])
def test_side_branches_match_oracle(device, config, use_graph, tmp_path):
    """Independent runs of launches issued on two streams (fork, two branches, join), forced on the small graphs by
    a zero threshold: same results as the oracle, replay after replay, in a captured graph and launch by launch; what
    the side branch writes lives in buffers of its own."""
    from fluidml_amd import fluidml

    make_net, make_feeds = _cases()[config]
    net, feeds = make_net(), make_feeds()
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / f"{config}.onnx"))
    ex = fluidml.Executor.make_plain_greedy(config, 2)
    ex.context().set_branch_min_us(0.0)
    ex.context().set_branch_check(False)  # keep every region, faster or not
    ex.context().set_use_graph(use_graph)
    ex.compile(path)
    plan = ex.plan()
    print("[case]", config, "regions", plan["regions"], flush=True)
    if config != "efficientnet_b0":  # (a chain of blocks: nothing runs side by side there)
        assert len(plan["regions"]) >= 2
    for a, b, e in plan["regions"]:
        for l in plan["launches"][b:e]:
            assert all(w["space"] in ("private", "interface") for w in l["writes"])
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    for _ in range(3):
        assert ex.invoke(args) > 0
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"{config} side branches {name}")


OTHER_EXTENTS = [("convbert", (8, 1, 32, 2, 64)), ("convbert", (56, 2, 128, 4, 320)), ("convbert", (33, 3, 64, 4, 100)),
                 ("bert", (24, 2, 96, 6, 128)), ("bert", (72, 1, 192, 12, 256)),
                 ("gpt_neox", (8, 1, 64, 2, 64)), ("gpt_neox", (64, 3, 256, 4, 512)), ("gpt_neox", (25, 2, 128, 8, 128))]


@pytest.mark.parametrize("family,dims", OTHER_EXTENTS, ids=str)
def test_other_extents_match_oracle(device, family, dims, tmp_path):
    """The transformer builders at a spread of extents (sequence lengths that are not multiples of the tiles, one to
    three layers, 2 to 12 heads): every extent gives the memory plan other offsets and the fusion passes other
    conflicts to respect.  With the schedule's default choices and with side branches forced, against the oracle."""
    from fluidml_amd import fluidml, models

    seq, layers, hidden, heads, ffn = dims
    if family == "gpt_neox":
        net, feeds = models.gpt_neox(seq=seq, layers=layers, hidden=hidden, heads=heads, ffn=ffn, vocab=70), models.gpt_neox_inputs(seq, 70, seed=4)
    else:
        make = models.convbert_base if family == "convbert" else models.bert_base
        net = make(seq=seq, layers=layers, hidden=hidden, heads=heads, ffn=ffn, vocab=50, max_pos=128)
        feeds = models.bert_inputs(seq, 50, seed=3)
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / "net.onnx"))
    for forced in (False, True):
        print("[case]", family, dims, "side branches forced" if forced else "default", flush=True)
        ex = fluidml.Executor.make_plain_greedy("extents", 1)
        if forced:
            ex.context().set_branch_min_us(0.0)
            ex.context().set_branch_check(False)
        ex.compile(path)
        args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
        outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
        args.update(outs)
        for _ in range(2):
            assert ex.invoke(args) > 0
            for name, ref in want.items():
                assert_close(outs[name], ref, what=f"{family} {dims} {name}")


@pytest.mark.parametrize("family,dims", [("efficientnet_b0", (96, 2)), ("efficientnet_b0", (160, 4)), ("vgg16", (3, 48, 8)),
                                         ("vgg16", (2, 96, 4)), ("vgg16", (8, 32, 4))], ids=str)
@pytest.mark.parametrize("flavour", ["plain_greedy", "dp_greedy"])
def test_conv_nets_other_extents_match_oracle(device, family, dims, flavour, tmp_path, monkeypatch):
    """The convolutional builders at other image sizes, widths and batches (other tile counts: split and unsplit
    staged-patch convolutions, plane kernels, one- and two-launch squeeze-and-excitation pairs), default and reversed
    layouts, against the oracle."""
    from fluidml_amd import fluidml, models

    if family == "efficientnet_b0":
        image, width_div = dims
        net, feeds = models.efficientnet_b0(image=image, classes=7, width_div=width_div), models.image_input((1, 3, image, image), seed=9)
    else:
        batch, image, width_div = dims
        net = models.vgg16(batch=batch, image=image, classes=10, width_div=width_div, fc=256)
        feeds = models.image_input((batch, 3, image, image), seed=10)
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / "net.onnx"))
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    print("[case]", family, dims, flavour, flush=True)
    ex = getattr(fluidml.Executor, "make_" + flavour)("extents", 1)
    ex.compile(path)
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    for _ in range(2):
        assert ex.invoke(args) > 0
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"{family} {dims} {flavour} {name}")


@pytest.mark.parametrize("which", [0, 1], ids=["matmul_residual", "conv_skip"])
def test_residual_launch_beside_a_concat_matches_oracle(device, which, tmp_path):
    """MatMul + residual and Conv + skip connection whose result is one input of a Concat2 (last axis, and channel
    axis at batch 2): the launch keeps its own output tensor and the graph runs and matches the oracle."""
    from fluidml_amd import fluidml, models

    net, feeds = models.residual_concat_nets()[which]
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / (net.name + ".onnx")))
    for fuse in (True, False):
        ex = fluidml.Executor.make_plain_greedy(net.name)
        ex.context().set_fuse(fuse)
        print("[case]", net.name, "fuse", fuse, flush=True)
        ex.compile(path)
        args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
        outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
        args.update(outs)
        assert ex.invoke(args) > 0
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"{net.name} fuse={fuse} {name}")


def test_side_branch_decision_is_written_and_replayed(device, tmp_path):
    """Whether the side branches of a schedule stay is decided by timing at Compile, written into the executor's
    JSON ("side_branches": {"kept": ...}) and repeated, without timing, by a compile that is given that file --
    also when the file says the opposite of what this machine would measure."""
    import json

    from fluidml_amd import fluidml

    make_net, make_feeds = _cases()["gpt_neox"]
    net, feeds = make_net(), make_feeds()
    want = graph_runner.run_graph(net, feeds)
    path = net.save(str(tmp_path / "neox.onnx"))

    def compile_with(saved, name):
        ex = fluidml.Executor.make_plain_greedy(name)
        ex.context().set_branch_min_us(0.0)  # regions exist even on this small graph
        if saved is not None:
            ex.context().set_tune(saved)
        out = str(tmp_path / (name + ".json"))
        print("[case] compile", name, "saved decisions:", saved, flush=True)
        ex.compile(path, json=out)
        args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
        outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
        args.update(outs)
        assert ex.invoke(args) > 0
        for k, ref in want.items():
            assert_close(outs[k], ref, what=f"{name} {k}")
        return ex, json.load(open(out))

    first, doc = compile_with(None, "timed")
    assert first.branch_decision() in (0, 1)
    assert doc["side_branches"]["kept"] == bool(first.branch_decision())
    for kept in (True, False):
        saved = str(tmp_path / f"kept_{kept}.json")
        json.dump({"side_branches": {"kept": kept}, "contraction_table": doc.get("contraction_table", {})}, open(saved, "w"))
        ex, again = compile_with(saved, f"replayed_{kept}")
        assert ex.branch_decision() == int(kept) and again["side_branches"]["kept"] == kept
        assert (len(ex.plan()["regions"]) > 0) == kept
