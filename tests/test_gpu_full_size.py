"""The benchmark configurations at their full extents and full depth, against the oracle.

Every configuration (BERT-base, ConvBERT-base, GPT-NeoX prefill, EfficientNet-B0, VGG-16 at batch 1 and at
batch 8) is compiled from its ONNX file and run three ways on the same seeded weights and inputs:

* the oracle's graph runner on the CPU (scalar loop nests: 1 s for EfficientNet-B0, 30-90 s for the others),
* the fused launch schedule (what bench.py times),
* the one-launch-per-node schedule (FLUIDML_FUSE=0) of the same plan.

Both GPU schedules have to meet the oracle within the tolerance the configurations are specified with
(rel 1e-4 / abs 1e-5, fp32), element by element.  Only for VGG-16 (LONGEST_SUM below) an element outside it is
referred to the float64 evaluation of the network (tests/torch_reference.py, pinned against the oracle on small
instances by tests/test_oracle_graphs.py): it passes if the GPU value is within the same tolerance of the float64
value, or within rel 1e-4 / abs 3e-5 of it, and at most 1 % of an output may pass that way.  The oracle adds the
products of each dot product one after the other in fp32 like the reference's loop nests, and over the 4,608 to
25,088 terms of VGG-16's late layers that rounding alone exceeds the tolerance on a few logits whose terms cancel
(the test prints the counts: about 10 of 1000 oracle logits are outside the tolerance of the float64 value, with
errors up to 4e-5, against 2e-5 for the GPU).  For VGG-16 at batch 8 the oracle runs the batch-1 graph (same seed, hence the
same weights; tests/test_oracle_graphs.py checks that rows of a batch are independent images) on images 0
and 7.  A BERT-base case with the layouts of the DP executor (constant costs: every tensor stored with its
dimensions reversed) runs the same comparison on non-identity strides at real extents.
"""
import functools

import numpy as np
import pytest

from oracle import graph_runner
from tests.util import assert_close, assert_close_or_exact

pytestmark = pytest.mark.gpu

# Terms of the longest fp32 sum behind an element of the configuration's output.  Only VGG-16's logits (25,088 products
# in its first Gemm, 4,096 in the next two) are long enough for sequential fp32 summation to miss the tolerance by
# itself; every other configuration is held to the plain rule (no entry = no escape).
LONGEST_SUM = {"vgg16_b1": 25088, "vgg16_b8": 25088}


def _run(fluidml, net, feeds, path, name, flavour="plain_greedy"):
    ex = getattr(fluidml.Executor, "make_" + flavour)(name, 1)
    ex.compile(path)
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    assert ex.invoke(args) > 0
    return outs, ex.plan()


def _full_configs():
    from fluidml_amd import models

    return {
        "bert_base": (models.bert_base, lambda: models.bert_inputs(128, 30522, seed=12)),
        "convbert_base": (models.convbert_base, lambda: models.bert_inputs(128, 30522, seed=13)),
        "gpt_neox": (models.gpt_neox, lambda: models.gpt_neox_inputs(256, 50304, seed=14)),
        "efficientnet_b0": (models.efficientnet_b0, lambda: models.image_input((1, 3, 224, 224), seed=15)),
        # batch 1 runs image 0 of the batch of 8, so the oracle's pass over that image serves both
        "vgg16_b1": (lambda: models.vgg16(batch=1), lambda: {"input": _vgg_images()[:1].copy()}),
        "vgg16_b8": (lambda: models.vgg16(batch=8), lambda: {"input": _vgg_images()}),
    }


# the launch kinds each configuration is expected to exercise at full size
_EXPECTED_KINDS = {
    "bert_base": {"Attention", "MatMulGroup", "GatherAddLayerNormalization"},
    "convbert_base": {"Attention", "SoftmaxMatVec"},
    "gpt_neox": {"Attention", "RotaryPair"},
    "efficientnet_b0": {"ConvChain", "ConvPair"},
    "vgg16_b1": {"ConvChain", "GemmChain"},
    "vgg16_b8": {"ConvChain", "GemmChain"},
}


@functools.lru_cache(maxsize=None)
def _vgg_images():
    from fluidml_amd import models

    return models.image_input((8, 3, 224, 224), seed=17)["input"]


@functools.lru_cache(maxsize=None)
def _vgg_oracle(image):
    """the oracle's VGG-16 (batch-1 graph) on one image of the batch: about a minute and a half of loop nests"""
    from fluidml_amd import models

    (ref,) = graph_runner.run_graph(models.vgg16(batch=1), {"input": _vgg_images()[image:image + 1].copy()}).values()
    return ref


def _exact(config, net, feeds, rows):
    """float64 torch forward pass of the configuration (tests/torch_reference.py), rows `rows` of its output"""
    from tests import torch_reference as tr

    if config == "bert_base":
        out = tr.bert(net, feeds, seq=128, layers=12, hidden=768, heads=12, ffn=3072, vocab=30522)
    elif config == "convbert_base":
        out = tr.convbert(net, feeds, seq=128, layers=12, hidden=768, heads=12, ffn=3072, vocab=30522)
    elif config == "gpt_neox":
        out = tr.gpt_neox(net, feeds, seq=256, layers=6, hidden=512, heads=8, ffn=2048, vocab=50304)
    elif config == "efficientnet_b0":
        out = tr.efficientnet_b0(net, feeds)
    else:
        out = tr.vgg16(net, feeds)
    return out.numpy()[rows]


def _oracle(config, net, feeds, progress):
    """name -> (rows of the output the oracle computed, expected values)"""
    if not config.startswith("vgg16"):
        return {name: (slice(None), ref) for name, ref in graph_runner.run_graph(net, feeds).items()}
    (out_name,) = [v.name for v in net.outputs]
    rows, refs = ([0], []) if config == "vgg16_b1" else ([0, 7], [])
    for b in rows:
        progress("[oracle] vgg16 image", b)
        refs.append(_vgg_oracle(b))
    return {out_name: (rows, np.concatenate(refs, axis=0))}


@pytest.mark.parametrize("config", ["efficientnet_b0", "bert_base", "convbert_base", "gpt_neox", "vgg16_b1", "vgg16_b8"])
def test_full_size_matches_oracle(device, config, tmp_path, monkeypatch, progress):
    from fluidml_amd import fluidml

    make_net, make_feeds = _full_configs()[config]
    net, feeds = make_net(), make_feeds()
    path = net.save(str(tmp_path / f"{config}.onnx"))
    progress("[case] full size", config, len(net.nodes), "nodes: oracle")
    want = _oracle(config, net, feeds, progress)
    progress("[case] full size", config, "per-node launches")
    monkeypatch.setenv("FLUIDML_FUSE", "0")
    plain, plain_plan = _run(fluidml, net, feeds, path, config + "_plain")
    progress("[case] full size", config, "fused launches")
    monkeypatch.setenv("FLUIDML_FUSE", "1")
    fused, fused_plan = _run(fluidml, net, feeds, path, config + "_fused")
    assert len(plain_plan["launches"]) == len(net.nodes) > len(fused_plan["launches"])
    assert _EXPECTED_KINDS[config] <= {l["kind"] for l in fused_plan["launches"]}
    cache = {}

    def exact_rows(rows):
        if "out" not in cache:
            progress("[case] full size", config, "float64 torch forward pass")
            cache["out"] = _exact(config, net, feeds, slice(None))
        return cache["out"][rows]

    for name, (rows, ref) in want.items():
        assert np.isfinite(ref).all()
        for what, got in (("per-node launches", plain), ("fused launches", fused)):
            assert_close_or_exact(got[name][rows], ref, lambda: exact_rows(rows), LONGEST_SUM.get(config),
                                  what=f"{config} {what} vs oracle, {name}", report=progress)
    for name, ref in plain.items():  # every row, also those the oracle did not compute
        assert np.isfinite(ref).all()
        assert_close(fused[name], ref, what=f"{config} fused vs per-node {name}")


def test_bert_base_dp_layouts_match_oracle(device, tmp_path, monkeypatch, progress):
    """DP executor at BERT-base extents (4 layers): with constant costs every internal tensor is stored with its
    dimensions reversed, so every kernel and every fused launch runs on non-identity strides at the real shapes."""
    from fluidml_amd import fluidml, models

    net = models.bert_base(layers=4)
    feeds = models.bert_inputs(128, 30522, seed=18)
    path = net.save(str(tmp_path / "bert4.onnx"))
    progress("[case] bert_base extents, 4 layers, dp_greedy with constant costs: oracle")
    want = graph_runner.run_graph(net, feeds)
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    for fuse in ("0", "1"):
        progress("[case] bert_base extents, dp_greedy, FLUIDML_FUSE =", fuse)
        monkeypatch.setenv("FLUIDML_FUSE", fuse)
        outs, plan = _run(fluidml, net, feeds, path, "bert4_dp" + fuse, flavour="dp_greedy")
        layouts = [list(s["output_layout"]) for s in plan["steps"]]
        assert sum(l != sorted(l) for l in layouts) > len(layouts) // 2, "the DP plan should hold non-identity layouts"
        for name, ref in want.items():
            assert_close(outs[name], ref, what=f"bert_base (4 layers) dp_greedy fuse={fuse} {name}")


def test_vgg16_dp_layouts_match_oracle(device, tmp_path, monkeypatch, progress):
    """A convolutional network under the DP executor at full size (VGG-16, batch 1): with constant costs every
    internal tensor and every weight is stored with its dimensions reversed, so the convolutions, pools and Gemm
    layers run on non-default strides at their real extents (the direct and implicit-GEMM convolution paths that the
    default layouts never reach at these sizes)."""
    from fluidml_amd import fluidml, models

    net = models.vgg16(batch=1)
    feeds = {"input": _vgg_images()[:1].copy()}
    path = net.save(str(tmp_path / "vgg16.onnx"))
    progress("[case] vgg16_b1, dp_greedy with constant costs: oracle (cached if the full-size case ran)")
    ref = _vgg_oracle(0)
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    progress("[case] vgg16_b1, dp_greedy with constant costs: compile + invoke")
    outs, plan = _run(fluidml, net, feeds, path, "vgg16_dp", flavour="dp_greedy")
    layouts = [list(s["output_layout"]) for s in plan["steps"]]
    assert sum(l != sorted(l) for l in layouts) > len(layouts) // 2, "the DP plan should hold non-identity layouts"
    (name,) = [v.name for v in net.outputs]
    assert_close_or_exact(outs[name][[0]], ref, lambda: _exact("vgg16_b1", net, feeds, [0]), LONGEST_SUM["vgg16_b1"],
                          what=f"vgg16_b1 dp_greedy (constant costs) {name}", report=progress)
