"""The benchmark configurations at their full extents.

* BERT-base with its real extents (seq 128, hidden 768, 12 heads, FFN 3072, vocab 30522) and two of its
  twelve layers against the oracle's graph runner (a few seconds of scalar loop nests): every launch of a
  layer at the shape bench.py times it at.
* Every configuration at full size and full depth, where the oracle would take minutes: the fused launch
  schedule against the one-launch-per-node schedule (FLUIDML_FUSE=0) of the same plan on the same inputs.
  The per-node kernels are the ones the kernel tests pin against the oracle; the fused launches re-associate
  sums (attention, split K, grouped projections), so the two agree within the fp32 tolerance the
  configurations are specified with (rel 1e-4 / abs 1e-5), not bit for bit.
"""
import sys

import numpy as np
import pytest

from oracle import graph_runner
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _run(fluidml, net, feeds, path, name):
    ex = fluidml.Executor.make_plain_greedy(name, 1)
    ex.compile(path)
    args = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    outs = {v.name: np.full(v.shape, np.nan, dtype=v.dtype) for v in net.outputs}
    args.update(outs)
    assert ex.invoke(args) > 0
    return outs, ex.plan()


def test_bert_base_extents_match_oracle(device, tmp_path):
    from fluidml_amd import fluidml, models

    net = models.bert_base(layers=2)
    feeds = models.bert_inputs(128, 30522, seed=11)
    print("[case] bert_base extents, 2 layers,", len(net.nodes), "nodes", flush=True)
    sys.stdout.flush()
    want = graph_runner.run_graph(net, feeds)
    outs, plan = _run(fluidml, net, feeds, net.save(str(tmp_path / "bert2.onnx")), "bert2")
    kinds = {l["kind"] for l in plan["launches"]}
    assert {"Attention", "MatMulGroup", "AddLayerNormalization"} <= kinds
    for name, ref in want.items():
        assert_close(outs[name], ref, what=f"bert_base (2 layers) {name}")


def _full_configs():
    from fluidml_amd import models

    return {
        "bert_base": (models.bert_base, lambda: models.bert_inputs(128, 30522, seed=12)),
        "convbert_base": (models.convbert_base, lambda: models.bert_inputs(128, 30522, seed=13)),
        "gpt_neox": (models.gpt_neox, lambda: models.gpt_neox_inputs(256, 50304, seed=14)),
        "efficientnet_b0": (models.efficientnet_b0, lambda: models.image_input((1, 3, 224, 224), seed=15)),
        "vgg16_b1": (lambda: models.vgg16(batch=1), lambda: models.image_input((1, 3, 224, 224), seed=16)),
    }


@pytest.mark.parametrize("config", ["bert_base", "convbert_base", "gpt_neox", "efficientnet_b0", "vgg16_b1"])
def test_full_size_fused_matches_unfused(device, config, tmp_path, monkeypatch):
    from fluidml_amd import fluidml

    make_net, make_feeds = _full_configs()[config]
    net, feeds = make_net(), make_feeds()
    path = net.save(str(tmp_path / f"{config}.onnx"))
    print("[case] full size", config, len(net.nodes), "nodes", flush=True)
    sys.stdout.flush()
    monkeypatch.setenv("FLUIDML_FUSE", "0")
    plain, plain_plan = _run(fluidml, net, feeds, path, config + "_plain")
    monkeypatch.setenv("FLUIDML_FUSE", "1")
    fused, fused_plan = _run(fluidml, net, feeds, path, config + "_fused")
    assert len(plain_plan["launches"]) == len(net.nodes) > len(fused_plan["launches"])
    # the launch kinds each configuration is expected to exercise at full size
    expected = {"bert_base": {"Attention", "MatMulGroup", "GatherAdd"}, "convbert_base": {"Attention", "SoftmaxMatVec"},
                "gpt_neox": {"Attention", "Rotary", "AddAdd"}, "efficientnet_b0": {"ConvChain", "ConvPair"},
                "vgg16_b1": {"ConvChain", "GemmChain"}}[config]
    assert expected <= {l["kind"] for l in fused_plan["launches"]}
    for name, ref in plain.items():
        assert np.isfinite(ref).all()
        assert_close(fused[name], ref, what=f"{config} fused vs per-node {name}")
