"""Writes tests/golden/bert_base_s128_plan.json and tests/golden/config_plans.json: the arena plans this
backend computes for the headline workload (BERT-base, batch 1, seq 128) and for the other benchmark
configurations at full size, frozen as regression fixtures.

The reference itself cannot produce this fixture here (its pipeline needs MLIR/LLVM 18 and the ONNX
protobuf library), so the fixture pins *this* implementation; the planner core underneath is checked
against the reference's own sources in tests/test_memory_plan.py.

    python tests/golden/make_plan_fixture.py
"""
import json
import os
import sys
import tempfile
import zlib

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from fluidml_amd import fluidml, models  # noqa: E402


# name -> (description, graph factory); the CPU suite rebuilds each graph and compares
CONFIGS = {
    "convbert_base_s128": ("ConvBERT-base, batch 1, seq 128 (models.convbert_base(), seed 2345)", lambda: models.convbert_base()),
    "gpt_neox_s256": ("GPT-NeoX-style prefill, batch 1, seq 256 (models.gpt_neox(), seed 3456)", lambda: models.gpt_neox()),
    "efficientnet_b0": ("EfficientNet-B0, batch 1, 224x224 (models.efficientnet_b0(), seed 4567)", lambda: models.efficientnet_b0()),
    "vgg16_b1": ("VGG-16, batch 1, 224x224 (models.vgg16(1), seed 5678)", lambda: models.vgg16(1)),
    "vgg16_b8": ("VGG-16, batch 8, 224x224 (models.vgg16(8), seed 5678)", lambda: models.vgg16(8)),
}


def plan_of(net, tmp):
    path = net.save(os.path.join(tmp, net.name + ".onnx"))
    graph = fluidml.Parser.make().run(path)
    os.remove(path)
    flow = fluidml.Converter.make().run(graph)
    sequence, index, _ = fluidml.Context().make_plain_greedy_planner().run(flow)
    items = index.items()
    names = sorted(items)
    return {
        "planner": "plain greedy",
        "nodes": len(sequence.node_names()),
        "arena_bytes": index.get_maximum(),
        "offsets_crc32": zlib.crc32(json.dumps(sorted((k, v[0], v[1]) for k, v in items.items())).encode()),
        "order_crc32": zlib.crc32("\n".join(sequence.node_names()).encode()),
        "sample": {n: list(items[n]) for n in names[:: max(1, len(names) // 24)]},
    }


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    with tempfile.TemporaryDirectory() as tmp:
        doc = plan_of(models.bert_base(), tmp)
        doc["workload"] = "BERT-base encoder, batch 1, seq 128 (fluidml_amd.models.bert_base(), seed 1234)"
        out = os.path.join(here, "bert_base_s128_plan.json")
        json.dump(doc, open(out, "w"), indent=1, sort_keys=True)
        print("wrote", out, "arena bytes", doc["arena_bytes"])
        docs = {}
        for name, (what, make) in CONFIGS.items():
            docs[name] = plan_of(make(), tmp)
            docs[name]["workload"] = what
            print(name, "arena bytes", docs[name]["arena_bytes"], "nodes", docs[name]["nodes"])
        out = os.path.join(here, "config_plans.json")
        json.dump(docs, open(out, "w"), indent=1, sort_keys=True)
        print("wrote", out)


if __name__ == "__main__":
    main()
