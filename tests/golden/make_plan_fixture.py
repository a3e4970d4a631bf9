"""Writes tests/golden/bert_base_s128_plan.json: the arena plan this backend computes for the
headline workload (BERT-base, batch 1, seq 128), frozen as a regression fixture.

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


def main():
    net = models.bert_base()
    with tempfile.TemporaryDirectory() as tmp:
        path = net.save(os.path.join(tmp, "bert.onnx"))
        graph = fluidml.Parser.make().run(path)
        flow = fluidml.Converter.make().run(graph)
        sequence, index, _ = fluidml.Context().make_plain_greedy_planner().run(flow)
    items = index.items()
    names = sorted(items)
    sample = {n: list(items[n]) for n in names[:: max(1, len(names) // 24)]}
    doc = {
        "workload": "BERT-base encoder, batch 1, seq 128 (fluidml_amd.models.bert_base(), seed 1234)",
        "planner": "plain greedy",
        "nodes": len(sequence.node_names()),
        "arena_bytes": index.get_maximum(),
        "offsets_crc32": zlib.crc32(json.dumps(sorted((k, v[0], v[1]) for k, v in items.items())).encode()),
        "order_crc32": zlib.crc32("\n".join(sequence.node_names()).encode()),
        "sample": sample,
    }
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bert_base_s128_plan.json")
    json.dump(doc, open(out, "w"), indent=1, sort_keys=True)
    print("wrote", out, "arena bytes", doc["arena_bytes"])


if __name__ == "__main__":
    main()
