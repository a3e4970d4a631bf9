"""Host pipeline without a GPU: ONNX codec, graph -> flow conversion, execution order, lifetimes,
arena plan and layout DP.  Nothing here launches a kernel."""
import itertools
import json
import os
import zlib

import numpy as np
import pytest

from oracle import memory_plan, ref_memory


@pytest.fixture(scope="module")
def mods():
    from fluidml_amd import fluidml, models, onnx_writer

    return fluidml, models, onnx_writer


@pytest.fixture(scope="module")
def tiny(mods, tmp_path_factory):
    fluidml, models, _ = mods
    net = models.bert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32, seed=5)
    path = str(tmp_path_factory.mktemp("onnx") / "tiny_bert.onnx")
    net.save(path)
    return net, path


def staged(fluidml, path, planner="make_plain_greedy_planner"):
    graph = fluidml.Parser.make().run(path)
    flow = fluidml.Converter.make().run(graph)
    ctx = fluidml.Context()
    ctx.set_cost_mode("constant")
    sequence, index, report = getattr(ctx, planner)().run(flow)
    return flow, sequence, index, report


# ------------------------------------------------------------------ ONNX codec

def _onnx_messages():
    """The slice of onnx.proto this backend reads, declared to the protobuf runtime so that the
    protobuf library itself (not this repository's codec) produces and parses the bytes."""
    pytest.importorskip("google.protobuf")
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

    f = descriptor_pb2.FileDescriptorProto(name="onnx_subset.proto", package="onnxsub", syntax="proto2")
    T = descriptor_pb2.FieldDescriptorProto

    def msg(name, fields):
        m = f.message_type.add(name=name)
        for fname, number, ftype, label, type_name in fields:
            fd = m.field.add(name=fname, number=number, type=ftype, label=label)
            if type_name:
                fd.type_name = ".onnxsub." + type_name
        return m

    O, R = T.LABEL_OPTIONAL, T.LABEL_REPEATED
    msg("TensorProto", [("dims", 1, T.TYPE_INT64, R, None), ("data_type", 2, T.TYPE_INT32, O, None),
                        ("float_data", 4, T.TYPE_FLOAT, R, None), ("int32_data", 5, T.TYPE_INT32, R, None),
                        ("int64_data", 7, T.TYPE_INT64, R, None), ("name", 8, T.TYPE_STRING, O, None),
                        ("raw_data", 9, T.TYPE_BYTES, O, None), ("double_data", 10, T.TYPE_DOUBLE, R, None)])
    msg("AttributeProto", [("name", 1, T.TYPE_STRING, O, None), ("f", 2, T.TYPE_FLOAT, O, None),
                           ("i", 3, T.TYPE_INT64, O, None), ("s", 4, T.TYPE_BYTES, O, None),
                           ("t", 5, T.TYPE_MESSAGE, O, "TensorProto"), ("floats", 7, T.TYPE_FLOAT, R, None),
                           ("ints", 8, T.TYPE_INT64, R, None), ("type", 20, T.TYPE_INT32, O, None)])
    msg("NodeProto", [("input", 1, T.TYPE_STRING, R, None), ("output", 2, T.TYPE_STRING, R, None),
                      ("name", 3, T.TYPE_STRING, O, None), ("op_type", 4, T.TYPE_STRING, O, None),
                      ("attribute", 5, T.TYPE_MESSAGE, R, "AttributeProto")])
    msg("Dimension", [("dim_value", 1, T.TYPE_INT64, O, None), ("dim_param", 2, T.TYPE_STRING, O, None)])
    msg("TensorShapeProto", [("dim", 1, T.TYPE_MESSAGE, R, "Dimension")])
    msg("TypeTensor", [("elem_type", 1, T.TYPE_INT32, O, None), ("shape", 2, T.TYPE_MESSAGE, O, "TensorShapeProto")])
    msg("TypeProto", [("tensor_type", 1, T.TYPE_MESSAGE, O, "TypeTensor")])
    msg("ValueInfoProto", [("name", 1, T.TYPE_STRING, O, None), ("type", 2, T.TYPE_MESSAGE, O, "TypeProto")])
    msg("GraphProto", [("node", 1, T.TYPE_MESSAGE, R, "NodeProto"), ("name", 2, T.TYPE_STRING, O, None),
                       ("initializer", 5, T.TYPE_MESSAGE, R, "TensorProto"), ("input", 11, T.TYPE_MESSAGE, R, "ValueInfoProto"),
                       ("output", 12, T.TYPE_MESSAGE, R, "ValueInfoProto"), ("value_info", 13, T.TYPE_MESSAGE, R, "ValueInfoProto")])
    msg("OperatorSetId", [("domain", 1, T.TYPE_STRING, O, None), ("version", 2, T.TYPE_INT64, O, None)])
    msg("ModelProto", [("ir_version", 1, T.TYPE_INT64, O, None), ("producer_name", 2, T.TYPE_STRING, O, None),
                       ("graph", 7, T.TYPE_MESSAGE, O, "GraphProto"), ("opset_import", 8, T.TYPE_MESSAGE, R, "OperatorSetId")])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(f)
    get = getattr(message_factory, "GetMessageClass", None)
    if get is None:
        factory = message_factory.MessageFactory(pool)
        return lambda n: factory.GetPrototype(pool.FindMessageTypeByName("onnxsub." + n))
    return lambda n: get(pool.FindMessageTypeByName("onnxsub." + n))


def test_writer_output_parses_with_the_protobuf_library(mods, tiny):
    """The writer's bytes, read back by google.protobuf against onnx.proto's field numbers."""
    net, path = tiny
    Model = _onnx_messages()("ModelProto")
    m = Model()
    m.ParseFromString(open(path, "rb").read())
    assert m.ir_version == 8 and m.opset_import[0].version == 17
    g = m.graph
    assert [n.name for n in g.node] == [n.name for n in net.nodes]
    assert [n.op_type for n in g.node] == [n.op_type for n in net.nodes]
    assert [i.name for i in g.input] == [v.name for v in net.inputs]
    assert [tuple(d.dim_value for d in i.type.tensor_type.shape.dim) for i in g.input] == [v.shape for v in net.inputs]
    assert len(g.value_info) == len(net.nodes) - len(net.outputs)
    init = {t.name: t for t in g.initializer}
    for v in net.initializers[:20]:
        t = init[v.name]
        assert tuple(t.dims) == v.shape
        assert np.array_equal(np.frombuffer(t.raw_data, dtype=v.dtype).reshape(v.shape), v.const)
    ln = next(n for n in g.node if n.op_type == "LayerNormalization")
    attrs = {a.name: a for a in ln.attribute}
    assert attrs["axis"].i == -1 and attrs["axis"].type == 2
    assert abs(attrs["epsilon"].f - 1e-12) < 1e-18 and attrs["epsilon"].type == 1


def test_reader_accepts_bytes_from_the_protobuf_library(mods, tmp_path):
    """A model serialised by google.protobuf (typed repeated fields, unpacked and packed, negative ints,
    rank-0 initialisers) goes through Parser -> Converter -> Planner."""
    fluidml, _, _ = mods
    cls = _onnx_messages()
    m = cls("ModelProto")()
    m.ir_version = 8
    g = m.graph
    g.name = "pb"

    def vi(lst, name, elem, shape):
        v = lst.add()
        v.name = name
        v.type.tensor_type.elem_type = elem
        for d in shape:
            v.type.tensor_type.shape.dim.add().dim_value = d

    vi(g.input, "x", 1, [2, 3, 4])
    vi(g.output, "y", 1, [2, 4, 3])
    vi(g.value_info, "t0", 1, [2, 3, 4])
    vi(g.value_info, "t1", 1, [2, 3, 4])
    c = g.initializer.add()
    c.name, c.data_type = "half", 1
    c.float_data.append(0.5)  # typed field, rank 0 -> scalar operand
    b = g.initializer.add()
    b.name, b.data_type = "bias", 1
    b.dims.append(4)
    b.float_data.extend([1.0, 2.0, 3.0, 4.0])
    n = g.node.add(name="mul", op_type="Mul")
    n.input.extend(["x", "half"])
    n.output.append("t0")
    n = g.node.add(name="add", op_type="Add")
    n.input.extend(["t0", "bias"])
    n.output.append("t1")
    n = g.node.add(name="tr", op_type="Transpose")
    n.input.append("t1")
    n.output.append("y")
    a = n.attribute.add(name="perm", type=7)
    a.ints.extend([0, 2, 1])
    path = str(tmp_path / "pb.onnx")
    open(path, "wb").write(m.SerializeToString())
    flow, seq, index, _ = staged(fluidml, path)
    assert seq.node_names() == ["mul", "add", "tr"]
    assert seq.kernel_names() == ["MulConstantKernel", "AddCommonKernel", "TransposeKernel"]
    assert index.get_maximum() == 2 * 96  # t0 and t1 live in adjacent steps


def test_converter_rejects_what_the_reference_leaves_unreachable(mods, tmp_path):
    fluidml, models, _ = mods
    g = models.Net("bad", 0)
    x = g.input("x", np.float32, (2, 3))
    y = g.node("Sub", [x, g.scalar(1.0)], (2, 3))  # x - scalar has no FluidML kernel
    g.output(y)
    path = g.save(str(tmp_path / "bad.onnx"))
    with pytest.raises(RuntimeError, match="scalar - x"):
        staged(fluidml, path)
    g = models.Net("bad2", 0)
    x = g.input("x", np.float32, (2, 3))
    g.output(g.node("Sigmoid", [x], (2, 3)))
    with pytest.raises(RuntimeError, match="not supported"):
        staged(fluidml, g.save(str(tmp_path / "bad2.onnx")))


# ------------------------------------------------------------------ order, lifetimes, plan

def users_of(net):
    producer, consumers = {}, {}
    for n in net.nodes:
        producer[n.outputs[0].name] = n.name
        for i in n.inputs:
            consumers.setdefault(i.name, []).append(n.name)
    return producer, consumers


@pytest.mark.parametrize("planner", ["make_plain_linear_planner", "make_plain_greedy_planner", "make_dp_greedy_planner"])
def test_order_lifetimes_and_plan(mods, tiny, planner):
    fluidml, _, _ = mods
    net, path = tiny
    flow, seq, index, _ = staged(fluidml, path, planner)
    order = seq.node_names()
    assert sorted(order) == sorted(n.name for n in net.nodes)
    pos = {name: i for i, name in enumerate(order)}
    producer, consumers = users_of(net)
    inner = {n.outputs[0].name: n.outputs[0] for n in net.nodes} 
    for out in net.outputs:
        inner.pop(out.name)
    # valid topological order
    for n in net.nodes:
        for i in n.inputs:
            if i.name in producer:
                assert pos[producer[i.name]] < pos[n.name]
    # rebuild the planner's requests from first principles, in the planner's push order
    # (reference planner.cpp:236-293): regions in Sequence::GetRegions() order, then node scratch
    requests, names = [], []
    for name in seq.region_names():
        if name in inner and consumers.get(name):
            steps = [pos[producer[name]]] + [pos[c] for c in consumers[name]]
            v = inner[name]
            requests.append((min(steps), max(steps), int(np.prod(v.shape)) * v.dtype.itemsize))
            names.append(name)
    for i, (name, scratch) in enumerate(zip(order, seq.buffer_sizes())):
        if scratch:
            requests.append((i, i, scratch))
            names.append(name)
    got = index.items()
    assert sorted(got) == sorted(names)
    kind = 0 if planner == "make_plain_linear_planner" else 1
    want_offsets, want_max = (memory_plan.linear_plan if kind == 0 else memory_plan.greedy_plan)(requests)
    assert [got[n][0] for n in names] == want_offsets
    assert index.get_maximum() == want_max
    if ref_memory.available():  # and the reference's own planner sources agree on the same requests
        assert ref_memory.plan(kind, requests) == (want_offsets, want_max)
    # tensors alive at a common step never share bytes
    for (a, ra), (b, rb) in itertools.combinations(zip(names, requests), 2):
        if ra[0] <= rb[1] and rb[0] <= ra[1]:
            oa, ob = got[a][0], got[b][0]
            assert oa + ra[2] <= ob or ob + rb[2] <= oa, (a, b)
    # scratch sizes: softmax / layernorm = input shape with the axis collapsed (reference flow/node.cpp:972-985, 1355-1368)
    sizes = dict(zip(order, seq.buffer_sizes()))
    for n in net.nodes:
        if n.op_type in ("Softmax", "LayerNormalization"):
            assert sizes[n.name] == int(np.prod(n.inputs[0].shape[:-1])) * 4
        else:
            assert sizes[n.name] == 0


def test_plan_is_independent_of_layouts(mods, tiny):
    """Layouts change strides, never sizes: DP and plain greedy plans coincide (reference meta.cpp:38-40)."""
    fluidml, _, _ = mods
    _, path = tiny
    _, s1, i1, _ = staged(fluidml, path, "make_plain_greedy_planner")
    _, s2, i2, _ = staged(fluidml, path, "make_dp_greedy_planner")
    assert s1.node_names() == s2.node_names()
    assert i1.items() == i2.items()


def test_golden_bert_base_plan(mods, tmp_path):
    """Arena plan of the headline workload, frozen: a change of container order, heap ties or best-fit
    behaviour shows up here.  (Regenerate with tests/golden/make_plan_fixture.py.)"""
    fluidml, models, _ = mods
    golden_path = os.path.join(os.path.dirname(__file__), "golden", "bert_base_s128_plan.json")
    golden = json.load(open(golden_path))
    net = models.bert_base()
    path = net.save(str(tmp_path / "bert.onnx"))
    _, seq, index, _ = staged(fluidml, path)
    assert index.get_maximum() == golden["arena_bytes"]
    assert len(seq.node_names()) == golden["nodes"]
    items = index.items()
    digest = zlib.crc32(json.dumps(sorted((k, v[0], v[1]) for k, v in items.items())).encode())
    assert digest == golden["offsets_crc32"]
    assert zlib.crc32("\n".join(seq.node_names()).encode()) == golden["order_crc32"]
    for name, (offset, size) in golden["sample"].items():
        assert items[name] == (offset, size), name


@pytest.mark.parametrize("config", ["convbert_base_s128", "gpt_neox_s256", "efficientnet_b0", "vgg16_b1", "vgg16_b8"])
def test_golden_config_plans(mods, tmp_path, config):
    """Arena plans of the other benchmark configurations at full size, frozen like the BERT-base one."""
    import importlib.util

    here = os.path.join(os.path.dirname(__file__), "golden")
    spec = importlib.util.spec_from_file_location("make_plan_fixture", os.path.join(here, "make_plan_fixture.py"))
    fixture = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(fixture)
    golden = json.load(open(os.path.join(here, "config_plans.json")))[config]
    got = fixture.plan_of(fixture.CONFIGS[config][1](), str(tmp_path))
    for key in ("nodes", "arena_bytes", "offsets_crc32", "order_crc32"):
        assert got[key] == golden[key], key
    assert got["sample"] == {k: list(v) for k, v in golden["sample"].items()}


# ------------------------------------------------------------------ graph-level fusion passes

def test_graph_fusion_passes(mods, tmp_path, monkeypatch):
    """The three graph passes (reference src/optimization/graph/*.cpp): each pattern collapses into one fused
    node whose inputs are the chain's constants followed by its variable input; everything else is untouched."""
    fluidml, models, _ = mods
    import numpy as np

    g = models.Net("passes", 11)
    ids = g.input("ids", np.int64, (1, 8))
    mask = g.input("mask", np.float32, (1, 8))
    emb = g.gather(g.normal((50, 16)), ids)                       # Gather(table) -> Add(CT) -> Add(CT)
    emb = g.add(emb, g.normal((1, 8, 16)))
    emb = g.add(emb, g.normal((16,)))
    ext = g.mul(g.sub(g.scalar(1.0), g.unsqueeze(mask, [1, 2])), g.scalar(-10000.0))   # Unsqueeze -> Sub -> Mul
    h = g.erf_gelu(g.linear(emb, g.normal((16, 32)), g.zeros((32,))))                   # Add(bias) -> GELU chain
    s = g.add(g.matmul(h, g.normal((32, 8))), g.reshape(ext, (1, 1, 8)))
    g.output(s)
    path = g.save(str(tmp_path / "passes.onnx"))
    graph = fluidml.Parser.make().run(path)
    before = {n["name"]: n for n in graph.nodes()}
    manager = fluidml.GraphPassesManager()
    manager.register_all_passes()
    manager.run(graph)
    after = {n["name"]: n for n in graph.nodes()}
    ops = sorted(n["op"] for n in after.values())
    assert ops == sorted(["AddDivErfAddMulMul", "GatherAddAdd", "UnsqueezeSubMul", "MatMul", "MatMul", "Add", "Reshape"])
    assert len(before) == 3 + 3 + 1 + 6 + 1 + 1 + 1
    gelu = next(n for n in after.values() if n["op"] == "AddDivErfAddMulMul")
    assert len(gelu["inputs"]) == 5 and len(gelu["name"].split("-")) == 6
    assert gelu["inputs"][4] == next(n for n in before.values() if n["op"] == "MatMul" and n["outputs"][0] == gelu["inputs"][4])["outputs"][0]
    gather = next(n for n in after.values() if n["op"] == "GatherAddAdd")
    assert gather["inputs"][3] == "ids" and len(gather["inputs"]) == 4
    um = next(n for n in after.values() if n["op"] == "UnsqueezeSubMul")
    assert um["inputs"][3] == "mask" and len(um["inputs"]) == 4
    # the fused graph converts and plans; fewer kernels than without the passes
    flow = fluidml.Converter.make().run(graph)
    seq, _, _ = fluidml.Context().make_plain_greedy_planner().run(flow)
    kernels = sorted(seq.kernel_names())
    assert "AddDivErfAddMulMulKernel" in kernels and "UnsqueezeSubLhsScalarMulRhsScalarKernel" in kernels
    assert "GatherConstantDataTensorAddTensorLhsAddTensorLhsKernel" in kernels
    assert len(kernels) == 7
    # through the Executor: off by default (the reference never calls the passes), on with the switch
    ex = fluidml.Executor.make_plain_greedy("no_passes")
    ex.compile(path)
    assert len(ex.plan()["steps"]) == len(before)
    monkeypatch.setenv("FLUIDML_GRAPH_PASSES", "1")
    ex = fluidml.Executor.make_plain_greedy("with_passes")
    ex.compile(path)
    assert len(ex.plan()["steps"]) == 7


# ------------------------------------------------------------------ launch schedule (fusion)

def _overlap(x, y):
    if x["space"] != y["space"]:
        return False
    if x["space"] != "arena":
        return x["name"] == y["name"]
    return x["offset"] < y["offset"] + y["bytes"] and y["offset"] < x["offset"] + x["bytes"]


SCHEDULE_NETS = {
    # the full-size headline graph: its memory plan reuses bytes in ways the small ones do not
    # (third entry: kinds expected with the default layouts only)
    "bert_base_full": (lambda m: m.bert_base(), {"MatMulGroup", "Attention"}, {"GatherAddLayerNormalization"}),
    # the embedding block as the separate launches (two lookups, the second with its Add, Add + LayerNormalization)
    "bert_base_full_separate_embedding": (lambda m: m.bert_base(), {"MatMulGroup", "AddLayerNormalization", "Attention", "GatherAdd"}),
    "bert": (lambda m: m.bert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32, seed=5),
             {"MatMulChain", "Attention", "ElementwiseChain"}, {"GatherAddLayerNormalization"}),
    "convbert": (lambda m: m.convbert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32),
                 {"MatMulChain"}, {"GatherAddLayerNormalization"}),  # whether its attention fuses depends on the plan's reuse of bytes
    # full size: the Concat2 of attention and convolution heads written in place (also into the Reshape behind it),
    # Softmax -> MatMul pairs and attention blocks matched after view elision
    "convbert_base_full": (lambda m: m.convbert_base(), {"MatMulChain"},
                           {"SoftmaxMatVec", "Attention", "Placed", "MatMulGroup", "GatherAddLayerNormalization"}),
    "gpt_neox": (lambda m: m.gpt_neox(seq=24, layers=2, hidden=64, heads=2, ffn=128, vocab=120), {"MatMulChain", "Attention", "View", "RotaryPair"}),
    # full size (vocabulary cut: the projection's weights play no part in the plan): the parallel-residual blocks with
    # both LayerNormalizations of a layer deferred into their readers, side by side with the plan's real reuse of bytes
    "gpt_neox_full": (lambda m: m.gpt_neox(vocab=1024), {"MatMulChain", "Attention", "View", "RotaryPair"}),
    # without the rotary launch its steps go through the general mechanisms: views, Concat2 inputs written in place
    "gpt_neox_no_rotary": (lambda m: m.gpt_neox(seq=24, layers=2, hidden=64, heads=2, ffn=128, vocab=120),
                           {"MatMulChain", "Attention", "View", "CopyInto", "MulAdd"}),
    # other extents: other plans, other reuse of bytes under the same passes
    "convbert_wide": (lambda m: m.convbert_base(seq=40, layers=3, hidden=96, heads=6, ffn=192, vocab=64, max_pos=64),
                      {"MatMulChain"}, {"GatherAddLayerNormalization"}),
    "gpt_neox_deep": (lambda m: m.gpt_neox(seq=48, layers=3, hidden=128, heads=4, ffn=256, vocab=90), {"MatMulChain", "Attention", "View"}),
    "efficientnet_b0": (lambda m: m.efficientnet_b0(image=64, classes=10, width_div=4), {"ConvChain", "ConvPair"}),
    "vgg16": (lambda m: m.vgg16(batch=2, image=32, classes=10, width_div=8, fc=512), {"ConvChain", "GemmChain"}),
}


@pytest.mark.parametrize("flavour", ["make_plain_greedy", "make_plain_linear", "make_dp_greedy"])
@pytest.mark.parametrize("which", list(SCHEDULE_NETS))
def test_fused_schedule_is_safe(mods, which, flavour, monkeypatch, tmp_path):
    """Independent re-check of what the launcher's fusion pass must guarantee: every step is issued once,
    an elided tensor has no reader outside its chain, and moving a chain's reads to its last member's
    position crosses no write to the bytes it reads (arena intervals of the memory plan)."""
    fluidml, models, _ = mods
    if "_full" in which and flavour == "make_plain_linear":
        pytest.skip("the linear plan reuses no bytes: the small graphs cover it, the full-size ones are here for their reuse")
    make, expected_kinds = SCHEDULE_NETS[which][:2]
    if flavour != "make_dp_greedy" and len(SCHEDULE_NETS[which]) > 2:
        expected_kinds = expected_kinds | SCHEDULE_NETS[which][2]
    path = make(models).save(str(tmp_path / "net.onnx"))
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    if which.endswith("_no_rotary"):
        monkeypatch.setenv("FLUIDML_ROTARY", "0")
    if which.endswith("_separate_embedding"):
        monkeypatch.setenv("FLUIDML_EMBEDDING", "0")
    ex = getattr(fluidml.Executor, flavour)("sched")
    ex.compile(path)
    plan = ex.plan()
    steps, launches = plan["steps"], plan["launches"]
    assert sorted(m for l in launches for m in l["members"]) == list(range(len(steps)))
    assert [l["position"] for l in launches] == sorted(l["position"] for l in launches)
    kinds = {l["kind"] for l in launches}
    assert expected_kinds <= kinds
    # A fused launch may write a tensor into a buffer of its own ("moved_out") when the bytes the memory plan holds
    # for it are in use at the time the launch writes it, or are reused before the last launch reads it.
    # Everything below is checked against where the tensor really is, after making sure that every launch reading it
    # was pointed there.
    for l in launches:
        for to in l["moved_out"]:
            assert to["space"] == "private"
            assert to["name"] in ({steps[m]["out"]["name"] for m in l["members"]} | {l.get("writes_into", {}).get("name")}
                                  | {w["into"]["name"] for w in l["writes_inside"]})
            assert any(w["space"] == "private" and w["name"] == to["name"] for w in l["writes"])
            for other in launches:
                assert all(r["space"] == "private" for r in other["reads"] if r["name"] == to["name"])
                if other["kind"] == "View" and other["source"]["name"] == to["name"]:
                    assert other["source"]["space"] == "private"
            for s in steps:
                for op in s["inputs"] + [s["out"]]:
                    if op["name"] == to["name"]:
                        op.update(space="private", offset=0, pool="")
    # (a tensor written into the interior of a padded buffer never touches the bytes the plan holds for it)
    for l in launches:
        for w in l["writes_inside"]:
            redirected = steps[w["step"]]["out"]["name"]
            for s in steps:
                for op in s["inputs"] + [s["out"]]:
                    if op["name"] == redirected:
                        op.update(space="private", offset=0, pool="")
    readers = {}
    for i, s in enumerate(steps):
        for op in s["inputs"]:
            readers.setdefault(op["name"], set()).add(i)
    issued = {}
    for l in launches:
        for m in l["members"]:
            issued[m] = (l["position"], l)
    # A zero Pad that does not run ("writes_inside"): the launch that produces the Pad's input writes it into the
    # interior of the padded tensor, which lives in a buffer of its own outside the arena (zero when it is created).
    # The border stays zero only if nothing else ever writes the buffer; the input has no other reader; the interior
    # is where the Pad would have put the input; the launch runs before the Pad's place.
    padded_in_place = set()
    for l in launches:
        for w in l["writes_inside"]:
            into = w["into"]
            (t,) = [i for i, st in enumerate(steps) if st["out"]["name"] == into["name"] and st["kernel"] == "PadKernel"]
            whole, x = steps[t]["out"], steps[t]["inputs"][0]
            assert whole["space"] == "private" and into["space"] == "private" and whole["pool"] == ""
            assert issued[t][1]["kind"] == "Placed" and issued[t][1]["written"] == [] and l["position"] < t
            assert w["step"] in l["members"] and w["step"] in l["written"]
            assert readers[x["name"]] == {t}, "a Pad input written in place has another reader"
            assert into["shape"] == x["shape"] and whole["layout"] == sorted(whole["layout"])
            strides = [int(np.prod(whole["shape"][d + 1:])) for d in range(len(whole["shape"]))]
            assert list(into["view_strides"]) == strides
            lead = into["view_offset"]
            for d, st in enumerate(strides):  # the interior starts `before` elements in along every dim and fits
                before, lead = divmod(lead, st)
                assert 0 <= before and before + x["shape"][d] <= whole["shape"][d]
            assert lead == 0
            for other in launches:
                if other is l:
                    assert sum(1 for ww in other["writes"] if ww["name"] == into["name"]) == 1
                else:
                    assert all(ww["name"] != into["name"] for ww in other["writes"]), "someone else writes a padded buffer"
            for q, st in enumerate(steps):  # (no step other than the Pad and the redirected producer names it as output)
                if st["out"]["name"] == into["name"]:
                    assert q == t or q == w["step"] or q in {ll["members"][0] for ll in launches if ll["kind"] == "View"}
            padded_in_place.add(t)
    # A step that is not run (kind "View"): its readers address `source`, the bytes of another tensor, when
    # they are issued.  Everything that writes between the view step and such a reader -- outputs of single
    # steps at their own position, outputs of fused launches at the launch's position -- must stay off those
    # bytes, and so must the reader's own launch.
    elided = {l["members"][0] for l in launches if l["kind"] == "View"}
    writes = []  # (position, operand, launch id)
    for k, l in enumerate(launches):
        if l["kind"] != "View":
            writes += [(l["position"], steps[m]["out"], k) for m in l["written"]]
    for l in launches:
        if l["kind"] != "View":
            continue
        (i,) = l["members"]
        assert l["written"] == [] and steps[i]["out"]["space"] in ("arena", "private")
        src = l["source"]
        # a view of a view reads through to a tensor that is materialised
        assert all(steps[j]["out"]["name"] != src["name"] for j in elided), "the source of a view is itself not run"
        pending = list(readers.get(steps[i]["out"]["name"], ()))
        seen = set()
        while pending:
            r = pending.pop()
            if r in seen:
                continue
            seen.add(r)
            assert r > i
            if r in elided:  # reads through: its own readers are the ones that touch the bytes
                pending += list(readers.get(steps[r]["out"]["name"], ()))
                continue
            pos, owner = issued[r]
            assert pos >= i, "a reader of an elided view was hoisted in front of it"
            for wpos, what, k in writes:
                own = launches[k] is owner
                if (i < wpos < pos) or own:
                    assert not _overlap(what, src), "the source of an elided view is overwritten before a reader runs"
    # A launch that writes an input of a Concat2 straight into the Concat2's output ("writes_into"): the plan
    # reserves those bytes only from the Concat2 on, so nothing else may read or write them between that launch
    # and the Concat2; the input itself must have no other reader; a "Placed" Concat2 has both inputs in place,
    # a "CopyInto" one exactly one.
    # (tensors between the members of a fused launch stay on chip: their planned bytes are neither written nor read)
    on_chip = {steps[m]["out"]["name"] for l in launches if l["kind"] not in ("Step", "View", "Placed", "CopyInto")
               for m in l["members"] if m not in l["written"]}
    in_place = {}
    filled = set()
    for l in launches:
        if "writes_into" not in l:
            continue
        into = l["writes_into"]
        (t,) = [i for i, s in enumerate(steps) if s["out"]["name"] == into["name"]]
        c, end = t, t
        if steps[t]["kernel"] != "Concat2Kernel":
            # a Reshape that keeps the bytes in order behind a Concat2 nobody else reads: the Concat2's output is
            # written into the Reshape's buffer (reserved from the Reshape on) and the Reshape does not run
            assert steps[t]["kernel"] in ("ReshapeKernel", "FlattenKernel") and issued[t][1]["kind"] == "Placed"
            source = steps[t]["inputs"][0]
            (c,) = [i for i, s in enumerate(steps) if s["out"]["name"] == source["name"]]
            assert steps[c]["kernel"] == "Concat2Kernel" and readers[source["name"]] == {t} and c < t
            assert source["bytes"] == steps[t]["out"]["bytes"]
            assert source["layout"] == sorted(source["layout"]) and steps[t]["out"]["layout"] == sorted(steps[t]["out"]["layout"])
            filled.add(t)
        in_place[c] = in_place.get(c, 0) + (0 if l["kind"] == "Step" and l["members"] == [c] else 1)
        if l["kind"] == "CopyInto":
            assert l["members"] == [c]
        if l["members"] == [c]:
            # the Concat2 itself (whole, or the copy of one input): only a redirected one has a window to check
            pos = c
        else:
            final = l["members"][-1]
            assert readers[steps[final]["out"]["name"]] == {c}, "an input written in place has another reader"
            pos = l["position"]
            assert pos < c
        for q, s in enumerate(steps):
            if q == c or q == end or q in elided or q in l["members"]:
                continue
            if pos <= q <= end or pos <= issued[q][0] <= end:
                for op in s["inputs"] + [s["out"]]:
                    if steps[c]["out"]["name"] == issued[q][1].get("writes_into", {}).get("name") and op is s["out"]:
                        continue  # the producer of the other input, writing its own part
                    if op["name"] in on_chip:
                        continue
                    made_by = [i for i, t in enumerate(steps) if t["out"]["name"] == op["name"]]
                    if op is not s["out"] and made_by and made_by[0] in elided:
                        op = issued[made_by[0]][1]["source"]  # read through a view that is not run: its source's bytes
                    assert not _overlap(op, into), "bytes of a Concat2 output written early are in use"
    for l in launches:
        if l["kind"] == "Placed" and steps[l["members"][0]]["kernel"] == "PadKernel":
            assert l["members"][0] in padded_in_place and l["written"] == []
        elif l["kind"] == "Placed" and steps[l["members"][0]]["kernel"] != "Concat2Kernel":
            assert l["members"][0] in filled and l["written"] == []
        elif l["kind"] == "Placed":
            assert in_place.get(l["members"][0]) == 2 and l["written"] == []
        if l["kind"] == "CopyInto":
            assert in_place.get(l["members"][0]) == 2  # its own copy and the producer of the other input
    never_materialised = {steps[m]["out"]["name"] for l in launches if l["kind"] not in ("Step", "View", "Placed", "CopyInto")
                          for m in l["members"] if m not in l["written"]}
    for l in launches:
        members = l["members"]
        assert members == sorted(members)
        if l["kind"] in ("Step", "View", "Placed", "CopyInto"):
            assert len(members) == 1
            continue
        written = set(l["written"])
        position = l["position"]  # the step index where the launch is issued
        assert position in members
        if l["kind"] != "MatMulGroup":
            assert position == members[-1] and members[-1] in written
            # a convolution that also delivers the ReduceMean of its result writes that result as well
            also = written - {members[-1]}
            if l["kind"] == "RotaryPair":  # two rotary blocks in one launch: both results are written
                assert len(also) == 1 and also < set(members)
            else:
                assert not also or (also == {members[-2]} and steps[members[-1]]["kernel"] == "ReduceMeanKernel")
        inside = {steps[m]["out"]["name"] for m in members if m not in written}
        producer = {s["out"]["name"]: i for i, s in enumerate(steps)}
        for m in members:
            out = steps[m]["out"]
            if m in written:
                # written at `position`: no reader may come earlier ...
                assert all(r in members or r > position for r in readers.get(out["name"], ())), "read before written"
                # ... and if that is earlier than planned, nothing in between may touch the bytes
                for s in range(position, m):
                    if s not in members:
                        for op in steps[s]["inputs"] + ([] if s in elided else [steps[s]["out"]]):
                            if op["name"] in never_materialised:
                                continue  # an intermediate inside a fused launch: neither written nor read
                            if op["name"] in producer and producer[op["name"]] in elided:
                                op = issued[producer[op["name"]]][1]["source"]  # a view that is not run: its source's bytes
                            assert not _overlap(op, out), "a hoisted output lands on bytes still in use"
            else:
                assert out["space"] in ("arena", "private")
                assert readers[out["name"]] <= set(members), "an elided tensor is read outside its chain"
        # the bytes the launch writes: the planned outputs, or the part of another tensor it was pointed at
        finals = [l["writes_into"] if "writes_into" in l and m == members[-1] else steps[m]["out"] for m in written]
        own = {steps[m]["out"]["name"] for m in written}
        for m in members:
            for op in steps[m]["inputs"]:
                if op["name"] in inside or (op["name"] in own and m in written and len(written) > 1):
                    continue  # (the second result of a launch is computed from its first inside the kernel)
                if op["name"] in producer and producer[op["name"]] in elided:
                    op = issued[producer[op["name"]]][1]["source"]  # read through a view: the bytes of its source
                # every tensor that is materialised is written where its launch is issued
                for s in range(len(steps)):
                    if s in members or steps[s]["out"]["name"] in never_materialised or s in elided:
                        continue
                    if m < issued[s][0] < position:
                        assert not _overlap(steps[s]["out"], op), "a read was moved across a write to its bytes"
                if m > position and op["name"] in producer:
                    assert producer[op["name"]] < position, "a hoisted read precedes its producer"
                for final in finals:
                    if _overlap(final, op):  # only row-wise / elementwise kernels may work in place, and only exactly
                        assert l["kind"] in ("DivAddSoftmax", "ElementwiseChain")
                        assert final["offset"] == op["offset"] and final["layout"] == op["layout"]
    # switched off: one launch per step
    monkeypatch.setenv("FLUIDML_FUSE", "0")
    ex = getattr(fluidml.Executor, flavour)("sched_off")
    ex.compile(path)
    plan = ex.plan()
    assert [l["members"] for l in plan["launches"]] == [[i] for i in range(len(plan["steps"]))]
    # literal-reference mode never fuses
    monkeypatch.setenv("FLUIDML_FUSE", "1")
    monkeypatch.setenv("FLUIDML_REF_QUIRKS", "4")
    ex = getattr(fluidml.Executor, flavour)("sched_ref")
    ex.compile(path)
    assert len(ex.plan()["launches"]) == len(ex.plan()["steps"])


BRANCH_NETS = {
    "gpt_neox": (lambda m: m.gpt_neox(seq=24, layers=2, hidden=64, heads=2, ffn=128, vocab=120), 0.0, 2),
    "convbert": (lambda m: m.convbert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32), 0.0, 2),
    "bert": (lambda m: m.bert_base(seq=16, layers=2, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32, seed=5), 0.0, 0),
    "convbert_wide": (lambda m: m.convbert_base(seq=40, layers=3, hidden=96, heads=6, ffn=192, vocab=64, max_pos=64), 0.0, 2),
    "gpt_neox_deep": (lambda m: m.gpt_neox(seq=48, layers=3, hidden=128, heads=4, ffn=256, vocab=90), 0.0, 2),
    # full size with the default threshold: the attention block of a layer beside its MLP
    "gpt_neox_full": (lambda m: m.gpt_neox(), None, 3),
    "convbert_full_forced": (lambda m: m.convbert_base(), 0.0, 6),
}


@pytest.mark.parametrize("which", list(BRANCH_NETS))
def test_side_branches_are_independent(mods, which, tmp_path):
    """Two runs of launches issued side by side on two streams: the second (B) must read nothing the first (A)
    writes, and since the memory plan was made for the serial order, everything B writes has to live outside the
    arena, in buffers nobody else writes and nobody reads before B."""
    fluidml, models, _ = mods
    make, min_us, at_least = BRANCH_NETS[which]
    path = make(models).save(str(tmp_path / "net.onnx"))
    ex = fluidml.Executor.make_plain_greedy("branches")
    if min_us is not None:
        ex.context().set_branch_min_us(min_us)
    ex.compile(path)
    plan = ex.plan()
    launches, regions = plan["launches"], plan["regions"]
    assert len(regions) >= at_least
    runs = lambda l: l["kind"] not in ("View", "Placed")

    def touches(x, y):  # bytes of the arena, or of one buffer outside it
        if x["space"] != y["space"]:
            return False
        if x["space"] in ("interface", "constant"):
            return x["name"] == y["name"]
        if x["space"] == "private" and (x["pool"] or x["name"]) != (y["pool"] or y["name"]):
            return False
        return x["offset"] < y["offset"] + y["bytes"] and y["offset"] < x["offset"] + x["bytes"]

    last = 0
    for a, b, e in regions:
        assert last <= a < b < e <= len(launches)
        last = e
        assert runs(launches[a]) and runs(launches[b]) and runs(launches[e - 1])
        first, second = [l for l in launches[a:b] if runs(l)], [l for l in launches[b:e] if runs(l)]
        own = []
        for y in second:
            for w in y["writes"]:
                assert w["space"] in ("private", "interface"), "a side branch writes into the arena"
                own.append(w)
            for r in y["reads"]:
                for x in first:
                    assert not any(touches(w, r) for w in x["writes"]), "a side branch reads what the other run writes"
        # The side branch's bytes (buffers the regions share, one after the other): it starts right behind the fork
        # in front of the first run, so whoever else touches them has to come before that fork or behind the join.
        for k, l in enumerate(launches):
            if not runs(l) or b <= k < e:
                continue
            for op in l["reads"] + l["writes"]:
                if any(touches(op, w) for w in own):
                    assert k < a or k >= e, "the first run touches what the side branch writes"
        # ... and a tensor of this branch is read for the last time before the fork of whichever later branch moves
        # into its bytes
        names = {w["name"] for w in own if w["space"] == "private"}
        for k in range(b, len(launches)):
            if not runs(launches[k]):
                continue
            for r in launches[k]["reads"]:
                if r["space"] == "private" and r["name"] in names:
                    for a2, b2, e2 in regions:
                        if a2 >= e and a2 <= k:
                            assert not any(touches(r, w2) for l2 in launches[b2:e2] if runs(l2) for w2 in l2["writes"]), \
                                "a side branch overwrites bytes an earlier one's reader still needs"
    # without regions nothing is moved out of the arena
    ex = fluidml.Executor.make_plain_greedy("no_branches")
    ex.context().set_branch_min_us(1e9)
    ex.compile(path)
    assert ex.plan()["regions"] == []


# ------------------------------------------------------------------ layout DP

def test_dp_constant_cost_closed_form(mods, tiny):
    """With every kernel cost equal, every tensor gets GenAllOrders(rank)[0], the reversed permutation
    (ties keep the first enumerated layout, reference dp.cpp:705-709, 787, 820)."""
    fluidml, _, _ = mods
    net, path = tiny
    flow, seq, _, report = staged(fluidml, path, "make_dp_greedy_planner")
    layouts = fluidml._dp_layouts(flow, "constant")
    shapes = {v.name: v.shape for n in net.nodes for v in n.outputs + n.inputs}
    assert len(layouts) >= len(net.nodes)
    for name, layout in layouts.items():
        assert layout == list(range(len(shapes[name])))[::-1], name
    doc = json.loads(report)
    assert set(doc) == {"dp_table", "plan"} and "evaluator" in doc["dp_table"]
    assert doc["plan"] == {k: v for k, v in layouts.items()}
    row = doc["dp_table"]["evaluator"]["SoftmaxKernel"][0]
    assert set(row) == {"input_shape", "output_shape", "input_layout", "output_layout", "time_cost"}


def test_dp_json_serves_the_reference_analyzer(mods, tiny):
    """The JSON a DP compile emits is what the reference's tools/analyzer.py reads (its `onnx` import is absent
    here, so its lookups are replayed on the generated graph): for every graph node, the row of the node's kernel
    with the operands' shapes and the DEFAULT layouts, and the row with the layouts of data["plan"], both found
    by the equality tests of find_single_input / find_double_inputs (reference tools/analyzer.py:19-93), operand
    names chosen per operator as in its main loop (:150-700): single-input kernels by their one runtime tensor,
    Add/Mul with a rank-0 initializer as the *Constant kernels, MatMul/Add with a weight by (lhs, rhs, output)
    with the weight's layout taken from data["plan"] too."""
    fluidml, _, _ = mods
    net, path = tiny
    _, _, _, report = staged(fluidml, path, "make_dp_greedy_planner")
    data = json.loads(report)
    dp_table, plan = data["dp_table"]["evaluator"], data["plan"]
    infos = {v.name: list(v.shape) for n in net.nodes for v in n.outputs + n.inputs}
    consts = {v.name for v in net.initializers}

    def single(kernel, x, out):
        rows = dp_table[kernel]
        for layouts in ([list(range(len(infos[x]))), list(range(len(infos[out])))], [plan[x], plan[out]]):
            hit = [r for r in rows if r["input_shape"] == infos[x] and r["output_shape"] == infos[out] and
                   r["input_layout"] == layouts[0] and r["output_layout"] == layouts[1]]
            assert hit and isinstance(hit[0]["time_cost"], int), (kernel, x, out, layouts)

    def double(kernel, lhs, rhs, out):
        rows = dp_table[kernel]
        for layouts in ([list(range(len(infos[t]))) for t in (lhs, rhs, out)], [plan[lhs], plan[rhs], plan[out]]):
            hit = [r for r in rows if r["lhs_shape"] == infos[lhs] and r["rhs_shape"] == infos[rhs] and
                   r["output_shape"] == infos[out] and r["lhs_layout"] == layouts[0] and r["rhs_layout"] == layouts[1] and
                   r["output_layout"] == layouts[2]]
            assert hit and isinstance(hit[0]["time_cost"], int), (kernel, lhs, rhs, out, layouts)

    seen = set()
    for n in net.nodes:
        ins, out, op = [v.name for v in n.inputs], n.outputs[0].name, n.op_type
        runtime = [i for i in ins if i not in consts]
        scalars = [i for i in ins if i in consts and infos[i] == []]
        seen.add(op)
        if op in ("Add", "Mul"):
            if scalars:
                single(op + "ConstantKernel", runtime[0], out)
            else:
                double(op + "CommonKernel", ins[0], ins[1], out)
        elif op == "Sub":
            single("SubConstantLhsKernel", ins[1], out)
        elif op == "Div":
            single("DivConstantRhsKernel", ins[0], out)
        elif op == "Gather":
            single("GatherConstantDataTensorKernel", ins[1], out)
        elif op == "MatMul":
            double("MatMulKernel", ins[0], ins[1], out)
        elif op == "LayerNormalization":
            single("LayerNormalizationConstantScaleBiasKernel", ins[0], out)
        else:
            assert op in ("Erf", "Softmax", "Reshape", "Transpose", "Unsqueeze"), op
            single(op + "Kernel", ins[0], out)
    assert {"Add", "Mul", "Sub", "Div", "Gather", "MatMul", "LayerNormalization", "Erf", "Softmax", "Reshape", "Transpose",
            "Unsqueeze"} <= seen


def synthetic_cost(kernel, layouts):
    return 1 + zlib.crc32(repr((kernel, layouts)).encode()) % 1000


def test_dp_is_optimal_on_a_chain(mods, tmp_path):
    """Brute force over every layout assignment of a 3-kernel chain with a synthetic cost table."""
    fluidml, models, _ = mods
    g = models.Net("chain", 0)
    x = g.input("x", np.float32, (2, 3, 4))
    t1 = g.unary("Relu", x)
    t2 = g.transpose(t1, (2, 0, 1))
    y = g.unary("Erf", t2)
    g.output(y)
    path = g.save(str(tmp_path / "chain.onnx"))
    flow, _, _, _ = staged(fluidml, path)
    perms = fluidml._gen_all_orders(3)
    kernels = [("ReluKernel", (2, 3, 4), (2, 3, 4)), ("TransposeKernel", (2, 3, 4), (4, 2, 3)), ("ErfKernel", (4, 2, 3), (4, 2, 3))]
    table = {}
    for name, ishape, oshape in kernels:
        table[name] = [{"input_shape": list(ishape), "output_shape": list(oshape), "input_layout": a, "output_layout": b,
                        "time_cost": synthetic_cost(name, (a, b))} for a in perms for b in perms]
    layouts = fluidml._dp_layouts(flow, json.dumps({"evaluator": table}))
    tensors = [x.name, t1.name, t2.name, y.name]
    assert sorted(layouts) == sorted(tensors)
    assert layouts[y.name] == perms[0]  # the result keeps the first enumerated layout

    def total(assign):
        return sum(synthetic_cost(k[0], (assign[i], assign[i + 1])) for i, k in enumerate(kernels))

    best = min(total([a, b, c, perms[0]]) for a in perms for b in perms for c in perms)
    assert total([layouts[t] for t in tensors]) == best


def test_dp_on_a_branching_flow_covers_every_tensor(mods, tmp_path):
    """Residual pattern (a value with two consumers): main chain + branch, merged first-writer-wins."""
    fluidml, models, _ = mods
    g = models.Net("residual", 0)
    x = g.input("x", np.float32, (2, 3, 4))
    a = g.unary("Relu", x)
    b = g.unary("Erf", a)
    c = g.unary("Tanh", b)
    d = g.add(c, a)  # `a` feeds both Erf and Add
    g.output(g.unary("Neg", d))
    path = g.save(str(tmp_path / "residual.onnx"))
    flow, _, _, _ = staged(fluidml, path)
    layouts = fluidml._dp_layouts(flow, "constant")
    produced = {n.outputs[0].name for n in g.nodes} | {x.name}
    assert produced <= set(layouts)
    assert all(sorted(l) == [0, 1, 2] for l in layouts.values())
    # determinism: same flow, same answer
    assert fluidml._dp_layouts(flow, "constant") == layouts


# ------------------------------------------------------------------ command-line compiler

def test_compiler_cli(mods, tmp_path, capsys, monkeypatch):
    """Same options as the reference's executable (reference bin/compiler.cpp:13-69); --mode selects the executor
    (the reference parses it and then ignores it), the three sinks are written, a bad mode is refused."""
    import json

    from fluidml_amd import compiler

    _, models, _ = mods
    path = models.bert_base(seq=16, layers=1, hidden=64, heads=4, ffn=128, vocab=100, max_pos=32, seed=5).save(
        str(tmp_path / "net.onnx"))
    monkeypatch.setenv("FLUIDML_DP_COST", "constant")
    plans = {}
    for mode in compiler.ALLOWED_MODES:
        sinks = {k: tmp_path / f"{mode}.{k}" for k in ("mlir", "llvm", "json")}
        rc = compiler.main(["--name", "cli_" + mode, "--input", path, "--mode", mode, "--mlir", str(sinks["mlir"]),
                            "--llvm", str(sinks["llvm"]), "--json", str(sinks["json"])])
        assert rc == 0
        plans[mode] = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
        assert plans[mode]["mode"] == mode and plans[mode]["steps"] > 0
        assert sinks["mlir"].read_text() == sinks["llvm"].read_text() != ""
        assert "cli_" + mode in sinks["mlir"].read_text()
        kinds = [a["kind"] for a in plans[mode]["arguments"]]
        assert kinds.count("output") == 1 and kinds.count("input") == len(kinds) - 1 >= 2
    # the linear plan never reuses bytes, the greedy one does: the mode reached the executor
    assert plans["plain_linear"]["arena_bytes"] > plans["plain_greedy"]["arena_bytes"]
    assert (tmp_path / "dp_greedy.json").stat().st_size > (tmp_path / "plain_greedy.json").stat().st_size
    with pytest.raises(SystemExit):
        compiler.main(["-n", "x", "-i", path, "-m", "fastest"])
    with pytest.raises(SystemExit):
        compiler.main(["-i", path])  # --name is required, as in the reference


def test_launch_with_a_residual_is_not_placed_into_a_concat(mods, tmp_path):
    """A MatMul or Conv launch that adds a residual (or scales by a gate) keeps its own output tensor when that tensor
    is an input of a Concat2: the kernels read the addend through the output's strides, and a part of the wider
    Concat2 output has other strides (such a launch used to be redirected and was then refused at its first Invoke)."""
    fluidml, models, _ = mods
    for net, _ in models.residual_concat_nets():
        path = net.save(str(tmp_path / (net.name + ".onnx")))
        ex = fluidml.Executor.make_plain_greedy("rc")
        ex.compile(path)
        launches = ex.plan()["launches"]
        carriers = [l for l in launches if l["kind"] in ("MatMulChain", "ConvChain") and len(l["reads"]) >= 3]
        assert carriers, [l["kind"] for l in launches]
        for l in carriers:
            assert "writes_into" not in l, l
        # the Concat2 still runs (at most its other input was written in place)
        assert any(l["kind"] in ("Step", "CopyInto") and len(l["members"]) == 1 for l in launches)


@pytest.mark.parametrize("which", ["bert_base_full", "bert"])
def test_layer_norms_are_deferred_into_contractions(mods, which, tmp_path, monkeypatch):
    """Add + LayerNormalization behind a contraction: the contraction takes the Add and writes the un-normalised sum
    plus partial row statistics; every reader of the normalised tensor normalises on the fly (left operand: folded
    into the epilogue; residual: on the way into the next Add).  The plan has to be consistent -- a tensor is kept
    un-normalised exactly when all of its readers know -- and BERT-base comes out at 66 launches or fewer."""
    fluidml, models, _ = mods
    path = SCHEDULE_NETS[which][0](models).save(str(tmp_path / "net.onnx"))

    def plan_of(defer):
        monkeypatch.setenv("FLUIDML_DEFER_NORM", defer)
        ex = fluidml.Executor.make_plain_greedy("defer" + defer)
        ex.compile(path)
        return ex.plan()

    off, on = plan_of("0"), plan_of("1")
    assert all(l["norm_mode"] == 0 and not l["norm_emits"] for l in off["launches"])
    steps, launches = on["steps"], on["launches"]
    assert len(launches) < len(off["launches"])
    if which == "bert_base_full":
        assert len([l for l in launches if l["kind"] not in ("View", "Placed")]) <= 66
    producer = {}
    for l in launches:
        for m in l["written"]:
            producer[steps[m]["out"]["name"]] = l
    emitted = {steps[l["members"][-1]]["out"]["name"] for l in launches if l["norm_emits"]}
    assert emitted, "no LayerNormalization was deferred"
    for name in emitted:
        (ln,) = [i for i, s in enumerate(steps) if s["out"]["name"] == name]
        assert steps[ln]["kernel"] == "LayerNormalizationConstantScaleBiasKernel"
        assert producer[name]["kind"] in ("MatMulChain", "GemmChain") and producer[name]["members"][-1] == ln
    # every reader of a tensor kept un-normalised normalises it, and nobody normalises anything else
    for l in launches:
        if l["kind"] in ("View", "Placed"):
            continue
        read = {op["name"] for m in l["members"] for op in steps[m]["inputs"]} - {steps[m]["out"]["name"] for m in l["members"]}
        deferred_inputs = read & emitted
        assert bool(deferred_inputs) == (l["norm_mode"] != 0), (l["kind"], l["members"], deferred_inputs)
        assert len(deferred_inputs) <= 1
        if l["norm_mode"] == 1:  # as the left operand of its contraction(s)
            assert l["kind"] in ("MatMulChain", "MatMulGroup")
        if l["norm_mode"] == 2:  # as the residual of an Add the launch absorbed
            assert l["kind"] == "MatMulChain"
    # the statistics and the tensors moved out of the arena are accounted for as private bytes
    assert on["private_bytes"] > off["private_bytes"]


def test_lone_layer_norms_are_deferred_into_their_readers(mods, tmp_path, monkeypatch):
    """Pre-norm blocks (GPT-NeoX): a LayerNormalization on its own whose input a contraction launch -- or, in the first
    layer, the embedding lookup -- produced becomes a view of that input; the producer also writes the row statistics
    and every reader -- the contractions behind the LayerNormalization -- normalises its left operand on the fly.
    Both LayerNormalizations of a layer (parallel residual: attention and MLP read the same tensor) go this way."""
    fluidml, models, _ = mods
    path = SCHEDULE_NETS["gpt_neox"][0](models).save(str(tmp_path / "net.onnx"))

    def plan_of(defer):
        monkeypatch.setenv("FLUIDML_DEFER_NORM", defer)
        ex = fluidml.Executor.make_plain_greedy("lone" + defer)
        ex.compile(path)
        return ex.plan()

    off, on = plan_of("0"), plan_of("1")
    steps, launches = on["steps"], on["launches"]
    running = lambda plan: [l for l in plan["launches"] if l["kind"] not in ("View", "Placed")]
    assert len(running(on)) <= len(running(off)) - 4
    lone = [l for l in launches if l["kind"] == "View" and steps[l["members"][0]]["kernel"] == "LayerNormalizationConstantScaleBiasKernel"]
    assert len(lone) == 4, [l["members"] for l in lone]
    producer = {steps[m]["out"]["name"]: l for l in launches for m in l["written"]}
    sources = set()
    for l in lone:
        (ln,) = l["members"]
        source = steps[ln]["inputs"][0]["name"]
        sources.add(source)
        assert producer[source]["kind"] in ("MatMulChain", "GatherStatistics") and producer[source]["norm_emits"]
        readers = [r for r in launches if r is not l and any(op["name"] == steps[ln]["out"]["name"] for m in r["members"] for op in steps[m]["inputs"])]
        assert readers
        for r in readers:
            assert r["kind"] in ("MatMulChain", "MatMulGroup") and r["norm_mode"] == 1, (r["kind"], r["members"])
    assert len(sources) == 2  # the two of a layer read the one un-normalised tensor
    assert sorted(producer[source]["kind"] for source in sources) == ["GatherStatistics", "MatMulChain"]
    # nobody else normalises anything
    normalising = [l for l in launches if l["norm_mode"]]
    outs = {steps[l["members"][0]]["out"]["name"] for l in lone}
    for l in normalising:
        assert outs & {op["name"] for m in l["members"] for op in steps[m]["inputs"]}, (l["kind"], l["members"])
