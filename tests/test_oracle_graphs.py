"""Pins the whole-graph oracle (oracle/graph_runner.run_graph) and the graph generators of
fluidml_amd/models.py WITHOUT the product beside them.

For a small instance of each of the five architectures the graph generator's output, executed by the
oracle's loop nests, has to agree with an independent float64 torch-functional forward pass that is
written in tests/torch_reference.py from the architecture descriptions alone (BERT: post-LN, erf-GELU, additive mask;
ConvBERT: mixed attention with span-based dynamic convolution, kernel 9; GPT-NeoX: rotary embedding on
a quarter of each head, causal mask, parallel residual; EfficientNet-B0: MBConv with squeeze-excite and
swish; VGG-16).  The forward passes take the weights from the graph's initializers in creation order,
asserting each one's shape; the generators' all-zero biases and all-one scales are first overwritten
with random values so that a bias or scale wired to the wrong place (or dropped) changes the result.

The second half checks the runner's operator-variant dispatch and attribute DEFAULTS against what the
reference's converter and flow nodes use (reference src/worker/converter.cpp:1394-1408 Gemm alpha = beta = 0;
include/structure/flow/node.h:672-673 LayerNormalization axis 1 / epsilon 1e-5, :924 Softmax axis -1,
:389/:517 Gather axis 0, :504 Flatten axis 1; converter.cpp:2413-2438 Transpose perm reversed;
converter.cpp:551-592 AveragePool strides 1), each on a graph that omits the attribute.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fluidml_amd import models
from fluidml_amd.onnx_writer import GraphBuilder
from oracle import graph_runner
from tests import torch_reference

# float64 forward against the oracle's fp32 loop nests on small nets: fp32 rounding only
RTOL, ATOL = 2e-4, 2e-5


def _check(net, feeds, want):
    got = graph_runner.run_graph(net, feeds)
    assert len(got) == 1
    (name, value), = got.items()
    want = want.numpy()
    assert value.shape == want.shape, (value.shape, want.shape)
    err = np.abs(value.astype(np.float64) - want)
    bound = ATOL + RTOL * np.abs(want)
    assert (err <= bound).all(), f"{net.name}: max err {err.max():.3e}, max |want| {np.abs(want).max():.3e}"
    assert np.abs(want).max() > 1e-2  # a forward pass that collapsed to zero would pin nothing


def test_bert_generator_and_runner_against_torch():
    dims = dict(seq=16, layers=2, hidden=32, heads=4, ffn=64, vocab=50)
    net = models.bert_base(max_pos=32, seed=5, **dims)
    feeds = models.bert_inputs(16, 50, seed=6)
    feeds["attention_mask"][0, -3:] = 0  # the additive mask must matter
    feeds["token_type_ids"][0, 8:] = 1
    _check(net, feeds, torch_reference.bert(net, feeds, randomize_seed=7, **dims))


def test_convbert_generator_and_runner_against_torch():
    dims = dict(seq=16, layers=2, hidden=32, heads=4, ffn=64, vocab=50)
    net = models.convbert_base(max_pos=32, seed=8, **dims)
    feeds = models.bert_inputs(16, 50, seed=9)
    feeds["attention_mask"][0, :2] = 0
    _check(net, feeds, torch_reference.convbert(net, feeds, randomize_seed=10, **dims))


def test_gpt_neox_generator_and_runner_against_torch():
    dims = dict(seq=24, layers=2, hidden=64, heads=2, ffn=128, vocab=70)
    net = models.gpt_neox(seed=11, **dims)
    feeds = models.gpt_neox_inputs(24, 70, seed=12)
    _check(net, feeds, torch_reference.gpt_neox(net, feeds, randomize_seed=13, **dims))


def test_efficientnet_generator_and_runner_against_torch():
    net = models.efficientnet_b0(image=32, classes=10, width_div=4, seed=14)
    feeds = models.image_input((1, 3, 32, 32), seed=15)
    _check(net, feeds, torch_reference.efficientnet_b0(net, feeds, classes=10, div=4, randomize_seed=16))


@pytest.mark.parametrize("batch", [1, 2])
def test_vgg16_generator_and_runner_against_torch(batch):
    net = models.vgg16(batch=batch, image=32, classes=10, width_div=8, seed=17)
    feeds = models.image_input((batch, 3, 32, 32), seed=18)
    _check(net, feeds, torch_reference.vgg16(net, feeds, classes=10, div=8, randomize_seed=19))


def test_vgg16_batch_rows_are_independent_images():
    """image b of a batch-B graph = the batch-1 graph on that image (same seed -> same weights): what lets the
    full-size batch-8 GPU test meet the oracle on single images."""
    image, div = 32, 8
    feeds = models.image_input((3, 3, image, image), seed=20)
    whole = graph_runner.run_graph(models.vgg16(batch=3, image=image, classes=10, width_div=div, seed=21), feeds)
    one_net = models.vgg16(batch=1, image=image, classes=10, width_div=div, seed=21)
    (out_b,), = [list(whole.values())]
    for b in (0, 2):
        (out_1,), = [list(graph_runner.run_graph(one_net, {"input": feeds["input"][b:b + 1]}).values())]
        np.testing.assert_array_equal(out_b[b:b + 1], out_1)


# ------------------------------------------------------------------ dispatch and attribute defaults

def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _single(op, ins, out_shape, out_dtype=np.float32, **attrs):
    """one-node graph; `ins` = list of ("in", array) graph inputs or ("const", array) initializers"""
    g = GraphBuilder("one")
    vals, feeds = [], {}
    for i, (kind, arr) in enumerate(ins):
        arr = np.asarray(arr)
        if kind == "in":
            vals.append(g.input(f"x{i}", arr.dtype, arr.shape))
            feeds[f"x{i}"] = arr
        else:
            vals.append(g.const(arr))
    g.output(g.node(op, vals, out_shape, out_dtype, **attrs))
    (out,) = graph_runner.run_graph(g, feeds).values()
    return out


def test_gemm_alpha_beta_default_to_zero():
    r = _rng(1)
    a, w, b = (r.standard_normal(s).astype(np.float32) for s in ((3, 5), (4, 5), (4,)))
    out = _single("Gemm", [("in", a), ("const", w), ("const", b)], (3, 4), transB=1)
    np.testing.assert_array_equal(out, np.zeros((3, 4), np.float32))
    out = _single("Gemm", [("in", a), ("const", w), ("const", b)], (3, 4), transB=1, alpha=1.0)
    np.testing.assert_allclose(out, a @ w.T, rtol=1e-5, atol=1e-6)
    out = _single("Gemm", [("in", a), ("const", w), ("const", b)], (3, 4), transB=1, alpha=2.0, beta=0.5)
    np.testing.assert_allclose(out, 2.0 * (a @ w.T) + 0.5 * b, rtol=1e-5, atol=1e-6)
    out = _single("Gemm", [("in", a), ("const", w.T.copy()), ("const", b)], (3, 4), alpha=1.0, beta=1.0)  # transB defaults to 0
    np.testing.assert_allclose(out, a @ w.T + b, rtol=1e-5, atol=1e-6)
    # the reference's own line applies the scalars the other way round (gemm.cpp:57-61): out = alpha * bias + beta * AB
    g = GraphBuilder("swapped")
    x = g.input("x", np.float32, a.shape)
    g.output(g.node("Gemm", [x, g.const(w), g.const(b)], (3, 4), transB=1, alpha=2.0, beta=0.5))
    (out,) = graph_runner.run_graph(g, {"x": a}, flags=graph_runner.FL_REF_GEMM_SWAPPED_SCALARS).values()
    np.testing.assert_allclose(out, 2.0 * b + 0.5 * (a @ w.T), rtol=1e-5, atol=1e-6)


def test_layer_norm_defaults_axis_one_epsilon_1e5():
    r = _rng(2)
    x = (r.standard_normal((2, 6, 3)) * 1e-2).astype(np.float32)  # small values: epsilon matters
    gamma, beta = r.standard_normal((6, 1)).astype(np.float32), r.standard_normal((6, 1)).astype(np.float32)
    out = _single("LayerNormalization", [("in", x), ("const", gamma), ("const", beta)], x.shape)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)  # one axis only, biased variance
    want = (x64 - mean) / np.sqrt(var + 1e-5) * gamma + beta
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
    # negative axis counts from the back (flow/node.cpp:931-933)
    g2, b2 = r.standard_normal((3,)).astype(np.float32), r.standard_normal((3,)).astype(np.float32)
    out = _single("LayerNormalization", [("in", x), ("const", g2), ("const", b2)], x.shape, axis=-1, epsilon=1e-12)
    mean = x64.mean(axis=2, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=2, keepdims=True)
    np.testing.assert_allclose(out, (x64 - mean) / np.sqrt(var + 1e-12) * g2 + b2, rtol=1e-4, atol=1e-5)


def test_softmax_transpose_flatten_gather_pool_defaults():
    r = _rng(3)
    x = r.standard_normal((2, 3, 4)).astype(np.float32)
    out = _single("Softmax", [("in", x)], x.shape)
    np.testing.assert_allclose(out, torch.softmax(torch.from_numpy(x).double(), -1).numpy(), rtol=1e-5, atol=1e-6)
    out = _single("Softmax", [("in", x)], x.shape, axis=1)
    np.testing.assert_allclose(out, torch.softmax(torch.from_numpy(x).double(), 1).numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(_single("Transpose", [("in", x)], (4, 3, 2)), x.transpose(2, 1, 0))
    np.testing.assert_array_equal(_single("Transpose", [("in", x)], (3, 2, 4), perm=[1, 0, 2]), x.transpose(1, 0, 2))
    np.testing.assert_array_equal(_single("Flatten", [("in", x)], (2, 12)), x.reshape(2, 12))
    # Gather: which of the three kernels runs depends on which operand is an initializer; axis defaults to 0
    table = r.standard_normal((7, 5)).astype(np.float32)
    ids = np.array([[1, 6, 0], [3, 3, 2]], np.int64)
    np.testing.assert_array_equal(_single("Gather", [("const", table), ("in", ids)], (2, 3, 5)), table[ids])
    np.testing.assert_array_equal(_single("Gather", [("in", x), ("const", np.array([1, 0, 1], np.int64))], (3, 3, 4)), x[[1, 0, 1]])
    np.testing.assert_array_equal(_single("Gather", [("in", x), ("const", np.array([2, 0], np.int64))], (2, 2, 4), axis=1), x[:, [2, 0]])
    np.testing.assert_array_equal(_single("Gather", [("in", x), ("const", np.array(1, np.int64))], (3, 4)), x[1])
    np.testing.assert_array_equal(_single("Gather", [("in", x), ("const", np.array(2, np.int64))], (2, 4), axis=1), x[:, 2])
    # AveragePool: strides default to 1; MaxPool takes them from the attribute
    img = r.standard_normal((1, 2, 5, 5)).astype(np.float32)
    t = torch.from_numpy(img).double()
    np.testing.assert_allclose(_single("AveragePool", [("in", img)], (1, 2, 4, 4), kernel_shape=[2, 2]), F.avg_pool2d(t, 2, 1).numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(_single("MaxPool", [("in", img)], (1, 2, 2, 2), kernel_shape=[2, 2], pads=[0] * 4, strides=[2, 2]),
                                  F.max_pool2d(t, 2, 2).numpy().astype(np.float32))


def test_scalar_and_tensor_operand_variants():
    r = _rng(4)
    x = r.standard_normal((2, 3, 4)).astype(np.float32)
    y = r.standard_normal((4,)).astype(np.float32)
    c = np.array(1.75, np.float32)
    np.testing.assert_array_equal(_single("Add", [("in", x), ("const", c)], x.shape), x + c)
    np.testing.assert_array_equal(_single("Add", [("const", c), ("in", x)], x.shape), x + c)
    np.testing.assert_array_equal(_single("Add", [("const", y), ("in", x)], x.shape), x + y)
    np.testing.assert_array_equal(_single("Mul", [("in", x), ("const", c)], x.shape), x * c)
    np.testing.assert_array_equal(_single("Sub", [("const", c), ("in", x)], x.shape), c - x)      # only scalar - x exists
    np.testing.assert_array_equal(_single("Div", [("in", x), ("const", c)], x.shape), x / c)      # true division
    np.testing.assert_array_equal(_single("Sub", [("in", x), ("in", x[:, :1] * 2)], x.shape), x - x[:, :1] * 2)
    np.testing.assert_array_equal(_single("Div", [("in", x), ("in", np.abs(x[..., :1]) + 1)], x.shape), x / (np.abs(x[..., :1]) + 1))
    with pytest.raises(AssertionError):
        _single("Sub", [("in", x), ("const", c)], x.shape)
    with pytest.raises(AssertionError):
        _single("Div", [("const", c), ("in", x)], x.shape)
    cond = r.integers(0, 2, size=(3, 4)).astype(np.bool_)
    np.testing.assert_array_equal(_single("Where", [("const", cond), ("in", x), ("const", np.array(-3.0, np.float32))], x.shape), np.where(cond, x, np.float32(-3)))
    other = r.standard_normal((3, 4)).astype(np.float32)
    np.testing.assert_array_equal(_single("Where", [("const", cond), ("in", x), ("const", other)], x.shape), np.where(cond, x, other))
    np.testing.assert_allclose(_single("Pow", [("in", np.abs(x) + 0.1), ("const", np.array(2.5, np.float32))], x.shape),
                               (np.abs(x).astype(np.float64) + 0.1) ** 2.5, rtol=1e-5)
    np.testing.assert_array_equal(_single("Clip", [("in", x), ("const", np.array(-0.5, np.float32)), ("const", np.array(0.25, np.float32))], x.shape),
                                  np.clip(x, -0.5, 0.25))
    np.testing.assert_array_equal(_single("Clip", [("in", x)], x.shape, min=-0.5, max=0.25), np.clip(x, -0.5, 0.25))


def test_conv_variants_against_torch():
    r = _rng(5)
    x = r.standard_normal((2, 4, 7, 6)).astype(np.float32)
    w = r.standard_normal((5, 4, 3, 3)).astype(np.float32)
    b = r.standard_normal((5,)).astype(np.float32)
    t = torch.from_numpy(x).double()
    want = F.conv2d(t, torch.from_numpy(w).double(), torch.from_numpy(b).double(), stride=(2, 1), padding=1).numpy()
    out = _single("Conv", [("in", x), ("const", w), ("const", b)], want.shape, dilations=[1, 1], group=1, kernel_shape=[3, 3],
                  pads=[1, 1, 1, 1], strides=[2, 1])
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
    wd = r.standard_normal((4, 1, 3, 3)).astype(np.float32)
    want = F.conv2d(t, torch.from_numpy(wd).double(), None, padding=0, groups=4, dilation=(2, 1)).numpy()
    out = _single("Conv", [("in", x), ("const", wd)], want.shape, dilations=[2, 1], group=4, kernel_shape=[3, 3], pads=[0] * 4, strides=[1, 1])
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
