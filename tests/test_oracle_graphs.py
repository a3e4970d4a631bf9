"""Pins the whole-graph oracle (oracle/graph_runner.run_graph) and the graph generators of
fluidml_amd/models.py WITHOUT the product beside them.

For a small instance of each of the five architectures the graph generator's output, executed by the
oracle's loop nests, has to agree with an independent float64 torch-functional forward pass that is
written here from the architecture descriptions alone (BERT: post-LN, erf-GELU, additive mask;
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
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fluidml_amd import models
from fluidml_amd.onnx_writer import GraphBuilder
from oracle import graph_runner

# float64 forward against the oracle's fp32 loop nests on small nets: fp32 rounding only
RTOL, ATOL = 2e-4, 2e-5


class Params:
    """The float initializers of rank >= 1 in creation order, handed out one by one as float64 tensors."""

    def __init__(self, net, seed):
        rng = np.random.Generator(np.random.PCG64(seed))
        self.items = []
        for v in net.initializers:
            c = v.const
            if c.dtype != np.float32 or c.ndim == 0:
                continue
            if c.size > 1 and (not c.any() or (c == 1).all()):  # the generators' zero biases and unit scales
                c[...] = rng.standard_normal(c.shape).astype(np.float32) * np.float32(0.5) + (1 if c.flat[0] == 1 else 0)
            self.items.append(c)
        self.at = 0

    def take(self, *shape):
        c = self.items[self.at]
        self.at += 1
        assert tuple(c.shape) == tuple(shape), f"initializer {self.at - 1}: shape {c.shape}, architecture wants {shape}"
        return torch.from_numpy(c.astype(np.float64))

    def done(self):
        assert self.at == len(self.items), f"{len(self.items) - self.at} float initializers were never used"


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


def _gelu(x):
    return x * 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))


def _attention(q, k, v, heads, bias=None, causal=False):
    """q, k, v [1, S, heads*d] -> context [1, S, heads, d]"""
    S, d = q.shape[1], q.shape[2] // heads
    qh, kh, vh = (t.view(1, S, heads, d).permute(0, 2, 1, 3) for t in (q, k, v))
    s = qh @ kh.transpose(-1, -2) / math.sqrt(d)
    if bias is not None:
        s = s + bias
    if causal:
        s = torch.where(torch.tril(torch.ones(S, S, dtype=torch.bool)), s, torch.tensor(torch.finfo(torch.float32).min, dtype=s.dtype))
    return (torch.softmax(s, -1) @ vh).permute(0, 2, 1, 3)


def _embeddings(p, feeds, vocab, types, hidden, seq, eps):
    ids = torch.from_numpy(feeds["input_ids"])
    tok = torch.from_numpy(feeds["token_type_ids"])
    word, typ, pos = p.take(vocab, hidden), p.take(types, hidden), p.take(1, seq, hidden)
    x = word[ids] + typ[tok] + pos
    return F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)


def test_bert_generator_and_runner_against_torch():
    seq, layers, hidden, heads, ffn, vocab, eps = 16, 2, 32, 4, 64, 50, 1e-12
    net = models.bert_base(seq=seq, layers=layers, hidden=hidden, heads=heads, ffn=ffn, vocab=vocab, max_pos=32, seed=5)
    feeds = models.bert_inputs(seq, vocab, seed=6)
    feeds["attention_mask"][0, -3:] = 0  # the additive mask must matter
    feeds["token_type_ids"][0, seq // 2:] = 1
    p = Params(net, 7)
    x = _embeddings(p, feeds, vocab, 2, hidden, seq, eps)
    bias = (1.0 - torch.from_numpy(feeds["attention_mask"]).double())[:, None, None, :] * -10000.0
    for _ in range(layers):
        q = x @ p.take(hidden, hidden) + p.take(hidden)
        k = x @ p.take(hidden, hidden) + p.take(hidden)
        v = x @ p.take(hidden, hidden) + p.take(hidden)
        c = _attention(q, k, v, heads, bias).reshape(1, seq, hidden)
        o = c @ p.take(hidden, hidden) + p.take(hidden)
        x = F.layer_norm(o + x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(x @ p.take(hidden, ffn) + p.take(ffn))
        f = h @ p.take(ffn, hidden) + p.take(hidden)
        x = F.layer_norm(f + x, (hidden,), p.take(hidden), p.take(hidden), eps)
    p.done()
    _check(net, feeds, x)


def test_convbert_generator_and_runner_against_torch():
    seq, layers, hidden, heads, ffn, vocab, eps, ck = 16, 2, 32, 4, 64, 50, 1e-12, 9
    net = models.convbert_base(seq=seq, layers=layers, hidden=hidden, heads=heads, ffn=ffn, vocab=vocab, max_pos=32, seed=8)
    feeds = models.bert_inputs(seq, vocab, seed=9)
    feeds["attention_mask"][0, :2] = 0
    p = Params(net, 10)
    nh = heads // 2
    hd = hidden // heads
    inner = nh * hd
    x = _embeddings(p, feeds, vocab, 2, hidden, seq, eps)
    bias = (1.0 - torch.from_numpy(feeds["attention_mask"]).double())[:, None, None, :] * -10000.0
    for _ in range(layers):
        q = x @ p.take(hidden, inner) + p.take(inner)
        k = x @ p.take(hidden, inner) + p.take(inner)
        v = x @ p.take(hidden, inner) + p.take(inner)
        # separable convolution of the layer input over the sequence: depthwise k=9 (no bias), pointwise (+ bias)
        dw = F.conv1d(x.transpose(1, 2), p.take(hidden, 1, ck), None, padding=ck // 2, groups=hidden)
        key_conv = F.conv1d(dw, p.take(inner, hidden, 1), p.take(inner)).transpose(1, 2)
        conv_attn = key_conv * q
        kernel = conv_attn @ p.take(inner, nh * ck) + p.take(nh * ck)
        kernel = torch.softmax(kernel.reshape(seq * nh, ck, 1), dim=1)
        conv_out = x @ p.take(hidden, inner) + p.take(inner)
        windows = F.pad(conv_out, (0, 0, ck // 2, ck // 2)).unfold(1, ck, 1)        # [1, S, inner, k]
        conv_out = (windows.reshape(seq * nh, hd, ck) @ kernel).reshape(1, seq, nh, hd)
        c = torch.cat([_attention(q, k, v, nh, bias), conv_out], dim=2).reshape(1, seq, hidden)
        o = c @ p.take(hidden, hidden) + p.take(hidden)
        x = F.layer_norm(o + x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(x @ p.take(hidden, ffn) + p.take(ffn))
        f = h @ p.take(ffn, hidden) + p.take(hidden)
        x = F.layer_norm(f + x, (hidden,), p.take(hidden), p.take(hidden), eps)
    p.done()
    _check(net, feeds, x)


def test_gpt_neox_generator_and_runner_against_torch():
    seq, layers, hidden, heads, ffn, vocab, eps = 24, 2, 64, 2, 128, 70, 1e-5
    net = models.gpt_neox(seq=seq, layers=layers, hidden=hidden, heads=heads, ffn=ffn, vocab=vocab, seed=11)
    feeds = models.gpt_neox_inputs(seq, vocab, seed=12)
    p = Params(net, 13)
    hd = hidden // heads
    rot = hd // 4
    x = p.take(vocab, hidden)[torch.from_numpy(feeds["input_ids"])]
    # rotary tables, base 10000, over the first quarter of each head; the graph's constants must equal them
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    ang = torch.arange(seq, dtype=torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    cos, sin = p.take(1, 1, seq, rot), p.take(1, 1, seq, rot)
    assert torch.allclose(cos[0, 0], emb.cos(), atol=1e-6, rtol=0) and torch.allclose(sin[0, 0], emb.sin(), atol=1e-6, rtol=0)

    def rotary(t):  # [1, heads, S, hd]
        t_rot, t_pass = t[..., :rot], t[..., rot:]
        half = torch.cat([-t_rot[..., rot // 2:], t_rot[..., : rot // 2]], dim=-1)
        return torch.cat([t_rot * emb.cos() + half * emb.sin(), t_pass], dim=-1)

    for _ in range(layers):
        a_in = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
        qkv = (a_in @ p.take(hidden, 3 * hidden) + p.take(3 * hidden)).view(1, seq, heads, 3 * hd)
        q, k, v = (qkv[..., i * hd:(i + 1) * hd].permute(0, 2, 1, 3) for i in range(3))
        q, k = rotary(q), rotary(k)
        s = (q @ k.transpose(-1, -2)) * (1.0 / math.sqrt(hd))
        s = torch.where(torch.tril(torch.ones(seq, seq, dtype=torch.bool)), s, torch.tensor(float(np.finfo(np.float32).min), dtype=s.dtype))
        c = (torch.softmax(s, -1) @ v).permute(0, 2, 1, 3).reshape(1, seq, hidden)
        attn = c @ p.take(hidden, hidden) + p.take(hidden)
        m_in = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(m_in @ p.take(hidden, ffn) + p.take(ffn))
        mlp = h @ p.take(ffn, hidden) + p.take(hidden)
        x = mlp + attn + x
    x = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
    logits = x @ p.take(hidden, vocab)
    p.done()
    _check(net, feeds, logits)


def _swish(x):
    return x * torch.sigmoid(x)


def test_efficientnet_generator_and_runner_against_torch():
    image, classes, div = 32, 10, 4
    net = models.efficientnet_b0(image=image, classes=classes, width_div=div, seed=14)
    feeds = models.image_input((1, 3, image, image), seed=15)
    p = Params(net, 16)

    def ch(c):
        return max(4, c // div)

    def conv(x, cout, k, stride, groups=1):
        cin = x.shape[1]
        return F.conv2d(x, p.take(cout, cin // groups, k, k), p.take(cout), stride=stride, padding=(k - 1) // 2, groups=groups)

    x = _swish(conv(torch.from_numpy(feeds["input"]).double(), ch(32), 3, 2))
    stages = [(1, 3, 1, 16, 1), (6, 3, 2, 24, 2), (6, 5, 2, 40, 2), (6, 3, 2, 80, 3), (6, 5, 1, 112, 3), (6, 5, 2, 192, 4), (6, 3, 1, 320, 1)]
    for expand, k, stride, cout, repeats in stages:
        for r in range(repeats):
            inp, cin = x, x.shape[1]
            mid = cin * expand
            h = _swish(conv(x, mid, 1, 1)) if expand != 1 else x
            h = _swish(conv(h, mid, k, stride if r == 0 else 1, groups=mid))
            se = h.mean(dim=(2, 3), keepdim=True)
            se = _swish(conv(se, max(1, cin // 4), 1, 1))
            se = torch.sigmoid(conv(se, mid, 1, 1))
            h = conv(h * se, ch(cout), 1, 1)
            x = h + inp if h.shape == inp.shape and (r > 0 or stride == 1) else h
    x = _swish(conv(x, ch(1280), 1, 1)).mean(dim=(2, 3))
    logits = x @ p.take(classes, x.shape[1]).T + p.take(classes)
    p.done()
    _check(net, feeds, logits)


@pytest.mark.parametrize("batch", [1, 2])
def test_vgg16_generator_and_runner_against_torch(batch):
    image, classes, div = 32, 10, 8
    net = models.vgg16(batch=batch, image=image, classes=classes, width_div=div, seed=17)
    feeds = models.image_input((batch, 3, image, image), seed=18)
    p = Params(net, 19)
    x = torch.from_numpy(feeds["input"]).double()
    for item in [64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M"]:
        if item == "M":
            x = F.max_pool2d(x, 2, 2)
        else:
            cout = max(4, item // div)
            x = F.relu(F.conv2d(x, p.take(cout, x.shape[1], 3, 3), p.take(cout), padding=1))
    x = x.flatten(1)
    for i, n in enumerate([4096 // div, 4096 // div, classes]):
        x = x @ p.take(n, x.shape[1]).T + p.take(n)
        if i < 2:
            x = F.relu(x)
    p.done()
    _check(net, feeds, x)


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
