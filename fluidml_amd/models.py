"""ONNX graphs of the benchmark configurations, generated offline with seeded weights.

Each builder emits the operator patterns FluidML's converter accepts (reference
src/worker/converter.cpp; e.g. Gemm with explicit alpha/beta, LayerNormalization with an
explicit axis, scalars as rank-0 initializers, Reshape with a constant shape tensor) in the
shape a HuggingFace/torchvision export simplified by onnxsim has.  Weights come from
numpy.random.Generator(PCG64(seed)).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import numpy as np

from .onnx_writer import GraphBuilder, Value


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


class Net(GraphBuilder):
    """GraphBuilder plus shape-inferring helpers for the operators used below."""

    def __init__(self, name: str, seed: int):
        super().__init__(name)
        self.rng = _rng(seed)

    # ---- weights
    def normal(self, shape, std=0.02, name=None) -> Value:
        w = self.rng.standard_normal(shape, dtype=np.float32)
        w *= np.float32(std)
        return self.const(w, name)

    def zeros(self, shape, name=None) -> Value:
        return self.const(np.zeros(shape, np.float32), name)

    def ones(self, shape, name=None) -> Value:
        return self.const(np.ones(shape, np.float32), name)

    # ---- operators
    def binary(self, op: str, a: Value, b: Value) -> Value:
        shape = np.broadcast_shapes(a.shape, b.shape)
        dtype = a.dtype if not (a.const is not None and a.const.ndim == 0) else b.dtype
        return self.node(op, [a, b], shape, dtype)

    def add(self, a, b):
        return self.binary("Add", a, b)

    def sub(self, a, b):
        return self.binary("Sub", a, b)

    def mul(self, a, b):
        return self.binary("Mul", a, b)

    def div(self, a, b):
        return self.binary("Div", a, b)

    def unary(self, op: str, x: Value, **attrs) -> Value:
        return self.node(op, [x], x.shape, x.dtype, **attrs)

    def matmul(self, a: Value, b: Value) -> Value:
        shape = np.matmul(np.empty(a.shape, np.int8), np.empty(b.shape, np.int8)).shape
        return self.node("MatMul", [a, b], shape)

    def linear(self, x: Value, w: Value, b: Optional[Value]) -> Value:
        y = self.matmul(x, w)
        return self.add(b, y) if b is not None else y  # HF exports put the bias first

    def gather(self, table: Value, ids: Value, axis: int = 0) -> Value:
        shape = table.shape[:axis] + ids.shape + table.shape[axis + 1:]
        return self.node("Gather", [table, ids], shape, table.dtype, axis=axis)

    def reshape(self, x: Value, shape: Sequence[int]) -> Value:
        return self.node("Reshape", [x, self.const(np.array(shape, np.int64))], shape)

    def transpose(self, x: Value, perm: Sequence[int]) -> Value:
        return self.node("Transpose", [x], [x.shape[p] for p in perm], perm=list(perm))

    def unsqueeze(self, x: Value, axes: Sequence[int]) -> Value:
        shape = list(x.shape)
        for ax in sorted(axes):
            shape.insert(ax, 1)
        return self.node("Unsqueeze", [x, self.const(np.array(axes, np.int64))], shape)

    def softmax(self, x: Value, axis: int = -1) -> Value:
        return self.unary("Softmax", x, axis=axis)

    def layer_norm(self, x: Value, gamma: Value, beta: Value, eps: float) -> Value:
        return self.node("LayerNormalization", [x, gamma, beta], x.shape, axis=-1, epsilon=float(eps))

    def erf_gelu(self, x: Value) -> Value:
        """x * 0.5 * (1 + erf(x / sqrt(2))) as Div, Erf, Add, Mul, Mul (the unfused chain)."""
        t = self.div(x, self.scalar(1.4142135381698608))
        t = self.unary("Erf", t)
        t = self.add(t, self.scalar(1.0))
        t = self.mul(x, t)
        return self.mul(t, self.scalar(0.5))

    def slice(self, x: Value, starts, ends, axes, steps=None) -> Value:
        steps = steps or [1] * len(axes)
        shape = list(x.shape)
        for s, e, a, st in zip(starts, ends, axes, steps):
            e = min(e, x.shape[a])
            shape[a] = (e - s + st - 1) // st
        ins = [x] + [self.const(np.array(v, np.int64)) for v in (starts, ends, axes, steps)]
        return self.node("Slice", ins, shape)

    def concat2(self, a: Value, b: Value, axis: int) -> Value:
        shape = list(a.shape)
        shape[axis] += b.shape[axis]
        return self.node("Concat", [a, b], shape, axis=axis)

    def he_normal(self, shape, fan_in: int, name=None) -> Value:
        return self.normal(shape, std=float(np.sqrt(2.0 / fan_in)), name=name)

    def neg(self, x: Value) -> Value:
        return self.unary("Neg", x)

    def relu(self, x: Value) -> Value:
        return self.unary("Relu", x)

    def sigmoid(self, x: Value) -> Value:
        """sigmoid(x) = 0.5 * (1 + tanh(x / 2)): FluidML has no Sigmoid node (reference converter.cpp has no case)."""
        t = self.unary("Tanh", self.div(x, self.scalar(2.0)))
        return self.mul(self.add(t, self.scalar(1.0)), self.scalar(0.5))

    def swish(self, x: Value) -> Value:
        return self.mul(x, self.sigmoid(x))

    def where_const(self, cond: np.ndarray, x: Value, y) -> Value:
        """Where with a constant boolean condition and a scalar or constant-tensor y."""
        yv = self.scalar(y) if np.ndim(y) == 0 else self.const(np.asarray(y, np.float32))
        return self.node("Where", [self.const(np.asarray(cond, np.bool_)), x, yv], x.shape, x.dtype)

    def pad(self, x: Value, before: Sequence[int], after: Sequence[int]) -> Value:
        shape = [d + b + a for d, b, a in zip(x.shape, before, after)]
        return self.node("Pad", [x, self.const(np.array(list(before) + list(after), np.int64))], shape)

    def gather_const_indices(self, x: Value, indices: np.ndarray, axis: int) -> Value:
        indices = np.asarray(indices, np.int64)
        shape = x.shape[:axis] + indices.shape + x.shape[axis + 1:]
        return self.node("Gather", [x, self.const(indices)], shape, x.dtype, axis=axis)

    def reduce_mean(self, x: Value, axes: Sequence[int]) -> Value:
        shape = [1 if i in axes else d for i, d in enumerate(x.shape)]
        return self.node("ReduceMean", [x], shape, axes=list(axes), keepdims=1)

    def max_pool(self, x: Value, kernel: Sequence[int], strides: Sequence[int]) -> Value:
        out = list(x.shape[:2]) + [(d - k) // s + 1 for d, k, s in zip(x.shape[2:], kernel, strides)]
        return self.node("MaxPool", [x], out, kernel_shape=list(kernel), pads=[0] * (2 * len(kernel)), strides=list(strides))

    def flatten(self, x: Value, axis: int = 1) -> Value:
        return self.node("Flatten", [x], [int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis:]))], axis=axis)

    def gemm(self, x: Value, w: Value, b: Value, trans_b: bool = True) -> Value:
        """Gemm with alpha = beta = 1 written out: FluidML defaults both to 0 (reference converter.cpp:1394-1403)."""
        n = w.shape[0] if trans_b else w.shape[1]
        return self.node("Gemm", [x, w, b], [x.shape[0], n], alpha=1.0, beta=1.0, transA=0, transB=int(trans_b))

    def conv(self, x: Value, w: Value, b: Optional[Value], strides, pads, dilations=None, group=1) -> Value:
        ns = len(x.shape) - 2
        dilations = dilations or [1] * ns
        out = [x.shape[0], w.shape[0]]
        for d in range(ns):
            out.append((x.shape[2 + d] + pads[d] + pads[d + ns] - dilations[d] * (w.shape[2 + d] - 1) - 1) // strides[d] + 1)
        ins = [x, w] + ([b] if b is not None else [])
        return self.node("Conv", ins, out, dilations=list(dilations), group=int(group), kernel_shape=list(w.shape[2:]),
                         pads=list(pads), strides=list(strides))


def bert_base(seq: int = 128, layers: int = 12, hidden: int = 768, heads: int = 12, ffn: int = 3072,
              vocab: int = 30522, max_pos: int = 512, types: int = 2, eps: float = 1e-12, seed: int = 1234) -> Net:
    """BERT-base encoder, batch 1: post-LN layers, erf-GELU, learned positions; output = last hidden state.

    Inputs: input_ids int64 [1,seq], attention_mask float32 [1,seq] (the reference's model takes it as
    float, reference test/python/model_test.py:30), token_type_ids int64 [1,seq].
    """
    g = Net("bert_base", seed)
    head_dim = hidden // heads
    ids = g.input("input_ids", np.int64, (1, seq))
    mask = g.input("attention_mask", np.float32, (1, seq))
    tok = g.input("token_type_ids", np.int64, (1, seq))

    word = g.gather(g.normal((vocab, hidden), name="embeddings.word_embeddings.weight"), ids)
    typ = g.gather(g.normal((types, hidden), name="embeddings.token_type_embeddings.weight"), tok)
    pos_table = g.rng.standard_normal((max_pos, hidden), dtype=np.float32) * np.float32(0.02)
    x = g.add(word, typ)
    x = g.add(x, g.const(pos_table[:seq][None], name="embeddings.position_embeddings.slice"))
    x = g.layer_norm(x, g.ones((hidden,)), g.zeros((hidden,)), eps)

    ext = g.unsqueeze(mask, [1, 2])
    ext = g.sub(g.scalar(1.0), ext)
    ext = g.mul(ext, g.scalar(-10000.0))

    for _ in range(layers):
        q = g.linear(x, g.normal((hidden, hidden)), g.zeros((hidden,)))
        k = g.linear(x, g.normal((hidden, hidden)), g.zeros((hidden,)))
        v = g.linear(x, g.normal((hidden, hidden)), g.zeros((hidden,)))
        q = g.transpose(g.reshape(q, (1, seq, heads, head_dim)), (0, 2, 1, 3))
        k = g.transpose(g.reshape(k, (1, seq, heads, head_dim)), (0, 2, 3, 1))
        v = g.transpose(g.reshape(v, (1, seq, heads, head_dim)), (0, 2, 1, 3))
        s = g.matmul(q, k)
        s = g.div(s, g.scalar(float(np.sqrt(head_dim))))
        s = g.add(s, ext)
        p = g.softmax(s, -1)
        c = g.matmul(p, v)
        c = g.reshape(g.transpose(c, (0, 2, 1, 3)), (1, seq, hidden))
        o = g.linear(c, g.normal((hidden, hidden)), g.zeros((hidden,)))
        x = g.layer_norm(g.add(o, x), g.ones((hidden,)), g.zeros((hidden,)), eps)
        h = g.linear(x, g.normal((hidden, ffn)), g.zeros((ffn,)))
        h = g.erf_gelu(h)
        f = g.linear(h, g.normal((ffn, hidden)), g.zeros((hidden,)))
        x = g.layer_norm(g.add(f, x), g.ones((hidden,)), g.zeros((hidden,)), eps)
    g.output(x)
    return g


def bert_inputs(seq: int = 128, vocab: int = 30522, seed: int = 99) -> Dict[str, np.ndarray]:
    r = _rng(seed)
    return {
        "input_ids": r.integers(0, vocab, size=(1, seq), dtype=np.int64),
        "attention_mask": np.ones((1, seq), np.float32),
        "token_type_ids": np.zeros((1, seq), np.int64),
    }


def convbert_base(seq: int = 128, layers: int = 12, hidden: int = 768, heads: int = 12, head_ratio: int = 2,
                  conv_kernel: int = 9, ffn: int = 3072, vocab: int = 30522, max_pos: int = 512, types: int = 2,
                  eps: float = 1e-12, seed: int = 2345) -> Net:
    """ConvBERT-base encoder, batch 1: mixed attention = self-attention on heads/head_ratio heads plus
    span-based dynamic convolution (depthwise k=9 separable conv on the keys, a per-position softmaxed
    kernel of 9 taps applied to a window of the value projection), concatenated; output last hidden state.

    The window extraction (torch unfold) is written as Pad + Gather with a constant [seq, k] index table,
    which is what an exporter produces and what FluidML's GatherConstantIndicesTensor accepts.
    """
    g = Net("convbert_base", seed)
    head_dim = hidden // heads
    nh = heads // head_ratio  # heads of each branch
    inner = nh * head_dim
    ids = g.input("input_ids", np.int64, (1, seq))
    mask = g.input("attention_mask", np.float32, (1, seq))
    tok = g.input("token_type_ids", np.int64, (1, seq))
    word = g.gather(g.normal((vocab, hidden)), ids)
    typ = g.gather(g.normal((types, hidden)), tok)
    pos_table = g.rng.standard_normal((max_pos, hidden), dtype=np.float32) * np.float32(0.02)
    x = g.add(g.add(word, typ), g.const(pos_table[:seq][None]))
    x = g.layer_norm(x, g.ones((hidden,)), g.zeros((hidden,)), eps)
    ext = g.mul(g.sub(g.scalar(1.0), g.unsqueeze(mask, [1, 2])), g.scalar(-10000.0))
    window = np.arange(seq)[:, None] + np.arange(conv_kernel)[None, :]  # rows of the padded sequence
    half = conv_kernel // 2

    for _ in range(layers):
        q = g.linear(x, g.normal((hidden, inner)), g.zeros((inner,)))
        k = g.linear(x, g.normal((hidden, inner)), g.zeros((inner,)))
        v = g.linear(x, g.normal((hidden, inner)), g.zeros((inner,)))
        # separable conv over the sequence: [1, S, H] -> [1, H, S], depthwise k=9 pad 4, pointwise H -> inner (+bias)
        xt = g.transpose(x, (0, 2, 1))
        dw = g.conv(xt, g.normal((hidden, 1, conv_kernel)), None, [1], [half, half], group=hidden)
        pw = g.conv(dw, g.normal((inner, hidden, 1)), g.zeros((inner,)), [1], [0, 0])
        key_conv = g.transpose(pw, (0, 2, 1))                       # [1, S, inner]
        conv_attn = g.mul(key_conv, q)
        ck = g.linear(conv_attn, g.normal((inner, nh * conv_kernel)), g.zeros((nh * conv_kernel,)))
        ck = g.softmax(g.reshape(ck, (seq * nh, conv_kernel, 1)), 1)  # softmax over the taps
        co = g.linear(x, g.normal((hidden, inner)), g.zeros((inner,)))
        co = g.pad(co, [0, half, 0], [0, half, 0])                  # [1, S + 8, inner]
        co = g.gather_const_indices(co, window, 1)                  # [1, S, k, inner]
        co = g.reshape(g.transpose(co, (0, 1, 3, 2)), (seq * nh, head_dim, conv_kernel))
        co = g.reshape(g.matmul(co, ck), (1, seq, nh, head_dim))    # [S*nh, d, 1] -> [1, S, nh, d]
        # self-attention on nh heads
        qh = g.transpose(g.reshape(q, (1, seq, nh, head_dim)), (0, 2, 1, 3))
        kh = g.transpose(g.reshape(k, (1, seq, nh, head_dim)), (0, 2, 3, 1))
        vh = g.transpose(g.reshape(v, (1, seq, nh, head_dim)), (0, 2, 1, 3))
        s = g.add(g.div(g.matmul(qh, kh), g.scalar(float(np.sqrt(head_dim)))), ext)
        c = g.transpose(g.matmul(g.softmax(s, -1), vh), (0, 2, 1, 3))  # [1, S, nh, d]
        c = g.reshape(g.concat2(c, co, 2), (1, seq, hidden))
        o = g.linear(c, g.normal((hidden, hidden)), g.zeros((hidden,)))
        x = g.layer_norm(g.add(o, x), g.ones((hidden,)), g.zeros((hidden,)), eps)
        h = g.erf_gelu(g.linear(x, g.normal((hidden, ffn)), g.zeros((ffn,))))
        f = g.linear(h, g.normal((ffn, hidden)), g.zeros((hidden,)))
        x = g.layer_norm(g.add(f, x), g.ones((hidden,)), g.zeros((hidden,)), eps)
    g.output(x)
    return g


def gpt_neox(seq: int = 256, layers: int = 6, hidden: int = 512, heads: int = 8, rotary_pct: float = 0.25,
             rotary_base: float = 10000.0, ffn: int = 2048, vocab: int = 50304, eps: float = 1e-5, seed: int = 3456) -> Net:
    """GPT-NeoX-style decoder, prefill of `seq` tokens, batch 1: fused QKV projection, rotary embedding on the
    first rotary_pct of each head, full causal mask through Where(constant condition), parallel residual
    x + attn(ln1(x)) + mlp(ln2(x)), final LayerNorm, untied LM head; output logits [1, seq, vocab]."""
    g = Net("gpt_neox", seed)
    hd = hidden // heads
    rot = int(hd * rotary_pct)
    ids = g.input("input_ids", np.int64, (1, seq))
    x = g.gather(g.normal((vocab, hidden)), ids)
    inv_freq = 1.0 / (rotary_base ** (np.arange(0, rot, 2, dtype=np.float64) / rot))
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv_freq[None, :]
    emb = np.concatenate([ang, ang], axis=-1)                       # [S, rot]
    cos = g.const(np.cos(emb).astype(np.float32)[None, None])
    sin = g.const(np.sin(emb).astype(np.float32)[None, None])
    causal = np.tril(np.ones((seq, seq), np.bool_))[None, None]
    min_value = float(np.finfo(np.float32).min)

    def rotary(t: Value) -> Value:
        t_rot = g.slice(t, [0], [rot], [3])
        t_pass = g.slice(t, [rot], [hd], [3])
        x1 = g.slice(t_rot, [0], [rot // 2], [3])
        x2 = g.slice(t_rot, [rot // 2], [rot], [3])
        rotated = g.concat2(g.neg(x2), x1, 3)
        t_emb = g.add(g.mul(t_rot, cos), g.mul(rotated, sin))
        return g.concat2(t_emb, t_pass, 3)

    for _ in range(layers):
        a_in = g.layer_norm(x, g.ones((hidden,)), g.zeros((hidden,)), eps)
        qkv = g.linear(a_in, g.normal((hidden, 3 * hidden)), g.zeros((3 * hidden,)))
        qkv = g.reshape(qkv, (1, seq, heads, 3 * hd))
        q = g.transpose(g.slice(qkv, [0], [hd], [3]), (0, 2, 1, 3))
        k = g.transpose(g.slice(qkv, [hd], [2 * hd], [3]), (0, 2, 1, 3))
        v = g.transpose(g.slice(qkv, [2 * hd], [3 * hd], [3]), (0, 2, 1, 3))
        q, k = rotary(q), rotary(k)
        s = g.matmul(q, g.transpose(k, (0, 1, 3, 2)))
        s = g.mul(s, g.scalar(float(1.0 / np.sqrt(hd))))
        s = g.where_const(causal, s, min_value)
        c = g.matmul(g.softmax(s, -1), v)
        c = g.reshape(g.transpose(c, (0, 2, 1, 3)), (1, seq, hidden))
        attn = g.linear(c, g.normal((hidden, hidden)), g.zeros((hidden,)))
        m_in = g.layer_norm(x, g.ones((hidden,)), g.zeros((hidden,)), eps)
        h = g.erf_gelu(g.linear(m_in, g.normal((hidden, ffn)), g.zeros((ffn,))))
        mlp = g.linear(h, g.normal((ffn, hidden)), g.zeros((hidden,)))
        x = g.add(g.add(mlp, attn), x)
    x = g.layer_norm(x, g.ones((hidden,)), g.zeros((hidden,)), eps)
    g.output(g.matmul(x, g.normal((hidden, vocab))))
    return g


def gpt_neox_inputs(seq: int = 256, vocab: int = 50304, seed: int = 98) -> Dict[str, np.ndarray]:
    return {"input_ids": _rng(seed).integers(0, vocab, size=(1, seq), dtype=np.int64)}


# (expand ratio, kernel, stride, out channels, repeats) of the seven MBConv stages of EfficientNet-B0
_B0_STAGES = [(1, 3, 1, 16, 1), (6, 3, 2, 24, 2), (6, 5, 2, 40, 2), (6, 3, 2, 80, 3), (6, 5, 1, 112, 3), (6, 5, 2, 192, 4),
              (6, 3, 1, 320, 1)]


def efficientnet_b0(image: int = 224, classes: int = 1000, width_div: int = 1, seed: int = 4567) -> Net:
    """EfficientNet-B0, batch 1, BatchNorm folded into each conv (weights + bias), swish through the tanh
    identity, squeeze-excite with ratio 0.25 of the block input; symmetric (k-1)/2 padding.
    `width_div` divides every channel count (tests use a narrow net on a small image)."""
    g = Net("efficientnet_b0", seed)

    def ch(c):
        return max(4, c // width_div)

    def conv_bn(x, cout, k, stride, group=1):
        cin = x.shape[1]
        w = g.he_normal((cout, cin // group, k, k), fan_in=(cin // group) * k * k)
        b = g.normal((cout,), std=0.05)
        p = (k - 1) // 2
        return g.conv(x, w, b, [stride, stride], [p, p, p, p], group=group)

    x = g.input("input", np.float32, (1, 3, image, image))
    x = g.swish(conv_bn(x, ch(32), 3, 2))
    for expand, k, stride, cout, repeats in _B0_STAGES:
        for r in range(repeats):
            cin = x.shape[1]
            inp = x
            mid = cin * expand
            h = g.swish(conv_bn(x, mid, 1, 1)) if expand != 1 else x
            h = g.swish(conv_bn(h, mid, k, stride if r == 0 else 1, group=mid))
            se = g.reduce_mean(h, [2, 3])
            se = g.swish(conv_bn(se, max(1, cin // 4), 1, 1))
            se = g.sigmoid(conv_bn(se, mid, 1, 1))
            h = g.mul(h, se)
            h = conv_bn(h, ch(cout), 1, 1)
            x = g.add(h, inp) if (r > 0 or stride == 1) and h.shape == inp.shape else h
    x = g.swish(conv_bn(x, ch(1280), 1, 1))
    x = g.flatten(g.reduce_mean(x, [2, 3]), 1)
    feat = x.shape[1]
    g.output(g.gemm(x, g.normal((classes, feat), std=float(np.sqrt(1.0 / feat))), g.zeros((classes,))))
    return g


_VGG16 = [64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M"]


def vgg16(batch: int = 1, image: int = 224, classes: int = 1000, width_div: int = 1, fc: int = 4096, seed: int = 5678) -> Net:
    """VGG-16: 13 conv3x3 pad 1 + ReLU, 5 maxpool 2x2 stride 2, Flatten, three Gemm (ReLU between)."""
    g = Net("vgg16", seed)
    x = g.input("input", np.float32, (batch, 3, image, image))
    for item in _VGG16:
        if item == "M":
            x = g.max_pool(x, [2, 2], [2, 2])
        else:
            cout, cin = max(4, item // width_div), x.shape[1]
            x = g.relu(g.conv(x, g.he_normal((cout, cin, 3, 3), fan_in=cin * 9), g.zeros((cout,)), [1, 1], [1, 1, 1, 1]))
    x = g.flatten(x, 1)
    for i, n in enumerate([fc // width_div, fc // width_div, classes]):
        feat = x.shape[1]
        x = g.gemm(x, g.he_normal((n, feat), fan_in=feat), g.zeros((n,)))
        if i < 2:
            x = g.relu(x)
    g.output(x)
    return g


def image_input(shape, seed: int = 97) -> Dict[str, np.ndarray]:
    return {"input": _rng(seed).standard_normal(shape, dtype=np.float32)}


def residual_concat_nets():
    """Two small graphs in which a contraction that carries a residual addend feeds one half of a Concat2:
    MatMul(relu(x), W) + relu(x) beside tanh(relu(x)) on the last axis, and a pointwise Conv with a skip connection
    beside a second Conv on the channel axis at batch 2.  The launch that adds the residual reads it through the
    strides of its own output tensor, so it must not be redirected into a part of the wider Concat2 output."""
    g = Net("matmul_residual_concat", 21)
    x = g.input("x", np.float32, (1, 16, 32))
    r = g.relu(x)
    y = g.add(g.matmul(r, g.normal((32, 32), 0.2)), r)
    g.output(g.concat2(y, g.unary("Tanh", r), 2))
    rng = _rng(22)
    first = (g, {"x": rng.standard_normal((1, 16, 32), dtype=np.float32)})

    h = Net("conv_skip_concat", 23)
    img = h.input("input", np.float32, (2, 8, 6, 6))
    s = h.relu(img)
    a = h.add(h.conv(s, h.he_normal((8, 8, 1, 1), fan_in=8), h.zeros((8,)), [1, 1], [0, 0, 0, 0]), s)
    b = h.relu(h.conv(s, h.he_normal((4, 8, 3, 3), fan_in=72), h.normal((4,), 0.1), [1, 1], [1, 1, 1, 1]))
    h.output(h.concat2(a, b, 1))
    second = (h, {"input": rng.standard_normal((2, 8, 6, 6), dtype=np.float32)})
    return [first, second]
