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
