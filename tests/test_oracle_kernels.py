"""Pins oracle/kernels.c before anything is checked against it.

The reference holds no golden vectors for its kernels: its per-operator tests
(test/python/node/node_test.py) compare against onnxruntime on unseeded random
inputs, and onnxruntime is not installed here.  So each oracle function is
pinned against the library routine its loop nest reduces to (numpy / torch on
CPU), on the reference's own node-test shapes, for every layout permutation
where that is cheap -- a wrong stride, a transposed operand, a dropped pass or
a wrong broadcast rule changes the result far beyond the bounds used here.
The literal-reference modes (FL_REF_*) are pinned by closed forms derived from
the cited reference lines.
"""
import zlib

import numpy as np
import pytest
import torch

from oracle import kernels as ok
from tests.util import all_layouts, some_layouts


def rng_for(*what):
    return np.random.default_rng(zlib.crc32(repr(what).encode()))


def rand(rng, shape, lo=-2.0, hi=2.0):
    return rng.uniform(lo, hi, size=shape).astype(np.float32)


def close(got, want, rtol=1e-5, atol=1e-6):
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)


def test_unary_closed_forms():
    rng = rng_for("unary")
    x = rand(rng, (3, 5, 7))
    pos = np.abs(x) + 0.1
    t = torch.from_numpy
    table = [
        (ok.OP_ADD_C, x, (1.5, 0), x + np.float32(1.5)),
        (ok.OP_RSUB_C, x, (1.0, 0), np.float32(1.0) - x),
        (ok.OP_MUL_C, x, (-10000.0, 0), x * np.float32(-10000.0)),
        (ok.OP_DIV_C, x, (8.0, 0), x / np.float32(8.0)),
        (ok.OP_POW_C, pos, (3.0, 0), pos**3),
        (ok.OP_ERF, x, (0, 0), torch.erf(t(x)).numpy()),
        (ok.OP_RELU, x, (0, 0), np.maximum(x, 0)),
        (ok.OP_CLIP, 4 * x, (0.0, 6.0), np.clip(4 * x, 0, 6)),
        (ok.OP_TANH, x, (0, 0), np.tanh(x)),
        (ok.OP_SQRT, pos, (0, 0), np.sqrt(pos)),
        (ok.OP_NEG, x, (0, 0), -x),
        (ok.OP_COPY, x, (0, 0), x),
    ]
    for op, inp, (c0, c1), want in table:
        for lin in all_layouts(3):
            for lout in ([0, 1, 2], [2, 1, 0], [1, 2, 0]):
                hx, ho = ok.View(inp, lin), ok.View.empty(inp.shape, np.float32, lout)
                ok.unary_f32(op, hx, ho, c0, c1)
                close(ho.logical(), want)


def test_relu_and_clip_propagate_nan():
    # arith.maximumf / minimumf propagate NaN (reference relu.cpp:12-46, clip.cpp:13-48)
    x = np.array([np.nan, -1.0, 2.0], dtype=np.float32)
    ho = ok.View.empty((3,))
    ok.unary_f32(ok.OP_RELU, ok.View(x), ho)
    assert np.isnan(ho.logical()[0]) and ho.logical()[1] == 0 and ho.logical()[2] == 2
    ok.unary_f32(ok.OP_CLIP, ok.View(x), ho, 0.0, 1.0)
    assert np.isnan(ho.logical()[0]) and ho.logical()[1] == 0 and ho.logical()[2] == 1


def test_integer_kernels():
    rng = rng_for("int")
    ids = rng.integers(-3, 5, size=(4, 6)).astype(np.int64)
    for lin in all_layouts(2):
        hx = ok.View(ids, lin)
        ho = ok.View.empty(ids.shape, np.int64)
        ok.unary_int(ok.IOP_ADD_C, hx, ho, 2)
        assert (ho.logical() == ids + 2).all()
        hb = ok.View.empty(ids.shape, np.bool_)
        ok.unary_int(ok.IOP_EQ_C, hx, hb, 1)
        assert (hb.logical() == (ids == 1)).all()
        hn = ok.View.empty(ids.shape, np.bool_)
        ok.unary_int(ok.IOP_NOT, hb, hn)
        assert (hn.logical() == ~(ids == 1)).all()
        hc = ok.View.empty(ids.shape, np.int32)
        ok.unary_int(ok.IOP_CAST, hx, hc)
        assert (hc.logical() == ids.astype(np.int32)).all()
        hz = ok.View.empty(ids.shape, np.int64)
        ok.unary_int(ok.IOP_CAST, hb, hz)  # true must become 1, not -1 (reference cast.cpp:33-40)
        assert (hz.logical() == (ids == 1).astype(np.int64)).all()
        for axis in (0, 1):
            hs = ok.View.empty(ids.shape, np.int64)
            ok.cum_sum(hx, hs, axis)
            assert (hs.logical() == np.cumsum(ids, axis=axis)).all()
    a = rng.integers(-9, 9, size=(2, 16)).astype(np.int64)
    b = rng.integers(-9, 9, size=(16,)).astype(np.int64)
    ho = ok.View.empty((2, 16), np.int64)
    ok.mul_int(ok.View(a), ok.View(b), ho)
    assert (ho.logical() == a * b).all()


@pytest.mark.parametrize("lshape,rshape", [((1, 128, 768), (1, 128, 768)), ((1, 128, 768), (768,)),
                                           ((1, 12, 16, 16), (1, 1, 1, 16)), ((2, 5, 7), (5, 1)), ((3, 1, 6), (3, 4, 6))])
def test_binary_broadcast(lshape, rshape):
    rng = rng_for(lshape, rshape)
    a, b = rand(rng, lshape), rand(rng, rshape, 0.5, 2)
    for op, fn in [(ok.BOP_ADD, np.add), (ok.BOP_SUB, np.subtract), (ok.BOP_MUL, np.multiply), (ok.BOP_DIV, np.divide)]:
        want = fn(a, b)
        for la in some_layouts(len(lshape), rng, 3):
            for lb in some_layouts(len(rshape), rng, 2):
                ho = ok.View.empty(want.shape, np.float32, some_layouts(want.ndim, rng, 2)[-1])
                ok.binary_f32(op, ok.View(a, la), ok.View(b, lb), ho)
                assert (ho.logical() == want).all()


def test_where_and_fused():
    rng = rng_for("where")
    cond = np.tril(np.ones((1, 1, 16, 16), dtype=np.bool_))
    x = rand(rng, (2, 3, 16, 16))
    y = rand(rng, (16,))
    for lx in all_layouts(4)[::5]:
        ho = ok.View.empty(x.shape, np.float32, lx)
        ok.where(ok.View(cond), ok.View(x, lx), None, -7.0, ho)
        assert (ho.logical() == np.where(cond, x, np.float32(-7.0))).all()
        ok.where(ok.View(cond), ok.View(x, lx), ok.View(y), 0.0, ho)
        assert (ho.logical() == np.where(cond, x, y)).all()
    # erf-GELU with bias: 0.5 * t * (1 + erf(t / sqrt(2))), t = x + b
    xb, b = rand(rng, (2, 8, 32)), rand(rng, (32,))
    ho = ok.View.empty(xb.shape)
    ok.add_div_erf_add_mul_mul(ok.View(xb), ok.View(b), ho, np.sqrt(2.0), 1.0, 0.5)
    want = torch.nn.functional.gelu(torch.from_numpy(xb + b)).numpy()
    close(ho.logical(), want, rtol=1e-5, atol=1e-6)
    m = rand(rng, (2, 16), 0, 1)
    ho = ok.View.empty((2, 1, 1, 16))
    ok.unsqueeze_sub_mul(ok.View(m), ho, [1, 2], 1.0, -10000.0)
    assert (ho.logical() == ((np.float32(1.0) - m) * np.float32(-10000.0)).reshape(2, 1, 1, 16)).all()


def test_data_movement():
    rng = rng_for("move")
    x = rand(rng, (2, 3, 4, 5))
    for perm in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 3, 2)]:
        for lin in all_layouts(4)[::7]:
            for lout in all_layouts(4)[::5]:
                ho = ok.View.empty(tuple(x.shape[p] for p in perm), np.float32, lout)
                ok.transpose(ok.View(x, lin), ho, perm)
                assert (ho.logical() == np.transpose(x, perm)).all()
    for oshape in [(6, 20), (2, 12, 5), (120,), (1, 2, 3, 4, 5)]:
        for lin in all_layouts(4)[::7]:
            for lout in some_layouts(len(oshape), rng, 3):
                ho = ok.View.empty(oshape, np.float32, lout)
                ok.reshape(ok.View(x, lin), ho)
                assert (ho.logical() == x.reshape(oshape)).all()
    s = rand(rng, (1, 6, 1, 5))
    ho = ok.View.empty((6, 5), np.float32, [1, 0])
    ok.squeeze(ok.View(s, [3, 1, 0, 2]), ho, [0, 2])
    assert (ho.logical() == s.reshape(6, 5)).all()
    ho = ok.View.empty((1, 6, 1, 5), np.float32, [2, 0, 3, 1])
    ok.unsqueeze(ok.View(s.reshape(6, 5), [1, 0]), ho, [0, 2])
    assert (ho.logical() == s).all()
    ho = ok.View.empty((2, 3, 2, 2))
    ok.slice_(ok.View(x, [3, 0, 2, 1]), ho, [1, 0], [2, 3], [2, 3])
    assert (ho.logical() == x[:, :, 1::2, 0::3][:, :, :2, :2]).all()
    a, b = rand(rng, (2, 3, 4)), rand(rng, (2, 5, 4))
    ho = ok.View.empty((2, 8, 4), np.float32, [1, 2, 0])
    ok.concat2(ok.View(a, [2, 1, 0]), ok.View(b), ho, 1)
    assert (ho.logical() == np.concatenate([a, b], axis=1)).all()
    p = rand(rng, (2, 3, 5))
    ho = ok.View.empty((2, 4, 8), np.float32, [2, 0, 1], fill=7)
    ok.pad(ok.View(p), ho, [0, 1, 2], 1 << 5)  # FL_REF_PAD_BORDER_UNWRITTEN
    want = np.full((2, 4, 8), 7, np.float32)
    want[:, 1:4, 2:7] = p  # border keeps its previous contents (reference pad.cpp:15-51)
    assert (ho.logical() == want).all()
    ho = ok.View.empty((2, 4, 8), np.float32, [2, 0, 1], fill=7)
    ok.pad(ok.View(p, [1, 0, 2]), ho, [0, 1, 2])  # default: ONNX constant mode, value 0
    assert (ho.logical() == np.pad(p, [(0, 0), (1, 0), (2, 1)])).all()


def test_gathers():
    rng = rng_for("gather")
    table = rand(rng, (50, 24))
    ids = rng.integers(0, 50, size=(2, 7)).astype(np.int64)
    pos, typ = rand(rng, (7, 24)), rand(rng, (24,))
    for lout in all_layouts(3):
        ho = ok.View.empty((2, 7, 24), np.float32, lout)
        ok.gather_data_tensor(ok.View(ids, [1, 0]), ok.View(table), ho)
        assert (ho.logical() == table[ids]).all()
        ok.gather_data_tensor(ok.View(ids), ok.View(table), ho, ok.View(pos), ok.View(typ))
        assert (ho.logical() == (table[ids] + pos) + typ).all()
    x = rand(rng, (4, 9, 6))
    for lin in all_layouts(3):
        for axis, index in [(0, 3), (1, 0), (2, 5), (-1, 2)]:
            ax = axis % 3
            ho = ok.View.empty(tuple(s for i, s in enumerate(x.shape) if i != ax))
            ok.gather_index_scalar(ok.View(x, lin), ho, axis, index)
            assert (ho.logical() == np.take(x, index, axis=ax)).all()
        idx = rng.integers(0, 9, size=(2, 5)).astype(np.int64)
        ho = ok.View.empty((4, 2, 5, 6))
        ok.gather_indices_tensor(ok.View(x, lin), ok.View(idx), ho, 1)
        assert (ho.logical() == np.take(x, idx, axis=1)).all()
    # literal mode: a negative axis is compared un-normalised (reference gather.cpp:116) -> no valid map
    with pytest.raises(RuntimeError):
        ok.gather_index_scalar(ok.View(x), ok.View.empty((4, 9)), -1, 2, flags=1 << 4)


@pytest.mark.parametrize("shape,axis", [((1, 12, 128, 768), 3), ((1, 12, 128, 128), 3), ((2, 17, 5), 1), ((3, 40), 0)])
def test_softmax(shape, axis):
    # (1,12,128,768) is the reference's own softmax.py shape
    rng = rng_for(shape, axis)
    x = rand(rng, shape, -6, 6)
    want = torch.softmax(torch.from_numpy(x).double(), dim=axis).float().numpy()
    for lin in some_layouts(len(shape), rng, 3):
        ho = ok.View.empty(shape, np.float32, some_layouts(len(shape), rng, 2)[-1])
        ok.softmax(ok.View(x, lin), ho, axis)
        close(ho.logical(), want, rtol=2e-5, atol=1e-7)
        close(ho.logical().sum(axis=axis), 1.0, rtol=1e-4)


@pytest.mark.parametrize("shape,axis,eps", [((1, 128, 768), 2, 1e-12), ((2, 7, 33), 2, 1e-5), ((3, 20, 5), 1, 1e-5)])
def test_layer_norm(shape, axis, eps):
    # (1,128,768) axis 2 is the reference's layer_normalization.py case
    rng = rng_for(shape, axis)
    x = rand(rng, shape, -3, 3)
    pshape = shape[axis:]
    g, b = rand(rng, pshape, 0.5, 1.5), rand(rng, pshape, -0.5, 0.5)
    xd = x.astype(np.float64)
    mean = xd.mean(axis=axis, keepdims=True)
    var = ((xd - mean) ** 2).mean(axis=axis, keepdims=True)  # biased
    want = (xd - mean) / np.sqrt(var + np.float32(eps)) * g + b
    if len(pshape) == 1:
        tl = torch.nn.functional.layer_norm(torch.from_numpy(x), pshape, torch.from_numpy(g), torch.from_numpy(b), eps)
        close(tl.numpy(), want, rtol=1e-4, atol=1e-5)
    for lin in some_layouts(len(shape), rng, 3):
        ho = ok.View.empty(shape, np.float32, some_layouts(len(shape), rng, 2)[-1])
        ok.layer_norm(ok.View(x, lin), ok.View(g), ok.View(b), ho, axis, eps)
        if len(pshape) == 1:
            close(ho.logical(), want, rtol=1e-4, atol=1e-5)
    if len(pshape) == 1:
        # literal mode (reference layer_normalization.cpp:126 vs :165): a stale scratch value s
        # shifts the mean by s/N, which then also enters the variance
        rows = int(np.prod(shape)) // shape[axis]
        stale = rng.uniform(-50, 50, size=rows).astype(np.float32)
        ho = ok.View.empty(shape)
        ok.layer_norm(ok.View(x), ok.View(g), ok.View(b), ho, axis, eps, scratch=stale)
        sshape = list(shape)
        sshape[axis] = 1
        mean_q = (xd.sum(axis=axis, keepdims=True) + stale.reshape(sshape)) / shape[axis]
        var_q = ((xd - mean_q) ** 2).mean(axis=axis, keepdims=True)
        want_q = (xd - mean_q) / np.sqrt(var_q + np.float32(eps)) * g + b
        close(ho.logical(), want_q, rtol=1e-4, atol=1e-5)
        assert np.abs(want_q - want).max() > 1e-2  # the literal mode really differs


def test_reduce_mean_and_pools():
    rng = rng_for("reduce")
    for shape, axes in [((1, 32, 14, 14), [2, 3]), ((3, 4, 5), [0]), ((2, 6, 5, 3), [1, 3])]:
        x = rand(rng, shape)
        want = x.astype(np.float64).mean(axis=tuple(axes), keepdims=True)
        for lin in some_layouts(len(shape), rng, 3):
            ho = ok.View.empty(want.shape)
            ok.reduce_mean(ok.View(x, lin), ho, axes)
            close(ho.logical(), want, rtol=1e-5, atol=1e-6)
    # reference maxpool.py [1,64,224,224] 2x2 s2 and averagepool.py [1,1280,7,7] k7 (channels cut down)
    for shape, k, s in [((1, 4, 224, 224), (2, 2), (2, 2)), ((1, 40, 7, 7), (7, 7), (1, 1)), ((2, 3, 9, 11), (3, 2), (2, 3))]:
        x = rand(rng, shape)
        t = torch.from_numpy(x)
        want_max = torch.nn.functional.max_pool2d(t, k, s).numpy()
        want_avg = torch.nn.functional.avg_pool2d(t, k, s).numpy()
        for lin in some_layouts(4, rng, 3):
            ho = ok.View.empty(want_max.shape, np.float32, lin)
            ok.pool(True, ok.View(x, lin), ho, k, s)
            assert (ho.logical() == want_max).all()
            ok.pool(False, ok.View(x, lin), ho, k, s)
            close(ho.logical(), want_avg, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("lshape,rshape", [((1, 12, 128, 64), (1, 12, 64, 128)), ((1, 128, 768), (768, 768)),
                                           ((2, 1, 33, 17), (3, 17, 29)), ((5, 7), (7, 3))])
def test_matmul(lshape, rshape):
    # first two: the reference's matmul0.py / matmul1.py shapes
    rng = rng_for(lshape, rshape)
    a, b = rand(rng, lshape, -1, 1), rand(rng, rshape, -1, 1)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    for la in some_layouts(len(lshape), rng, 2):
        for lb in some_layouts(len(rshape), rng, 2):
            ho = ok.View.empty(want.shape, np.float32, some_layouts(want.ndim, rng, 2)[-1], fill=5)
            ok.matmul(ok.View(a, la), ok.View(b, lb), ho)
            close(ho.logical(), want, rtol=1e-4, atol=1e-4)


def test_gemm_both_scalar_conventions():
    rng = rng_for("gemm")
    # reference gemm.py: [1,768] x [768,768]^T + [768]
    for ashape, bshape, cshape, alpha, beta, ta, tb in [((1, 768), (768, 768), (768,), 1.0, 1.0, 0, 1),
                                                        ((8, 100), (100, 50), (50,), 0.5, 2.0, 0, 0),
                                                        ((100, 8), (50, 100), (8, 50), 1.5, 0.25, 1, 1)]:
        a, b, c = rand(rng, ashape, -1, 1), rand(rng, bshape, -1, 1), rand(rng, cshape, -1, 1)
        A = a.T if ta else a
        B = b.T if tb else b
        ab = A.astype(np.float64) @ B.astype(np.float64)
        ho = ok.View.empty(ab.shape)
        ok.gemm(ok.View(a, [1, 0]), ok.View(b), ok.View(c), ho, alpha, beta, ta, tb, 0)
        close(ho.logical(), alpha * ab + beta * c, rtol=1e-4, atol=1e-4)  # ONNX
        ok.gemm(ok.View(a), ok.View(b, [1, 0]), ok.View(c), ho, alpha, beta, ta, tb, 1 << 3)
        close(ho.logical(), alpha * c + beta * ab, rtol=1e-4, atol=1e-4)  # reference gemm.cpp:176-179


CONV_CASES = [
    ((1, 768, 128), (768, 1, 9), [4, 4], [1], [1], 768, False),  # reference conv0.py
    ((1, 768, 128), (384, 768, 1), None, [1], [1], 1, True),  # reference conv1.py
    ((1, 3, 34, 34), (8, 3, 3, 3), [1, 1, 1, 1], [1, 1], [1, 1], 1, True),
    ((2, 4, 19, 17), (6, 4, 3, 5), [1, 2, 1, 2], [2, 2], [1, 1], 1, True),
    ((1, 6, 15, 15), (6, 1, 5, 5), [2, 2, 2, 2], [2, 2], [1, 1], 6, True),
    ((1, 2, 12, 12), (3, 2, 3, 3), [2, 2, 2, 2], [1, 1], [2, 2], 1, False),
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: str(c[:2]))
def test_conv(case):
    xshape, wshape, pads, strides, dilations, group, with_bias = case
    rng = rng_for(xshape, wshape)
    x, w = rand(rng, xshape, -1, 1), rand(rng, wshape, -1, 1)
    bias = rand(rng, (wshape[0],), -1, 1) if with_bias else None
    ns = len(xshape) - 2
    p = pads if pads is not None else [0] * (2 * ns)
    assert all(p[d] == p[d + ns] for d in range(ns))  # torch takes symmetric padding
    tx, tw = torch.from_numpy(x).double(), torch.from_numpy(w).double()
    tb = torch.from_numpy(bias).double() if with_bias else None
    fn = torch.nn.functional.conv1d if ns == 1 else torch.nn.functional.conv2d
    want = fn(tx, tw, tb, stride=strides, padding=p[:ns], dilation=dilations, groups=group).numpy()
    for lx in some_layouts(len(xshape), rng, 2):
        ho = ok.View.empty(want.shape, np.float32, some_layouts(len(xshape), rng, 2)[-1])
        ok.conv(ok.View(x, lx), ok.View(w), ok.View(bias) if with_bias else None, ho, pads, strides, dilations, group, 0)
        close(ho.logical(), want, rtol=1e-4, atol=1e-4)
    # literal mode: taps at o + k whatever the attributes say, and bias[1] everywhere
    # (reference conv.cpp:71,118,181-182) == a unit-stride, undilated convolution cropped to the
    # graph's output shape, with a constant bias
    want_unit = fn(tx, tw, None, stride=1, padding=p[:ns], dilation=1, groups=group).numpy()
    crop = tuple(slice(0, s) for s in want.shape)
    if all(want_unit.shape[i] >= want.shape[i] for i in range(len(want.shape))):
        ho = ok.View.empty(want.shape)
        flags = (1 << 0) | ((1 << 1) if with_bias else 0)
        ok.conv(ok.View(x), ok.View(w), ok.View(bias) if with_bias else None, ho, pads, strides, dilations, group, flags)
        lit = want_unit[crop] + (bias[1] if with_bias else 0.0)
        close(ho.logical(), lit, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("shape", [(3, 5), (4, 4), (2, 3, 4), (3, 3, 3)], ids=str)
def test_reference_constant_relayout(shape):
    """The reference's re-layout of constants (builder.cpp:279-297), pinned by the loop the cited lines spell out,
    written index by index, and by what the numbering implies: the default layout and every layout whose strided
    numbering is its own inverse (a square matrix stored transposed) read back unchanged; a non-square matrix stored
    transposed does not."""
    import itertools

    rng = rng_for("reference constant", shape)
    logical = rand(rng, shape)
    for layout in all_layouts(len(shape)):
        strides = ok.layout_strides(list(shape), layout)
        stored, as_read = ok.reference_constant(logical, layout)
        buffer = logical.reshape(-1)
        data = []
        for indices in itertools.product(*[range(n) for n in shape]):  # GenAllIndicesInOrder
            data.append(buffer[sum(i * s for i, s in zip(indices, strides))])  # data.push_back(buffer[GenIndex(..)])
        assert np.array_equal(stored, np.asarray(data, dtype=np.float32))
        for indices in itertools.product(*[range(n) for n in shape]):
            assert as_read[indices] == data[sum(i * s for i, s in zip(indices, strides))]
        if list(layout) == sorted(layout):
            assert np.array_equal(as_read, logical)
    if shape == (4, 4):
        assert np.array_equal(ok.reference_constant(logical, [1, 0])[1], logical)
    if shape == (3, 5):
        assert not np.array_equal(ok.reference_constant(logical, [1, 0])[1], logical)
