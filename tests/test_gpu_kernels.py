"""Parity of every HIP kernel (through the C ABI) against the C oracle on the
same seeded inputs and the same layout permutations.

Shapes follow the reference's per-operator tests (test/python/node/*.py) where
the oracle finishes in seconds, plus ragged / unaligned cases.  Bit-exact for
integer, copy and single-operation fp32 kernels; rel 1e-4 / abs 1e-5 (the
tolerance BASELINE.json states) where device libm or summation order differ.
"""
import ctypes
import sys
import zlib

import numpy as np
import pytest

from oracle import kernels as ok
from tests.util import DeviceView, all_layouts, assert_close, some_layouts

pytestmark = pytest.mark.gpu


def _cabi():
    from fluidml_amd import cabi

    return cabi


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def seed_of(*what):
    return zlib.crc32(repr(what).encode())


def rand(rng, shape, lo=-2.0, hi=2.0):
    return rng.uniform(lo, hi, size=shape).astype(np.float32)


# --------------------------------------------------------------------------- unary f32

UNARY = [
    # name, oracle op, c0, c1, exact, input range
    ("add_constant", ok.OP_ADD_C, 1.5, 0, True, (-2, 2)),
    ("sub_constant_lhs", ok.OP_RSUB_C, 1.0, 0, True, (-2, 2)),
    ("mul_constant", ok.OP_MUL_C, -10000.0, 0, True, (-2, 2)),
    ("div_constant_rhs", ok.OP_DIV_C, 8.0, 0, True, (-2, 2)),
    ("pow", ok.OP_POW_C, 2.0, 0, False, (0.1, 3)),
    ("erf", ok.OP_ERF, 0, 0, False, (-3, 3)),
    ("relu", ok.OP_RELU, 0, 0, True, (-2, 2)),
    ("clip", ok.OP_CLIP, 0.0, 6.0, True, (-8, 8)),
    ("tanh", ok.OP_TANH, 0, 0, False, (-3, 3)),
    ("sqrt", ok.OP_SQRT, 0, 0, True, (0, 4)),
    ("neg", ok.OP_NEG, 0, 0, True, (-2, 2)),
    ("dropout", ok.OP_COPY, 0, 0, True, (-2, 2)),
]


@pytest.mark.parametrize("name,op,c0,c1,exact,rng_range", UNARY, ids=[u[0] for u in UNARY])
@pytest.mark.parametrize("shape", [(1, 128, 768), (3, 5, 7), (2, 3, 4, 6)], ids=str)
def test_unary_f32(device, name, op, c0, c1, exact, rng_range, shape):
    cabi = _cabi()
    rng = np.random.default_rng(seed_of(name, shape))
    x = rand(rng, shape, *rng_range)
    for lin in some_layouts(len(shape), rng, 3):
        for lout in some_layouts(len(shape), rng, 3):
            announce(name, shape, lin, lout)
            hx, ho = ok.View(x, lin), ok.View.empty(shape, np.float32, lout)
            ok.unary_f32(op, hx, ho, c0, c1)
            dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(shape, np.float32, lout), device)
            if name in ("add_constant", "sub_constant_lhs", "mul_constant", "div_constant_rhs", "pow"):
                cabi.call(name, dx.ref(), do.ref(), ctypes.c_double(c0), None)
            elif name == "clip":
                cabi.call(name, dx.ref(), do.ref(), ctypes.c_float(c0), ctypes.c_float(c1), None)
            else:
                cabi.call(name, dx.ref(), do.ref(), None)
            assert_close(do.logical(), ho.logical(), exact=exact, what=f"{name} {shape} {lin}->{lout}")


def test_unary_unaligned_base(device):
    """Arena offsets are only 4-byte aligned in general: the 128-bit path must not be taken."""
    cabi = _cabi()
    rng = np.random.default_rng(7)
    x = rand(rng, (4, 64))
    hx, ho = ok.View(x), ok.View.empty((4, 64))
    ok.unary_f32(ok.OP_ADD_C, hx, ho, 2.0)
    for mis_in, mis_out in [(1, 0), (0, 3), (1, 2)]:
        announce("add_constant unaligned", mis_in, mis_out)
        dx = DeviceView(hx, device, misalign_elems=mis_in)
        do = DeviceView(ok.View.empty((4, 64)), device, misalign_elems=mis_out)
        cabi.call("add_constant", dx.ref(), do.ref(), ctypes.c_double(2.0), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="unaligned add")


def test_integer_and_bool_kernels(device):
    cabi = _cabi()
    rng = np.random.default_rng(11)
    shape = (2, 128)
    ids = rng.integers(0, 5, size=shape).astype(np.int64)
    for lin in all_layouts(2):
        announce("int kernels", lin)
        hx = ok.View(ids, lin)
        # add constant int64
        ho = ok.View.empty(shape, np.int64)
        ok.unary_int(ok.IOP_ADD_C, hx, ho, 2)
        dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(shape, np.int64), device)
        cabi.call("add_constant", dx.ref(), do.ref(), ctypes.c_double(2), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="add_constant i64")
        # equal -> bool
        hb = ok.View.empty(shape, np.bool_)
        ok.unary_int(ok.IOP_EQ_C, hx, hb, 1)
        db = DeviceView(ok.View.empty(shape, np.bool_), device)
        cabi.call("equal", dx.ref(), db.ref(), ctypes.c_double(1), None)
        assert_close(db.logical(), hb.logical(), exact=True, what="equal")
        # not
        hn = ok.View.empty(shape, np.bool_)
        ok.unary_int(ok.IOP_NOT, hb, hn)
        dn = DeviceView(ok.View.empty(shape, np.bool_), device)
        dbin = DeviceView(hb, device)
        cabi.call("not", dbin.ref(), dn.ref(), None)
        assert_close(dn.logical(), hn.logical(), exact=True, what="not")
        # cast bool -> int64, int64 -> int32
        for src, dst_np in [(hb, np.int64), (hx, np.int32), (hb, np.int32)]:
            hc = ok.View.empty(shape, dst_np)
            ok.unary_int(ok.IOP_CAST, src, hc)
            dc = DeviceView(ok.View.empty(shape, dst_np), device)
            ds = DeviceView(src, device)
            cabi.call("cast", ds.ref(), dc.ref(), None)
            assert_close(dc.logical(), hc.logical(), exact=True, what=f"cast ->{dst_np}")
        # cumsum along both axes
        for axis in (0, 1):
            hs = ok.View.empty(shape, np.int64)
            ok.cum_sum(hx, hs, axis)
            assert (hs.logical() == np.cumsum(ids, axis=axis)).all()
            dsum = DeviceView(ok.View.empty(shape, np.int64), device)
            cabi.call("cum_sum", dx.ref(), dsum.ref(), ctypes.c_int64(axis), None)
            assert_close(dsum.logical(), hs.logical(), exact=True, what=f"cum_sum axis {axis}")


# --------------------------------------------------------------------------- binary

BINARY = [("add_common", ok.BOP_ADD), ("sub_common", ok.BOP_SUB), ("mul_common", ok.BOP_MUL), ("div_common", ok.BOP_DIV)]
BINARY_SHAPES = [
    ((1, 128, 768), (1, 128, 768)),  # reference add0.py / mul0.py / sub1.py / div1.py
    ((1, 128, 768), (768,)),  # bias
    ((1, 12, 128, 128), (1, 1, 1, 128)),  # additive attention mask
    ((2, 5, 7), (5, 1)),
    ((3, 1, 6), (3, 4, 6)),
]


@pytest.mark.parametrize("name,op", BINARY, ids=[b[0] for b in BINARY])
@pytest.mark.parametrize("lshape,rshape", BINARY_SHAPES, ids=str)
def test_binary_f32(device, name, op, lshape, rshape):
    cabi = _cabi()
    rng = np.random.default_rng(seed_of(name, lshape, rshape))
    a, b = rand(rng, lshape), rand(rng, rshape, 0.5, 2.0)
    oshape = np.broadcast_shapes(lshape, rshape)
    for la in some_layouts(len(lshape), rng, 3):
        for lb in some_layouts(len(rshape), rng, 2):
            for lo in some_layouts(len(oshape), rng, 2):
                announce(name, lshape, rshape, la, lb, lo)
                ha, hb, ho = ok.View(a, la), ok.View(b, lb), ok.View.empty(oshape, np.float32, lo)
                ok.binary_f32(op, ha, hb, ho)
                da, db = DeviceView(ha, device), DeviceView(hb, device)
                do = DeviceView(ok.View.empty(oshape, np.float32, lo), device)
                cabi.call(name, da.ref(), db.ref(), do.ref(), None)
                assert_close(do.logical(), ho.logical(), exact=True, what=f"{name} {la} {lb} {lo}")


def test_mul_common_int(device):
    cabi = _cabi()
    rng = np.random.default_rng(5)
    a = rng.integers(-9, 9, size=(2, 16)).astype(np.int64)
    b = rng.integers(-9, 9, size=(16,)).astype(np.int64)
    ha, hb, ho = ok.View(a), ok.View(b), ok.View.empty((2, 16), np.int64)
    ok.mul_int(ha, hb, ho)
    da, db, do = DeviceView(ha, device), DeviceView(hb, device), DeviceView(ok.View.empty((2, 16), np.int64), device)
    announce("mul_common int64")
    cabi.call("mul_common", da.ref(), db.ref(), do.ref(), None)
    assert_close(do.logical(), ho.logical(), exact=True, what="mul int")


def test_where(device):
    cabi = _cabi()
    rng = np.random.default_rng(3)
    S = 64
    cond = np.tril(np.ones((1, 1, S, S), dtype=np.bool_))
    x = rand(rng, (1, 8, S, S))
    y = rand(rng, (1,))
    for lx in some_layouts(4, rng, 3):
        announce("where", lx)
        hc, hx, hy = ok.View(cond), ok.View(x, lx), ok.View(y)
        ho = ok.View.empty(x.shape, np.float32, lx)
        ok.where(hc, hx, None, -3.4e38, ho)
        dc, dx = DeviceView(hc, device), DeviceView(hx, device)
        do = DeviceView(ok.View.empty(x.shape, np.float32, lx), device)
        cabi.call("where_constant_cond_constant_scalar_y", dc.ref(), dx.ref(), do.ref(), ctypes.c_double(-3.4e38), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="where scalar y")
        ho2 = ok.View.empty(x.shape, np.float32, lx)
        ok.where(hc, hx, hy, 0.0, ho2)
        dy = DeviceView(hy, device)
        do2 = DeviceView(ok.View.empty(x.shape, np.float32, lx), device)
        cabi.call("where_constant_cond_constant_tensor_y", dc.ref(), dx.ref(), dy.ref(), do2.ref(), None)
        assert_close(do2.logical(), ho2.logical(), exact=True, what="where tensor y")


def test_fused_elementwise(device):
    cabi = _cabi()
    rng = np.random.default_rng(21)
    x, b = rand(rng, (1, 128, 3072)), rand(rng, (3072,))
    for lx in some_layouts(3, rng, 3):
        announce("add_div_erf_add_mul_mul", lx)
        hx, hb, ho = ok.View(x, lx), ok.View(b), ok.View.empty(x.shape, np.float32, lx)
        ok.add_div_erf_add_mul_mul(hx, hb, ho, 1.4142135381698608, 1.0, 0.5)
        dx, db = DeviceView(hx, device), DeviceView(hb, device)
        do = DeviceView(ok.View.empty(x.shape, np.float32, lx), device)
        cabi.call("add_div_erf_add_mul_mul", dx.ref(), db.ref(), do.ref(), ctypes.c_double(1.4142135381698608),
                  ctypes.c_double(1.0), ctypes.c_double(0.5), None)
        assert_close(do.logical(), ho.logical(), what="gelu chain")
    m = rand(rng, (1, 128), 0, 1)
    hm, ho = ok.View(m), ok.View.empty((1, 1, 1, 128))
    ok.unsqueeze_sub_mul(hm, ho, [1, 2], 1.0, -10000.0)
    dm, do = DeviceView(hm, device), DeviceView(ok.View.empty((1, 1, 1, 128)), device)
    announce("unsqueeze_sub_mul")
    cabi.call("unsqueeze_sub_lhs_scalar_mul_rhs_scalar", dm.ref(), do.ref(), cabi.i64_array([1, 2]), 2,
              ctypes.c_double(1.0), ctypes.c_double(-10000.0), None)
    assert_close(do.logical(), ho.logical(), exact=True, what="unsqueeze_sub_mul")


# --------------------------------------------------------------------------- data movement


def test_transpose(device):
    cabi = _cabi()
    rng = np.random.default_rng(31)
    for shape, perm in [((1, 128, 12, 64), (0, 2, 1, 3)), ((1, 12, 128, 64), (0, 1, 3, 2)), ((3, 5, 7), (2, 0, 1)),
                        ((33, 65), (1, 0))]:
        x = rand(rng, shape)
        oshape = tuple(shape[p] for p in perm)
        for lin in some_layouts(len(shape), rng, 3):
            for lout in some_layouts(len(shape), rng, 3):
                announce("transpose", shape, perm, lin, lout)
                hx, ho = ok.View(x, lin), ok.View.empty(oshape, np.float32, lout)
                ok.transpose(hx, ho, perm)
                assert (ho.logical() == np.transpose(x, perm)).all()
                dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape, np.float32, lout), device)
                cabi.call("transpose", dx.ref(), do.ref(), cabi.i64_array(perm), len(perm), None)
                assert_close(do.logical(), ho.logical(), exact=True, what="transpose")


def test_reshape_flatten(device):
    cabi = _cabi()
    rng = np.random.default_rng(32)
    cases = [((1, 128, 768), (1, 128, 12, 64)), ((1, 12, 128, 64), (12, 128, 64)), ((2, 3, 4), (4, 6)), ((6,), (2, 3))]
    for ishape, oshape in cases:
        x = rand(rng, ishape)
        for lin in some_layouts(len(ishape), rng, 3):
            for lout in some_layouts(len(oshape), rng, 3):
                announce("reshape", ishape, oshape, lin, lout)
                hx, ho = ok.View(x, lin), ok.View.empty(oshape, np.float32, lout)
                ok.reshape(hx, ho)
                assert (ho.logical() == x.reshape(oshape)).all()
                dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape, np.float32, lout), device)
                cabi.call("reshape", dx.ref(), do.ref(), None)
                assert_close(do.logical(), ho.logical(), exact=True, what="reshape")
    x = rand(rng, (2, 3, 4, 5))
    for axis in (0, 1, 2, -1):
        ax = axis % 4
        oshape = (int(np.prod(x.shape[:ax])), int(np.prod(x.shape[ax:])))
        for lin in some_layouts(4, rng, 3):
            announce("flatten", axis, lin)
            hx, ho = ok.View(x, lin), ok.View.empty(oshape, np.float32, [1, 0])
            ok.reshape(hx, ho)
            dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape, np.float32, [1, 0]), device)
            cabi.call("flatten", dx.ref(), do.ref(), ctypes.c_int64(axis), None)
            assert_close(do.logical(), ho.logical(), exact=True, what="flatten")


def test_squeeze_unsqueeze_slice_concat_pad(device):
    cabi = _cabi()
    rng = np.random.default_rng(33)
    x = rand(rng, (1, 128, 1, 64))
    for lin in some_layouts(4, rng, 3):
        announce("squeeze", lin)
        hx, ho = ok.View(x, lin), ok.View.empty((128, 64), np.float32, [1, 0])
        ok.squeeze(hx, ho, [0, 2])
        assert (ho.logical() == x.reshape(128, 64)).all()
        dx, do = DeviceView(hx, device), DeviceView(ok.View.empty((128, 64), np.float32, [1, 0]), device)
        cabi.call("squeeze", dx.ref(), do.ref(), cabi.i64_array([0, 2]), 2, None)
        assert_close(do.logical(), ho.logical(), exact=True, what="squeeze")
    y = rand(rng, (128, 64))
    for lout in some_layouts(4, rng, 3):
        announce("unsqueeze", lout)
        hy, ho = ok.View(y, [1, 0]), ok.View.empty((1, 128, 1, 64), np.float32, lout)
        ok.unsqueeze(hy, ho, [0, 2])
        assert (ho.logical() == y.reshape(1, 128, 1, 64)).all()
        dy, do = DeviceView(hy, device), DeviceView(ok.View.empty((1, 128, 1, 64), np.float32, lout), device)
        cabi.call("unsqueeze", dy.ref(), do.ref(), cabi.i64_array([0, 2]), 2, None)
        assert_close(do.logical(), ho.logical(), exact=True, what="unsqueeze")
    z = rand(rng, (1, 8, 256, 64))
    for lin in some_layouts(4, rng, 3):
        announce("slice/concat", lin)
        # rotary halves: z[..., :8], z[..., 8:16], and a strided slice
        for starts, axes, steps, oshape in [([0], [3], [1], (1, 8, 256, 8)), ([8], [3], [1], (1, 8, 256, 8)),
                                            ([1, 2], [2, 3], [2, 3], (1, 8, 100, 20))]:
            hz, ho = ok.View(z, lin), ok.View.empty(oshape, np.float32, lin)
            ok.slice_(hz, ho, starts, axes, steps)
            dz, do = DeviceView(hz, device), DeviceView(ok.View.empty(oshape, np.float32, lin), device)
            cabi.call("slice", dz.ref(), do.ref(), cabi.i64_array(starts), cabi.i64_array(axes), cabi.i64_array(steps),
                      len(axes), None)
            assert_close(do.logical(), ho.logical(), exact=True, what="slice")
        a, b = rand(rng, (1, 8, 256, 8)), rand(rng, (1, 8, 256, 24))
        ha, hb, ho = ok.View(a, lin), ok.View(b), ok.View.empty((1, 8, 256, 32), np.float32, lin)
        ok.concat2(ha, hb, ho, 3)
        assert (ho.logical() == np.concatenate([a, b], axis=3)).all()
        da, db = DeviceView(ha, device), DeviceView(hb, device)
        do = DeviceView(ok.View.empty((1, 8, 256, 32), np.float32, lin), device)
        cabi.call("concat2", da.ref(), db.ref(), do.ref(), ctypes.c_int64(3), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="concat2")
    p = rand(rng, (2, 3, 5))
    for flags, what in ((0, "pad (zero border)"), (cabi.FL_REF_PAD_BORDER_UNWRITTEN, "pad (border untouched)")):
        for lin, lout in (([0, 1, 2], [2, 0, 1]), ([1, 2, 0], [0, 1, 2])):
            hp, ho = ok.View(p, lin), ok.View.empty((2, 4, 8), np.float32, lout, fill=7)
            ok.pad(hp, ho, [0, 1, 2], flags)
            if flags == 0:
                assert (ho.logical() == np.pad(p, [(0, 0), (1, 0), (2, 1)])).all()
            dp = DeviceView(hp, device)
            do = DeviceView(ok.View.empty((2, 4, 8), np.float32, lout, fill=7), device)
            announce(what, lin, lout)
            cabi.call("pad", dp.ref(), do.ref(), cabi.i64_array([0, 1, 2]), 3, ctypes.c_uint32(flags), None)
            assert_close(do.logical(), ho.logical(), exact=True, what=what)


def test_pad_view_copy(device):
    """Pad along the sequence -> Gather of sliding windows -> Transpose -> Reshape as one copy that reads the Pad's
    input (the unfold of ConvBERT's span-based convolution), and a Pad on two dims seen through a Slice and a
    Transpose; checked against numpy on the padded tensor."""
    cabi = _cabi()
    rng = np.random.default_rng(29)
    # [1, S, C] padded by 4 on both sides of S, windows of 9 -> [1, S, 9, C] -> [1, S, C, 9] -> [S * H, C / H, 9]
    S, C, H, K = 40, 96, 6, 9
    x = rand(rng, (1, S, C))
    padded = np.zeros((1, S + K - 1, C), np.float32)
    padded[:, 4:4 + S] = x
    windows = np.stack([padded[:, j:j + S] for j in range(K)], axis=2)  # [1, S, K, C]
    want = np.transpose(windows, (0, 1, 3, 2)).reshape(S * H, C // H, K)
    # strides of the result inside the padded tensor: row b = (s, h) -> s * C + h * (C / H) = b * (C / H)
    strides = [C // H, 1, C]
    dx = DeviceView(ok.View(x), device)
    for lo in (None, [2, 0, 1]):
        announce("pad_view_copy unfold", lo)
        do = DeviceView(ok.View.empty(want.shape, np.float32, lo, fill=7), device)
        cabi.call("pad_view_copy", dx.ref(), cabi.i64_array([0, 4, 0]), cabi.i64_array([1, S + K - 1, C]), 3, ctypes.c_int64(0),
                  cabi.i64_array(strides), do.ref(), None)
        assert_close(do.logical(), want, exact=True, what="pad_view_copy unfold")
    # two padded dims, then Slice [1:, 2:9] and Transpose
    y = rand(rng, (5, 7))
    py = np.zeros((8, 12), np.float32)
    py[2:7, 3:10] = y
    want = py[1:, 2:9].T  # [7, 7]
    dy = DeviceView(ok.View(y), device)
    do = DeviceView(ok.View.empty(want.shape, np.float32, None, fill=7), device)
    cabi.call("pad_view_copy", dy.ref(), cabi.i64_array([2, 3]), cabi.i64_array([8, 12]), 2, ctypes.c_int64(1 * 12 + 2),
              cabi.i64_array([1, 12]), do.ref(), None)
    assert_close(do.logical(), np.ascontiguousarray(want), exact=True, what="pad_view_copy slice + transpose")
    # a view that leaves the padded tensor is refused
    assert cabi.lib.fluidml_hip_pad_view_copy(dy.ref(), cabi.i64_array([2, 3]), cabi.i64_array([8, 12]), 2, 30, cabi.i64_array([1, 12]),
                                              do.ref(), None) == -3  # FL_ERR_SHAPE


def test_gathers(device):
    cabi = _cabi()
    rng = np.random.default_rng(34)
    table = rand(rng, (1000, 768))
    ids = rng.integers(0, 1000, size=(1, 128)).astype(np.int64)
    pos, typ = rand(rng, (128, 768)), rand(rng, (768,))
    for lout in some_layouts(3, rng, 3):
        announce("gather_constant_data_tensor", lout)
        hi, ht, ho = ok.View(ids), ok.View(table), ok.View.empty((1, 128, 768), np.float32, lout)
        ok.gather_data_tensor(hi, ht, ho)
        assert (ho.logical() == table[ids]).all()
        di, dt = DeviceView(hi, device), DeviceView(ht, device)
        do = DeviceView(ok.View.empty((1, 128, 768), np.float32, lout), device)
        cabi.call("gather_constant_data_tensor", di.ref(), dt.ref(), do.ref(), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="gather data tensor")
        hp, hy = ok.View(pos), ok.View(typ)
        ho2 = ok.View.empty((1, 128, 768), np.float32, lout)
        ok.gather_data_tensor(hi, ht, ho2, hp, hy)
        dp, dy = DeviceView(hp, device), DeviceView(hy, device)
        do2 = DeviceView(ok.View.empty((1, 128, 768), np.float32, lout), device)
        cabi.call("gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs", di.ref(), dt.ref(), dp.ref(), dy.ref(),
                  do2.ref(), None)
        assert_close(do2.logical(), ho2.logical(), exact=True, what="gather+add+add")
        # one addend: Gather -> AddCommon as the separate oracle steps
        ho3 = ok.View.empty((1, 128, 768), np.float32, lout)
        ok.binary_f32(ok.BOP_ADD, ho, hp, ho3)
        do3 = DeviceView(ok.View.empty((1, 128, 768), np.float32, lout), device)
        cabi.call("gather_constant_data_tensor_add", di.ref(), dt.ref(), dp.ref(), do3.ref(), None)
        assert_close(do3.logical(), ho3.logical(), exact=True, what="gather+add")
    x = rand(rng, (4, 9, 6))
    for lin in some_layouts(3, rng, 3):
        for axis, index in [(0, 3), (1, 0), (2, 5), (-1, 2)]:
            announce("gather_constant_index_scalar", lin, axis, index)
            ax = axis % 3
            oshape = tuple(s for i, s in enumerate(x.shape) if i != ax)
            hx, ho = ok.View(x, lin), ok.View.empty(oshape)
            ok.gather_index_scalar(hx, ho, axis, index)
            assert (ho.logical() == np.take(x, index, axis=ax)).all()
            dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape), device)
            cabi.call("gather_constant_index_scalar", dx.ref(), do.ref(), ctypes.c_int64(axis), ctypes.c_int64(index),
                      ctypes.c_uint32(0), None)
            assert_close(do.logical(), ho.logical(), exact=True, what="gather index scalar")
        idx = rng.integers(0, 9, size=(2, 5)).astype(np.int64)
        announce("gather_constant_indices_tensor", lin)
        hx, hi, ho = ok.View(x, lin), ok.View(idx), ok.View.empty((4, 2, 5, 6))
        ok.gather_indices_tensor(hx, hi, ho, 1)
        assert (ho.logical() == np.take(x, idx, axis=1)).all()
        dx, di, do = DeviceView(hx, device), DeviceView(hi, device), DeviceView(ok.View.empty((4, 2, 5, 6)), device)
        cabi.call("gather_constant_indices_tensor", dx.ref(), di.ref(), do.ref(), ctypes.c_int64(1), None)
        assert_close(do.logical(), ho.logical(), exact=True, what="gather indices tensor")


# --------------------------------------------------------------------------- row reductions

SOFTMAX_CASES = [((1, 12, 128, 128), 3), ((1, 8, 256, 256), 3), ((2, 3, 9), 2), ((2, 17, 5), 1), ((4, 1500), 1),
                 ((1, 6, 128, 9), 3), ((3, 40), 0)]


@pytest.mark.parametrize("shape,axis", SOFTMAX_CASES, ids=str)
def test_softmax(device, shape, axis):
    cabi = _cabi()
    rng = np.random.default_rng(seed_of(shape, axis))
    x = rand(rng, shape, -6, 6)
    for lin in some_layouts(len(shape), rng, 3):
        for lout in some_layouts(len(shape), rng, 2):
            announce("softmax", shape, axis, lin, lout)
            hx, ho = ok.View(x, lin), ok.View.empty(shape, np.float32, lout)
            ok.softmax(hx, ho, axis)
            dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(shape, np.float32, lout), device)
            cabi.call("softmax", dx.ref(), do.ref(), None, 0, ctypes.c_int64(axis), None)
            assert_close(do.logical(), ho.logical(), what=f"softmax {shape} {lin}->{lout}")


LN_CASES = [((1, 128, 768), 2, 1e-12), ((1, 256, 512), 2, 1e-5), ((2, 7, 33), 2, 1e-5), ((3, 20, 5), 1, 1e-5),
            ((2, 5000), 1, 1e-5)]


@pytest.mark.parametrize("shape,axis,eps", LN_CASES, ids=str)
def test_layer_norm(device, shape, axis, eps):
    cabi = _cabi()
    rng = np.random.default_rng(seed_of(shape, axis))
    x = rand(rng, shape, -3, 3)
    pshape = shape[axis:]
    g, b = rand(rng, pshape, 0.5, 1.5), rand(rng, pshape, -0.5, 0.5)
    rows = int(np.prod(shape)) // shape[axis]
    for lin in some_layouts(len(shape), rng, 3):
        for lout in some_layouts(len(shape), rng, 2):
            announce("layer_norm", shape, axis, lin, lout)
            hx, hg, hb = ok.View(x, lin), ok.View(g), ok.View(b)
            ho = ok.View.empty(shape, np.float32, lout)
            ok.layer_norm(hx, hg, hb, ho, axis, eps)
            dx, dg, db = DeviceView(hx, device), DeviceView(hg, device), DeviceView(hb, device)
            do = DeviceView(ok.View.empty(shape, np.float32, lout), device)
            cabi.call("layer_normalization_constant_scale_bias", dx.ref(), dg.ref(), db.ref(), do.ref(), None, 0,
                      ctypes.c_int64(axis), ctypes.c_double(eps), ctypes.c_uint32(0), None)
            assert_close(do.logical(), ho.logical(), what=f"layer_norm {shape} {lin}->{lout}")
    # literal mode: the row sum starts from what the scratch holds
    import torch

    stale = rng.uniform(-50, 50, size=rows).astype(np.float32)
    hx, hg, hb = ok.View(x), ok.View(g), ok.View(b)
    ho = ok.View.empty(shape)
    ok.layer_norm(hx, hg, hb, ho, axis, eps, scratch=stale)
    dx, dg, db = DeviceView(hx, device), DeviceView(hg, device), DeviceView(hb, device)
    do = DeviceView(ok.View.empty(shape), device)
    dscratch = torch.from_numpy(stale).to(device)
    announce("layer_norm stale scratch", shape)
    cabi.call("layer_normalization_constant_scale_bias", dx.ref(), dg.ref(), db.ref(), do.ref(),
              ctypes.c_void_p(dscratch.data_ptr()), rows * 4, ctypes.c_int64(axis), ctypes.c_double(eps),
              ctypes.c_uint32(cabi.FL_REF_LN_STALE_SCRATCH), None)
    assert_close(do.logical(), ho.logical(), what="layer_norm stale scratch")


def test_reduce_mean(device):
    cabi = _cabi()
    rng = np.random.default_rng(41)
    # the last three: long unit-stride runs (a workgroup per output), runs that start off a 16-byte boundary
    # (169 elements per channel), and many short runs
    for shape, axes in [((1, 32, 14, 14), [2, 3]), ((1, 128, 768), [2]), ((3, 4, 5), [0]), ((2, 6, 5, 3), [1, 3]),
                        ((1, 32, 112, 112), [2, 3]), ((1, 96, 13, 13), [2, 3]), ((2, 600, 9, 9), [2, 3])]:
        x = rand(rng, shape)
        oshape = tuple(1 if i in axes else s for i, s in enumerate(shape))
        for lin in some_layouts(len(shape), rng, 3):
            announce("reduce_mean", shape, axes, lin)
            hx, ho = ok.View(x, lin), ok.View.empty(oshape)
            ok.reduce_mean(hx, ho, axes)
            dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape), device)
            cabi.call("reduce_mean", dx.ref(), do.ref(), cabi.i64_array(axes), len(axes), None)
            assert_close(do.logical(), ho.logical(), what="reduce_mean")


def test_pools(device):
    cabi = _cabi()
    rng = np.random.default_rng(42)
    cases = [((1, 8, 56, 56), (2, 2), (2, 2)), ((1, 40, 7, 7), (7, 7), (1, 1)), ((2, 3, 9, 11), (3, 2), (2, 3)),
             ((1, 4, 30), (3,), (2,)), ((2, 5, 14, 28), (2, 2), (2, 2)), ((1, 3, 13, 12), (2, 2), (3, 2)),
             ((1, 2, 10, 10), (2, 2), (2, 2)), ((1, 3, 8, 16), (2, 2), (2, 1))]
    for shape, k, s in cases:
        x = rand(rng, shape)
        n = len(k)
        oshape = tuple(shape[: len(shape) - n]) + tuple((shape[len(shape) - n + i] - k[i]) // s[i] + 1 for i in range(n))
        for lin in some_layouts(len(shape), rng, 3):
            for is_max, name in [(True, "max_pool_without_padding"), (False, "average_pool_without_padding")]:
                announce(name, shape, k, s, lin)
                hx, ho = ok.View(x, lin), ok.View.empty(oshape, np.float32, lin)
                ok.pool(is_max, hx, ho, k, s)
                dx, do = DeviceView(hx, device), DeviceView(ok.View.empty(oshape, np.float32, lin), device)
                cabi.call(name, dx.ref(), do.ref(), cabi.i64_array(k), cabi.i64_array(s), n, None)
                assert_close(do.logical(), ho.logical(), exact=True, what=name)


def test_large_outputs(device):
    """Outputs of 64 MiB and more take the non-temporal store path (and the widest launch grids): the same
    oracle comparison as the small cases, one layout each."""
    cabi = _cabi()
    rng = np.random.default_rng(2718)

    def run(what, host_inputs, oshape, oracle, call, exact):
        announce("large", what, oshape)
        ho = ok.View.empty(oshape, np.float32)
        oracle(*host_inputs, ho)
        devs = [DeviceView(h, device) for h in host_inputs]
        do = DeviceView(ok.View.empty(oshape, np.float32), device)
        call(*[d.ref() for d in devs], do.ref())
        assert_close(do.logical(), ho.logical(), exact=exact, what=f"large {what}")

    shape = (4100, 4096)  # 64.06 MiB
    x = rand(rng, shape)
    run("relu", [ok.View(x)], shape, lambda a, o: ok.unary_f32(ok.OP_RELU, a, o, 0, 0),
        lambda a, o: cabi.call("relu", a, o, None), True)
    row = rand(rng, (4096,))
    run("add_common (row broadcast)", [ok.View(x), ok.View(row)], shape, lambda a, b, o: ok.binary_f32(ok.BOP_ADD, a, b, o),
        lambda a, b, o: cabi.call("add_common", a, b, o, None), True)
    chain = cabi.make_chain([(cabi.EW_MUL_C, 0.5), (cabi.EW_RELU, 0), (cabi.EW_ADD_X, 0)])

    def chain_oracle(a, o):
        t0, t1 = ok.View.empty(shape, np.float32), ok.View.empty(shape, np.float32)
        ok.unary_f32(ok.OP_MUL_C, a, t0, 0.5, 0)
        ok.unary_f32(ok.OP_RELU, t0, t1, 0, 0)
        ok.binary_f32(ok.BOP_ADD, t1, a, o)

    run("elementwise_chain", [ok.View(x)], shape, chain_oracle,
        lambda a, o: cabi.call("elementwise_chain", a, o, ctypes.byref(chain), None), True)
    for sshape in [(131080, 128), (16400, 1024)]:
        xs = rand(rng, sshape, -6, 6)
        run(f"softmax {sshape}", [ok.View(xs)], sshape, lambda a, o: ok.softmax(a, o, 1),
            lambda a, o: cabi.call("softmax", a, o, None, 0, ctypes.c_int64(1), None), False)
    lshape = (21900, 768)
    xl, g, b = rand(rng, lshape, -3, 3), rand(rng, (768,), 0.5, 1.5), rand(rng, (768,), -0.5, 0.5)
    run("layer_norm", [ok.View(xl), ok.View(g), ok.View(b)], lshape, lambda a, gg, bb, o: ok.layer_norm(a, gg, bb, o, 1, 1e-5),
        lambda a, gg, bb, o: cabi.call("layer_normalization_constant_scale_bias", a, gg, bb, o, None, 0, ctypes.c_int64(1),
                                       ctypes.c_double(1e-5), ctypes.c_uint32(0), None), False)
    tshape = (4160, 4128)
    xt = rand(rng, tshape)
    run("transpose", [ok.View(xt)], (4128, 4160), lambda a, o: ok.transpose(a, o, (1, 0)),
        lambda a, o: cabi.call("transpose", a, o, cabi.i64_array((1, 0)), 2, None), True)
    pshape, two = (16, 64, 264, 256), cabi.i64_array((2, 2))
    xp = rand(rng, pshape)
    for is_max, name in [(True, "max_pool_without_padding"), (False, "average_pool_without_padding")]:
        run(name, [ok.View(xp)], (16, 64, 132, 128), lambda a, o, m=is_max: ok.pool(m, a, o, (2, 2), (2, 2)),
            lambda a, o, nm=name: cabi.call(nm, a, o, two, two, 2, None), True)


# --------------------------------------------------------------------------- contractions

MATMUL_CASES = [
    ((1, 12, 128, 64), (1, 12, 64, 128)),  # reference matmul0.py
    ((1, 128, 768), (768, 768)),  # reference matmul1.py
    ((1, 12, 128, 128), (1, 12, 128, 64)),
    ((2, 1, 33, 17), (3, 17, 29)),  # broadcast both ways, ragged
    ((5, 7), (7, 3)),
    ((1, 130, 70), (70, 258)),  # tile edges
    ((64, 6), (6, 64)),  # K not a multiple of 4
    ((192, 1152), (1152, 49)),  # wide loads for the left operand only, K split over workgroups
    ((900, 64), (64, 1001)),  # the same on the 64x64 tile
    ((64, 1000), (1000, 40)),  # four tiles, a workgroup per chunk of K, the last chunk ragged
]


@pytest.mark.parametrize("lshape,rshape", MATMUL_CASES, ids=str)
def test_matmul(device, lshape, rshape):
    cabi = _cabi()
    rng = np.random.default_rng(seed_of(lshape, rshape))
    # activations in [-1, 1], weights at the N(0, 0.02)-like scale of the BASELINE configs: the stated
    # rel 1e-4 / abs 1e-5 bound is about such data (a K=768 fp32 sum of O(1) products already differs by
    # more than 1e-5 between two summation orders)
    a, b = rand(rng, lshape, -1, 1), rand(rng, rshape, -0.05, 0.05)
    oshape = np.matmul(np.zeros(lshape, np.int8), np.zeros(rshape, np.int8)).shape
    for la in some_layouts(len(lshape), rng, 3):
        for lb in some_layouts(len(rshape), rng, 3):
            for lo in some_layouts(len(oshape), rng, 2):
                announce("matmul", lshape, rshape, la, lb, lo)
                ha, hb, ho = ok.View(a, la), ok.View(b, lb), ok.View.empty(oshape, np.float32, lo)
                ok.matmul(ha, hb, ho)
                da, db = DeviceView(ha, device), DeviceView(hb, device)
                do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=9), device)
                cabi.call("matmul", da.ref(), db.ref(), do.ref(), None)
                assert_close(do.logical(), ho.logical(), what=f"matmul {la} {lb} {lo}")


def test_matmul_large_tiles(device):
    """Shapes that select the 64x64 and 128x128 workgroup tiles."""
    cabi = _cabi()
    rng = np.random.default_rng(77)
    for M, K, N in [(1024, 96, 1024), (2048, 64, 2048), (520, 40, 1000)]:
        a, b = rand(rng, (M, K), -1, 1), rand(rng, (K, N), -0.05, 0.05)
        want = a.astype(np.float64) @ b.astype(np.float64)
        for la, lb in [([0, 1], [0, 1]), ([1, 0], [1, 0]), ([0, 1], [1, 0])]:
            announce("matmul large", M, K, N, la, lb)
            da, db = DeviceView(ok.View(a, la), device), DeviceView(ok.View(b, lb), device)
            do = DeviceView(ok.View.empty((M, N)), device)
            cabi.call("matmul", da.ref(), db.ref(), do.ref(), None)
            assert_close(do.logical(), want.astype(np.float32), what="matmul large vs float64 numpy")


def test_matmul_split_k(device):
    """Few tiles and a long K: the tile's K range is split over several workgroups whose partial tiles are
    added in split order by the last one to arrive -- the result must not depend on arrival order."""
    cabi = _cabi()
    rng = np.random.default_rng(80)
    for M, K, N in [(128, 768, 768), (128, 3072, 768), (100, 1000, 70), (1, 4096, 512)]:
        a, b = rand(rng, (M, K), -1, 1), rand(rng, (K, N), -0.05, 0.05)
        want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
        announce("matmul split k", M, K, N)
        da, db = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device)
        runs = []
        for _ in range(4):
            do = DeviceView(ok.View.empty((M, N), fill=3), device)
            cabi.call("matmul", da.ref(), db.ref(), do.ref(), None)
            runs.append(do.logical())
        assert_close(runs[0], want, what="matmul split k vs float64 numpy")
        for r in runs[1:]:
            assert (r == runs[0]).all(), "split-K sum depends on the run"


def _round_bf16(x):
    """float32 -> nearest-even bf16 -> float32"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(x.shape)


def test_matmul_bf16(device):
    """Opt-in path: both operands rounded to bf16, products and sums in fp32.  Checked to the fp32 tolerance
    against the oracle run on the rounded operands; the distance to the unrounded fp32 result is printed."""
    cabi = _cabi()
    rng = np.random.default_rng(81)
    # (the last two reach the 128x128 tile; the last one with ragged extents and K not a multiple of the chunk)
    for ashape, bshape in [((1, 128, 768), (768, 768)), ((2, 3, 70, 40), (40, 50)), ((1024, 96), (96, 1024)),
                           ((2048, 64), (64, 2048)), ((2100, 72), (72, 2060))]:
        a, b = rand(rng, ashape, -1, 1), rand(rng, bshape, -0.05, 0.05)
        oshape = np.matmul(np.empty(ashape, np.int8), np.empty(bshape, np.int8)).shape
        want = ok.View.empty(oshape)
        ok.matmul(ok.View(_round_bf16(a)), ok.View(_round_bf16(b)), want)
        exact = ok.View.empty(oshape)
        ok.matmul(ok.View(a), ok.View(b), exact)
        for la in (None, list(range(len(ashape)))[::-1]):
            announce("matmul bf16", ashape, bshape, la)
            da, db = DeviceView(ok.View(a, la), device), DeviceView(ok.View(b), device)
            do = DeviceView(ok.View.empty(oshape, fill=4), device)
            cabi.call("matmul_bf16", da.ref(), db.ref(), do.ref(), None)
            assert_close(do.logical(), want.logical(), what="matmul_bf16 vs oracle on bf16-rounded operands")
        err = np.abs(do.logical() - exact.logical())
        print(f"[bf16] {ashape}x{bshape}: max abs err vs fp32 {err.max():.3e}, relative to max |c| {err.max() / np.abs(exact.logical()).max():.3e}")
        assert err.max() / np.abs(exact.logical()).max() < 2e-2


def test_matmul_unaligned(device):
    cabi = _cabi()
    rng = np.random.default_rng(78)
    a, b = rand(rng, (40, 24), -1, 1), rand(rng, (24, 36), -0.05, 0.05)
    ha, hb, ho = ok.View(a), ok.View(b), ok.View.empty((40, 36))
    ok.matmul(ha, hb, ho)
    announce("matmul unaligned")
    da, db = DeviceView(ha, device, misalign_elems=1), DeviceView(hb, device, misalign_elems=3)
    do = DeviceView(ok.View.empty((40, 36)), device, misalign_elems=1)
    cabi.call("matmul", da.ref(), db.ref(), do.ref(), None)
    assert_close(do.logical(), ho.logical(), what="matmul unaligned bases")


def test_gemm(device):
    cabi = _cabi()
    rng = np.random.default_rng(51)
    # reference gemm.py: [1,768] x [768,768]^T + [768], alpha = beta = 1
    cases = [((1, 768), (768, 768), (768,), 1.0, 1.0, 0, 1), ((8, 100), (100, 50), (50,), 0.5, 2.0, 0, 0),
             ((100, 8), (50, 100), (8, 50), 1.5, 0.25, 1, 1), ((33, 65), (65, 17), (33, 17), 2.0, 3.0, 0, 0),
             # few rows against k-contiguous weights: the weight-streaming kernel (1, 2, 3..4 and 5..8 row variants)
             ((8, 2048), (1000, 2048), (1000,), 1.0, 1.0, 0, 1), ((3, 4096), (515, 4096), (515,), 1.0, 1.0, 0, 1),
             ((2, 1024), (300, 1024), (2, 300), 0.5, 2.0, 0, 1), ((5, 512), (257, 512), (257,), 1.0, 1.0, 0, 1),
             # long K: a workgroup per one or two weight rows, K split over its waves (K not a multiple of the step)
             ((1, 3588), (4099, 3588), (4099,), 1.0, 1.0, 0, 1), ((6, 2052), (4100, 2052), (4100,), 1.0, 0.5, 0, 1)]
    for ashape, bshape, cshape, alpha, beta, ta, tb in cases:
        a, b, c = rand(rng, ashape, -1, 1), rand(rng, bshape, -0.05, 0.05), rand(rng, cshape, -1, 1)
        M = ashape[1] if ta else ashape[0]
        N = bshape[0] if tb else bshape[1]
        for flags in (0, cabi.FL_REF_GEMM_SWAPPED_SCALARS):
            for la, lb in [([0, 1], [0, 1]), ([1, 0], [1, 0])]:
                announce("gemm", ashape, bshape, cshape, alpha, beta, ta, tb, flags, la, lb)
                ha, hb, hc, ho = ok.View(a, la), ok.View(b, lb), ok.View(c), ok.View.empty((M, N))
                ok.gemm(ha, hb, hc, ho, alpha, beta, ta, tb, flags)
                da, db, dc = DeviceView(ha, device), DeviceView(hb, device), DeviceView(hc, device)
                do = DeviceView(ok.View.empty((M, N)), device)
                cabi.call("gemm_constant_weights_bias", da.ref(), db.ref(), dc.ref(), do.ref(), ctypes.c_double(alpha),
                          ctypes.c_double(beta), ta, tb, ctypes.c_uint32(flags), None)
                assert_close(do.logical(), ho.logical(), what="gemm")


# --------------------------------------------------------------------------- launch-level fusions
# Each fused entry point is checked against the oracle's UNFUSED chain of kernels.

def test_fused_matmul_add_and_gelu(device):
    cabi = _cabi()
    rng = np.random.default_rng(91)
    for ashape, bshape in [((1, 128, 768), (768, 3072)), ((1, 128, 768), (768, 768)), ((2, 3, 17, 40), (40, 29)),
                           ((1, 5, 64), (64, 8))]:
        a, b = rand(rng, ashape, -1, 1), rand(rng, bshape, -0.05, 0.05)
        oshape = ashape[:-1] + (bshape[-1],)
        bias = rand(rng, (bshape[-1],), -0.5, 0.5)
        for la, lb, lo in [(None, None, None), (list(range(len(ashape)))[::-1], [1, 0], list(range(len(oshape)))[::-1])]:
            announce("fused matmul+add(+gelu)", ashape, bshape, la, lb, lo)
            ha, hb, hbias = ok.View(a, la), ok.View(b, lb), ok.View(bias)
            t0, t1 = ok.View.empty(oshape), ok.View.empty(oshape)
            ok.matmul(ha, hb, t0)
            ok.binary_f32(ok.BOP_ADD, hbias, t0, t1)  # bias first, like the exported graphs
            da, db, dbias = DeviceView(ha, device), DeviceView(hb, device), DeviceView(hbias, device)
            do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
            cabi.call("matmul_add", da.ref(), db.ref(), dbias.ref(), do.ref(), None)
            assert_close(do.logical(), t1.logical(), what="matmul_add")
            # Div -> Erf -> Add -> Mul(t, .) -> Mul
            u0, u1, u2, u3, u4 = (ok.View.empty(oshape) for _ in range(5))
            ok.unary_f32(ok.OP_DIV_C, t1, u0, 1.4142135381698608)
            ok.unary_f32(ok.OP_ERF, u0, u1)
            ok.unary_f32(ok.OP_ADD_C, u1, u2, 1.0)
            ok.binary_f32(ok.BOP_MUL, t1, u2, u3)
            ok.unary_f32(ok.OP_MUL_C, u3, u4, 0.5)
            do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
            gelu = cabi.make_chain([(cabi.EW_DIV_C, 1.4142135381698608), (cabi.EW_ERF, 0), (cabi.EW_ADD_C, 1.0),
                                    (cabi.EW_MUL_X, 0), (cabi.EW_MUL_C, 0.5)])
            cabi.call("matmul_chain", da.ref(), db.ref(), dbias.ref(), do.ref(), ctypes.byref(gelu), ctypes.c_uint32(0), None)
            assert_close(do.logical(), u4.logical(), what="matmul_chain bias + erf-GELU")
            # no bias, chain only: relu(a.b) * 0.5
            ok.unary_f32(ok.OP_RELU, t0, u0)
            ok.unary_f32(ok.OP_MUL_C, u0, u1, 0.5)
            do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
            chain = cabi.make_chain([(cabi.EW_RELU, 0), (cabi.EW_MUL_C, 0.5)])
            cabi.call("matmul_chain", da.ref(), db.ref(), None, do.ref(), ctypes.byref(chain), ctypes.c_uint32(0), None)
            assert_close(do.logical(), u1.logical(), what="matmul_chain relu, scale")


def test_matmul_chain_add(device):
    """MatMul + bias [+ chain] followed by one or two AddCommon with tensors of the output's shape, as one launch; the
    sums are taken in the order of the separate kernels.  Small and large tiles, batch dims, a transposed output."""
    cabi = _cabi()
    rng = np.random.default_rng(93)
    relu = cabi.make_chain([(cabi.EW_RELU, 0)])
    none = cabi.make_chain([])
    for ashape, bshape, lo, two, with_chain in [((1, 256, 512), (512, 512), None, True, False),
                                                ((1, 128, 768), (768, 768), None, False, False),
                                                ((2, 3, 70, 40), (40, 96), None, True, True),
                                                ((1, 300, 256), (256, 1024), [0, 2, 1], True, False),
                                                ((1, 80, 256), (256, 49), None, True, False)]:  # rows of B unaligned
        a, b = rand(rng, ashape, -1, 1), rand(rng, bshape, -0.05, 0.05)
        oshape = ashape[:-1] + (bshape[-1],)
        bias, r1, r2 = rand(rng, (bshape[-1],), -0.5, 0.5), rand(rng, oshape, -1, 1), rand(rng, oshape, -1, 1)
        # (second pass: the opt-in bf16 operands, against the oracle on the rounded operands)
        # (rows of B that are not 16-byte aligned keep the launch in fp32 whatever the flag says)
        rounds = bshape[-1] % 4 == 0
        for flags, opa, opb in ((0, a, b), (cabi.FL_CONTRACT_BF16, _round_bf16(a) if rounds else a, _round_bf16(b) if rounds else b)):
            announce("matmul_chain_add", ashape, bshape, lo, two, with_chain, "flags", flags)
            t0, t1 = ok.View.empty(oshape), ok.View.empty(oshape)
            ok.matmul(ok.View(opa), ok.View(opb), t0)
            ok.binary_f32(ok.BOP_ADD, ok.View(bias), t0, t1)
            if with_chain:
                t = ok.View.empty(oshape)
                ok.unary_f32(ok.OP_RELU, t1, t)
                t1 = t
            want = ok.View.empty(oshape)
            ok.binary_f32(ok.BOP_ADD, ok.View(r1), t1, want)
            if two:
                t = ok.View.empty(oshape)
                ok.binary_f32(ok.BOP_ADD, want, ok.View(r2), t)
                want = t
            h1, h2 = ok.View.empty(oshape, np.float32, lo), ok.View.empty(oshape, np.float32, lo)
            h1.logical()[...] = r1
            h2.logical()[...] = r2
            da, db, dbias = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device), DeviceView(ok.View(bias), device)
            d1, d2 = DeviceView(h1, device), DeviceView(h2, device)
            do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
            cabi.call("matmul_chain_add", da.ref(), db.ref(), dbias.ref(), do.ref(), ctypes.byref(relu if with_chain else none),
                      d1.ref(), d2.ref() if two else None, ctypes.c_uint32(flags), None)
            assert_close(do.logical(), want.logical(), what=f"matmul_chain_add, flags {flags}")
    # a right operand stored k-fastest is refused
    bt = DeviceView(ok.View(rand(rng, (40, 96)), [1, 0]), device)
    a = DeviceView(ok.View(rand(rng, (70, 40))), device)
    o, r = DeviceView(ok.View.empty((70, 96)), device), DeviceView(ok.View(rand(rng, (70, 96))), device)
    assert cabi.lib.fluidml_hip_matmul_chain_add(a.ref(), bt.ref(), None, o.ref(), ctypes.byref(none), r.ref(), None, 0, None) == cabi.FL_ERR_UNSUPPORTED


def test_matmul_chain_view(device):
    """MatMul + bias written straight into the buffer of a following Reshape (last dim split into heads) and
    Transpose: the head-split copies of an attention block folded into the contraction's output addressing."""
    cabi = _cabi()
    rng = np.random.default_rng(96)
    S, H, heads, d = 24, 48, 4, 12
    a, b, bias = rand(rng, (1, S, H), -1, 1), rand(rng, (H, H), -0.2, 0.2), rand(rng, (H,), -0.5, 0.5)
    t0, t1 = ok.View.empty((1, S, H)), ok.View.empty((1, S, H))
    ok.matmul(ok.View(a), ok.View(b), t0)
    ok.binary_f32(ok.BOP_ADD, ok.View(bias), t0, t1)
    r = ok.View.empty((1, S, heads, d))
    ok.reshape(t1, r)
    for perm, lout in [((0, 2, 1, 3), None), ((0, 2, 3, 1), None), ((0, 2, 1, 3), [3, 1, 0, 2])]:
        oshape = tuple((1, S, heads, d)[p] for p in perm)
        want = ok.View.empty(oshape)
        ok.transpose(r, want, list(perm))
        announce("matmul chain view", perm, lout)
        final = ok.View.empty(oshape, np.float32, lout, fill=5)
        dfinal = DeviceView(final, device)
        fs = final.strides  # strides of the transposed tensor's dims
        pos = {p: k for k, p in enumerate(perm)}  # reshape dim -> transposed dim
        # logical [1, S, H]: dim 0 and dim 1 map to reshape dims 0 and 1, H splits into (heads, d)
        view = cabi.make_tensor(dfinal.tensor.base, cabi.FL_FLOAT32, [1, S, H], [fs[pos[0]], fs[pos[1]], fs[pos[3]]])
        da, db, dbias = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device), DeviceView(ok.View(bias), device)
        cabi.call("matmul_chain_view", da.ref(), db.ref(), dbias.ref(), ctypes.byref(view), ctypes.c_int64(d),
                  ctypes.c_int64(fs[pos[2]]), None, ctypes.c_uint32(0), None)
        assert_close(dfinal.logical(), want.logical(), what="matmul_chain_view")


def test_matmul_chain_group(device):
    """Three contractions that share the left operand in one launch (query / key / value projections), each
    with its own weights, bias and output addressing."""
    cabi = _cabi()
    rng = np.random.default_rng(97)
    S, H = 40, 64
    a = rand(rng, (1, S, H), -1, 1)
    ws = [rand(rng, (H, H), -0.2, 0.2) for _ in range(3)]
    bs = [rand(rng, (H,), -0.5, 0.5) for _ in range(3)]
    louts = [None, [2, 1, 0], [0, 2, 1]]
    wants, douts = [], []
    for w, b, lo in zip(ws, bs, louts):
        t0, t1 = ok.View.empty((1, S, H)), ok.View.empty((1, S, H))
        ok.matmul(ok.View(a), ok.View(w), t0)
        ok.binary_f32(ok.BOP_ADD, ok.View(b), t0, t1)
        wants.append(t1.logical())
        douts.append(DeviceView(ok.View.empty((1, S, H), np.float32, lo, fill=2), device))
    da = DeviceView(ok.View(a), device)
    dws = [DeviceView(ok.View(w), device) for w in ws]
    dbs = [DeviceView(ok.View(b), device) for b in bs]
    ptr = ctypes.POINTER(cabi.FlTensor)
    rhs = (ptr * 3)(*[ctypes.pointer(d.tensor) for d in dws])
    bias = (ptr * 3)(*[ctypes.pointer(d.tensor) for d in dbs])
    out = (ptr * 3)(*[ctypes.pointer(d.tensor) for d in douts])
    announce("matmul chain group")
    cabi.call("matmul_chain_group", 3, da.ref(), rhs, bias, out, ctypes.c_int64(0), None, None, ctypes.c_uint32(0), None)
    for d, want in zip(douts, wants):
        assert_close(d.logical(), want, what="matmul_chain_group")
    # mismatching sibling shapes are rejected
    bad = DeviceView(ok.View(rand(rng, (H, H + 4), -1, 1)), device)
    rhs_bad = (ptr * 2)(ctypes.pointer(dws[0].tensor), ctypes.pointer(bad.tensor))
    assert cabi.lib.fluidml_hip_matmul_chain_group(2, da.ref(), rhs_bad, bias, out, 0, None, None, 0, None) == -3  # FL_ERR_SHAPE


def test_fused_pointwise_conv_pair(device):
    """Conv 1x1 -> swish -> Conv 1x1 -> sigmoid on one-pixel tensors against the oracle's separate kernels."""
    cabi = _cabi()
    rng = np.random.default_rng(77)
    swish = [(cabi.EW_DIV_C, 2.0), (cabi.EW_TANH, 0), (cabi.EW_ADD_C, 1.0), (cabi.EW_MUL_C, 0.5), (cabi.EW_MUL_X, 0)]
    sigmoid = swish[:4]
    oracle_op = {cabi.EW_DIV_C: ok.OP_DIV_C, cabi.EW_TANH: ok.OP_TANH, cabi.EW_ADD_C: ok.OP_ADD_C, cabi.EW_MUL_C: ok.OP_MUL_C}

    def chain_on_host(v, steps):
        cur = v
        for op, c in steps:
            nxt = ok.View.empty(v.shape, np.float32)
            if op == cabi.EW_MUL_X:
                ok.binary_f32(ok.BOP_MUL, cur, v, nxt)
            else:
                ok.unary_f32(oracle_op[op], cur, nxt, c, 0)
            cur = nxt
        return cur

    for n, c, hidden, f, with_bias in [(1, 96, 4, 96, True), (2, 1152, 48, 1152, True), (3, 40, 10, 300, False),
                                          (1, 2600, 6, 1030, True), (2, 37, 5, 9, True),
                                          (1, 1154, 50, 1201, True)]:  # many weights, rows not 16-byte aligned: two launches
        announce("pointwise_conv_pair", n, c, hidden, f, with_bias)
        x = rand(rng, (n, c, 1, 1))
        w1, w2 = rand(rng, (hidden, c, 1, 1), -0.2, 0.2), rand(rng, (f, hidden, 1, 1), -0.5, 0.5)
        b1, b2 = rand(rng, (hidden,)), rand(rng, (f,))
        hx, hw1, hw2, hb1, hb2 = ok.View(x), ok.View(w1), ok.View(w2), ok.View(b1), ok.View(b2)
        mid, res = ok.View.empty((n, hidden, 1, 1), np.float32), ok.View.empty((n, f, 1, 1), np.float32)
        ok.conv(hx, hw1, hb1 if with_bias else None, mid, None, (1, 1), (1, 1), 1, 0)
        ok.conv(chain_on_host(mid, swish), hw2, hb2 if with_bias else None, res, None, (1, 1), (1, 1), 1, 0)
        want = chain_on_host(res, sigmoid)
        dx, dw1, dw2, db1, db2 = (DeviceView(h, device) for h in (hx, hw1, hw2, hb1, hb2))
        do = DeviceView(ok.View.empty((n, f, 1, 1), np.float32), device)
        p1, p2 = cabi.make_chain(swish), cabi.make_chain(sigmoid)
        cabi.call("pointwise_conv_pair", dx.ref(), dw1.ref(), db1.ref() if with_bias else None, ctypes.byref(p1), dw2.ref(),
                  db2.ref() if with_bias else None, ctypes.byref(p2), do.ref(), None)
        assert_close(do.logical(), want.logical(), what="pointwise_conv_pair")


def test_fused_softmax_matvec(device):
    """Softmax over a few logits -> MatMul with the result against the oracle's two kernels; the output is written
    through the strides of a reshaped buffer."""
    cabi = _cabi()
    rng = np.random.default_rng(123)
    for batch, rows, k in [(768, 64, 9), (32, 16, 9), (5, 7, 16), (3, 130, 1)]:
        announce("softmax_matvec", batch, rows, k)
        a, v = rand(rng, (batch, rows, k)), rand(rng, (batch, k, 1), -4, 4)
        ha, hv = ok.View(a), ok.View(v)
        hs, ho = ok.View.empty((batch, k, 1), np.float32), ok.View.empty((batch, rows, 1), np.float32)
        ok.softmax(hv, hs, 1)
        ok.matmul(ha, hs, ho)
        da, dv = DeviceView(ha, device), DeviceView(hv, device)
        do = DeviceView(ok.View.empty((batch, rows, 1), np.float32), device)
        cabi.call("softmax_matvec", da.ref(), dv.ref(), do.ref(), None)
        assert_close(do.logical(), ho.logical(), what="softmax_matvec")
        # transposed storage of the matrix and of the output
        ha2 = ok.View(a, [2, 0, 1])
        da2 = DeviceView(ha2, device)
        do2 = DeviceView(ok.View.empty((batch, rows, 1), np.float32, [1, 0, 2]), device)
        cabi.call("softmax_matvec", da2.ref(), dv.ref(), do2.ref(), None)
        assert_close(do2.logical(), ho.logical(), what="softmax_matvec (strided)")
        # the batches as `inner` heads of each position inside the second half of a [positions, 2 * inner, rows] buffer
        inner = 6 if batch % 6 == 0 else 1
        whole = DeviceView(ok.View.empty((batch // inner, 2 * inner, rows), np.float32, fill=3), device)
        part = cabi.make_tensor(whole.storage.data_ptr() + inner * rows * 4, ok.FL_FLOAT32, (batch // inner, inner, rows, 1),
                                (2 * inner * rows, rows, 1, 1))
        cabi.call("softmax_matvec", da.ref(), dv.ref(), ctypes.byref(part), None)
        got = whole.logical()
        assert_close(got[:, inner:, :].reshape(batch, rows, 1), ho.logical(), what="softmax_matvec (split batch)")
        assert np.all(got[:, :inner, :] == 3), "softmax_matvec wrote outside its part"
    big = DeviceView(ok.View(rand(rng, (2, 3, 17))), device)
    logits = DeviceView(ok.View(rand(rng, (2, 17, 1))), device)
    res = DeviceView(ok.View.empty((2, 3, 1), np.float32), device)
    with pytest.raises(cabi.FluidmlHipError):
        cabi.call("softmax_matvec", big.ref(), logits.ref(), res.ref(), None)


def test_fused_mul_add(device):
    """MulCommon -> AddCommon in one launch: the product is rounded before the sum, so the result is the two
    kernels' bit for bit; all three inputs broadcast."""
    cabi = _cabi()
    rng = np.random.default_rng(171)
    for sa, sb, sc, so in [((1, 2, 24, 8), (24, 8), (1, 2, 24, 8), (1, 2, 24, 8)), ((4, 1, 6), (1, 5, 6), (6,), (4, 5, 6)),
                           ((1, 96, 14, 14), (1, 96, 1, 1), (1, 96, 14, 14), (1, 96, 14, 14))]:
        a, b, c = rand(rng, sa), rand(rng, sb), rand(rng, sc)
        for lo in some_layouts(len(so), rng, 2):
            announce("mul_add", sa, sb, sc, lo)
            t, want = ok.View.empty(np.broadcast_shapes(sa, sb)), ok.View.empty(so)
            ok.binary_f32(ok.BOP_MUL, ok.View(a), ok.View(b), t)
            ok.binary_f32(ok.BOP_ADD, t, ok.View(c), want)
            da, db, dc = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device), DeviceView(ok.View(c), device)
            do = DeviceView(ok.View.empty(so, np.float32, lo, fill=5), device)
            cabi.call("mul_add", da.ref(), db.ref(), dc.ref(), do.ref(), None)
            assert_close(do.logical(), want.logical(), exact=True, what="mul_add")
            # AddCommon -> AddCommon on the same operands
            ok.binary_f32(ok.BOP_ADD, ok.View(a), ok.View(b), t)
            ok.binary_f32(ok.BOP_ADD, t, ok.View(c), want)
            do = DeviceView(ok.View.empty(so, np.float32, lo, fill=5), device)
            cabi.call("add_add", da.ref(), db.ref(), dc.ref(), do.ref(), None)
            assert_close(do.logical(), want.logical(), exact=True, what="add_add")


def test_fused_rotary(device):
    """The rotary embedding's Slice / Neg / Concat2 / MulCommon / AddCommon / Concat2 steps as one launch: the
    result is the oracle's nine steps bit for bit, for any layouts of x and out, with and without a pass-through
    part, tables that broadcast over heads."""
    cabi = _cabi()
    rng = np.random.default_rng(173)
    for shape, rot, tshape in [((1, 8, 256, 64), 16, (1, 1, 256, 16)), ((2, 3, 10, 8), 8, (10, 8)),
                               ((1, 2, 7, 12), 4, (1, 2, 7, 4)), ((5, 6), 6, (5, 6))]:
        x = rand(rng, shape)
        cos_t, sin_t = rand(rng, tshape, -1, 1), rand(rng, tshape, -1, 1)
        rank, last, half = len(shape), len(shape) - 1, rot // 2
        hx = ok.View(x)
        want = ok.View.empty(shape)
        if rot > 0:
            head = shape[:-1]
            xr, x1, x2, neg, turned = (ok.View.empty(head + (n,)) for n in (rot, half, half, half, rot))
            ok.slice_(hx, xr, [0], [last], [1])
            ok.slice_(xr, x1, [0], [last], [1])
            ok.slice_(xr, x2, [half], [last], [1])
            ok.unary_f32(ok.OP_NEG, x2, neg)
            ok.concat2(neg, x1, turned, last)
            m1, m2, summed = (ok.View.empty(head + (rot,)) for _ in range(3))
            ok.binary_f32(ok.BOP_MUL, xr, ok.View(cos_t), m1)
            ok.binary_f32(ok.BOP_MUL, turned, ok.View(sin_t), m2)
            ok.binary_f32(ok.BOP_ADD, m1, m2, summed)
            if rot == shape[-1]:
                want = summed
            else:
                rest = ok.View.empty(head + (shape[-1] - rot,))
                ok.slice_(hx, rest, [rot], [last], [1])
                ok.concat2(summed, rest, want, last)
        for lx, lo in [(None, None), (list(range(rank))[::-1], None), (None, list(range(rank))[::-1])]:
            announce("rotary", shape, rot, tshape, lx, lo)
            dx = DeviceView(ok.View(x, lx), device)
            dc, ds = DeviceView(ok.View(cos_t), device), DeviceView(ok.View(sin_t), device)
            do = DeviceView(ok.View.empty(shape, np.float32, lo, fill=5), device)
            cabi.call("rotary", dx.ref(), dc.ref(), ds.ref(), do.ref(), ctypes.c_int64(rot), None)
            assert_close(do.logical(), want.logical(), exact=True, what="rotary")
        # two tensors in one launch: x and 2x against the same tables, outputs in different layouts
        announce("rotary pair", shape, rot, tshape)
        d0, d1 = DeviceView(ok.View(x), device), DeviceView(ok.View((2 * x).astype(np.float32), list(range(rank))[::-1]), device)
        dc, ds = DeviceView(ok.View(cos_t), device), DeviceView(ok.View(sin_t), device)
        o0 = DeviceView(ok.View.empty(shape, np.float32, list(range(rank))[::-1], fill=5), device)
        o1 = DeviceView(ok.View.empty(shape, np.float32, None, fill=5), device)
        cabi.call("rotary_pair", d0.ref(), o0.ref(), d1.ref(), o1.ref(), dc.ref(), ds.ref(), ctypes.c_int64(rot), None)
        assert_close(o0.logical(), want.logical(), exact=True, what="rotary pair, first")
        assert_close(o1.logical(), 2 * want.logical(), exact=True, what="rotary pair, second")  # (doubling is exact)
    dx = DeviceView(ok.View.empty((2, 8)), device)
    dt = DeviceView(ok.View.empty((2, 3)), device)
    assert cabi.lib.fluidml_hip_rotary(dx.ref(), dt.ref(), dt.ref(), dx.ref(), 3, None) == -5  # FL_ERR_ATTR: odd
    assert cabi.lib.fluidml_hip_rotary(dx.ref(), dt.ref(), dt.ref(), dx.ref(), 4, None) == -3  # FL_ERR_SHAPE: tables


def test_elementwise_chain(device):
    """Every chain operation against the oracle's standalone kernels, applied one after the other."""
    cabi = _cabi()
    rng = np.random.default_rng(94)
    shape = (3, 17, 40)
    x = rand(rng, shape, 0.2, 3.0)  # positive: sqrt and pow stay real
    unary = {cabi.EW_ADD_C: ok.OP_ADD_C, cabi.EW_RSUB_C: ok.OP_RSUB_C, cabi.EW_MUL_C: ok.OP_MUL_C, cabi.EW_DIV_C: ok.OP_DIV_C,
             cabi.EW_POW_C: ok.OP_POW_C, cabi.EW_ERF: ok.OP_ERF, cabi.EW_RELU: ok.OP_RELU, cabi.EW_TANH: ok.OP_TANH,
             cabi.EW_SQRT: ok.OP_SQRT, cabi.EW_NEG: ok.OP_NEG}
    programs = [
        [(cabi.EW_DIV_C, 2.0), (cabi.EW_TANH, 0), (cabi.EW_ADD_C, 1.0), (cabi.EW_MUL_C, 0.5), (cabi.EW_MUL_X, 0)],  # swish
        [(cabi.EW_SQRT, 0), (cabi.EW_RSUB_C, 1.5), (cabi.EW_RELU, 0), (cabi.EW_ADD_X, 0), (cabi.EW_POW_C, 1.7), (cabi.EW_NEG, 0),
         (cabi.EW_ERF, 0), (cabi.EW_SUB_X, 0)],
        [(cabi.EW_MUL_C, 0.3), (cabi.EW_RSUB_X, 0), (cabi.EW_DIV_X, 0), (cabi.EW_ADD_C, 2.0), (cabi.EW_RDIV_X, 0)],
    ]
    for steps in programs:
        for lin, lout in [(None, None), ([2, 1, 0], [1, 0, 2])]:
            announce("elementwise chain", [s[0] for s in steps], lin, lout)
            hx = ok.View(x, lin)
            cur = hx
            for op, c in steps:
                nxt = ok.View.empty(shape)
                if op in unary:
                    ok.unary_f32(unary[op], cur, nxt, c)
                elif op in (cabi.EW_ADD_X, cabi.EW_MUL_X):
                    ok.binary_f32(ok.BOP_ADD if op == cabi.EW_ADD_X else ok.BOP_MUL, cur, hx, nxt)
                elif op in (cabi.EW_SUB_X, cabi.EW_DIV_X):
                    ok.binary_f32(ok.BOP_SUB if op == cabi.EW_SUB_X else ok.BOP_DIV, cur, hx, nxt)
                else:
                    ok.binary_f32(ok.BOP_SUB if op == cabi.EW_RSUB_X else ok.BOP_DIV, hx, cur, nxt)
                cur = nxt
            dx = DeviceView(hx, device)
            do = DeviceView(ok.View.empty(shape, np.float32, lout), device)
            chain = cabi.make_chain(steps)
            cabi.call("elementwise_chain", dx.ref(), do.ref(), ctypes.byref(chain), None)
            assert_close(do.logical(), cur.logical(), what="elementwise_chain")
    bad = cabi.make_chain([(99, 0)])
    assert cabi.lib.fluidml_hip_elementwise_chain(dx.ref(), do.ref(), ctypes.byref(bad), None) == -5  # FL_ERR_ATTR


def test_conv_and_gemm_chain(device):
    cabi = _cabi()
    rng = np.random.default_rng(95)
    swish = [(cabi.EW_DIV_C, 2.0), (cabi.EW_TANH, 0), (cabi.EW_ADD_C, 1.0), (cabi.EW_MUL_C, 0.5), (cabi.EW_MUL_X, 0)]

    def swish_ref(t):
        u = [ok.View.empty(t.shape) for _ in range(5)]
        ok.unary_f32(ok.OP_DIV_C, t, u[0], 2.0)
        ok.unary_f32(ok.OP_TANH, u[0], u[1])
        ok.unary_f32(ok.OP_ADD_C, u[1], u[2], 1.0)
        ok.unary_f32(ok.OP_MUL_C, u[2], u[3], 0.5)
        ok.binary_f32(ok.BOP_MUL, u[3], t, u[4])
        return u[4]

    # dense 3x3 (matrix cores) and depthwise 5x5 stride 2 (direct kernel)
    for xshape, wshape, pads, strides, group in [((2, 8, 20, 20), (16, 8, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((1, 6, 15, 15), (6, 1, 5, 5), [2, 2, 2, 2], [2, 2], 6)]:
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.3, 0.3), rand(rng, (wshape[0],), -1, 1)
        od = tuple((xshape[2 + d] + 2 * pads[d] - wshape[2 + d]) // strides[d] + 1 for d in range(2))
        oshape = (xshape[0], wshape[0]) + od
        hx, hw, hb, t = ok.View(x), ok.View(w), ok.View(bias), ok.View.empty(oshape)
        ok.conv(hx, hw, hb, t, pads, strides, [1, 1], group, 0)
        want = swish_ref(t)
        announce("conv chain", xshape, wshape, group)
        dx, dw, db = DeviceView(hx, device), DeviceView(hw, device), DeviceView(hb, device)
        do = DeviceView(ok.View.empty(oshape, np.float32, [0, 3, 1, 2]), device)
        chain = cabi.make_chain(swish)
        cabi.call("conv_chain", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads), cabi.i64_array(strides),
                  cabi.i64_array([1, 1]), ctypes.c_int64(group), ctypes.byref(chain), ctypes.c_uint32(0), None)
        assert_close(do.logical(), want.logical(), what="conv_chain swish")
    # Gemm -> Relu (transB, alpha = beta = 1)
    a, b, c = rand(rng, (8, 100), -1, 1), rand(rng, (50, 100), -0.05, 0.05), rand(rng, (50,), -0.2, 0.2)
    ha, hb, hc, t, want = ok.View(a), ok.View(b), ok.View(c), ok.View.empty((8, 50)), ok.View.empty((8, 50))
    ok.gemm(ha, hb, hc, t, 1.0, 1.0, 0, 1, 0)
    ok.unary_f32(ok.OP_RELU, t, want)
    announce("gemm chain")
    da, db, dc = DeviceView(ha, device), DeviceView(hb, device), DeviceView(hc, device)
    do = DeviceView(ok.View.empty((8, 50)), device)
    relu = cabi.make_chain([(cabi.EW_RELU, 0)])
    cabi.call("gemm_chain", da.ref(), db.ref(), dc.ref(), do.ref(), ctypes.c_double(1.0), ctypes.c_double(1.0), 0, 1,
              ctypes.byref(relu), ctypes.c_uint32(0), None)
    assert_close(do.logical(), want.logical(), what="gemm_chain relu")


def test_gemm_and_conv_bf16(device):
    """The opt-in path on Gemm and on convolutions that run as implicit GEMM: operands rounded to bf16, products and
    sums in fp32.  Checked to the fp32 tolerance against the oracle run on the rounded operands (bias unrounded), through
    the plain entry points (option in the upper half of `flags`) and the fused ones."""
    cabi = _cabi()
    rng = np.random.default_rng(96)
    bits = cabi.FL_CONTRACT_BF16 << cabi.FL_CONTRACT_SHIFT
    # Gemm with more than 8 rows (matrix cores); transB, alpha = beta = 1
    for M, K, N in [(64, 256, 96), (200, 1000, 130), (2048, 96, 2100)]:  # (the last: 128x128 tiles, both tiles kept k-contiguous)
        a, b, c = rand(rng, (M, K), -1, 1), rand(rng, (N, K), -0.05, 0.05), rand(rng, (N,), -0.2, 0.2)
        want, exact = ok.View.empty((M, N)), ok.View.empty((M, N))
        ok.gemm(ok.View(_round_bf16(a)), ok.View(_round_bf16(b)), ok.View(c), want, 1.0, 1.0, 0, 1, 0)
        ok.gemm(ok.View(a), ok.View(b), ok.View(c), exact, 1.0, 1.0, 0, 1, 0)
        announce("gemm bf16", M, K, N)
        da, db, dc = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device), DeviceView(ok.View(c), device)
        do = DeviceView(ok.View.empty((M, N), fill=4), device)
        cabi.call("gemm_constant_weights_bias", da.ref(), db.ref(), dc.ref(), do.ref(), ctypes.c_double(1.0), ctypes.c_double(1.0),
                  0, 1, ctypes.c_uint32(bits), None)
        assert_close(do.logical(), want.logical(), what="gemm bf16 vs oracle on bf16-rounded operands")
        assert not np.array_equal(do.logical(), exact.logical()), "the bf16 option had no effect"
        do2 = DeviceView(ok.View.empty((M, N), fill=4), device)
        none = cabi.make_chain([])
        cabi.call("gemm_chain", da.ref(), db.ref(), dc.ref(), do2.ref(), ctypes.c_double(1.0), ctypes.c_double(1.0), 0, 1,
                  ctypes.byref(none), ctypes.c_uint32(cabi.FL_CONTRACT_BF16), None)
        assert_close(do2.logical(), do.logical(), exact=True, what="gemm_chain bf16 vs gemm bf16")
        err = np.abs(do.logical().astype(np.float64) - exact.logical())
        print(f"[bf16] gemm {M}x{K}x{N}: max abs err vs fp32 {err.max():.3e}, relative to max |c| {err.max() / np.abs(exact.logical()).max():.3e}")
    # 3x3 pad 1 (gather path, 32x32 and 64x64 tiles), 1x1 (plain batched contraction), strided 3x3; depthwise ignores the option
    for xshape, wshape, pads, strides, group in [((2, 8, 20, 20), (16, 8, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((4, 12, 64, 64), (128, 12, 3, 3), [1, 1, 1, 1], [1, 1], 1),  # 12 channels: not the staged-patch kernel
                                                 ((8, 12, 64, 64), (256, 12, 3, 3), [1, 1, 1, 1], [1, 1], 1),  # the same on 128x128 tiles
                                                 # channels in chunks of 16: the staged-patch kernel with bf16 operands -- one
                                                 # pixel tile per wave, two, ragged filters, and channels split over workgroups
                                                 ((4, 32, 64, 64), (64, 32, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((8, 16, 160, 160), (64, 16, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((3, 48, 30, 62), (96, 48, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((1, 512, 28, 28), (512, 512, 3, 3), [1, 1, 1, 1], [1, 1], 1),
                                                 ((2, 24, 14, 14), (40, 24, 1, 1), [0, 0, 0, 0], [1, 1], 1),
                                                 ((1, 8, 21, 21), (12, 8, 3, 3), [1, 1, 1, 1], [2, 2], 1),
                                                 ((1, 6, 15, 15), (6, 1, 5, 5), [2, 2, 2, 2], [2, 2], 6)]:
        wmax = 0.3 if wshape[1] < 256 else 0.03  # (sums of 4608 products: keep them of order 1, like the shorter ones)
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -wmax, wmax), rand(rng, (wshape[0],), -1, 1)
        od = tuple((xshape[2 + d] + 2 * pads[d] - wshape[2 + d]) // strides[d] + 1 for d in range(2))
        oshape = (xshape[0], wshape[0]) + od
        want, exact = ok.View.empty(oshape), ok.View.empty(oshape)
        rounded = group == 1
        ok.conv(ok.View(_round_bf16(x) if rounded else x), ok.View(_round_bf16(w) if rounded else w), ok.View(bias), want, pads, strides,
                [1, 1], group, 0)
        ok.conv(ok.View(x), ok.View(w), ok.View(bias), exact, pads, strides, [1, 1], group, 0)
        announce("conv bf16", xshape, wshape, group)
        dx, dw, db = DeviceView(ok.View(x), device), DeviceView(ok.View(w), device), DeviceView(ok.View(bias), device)
        do = DeviceView(ok.View.empty(oshape, fill=4), device)
        cabi.call("conv_with_padding", dx.ref(), dw.ref(), db.ref(), do.ref(), None, 0, cabi.i64_array(pads), cabi.i64_array(strides),
                  cabi.i64_array([1, 1]), ctypes.c_int64(group), ctypes.c_uint32(bits), None)
        assert_close(do.logical(), want.logical(), what="conv bf16 vs oracle on bf16-rounded operands")
        if rounded:
            assert not np.array_equal(do.logical(), exact.logical()), "the bf16 option had no effect"
        do2 = DeviceView(ok.View.empty(oshape, fill=4), device)
        none = cabi.make_chain([])
        cabi.call("conv_chain", dx.ref(), dw.ref(), db.ref(), do2.ref(), cabi.i64_array(pads), cabi.i64_array(strides),
                  cabi.i64_array([1, 1]), ctypes.c_int64(group), ctypes.byref(none), ctypes.c_uint32(cabi.FL_CONTRACT_BF16), None)
        assert_close(do2.logical(), do.logical(), exact=True, what="conv_chain bf16 vs conv bf16")
        err = np.abs(do.logical().astype(np.float64) - exact.logical())
        print(f"[bf16] conv {xshape} * {wshape}: max abs err vs fp32 {err.max():.3e}, relative to max |out| {err.max() / np.abs(exact.logical()).max():.3e}")


def test_fused_div_add_softmax(device):
    cabi = _cabi()
    rng = np.random.default_rng(92)
    for shape, mshape, axis in [((1, 12, 128, 128), (1, 1, 1, 128), 3), ((2, 3, 9, 70), (2, 1, 9, 70), 3),
                                ((2, 17, 5), (17, 1), 1), ((4, 1500), (1500,), 1)]:
        x, mask = rand(rng, shape, -40, 40), rand(rng, mshape, -5, 0)
        for lin, lout in [(None, None), (list(range(len(shape)))[::-1], None), (None, list(range(len(shape)))[::-1])]:
            announce("fused div+add+softmax", shape, mshape, axis, lin, lout)
            hx, hm = ok.View(x, lin), ok.View(mask)
            t0, t1, ho = ok.View.empty(shape), ok.View.empty(shape), ok.View.empty(shape, np.float32, lout)
            ok.unary_f32(ok.OP_DIV_C, hx, t0, 8.0)
            ok.binary_f32(ok.BOP_ADD, t0, hm, t1)
            ok.softmax(t1, ho, axis)
            dx, dm = DeviceView(hx, device), DeviceView(hm, device)
            do = DeviceView(ok.View.empty(shape, np.float32, lout), device)
            cabi.call("div_add_softmax", dx.ref(), ctypes.c_double(8.0), dm.ref(), do.ref(), ctypes.c_int64(axis), None)
            assert_close(do.logical(), ho.logical(), what="div_add_softmax")
    # in place on the input (what the launcher does when the plan put the output over the dead input)
    x, mask = rand(rng, (1, 4, 64, 64), -40, 40), rand(rng, (1, 1, 1, 64), -5, 0)
    hx, hm = ok.View(x), ok.View(mask)
    t0, t1, ho = (ok.View.empty(x.shape) for _ in range(3))
    ok.unary_f32(ok.OP_DIV_C, hx, t0, 8.0)
    ok.binary_f32(ok.BOP_ADD, t0, hm, t1)
    ok.softmax(t1, ho, 3)
    dx, dm = DeviceView(hx, device), DeviceView(hm, device)
    announce("fused div+add+softmax in place")
    cabi.call("div_add_softmax", dx.ref(), ctypes.c_double(8.0), dm.ref(), dx.ref(), ctypes.c_int64(3), None)
    assert_close(dx.logical(), ho.logical(), what="div_add_softmax in place")


def test_fused_attention(device):
    """scores -> scale -> mask / where -> softmax -> context in one launch, against the oracle's chain of
    MatMul, Div | Mul, Add | Where, Softmax, MatMul; operands as the strided views an attention block has."""
    cabi = _cabi()
    rng = np.random.default_rng(98)
    # (batch dims, Sq, Skv, D, additive mask?, causal where?, scale is divisor?, keys stored transposed?)
    # keys stored as [.., D, Skv] with every extent a multiple of four take the kernel's 128-bit path
    cases = [((1, 12), 128, 128, 64, True, False, True, True), ((2, 3), 40, 40, 16, True, False, True, False),
             ((1, 4), 200, 200, 64, False, True, False, True), ((3,), 33, 70, 32, False, False, True, True),
             ((1, 2), 256, 256, 64, True, True, False, False), ((2, 2), 24, 36, 48, True, True, True, True),
             ((1, 1), 5, 3, 7, True, False, False, False)]
    for bdims, sq, skv, d, use_mask, use_where, divisor, kt_stored in cases:
        q = rand(rng, bdims + (sq, d), -1, 1)
        k = rand(rng, bdims + (skv, d), -1, 1)
        v = rand(rng, bdims + (skv, d), -1, 1)
        scale = float(np.sqrt(d)) if divisor else float(1.0 / np.sqrt(d))
        mask = rand(rng, (1,) * len(bdims) + (1, skv), -8, 0) if use_mask else None
        cond = np.tril(np.ones((sq, skv), np.bool_))[(None,) * len(bdims)] if use_where else None
        fill = float(np.finfo(np.float32).min)
        # oracle chain
        kt = np.ascontiguousarray(np.swapaxes(k, -1, -2))
        s0 = ok.View.empty(bdims + (sq, skv))
        ok.matmul(ok.View(q), ok.View(kt), s0)
        s1 = ok.View.empty(s0.shape)
        ok.unary_f32(ok.OP_DIV_C if divisor else ok.OP_MUL_C, s0, s1, scale)
        if use_mask:
            s2 = ok.View.empty(s0.shape)
            ok.binary_f32(ok.BOP_ADD, s1, ok.View(mask), s2)
            s1 = s2
        if use_where:
            s2 = ok.View.empty(s0.shape)
            ok.where(ok.View(cond), s1, None, fill, s2)
            s1 = s2
        p = ok.View.empty(s0.shape)
        ok.softmax(s1, p, len(s0.shape) - 1)
        want = ok.View.empty(bdims + (sq, d))
        ok.matmul(p, ok.View(v), want)
        announce("fused attention", bdims, sq, skv, d, use_mask, use_where, divisor, kt_stored)
        dq, dv = DeviceView(ok.View(q), device), DeviceView(ok.View(v), device)
        rank = len(bdims) + 2
        if kt_stored:
            dk = DeviceView(ok.View(kt), device)
            ktv = dk.tensor
        else:  # keys as the projection wrote them, [.., Skv, D]; the kernel sees K^T as a strided view
            dk = DeviceView(ok.View(k), device)
            kst = list(dk.tensor.strides[:rank])
            ktv = cabi.make_tensor(dk.tensor.base, cabi.FL_FLOAT32, list(bdims) + [d, skv], kst[:-2] + [kst[-1], kst[-2]])
        # output stored head-merged: [.., Sq, heads * D] like the Transpose + Reshape after the context matmul
        lo = None if len(bdims) < 2 else list(range(len(bdims) - 1)) + [len(bdims), len(bdims) - 1, len(bdims) + 1]
        do = DeviceView(ok.View.empty(bdims + (sq, d), np.float32, lo, fill=3), device)
        dm = DeviceView(ok.View(mask), device) if use_mask else None
        dc = DeviceView(ok.View(cond), device) if use_where else None
        cabi.call("attention", dq.ref(), ctypes.byref(ktv), dv.ref(), do.ref(), ctypes.c_double(scale), int(divisor),
                  dm.ref() if dm else None, dc.ref() if dc else None, ctypes.c_double(fill), None)
        assert_close(do.logical(), want.logical(), what="attention")
    big = DeviceView(ok.View.empty((1, 1, 8, 128)), device)
    assert cabi.lib.fluidml_hip_attention(big.ref(), big.ref(), big.ref(), big.ref(), 1.0, 1, None, None, 0.0, None) != 0


def test_fused_add_layer_norm(device):
    cabi = _cabi()
    rng = np.random.default_rng(93)
    for shape, axis, eps in [((1, 128, 768), 2, 1e-12), ((2, 7, 33), 2, 1e-5), ((3, 20, 5), 1, 1e-5), ((2, 5000), 1, 1e-5)]:
        x, y = rand(rng, shape, -3, 3), rand(rng, shape, -3, 3)
        g, b = rand(rng, shape[axis:], 0.5, 1.5), rand(rng, shape[axis:], -0.5, 0.5)
        for lx, ly, lo in [(None, None, None), (list(range(len(shape)))[::-1], None, None),
                           (None, list(range(len(shape)))[::-1], list(range(len(shape)))[::-1])]:
            announce("fused add+layer_norm", shape, axis, lx, ly, lo)
            hx, hy, hg, hb = ok.View(x, lx), ok.View(y, ly), ok.View(g), ok.View(b)
            t0, ho = ok.View.empty(shape), ok.View.empty(shape, np.float32, lo)
            ok.binary_f32(ok.BOP_ADD, hx, hy, t0)
            ok.layer_norm(t0, hg, hb, ho, axis, eps)
            dx, dy, dg, db = (DeviceView(h, device) for h in (hx, hy, hg, hb))
            do = DeviceView(ok.View.empty(shape, np.float32, lo), device)
            cabi.call("add_layer_normalization", dx.ref(), dy.ref(), dg.ref(), db.ref(), do.ref(), ctypes.c_int64(axis),
                      ctypes.c_double(eps), None)
            assert_close(do.logical(), ho.logical(), what="add_layer_normalization")


def test_gather_with_row_statistics(device):
    """The lookup that also leaves the partial row statistics of its result (mean and sum of squared deviations of
    every run of 32 columns): rows bit-identical to the oracle's Gather, statistics against float64."""
    import torch

    cabi = _cabi()
    rng = np.random.default_rng(223)
    for lead, length, rows in [((1, 256), 512, 1000), ((3, 5), 33, 17), ((7,), 300, 9), ((2, 2), 1056, 6)]:
        announce("gather_constant_data_tensor_stats", lead, length, rows)
        table = rand(rng, (rows, length), -2, 2)
        ids = rng.integers(0, rows, size=lead).astype(np.int64)
        hi, ht, want = ok.View(ids), ok.View(table), ok.View.empty(lead + (length,))
        ok.gather_data_tensor(hi, ht, want)
        di, dt = DeviceView(hi, device), DeviceView(ht, device)
        do = DeviceView(ok.View.empty(lead + (length,), np.float32, None, fill=5), device)
        n_rows, parts = int(np.prod(lead)), (length + 31) // 32
        stats = torch.full((n_rows, parts, 2), 7.0, dtype=torch.float32, device=device)
        cabi.call("gather_constant_data_tensor_stats", di.ref(), dt.ref(), do.ref(), ctypes.c_void_p(stats.data_ptr()), None)
        assert_close(do.logical(), want.logical(), exact=True, what="gather with statistics: rows")
        got = stats.cpu().numpy()
        x = want.logical().reshape(n_rows, length).astype(np.float64)
        for j in range(parts):
            run = x[:, 32 * j:32 * (j + 1)]
            np.testing.assert_allclose(got[:, j, 0], run.mean(axis=1), rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(got[:, j, 1], ((run - run.mean(axis=1, keepdims=True)) ** 2).sum(axis=1), rtol=1e-4, atol=1e-5)


def test_gather_add_layer_norm(device):
    """The embedding block as one launch against the oracle's separate Gather, Add, Add and LayerNormalization: with
    one table or two, a second addend or none, addends that repeat along the leading dims."""
    cabi = _cabi()
    rng = np.random.default_rng(211)
    for lead, length, rows0, rows1, eps in [((1, 128), 768, 1000, 2, 1e-12), ((3, 5), 33, 17, 4, 1e-5), ((7,), 2048, 9, 3, 1e-5),
                                             ((2, 6), 300, 50, 5, 1e-5)]:
        shape = lead + (length,)
        t0, t1 = rand(rng, (rows0, length), -1, 1), rand(rng, (rows1, length), -1, 1)
        i0 = rng.integers(0, rows0, size=lead).astype(np.int64)
        i1 = rng.integers(0, rows1, size=lead).astype(np.int64)
        g, b = rand(rng, (length,), 0.5, 1.5), rand(rng, (length,), -0.5, 0.5)
        full = rand(rng, shape, -1, 1)
        repeated = rand(rng, (1,) * (len(lead) - 1) + lead[-1:] + (length,), -1, 1)  # like a position embedding
        hi0, hi1, ht0, ht1, hg, hb = (ok.View(v) for v in (i0, i1, t0, t1, g, b))
        di0, di1, dt0, dt1, dg, db = (DeviceView(h, device) for h in (hi0, hi1, ht0, ht1, hg, hb))
        for two_tables in (True, False):
            for third in (None, full, repeated):
                announce("gather_add_layer_normalization", shape, two_tables, None if third is None else third.shape)
                first, second = ok.View.empty(shape), ok.View.empty(shape)
                ok.gather_data_tensor(hi0, ht0, first)
                if two_tables:
                    ok.gather_data_tensor(hi1, ht1, second)
                else:
                    second = ok.View(repeated if third is full else full)
                summed = ok.View.empty(shape)
                ok.binary_f32(ok.BOP_ADD, first, second, summed)
                if third is not None:
                    both = ok.View.empty(shape)
                    ok.binary_f32(ok.BOP_ADD, summed, ok.View(third), both)
                    summed = both
                want = ok.View.empty(shape)
                ok.layer_norm(summed, hg, hb, want, len(shape) - 1, eps)
                dsecond = dt1 if two_tables else DeviceView(second, device)
                dthird = None if third is None else DeviceView(ok.View(third), device)
                do = DeviceView(ok.View.empty(shape, np.float32, None, fill=5), device)
                cabi.call("gather_add_layer_normalization", di0.ref(), dt0.ref(), di1.ref() if two_tables else None,
                          dsecond.ref(), dthird.ref() if dthird else None, dg.ref(), db.ref(), do.ref(),
                          ctypes.c_double(eps), None)
                assert_close(do.logical(), want.logical(), what="gather_add_layer_normalization")
    # refused, nothing launched: a row longer than the kernel keeps in registers, an addend that repeats along the row
    long_t = DeviceView(ok.View(rand(rng, (4, 4096), -1, 1)), device)
    ids = DeviceView(ok.View(np.zeros((2,), np.int64)), device)
    vec = DeviceView(ok.View(rand(rng, (4096,), -1, 1)), device)
    out = DeviceView(ok.View.empty((2, 4096)), device)
    assert cabi.lib.fluidml_hip_gather_add_layer_normalization(ids.ref(), long_t.ref(), None, out.ref(), None, vec.ref(),
                                                               vec.ref(), out.ref(), 1e-5, None) == cabi.FL_ERR_UNSUPPORTED
    small_t = DeviceView(ok.View(rand(rng, (4, 8), -1, 1)), device)
    col = DeviceView(ok.View(rand(rng, (2, 1), -1, 1)), device)
    v8 = DeviceView(ok.View(rand(rng, (8,), -1, 1)), device)
    out8 = DeviceView(ok.View.empty((2, 8)), device)
    assert cabi.lib.fluidml_hip_gather_add_layer_normalization(ids.ref(), small_t.ref(), None, col.ref(), None, v8.ref(),
                                                               v8.ref(), out8.ref(), 1e-5, None) == cabi.FL_ERR_UNSUPPORTED


@pytest.mark.parametrize("M,H,K0,N1", [(128, 256, 128, 384), (100, 200, 96, 72), (33, 768, 256, 768)], ids=str)
def test_matmul_with_deferred_layer_norm(device, M, H, K0, N1):
    """A LayerNormalization that never reaches memory (fluidml_hip_matmul_chain_group_norm) against the oracle's
    MatMul -> Add -> Add -> LayerNormalization -> MatMul chain.  Three calls: (1) the contraction that produces the
    residual sum s leaves the partial row statistics of s beside it; (2) a grouped pair of projections reads s as if
    it were LayerNorm(s) (scale folded into the weights, per-row mean and rstd applied in the epilogue); (3) a
    contraction adds LayerNorm(s) as its residual and leaves the statistics of its own result.  Widths with a
    ragged last run of 32 columns, rows that do not fill the tiles, and every tile configuration the flags name."""
    import torch

    cabi = _cabi()
    rng = np.random.default_rng(M + H)
    eps = 1e-5
    a0, w0, b0 = rand(rng, (1, M, K0), -1, 1), rand(rng, (K0, H), -0.3, 0.3), rand(rng, (H,), -0.5, 0.5)
    x = rand(rng, (1, M, H), -2, 2) + 0.75  # rows with a mean well away from zero
    gamma, beta = rand(rng, (H,), 0.5, 1.5), rand(rng, (H,), -0.5, 0.5)
    w1 = [rand(rng, (H, N1), -0.2, 0.2) for _ in range(2)]
    b1 = [rand(rng, (N1,), -0.5, 0.5) for _ in range(2)]
    a2, w2, b2 = rand(rng, (1, M, K0), -1, 1), rand(rng, (K0, H), -0.3, 0.3), rand(rng, (H,), -0.5, 0.5)

    # the oracle's unfused chain
    def V(shape):
        return ok.View.empty(shape)

    t, t1, s_ref, h_ref = V((1, M, H)), V((1, M, H)), V((1, M, H)), V((1, M, H))
    ok.matmul(ok.View(a0), ok.View(w0), t)
    ok.binary_f32(ok.BOP_ADD, ok.View(b0), t, t1)
    ok.binary_f32(ok.BOP_ADD, t1, ok.View(x), s_ref)
    ok.layer_norm(s_ref, ok.View(gamma), ok.View(beta), h_ref, 2, eps)
    x2 = rand(rng, (1, M, H), -1, 1)
    s3_ref = V((1, M, H))
    ok.binary_f32(ok.BOP_ADD, s_ref, ok.View(x2), s3_ref)
    z_ref = []
    for w, b in zip(w1, b1):
        z0, z = V((1, M, N1)), V((1, M, N1))
        ok.matmul(h_ref, ok.View(w), z0)
        ok.binary_f32(ok.BOP_ADD, ok.View(b), z0, z)
        z_ref.append(z.logical())
    u0, u1, u_ref = V((1, M, H)), V((1, M, H)), V((1, M, H))
    ok.matmul(ok.View(a2), ok.View(w2), u0)
    ok.binary_f32(ok.BOP_ADD, ok.View(b2), u0, u1)
    ok.binary_f32(ok.BOP_ADD, u1, h_ref, u_ref)

    parts = (H + 31) // 32
    ptr = ctypes.POINTER(cabi.FlTensor)

    def dev(arr):
        return DeviceView(ok.View(np.ascontiguousarray(arr, dtype=np.float32)), device)

    def one(v):
        return (ptr * 1)(ctypes.pointer(v.tensor))

    def partial_stats(rows):
        want = np.zeros((rows.shape[0], parts, 2))
        for j in range(parts):
            run = rows[:, 32 * j:32 * j + 32].astype(np.float64)
            want[:, j, 0] = run.mean(axis=1)
            want[:, j, 1] = ((run - run.mean(axis=1, keepdims=True)) ** 2).sum(axis=1)
        return want

    da0, dw0, db0, dx, dx2 = dev(a0), dev(w0), dev(b0), dev(x), dev(x2)
    dgamma, dbeta = dev(gamma), dev(beta)
    # what a caller folds at compile time: scale into the weights, their column sums, shift . W + bias
    dw1 = [dev(gamma[:, None] * w) for w in w1]
    dc1 = [dev((gamma[:, None].astype(np.float64) * w).sum(axis=0)) for w in w1]
    dc2 = [dev(beta.astype(np.float64) @ w.astype(np.float64) + b) for w, b in zip(w1, b1)]
    da2, dw2, db2 = dev(a2), dev(w2), dev(b2)
    for tile in range(0, 9):
        flags = ctypes.c_uint32(tile << 4)
        ds = DeviceView(ok.View.empty((1, M, H), np.float32, None, fill=3), device)
        stats = torch.full((M, parts, 2), 7.0, device=device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.stats_out = cabi.FL_NORM_NONE, stats.data_ptr()
        announce("deferred layer norm: producer", (M, H, K0), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, da0.ref(), one(dw0), one(db0), None, one(ds), 0, None, None, dx.ref(),
                                                          ctypes.byref(norm), flags, None)
        if rc == -8:
            assert tile >= 3  # the rule and the register-staged tiles take every operand
            continue
        assert rc == 0, cabi.error_string(rc)
        s_got = ds.logical()
        assert_close(s_got, s_ref.logical(), what=f"residual sum, tile {tile}")
        got_stats = stats.cpu().numpy().astype(np.float64)
        want_stats = partial_stats(s_got[0])
        assert np.allclose(got_stats[..., 0], want_stats[..., 0], rtol=1e-5, atol=1e-6), "partial means"
        assert np.allclose(got_stats[..., 1], want_stats[..., 1], rtol=1e-4, atol=1e-5), "partial sums of squared deviations"

        # the same producer with a second plain addend (a parallel residual: x + attention + mlp)
        ds3 = DeviceView(ok.View.empty((1, M, H), np.float32, None, fill=3), device)
        stats3 = torch.full((M, parts, 2), 7.0, device=device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.stats_out, norm.addend2 = cabi.FL_NORM_NONE, stats3.data_ptr(), ctypes.pointer(dx2.tensor)
        announce("deferred layer norm: producer with two addends", (M, H, K0), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, da0.ref(), one(dw0), one(db0), None, one(ds3), 0, None, None, dx.ref(),
                                                          ctypes.byref(norm), flags, None)
        assert rc == 0, cabi.error_string(rc)
        assert_close(ds3.logical(), s3_ref.logical(), what=f"residual sum of two addends, tile {tile}")
        want3 = partial_stats(ds3.logical()[0])
        got3 = stats3.cpu().numpy().astype(np.float64)
        assert np.allclose(got3[..., 0], want3[..., 0], rtol=1e-5, atol=1e-6) and np.allclose(got3[..., 1], want3[..., 1], rtol=1e-4, atol=1e-5)

        douts = [DeviceView(ok.View.empty((1, M, N1), np.float32, None, fill=3), device) for _ in range(2)]
        norm = cabi.FlNormFusion()
        norm.deferred, norm.width, norm.epsilon, norm.stats = cabi.FL_NORM_LHS, H, eps, stats.data_ptr()
        rhs = (ptr * 2)(*[ctypes.pointer(d.tensor) for d in dw1])
        bias = (ptr * 2)(*[ctypes.pointer(d.tensor) for d in dc2])
        csum = (ptr * 2)(*[ctypes.pointer(d.tensor) for d in dc1])
        outs = (ptr * 2)(*[ctypes.pointer(d.tensor) for d in douts])
        announce("deferred layer norm: normalised left operand, two projections", (M, H, N1), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(2, ds.ref(), rhs, bias, csum, outs, 0, None, None, None,
                                                          ctypes.byref(norm), flags, None)
        if rc == -8:
            assert tile >= 3
        else:
            assert rc == 0, cabi.error_string(rc)
            for d, want in zip(douts, z_ref):
                assert_close(d.logical(), want, what=f"projection of the deferred LayerNorm, tile {tile}")

        du = DeviceView(ok.View.empty((1, M, H), np.float32, None, fill=3), device)
        stats2 = torch.full((M, parts, 2), 7.0, device=device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.width, norm.epsilon, norm.stats = cabi.FL_NORM_ADDEND, H, eps, stats.data_ptr()
        norm.scale, norm.shift = ctypes.pointer(dgamma.tensor), ctypes.pointer(dbeta.tensor)
        norm.stats_out = stats2.data_ptr()
        announce("deferred layer norm: normalised residual", (M, K0, H), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, da2.ref(), one(dw2), one(db2), None, one(du), 0, None, None, ds.ref(),
                                                          ctypes.byref(norm), flags, None)
        if rc == -8:
            assert tile >= 3
            continue
        assert rc == 0, cabi.error_string(rc)
        assert_close(du.logical(), u_ref.logical(), what=f"contraction + deferred LayerNorm residual, tile {tile}")
        want2 = partial_stats(du.logical()[0])
        got2 = stats2.cpu().numpy().astype(np.float64)
        assert np.allclose(got2[..., 0], want2[..., 0], rtol=1e-5, atol=1e-6) and np.allclose(got2[..., 1], want2[..., 1], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("M,H,K0,N1", [(128, 256, 128, 384), (33, 768, 256, 768), (300, 512, 128, 4096)], ids=str)
def test_matmul_with_deferred_layer_norm_bf16(device, M, H, K0, N1):
    """The three forms of fluidml_hip_matmul_chain_group_norm with FL_CONTRACT_BF16: both operands of the contraction
    are rounded to bf16 on their way into LDS (the un-normalised sum and the pre-scaled weights where the left operand
    carries the deferred LayerNormalization), everything else -- accumulation, row statistics, the epilogue's
    correction, the residual's normalisation -- stays fp32.  Expected values: the same formulas in float64 on the
    rounded operands.  The rule's tile, the 64x64 tile and, where the rows fit its two lanes per row, the 128x128 one."""
    import torch

    cabi = _cabi()
    rng = np.random.default_rng(M + H + 1)
    eps = 1e-5
    a0, w0, b0 = rand(rng, (1, M, K0), -1, 1), rand(rng, (K0, H), -0.3, 0.3), rand(rng, (H,), -0.5, 0.5)
    x = rand(rng, (1, M, H), -2, 2) + 0.75
    gamma, beta = rand(rng, (H,), 0.5, 1.5), rand(rng, (H,), -0.5, 0.5)
    w1, b1 = rand(rng, (H, N1), -0.2, 0.2), rand(rng, (N1,), -0.5, 0.5)
    a2, w2, b2 = rand(rng, (1, M, K0), -1, 1), rand(rng, (K0, H), -0.3, 0.3), rand(rng, (H,), -0.5, 0.5)
    parts = (H + 31) // 32
    ptr = ctypes.POINTER(cabi.FlTensor)
    f64 = np.float64

    def dev(arr):
        return DeviceView(ok.View(np.ascontiguousarray(arr, dtype=np.float32)), device)

    def one(v):
        return (ptr * 1)(ctypes.pointer(v.tensor))

    r = _round_bf16
    s_want = (r(a0[0]).astype(f64) @ r(w0).astype(f64) + b0 + x[0]).astype(np.float32)
    da0, dw0, db0, dx = dev(a0), dev(w0), dev(b0), dev(x)
    gw = (gamma[:, None] * w1).astype(np.float32)
    dw1, dc1 = dev(gw), dev(gw.astype(f64).sum(axis=0))
    dc2 = dev(beta.astype(f64) @ w1.astype(f64) + b1)
    dgamma, dbeta, da2, dw2, db2 = dev(gamma), dev(beta), dev(a2), dev(w2), dev(b2)
    for tile in (0, 2, 8):
        flags = ctypes.c_uint32(cabi.FL_CONTRACT_BF16 | tile << 4)
        ds = DeviceView(ok.View.empty((1, M, H), np.float32, None, fill=3), device)
        stats = torch.full((M, parts, 2), 7.0, device=device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.stats_out = cabi.FL_NORM_NONE, stats.data_ptr()
        announce("deferred layer norm, bf16 operands: producer", (M, H, K0), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, da0.ref(), one(dw0), one(db0), None, one(ds), 0, None, None, dx.ref(),
                                                          ctypes.byref(norm), flags, None)
        assert rc == 0, cabi.error_string(rc)
        s_got = ds.logical()[0]
        assert_close(s_got, s_want, what=f"bf16 residual sum, tile {tile}")
        # row statistics of what was written
        mean = s_got.astype(f64).mean(axis=1, keepdims=True)
        rstd = 1.0 / np.sqrt(((s_got.astype(f64) - mean) ** 2).mean(axis=1, keepdims=True) + eps)

        dz = DeviceView(ok.View.empty((1, M, N1), np.float32, None, fill=3), device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.width, norm.epsilon, norm.stats = cabi.FL_NORM_LHS, H, eps, stats.data_ptr()
        announce("deferred layer norm, bf16 operands: normalised left operand", (M, H, N1), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, ds.ref(), one(dw1), one(dc2), one(dc1), one(dz), 0, None, None, None,
                                                          ctypes.byref(norm), flags, None)
        if tile == 8 and H > 512:
            assert rc == cabi.FL_ERR_UNSUPPORTED  # two lanes per row merge at most 16 partials
        else:
            assert rc == 0, cabi.error_string(rc)
            acc = r(s_got).astype(f64) @ r(gw).astype(f64)
            z_want = rstd * (acc - mean * dc1.logical().astype(f64)) + dc2.logical().astype(f64)
            np.testing.assert_allclose(dz.logical()[0], z_want, rtol=2e-4, atol=2e-4, err_msg=f"bf16 projection of the deferred LayerNorm, tile {tile}")

        du = DeviceView(ok.View.empty((1, M, H), np.float32, None, fill=3), device)
        norm = cabi.FlNormFusion()
        norm.deferred, norm.width, norm.epsilon, norm.stats = cabi.FL_NORM_ADDEND, H, eps, stats.data_ptr()
        norm.scale, norm.shift = ctypes.pointer(dgamma.tensor), ctypes.pointer(dbeta.tensor)
        announce("deferred layer norm, bf16 operands: normalised residual", (M, K0, H), "tile", tile)
        rc = cabi.lib.fluidml_hip_matmul_chain_group_norm(1, da2.ref(), one(dw2), one(db2), None, one(du), 0, None, None, ds.ref(),
                                                          ctypes.byref(norm), flags, None)
        if tile == 8 and H > 512:
            assert rc == cabi.FL_ERR_UNSUPPORTED
            continue
        assert rc == 0, cabi.error_string(rc)
        h = (s_got.astype(f64) - mean) * rstd * gamma + beta
        u_want = r(a2[0]).astype(f64) @ r(w2).astype(f64) + b2 + h
        np.testing.assert_allclose(du.logical()[0], u_want, rtol=1e-4, atol=1e-4, err_msg=f"bf16 contraction + deferred LayerNorm residual, tile {tile}")


CONV_CASES = [
    # x shape, w shape, pads, strides, dilations, group, bias
    ((1, 768, 128), (768, 1, 9), [4, 4], [1], [1], 768, False),  # reference conv0.py (depthwise 1-d, pad 4)
    ((1, 768, 128), (384, 768, 1), None, [1], [1], 1, True),  # reference conv1.py (pointwise + bias)
    ((1, 3, 34, 34), (8, 3, 3, 3), [1, 1, 1, 1], [1, 1], [1, 1], 1, True),  # VGG-style 3x3 pad 1
    ((2, 4, 19, 17), (6, 4, 3, 5), [1, 2, 1, 2], [2, 2], [1, 1], 1, True),  # stride 2
    ((1, 6, 15, 15), (6, 1, 5, 5), [2, 2, 2, 2], [2, 2], [1, 1], 6, True),  # depthwise 5x5 stride 2
    ((1, 2, 12, 12), (3, 2, 3, 3), [2, 2, 2, 2], [1, 1], [2, 2], 1, False),  # dilation 2
    ((2, 24, 14, 14), (40, 24, 1, 1), None, [1, 1], [1, 1], 1, True),  # pointwise 2-d, two images (plain contraction)
    ((1, 8, 12, 12), (16, 8, 1, 1), None, [2, 2], [1, 1], 1, True),  # pointwise with stride 2 (gather path)
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: str(c[:2]))
def test_conv(device, case):
    cabi = _cabi()
    xshape, wshape, pads, strides, dilations, group, with_bias = case
    rng = np.random.default_rng(seed_of(xshape, wshape))
    x, w = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.05, 0.05)
    bias = rand(rng, (wshape[0],), -1, 1) if with_bias else None
    ns = len(xshape) - 2
    p = pads if pads is not None else [0] * (2 * ns)

    def out_dims(st, di):
        return tuple((xshape[2 + d] + p[d] + p[d + ns] - di[d] * (wshape[2 + d] - 1) - 1) // st[d] + 1 for d in range(ns))

    for flags in (0, cabi.FL_REF_CONV_UNIT_STRIDE | (cabi.FL_REF_CONV_BIAS_INDEX1 if with_bias else 0)):
        # the output shape comes from the graph's value_info (ONNX semantics) in both modes
        oshape = (xshape[0], wshape[0]) + out_dims(strides, dilations)
        for lx in some_layouts(len(xshape), rng, 2):
            for lo in some_layouts(len(xshape), rng, 2):
                announce("conv", case[:2], flags, lx, lo)
                hx, hw, ho = ok.View(x, lx), ok.View(w), ok.View.empty(oshape, np.float32, lo)
                hb = ok.View(bias) if with_bias else None
                ok.conv(hx, hw, hb, ho, pads, strides, dilations, group, flags)
                dx, dw = DeviceView(hx, device), DeviceView(hw, device)
                db = DeviceView(hb, device) if with_bias else None
                do = DeviceView(ok.View.empty(oshape, np.float32, lo), device)
                bref = db.ref() if with_bias else None
                if pads is None:
                    cabi.call("conv_without_padding", dx.ref(), dw.ref(), bref, do.ref(), cabi.i64_array(strides),
                              cabi.i64_array(dilations), ctypes.c_int64(group), ctypes.c_uint32(flags), None)
                else:
                    cabi.call("conv_with_padding", dx.ref(), dw.ref(), bref, do.ref(), None, 0, cabi.i64_array(pads),
                              cabi.i64_array(strides), cabi.i64_array(dilations), ctypes.c_int64(group),
                              ctypes.c_uint32(flags), None)
                assert_close(do.logical(), ho.logical(), what=f"conv flags={flags}")


def test_conv_large_tiles(device):
    """Shapes that select the 64x64 and 128x128 workgroup tiles of the implicit-GEMM path, and a weight
    tensor whose layout is not (c, kh, kw)-contiguous, which has to take the direct kernel."""
    cabi = _cabi()
    rng = np.random.default_rng(79)
    for xshape, wshape, lw in [((2, 8, 64, 64), (128, 8, 3, 3), None), ((4, 8, 64, 64), (256, 8, 3, 3), None),
                               ((1, 8, 20, 20), (16, 8, 3, 3), [3, 2, 1, 0])]:
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.05, 0.05), rand(rng, (wshape[0],), -1, 1)
        oshape = (xshape[0], wshape[0]) + xshape[2:]
        for lx, lo in [(None, None), ([0, 3, 1, 2], [0, 3, 1, 2])]:  # NCHW and channels-last storage
            announce("conv large", xshape, wshape, lx, lo, lw)
            hx, hw, hb, ho = ok.View(x, lx), ok.View(w, lw), ok.View(bias), ok.View.empty(oshape, np.float32, lo)
            ok.conv(hx, hw, hb, ho, [1, 1, 1, 1], [1, 1], [1, 1], 1, 0)
            dx, dw, db = DeviceView(hx, device), DeviceView(hw, device), DeviceView(hb, device)
            do = DeviceView(ok.View.empty(oshape, np.float32, lo), device)
            cabi.call("conv_with_padding", dx.ref(), dw.ref(), db.ref(), do.ref(), None, 0, cabi.i64_array([1, 1, 1, 1]),
                      cabi.i64_array([1, 1]), cabi.i64_array([1, 1]), ctypes.c_int64(1), ctypes.c_uint32(0), None)
            assert_close(do.logical(), ho.logical(), what="conv large")


def test_conv_staged_patch(device):
    """3x3 unit-stride convolutions that take the kernel with the input patch staged in LDS: one and two pixel tiles per
    wave, image extents that leave the last tiles ragged, a filter count that leaves the last filter tile half empty,
    no padding, channels-last output, bias and a ReLU chain, fewer than eight input channels, input channels split
    over several workgroups per tile."""
    cabi = _cabi()
    rng = np.random.default_rng(83)
    relu = cabi.make_chain([(cabi.EW_RELU, 0)])
    for xshape, filters, pads, lo, with_chain in [((8, 8, 96, 150), 96, [1, 1, 1, 1], None, True),     # two tiles per wave
                                                  ((3, 16, 30, 62), 160, [1, 1, 1, 1], [0, 3, 1, 2], False),  # ragged rows
                                                  ((2, 8, 66, 66), 128, [0, 0, 0, 0], None, True),     # no padding
                                                  ((4, 3, 64, 80), 64, [1, 1, 1, 1], None, True),      # three channels, two tiles per wave
                                                  ((2, 5, 33, 70), 40, [1, 1, 1, 1], None, False),     # five channels, ragged
                                                  # few tiles: the input channels split over workgroups (8, 4 and 2 ways, the last uneven)
                                                  ((1, 512, 14, 14), 512, [1, 1, 1, 1], None, True),
                                                  ((1, 256, 28, 28), 256, [1, 1, 1, 1], None, False),
                                                  ((2, 136, 24, 40), 192, [1, 1, 1, 1], None, True)]:
        wshape = (filters, xshape[1], 3, 3)
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.1, 0.1), rand(rng, (filters,), -1, 1)
        oh, ow = xshape[2] + 2 * pads[0] - 2, xshape[3] + 2 * pads[1] - 2
        oshape = (xshape[0], filters, oh, ow)
        announce("conv staged patch", xshape, wshape, pads, lo)
        hx, hw, hb, ho = ok.View(x), ok.View(w), ok.View(bias), ok.View.empty(oshape, np.float32, lo)
        ok.conv(hx, hw, hb, ho, pads if any(pads) else None, [1, 1], [1, 1], 1, 0)
        want = ho
        if with_chain:
            want = ok.View.empty(oshape, np.float32, lo)
            ok.unary_f32(ok.OP_RELU, ho, want)
        dx, dw, db = DeviceView(hx, device), DeviceView(hw, device), DeviceView(hb, device)
        do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
        none = cabi.make_chain([])
        cabi.call("conv_chain", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads), cabi.i64_array([1, 1]),
                  cabi.i64_array([1, 1]), ctypes.c_int64(1), ctypes.byref(relu if with_chain else none), ctypes.c_uint32(0), None)
        assert_close(do.logical(), want.logical(), what="conv with staged patch")
        # (partial tiles of split channels are added in split order whichever workgroup arrives last: every run the same bits)
        first = do.logical().copy()
        for _ in range(3):
            cabi.call("conv_chain", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads), cabi.i64_array([1, 1]),
                      cabi.i64_array([1, 1]), ctypes.c_int64(1), ctypes.byref(relu if with_chain else none), ctypes.c_uint32(0), None)
            assert np.array_equal(do.logical(), first), "conv with staged patch: runs differ"


def test_conv_paths_against_their_fallbacks(device, monkeypatch):
    """The specialised convolution kernels against the kernels behind them, on the same inputs: the 3x3 kernel with the
    input patch staged in LDS against the implicit GEMM (FLUIDML_CONV_HALO=0), and the depthwise kernel that owns a
    channel plane per workgroup against the direct kernel (FLUIDML_CONV_PLANE=0).  The switches are read at every call,
    so both sides run inside this process; each side has to meet the oracle, and the two sides each other."""
    cabi = _cabi()
    rng = np.random.default_rng(97)
    none = cabi.make_chain([])
    cases = [("FLUIDML_CONV_HALO", (2, 64, 28, 28), 96, 1, 3), ("FLUIDML_CONV_HALO", (1, 128, 14, 14), 128, 1, 3),
             ("FLUIDML_CONV_PLANE", (1, 96, 28, 28), 96, 96, 3), ("FLUIDML_CONV_PLANE", (2, 40, 31, 29), 40, 40, 5)]
    for switch, xshape, filters, group, k in cases:
        wshape = (filters, xshape[1] // group, k, k)
        pads = [k // 2] * 4
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.1, 0.1), rand(rng, (filters,), -1, 1)
        oshape = (xshape[0], filters, xshape[2], xshape[3])
        hx, hw, hb, ho = ok.View(x), ok.View(w), ok.View(bias), ok.View.empty(oshape)
        ok.conv(hx, hw, hb, ho, pads, [1, 1], [1, 1], group, 0)
        dx, dw, db = DeviceView(hx, device), DeviceView(hw, device), DeviceView(hb, device)
        got = {}
        for value in ("1", "0"):
            announce("conv path", switch, value, xshape, wshape)
            monkeypatch.setenv(switch, value)
            do = DeviceView(ok.View.empty(oshape, np.float32, None, fill=7), device)
            cabi.call("conv_chain", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads), cabi.i64_array([1, 1]),
                      cabi.i64_array([1, 1]), ctypes.c_int64(group), ctypes.byref(none), ctypes.c_uint32(0), None)
            got[value] = do.logical().copy()
            assert_close(got[value], ho.logical(), what=f"conv with {switch}={value}")
        monkeypatch.delenv(switch)
        assert_close(got["1"], got["0"], what=f"conv, {switch} on against off")
        if group > 1:  # the plane kernel folds the window in the direct kernel's order: the same bits
            assert np.array_equal(got["1"], got["0"]) or np.allclose(got["1"], got["0"], rtol=1e-6, atol=1e-7)


def test_conv_scale_add(device):
    """MulCommon (one factor per channel) -> Conv -> chain -> AddCommon (tensor of the output's shape) as one launch, against
    the oracle's four kernels: pointwise convolutions on both tile sizes with the gate, the skip connection or both,
    two images, a 1-d convolution."""
    cabi = _cabi()
    rng = np.random.default_rng(97)
    relu = cabi.make_chain([(cabi.EW_RELU, 0)])
    none = cabi.make_chain([])
    cases = [((1, 96, 28, 28), 40, 1, True, True, False, None),      # small tile, gate and skip connection
             ((1, 240, 56, 56), 80, 1, True, False, True, None),     # 64x64 tile, gate, ReLU
             ((1, 37, 9, 11), 50, 1, True, True, False, None),       # ragged extents, scalar loads
             ((2, 64, 20, 20), 64, 1, False, True, True, None),      # two images, skip connection
             ((1, 1152, 7, 7), 192, 1, True, True, False, None)]     # 49 pixels: wide loads for the weights alone
    for xshape, filters, k, gate, skip, with_chain, lo in cases:
        pads = [k // 2] * 4
        wshape = (filters, xshape[1], k, k)
        oshape = (xshape[0], filters, xshape[2], xshape[3])
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.2, 0.2), rand(rng, (filters,), -1, 1)
        scale, res = rand(rng, (1, xshape[1], 1, 1), 0, 1), rand(rng, oshape, -1, 1)
        announce("conv scale/add", xshape, wshape, gate, skip, with_chain, lo)
        hx = ok.View(x)
        if gate:
            hx = ok.View.empty(xshape)
            ok.binary_f32(ok.BOP_MUL, ok.View(x), ok.View(scale), hx)
        want = ok.View.empty(oshape, np.float32, lo)
        ok.conv(hx, ok.View(w), ok.View(bias), want, pads if k > 1 else None, [1, 1], [1, 1], 1, 0)
        if with_chain:
            t = ok.View.empty(oshape, np.float32, lo)
            ok.unary_f32(ok.OP_RELU, want, t)
            want = t
        hres = ok.View.empty(oshape, np.float32, lo)
        hres.logical()[...] = res
        if skip:
            t = ok.View.empty(oshape, np.float32, lo)
            ok.binary_f32(ok.BOP_ADD, want, hres, t)
            want = t
        dx, dw, db = DeviceView(ok.View(x), device), DeviceView(ok.View(w), device), DeviceView(ok.View(bias), device)
        ds, dr = DeviceView(ok.View(scale), device), DeviceView(hres, device)
        do = DeviceView(ok.View.empty(oshape, np.float32, lo, fill=7), device)
        cabi.call("conv_chain_scale_add", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads) if k > 1 else None,
                  cabi.i64_array([1, 1]), cabi.i64_array([1, 1]), ctypes.c_int64(1), ctypes.byref(relu if with_chain else none),
                  ds.ref() if gate else None, dr.ref() if skip else None, ctypes.c_uint32(0), None)
        assert_close(do.logical(), want.logical(), what="conv with channel scale / addend")
    # what the entry point refuses: anything but a pointwise convolution
    x, w = DeviceView(ok.View(rand(rng, (1, 8, 6, 6))), device), DeviceView(ok.View(rand(rng, (8, 8, 3, 3))), device)
    o, sc = DeviceView(ok.View.empty((1, 8, 6, 6)), device), DeviceView(ok.View(rand(rng, (1, 8, 1, 1))), device)
    assert cabi.lib.fluidml_hip_conv_chain_scale_add(x.ref(), w.ref(), None, o.ref(), cabi.i64_array([1, 1, 1, 1]), cabi.i64_array([1, 1]),
                                                     cabi.i64_array([1, 1]), 1, ctypes.byref(none), sc.ref(), None, 0, None) == cabi.FL_ERR_UNSUPPORTED


def test_conv_times_tensor_through_transpose(device):
    """Pointwise 1-d convolution -> [Transpose (0, 2, 1)] -> MulCommon with a tensor of the result's shape as one call:
    FL_CONTRACT_ADDEND_IS_FACTOR makes the entry point multiply by its `addend`, and the Transpose is expressed by
    handing over `out` and `addend` stored with their last two dims swapped (ConvBERT's convolved keys times queries).
    Against the oracle's conv and mul, for the 32x32 and 64x64 tiles and ragged extents."""
    cabi = _cabi()
    rng = np.random.default_rng(91)
    none = cabi.make_chain([])
    for C, F, S, lo in [(768, 384, 128, [0, 2, 1]), (64, 32, 16, [0, 2, 1]), (96, 50, 37, [0, 2, 1]), (512, 1024, 256, [0, 2, 1]),
                        (128, 64, 40, None)]:
        announce("conv x tensor", C, F, S, lo)
        x, w, bias = rand(rng, (1, C, S), -1, 1), rand(rng, (F, C, 1), -0.2, 0.2), rand(rng, (F,), -1, 1)
        q = rand(rng, (1, F, S), -1, 1)
        conv = ok.View.empty((1, F, S))
        ok.conv(ok.View(x), ok.View(w), ok.View(bias), conv, None, [1], [1], 1, 0)
        hq = ok.View.empty((1, F, S), np.float32, lo)
        hq.logical()[...] = q
        want = ok.View.empty((1, F, S), np.float32, lo)
        ok.binary_f32(ok.BOP_MUL, conv, hq, want)
        dx, dw, db = (DeviceView(ok.View(t), device) for t in (x, w, bias))
        dq = DeviceView(hq, device)
        do = DeviceView(ok.View.empty((1, F, S), np.float32, lo, fill=7), device)
        cabi.call("conv_chain_scale_add", dx.ref(), dw.ref(), db.ref(), do.ref(), None, cabi.i64_array([1]), cabi.i64_array([1]),
                  ctypes.c_int64(1), ctypes.byref(none), None, dq.ref(), ctypes.c_uint32(cabi.FL_CONTRACT_ADDEND_IS_FACTOR), None)
        assert_close(do.logical(), want.logical(), what="pointwise conv times a tensor")
    # the factor flag without a tensor is refused
    assert cabi.lib.fluidml_hip_conv_chain_scale_add(dx.ref(), dw.ref(), db.ref(), do.ref(), None, cabi.i64_array([1]), cabi.i64_array([1]), 1,
                                                     ctypes.byref(none), None, None, cabi.FL_CONTRACT_ADDEND_IS_FACTOR, None) == cabi.FL_ERR_NULL


def test_conv_chain_mean(device):
    """Convolution -> swish chain -> ReduceMean over the spatial dims with both results from one call: depthwise 3x3 and
    5x5, strides 1 and 2 (one workgroup per plane), a channels-last input, and the shapes that take the two-launch
    route (few planes, a dense convolution)."""
    cabi = _cabi()
    rng = np.random.default_rng(57)
    swish = cabi.make_chain([(cabi.EW_DIV_C, 2.0), (cabi.EW_TANH, 0), (cabi.EW_ADD_C, 1.0), (cabi.EW_MUL_C, 0.5), (cabi.EW_MUL_X, 0)])
    none = cabi.make_chain([])

    def swish_ref(t):
        u0, u1, u2, u3, u4 = (ok.View.empty(t.shape) for _ in range(5))
        ok.unary_f32(ok.OP_DIV_C, t, u0, 2.0)
        ok.unary_f32(ok.OP_TANH, u0, u1)
        ok.unary_f32(ok.OP_ADD_C, u1, u2, 1.0)
        ok.unary_f32(ok.OP_MUL_C, u2, u3, 0.5)
        ok.binary_f32(ok.BOP_MUL, u3, t, u4)
        return u4

    cases = [((1, 144, 56, 56), 3, 1, 144, True, None),
             ((1, 96, 57, 57), 3, 2, 96, True, None),
             ((2, 120, 28, 28), 5, 1, 120, True, [0, 2, 3, 1]),
             ((1, 240, 29, 31), 5, 2, 240, False, None),
             ((1, 32, 20, 20), 3, 1, 32, True, None),    # few planes: convolution, then reduction
             ((2, 8, 12, 12), 3, 1, 1, True, None)]      # dense convolution: the same
    for xshape, k, st, group, with_chain, li in cases:
        filters = xshape[1] if group != 1 else 16
        wshape = (filters, 1 if group != 1 else xshape[1], k, k)
        pads = [k // 2] * 4
        od = tuple((xshape[2 + d] + 2 * (k // 2) - k) // st + 1 for d in range(2))
        oshape = (xshape[0], filters) + od
        x, w, bias = rand(rng, xshape, -1, 1), rand(rng, wshape, -0.3, 0.3), rand(rng, (filters,), -1, 1)
        announce("conv_chain_mean", xshape, wshape, st, li)
        hx = ok.View.empty(xshape, np.float32, li)
        hx.logical()[...] = x
        t = ok.View.empty(oshape)
        ok.conv(hx, ok.View(w), ok.View(bias), t, pads, [st, st], [1, 1], group, 0)
        want = swish_ref(t) if with_chain else t
        want_mean = ok.View.empty((xshape[0], filters, 1, 1))
        ok.reduce_mean(want, want_mean, [2, 3])
        dx, dw, db = DeviceView(hx, device), DeviceView(ok.View(w), device), DeviceView(ok.View(bias), device)
        do = DeviceView(ok.View.empty(oshape, fill=7), device)
        dm = DeviceView(ok.View.empty((xshape[0], filters, 1, 1), fill=7), device)
        cabi.call("conv_chain_mean", dx.ref(), dw.ref(), db.ref(), do.ref(), cabi.i64_array(pads), cabi.i64_array([st, st]),
                  cabi.i64_array([1, 1]), ctypes.c_int64(group), ctypes.byref(swish if with_chain else none), dm.ref(),
                  ctypes.c_uint32(0), None)
        assert_close(do.logical(), want.logical(), what="conv_chain_mean: result")
        assert_close(dm.logical(), want_mean.logical(), what="conv_chain_mean: mean")


def test_argument_errors(device):
    """Rejected arguments return negative codes and launch nothing."""
    cabi = _cabi()
    a = DeviceView(ok.View.empty((4, 5)), device)
    b = DeviceView(ok.View.empty((6, 3)), device)
    o = DeviceView(ok.View.empty((4, 3)), device)
    assert cabi.lib.fluidml_hip_matmul(a.ref(), b.ref(), o.ref(), None) == -3  # FL_ERR_SHAPE
    assert cabi.lib.fluidml_hip_matmul(None, b.ref(), o.ref(), None) == -1  # FL_ERR_NULL
    assert cabi.lib.fluidml_hip_softmax(a.ref(), a.ref(), None, 0, 5, None) == -5  # FL_ERR_ATTR
    i = DeviceView(ok.View.empty((4, 5), np.int64), device)
    assert cabi.lib.fluidml_hip_erf(i.ref(), a.ref(), None) == -4  # FL_ERR_DTYPE
    with pytest.raises(cabi.FluidmlHipError):
        cabi.call("add_common", a.ref(), b.ref(), o.ref(), None)
