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


def assert_close_or_exact(got, ref, exact_fn, what="", report=None):
    """`got` has to be within rel RTOL / abs ATOL of the oracle's result `ref`, element by element.  Where it
    is not, the float64 evaluation of the same network (`exact_fn()`) decides whose rounding the difference is:
    the element passes if `got` is within the same tolerance of the float64 value, or at least no farther from
    it than the oracle's own worst element on this output is.  The oracle adds the products of a dot product
    one after the other in fp32 like the reference's loop nests, and over the 4,608 to 25,088 terms of the late
    VGG-16 layers that alone moves logits whose terms cancel by more than the tolerance; a result that is closer
    to the exact value than the reference's own arithmetic gets is not in error."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bad = err > ATOL + RTOL * np.abs(ref.astype(np.float64))
    if not bad.any():
        return
    exact = np.asarray(exact_fn(), np.float64)
    assert exact.shape == got.shape
    bound = ATOL + RTOL * np.abs(exact)
    err_got = np.abs(got.astype(np.float64) - exact)
    err_ref = np.abs(ref.astype(np.float64) - exact)
    if report is not None:
        report(f"[tolerance] {what}: {np.count_nonzero(bad)} of {bad.size} elements differ from the oracle by more than rel {RTOL} / "
               f"abs {ATOL} (max {err.max():.3e}); distance to the float64 evaluation: oracle max {err_ref.max():.3e} "
               f"({np.count_nonzero(err_ref > bound)} outside), this result max {err_got.max():.3e} ({np.count_nonzero(err_got > bound)} outside)")
    still = bad & (err_got > np.maximum(bound, err_ref.max()))
    assert not still.any(), (
        f"{what}: {np.count_nonzero(still)} of {bad.size} elements are outside rel {RTOL}/abs {ATOL} of the oracle and farther from the "
        f"float64 evaluation than the oracle ever is; max distance to the oracle {err.max():.3e}, to float64 {err_got.max():.3e} "
        f"(oracle to float64 {err_ref.max():.3e})"
    )
