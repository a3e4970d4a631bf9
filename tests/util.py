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
