"""fluidml_hip_matmul_no_alloc: the matmul entry point that allocates nothing keeps the split-K partial tiles
and arrival counters in a fixed device array inside the library.  Through the C ABI its output has to equal
fluidml_hip_matmul's bit for bit (same kernels, same split), on calls in a row that share the array -- the
second on a smaller problem, so stale partial tiles and counters of the first lie behind it -- and a problem
whose split does not fit the array has to be refused with nothing launched."""
import numpy as np
import pytest

from oracle import kernels as ok
from tests.util import DeviceView, assert_close

pytestmark = pytest.mark.gpu


def _pair(cabi, device, rng, M, K, N):
    a = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    b = rng.uniform(-0.05, 0.05, size=(K, N)).astype(np.float32)
    da, db = DeviceView(ok.View(a), device), DeviceView(ok.View(b), device)
    ref = DeviceView(ok.View.empty((M, N), fill=3), device)
    got = DeviceView(ok.View.empty((M, N), fill=5), device)
    return a, b, da, db, ref, got


def test_no_alloc_matmul_equals_matmul(device):
    import torch

    from fluidml_amd import cabi

    rng = np.random.default_rng(90)
    # a stream the library has never seen: fluidml_hip_matmul would allocate its 16 MiB workspace on first use
    side = torch.cuda.Stream()
    warm = torch.zeros(16, device=device)
    with torch.cuda.stream(side):
        warm.add_(1)  # the runtime's own first-use set-up of the stream (queue, signals) happens here
    torch.cuda.synchronize()
    # split-K launches (K >= 768 on few tiles), the second smaller than the first; then one without a split and
    # one that the weight-streaming kernel takes (no scratch at all)
    for M, K, N in [(128, 3072, 768), (96, 768, 320), (128, 3072, 768), (64, 1536, 64), (256, 64, 256), (1, 4096, 512)]:
        print("[case] matmul_no_alloc", M, K, N, flush=True)
        a, b, da, db, ref, got = _pair(cabi, device, rng, M, K, N)
        cabi.call("matmul", da.ref(), db.ref(), ref.ref(), None)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        cabi.call("matmul_no_alloc", da.ref(), db.ref(), got.ref(), side.cuda_stream)
        torch.cuda.synchronize()
        assert free_before - torch.cuda.mem_get_info()[0] < (8 << 20), "the call took device memory"
        want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
        assert_close(ref.logical(), want, what="matmul vs float64 numpy")
        assert_close(got.logical(), ref.logical(), exact=True, what=f"matmul_no_alloc vs matmul {M}x{K}x{N}")


def test_no_alloc_matmul_refuses_what_does_not_fit(device):
    from fluidml_amd import cabi

    rng = np.random.default_rng(91)
    # 8 x 20 = 160 tiles of 32x32, K = 2048 -> 4 splits: 640 partial tiles of 4 KiB > the 2 MiB array
    M, K, N = 256, 2048, 640
    a, b, da, db, ref, got = _pair(cabi, device, rng, M, K, N)
    rc = cabi.lib.fluidml_hip_matmul_no_alloc(da.ref(), db.ref(), got.ref(), None)
    assert rc == cabi.FL_ERR_STATIC_SCRATCH
    assert "fluidml_hip_matmul_no_alloc" in cabi.error_string(rc)
    assert (got.logical() == 5).all(), "a refused call must not launch anything"
    # the array still works afterwards
    M, K, N = 64, 1536, 96
    a, b, da, db, ref, got = _pair(cabi, device, rng, M, K, N)
    cabi.call("matmul", da.ref(), db.ref(), ref.ref(), None)
    cabi.call("matmul_no_alloc", da.ref(), db.ref(), got.ref(), None)
    assert_close(got.logical(), ref.logical(), exact=True, what="matmul_no_alloc after a refusal")
