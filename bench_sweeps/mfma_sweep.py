"""The contraction kernel (MatMul / implicit-GEMM convolution on fp32 MFMA) on problems of growing size:
achieved TFLOP/s against the 157.3 TFLOP/s fp32 matrix peak of an MI355X.

Each case calls one entry point of the C ABI and reports the median of the dispatch's own begin/end interval
over `repeats` launches; flops are 2*M*N*K (convolution: M = filters, N = images * output pixels,
K = channels * taps).  `python bench.py --mfma-kernels` prints the table and one JSON line.
"""
import ctypes
import json

FP32_MFMA_PEAK_TFLOPS = 157.3


def run(repeats: int = 20, out=None) -> dict:
    import torch

    from fluidml_amd import cabi

    if not torch.cuda.is_available():
        raise SystemExit("mfma_sweep: no GPU visible")
    dev = torch.device("cuda:0")
    ref = ctypes.byref

    def view(t):
        return cabi.make_tensor(t.data_ptr(), cabi.FL_FLOAT32, list(t.shape), list(t.stride()))

    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    cabi.call("event_create", ref(e0))
    cabi.call("event_create", ref(e1))

    def median_ns(fn):
        ts = []
        for _ in range(repeats):
            cabi.call("time_kernels", e0, e1)
            fn()
            cabi.call("time_kernels", None, None)
            torch.cuda.synchronize()
            ns = ctypes.c_double()
            cabi.call("event_elapsed_ns", e0, e1, ref(ns))
            ts.append(ns.value)
        ts.sort()
        return ts[len(ts) // 2]

    rows = []

    def report(name, fn, flops):
        ns = median_ns(fn)
        row = {"case": name, "us": ns / 1e3, "flops": float(flops), "TFLOP/s": flops / ns / 1e3,
               "frac_of_fp32_mfma_peak": flops / ns / 1e3 / FP32_MFMA_PEAK_TFLOPS}
        rows.append(row)
        print(f"{name:52s} {row['us']:9.1f} us {row['TFLOP/s']:7.1f} TFLOP/s  {100 * row['frac_of_fp32_mfma_peak']:5.1f} % of 157.3",
              file=out, flush=True)

    for m, k, n in [(128, 768, 768), (128, 768, 3072), (128, 3072, 768), (256, 512, 50304), (1024, 1024, 1024),
                    (2048, 2048, 2048), (4096, 4096, 4096), (8192, 4096, 8192)]:
        a = torch.randn(m, k, device=dev)
        b = torch.randn(k, n, device=dev)
        c = torch.empty(m, n, device=dev)
        va, vb, vc = view(a), view(b), view(c)
        report(f"MatMul [{m},{k}] x [{k},{n}]", lambda: cabi.call("matmul", ref(va), ref(vb), ref(vc), None), 2.0 * m * n * k)
        del a, b, c
    one, pad = cabi.i64_array([1, 1]), cabi.i64_array([1, 1, 1, 1])
    for images, channels, size, filters in [(8, 64, 224, 64), (8, 128, 112, 128), (8, 256, 56, 256), (8, 512, 28, 512),
                                            (8, 512, 14, 512), (1, 512, 14, 512), (32, 256, 56, 256)]:
        x = torch.randn(images, channels, size, size, device=dev)
        w = torch.randn(filters, channels, 3, 3, device=dev) * 0.05
        bias = torch.zeros(filters, device=dev)
        y = torch.empty(images, filters, size, size, device=dev)
        vx, vw, vbias, vy = view(x), view(w), view(bias), view(y)
        report(f"Conv 3x3 pad 1 [{images},{channels},{size},{size}] -> {filters} filters",
               lambda: cabi.call("conv_with_padding", ref(vx), ref(vw), ref(vbias), ref(vy), None, 0, pad, one, one,
                                 ctypes.c_int64(1), ctypes.c_uint32(0), None),
               2.0 * images * filters * size * size * channels * 9)
        del x, w, y
    return {"metric": "achieved fp32 MFMA throughput of the contraction kernel", "unit": "TFLOP/s",
            "peak": FP32_MFMA_PEAK_TFLOPS, "repeats": repeats, "cases": rows}


if __name__ == "__main__":
    print(json.dumps(run()))
