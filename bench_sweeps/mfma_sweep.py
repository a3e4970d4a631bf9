"""The contraction kernel (MatMul / implicit-GEMM convolution on fp32 MFMA) on problems of growing size:
achieved TFLOP/s against the 157.3 TFLOP/s fp32 matrix peak of an MI355X.

Each case calls one entry point of the C ABI and reports the median of the dispatch's own begin/end interval
over `repeats` launches; flops are 2*M*N*K (convolution: M = filters, N = images * output pixels,
K = channels * taps).  `python bench.py --mfma-kernels` prints the table and one JSON line.
"""
import ctypes
import json

FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 matrix peak; the opt-in bf16 rows are priced against it


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

    def report(name, fn, flops, bf16=False):
        ns = median_ns(fn)
        row = {"case": name, "us": ns / 1e3, "flops": float(flops), "TFLOP/s": flops / ns / 1e3}
        if bf16:
            # operands in memory stay fp32 (rounded to bf16 on their way into LDS), so the delivery of the operands,
            # not the bf16 matrix rate, is what this path can reach; both fractions are given
            row["frac_of_bf16_mfma_peak"] = flops / ns / 1e3 / BF16_MFMA_PEAK_TFLOPS
            row["speedup_over_fp32"] = rows[-1]["us"] / row["us"]
            tail = f"{100 * row['frac_of_bf16_mfma_peak']:5.1f} % of 2500, {row['speedup_over_fp32']:.2f}x the fp32 row above"
        else:
            row["frac_of_fp32_mfma_peak"] = flops / ns / 1e3 / FP32_MFMA_PEAK_TFLOPS
            tail = f"{100 * row['frac_of_fp32_mfma_peak']:5.1f} % of 157.3"
        rows.append(row)
        print(f"{name:58s} {row['us']:9.1f} us {row['TFLOP/s']:7.1f} TFLOP/s  {tail}", file=out, flush=True)

    for m, k, n in [(128, 768, 768), (128, 768, 3072), (128, 3072, 768), (256, 512, 50304), (1024, 1024, 1024),
                    (2048, 2048, 2048), (4096, 4096, 4096), (8192, 4096, 8192)]:
        a = torch.randn(m, k, device=dev)
        b = torch.randn(k, n, device=dev)
        c = torch.empty(m, n, device=dev)
        va, vb, vc = view(a), view(b), view(c)
        report(f"MatMul [{m},{k}] x [{k},{n}]", lambda: cabi.call("matmul", ref(va), ref(vb), ref(vc), None), 2.0 * m * n * k)
        if m >= 256:
            report(f"  bf16 operands: MatMul [{m},{k}] x [{k},{n}]", lambda: cabi.call("matmul_bf16", ref(va), ref(vb), ref(vc), None),
                   2.0 * m * n * k, bf16=True)
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
        if images >= 8:
            bits = ctypes.c_uint32(cabi.FL_CONTRACT_BF16 << cabi.FL_CONTRACT_SHIFT)
            report(f"  bf16 operands: Conv 3x3 [{images},{channels},{size},{size}] -> {filters}",
                   lambda: cabi.call("conv_with_padding", ref(vx), ref(vw), ref(vbias), ref(vy), None, 0, pad, one, one,
                                     ctypes.c_int64(1), bits, None),
                   2.0 * images * filters * size * size * channels * 9, bf16=True)
        del x, w, y
    # what the matrix pipes deliver when a wave does nothing but issue dependent fp32 MFMAs, at the clock the
    # device actually runs at: the ceiling of any contraction kernel here
    loop = {}
    for waves in (1, 2):
        ns, ticks = ctypes.c_double(), ctypes.c_double()
        count = 2048
        cabi.call("mfma_rate", waves, count, ref(ns), ref(ticks))
        simds = 4 * torch.cuda.get_device_properties(dev).multi_processor_count
        tflops = 4096.0 * count * waves * simds / (ns.value * 1e-9) / 1e12
        loop[f"{waves}_per_simd"] = {"us": ns.value / 1e3, "shader_clock_ghz": ticks.value / ns.value,
                                     "ticks_per_mfma": ticks.value / (count * waves), "TFLOP/s": tflops}
        print(f"{waves} wave(s) per SIMD, {count} dependent v_mfma_f32_32x32x2_f32 each: {ns.value / 1e3:8.1f} us, shader clock "
              f"{ticks.value / ns.value:.2f} GHz, {tflops:6.1f} TFLOP/s = {100 * tflops / FP32_MFMA_PEAK_TFLOPS:.1f} % of the published peak",
              file=out, flush=True)
    return {"metric": "achieved fp32 MFMA throughput of the contraction kernel", "unit": "TFLOP/s",
            "peak": FP32_MFMA_PEAK_TFLOPS, "repeats": repeats, "cases": rows, "mfma_only_loop": loop}


if __name__ == "__main__":
    print(json.dumps(run()))
