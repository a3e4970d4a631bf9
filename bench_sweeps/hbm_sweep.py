"""Bandwidth-bound kernels at sizes that do not fit any cache: achieved HBM GB/s per kernel class.

Each case calls one entry point of the C ABI on device buffers of 128-512 MiB and reports the median of the
dispatch's own begin/end interval (the interval a profiler reports for the kernel) over `repeats` launches.
Bytes are the algorithmic ones: every input once plus the output once.  `python bench.py --hbm-kernels`
prints the table and one JSON line.
"""
import ctypes
import json

HBM_PEAK_GBPS = 8000.0


def run(repeats: int = 20, out=None) -> dict:
    import torch

    from fluidml_amd import cabi

    if not torch.cuda.is_available():
        raise SystemExit("hbm_sweep: no GPU visible")
    dev = torch.device("cuda:0")
    ref = ctypes.byref

    def view(t, shape=None, strides=None, dtype=cabi.FL_FLOAT32):
        return cabi.make_tensor(t.data_ptr(), dtype, list(t.shape) if shape is None else shape,
                                list(t.stride()) if strides is None else strides)

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

    def report(name, fn, nbytes):
        ns = median_ns(fn)
        row = {"kernel": name, "us": ns / 1e3, "bytes": int(nbytes), "GB/s": nbytes / ns,
               "frac_of_hbm_peak": nbytes / ns / HBM_PEAK_GBPS}
        rows.append(row)
        print(f"{name:46s} {row['us']:9.1f} us {row['GB/s']:8.1f} GB/s  {100 * row['frac_of_hbm_peak']:5.1f} % of 8 TB/s",
              file=out, flush=True)

    n = 64 * 1024 * 1024
    x = torch.randn(n, device=dev)
    y = torch.randn(n, device=dev)
    o = torch.empty(n, device=dev)
    vx, vy, vo = view(x), view(y), view(o)
    report("Relu 256 MiB", lambda: cabi.call("relu", ref(vx), ref(vo), None), 2 * n * 4)
    report("AddCommon 256 MiB", lambda: cabi.call("add_common", ref(vx), ref(vy), ref(vo), None), 3 * n * 4)
    # (a chain with tanh or erf in it is bound by the transcendental, not by memory, at this size)
    chain = cabi.make_chain([(cabi.EW_MUL_C, 0.5), (cabi.EW_ADD_C, 1.0), (cabi.EW_RELU, 0), (cabi.EW_MUL_X, 0)])
    report("elementwise chain (x*relu(x/2+1)) 256 MiB",
           lambda: cabi.call("elementwise_chain", ref(vx), ref(vo), ref(chain), None), 2 * n * 4)
    for length in (128, 1024, 4096):
        r = n // length
        vi, vt = view(x, [r, length], [length, 1]), view(o, [r, length], [length, 1])
        report(f"Softmax [{r},{length}]",
               lambda: cabi.call("softmax", ref(vi), ref(vt), None, 0, ctypes.c_int64(1), None), 2 * n * 4)
    for length in (768, 4096):
        r = n // length
        gamma, beta = torch.ones(length, device=dev), torch.zeros(length, device=dev)
        vi, vt = view(x[:r * length], [r, length], [length, 1]), view(o[:r * length], [r, length], [length, 1])
        vg, vb = view(gamma), view(beta)
        report(f"LayerNormalization [{r},{length}]",
               lambda: cabi.call("layer_normalization_constant_scale_bias", ref(vi), ref(vg), ref(vb), ref(vt), None, 0,
                                 ctypes.c_int64(1), ctypes.c_double(1e-5), ctypes.c_uint32(0), None), 2 * r * length * 4)
    a, b = 4096, 16384
    vi, vt = view(x, [a, b], [b, 1]), view(o, [b, a], [a, 1])
    perm = cabi.i64_array([1, 0])
    report(f"Transpose [{a},{b}] -> [{b},{a}]", lambda: cabi.call("transpose", ref(vi), ref(vt), perm, 2, None), 2 * n * 4)
    vi = view(x, [64, 128, 16, 512], [128 * 16 * 512, 16 * 512, 512, 1])
    vt = view(o, [64, 16, 128, 512], [16 * 128 * 512, 128 * 512, 512, 1])
    perm2 = cabi.i64_array([0, 2, 1, 3])
    report("Transpose (0,2,1,3), unit-stride runs of 512",
           lambda: cabi.call("transpose", ref(vi), ref(vt), perm2, 4, None), 2 * n * 4)
    xi = torch.randn(32, 64, 224, 224, device=dev)
    xo = torch.empty(32, 64, 112, 112, device=dev)
    vi, vt = view(xi), view(xo)
    two = cabi.i64_array([2, 2])
    report("MaxPool 2x2/2 [32,64,224,224]",
           lambda: cabi.call("max_pool_without_padding", ref(vi), ref(vt), two, two, 2, None), xi.numel() * 4 * 1.25)
    report("AveragePool 2x2/2 [32,64,224,224]",
           lambda: cabi.call("average_pool_without_padding", ref(vi), ref(vt), two, two, 2, None), xi.numel() * 4 * 1.25)
    xi = torch.randn(64, 512, 56, 56, device=dev)
    xo = torch.empty(64, 512, 1, 1, device=dev)
    vi, vt = view(xi), view(xo)
    axes = cabi.i64_array([2, 3])
    report("ReduceMean over H,W [64,512,56,56]", lambda: cabi.call("reduce_mean", ref(vi), ref(vt), axes, 2, None),
           xi.numel() * 4)
    table = torch.randn(30522, 768, device=dev)
    ids = torch.randint(0, 30522, (128, 512), device=dev)
    og = torch.empty(128, 512, 768, device=dev)
    vid = cabi.make_tensor(ids.data_ptr(), cabi.FL_INT64, [128, 512], [512, 1])
    vtab, vog = view(table), view(og)
    report("Gather [128,512] rows of 768 floats",
           lambda: cabi.call("gather_constant_data_tensor", ref(vid), ref(vtab), ref(vog), None), 2 * og.numel() * 4)
    del table, ids, og, xi, xo
    weights = torch.randn(4096, 25088, device=dev) * 0.01
    bias = torch.zeros(4096, device=dev)
    for batch in (1, 8):
        act = torch.randn(batch, 25088, device=dev)
        res = torch.empty(batch, 4096, device=dev)
        va, vw, vbias, vres = view(act), view(weights), view(bias), view(res)
        report(f"Gemm [{batch},25088] x [4096,25088]^T (weight streaming)",
               lambda: cabi.call("gemm_constant_weights_bias", ref(va), ref(vw), ref(vbias), ref(vres), ctypes.c_double(1.0),
                                 ctypes.c_double(1.0), 0, 1, ctypes.c_uint32(0), None),
               (weights.numel() + act.numel() + res.numel() + bias.numel()) * 4)
    return {"metric": "achieved HBM bandwidth of the bandwidth-bound kernels", "unit": "GB/s", "peak": HBM_PEAK_GBPS,
            "repeats": repeats, "kernels": rows}


if __name__ == "__main__":
    print(json.dumps(run()))
