"""TEST INFRASTRUCTURE -- whole-graph CPU execution with the oracle's loop nests.

Walks the node list of a `fluidml_amd.onnx_writer.GraphBuilder` in order, picks the FluidML
operator variant from which inputs are initializers (the rules of reference
src/worker/converter.cpp, per operator) and runs the matching function of oracle/kernels.c on
dense row-major tensors (the layout of the reference's plain executors).  This is the
"FluidML-equivalent CPU loop nests" execution that whole-model parity tests compare the GPU
path with, and what the cpu_baseline leg of bench.py times.
"""
from __future__ import annotations

import time
from typing import Dict, Optional

import numpy as np

from . import kernels as ok

FL_REF_CONV_UNIT_STRIDE, FL_REF_CONV_BIAS_INDEX1, FL_REF_LN_STALE_SCRATCH, FL_REF_GEMM_SWAPPED_SCALARS = 1, 2, 4, 8


def _is_scalar(v) -> bool:
    return v.const is not None and v.const.ndim == 0


def _is_tensor_const(v) -> bool:
    return v.const is not None and v.const.ndim > 0


def run_graph(net, feeds: Dict[str, np.ndarray], flags: int = 0, timings: Optional[dict] = None) -> Dict[str, np.ndarray]:
    env: Dict[str, np.ndarray] = {k: np.ascontiguousarray(v) for k, v in feeds.items()}
    for v in net.initializers:
        env[v.name] = v.const

    def val(v):
        return env[v.name]

    def new(v, fill=0):
        return ok.View.empty(v.shape, v.dtype, fill=fill)

    for n in net.nodes:
        t0 = time.perf_counter()
        op, ins, out = n.op_type, n.inputs, n.outputs[0]
        o = new(out)
        a = n.attrs
        if op in ("Add", "Sub", "Mul", "Div"):
            x, y = ins
            if _is_scalar(x) or _is_scalar(y):
                t, c = (y, x) if _is_scalar(x) else (x, y)
                cv = float(val(c))
                tv = ok.View(val(t))
                if op == "Add":
                    if t.dtype == np.float32:
                        ok.unary_f32(ok.OP_ADD_C, tv, o, cv)
                    else:
                        ok.unary_int(ok.IOP_ADD_C, tv, o, cv)
                elif op == "Mul":
                    ok.unary_f32(ok.OP_MUL_C, tv, o, cv)
                elif op == "Sub":
                    assert _is_scalar(x), "FluidML only has scalar - x (reference converter.cpp:2284-2344)"
                    ok.unary_f32(ok.OP_RSUB_C, tv, o, cv)
                else:
                    assert _is_scalar(y), "FluidML only has x / scalar (reference converter.cpp:941-993)"
                    ok.unary_f32(ok.OP_DIV_C, tv, o, cv)
            elif op == "Mul" and out.dtype != np.float32:
                ok.mul_int(ok.View(val(x)), ok.View(val(y)), o)
            else:
                code = {"Add": ok.BOP_ADD, "Sub": ok.BOP_SUB, "Mul": ok.BOP_MUL, "Div": ok.BOP_DIV}[op]
                ok.binary_f32(code, ok.View(val(x)), ok.View(val(y)), o)
        elif op in ("Erf", "Relu", "Tanh", "Sqrt", "Neg", "Dropout"):
            code = {"Erf": ok.OP_ERF, "Relu": ok.OP_RELU, "Tanh": ok.OP_TANH, "Sqrt": ok.OP_SQRT, "Neg": ok.OP_NEG,
                    "Dropout": ok.OP_COPY}[op]
            ok.unary_f32(code, ok.View(val(ins[0])), o)
        elif op == "Pow":
            ok.unary_f32(ok.OP_POW_C, ok.View(val(ins[0])), o, float(val(ins[1])))
        elif op == "Clip":
            lo, hi = (float(val(ins[1])), float(val(ins[2]))) if len(ins) == 3 else (a["min"], a["max"])
            ok.unary_f32(ok.OP_CLIP, ok.View(val(ins[0])), o, lo, hi)
        elif op == "Cast":
            ok.unary_int(ok.IOP_CAST, ok.View(val(ins[0])), o)
        elif op == "Equal":
            ok.unary_int(ok.IOP_EQ_C, ok.View(val(ins[0])), o, float(val(ins[1])))
        elif op == "Not":
            ok.unary_int(ok.IOP_NOT, ok.View(val(ins[0])), o)
        elif op == "CumSum":
            ok.cum_sum(ok.View(val(ins[0])), o, int(val(ins[1])))
        elif op == "Where":
            cond, x, y = ins
            if _is_scalar(y):
                ok.where(ok.View(val(cond)), ok.View(val(x)), None, float(val(y)), o)
            else:
                ok.where(ok.View(val(cond)), ok.View(val(x)), ok.View(val(y)), 0.0, o)
        elif op == "Gather":
            data, idx = ins
            axis = a.get("axis", 0)
            if _is_tensor_const(data):
                ok.gather_data_tensor(ok.View(val(idx)), ok.View(val(data)), o)
            elif _is_scalar(idx):
                ok.gather_index_scalar(ok.View(val(data)), o, axis, int(val(idx)), flags & (1 << 4))
            else:
                ok.gather_indices_tensor(ok.View(val(data)), ok.View(val(idx)), o, axis % len(data.shape))
        elif op in ("Reshape", "Flatten"):
            ok.reshape(ok.View(val(ins[0])), o)
        elif op == "Transpose":
            perm = a.get("perm", list(range(len(ins[0].shape)))[::-1])
            ok.transpose(ok.View(val(ins[0])), o, perm)
        elif op == "Squeeze":
            axes = [int(v) for v in val(ins[1])] if len(ins) == 2 else a["axes"]
            ok.squeeze(ok.View(val(ins[0])), o, axes)
        elif op == "Unsqueeze":
            ok.unsqueeze(ok.View(val(ins[0])), o, [int(v) for v in val(ins[1])])
        elif op == "Slice":
            starts, axes, steps = ([int(v) for v in val(ins[i])] for i in (1, 3, 4))
            rank = len(ins[0].shape)
            axes = [ax % rank for ax in axes]
            starts = [s + ins[0].shape[ax] if s < 0 else s for s, ax in zip(starts, axes)]
            ok.slice_(ok.View(val(ins[0])), o, starts, axes, steps)
        elif op == "Concat":
            ok.concat2(ok.View(val(ins[0])), ok.View(val(ins[1])), o, a["axis"] % len(out.shape))
        elif op == "Pad":
            p = [int(v) for v in val(ins[1])]
            ok.pad(ok.View(val(ins[0])), o, p[: len(p) // 2], flags & (1 << 5))
        elif op == "Softmax":
            ok.softmax(ok.View(val(ins[0])), o, a.get("axis", -1) % len(out.shape))
        elif op == "LayerNormalization":
            ok.layer_norm(ok.View(val(ins[0])), ok.View(val(ins[1])), ok.View(val(ins[2])), o,
                          a.get("axis", 1) % len(out.shape), a.get("epsilon", 1e-5))
        elif op == "ReduceMean":
            axes = [int(v) for v in val(ins[1])] if len(ins) == 2 else a["axes"]
            ok.reduce_mean(ok.View(val(ins[0])), o, [ax % len(ins[0].shape) for ax in axes])
        elif op in ("MaxPool", "AveragePool"):
            k = a["kernel_shape"]
            ok.pool(op == "MaxPool", ok.View(val(ins[0])), o, k, a.get("strides", [1] * len(k)))
        elif op == "MatMul":
            ok.matmul(ok.View(val(ins[0])), ok.View(val(ins[1])), o)
        elif op == "Gemm":
            ok.gemm(ok.View(val(ins[0])), ok.View(val(ins[1])), ok.View(val(ins[2])), o, a.get("alpha", 0.0),
                    a.get("beta", 0.0), a.get("transA", 0), a.get("transB", 0), flags & FL_REF_GEMM_SWAPPED_SCALARS)
        elif op == "Conv":
            bias = ok.View(val(ins[2])) if len(ins) == 3 else None
            pads = a["pads"] if any(a["pads"]) else None
            ok.conv(ok.View(val(ins[0])), ok.View(val(ins[1])), bias, o, pads, a["strides"], a["dilations"],
                    a.get("group", 1), flags & (FL_REF_CONV_UNIT_STRIDE | FL_REF_CONV_BIAS_INDEX1))
        else:
            raise NotImplementedError(f"oracle graph runner: {op}")
        env[out.name] = o.logical()
        if timings is not None:
            timings[n.name] = (op, time.perf_counter() - t0)
    return {v.name: env[v.name] for v in net.outputs}
