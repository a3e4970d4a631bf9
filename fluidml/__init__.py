"""``import fluidml`` -- the module name the reference's Python binding has (reference
src/python/pybind.cpp:23, setup.py:76), so code written against it runs unchanged:

    import fluidml
    ex = fluidml.Executor.make_plain_greedy("bert")
    ex.compile("bert.onnx")
    ns = ex.invoke({"input_ids": ids, ..., "last_hidden_state": out})

Everything comes from the compiled host module ``fluidml_amd.fluidml`` (HIP launcher, planner, DP); there
is no CPU fallback, importing fails when the libraries are not built.
"""
from fluidml_amd import fluidml as _impl

for _name in dir(_impl):
    if not (_name.startswith("__") and _name.endswith("__")):
        globals()[_name] = getattr(_impl, _name)
del _name

__all__ = [n for n in dir(_impl) if not n.startswith("_")]
