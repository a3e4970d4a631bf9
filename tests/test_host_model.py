"""Host data model and API surface.

The vectors are the reference's own unit tests: test/utils/gen_test.cpp:5-51 (GenAllOrders(8) yields 8!
distinct permutations; GenAllIndicesInOrder({2,3,4}) is row-major; GenStrides({2,3,4}) == {12,4,1}),
test/tensor/meta_test.cpp:6-26 (BroadcastShape, BroadcastMatMulShape) and test/python/import_test.py:10-61
(the attribute checklist of the Python module)."""
import ctypes
import itertools
import math
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def fluidml():
    from fluidml_amd import fluidml as module

    return module


def test_gen_all_orders(fluidml):
    orders = [tuple(o) for o in fluidml._gen_all_orders(8)]
    assert len(orders) == math.factorial(8)  # gen_test.cpp:5-24
    assert len(set(orders)) == len(orders)
    assert all(sorted(o) == list(range(8)) for o in orders)
    # enumeration order matters to the DP (ties keep the first): element 0 is the reversed permutation
    assert fluidml._gen_all_orders(3) == [[2, 1, 0], [1, 2, 0], [1, 0, 2], [2, 0, 1], [0, 2, 1], [0, 1, 2]]
    assert fluidml._gen_all_orders(0) == [[]]
    for n in range(1, 6):
        assert fluidml._gen_all_orders(n)[0] == list(range(n))[::-1]


def test_gen_all_indices_in_order(fluidml):
    got = fluidml._gen_all_indices_in_order([2, 3, 4])  # gen_test.cpp:26-42
    assert got == [list(i) for i in itertools.product(range(2), range(3), range(4))]


def test_gen_strides(fluidml):
    assert fluidml._gen_strides([2, 3, 4]) == [12, 4, 1]  # gen_test.cpp:44-51
    # physical_shape[layout[i]] = shape[i]; strides[i] = rowmajor(physical)[layout[i]] (utils.cpp:64-102)
    assert fluidml._gen_physical_shape([2, 3, 4], [2, 0, 1]) == [3, 4, 2]
    assert fluidml._gen_strides_layout([2, 3, 4], [2, 0, 1]) == [1, 8, 2]
    import numpy as np

    rng = np.random.default_rng(0)
    for layout in itertools.permutations(range(4)):
        shape = rng.integers(1, 6, size=4).tolist()
        strides = fluidml._gen_strides_layout(shape, list(layout))
        phys = fluidml._gen_physical_shape(shape, list(layout))
        # every logical index maps to a distinct physical slot inside the dense block
        seen = {sum(i * s for i, s in zip(idx, strides)) for idx in itertools.product(*[range(d) for d in shape])}
        assert seen == set(range(int(np.prod(phys))))


def test_constant_bytes_for_a_layout(fluidml):
    """Tensor::Pack, the bytes uploaded for a constant: element i at its strided position; with
    FL_REF_CONSTANT_GATHERED the reference's form (builder.cpp:290-297), against the oracle's restatement."""
    import numpy as np

    from oracle import kernels as ok

    rng = np.random.default_rng(12)
    for shape in [(3, 5), (2, 3, 4), (7,)]:
        logical = rng.uniform(-1, 1, size=shape).astype(np.float32)
        for layout in itertools.permutations(range(len(shape))):
            plain = np.frombuffer(fluidml._pack_constant_f32(logical.reshape(-1).tolist(), list(shape), list(layout)), dtype=np.float32)
            view = ok.View(logical, list(layout))
            assert np.array_equal(plain, view.physical.reshape(-1)), (shape, layout)
            got = np.frombuffer(fluidml._pack_constant_f32(logical.reshape(-1).tolist(), list(shape), list(layout), True), dtype=np.float32)
            assert np.array_equal(got, ok.reference_constant(logical, list(layout))[0]), (shape, layout)


def test_broadcast_shapes(fluidml):
    assert fluidml._broadcast_shape([1, 1, 3], [2, 3]) == [1, 2, 3]  # meta_test.cpp:6-15
    assert fluidml._broadcast_matmul_shape([2, 1, 3], [3, 2]) == [2, 1, 2]  # meta_test.cpp:17-26
    assert fluidml._broadcast_shape([2, 3], [4, 3]) is None
    assert fluidml._broadcast_matmul_shape([3], [3, 2]) is None
    assert fluidml._broadcast_matmul_shape([1, 12, 128, 64], [1, 12, 64, 128]) == [1, 12, 128, 128]


def test_python_surface(fluidml):
    """test/python/import_test.py, attribute for attribute."""
    for name in ["Context", "Flow", "Sequence", "Graph", "Index", "Builder", "GeneralBuilder", "Converter", "Executor",
                 "Lower", "Parser", "Planner", "Runner"]:
        assert hasattr(fluidml, name), name
    assert hasattr(fluidml.GeneralBuilder, "run")
    assert hasattr(fluidml.Converter, "run") and hasattr(fluidml.Converter, "make")
    for attr in ["compile", "invoke", "make_plain_linear", "make_plain_greedy", "make_dp_greedy"]:
        assert hasattr(fluidml.Executor, attr), attr
    assert hasattr(fluidml.Lower, "run")
    assert hasattr(fluidml.Parser, "run") and hasattr(fluidml.Parser, "make")
    assert hasattr(fluidml.Planner, "run")
    assert hasattr(fluidml.Runner, "run")
    for attr in ["make_plain_general_builder", "make_dp_general_builder", "make_kernel_builder", "make_plain_linear_planner",
                 "make_plain_greedy_planner", "make_dp_greedy_planner", "make_lower", "make_runner"]:
        assert hasattr(fluidml.Context, attr), attr


def test_top_level_module_name(fluidml):
    """the reference's module is called `fluidml` (pybind.cpp:23): the same import line works here"""
    import fluidml as top

    for name in ["Context", "Flow", "Sequence", "Graph", "Index", "Builder", "GeneralBuilder", "Converter", "Executor",
                 "Lower", "Parser", "Planner", "Runner"]:
        assert getattr(top, name) is getattr(fluidml, name)
    assert top.Executor.make_dp_greedy is fluidml.Executor.make_dp_greedy


# kKernelName of every kernel class of the reference (include/structure/kernel/kernel/*.h; e.g. gemm.h:13
# "GemmConstantWeightsBiasKernel" for class GemmConstantBiasKernel, where.h:13-14, 34-35, gather_add_add.h:13-14)
REFERENCE_KERNEL_NAMES = """
AddCommonKernel AddConstantKernel AddDivErfAddMulMulKernel AveragePoolWithoutPaddingKernel CastKernel ClipKernel
Concat2Kernel ConvWithPaddingKernel ConvWithoutPaddingKernel CumSumKernel DivCommonKernel DivConstantRhsKernel
DropoutKernel EqualKernel ErfKernel FlattenKernel GatherConstantDataTensorKernel GatherConstantIndexScalarKernel
GatherConstantIndicesTensorKernel GemmConstantWeightsBiasKernel MatMulKernel MaxPoolWithoutPaddingKernel
MulCommonKernel MulConstantKernel NegKernel NotKernel PadKernel PowKernel ReduceMeanKernel ReluKernel ReshapeKernel
SliceKernel SoftmaxKernel SqrtKernel SqueezeKernel SubCommonKernel SubConstantLhsKernel TanhKernel TransposeKernel
UnsqueezeKernel GatherConstantDataTensorAddTensorLhsAddTensorLhsKernel LayerNormalizationConstantScaleBiasKernel
UnsqueezeSubLhsScalarMulRhsScalarKernel WhereConstantCondConstantScalarYKernel WhereConstantCondConstantTensorYKernel
""".split()


def test_kernel_names_are_the_references(fluidml):
    names = fluidml._kernel_names()
    assert len(names) == len(set(names)) == len(REFERENCE_KERNEL_NAMES) == 45
    assert set(names) == set(REFERENCE_KERNEL_NAMES)


def test_c_abi_exports_every_declared_symbol():
    """The shared library loads and exports each entry point include/fluidml_hip.h declares (no compute call)."""
    header = open(os.path.join(ROOT, "include", "fluidml_hip.h")).read()
    declared = set(re.findall(r"\b(fluidml_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) > 60
    lib = ctypes.CDLL(os.path.join(ROOT, "fluidml_amd", "lib", "libfluidml_hip.so"))
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, missing
    from fluidml_amd import cabi

    assert set(cabi.SIGNATURES) | {"fluidml_hip_error_string"} == declared
    assert cabi.lib.fluidml_hip_abi_version() == 3
    assert cabi.error_string(-3).startswith("shapes")


def test_header_compiles_as_c(tmp_path):
    import subprocess

    src = tmp_path / "t.c"
    src.write_text('#include "fluidml_hip.h"\nint main(void) { fl_tensor t; t.rank = 0; return t.rank; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)
