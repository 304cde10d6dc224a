"""The host side of the engine (batch layout, block tables, page reuse) with the torch test double in place of
the HIP kernels, in float32, for the same cuttings as on the GPU.  No kernel is tested here."""

import pytest

import engine_cases as cases
from torch_kernels import TorchKernels


@pytest.fixture(scope="module", params=["A", "B"])
def case(request, model_folders):
    return cases.make_case(request.param, model_folders)


@pytest.fixture(scope="module")
def engine(case):
    return cases.make_engine(case, "float32", "cpu", kernels=TorchKernels())


@pytest.mark.parametrize("cutting", [n[5:] for n in dir(cases) if n.startswith("case_")])
def test_cutting(engine, case, cutting):
    getattr(cases, "case_" + cutting)(engine, case)
