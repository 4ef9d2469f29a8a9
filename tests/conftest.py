import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run on the GPU box only")


@pytest.fixture(scope="session")
def native_build():
    """The native libraries and C++ test programs: used as built; compiled here only when nothing has been built yet."""
    import fusedkernellibrary_amd as lib
    from fusedkernellibrary_amd import build
    wanted = list(lib.library_paths()) + [os.path.join(ROOT, "tests", "cpp", n) for n in ("conformance", "readme_dropin", "api_gpu", "host_plan_check", "staging_ring_check")]
    wanted.append(os.path.join(ROOT, "fusedkernellibrary_amd", "benchmarks", "reference_sweeps"))
    if not all(os.path.exists(p) for p in wanted):
        build.build_all()
    return wanted


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    return binding.oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference-headers build (literal host semantics); tests that need it skip when it was not built."""
    from oracle import binding
    ref = binding.reference()
    if ref is None:
        pytest.skip("oracle/_ref/libfkref.so not built (needs the reference tree)")
    return ref


@pytest.fixture(scope="session")
def fk():
    """The native library on the GPU.  Never falls back: a missing library is an error, not a skip."""
    import torch
    import fusedkernellibrary_amd as lib
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    lib.load()
    return lib


def same_bits(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()
