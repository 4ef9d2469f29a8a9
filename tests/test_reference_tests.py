"""The reference's own test headers as a check of the drop-in operator API: each is compiled unchanged, from where it lies
in the reference checkout, against include/ of this library (fusedkernellibrary_amd/build.py: build_reference_tests), and
the resulting programs run on the GPU.  Most of what they check is static_assert'ed, so the CPU leg (they all compile) is
the larger half; the GPU leg runs each program's launch() and expects 0.  Nothing of the reference is kept in this
repository: without a reference checkout the CPU leg skips, and the GPU leg runs whatever programs were built before."""
import os
import subprocess

import pytest

from fusedkernellibrary_amd import build

NAMES = [os.path.splitext(os.path.basename(h))[0] for h in build.REFERENCE_TESTS]


def program(name):
    return os.path.join(build.REFERENCE_TESTS_DIR, name)


def test_reference_test_headers_compile_unchanged(native_build):
    if not os.path.isfile(os.path.join(build.REFERENCE_ROOT, build.REFERENCE_TESTS[0])):
        pytest.skip("no reference checkout here")
    if not all(os.path.exists(program(n)) for n in NAMES):
        build.build_reference_tests()  # raises with the compiler's output when one does not compile
    assert all(os.path.exists(program(n)) for n in NAMES)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_reference_test_program_passes(name):
    if not os.path.exists(program(name)):
        pytest.skip("not built (needs the reference checkout at build time)")
    done = subprocess.run([program(name)], capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, (done.stdout[-2000:], done.stderr[-2000:])
