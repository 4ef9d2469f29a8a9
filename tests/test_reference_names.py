"""The drop-in surface by name: every public name of the reference's namespace fk is either required of this library
(tests/cpp/reference_names.inc, which tests/cpp/conformance.cpp turns into using-declarations, so a missing name does not
compile) or listed as deliberately absent with a reason.  Where the reference checkout is present, the committed lists are
what the generator writes today."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
REFERENCE = os.environ.get("FK_REFERENCE_ROOT", "/root/reference")


def read_names(path):
    return [line.split("\t")[0].strip() for line in open(path) if line.strip() and not line.startswith("#")]


def test_every_reference_name_is_required_or_explained():
    names = read_names(os.path.join(GOLDEN, "reference_public_names.txt"))
    absent = {}
    for line in open(os.path.join(GOLDEN, "reference_names_absent.txt")):
        if line.strip() and not line.startswith("#"):
            name, _, reason = line.rstrip("\n").partition("\t")
            absent[name.strip()] = reason.strip()
    required = [line[len("FK_REFERENCE_NAME("):-2] for line in open(os.path.join(HERE, "cpp", "reference_names.inc")) if line.startswith("FK_REFERENCE_NAME(")]
    assert len(names) > 350 and len(set(names)) == len(names)
    assert set(required) | set(absent) == set(names) and not set(required) & set(absent)
    assert all(len(reason) > 20 for reason in absent.values()), "every absent name states why"
    assert len(absent) <= 20, "the absent list is for scaffolding of the reference's implementation, not for missing features"
    # the names the hot path is built from must be among the required ones
    for name in ("executeOperations" if False else "Executor", "TransformDPP", "PerThreadRead", "BatchRead", "Crop", "Resize", "Mul", "Sub", "Div",
                 "ColorConversion", "TensorWrite", "Tensor", "Ptr2D", "Stream_", "BaseStream", "Saturate", "PtrT3D", "Slice2x2"):
        assert name in required, name
    source = open(os.path.join(HERE, "cpp", "conformance.cpp")).read()
    assert '#include "reference_names.inc"' in source and "using fk::name;" in source


def test_the_committed_lists_are_what_the_generator_writes():
    if not os.path.isdir(os.path.join(REFERENCE, "include", "fused_kernel")):
        import pytest
        pytest.skip("no reference checkout here")
    before = {p: open(p).read() for p in (os.path.join(GOLDEN, "reference_public_names.txt"), os.path.join(HERE, "cpp", "reference_names.inc"))}
    subprocess.run([sys.executable, os.path.join(GOLDEN, "make_reference_names.py")], check=True, stdout=subprocess.DEVNULL)
    for path, text in before.items():
        assert open(path).read() == text, path + " is stale: run tests/golden/make_reference_names.py"
