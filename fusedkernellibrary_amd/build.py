"""Build recipe of the native libraries (hipcc, gfx950 only).

  libfk_hip_rt.so   the C runtime ABI of include/fk_hip_rt.h (csrc/fk_hip_rt.cpp)
  libfk_capi.so     the chain entry points of include/fk_capi.h (csrc/fk_capi*.hip), i.e. the
                    fused kernels instantiated from the fk:: templates under include/fk/

  benchmarks/reference_sweeps   the reference's benchmark sweeps (benchmarks/reference_sweeps.cpp), a program

Run as `python -m fusedkernellibrary_amd.build`; outputs land beside this file.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
CSRC = os.path.join(HERE, "csrc")

# -ffp-contract=off: no FMA contraction, so results equal an unfused evaluation bit for bit.
# packed-fp32-ops is switched off for device code (the host pass warns that it does not know the feature).
DEVICE_FLAGS = ["--offload-arch=gfx950", "-std=c++17", "-O3", "-ffp-contract=off", "-ftemplate-depth=1024",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the native libraries cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError("build step failed: " + " ".join(cmd))
    return proc.stdout


def build_runtime():
    out = os.path.join(HERE, "libfk_hip_rt.so")
    # compiled as HIP: it holds the kernel-argument probe kernel
    _run([hipcc(), "-x", "hip", os.path.join(CSRC, "fk_hip_rt.cpp"), "-I" + INCLUDE, "--offload-arch=gfx950", "-std=c++17", "-O2",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fPIC", "-shared", "-o", out])
    return out


CAPI_SOURCES = ("fk_capi.hip", "fk_capi_yuv.hip", "fk_capi_border_warp.hip", "fk_capi_circular.hip", "fk_capi_paths.hip", "fk_capi_noalloc.hip")


def build_capi(extra_defines=(), name="libfk_capi.so"):
    """One object per source (compiled side by side), linked into one shared library."""
    from concurrent.futures import ThreadPoolExecutor
    out = os.path.join(HERE, name)
    defines = ["-D" + d for d in extra_defines]
    objdir = os.path.join(HERE, "csrc", ".obj_" + name.replace(".so", ""))
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        _run([hipcc(), "-x", "hip", os.path.join(CSRC, src), "-I" + INCLUDE, *DEVICE_FLAGS, *defines, "-fPIC", "-c", "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=len(CAPI_SOURCES)) as pool:
        objs = list(pool.map(compile_one, CAPI_SOURCES))
    _run([hipcc(), *objs, "--offload-arch=gfx950", "-fPIC", "-shared", "-L" + HERE, "-lfk_hip_rt", "-Wl,-rpath,$ORIGIN", "-o", out])
    shutil.rmtree(objdir, ignore_errors=True)
    return out


def build_cpp_tests():
    """The C++ programs under tests/cpp: the host-side API conformance check, the README example and the executor surface as
    user code, and a translation unit that includes the HIP runtime's own header before the library's."""
    tests = os.path.join(ROOT, "tests", "cpp")
    outs = []
    for name in ("conformance", "readme_dropin", "api_gpu", "hip_header_coexistence"):
        out = os.path.join(tests, name)
        _run([hipcc(), "-x", "hip", os.path.join(tests, name + ".cpp"), "-I" + INCLUDE, *DEVICE_FLAGS, "-L" + HERE, "-lfk_hip_rt",
              "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/../../fusedkernellibrary_amd", "-o", out])
        outs.append(out)
    # host-only checks: the launch plans (no GPU call is made), and the staging ring's slot state machine with stand-ins
    # for the GPU runtime (plain g++, no GPU header)
    out = os.path.join(tests, "host_plan_check")
    _run([hipcc(), "-x", "hip", "--cuda-host-only", os.path.join(tests, "host_plan_check.cpp"), "-I" + INCLUDE, "-std=c++17", "-O1",
          "-L" + HERE, "-lfk_hip_rt", "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/../../fusedkernellibrary_amd", "-o", out])
    outs.append(out)
    out = os.path.join(tests, "staging_ring_check")
    _run([shutil.which("g++") or "g++", "-std=c++17", "-O2", "-pthread", "-I" + CSRC, os.path.join(tests, "staging_ring_check.cpp"), "-o", out])
    outs.append(out)
    return outs


def build_benchmarks():
    """benchmarks/reference_sweeps: the reference's four benchmark sweeps as user code of the operator API; and
    benchmarks/store_patterns."""
    src = os.path.join(HERE, "benchmarks", "reference_sweeps.cpp")
    out = os.path.join(HERE, "benchmarks", "reference_sweeps")
    _run([hipcc(), "-x", "hip", src, "-I" + INCLUDE, *DEVICE_FLAGS, "-L" + HERE, "-lfk_hip_rt", "-Wl,-rpath,$ORIGIN/..", "-o", out])
    # benchmarks/store_patterns: what the headline's output costs to write, by store pattern (a program of its own against the
    # HIP runtime; it uses nothing of the library)
    _run([hipcc(), os.path.join(HERE, "benchmarks", "store_patterns.hip"), "--offload-arch=gfx950", "-O3", "-Wno-unused-value",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", os.path.join(HERE, "benchmarks", "store_patterns")])
    return out


# The reference's own test headers that exercise this path's operator API (relative to the reference checkout); each
# defines `int launch()`.  Left out: benchmarks/ (their timing harness is written against the CUDA runtime's event and
# stream types; fusedkernellibrary_amd/benchmarks/reference_sweeps.cpp restates them).
REFERENCE_TESTS = (
    "tests/algorithm/test_batchresize_build.h", "tests/algorithm/test_border_reader.h", "tests/algorithm/test_crop.h",
    "tests/algorithm/test_deinterlace.h", "tests/algorithm/test_warp.h", "tests/data/basic_test.h", "tests/data/test_ptr_nd.h", "tests/data/test_rect.h",
    "tests/examples/readme_test_code.h",
    "tests/data/test_tuple.h", "tests/data/test_typelist.h", "tests/operation/test_filtered_index_sequence.h",
    "tests/operation/test_fused_operation.h", "tests/operation/test_instantiable_operations.h",
    "tests/operation/test_operation_fuser.h", "tests/operation/test_operation_tuple.h", "tests/operation/test_operation_types.h",
    "tests/thread_fusion/test_thread_fusion.h",
    "utests/algorithm/image_processing/utest_saturate.h", "utests/algorithm/image_processing/utest_color_conversion.h",
    "utests/algorithm/image_processing/utest_deinterlace.h", "utests/core/constexpr_libs/utest_constexpr_cmath.h",
    "utests/core/utils/utest_VBase.h", "utests/core/utils/utest_cuda_vector_utils.h",
    "tests/string/test_fk_string.h", "tests/string/test_IOps_to_string.h", "tests/string/test_literal_to_string.h",
    "tests/string/test_struct_to_string.h",
    "tests/cudabug/test_nvcc124_126_BugReproducer.h", "tests/cudabug/test_nvcc1281_129_BugReproducer.h",
)
REFERENCE_ROOT = os.environ.get("FK_REFERENCE_ROOT", "/root/reference")
REFERENCE_TESTS_DIR = os.path.join(ROOT, "tests", "cpp", "reference_tests")


def build_reference_tests():
    """The reference's test headers compiled, unchanged and where they lie, against include/ of this library (their
    #include <fused_kernel/...> lines resolve to the forwarding headers): most of their checks are static_asserts, so
    compiling is already the larger part of the test; the programs run on the GPU box.  Nothing when no reference checkout
    is present."""
    if not os.path.isfile(os.path.join(REFERENCE_ROOT, REFERENCE_TESTS[0])):
        return []
    import tempfile
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(REFERENCE_TESTS_DIR, exist_ok=True)

    def compile_one(header):
        name = os.path.splitext(os.path.basename(header))[0]
        out = os.path.join(REFERENCE_TESTS_DIR, name)
        with tempfile.TemporaryDirectory() as tmp:
            main = os.path.join(tmp, name + ".cpp")
            with open(main, "w") as f:
                f.write("#include <%s>\nint main() { return launch(); }\n" % header)
            _run([hipcc(), "-x", "hip", main, "-I" + INCLUDE, "-I" + REFERENCE_ROOT, *DEVICE_FLAGS, "-L" + HERE, "-lfk_hip_rt",
                  "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/../../../fusedkernellibrary_amd", "-o", out])
        return out

    with ThreadPoolExecutor(max_workers=4) as pool:
        return list(pool.map(compile_one, REFERENCE_TESTS))


def build_literal_capi():
    """The same chain entry points built with the reference's host-branch interpolation (bilinear row index taken from
    the x coordinate): only there to show parity with the reference CPU backend's own output where that is defined."""
    return build_capi(extra_defines=("FK_INTERPOLATE_Y1_FROM_X",), name="libfk_capi_literal.so")


def build_all():
    """Everything, the independent hipcc runs side by side (each is single-threaded)."""
    from concurrent.futures import ThreadPoolExecutor
    outs = [build_runtime()]  # the others link against it
    with ThreadPoolExecutor(max_workers=4) as pool:
        jobs = [pool.submit(build_capi), pool.submit(build_literal_capi), pool.submit(build_cpp_tests), pool.submit(build_benchmarks),
                pool.submit(build_reference_tests)]
        for job in jobs:
            res = job.result()
            outs += res if isinstance(res, list) else [res]
    return outs


if __name__ == "__main__":
    for path in build_all():
        print(path)
