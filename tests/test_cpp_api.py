"""The C++ side as a user sees it: programs under tests/cpp compiled against include/ by the build step."""
import os
import subprocess

import numpy as np
import pytest

from conftest import same_bits
from oracle import binding as B

HERE = os.path.dirname(os.path.abspath(__file__))


def test_host_api_conformance(native_build):
    exe = os.path.join(HERE, "cpp", "conformance")
    assert os.path.exists(exe), "tests/cpp/conformance is not built (python -m fusedkernellibrary_amd.build)"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert proc.returncode == 0, proc.stdout
    assert "conformance ok" in proc.stdout


def test_launch_plans_on_the_host(native_build):
    """Decisions of the host-side plan that no GPU test can reach or see: a three-byte source whose window spans 4 GiB or
    more keeps 64-bit addressing (no tile, no touch); a ragged batch takes its alignment from the whole box; a batch
    launched in parts carries the whole batch's box.  No GPU call is made, the pointers are made up."""
    exe = os.path.join(HERE, "cpp", "host_plan_check")
    assert os.path.exists(exe), "tests/cpp/host_plan_check is not built (python -m fusedkernellibrary_amd.build)"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert proc.returncode == 0 and "host plans: ok" in proc.stdout, proc.stdout


def test_staging_ring_state_machine(native_build):
    """The slots behind fkrt_params_upload / fkrt_params_release with the GPU runtime replaced by stand-ins: a ninth block
    never overwrites one of eight that are leased, a slot comes back only after its event, the wait for an event does not
    hold the ring's mutex, twelve host threads never see each other's blocks."""
    exe = os.path.join(HERE, "cpp", "staging_ring_check")
    assert os.path.exists(exe), "tests/cpp/staging_ring_check is not built (python -m fusedkernellibrary_amd.build)"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and "staging ring: ok" in proc.stdout, proc.stdout


@pytest.mark.gpu
def test_readme_example_as_user_code(oracle, tmp_path):
    exe = os.path.join(HERE, "cpp", "readme_dropin")
    assert os.path.exists(exe), "tests/cpp/readme_dropin is not built"
    src = oracle.bytes(1, (2160, 3840, 3))
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    src.tofile(fin)
    proc = subprocess.run([exe, str(fin), str(fout)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0, proc.stdout
    got = np.fromfile(fout, np.float32).reshape(5, 60, 60, 3)
    rects = [(0, 0, 34, 25), (10, 10, 70, 15), (20, 20, 60, 59), (30, 30, 20, 23), (40, 40, 12, 11)]
    want = oracle.crop_resize_muls_bgr_tensor(src, rects, (60, 60), B.PRESERVE_AR, (0, 0, 0), (1.4,) * 3, (0.5,) * 3, (255.,) * 3)
    assert same_bits(got, want)


@pytest.mark.gpu
def test_executor_surface_as_user_code():
    exe = os.path.join(HERE, "cpp", "api_gpu")
    assert os.path.exists(exe), "tests/cpp/api_gpu is not built"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0 and "api_gpu ok" in proc.stdout, proc.stdout


@pytest.mark.gpu
def test_user_code_that_includes_the_hip_runtime_header_first():
    """<hip/hip_runtime.h> before <fused_kernel/fused_kernel.h> in one translation unit: a chain on a stream made by the
    HIP API, timed with HIP events."""
    exe = os.path.join(HERE, "cpp", "hip_header_coexistence")
    assert os.path.exists(exe), "tests/cpp/hip_header_coexistence is not built"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0 and "hip_header_coexistence ok" in proc.stdout, proc.stdout


@pytest.mark.gpu
def test_reference_benchmark_sweeps_run_and_check_themselves():
    """The reference's four benchmark sweeps as user code (two timed iterations here): every sweep point compares its two
    variants with each other and with the closed-form result, and the program exits non-zero on any mismatch."""
    import json
    exe = os.path.join(os.path.dirname(HERE), "fusedkernellibrary_amd", "benchmarks", "reference_sweeps")
    assert os.path.exists(exe), "benchmarks/reference_sweeps is not built (python -m fusedkernellibrary_amd.build)"
    proc = subprocess.run([exe, "all", "2"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    rows = [json.loads(line) for line in proc.stdout.splitlines() if line.startswith("{")]
    assert proc.returncode == 0 and len(rows) == 155 and all(r["passed"] for r in rows), proc.stdout[-2000:]
