"""The host side of libodc_hip.so under AddressSanitizer and UndefinedBehaviorSanitizer.

odc_amd/csrc/odc_host.cpp (the C ABI, the arena allocator, the argument and overflow checks,
the launch planning) is plain C++; linked with tests/cpu/no_device.cpp instead of the gfx950
device side it builds with g++ alone. This test builds that library with
``-fsanitize=address,undefined`` and runs the host-side test files against it in a child
interpreter (``ODC_HIP_LIBRARY`` points the binding at it; the sanitizer runtime has to be loaded
before Python, hence the preload in the child's environment only). A memory error or undefined
behaviour anywhere in the allocator model test, the dry-run launch plans or the error paths
aborts the child.
"""

import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "odc_amd" / "csrc"
HOST_TESTS = ["tests/test_host_launch_plans.py", "tests/test_host_logic.py"]


def _gcc_file(name: str) -> str:
    return subprocess.run(["gcc", f"-print-file-name={name}"], capture_output=True, text=True, check=True).stdout.strip()


@pytest.fixture(scope="module")
def sanitized_env(tmp_path_factory):
    lib = tmp_path_factory.mktemp("host_asan") / "libodc_host_check.so"
    cmd = [
        "g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
        "-Wall", "-Wextra", "-Werror", "-Wno-unknown-pragmas", "-shared", "-fPIC",
        f"-I{ROOT / 'include'}", f"-I{CSRC}", str(CSRC / "odc_host.cpp"), str(ROOT / "tests" / "cpu" / "no_device.cpp"),
        "-o", str(lib),
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    asan = _gcc_file("libasan.so")
    assert os.path.isabs(asan), "g++ has no AddressSanitizer runtime"
    env = dict(os.environ)
    # the sanitizer runtime must come first; whatever is preloaded already stays
    env["LD_PRELOAD"] = " ".join(x for x in (asan, env.get("LD_PRELOAD", "")) if x)
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"  # CPython itself does not free everything
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    env["ODC_HIP_LIBRARY"] = str(lib)
    env["ODC_EXPECT_SANITIZED"] = "1"
    probe = subprocess.run([sys.executable, "-c", "pass"], env=env, capture_output=True, text=True)
    if probe.returncode != 0:
        pytest.skip(f"this environment does not let the sanitizer runtime be preloaded: {probe.stderr[-300:]}")
    return env


def test_host_side_tests_pass_under_asan_and_ubsan(sanitized_env):
    proc = subprocess.run(
        [sys.executable, "-m", "pytest", *HOST_TESTS, "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"],
        cwd=ROOT, env=sanitized_env, capture_output=True, text=True, timeout=900,
    )
    tail = proc.stdout[-3000:] + proc.stderr[-3000:]
    assert proc.returncode == 0, tail
    assert " passed" in proc.stdout and "failed" not in proc.stdout, tail
    assert "sanitized" in proc.stdout or "skipped" not in proc.stdout.splitlines()[-1], tail


def test_the_host_side_needs_no_hip_header():
    """odc_host.cpp must stay plain C++: everything HIP is behind odc_launch.h."""
    text = (CSRC / "odc_host.cpp").read_text()
    assert "hip/hip_runtime" not in text and "__global__" not in text and "hipLaunch" not in text
