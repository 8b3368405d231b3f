"""The product's plain-C host layer under AddressSanitizer + UBSan, on the CPU.

`make -C oracle asan` compiles iree_amd/csrc/uk_host.c and uk_plugin.c with
gcc's sanitizers against CPU stand-ins of the internal HIP C-ABI
(oracle/asan_hip_stubs.c: device memory is host memory, a launch runs the
oracle) and links the driver oracle/asan_host_driver.c, which checks staging of
host operands against the oracle over whole buffers, the contract-violation
reports, the early returns and the executable-plugin face. The reference offers
the same for its host code (CMakeLists.txt:552-555, IREE_ENABLE_ASAN). GPU code
is not involved: the sanitizers never see a kernel."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("gcc") is None or shutil.which("make") is None,
                    reason="needs gcc and make")
def test_host_layer_and_oracle_under_asan_ubsan():
    build = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    run = subprocess.run([os.path.join(ROOT, "oracle", "_asan", "asan_host_driver")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                         timeout=300)
    assert run.returncode == 0, run.stdout
    assert "asan_host_driver: ok" in run.stdout
