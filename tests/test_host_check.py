"""Host-side bounds check of the direct-to-LDS kernels (csrc/host_check.hpp, `make host-check`), run here in its short
form.

The library is rebuilt with -DMI_HOST_CHECK under AddressSanitizer and UndefinedBehaviorSanitizer: its own host code
(argument validation, workspace layout, cost model, step grouping, launchers) runs unchanged, and every launch of the
fast kernel is walked workgroup by workgroup and lane by lane through the address functions the device code itself
uses (the `MI_HD` functions of gemm_fast.hpp), each access checked against the buffers of the call.  The kernels that
guard their own accesses (normalisation passes, transposes, the general tile kernel, the per-head kernels) are checked
one level up: every launch site states the block of memory each pointer argument covers, and each block must lie inside
one buffer of the call (one segment of the workspace, for the single-call driver).  The driver program sweeps the C entry points over the benchmark shapes, the shapes of the GPU tests and sizes on both sides of
every tile edge.  No GPU is involved.
"""
import os
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "emerging-optimizers_amd", "csrc")


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("hostcheck")
    subprocess.run(["make", "-j8", "-C", CSRC, f"HCDIR={out}", f"{out}/host_check"], check=True, capture_output=True, timeout=900)
    return os.path.join(out, "host_check")


def test_checker_reports_undersized_buffers(checker):
    """A result one row short, an operand one K tile short and an addend 16 bytes short must each be reported, and so
    must a normalisation call whose output or whose array of partial sums is too small."""
    res = subprocess.run([checker, "--selftest"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "selftest" in res.stdout


def test_every_fast_kernel_access_stays_inside_its_buffers(checker):
    res = subprocess.run([checker, "--quick"], capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, (res.stdout + res.stderr)[-4000:]
    assert " 0 failures" in res.stdout and "ERROR: AddressSanitizer" not in res.stderr and "runtime error" not in res.stderr
    # the sweep really went through the launchers: hundreds of calls, thousands of launches
    words = res.stdout.split()
    calls, launches, others = int(words[1]), int(words[words.index("fast-kernel") - 1]), int(words[words.index("other") - 1])
    assert calls > 500 and launches > 2000 and others > 1000, res.stdout
