"""The backend's host code under AddressSanitizer and UndefinedBehaviorSanitizer, as the
reference builds its own test binary (-fsanitize=address,undefined, Makefile:4 there).
`make -C polygrad_amd/csrc asan` compiles the library's host side (kernel-graph analysis,
index simplifier, renderer, templates, plan-level fusion, plan-file loader) and the
host_check driver with both sanitizers; this test runs the driver over every committed
schedule, and over truncated and bit-flipped copies of the small ones (a damaged file may
be rejected, never crash).  A sanitizer report makes the driver exit non-zero."""
import glob
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "polygrad_amd", "csrc")
DRIVER = os.path.join(CSRC, "build_asan", "host_check")


@pytest.fixture(scope="module")
def driver():
    if not os.path.exists(DRIVER):
        subprocess.run(["make", "-C", CSRC, "-j8", "asan"], check=True, capture_output=True)
    return DRIVER


def run(driver, args, timeout):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    r = subprocess.run([driver] + args, capture_output=True, text=True, timeout=timeout, env=env)
    tail = "\n".join((r.stdout + r.stderr).splitlines()[-30:])
    assert r.returncode == 0, tail
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, tail
    return r.stdout


def test_every_golden_schedule_and_damaged_copies(driver):
    files = sorted(glob.glob(os.path.join(HERE, "golden", "*.polyplan")))
    small = [f for f in files if os.path.getsize(f) < 150_000]
    assert len(small) >= 20
    out = run(driver, ["--garbage"] + small, 600)
    assert "0 problems" in out
    rejected = int(out.split(" damaged copies rejected")[0].split()[-1])
    assert rejected > 8 * len(small), "truncated files must be rejected by the loader"


def test_benchmark_schedules(driver):
    """The full-size plans (GPT-2 small forward, the training block, the sweeps)."""
    files = sorted(glob.glob(os.path.join(HERE, "..", "polygrad_amd", "plans", "*.polyplan")))
    files += sorted(glob.glob(os.path.join(HERE, "golden", "fullsize", "*.polyplan")))
    files = [f for f in files if "b1_t1024" not in os.path.basename(f) or "block0" in f]   # the B=1 twin of the B=8 plan adds a minute and nothing new
    if not os.environ.get("POLY_SLOW_TESTS"):
        # the 24-layer training step is the one-block step 24 times over (2770 kernels, five
        # minutes under the sanitizers); the one-block plan goes through the same code
        files = [f for f in files if "train_24l" not in os.path.basename(f)]
    out = run(driver, files, 900)
    assert "0 problems" in out
