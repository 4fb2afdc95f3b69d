"""The reference's own unit tests (testing/*.cu, with its harness testing/unittest/) are compiled
unchanged against include/ — syntax and semantic analysis of the host and the device pass, no code
generation.  tests/golden/reference_unit_tests.json lists the files that compile; each must still
compile, and none may take a header from another Thrust on the include path.  Needs the reference
tree and hipcc; skipped where either is missing."""
import json
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_TESTING = "/root/reference/testing"
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

with open(os.path.join(ROOT, "tests", "golden", "reference_unit_tests.json")) as f:
    GOLDEN = json.load(f)


def _check(name):
    cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only", "-w", "-H", "-ferror-limit=3",
           "-I" + os.path.join(ROOT, "include"), "-I" + REF_TESTING, os.path.join(REF_TESTING, name + ".cu")]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    foreign = sorted({ln.split()[-1] for ln in p.stderr.splitlines()
                      if ln.startswith(".") and "/include/thrust/" in ln and not ln.split()[-1].startswith((ROOT, REF_TESTING))})
    errors = [ln for ln in p.stderr.splitlines() if " error: " in ln][:3]
    return name, p.returncode, errors, foreign


@pytest.mark.skipif(not os.path.isdir(REF_TESTING) or not os.path.exists(HIPCC), reason="needs the reference tree and hipcc")
def test_reference_unit_tests_compile_unchanged():
    present = {f[:-3] for f in os.listdir(REF_TESTING) if f.endswith(".cu")}
    assert set(GOLDEN["compiling"]) | set(GOLDEN["not_compiling"]) == present
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(_check, GOLDEN["compiling"]))
    broken = {name: errors for name, rc, errors, _ in results if rc != 0}
    assert not broken, broken
    leaked = {name: foreign for name, _, _, foreign in results if foreign}
    assert not leaked, leaked
