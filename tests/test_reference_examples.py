"""The reference's own example programs, compiled UNCHANGED against include/thrust (hipcc) and run:
their output must satisfy the golden outputs the reference keeps for them
(internal/test/thrust.example.*.filecheck, held as data in tests/golden/example_outputs.json).

The binaries are built from the reference tree where it is present (oracle/Makefile, target
ref_examples, into oracle/_ref/examples/); the GPU test runs whatever was built."""
import json
import os
import re
import subprocess

import pytest

from conftest import ROOT

REF = "/root/reference"
BIN_DIR = os.path.join(ROOT, "oracle", "_ref", "examples")
with open(os.path.join(ROOT, "tests", "golden", "example_outputs.json")) as f:
    GOLDEN = json.load(f)

# examples this device system runs: all of the reference's examples/ (none is left out today)
NOT_BUILT = {}
EXAMPLES = sorted(set(GOLDEN) - set(NOT_BUILT))


def pattern_of(text):
    """A FileCheck pattern: literal text with {{regex}} parts; runs of blanks match any blanks."""
    parts = re.split(r"(\{\{.*?\}\})", text.strip())
    rx = ""
    for p in parts:
        if p.startswith("{{") and p.endswith("}}"):
            rx += "(?:" + p[2:-2] + ")"
        else:
            rx += r"[ \t]+".join(re.escape(w) for w in re.split(r"[ \t]+", p))
    return re.compile(rx)


def filecheck(output, checks):
    """None when the output satisfies the directives, else a message.  CHECK: some later line
    matches; CHECK-NEXT: the line after the previous match does; CHECK-SAME: the rest of the line of
    the previous match does."""
    lines = output.splitlines()
    at, col = -1, 0  # line of the previous match and the column behind it
    for kind, text in checks:
        rx = pattern_of(text)
        if kind == "CHECK":
            for i in range(at + 1 if at >= 0 else 0, len(lines)):
                m = rx.search(lines[i])
                if m:
                    at, col = i, m.end()
                    break
            else:
                return f"no line after line {at + 1} matches CHECK: {text!r}"
        elif kind == "CHECK-NEXT":
            if at + 1 >= len(lines):
                return f"output ends before CHECK-NEXT: {text!r}"
            m = rx.search(lines[at + 1])
            if not m:
                return f"line {at + 2} is {lines[at + 1]!r}, expected CHECK-NEXT: {text!r}"
            at, col = at + 1, m.end()
        else:  # CHECK-SAME
            m = rx.search(lines[at], col) if at >= 0 else None
            if not m:
                return f"rest of line {at + 1} does not match CHECK-SAME: {text!r}"
            col = m.end()
    return None


def test_filecheck_matcher():
    assert filecheck("a\nsum is 45\nnext 7\n", [["CHECK", "sum is 45"], ["CHECK-NEXT", "next {{[0-9]+}}"]]) is None
    assert filecheck("x   y\n", [["CHECK", "x y"]]) is None
    assert filecheck("a\nb\nc\n", [["CHECK", "a"], ["CHECK-NEXT", "c"]]) is not None
    assert filecheck("a b\n", [["CHECK", "a"], ["CHECK-SAME", "b"]]) is None
    assert filecheck("a\n", [["CHECK", "b"]]) is not None


@pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "examples")), reason="the reference tree is not here")
def test_reference_examples_compile_unchanged():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-j", "8", "ref_examples"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    for name in EXAMPLES:
        assert os.path.exists(os.path.join(BIN_DIR, name)), name


@pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "examples")), reason="the reference tree is not here")
def test_a_header_that_is_not_provided_says_so(tmp_path):
    # never a silent fall-through to another Thrust on the include path (/opt/rocm/include/thrust)
    src = tmp_path / "t.cu"
    src.write_text("#include <thrust/system/cuda/vector.h>\nint main() { return 0; }\n")
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-fsyntax-only", "-I",
                        os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert r.returncode != 0
    assert "is not provided by the cdna4 device system" in r.stderr


def test_every_public_header_name_of_the_reference_exists_here():
    # implemented or an #error stub: nothing can resolve to a foreign <thrust/...>
    names = json.load(open(os.path.join(ROOT, "tests", "golden", "public_headers.json")))
    missing = [n for n in names if not os.path.exists(os.path.join(ROOT, "include", "thrust", n))]
    assert not missing, missing


@pytest.mark.gpu
@pytest.mark.parametrize("name", EXAMPLES)
def test_reference_example_output(name):
    path = os.path.join(BIN_DIR, name)
    if not os.path.exists(path):
        pytest.skip("not built (the reference tree was absent when the tree was built)")
    r = subprocess.run([path], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    problem = filecheck(r.stdout, GOLDEN[name]["checks"])
    assert problem is None, problem + "\n--- output ---\n" + r.stdout[-3000:]
