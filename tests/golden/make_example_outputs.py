"""Writes tests/golden/example_outputs.json from the golden outputs the reference keeps for its
example programs (internal/test/thrust.example.<name>.filecheck).  Only data is taken: the
expected output lines, as FileCheck directives (CHECK / CHECK-NEXT / CHECK-SAME, with {{regex}}
parts kept as they are).  Run in a container that has the reference tree:

    python tests/golden/make_example_outputs.py /root/reference
"""
import glob
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
out = {}
for path in sorted(glob.glob(os.path.join(ref, "internal", "test", "thrust.example.*.filecheck"))):
    name = os.path.basename(path)[len("thrust.example."):-len(".filecheck")]
    if name.startswith("cuda."):
        continue  # CUDA-runtime examples: outside this device system
    checks = []
    for line in open(path).read().splitlines():
        m = re.match(r"\s*(CHECK(?:-NEXT|-SAME)?):\s?(.*)$", line)
        if m:
            checks.append([m.group(1), m.group(2)])
    out[name] = {"source": f"internal/test/{os.path.basename(path)}", "checks": checks}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "example_outputs.json"), "w") as f:
    json.dump(out, f, indent=1)
print(len(out), "examples")
