"""CPU-only: the register budget of the precompiled kernels, from the compiler's own report.

The kernels of the hot path are written against a budget of 128 VGPRs (four wavefronts per SIMD);
a source change that looks neutral can push one of them over it, and the compiler then spills
registers to scratch memory without a word — the kernel stays correct and loses a third of its
throughput.  The build leaves `-Rpass-analysis=kernel-resource-usage` of every object in
thrust_amd/csrc/build/*.usage.txt; this test reads them."""
import glob
import os
import re
import subprocess

from conftest import ROOT

BUILD = os.path.join(ROOT, "thrust_amd", "csrc", "build")

# Known and accepted: the in-place (ticketed) scan of 64-bit elements with multiplies / maximum /
# minimum keeps 16 chunks of 64-bit values and the ticket bookkeeping live at once.
ACCEPTED = re.compile(r"_ZN3tcd11scan_kernelI[lmd]NS_(12OpMultiplies|9OpMaximum|9OpMinimum)ELi512ELi16ELb1E")
SMALL = 2  # a register or two spilled outside the main loop costs nothing measurable


def usage():
    files = sorted(glob.glob(os.path.join(BUILD, "*.usage.txt")))
    if len(files) < 9:  # normally left by __graft_entry__.build()
        subprocess.run(["make", "-C", os.path.join(ROOT, "thrust_amd", "csrc"), "-B", "-j", "8"], check=True,
                       capture_output=True)
        files = sorted(glob.glob(os.path.join(BUILD, "*.usage.txt")))
    kernels = {}
    for f in files:
        name = None
        for line in open(f):
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name = m.group(1)
                kernels[name] = {}
                continue
            m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
            if m and name:
                kernels[name][m.group(1).strip()] = int(m.group(2))
    return kernels


def test_every_object_reports_its_kernels():
    k = usage()
    for needle in ["onesweep_kernel", "radix_hist_kernel", "tile_sort_kernel", "scan_kernel", "scan_by_key_kernel",
                   "reduce_by_key_kernel", "histogram_kernel"]:
        assert any(needle in name for name in k), needle
    assert len(k) > 500  # every (type, operator, variant) instantiation


def test_hot_kernels_do_not_spill():
    bad = []
    for name, u in usage().items():
        if ACCEPTED.search(name):
            continue
        if u.get("VGPRs Spill", 0) > SMALL:
            bad.append((name, u.get("VGPRs"), u.get("VGPRs Spill")))
    assert not bad, bad[:10]


def test_hot_kernels_keep_four_wavefronts_per_simd():
    # 128 VGPRs at most for the kernels that are sized for two 512-thread (or one 1024-thread)
    # workgroups per CU
    over = []
    for name, u in usage().items():
        if any(s in name for s in ["onesweep_kernel", "scan_by_key_kernel", "reduce_by_key_kernel", "scan_kernel"]):
            if u.get("VGPRs", 0) > 128:
                over.append((name, u["VGPRs"]))
    assert not over, over[:10]


def test_lds_fits_the_workgroups_per_compute_unit_the_kernels_are_sized_for():
    # 160 KiB of LDS per compute unit: two 512-thread workgroups of the scan and by-key kernels, one
    # workgroup of a onesweep pass (the tile's keys are staged whole)
    over = []
    for name, u in usage().items():
        lds = u.get("LDS Size", 0)
        if any(s in name for s in ["scan_by_key_kernel", "reduce_by_key_kernel", "scan_kernel", "scan_packed_kernel"]) and lds > 80 * 1024:
            over.append((name, lds))
        if lds > 160 * 1024:
            over.append((name, lds))
    assert not over, over[:10]
    assert any(u.get("LDS Size", 0) > 60 * 1024 for u in usage().values())  # the report is being read


def test_the_by_key_objects_of_the_four_key_widths_share_no_symbol():
    """bykey.hip is compiled once per key width into one library, and the key type is a file-level
    alias: a template of one name in two of the objects can differ in its body, and a linker keeps
    one copy of a weak symbol.  A kernel's host stub folded like that makes every key width launch
    one width's kernel.  Each build has a namespace of its own; nothing weak may be common to two
    objects."""
    usage()  # builds the objects where they are missing
    weak = {}
    for k in (1, 2, 4, 8):
        out = subprocess.run(["nm", os.path.join(BUILD, "bykey_k%d.o" % k)], stdout=subprocess.PIPE, text=True, check=True).stdout
        weak[k] = {line.split()[-1] for line in out.splitlines() if len(line.split()) == 3 and line.split()[1] in "WVu"}
        assert len(weak[k]) >= 100, (k, len(weak[k]))  # the kernels' host stubs
    for a in (1, 2, 4, 8):
        for b in (1, 2, 4, 8):
            if a < b:
                assert not (weak[a] & weak[b]), (a, b, sorted(weak[a] & weak[b])[:5])
