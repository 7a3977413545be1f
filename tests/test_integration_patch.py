"""The LAPIS-side patch (integration/lapis_hip_kernels.patch): applies to the reference tree, carries the lit
tests kept unpacked beside it, and those tests say what they should."""
import os
import re
import shutil
import subprocess

import pytest

from conftest import ROOT

PATCH = os.path.join(ROOT, "integration", "lapis_hip_kernels.patch")
UNPACKED = os.path.join(ROOT, "integration", "tests", "Dialect", "Kokkos")
REFERENCE = "/root/reference"


def _new_files(patch_text):
    """{path: content} of the files the patch creates."""
    files = {}
    for block in re.split(r"^diff -ruN ", patch_text, flags=re.M)[1:]:
        m = re.search(r"^\+\+\+ b/(\S+)", block, re.M)
        hunks = re.findall(r"^@@ -(\d+),?(\d*) \+(\d+),?(\d*) @@\n((?:[ +\-\\].*\n?)*)", block, re.M)
        if len(hunks) == 1 and hunks[0][0] == "0":
            body = "".join(line[1:] + "\n" for line in hunks[0][4].splitlines() if line.startswith("+"))
            files[m.group(1)] = body
    return files


@pytest.mark.skipif(not (os.path.isdir(REFERENCE) and shutil.which("patch")),
                    reason="needs the reference tree and the patch tool on this machine")
def test_patch_applies_cleanly_to_the_reference_tree():
    proc = subprocess.run(["patch", "--dry-run", "-p1", "-d", REFERENCE, "-i", PATCH], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "FAILED" not in proc.stdout and "fuzz" not in proc.stdout and "offset" not in proc.stdout, proc.stdout
    for touched in ("TranslateToKokkosCpp.cpp", "KokkosLoopMapping.cpp", "lapis-translate.cpp", "Passes.td",
                    "CsrSpmvMatch.h", "hip_spmv_0.mlir.gold"):
        assert touched in proc.stdout


def test_patch_carries_the_unpacked_lit_tests():
    new = _new_files(open(PATCH).read())
    names = sorted(os.listdir(UNPACKED))
    assert names == ["hip_spmv_0.mlir", "hip_spmv_0.mlir.gold", "hip_spmv_1.mlir", "hip_spmv_1.mlir.gold",
                     "hip_spmv_translate_0.mlir", "hip_spmv_translate_0.mlir.gold", "hip_spmv_translate_1.mlir",
                     "hip_spmv_translate_1.mlir.gold"]
    for name in names:
        assert new["tests/Dialect/Kokkos/" + name] == open(os.path.join(UNPACKED, name)).read(), name


def _values_defined_in_order(ir):
    nums = [int(n) for n in re.findall(r"^\s*%(\d+) = ", ir, re.M)]
    return nums == list(range(len(nums)))


def test_gold_files_say_what_the_change_is_for():
    read = lambda n: open(os.path.join(UNPACKED, n)).read()
    pos_gold, neg_gold = read("hip_spmv_0.mlir.gold"), read("hip_spmv_1.mlir.gold")
    assert _values_defined_in_order(pos_gold) and _values_defined_in_order(neg_gold)
    before_launch = lambda ir: ir[:ir.index('"kokkos.thread_parallel"')]
    # matched nest: nothing is loaded on the host before the launch and the hint is the constant zero
    assert "memref.load" not in before_launch(pos_gold)
    assert '"kokkos.thread_parallel"(%dim, %c0)' in pos_gold
    # negative case: the estimate (R[N] - R[0] + N - 1) / N of KokkosLoopMapping.cpp:279-323 stays
    head = before_launch(neg_gold)
    assert head.count("memref.load %arg1[") == 2 and "arith.divui" in head and "arith.maximumf" in neg_gold
    assert '"kokkos.thread_parallel"(%dim, %7)' in neg_gold
    # both inputs are the same nest apart from the reduction
    strip = lambda s: re.sub(r"//[^\n]*\n", "", s)
    assert strip(read("hip_spmv_0.mlir")).replace("arith.addf", "arith.maximumf") == strip(read("hip_spmv_1.mlir"))
    # the translate tests feed the mapped IR (the golds above) to lapis-translate --hip-kernels
    assert strip(read("hip_spmv_translate_0.mlir")).strip() == pos_gold.strip()
    assert strip(read("hip_spmv_translate_1.mlir")).strip() == neg_gold.strip()
    assert read("hip_spmv_translate_0.mlir.gold") == "7\n" and read("hip_spmv_translate_1.mlir.gold") == "3\n"


def test_emitted_call_matches_the_library_header():
    # the argument order the patch prints is the one include/lapis_hip.h declares
    patch = open(PATCH).read()
    header = open(os.path.join(ROOT, "include", "lapis_hip.h")).read()
    decl = re.search(r"int lapis_hip_spmv_csr_f64_i32\(([^;]*)\);", header, re.S).group(1)
    params = [p.split()[-1].lstrip("*") for p in decl.replace("\n", " ").split(",")]
    assert params == ["plan", "nrows", "ncols", "pos", "crd", "val", "x", "y", "stream"]
    assert "for(Value v : {m.pos, m.crd, m.val, m.x, m.y})" in patch  # after plan, rows, columns
    create = re.search(r"int lapis_hip_csr_plan_create\(([^;]*)\);", header, re.S).group(1)
    cparams = [p.split()[-1].lstrip("*") for p in create.replace("\n", " ").split(",")]
    assert cparams == ["plan", "nrows", "ncols", "nnz", "pos", "crd", "value_bytes", "stream"]
