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
                    "CsrSpmvMatch.h", "LibraryLoopMatch.h", "hip_spmv_0.mlir.gold", "hip_spmm_translate_0.mlir",
                    "hip_depth1_translate_0.mlir"):
        assert touched in proc.stdout


def test_patch_carries_the_unpacked_lit_tests():
    new = _new_files(open(PATCH).read())
    names = sorted(os.listdir(UNPACKED))
    stems = ["hip_depth1_translate_0", "hip_depth1_translate_1", "hip_spmm_translate_0", "hip_spmm_translate_1",
             "hip_spmv_0", "hip_spmv_1", "hip_spmv_translate_0", "hip_spmv_translate_1", "hip_spmv_translate_2"]
    assert names == sorted(n + ext for n in stems for ext in (".mlir", ".mlir.gold"))
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
    # the same nest inside scf.while: one more line, the hand-over to lapis_hip_csr_plan_analyze
    inside = strip(read("hip_spmv_translate_2.mlir"))
    assert "scf.while" in inside and read("hip_spmv_translate_2.mlir.gold") == "8\n"
    nest = lambda ir: re.sub(r"\s+", " ", ir[ir.index('"kokkos.thread_parallel"'):ir.index("}) : (index, index) -> ()")])
    assert nest(inside) == nest(pos_gold)


def test_depth1_and_spmm_lit_tests_count_what_their_functions_say():
    read = lambda n: open(os.path.join(UNPACKED, n)).read()
    funcs = lambda ir: re.findall(r"func\.func @(\w+)", ir)
    # positives: one library call per function + lapis_hip_init + lapis_hip_finalize
    pos = read("hip_depth1_translate_0.mlir")
    assert funcs(pos) == ["inner", "combine", "hadamard", "duplicate", "clear"]
    assert read("hip_depth1_translate_0.mlir.gold") == "%d\n" % (len(funcs(pos)) + 2)
    # negatives: a device lambda per function that runs on the device (executionSpace = 1) + init + finalize
    neg = read("hip_depth1_translate_1.mlir")
    on_device = neg.count("executionSpace = 1 : i64, parallelLevel = 0 : i64")
    assert len(funcs(neg)) == 4 and on_device == 3
    assert read("hip_depth1_translate_1.mlir.gold") == "%d\n" % (on_device + 2)
    # SpMM: matches + create + call + destroy twice per function
    spmm = read("hip_spmm_translate_0.mlir")
    assert funcs(spmm) == ["rows_range", "rows_threads"] and "memref<?xi32>" in spmm
    assert read("hip_spmm_translate_0.mlir.gold") == "%d\n" % (5 * len(funcs(spmm)) + 2)
    neg = read("hip_spmm_translate_1.mlir")
    assert funcs(neg) == ["wide_positions", "transposed_operand"] and "memref<?xindex>" in neg
    assert "%arg4[%arg7, %6]" in neg and "%arg4[%4, %arg7]" in neg  # one multiplies by the transposed operand
    assert read("hip_spmm_translate_1.mlir.gold") == "%d\n" % (len(funcs(neg)) + 2)
    # the Python restatement of the matchers agrees on the same bodies written as scf loops (tests/loop_nests.py)
    import loop_nests
    from lapis_amd import loop_mapping as lm
    kinds = lambda text: [(bool(n.csr_spmv), (n.depth1 or {}).get("kind"), bool(n.csr_spmm))
                          for nests in lm.map_module(text, hip_kernels=True).values() for n in nests]
    assert kinds(loop_nests.DOT) == [(False, "dot", False)]
    assert kinds(loop_nests.DOT_PRODUCT_REDUCTION) == [(False, None, False)]
    assert kinds(loop_nests.elementwise(loop_nests.AXPBY_BODY)) == [(False, "axpby", False)]
    assert kinds(loop_nests.elementwise(loop_nests.CUBE_BODY)) == [(False, None, False)]
    assert kinds(loop_nests.spmm_i32("f32", "scf.parallel")) == kinds(loop_nests.spmm_i32("f64", "scf.for")) == [(False, None, True)]


def test_every_library_call_the_patch_emits_is_declared_in_the_header():
    patch = open(PATCH).read()
    header = open(os.path.join(ROOT, "include", "lapis_hip.h")).read()
    declared = set(re.findall(r"\b(lapis_hip_\w+)\s*\(", header))
    added = "\n".join(l[1:] for l in patch.splitlines() if l.startswith("+") and not l.startswith("+++"))
    emitter = added[added.index("// ---- gfx950 kernel library"):added.index("hip-kernels replaces device-level launches")]
    literal = set(re.findall(r'"[^"]*?\b(lapis_hip_[a-z0-9_]+)\(', emitter))
    assert {"lapis_hip_csr_plan_create", "lapis_hip_csr_plan_matches", "lapis_hip_csr_plan_analyze",
            "lapis_hip_csr_plan_destroy", "lapis_hip_spmv_csr_f64_i32", "lapis_hip_spmm_csr_f32_i32_plan",
            "lapis_hip_last_error", "lapis_hip_init", "lapis_hip_finalize"} <= literal
    assert literal <= declared, literal - declared
    # names built from an element type: lapis_hip_<op>_ << t << ...
    for stem, tail in re.findall(r'"(lapis_hip_[a-z_]+_)" << t << "(\w*)\(', emitter):
        for t in ("f64", "f32"):
            assert stem + t + tail in declared, stem + t + tail
    # the plan is keyed on the structure and on the generation of the operands, never on addresses alone
    assert "lapis_hip_operand_generation++" in added and "!= lapis_hip_operand_generation || !lapis_hip_csr_plan_matches(" in emitter
    matches = re.search(r"int lapis_hip_csr_plan_matches\(([^;]*)\);", header, re.S).group(1)
    assert [p.split()[-1].lstrip("*") for p in matches.replace("\n", " ").split(",")] == ["plan", "nrows", "ncols", "nnz", "pos", "crd"]


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
