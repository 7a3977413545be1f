"""The level-selection rules (lapis_amd/loop_mapping.py) against what the reference's loop-mapping pass
produces: its four gold files (structure kept in tests/golden/loop_mapping_expected.json, and the files
themselves when the reference tree is present), the gold files of this repository's LAPIS-side patch, and
hand-worked cases for the rules those leave open."""
import json
import os
import re

import pytest

import loop_nests as nests
from conftest import ROOT
from lapis_amd import loop_mapping as lm

REFERENCE = "/root/reference"
EXPECTED = json.load(open(os.path.join(ROOT, "tests", "golden", "loop_mapping_expected.json")))


def to_lists(summary):
    if isinstance(summary, tuple):
        return [summary[0], [to_lists(c) for c in summary[1]]]
    return summary


def number_values(expr):
    if expr is None:
        return None
    seen = {}
    return re.sub(r"%[\w.$-]+", lambda m: seen.setdefault(m.group(0), "v%d" % len(seen)), expr)


def decided(text, **kw):
    (fn, mapped), = lm.map_module(text, **kw).items()
    return mapped


@pytest.mark.parametrize("name", sorted(nests.SHAPES))
def test_own_worded_nests_map_as_the_reference_gold_says(name):
    mapped = decided(nests.SHAPES[name])
    want = EXPECTED[name]
    assert [to_lists(n.summary()) for n in mapped] == want["nests"]
    hints = [[number_values(n.vector_length_hint), number_values(n.team_size_hint)] for n in mapped if n.depth >= 2 and n.space == "device"]
    assert hints == want["hints"]


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference tree is not on this machine")
@pytest.mark.parametrize("k", range(4))
def test_reference_inputs_map_to_reference_golds(k):
    base = os.path.join(REFERENCE, "tests", "Dialect", "Kokkos", "loop_mapping_%d.mlir" % k)
    mapped = decided(open(base).read())
    gold = open(base + ".gold").read()
    (fn, want), = lm.mapped_summary(gold).items()
    assert [n.summary() for n in mapped] == want
    (_, hints), = lm.mapped_hints(gold).items()
    mine = [(number_values(n.vector_length_hint), number_values(n.team_size_hint)) for n in mapped
            if n.depth >= 2 and n.space == "device"]
    assert mine == [(number_values(v), number_values(t)) for v, t in hints]
    # the fixture the other tests use is what these gold files say
    assert EXPECTED["loop_mapping_%d" % k]["nests"] == [to_lists(w) for w in want]


@pytest.mark.parametrize("name, is_spmv", [("hip_spmv_0", True), ("hip_spmv_1", False)])
def test_patch_golds_follow_the_same_rules(name, is_spmv):
    base = os.path.join(ROOT, "integration", "tests", "Dialect", "Kokkos", name + ".mlir")
    mapped = decided(open(base).read(), hip_kernels=True)
    gold = open(base + ".gold").read()
    (fn, want), = lm.mapped_summary(gold).items()
    assert [n.summary() for n in mapped] == want
    (_, hints), = lm.mapped_hints(gold).items()
    assert bool(mapped[0].csr_spmv) == is_spmv
    # the nest the kernel library takes over keeps no estimate; any other nest keeps the mean row length
    assert (mapped[0].vector_length_hint is None) == is_spmv
    assert (hints[0][0] is None) == is_spmv
    assert number_values(mapped[0].vector_length_hint) == number_values(hints[0][0])


def test_spmv_nest_is_recognised_with_its_buffers_by_role():
    m = decided(nests.spmv_i32("f32"))[0]
    assert m.depth == 2 and m.space == "device"
    assert m.csr_spmv == {"y": "%y", "pos": "%rowptr", "crd": "%colidx", "val": "%vals", "x": "%x", "elem": "f32"}
    assert decided(nests.SPMV_INDEX)[0].csr_spmv["pos"] == "%rowptr"


@pytest.mark.parametrize("old, new", [
    ("arith.addf %rhs, %lhs", "arith.maximumf %rhs, %lhs"),                 # another reduction
    ("arith.mulf %xv, %a", "arith.addf %xv, %a"),                           # another product
    ("memref.load %x[%col]", "memref.load %x[%e]"),                         # x not gathered through the coordinates
    ("memref.load %vals[%e]", "memref.load %vals[%k]"),                     # values not taken at the entry
    ("memref.store %sum, %y[%row]", "memref.store %sum, %x[%row]"),         # result goes elsewhere
    ("init (%acc0)", "init (%fzero)"),                                      # does not start from y[i]
    ("arith.addi %one, %row", "arith.addi %row, %row"),                     # row end is not pos[i+1]
    ("memref.load %colidx[%e]", "memref.load %colidx[%row]"),               # coordinate not taken at the entry
])
def test_near_misses_of_the_spmv_nest_are_not_taken_for_it(old, new):
    text = nests.spmv_i32("f64")
    assert old in text
    text = text.replace(old, new).replace("%one = arith.constant 1 : index",
                                          "%one = arith.constant 1 : index\n    %fzero = arith.constant 0.0 : f64")
    m = decided(text)[0]
    assert m.csr_spmv is None
    assert m.summary()[0] == "thread_parallel results=0"  # still a two-level nest, mapped as such


THREE_LEVELS_NO_RESULTS = """
module {
  func.func @scale(%t: memref<?x?x?xf64>, %row_scale: memref<?xf64>, %counts: memref<?xindex>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %c2 = arith.constant 2 : index
    %n0 = memref.dim %t, %c0 : memref<?x?x?xf64>
    %n1 = memref.dim %t, %c1 : memref<?x?x?xf64>
    %n2 = memref.dim %t, %c2 : memref<?x?x?xf64>
    %two = arith.constant 2.0 : f64
    scf.parallel (%i) = (%c0) to (%n0) step (%c1) {
      // no loops of its own: every lane of the team
      scf.parallel (%q) = (%c0) to (%n2) step (%c1) {
        memref.store %two, %t[%i, %c0, %q] : memref<?x?x?xf64>
        scf.reduce
      }
      // has a loop of its own: threads of the team, lanes below
      scf.parallel (%j) = (%c0) to (%n1) step (%c1) {
        scf.parallel (%k) = (%c0) to (%n2) step (%c1) {
          %v = memref.load %t[%i, %j, %k] : memref<?x?x?xf64>
          %w = arith.mulf %v, %two : f64
          memref.store %w, %t[%i, %j, %k] : memref<?x?x?xf64>
          scf.reduce
        }
        %old = memref.atomic_rmw addi %c1, %counts[%i] : (index, memref<?xindex>) -> index
        scf.reduce
      }
      memref.store %two, %row_scale[%i] : memref<?xf64>
      scf.reduce
    }
    return
  }
}
"""


def test_team_level_rules_vector_loop_thread_loop_singles_and_barriers():
    m = decided(THREE_LEVELS_NO_RESULTS)[0]
    assert m.depth == 3 and m.space == "device"
    tv = "range_parallel space=2 level=%d ivs=1 results=0"
    assert m.summary() == (
        "team_parallel results=0", (
            # The reference asks "inside a vector loop?" only for operations inside a thread loop
            # (KokkosLoopMapping.cpp:686-706): a store in a TeamVector loop directly under the team loop is
            # wrapped per team, and the per-team single without results gets its barrier.
            (tv % lm.TEAM_VECTOR, (("single level=%d" % lm.PER_TEAM, ("store",)), "team_barrier")),
            "team_barrier",                               # a team-wide loop without results does not synchronise
            (tv % lm.TEAM_THREAD, (
                (tv % lm.THREAD_VECTOR, ("store",)),
                ("single level=%d" % lm.PER_THREAD, ("atomic_rmw",)),
            )),
            "team_barrier",
            ("single level=%d" % lm.PER_TEAM, ("store",)),
            "team_barrier",
        ))
    assert m.team_size_hint == "%n1" and m.vector_length_hint == "%n2"


def test_a_call_or_an_allocation_keeps_the_nest_on_the_host_and_serialises_inner_loops():
    text = THREE_LEVELS_NO_RESULTS.replace("%w = arith.mulf %v, %two : f64",
                                           "%w = func.call @g(%v) : (f64) -> f64")
    m = decided(text)[0]
    assert m.space == "host"
    head, body = m.summary()
    assert head == "range_parallel space=0 level=0 ivs=1 results=0"
    assert body == (("for", ("store",)), ("for", (("for", ("store",)), "atomic_rmw")), "store")
    assert m.vector_length_hint is None and m.team_size_hint is None


def test_middle_loops_of_a_deep_nest_become_sequential():
    m = decided(nests.DEEP4)[0]
    kinds = []

    def walk(s):
        if isinstance(s, tuple):
            kinds.append(s[0].split(" ")[0] + (" " + s[0].split("level=")[1].split(" ")[0] if "level=" in s[0] and s[0].startswith("range") else ""))
            for c in s[1]:
                walk(c)
    walk(m.summary())
    loops = [k for k in kinds if k.startswith(("team", "range", "for"))]
    assert loops == ["team_parallel", "range_parallel 2", "for", "range_parallel 3"]


def test_two_nests_in_one_function_are_mapped_one_by_one():
    text = nests.COUNT.replace("return %total : index", """%again = scf.parallel (%i2) = (%zero) to (%n) step (%one) init (%zero) -> index {
      scf.reduce(%one : index) {
      ^bb0(%lhs: index, %rhs: index):
        %s = arith.addi %lhs, %rhs : index
        scf.reduce.return %s : index
      }
    }
    return %total : index""")
    mapped = decided(text)
    assert len(mapped) == 2 and all(n.depth == 1 and n.space == "device" for n in mapped)


def test_row_length_bound_that_is_not_the_csr_pattern_gives_no_estimate():
    text = nests.SPMV_INDEX.replace("%next = arith.addi %row, %one : index", "%next = arith.addi %row, %row : index")
    assert decided(text)[0].vector_length_hint is None
    # a bound defined outside the nest is its own estimate
    text = nests.SPMV_INDEX.replace("to (%len) step", "to (%rows) step")
    assert decided(text)[0].vector_length_hint == "%rows"
