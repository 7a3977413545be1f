"""Writes tests/golden/loop_mapping_expected.json: what the reference's gold files
tests/Dialect/Kokkos/loop_mapping_{0,1,2,3}.mlir.gold say the four nests map to, as structure only
(which loops at which Kokkos level, where the singles and team barriers sit, and the vector-length /
team-size hints as expressions with values numbered in order of appearance).  The gold files are read as
text; nothing of the reference is imported or run.

    python tests/golden/make_loop_mapping_expected.py /root/reference
"""
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from lapis_amd import loop_mapping as lm  # noqa: E402


def number_values(expr):
    """%names replaced by v0, v1, ... in order of first appearance."""
    if expr is None:
        return None
    seen = {}
    return re.sub(r"%[\w.$-]+", lambda m: seen.setdefault(m.group(0), "v%d" % len(seen)), expr)


def to_lists(summary):
    if isinstance(summary, tuple):
        return [summary[0], [to_lists(c) for c in summary[1]]]
    return summary


def main(reference_root):
    out = {}
    for k in range(4):
        name = "loop_mapping_%d" % k
        path = os.path.join(reference_root, "tests", "Dialect", "Kokkos", name + ".mlir.gold")
        text = open(path).read()
        summaries = lm.mapped_summary(text)
        hints = lm.mapped_hints(text)
        (fn, nests), = summaries.items()
        out[name] = {
            "source": "tests/Dialect/Kokkos/%s.mlir.gold" % name,
            "nests": [to_lists(n) for n in nests],
            "hints": [[number_values(v), number_values(t)] for v, t in hints[fn]],
        }
    with open(os.path.join(HERE, "loop_mapping_expected.json"), "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
