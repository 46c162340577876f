"""Host logic of the level executor on a machine without a GPU.

tests/host_logic/null_abi.py turns include/ginn_hip.h into a recording stand-in
for the device library; tests/host_logic/host_logic.cpp runs a small graph
through LevelExecutor (ginn_amd/ginn/level_exec.h) against it and prints which
table launches every phase made.  Checked here: one launch per level whatever
the nodes compute, one zero fill for all gradients, a reduction for five users
of one gradient, successive launches for two users of one gradient on one
level, plans reused without uploads on the second pass, the frozen replay
making the same launches (and one reduction per pass into a leaf's gradient instead of one per
level), and plain execution making none of them.
"""
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "tests" / "host_logic"))


@pytest.fixture(scope="module")
def phases(tmp_path_factory):
    import null_abi
    tmp = tmp_path_factory.mktemp("host_logic")
    stub = tmp / "null_abi.c"
    assert null_abi.generate(ROOT / "include" / "ginn_hip.h", stub) > 40
    subprocess.run(["gcc", "-O1", f"-I{ROOT / 'include'}", "-c", str(stub), "-o", str(tmp / "null_abi.o")], check=True)
    subprocess.run(["g++", "-std=c++17", "-O1", f"-I{ROOT / 'ginn_amd'}", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "host_logic" / "host_logic.cpp"), str(tmp / "null_abi.o"),
                    "-o", str(tmp / "host_logic")], check=True)
    out = subprocess.run([str(tmp / "host_logic")], check=True, capture_output=True, text=True).stdout
    result = {}
    for line in out.splitlines():
        m = re.match(r"(.+?): \[(.*)\] uploads=(\d+) direct=(\d+)$", line)
        if m:
            calls = [tuple(c.split()) for c in m.group(2).split(", ") if c]
            result[m.group(1)] = ([(n, int(c)) for n, c in calls], int(m.group(3)), int(m.group(4)))
        else:
            k, _, v = line.partition(": ")
            result[k] = v
    return result


def test_one_launch_per_level(phases):
    calls, uploads, direct = phases["forward 1"]
    # sigmoid, tanh and relu of one tensor and relu of a shorter one: one launch
    assert calls[0] == ("multi_mixed", 4)
    assert calls[1] == ("multi_mixed", 2)  # the two products
    assert all(name == "multi_mixed" for name, _ in calls)
    assert direct == 2  # the two Sum nodes run themselves
    assert uploads >= 1


def test_reset_is_one_zero_fill(phases):
    calls, _, direct = phases["reset 1"]
    # one fill for every gradient that is zeroed; those with a single overwriting
    # user are only flagged (BaseNode::GradUse) and are in no launch
    assert len(calls) == 1 and calls[0][0] == "multi_zero" and calls[0][1] >= 5
    assert direct == 0


def test_backward_reduction_and_overlap_rounds(phases):
    calls, _, _ = phases["backward 1"]
    assert calls.count(("multi_reduce", 5)) == 1  # Add(s, s, s, s, s): five users of s.grad()
    # the two products both add into the gradient of Tanh(x): three operations
    # with distinct destinations first, the second user of that gradient after
    assert ("multi_mixed", 3) in calls
    i = max(k for k, c in enumerate(calls) if c == ("multi_mixed", 3))
    assert calls[i + 1] == ("multi_mixed", 1)


def test_plans_are_reused(phases):
    first = phases["forward 1"][0] + phases["reset 1"][0] + phases["backward 1"][0]
    calls, uploads, _ = phases["pass 2"]
    assert calls == first
    assert uploads == 0
    assert phases["rebuilt in pass 2"] == "0"


def test_frozen_replay_makes_the_same_launches(phases):
    calls, uploads, direct = phases["frozen pass"]
    assert calls == phases["pass 2"][0]
    assert uploads == 0 and direct == phases["pass 2"][2]
    assert phases["rebuilt frozen"] == "0"


def test_fused_levels_become_chain_launches(phases):
    """fuse(): consecutive levels without a self-running node in between are one
    chain launch; operations that touch each other's memory share a chain."""
    calls, uploads, direct = phases["fused forward"]
    # Sum(Relu(z)) runs itself on level 2, so level 1 stays a launch of its own; levels 2-5 (the products,
    # the two adds, the square) touch each other's memory: one chain; the last Add follows the Sum nodes
    assert calls == [("multi_mixed", 4), ("multi_chain", 1), ("multi_mixed", 1)]
    assert uploads == 0 and direct == phases["forward 1"][2]
    assert phases["fused reset"][0] == phases["reset 1"][0]
    bcalls, buploads, bdirect = phases["fused backward"]
    assert buploads == 0 and bdirect == phases["backward 1"][2]
    # the reduction stays a launch of its own and splits the levels around it; after it the gradients of
    # x (through Sigmoid / Tanh / Relu) and of z are two independent chains
    assert bcalls == [("multi_mixed", 2), ("multi_chain", 1), ("multi_reduce", 5), ("multi_mixed", 3),
                      ("multi_chain", 2)]
    assert int(phases["chain launches built"]) == 3


def test_frozen_pass_sums_a_leaf_gradient_once(phases):
    """Two levels each add five gradients into one bias: a reduction per level while every node is
    asked, ONE reduction over all ten sources at the end of a frozen backward pass."""
    calls, _, _ = phases["two-level backward"]
    assert calls.count(("multi_reduce", 5)) == 2
    frozen, uploads, _ = phases["two-level backward frozen"]
    assert [c for c in frozen if c[0] == "multi_reduce"] == [("multi_reduce", 10)]
    assert frozen[-1] == ("multi_reduce", 10) and uploads == 0
    assert [c for c in frozen if c[0] != "multi_reduce"] == [c for c in calls if c[0] != "multi_reduce"]


def test_plain_execution_launches_per_node(phases):
    calls, _, direct = phases["plain pass"]
    assert calls == []
    assert direct > len(phases["pass 2"][0]) + phases["pass 2"][2]


def test_autobatch_merges_products_by_left_operand_and_height(phases):
    """ginn/autobatch.h:42-202: every Affine becomes products + a broadcast bias
    + an Add; products with one left operand on one height are merged into ONE
    product over the row-wise concatenation of their right operands."""
    assert phases["autobatch"] == "affines 8 -> 0, prods 0 -> 2"
    assert phases["autobatch glue"] == "RowwiseCat 2 RowwiseUncat 8"
