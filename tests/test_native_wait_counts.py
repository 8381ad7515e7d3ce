"""The wait counts of the kernels that issue their loads by hand (anemone_amd/csrc/native_waits.h, used by
native_device.cuh) on the CPU: the header is compiled into a host program (g++) that prints loads_behind(step, total)
for the parameters of every kernel instance, and this file holds each number against a model of the order in which the
kernel's K loop issues its loads (written from the loop in native_device.cuh: steps() and one_step(), not from the
formula): at the top of a step, `s_waitcnt vmcnt(N)` must leave that step's columns and weights landed (N no larger than
the loads issued behind the later of them) and should wait for nothing more (N no smaller). No GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# (SLOTS, DEPTH, WEIGHTS_FIRST, VECTOR_LOADS, WEIGHT_LOADS) of the instances in kernel_native_linear.hip: VECTOR_LOADS is
# 2 loads a column block a wavefront brings (one or two) and one of scale words; WEIGHT_LOADS the tiles' halves and the
# scale loads of a wavefront's strip
INSTANCES = {
    "E2M1 gate/up (4 tiles, 2 scale words; 64 columns)": (3, 2, False, 3, 6),
    "E2M1 down (4 tiles, 1 scale word)": (3, 2, False, 3, 5),
    "E4M3 gate/up and down (2 tiles of two halves, 2 scale bytes; 128 columns)": (3, 3, True, 5, 6),
    "E4M3_BLOCK128 down (2 tiles of two halves, 1 scale)": (3, 3, True, 5, 5),
    "four sets of weight registers (measured, not kept)": (4, 3, True, 5, 6),
    "six sets": (6, 3, True, 5, 6),
    "weights behind the columns at three stages": (4, 3, False, 5, 6),
}
MOST_TOTAL = 24

HARNESS = r"""
#include <cstdio>
#include "native_waits.h"
template <uint32_t S, uint32_t D, bool W, uint32_t V, uint32_t L>
static void table(const char *name)
{
    for (uint32_t total = 1; total <= %d; total++) {
        for (uint32_t step = 0; step < total; step++) {
            std::printf("%%s %%u %%u %%u\n", name, total, step, native_waits<S, D, W, V, L>::loads_behind(step, total));
        }
    }
}
int main()
{
%s
    return 0;
}
"""


@pytest.fixture(scope="module")
def tables(tmp_path_factory):
    folder = tmp_path_factory.mktemp("waits")
    calls = "\n".join('    table<%du, %du, %s, %du, %du>("%d");' % (s, d, "true" if w else "false", v, l, index)
                      for index, (s, d, w, v, l) in enumerate(INSTANCES.values()))
    source = folder / "waits.cpp"
    source.write_text(HARNESS % (MOST_TOTAL, calls))
    program = folder / "waits"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "anemone_amd", "csrc"), str(source), "-o", str(program)],
                   check=True)
    printed = subprocess.run([str(program)], check=True, stdout=subprocess.PIPE, text=True).stdout
    found = {}
    for line in printed.splitlines():
        index, total, step, count = (int(word) for word in line.split())
        found[(index, total, step)] = count
    return found


def issue_order(slots, depth, weights_first, total):
    """The loads of a chain of `total` steps in the order the loop issues them, as (kind, step) with kind "V" (a step's
    columns) or "W" (its weights), and for every step the number of loads issued before its wait."""
    order, before_wait = [], []
    for k in range(depth - 1):  # steps(): the columns of the first stages
        if k < total:
            order.append(("V", k))
    for k in range(slots - 1):  # first_weights()
        if k < total:
            order.append(("W", k))
    for step in range(total):   # one_step(), step by step
        before_wait.append(len(order))
        ask = [("W", step + slots - 1)] if step + slots - 1 < total else []
        columns = [("V", step + depth - 1)] if step + depth - 1 < total else []
        order += ask + columns if weights_first else columns + ask
    return order, before_wait


@pytest.mark.parametrize("index,name", list(enumerate(INSTANCES)))
def test_a_steps_wait_leaves_its_loads_landed_and_no_more(tables, index, name):
    slots, depth, weights_first, vector_loads, weight_loads = INSTANCES[name]
    size = {"V": vector_loads, "W": weight_loads}
    for total in range(1, MOST_TOTAL + 1):
        order, before_wait = issue_order(slots, depth, weights_first, total)
        assert sorted(order) == sorted([("V", k) for k in range(total)] + [("W", k) for k in range(total)]), "every step's loads are asked for once"
        for step in range(total):
            issued = order[:before_wait[step]]
            assert ("V", step) in issued and ("W", step) in issued, "a step's loads are asked for before its wait"
            later = max(issued.index(("V", step)), issued.index(("W", step)))
            behind = sum(size[kind] for kind, _ in issued[later + 1:])  # loads complete in order: these may be outstanding
            assert tables[(index, total, step)] == behind, (name, total, step, tables[(index, total, step)], behind)
            assert behind < 64  # vmcnt's six bits


def test_the_counts_are_ones_the_kernel_has_an_instruction_for(tables):
    """wait_behind() of native_device.cuh has one s_waitcnt for W x WEIGHT_LOADS + V x VECTOR_LOADS with W below SLOTS and V
    below DEPTH - 1 (at least one): every count the formula gives is one of them."""
    for index, (slots, depth, weights_first, vector_loads, weight_loads) in enumerate(INSTANCES.values()):
        reachable = {w * weight_loads + v * vector_loads for w in range(slots) for v in range(max(1, depth - 1))}
        counts = {count for (i, _, _), count in tables.items() if i == index}
        assert counts <= reachable, (index, sorted(counts - reachable))
