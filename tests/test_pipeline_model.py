"""The compile-time model of the MFMA kernels' global -> LDS copy pipelines (nnabla_amd/csrc/kernels/copy_pipeline.hpp),
run on the host: the wait allowances the kernels take from it are the ones derived by hand, the allowance the
bit-weight kernel once used (one k step too many in flight at the mid-step wait, a race that the copies' head start
hid from every GPU test for a long time) is rejected, and so is every other way of breaking the hand-over that the
model is meant to catch (a missing barrier, a copy into the buffer being read, a wait after the read)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNELS = os.path.join(ROOT, "nnabla_amd", "csrc", "kernels")

PROGRAM = r"""
#include "copy_pipeline.hpp"
#include <cstdio>
using namespace nbla_hip::pipeline;

// the bit-weight loop with one element of its order changed
static Program two_tile_variant(int depth, int prologue_wait, int loop_wait, int steps, int variant) {
  Program p{};
  p.n = 0;
  p.steps = steps;
  for (int d = 0; d < depth; ++d)
    push(p, kIssue, d);
  push(p, kWait, prologue_wait);
  if (variant != 1) // 1: no barrier between the prologue's wait and the first read
    push(p, kBarrier, 0);
  push(p, kRead, 0);
  for (int ks = 0; ks < steps; ++ks) {
    push(p, kRead, ks);
    if (variant == 2) { // 2: the copy is issued before the barrier: other wavefronts may still read its buffer
      push(p, kWait, loop_wait);
      push(p, kIssue, ks + depth);
      push(p, kBarrier, 0);
    } else if (variant == 3) { // 3: barrier first, wait after it: own copies only
      push(p, kBarrier, 0);
      push(p, kWait, loop_wait);
      push(p, kIssue, ks + depth);
    } else {
      push(p, kWait, loop_wait);
      push(p, kBarrier, 0);
      push(p, kIssue, ks + depth);
    }
    if (ks + 1 < steps)
      push(p, kRead, ks + 1);
  }
  return p;
}

int main() {
  // compile-time use, as in the kernels
  static_assert(two_tile_safe(6, 5, two_tile_prologue_wait(6, 5), two_tile_loop_wait(6, 5)), "");
  static_assert(!two_tile_safe(6, 5, 4, 4), "");
  static_assert(one_tile_safe(3, 2, one_tile_loop_wait(3, 2)), "");
  for (int stages = 2; stages <= 12; ++stages) {
    const int depth = stages - 1, steps = model_steps(stages);
    printf("two_tile %d %d %d", stages, two_tile_prologue_wait(stages, depth), two_tile_loop_wait(stages, depth));
    // the allowances used before the fix: prologue depth - 1, loop depth - 1
    printf(" %d", check(two_tile_program(depth, depth - 1, depth - 1, steps), stages));
    // prologue allowance one too large
    printf(" %d", check(two_tile_program(depth, depth, depth - 2 < 0 ? 0 : depth - 2, steps), stages));
    for (int variant = 0; variant <= 3; ++variant) {
      // variant 2 with as many steps in flight as the ring has buffers: the copy of step ks + stages goes into the
      // buffer of step ks, which the shipped order allows only because the barrier comes first
      const int dp = variant == 2 ? stages : depth;
      printf(" %d", check(two_tile_variant(dp, dp - 1, dp - 2 < 0 ? 0 : dp - 2, steps, variant), stages));
    }
    printf(" %d", check(two_tile_program(stages, stages - 1, stages - 2, steps), stages));
    // one step of prefetch more than the ring has buffers for
    printf(" %d", check(two_tile_program(stages + 1, stages, 0, steps), stages));
    printf("\n");
    printf("read_ahead %d %d %d %d %d\n", stages, read_ahead_loop_wait(stages, depth),
           check(read_ahead_program(depth, depth - 1, depth - 2 < 0 ? 0 : depth - 2, steps), stages),
           check(read_ahead_program(depth, depth - 1, depth - 1, steps), stages),
           check(read_ahead_program(stages + 1, stages, 0, steps), stages));
    printf("one_tile %d %d %d %d %d\n", stages, one_tile_loop_wait(stages, depth),
           check(one_tile_program(depth, depth - 1, steps), stages), check(one_tile_program(depth, depth, steps), stages),
           check(one_tile_program(stages, 0, steps), stages));
  }
  printf("fits %d %d %d\n", (int)counter_fits(9, 7), (int)counter_fits(9, 8), (int)counter_fits(4, 6));
  return 0;
}
"""


@pytest.fixture(scope="module")
def table(tmp_path_factory):
    d = tmp_path_factory.mktemp("pipeline")
    src = d / "model.cpp"
    src.write_text(PROGRAM)
    exe = d / "model"
    subprocess.run(["g++", "-std=c++14", "-O1", "-I", KERNELS, "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE).stdout.decode()
    rows = {}
    for line in out.splitlines():
        f = line.split()
        rows.setdefault(f[0], []).append([int(v) for v in f[1:]])
    return rows


def test_bit_weight_loop_allowances(table):
    for stages, prologue, loop, old, big_prologue, v0, v1, v2, v3, full_ring, too_deep in table["two_tile"]:
        depth = stages - 1
        if stages == 2:  # one step ahead only: the step after the one being multiplied can never have landed
            assert prologue == -1 and loop == -1
            continue
        # by hand: before the mid-step wait of step ks the copies reach step ks + depth - 1, step ks + 1 must have
        # landed, so depth - 2 steps may stay in flight; the prologue has issued depth steps and needs step 0
        assert prologue == depth - 1 and loop == depth - 2
        assert old == 1, "the allowance of depth - 1 at the mid-step wait must be reported as a read before landing"
        assert big_prologue == 1
        assert v0 == 0, "the shipped order with the shipped allowances"
        assert v1 == 1, "no barrier after the prologue's wait"
        assert v2 == 2, "copy issued before the barrier into the buffer of the step being read"
        assert full_ring == 0, "the same depth with the barrier before the copy"
        assert v3 == 1, "wait after the barrier covers the wavefront's own copies only"
        assert too_deep == 2, "more steps in flight than buffers"


def test_digit_loop_allowances(table):
    for stages, loop, shipped, one_more, full_ring in table["one_tile"]:
        depth = stages - 1
        assert loop == depth - 1  # the wait at the top of tile kt: the copies reach kt + depth - 1, tile kt is needed
        assert shipped == 0 and one_more == 1
        assert full_ring == 2  # a ring with no spare buffer: the copy lands in the buffer being multiplied


def test_one_digit_loop_allowances(table):
    """The bit-weight kernel's loop for one-digit rows reads step ks+1 at the top of step ks: before that read the
    copies reach step ks + depth - 1, so depth - 2 steps may stay in flight; one step more in flight than the ring
    has buffers overwrites the step being read."""
    for stages, loop, shipped, one_more, too_deep in table["read_ahead"]:
        depth = stages - 1
        if stages == 2:
            assert loop == -1
            continue
        assert loop == depth - 2 and shipped == 0 and one_more == 1 and too_deep == 2


def test_counter_width(table):
    assert table["fits"] == [[1, 0, 1]]


def test_kernels_take_their_waits_from_the_model():
    bits = open(os.path.join(KERNELS, "gemm_bits.hip")).read()
    digits = open(os.path.join(KERNELS, "gemm_digits.hip")).read()
    waits = re.findall(r"wait_copies\(std::integral_constant<int, ([^>]+)>", bits)
    assert waits and set(waits) <= {"kPrologueWait", "kLoopWait", "kAheadWait"}, waits
    assert "pipeline::read_ahead_safe(kStages, kDepth, kPrologueWait, kAheadWait)" in bits
    assert "pipeline::two_tile_safe(kStages, kDepth, kPrologueWait, kLoopWait)" in bits
    loop_waits = [w for w in re.findall(r"^ +NBLA_WAIT_VMCNT\(([^;\n]+)\);", digits, re.M) if w.strip() != "0"]
    assert loop_waits == ["kLoopWait * kCopies"], loop_waits
    assert "pipeline::one_tile_safe(kStages, kStages - 1, kLoopWait)" in digits
    assert "copies_per_call(kOneA, kNarrow, kGroups) == kCopies" in digits
