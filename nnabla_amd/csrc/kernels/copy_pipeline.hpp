// Compile-time model of the global -> LDS copy pipelines of the MFMA kernels (host and device code, plain C++14).
//
// Both product kernels keep a ring of `stages` LDS buffers; k step s lives in buffer s % stages.  Every wavefront of
// a block issues its share of the copies of a step (asynchronous: they land some time later, in issue order, and the
// only way to know is the wavefront's own count of copies still in flight, s_waitcnt vmcnt(n)), reads the buffers
// of the step being multiplied, and meets the other wavefronts at fence-free barriers.  Two things can go wrong, and
// neither shows reliably in a test, because the copies usually have a head start:
//   * a wavefront reads a buffer before every wavefront's copies of that step have landed: each wavefront must have
//     waited its own copies of the step out, and a barrier must lie between that wait and the read;
//   * a copy is issued into a buffer that some wavefront may still read for the step it held before: a barrier must
//     lie between the last read of the old step and the issue.
// The model replays the order of issues, waits, barriers and reads of one wavefront -- every wavefront runs the same
// program; between two barriers they may be anywhere relative to each other -- and checks both conditions for every
// step.  The kernels take their wait allowances from the schedule they assert safe, so a change of the loop order
// or of the number of stages that breaks the hand-over fails to compile.
#pragma once

namespace nbla_hip {
namespace pipeline {

constexpr int kMaxEvents = 512;
constexpr int kMaxSteps = 64;

enum Op { kIssue, kWait, kBarrier, kRead };

struct Event {
  int op;
  int arg; // kIssue / kRead: the k step; kWait: the number of most recently issued steps that may stay in flight
};

struct Program {
  Event ev[kMaxEvents];
  int n;
  int steps; // k steps that are multiplied (issues run past them: the kernels copy the last step again)
};

constexpr void push(Program &p, int op, int arg) {
  if (p.n < kMaxEvents) {
    p.ev[p.n].op = op;
    p.ev[p.n].arg = arg;
  }
  ++p.n;
}

// Bit-weight kernel: two output tiles per k step, one wait and one barrier per step in the middle of it.
//   prologue: issue steps 0 .. depth-1; wait(prologue_wait); barrier; read step 0
//   step ks:  read ks; wait(loop_wait); barrier; issue ks+depth; read ks+1
constexpr Program two_tile_program(int depth, int prologue_wait, int loop_wait, int steps) {
  Program p{};
  p.n = 0;
  p.steps = steps;
  for (int d = 0; d < depth; ++d)
    push(p, kIssue, d);
  push(p, kWait, prologue_wait);
  push(p, kBarrier, 0);
  push(p, kRead, 0);
  for (int ks = 0; ks < steps; ++ks) {
    push(p, kRead, ks);
    push(p, kWait, loop_wait);
    push(p, kBarrier, 0);
    push(p, kIssue, ks + depth);
    if (ks + 1 < steps)
      push(p, kRead, ks + 1);
  }
  return p;
}

// Digit x digit kernel: one wait and one barrier at the top of every step.
//   prologue: issue steps 0 .. depth-1
//   step kt:  wait(loop_wait); barrier; issue kt+depth; read kt
constexpr Program one_tile_program(int depth, int loop_wait, int steps) {
  Program p{};
  p.n = 0;
  p.steps = steps;
  for (int d = 0; d < depth; ++d)
    push(p, kIssue, d);
  for (int kt = 0; kt < steps; ++kt) {
    push(p, kWait, loop_wait);
    push(p, kBarrier, 0);
    push(p, kIssue, kt + depth);
    push(p, kRead, kt);
  }
  return p;
}

// Bit-weight kernel, one-digit rows: a step's operands are few enough to be read one whole step ahead.
//   prologue: issue steps 0 .. depth-1; wait(prologue_wait); barrier; read step 0
//   step ks:  wait(loop_wait); barrier; read ks+1; (multiply step ks from registers); issue ks+depth
constexpr Program read_ahead_program(int depth, int prologue_wait, int loop_wait, int steps) {
  Program p{};
  p.n = 0;
  p.steps = steps;
  for (int d = 0; d < depth; ++d)
    push(p, kIssue, d);
  push(p, kWait, prologue_wait);
  push(p, kBarrier, 0);
  push(p, kRead, 0);
  for (int ks = 0; ks < steps; ++ks) {
    push(p, kWait, loop_wait);
    push(p, kBarrier, 0);
    if (ks + 1 < steps)
      push(p, kRead, ks + 1);
    push(p, kIssue, ks + depth);
  }
  return p;
}

// 0: safe; 1: a buffer is read before the step has landed for every wavefront; 2: a copy may overwrite a buffer that
// is still being read; 3: the program does not fit the model's tables; 4: a step is issued out of order
constexpr int check(const Program &p, int stages) {
  if (p.n > kMaxEvents || p.steps + stages + 1 > kMaxSteps || stages < 1)
    return 3;
  // epoch = number of barriers passed; events of different wavefronts in the same epoch are unordered
  int landed_epoch[kMaxSteps] = {}; // epoch in which the wavefront knows its copies of the step have landed
  int issue_epoch[kMaxSteps] = {};
  int last_read_epoch[kMaxSteps] = {};
  for (int s = 0; s < kMaxSteps; ++s) {
    landed_epoch[s] = -1;
    issue_epoch[s] = -1;
    last_read_epoch[s] = -1;
  }
  int epoch = 0, issued = 0; // steps 0 .. issued-1 have been issued, in order
  for (int i = 0; i < p.n; ++i) {
    const Event e = p.ev[i];
    if (e.op == kBarrier) {
      ++epoch;
    } else if (e.op == kIssue) {
      if (e.arg != issued || e.arg >= kMaxSteps)
        return e.arg >= kMaxSteps ? 3 : 4;
      issue_epoch[e.arg] = epoch;
      ++issued;
      const int old = e.arg - stages; // the step this buffer held before
      if (old >= 0) {
        // every wavefront's reads of the old step must lie before a barrier that precedes this issue; reads that
        // come later in the program are caught when they happen (the step is then no longer in its buffer)
        if (last_read_epoch[old] >= epoch)
          return 2;
      }
    } else if (e.op == kWait) {
      for (int s = 0; s < issued - e.arg; ++s)
        if (landed_epoch[s] < 0)
          landed_epoch[s] = epoch;
    } else { // kRead
      const int s = e.arg;
      if (s < 0 || s >= kMaxSteps || issue_epoch[s] < 0)
        return 1;
      // the other wavefronts' waits for this step lie in epoch landed_epoch[s] of their (identical) program: only a
      // barrier after it orders them before this read
      if (landed_epoch[s] < 0 || landed_epoch[s] >= epoch)
        return 1;
      // the buffer must still hold step s: no newer step may have been issued into it, even in this epoch
      if (s + stages < issued)
        return 2;
      last_read_epoch[s] = epoch;
    }
  }
  return 0;
}

// enough steps for the ring to wrap several times
constexpr int model_steps(int stages) { return 3 * stages + 2; }

constexpr bool two_tile_safe(int stages, int depth, int prologue_wait, int loop_wait) {
  return depth >= 1 && check(two_tile_program(depth, prologue_wait, loop_wait, model_steps(stages)), stages) == 0;
}
constexpr bool one_tile_safe(int stages, int depth, int loop_wait) {
  return depth >= 1 && check(one_tile_program(depth, loop_wait, model_steps(stages)), stages) == 0;
}

// The largest number of steps a wait may leave in flight (waiting for less than necessary costs time, more is the
// race): the schedules the kernels use.  -1: no allowance makes the loop safe.
constexpr int two_tile_loop_wait(int stages, int depth) {
  int best = -1;
  for (int w = 0; w <= depth; ++w)
    if (two_tile_safe(stages, depth, depth - 1, w))
      best = w;
  return best;
}
constexpr int two_tile_prologue_wait(int stages, int depth) {
  int best = -1;
  for (int w = 0; w <= depth; ++w)
    if (two_tile_safe(stages, depth, w, 0))
      best = w;
  return best;
}
constexpr bool read_ahead_safe(int stages, int depth, int prologue_wait, int loop_wait) {
  return depth >= 1 &&
         check(read_ahead_program(depth, prologue_wait, loop_wait, model_steps(stages)), stages) == 0;
}
constexpr int read_ahead_loop_wait(int stages, int depth) {
  int best = -1;
  for (int w = 0; w <= depth; ++w)
    if (read_ahead_safe(stages, depth, depth - 1, w))
      best = w;
  return best;
}
constexpr int one_tile_loop_wait(int stages, int depth) {
  int best = -1;
  for (int w = 0; w <= depth; ++w)
    if (one_tile_safe(stages, depth, w))
      best = w;
  return best;
}

// vmcnt is a 6-bit counter: a wait for "at most n copies in flight" can only be written for n <= 63.
constexpr bool counter_fits(int steps_in_flight, int copies_per_step) { return steps_in_flight * copies_per_step <= 63; }

} // namespace pipeline
} // namespace nbla_hip
