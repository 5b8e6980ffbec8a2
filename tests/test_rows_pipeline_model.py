"""The hand-over of LDS buffers in the one-walk BinaryAffine forward (nnabla_amd/csrc/kernels/binary_rows_mma.hip),
replayed on the host.  The kernel's two kinds of wavefronts issue global -> LDS copies (weights into a ring, digit
fragments into two stages) and ordinary stores (Wb) that all count on one in-order counter, and wait with
`s_waitcnt vmcnt(n)` for "all but my n youngest operations"; a wait that is one too generous is a race that the copies'
head start hides from GPU tests.  The model takes the kernel's own constants and wait expressions from the source text,
replays both programs operation by operation and checks every read of a buffer against the waits and barriers that
must precede it, and every overwrite against the reads that must be over -- and that each wait is the most generous
safe one (one more operation in flight breaks the hand-over)."""
import os
import re

import pytest

SRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nnabla_amd", "csrc", "kernels",
                   "binary_rows_mma.hip")


def kernel_text():
    return open(SRC).read()


def constants(text):
    c = {"kFragRows": 32, "kDigits": 3}   # gemm_layout.hpp
    for name in ("kChunkRows", "kRingDepth", "kWLoads", "kConvStores", "kAStages"):
        c[name] = int(re.search(r"constexpr int %s = (\d+);" % name, text).group(1))
    assert re.search(r"constexpr int kRowFrags = kChunkRows / kFragRows;", text)
    assert re.search(r"constexpr int kALoads = kRowFrags \* kDigits / 4;", text)
    c["kRowFrags"] = c["kChunkRows"] // c["kFragRows"]
    c["kALoads"] = c["kRowFrags"] * c["kDigits"] // 4
    c["D"] = c["kRingDepth"]
    return c


def wait_expressions(text):
    """The arguments of the kernel's vmcnt waits, in source order: prologue (weights), prologue (activations), loop
    (weights, k step still from the prologue), loop (weights, later), loop (activations), after the loop."""
    body = text[text.index("// ---- prologue: k steps 0 and 1 of W landed"):text.index("// ---- epilogue.  Column sums")]
    return re.findall(r"NBLA_ROWS_WAIT_VMCNT\(([^;]*)\);", body)


class Wave:
    """One wavefront's in-order memory operations: `issue` appends tagged operations, `wait(n)` marks all but the n
    youngest complete."""

    def __init__(self):
        self.ops = []
        self.done = 0

    def issue(self, tag, count):
        self.ops += [tag] * count

    def wait(self, n):
        self.done = max(self.done, len(self.ops) - n)

    def complete(self, tag):
        idx = [i for i, t in enumerate(self.ops) if t == tag]
        return bool(idx) and idx[-1] < self.done


def replay(c, waits, T, slack=None):
    """Replays T k steps.  `slack`: index of a wait to loosen by one operation.  Returns the list of violations."""
    D = c["D"]
    env = dict(c)
    w = [eval(e, {}, env) for e in waits]
    if slack is not None:
        w[slack] += 1
    slots, stages = D + 1, c["kAStages"]
    W, A = Wave(), Wave()                  # one representative wavefront of each kind (all of a kind run alike)
    epoch = 0
    landed_w, landed_a = {}, {}            # k step -> epoch in which its copies were known to have landed
    last_ring_read, last_stage_read, b_written, last_b_read = {}, {}, {}, {}
    ring_holds, stage_holds = {}, {}       # slot -> k step
    bad = []

    def note_landed():
        for s in list(ring_holds.values()):
            if s not in landed_w and W.complete(("w", s)):
                landed_w[s] = epoch
        for s in list(stage_holds.values()):
            if s not in landed_a and A.complete(("a", s)):
                landed_a[s] = epoch

    def issue_w(s):
        old = ring_holds.get(s % slots)
        if old is not None and last_ring_read.get(old, -1) >= epoch:
            bad.append("ring slot of k step %d overwritten by %d while it may still be converted" % (old, s))
        if old is not None and old not in last_ring_read and old < T:
            bad.append("ring slot of k step %d overwritten before it was converted" % old)
        ring_holds[s % slots] = s
        W.issue(("w", s), c["kWLoads"])

    def issue_a(s):
        old = stage_holds.get(s % stages)
        if old is not None and last_stage_read.get(old, -1) >= epoch:
            bad.append("digit stage of k step %d overwritten by %d while it may still be multiplied" % (old, s))
        stage_holds[s % stages] = s
        A.issue(("a", s), c["kALoads"])

    def convert(s, wave):   # every wavefront reads the ring slot of k step s, writes B tile s % 2, stores Wb
        if ring_holds.get(s % slots) != s:
            bad.append("k step %d is not in its ring slot when converted" % s)
        if landed_w.get(s, epoch) >= epoch:
            bad.append("k step %d converted before its copies were waited for and a barrier passed" % s)
        last_ring_read[s] = epoch
        if last_b_read.get(s - 2, -1) >= epoch:
            bad.append("B tile of k step %d rewritten while it may still be multiplied" % (s - 2))
        b_written[s] = epoch
        wave.issue(("st", s), c["kConvStores"])

    def multiply(s):
        if stage_holds.get(s % stages) != s:
            bad.append("digits of k step %d are not in their stage when multiplied" % s)
        if landed_a.get(s, epoch) >= epoch:
            bad.append("k step %d multiplied before its digits were waited for and a barrier passed" % s)
        if b_written.get(s, epoch) >= epoch:
            bad.append("k step %d multiplied before its B tile was written and a barrier passed" % s)
        last_stage_read[s] = epoch
        last_b_read[s] = epoch

    # prologue
    for t in range(D + 1):
        issue_w(t)
    W.wait(w[0])
    issue_a(0)
    note_landed()
    epoch += 1
    convert(0, W)
    convert(0, A)
    A.wait(w[1])
    note_landed()
    epoch += 1
    # main loop
    for i in range(T):
        if i + 1 < T:
            issue_w(i + 1 + D)
        issue_a(i + 1)
        if i + 1 < T:
            convert(i + 1, A)
        multiply(i)
        if i + 1 < T:
            convert(i + 1, W)
        W.wait(w[2] if i <= D - 2 else w[3])
        A.wait(w[4])
        note_landed()
        epoch += 1
    W.wait(w[5])
    A.wait(w[5])
    if W.done != len(W.ops) or A.done != len(A.ops):
        bad.append("copies in flight when the stages are reused after the loop")
    return bad


def test_the_kernel_waits_are_the_ones_the_model_reads():
    text = kernel_text()
    c = constants(text)
    assert c["kRingDepth"] >= 2 and c["kAStages"] == 2 and c["kWLoads"] == 4 and c["kALoads"] == 6
    waits = wait_expressions(text)
    assert len(waits) == 6 and waits[5].strip() == "0"
    # vmcnt is a six-bit counter
    assert all(0 <= eval(e, {}, dict(c)) <= 63 for e in waits)


@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 6, 7, 9, 16, 40])
def test_every_buffer_is_handed_over_behind_a_wait_and_a_barrier(T):
    text = kernel_text()
    assert replay(constants(text), wait_expressions(text), T) == []


def test_each_wait_is_as_generous_as_the_hand_over_allows():
    """One more operation left in flight at any of the waits that guard copies lets some k step be read before it has
    landed (for some number of k steps): the model would catch a miscounted wait."""
    text = kernel_text()
    c, waits = constants(text), wait_expressions(text)
    for slack in range(5):
        assert any(replay(c, waits, T, slack) for T in (1, 2, 3, 5, 8, 16, 40)), \
            "wait %d (%s) could leave one more operation in flight" % (slack, waits[slack])


def test_waits_counted_for_more_stores_than_are_issued_are_caught():
    """The stores of a conversion sit behind the copies on the same counter.  Waits computed for more stores per
    conversion than the wavefronts issue (the kernel once went from eight 32-bit to four 64-bit stores per conversion
    with the counts left behind) let copies stay in flight: the replay reports k steps read before they have landed."""
    text = kernel_text()
    c, waits = constants(text), wait_expressions(text)
    values = [str(eval(e, {}, dict(c, kConvStores=2 * c["kConvStores"]))) for e in waits]
    bad = replay(c, values, 12)
    assert any("before its copies were waited for" in b or "before its digits" in b for b in bad)
