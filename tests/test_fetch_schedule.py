"""The asynchronous fetch pipelines of the ring kernels, replayed against an adversarial memory.

The GEMM loops never synchronise on data: a direct-to-LDS (or register) load is assumed to have landed when an
`s_waitcnt vmcnt(N)` with a constant N allows only the N newest loads to be outstanding, and a ring slot is assumed free
when its last reader has been waited for.  A count that is one too high, or a fetch one step too early, passes every GPU
test on most runs, because loads usually land long before they are needed.  Here the issue / wait / read order of the
loops (gemm_m16.h stream_tile; gemm_mb.h stream_tile_mb and stream_tile_mbp) is restated step by step and run on a
memory that completes a load only when a wait forces it to (loads complete in issue order, as the counter assumes):

* every read of a step's words, activations or group scales finds the load that brought them complete;
* no load is issued into a slot, register set or scale slab that still holds data somebody is going to read;
* a wait never names more loads than can be in flight (a 6-bit counter).

Restated from the kernels: the order of loads inside a step's batch, where the load of group scales goes, the counts of
newer_step_ops / kWaitOdd / kWaitEven / the +1 for group scales, the slot rotation, the clamped redundant fetches past
the end.  The GPU tests run the compiled loops themselves.
"""
import itertools

import pytest


class Memory:
    """Loads complete in issue order, and only when a wait leaves them no choice."""

    def __init__(self):
        self.ops = []            # (id, what) in issue order
        self.done = 0            # ops[:done] have completed
        self.content = {}        # place -> (what, op index) as of the last load issued there
        self.pending_reads = {}  # place -> what a future read still expects there

    def load(self, place, what):
        slot = place[:2]                                       # (kind, slot): the unit that is handed back and forth
        assert slot not in self.pending_reads or self.pending_reads[slot] == what, \
            f"load of {what} into {place} which still holds unread {self.pending_reads[slot]}"
        self.content[place] = (what, len(self.ops))
        self.ops.append((place, what))

    def wait(self, n):
        assert 0 <= n <= 63
        self.done = max(self.done, len(self.ops) - n)

    def read(self, place, what):
        have, idx = self.content.get(place, (None, None))
        assert have == what, f"read of {what} from {place}, which holds {have}"
        assert idx < self.done, f"read of {what} from {place} before its load completed"
        self.pending_reads.pop(place[:2], None)

    def expect(self, place, what):
        """`what` has been fetched into the slot of `place` and somebody will read it from there later."""
        self.pending_reads[place[:2]] = what


def newer_step_ops(word_ops, a_ops, first, n):
    return word_ops * n + sum(a_ops for t in range(n) if (first + t) % 2 == 0)


def run_m16(steps, depth, arows, fp6, group):
    """gemm_m16.h stream_tile: one wave, `steps` k steps (even; a multiple of four with group scales)."""
    group = group and not fp6
    word_ops, a_ops = (3 if fp6 else 2), (2 if arows == 16 else 1)
    pair_slots = (depth + 2) // 2
    unroll = 4 if group else 2
    wait_odd = newer_step_ops(word_ops, a_ops, 1, depth - 2)
    wait_even = newer_step_ops(word_ops, a_ops, 0, depth - 2)
    mem = Memory()
    state = dict(issued=0, pairs_issued=0, pair_in=0)
    last, last_pair = steps - 1, steps // 2 - 1

    def issue(slot, even):
        step = state["issued"]
        if even:
            pair = state["pairs_issued"]
            for o in range(a_ops):
                mem.load(("A", state["pair_in"], o), ("A", pair))
            mem.expect(("A", state["pair_in"], 0), ("A", pair))
            state["pair_in"] = (state["pair_in"] + 1) % pair_slots
            if state["pairs_issued"] < last_pair:
                state["pairs_issued"] += 1
        for w in range(word_ops):
            mem.load(("W", slot, w), ("W", step))
        mem.expect(("W", slot, 0), ("W", step))
        scales = group and step % 4 == 0
        if scales:
            mem.load(("S", (step // 4) % 2), ("S", step // 4))
            mem.expect(("S", (step // 4) % 2), ("S", step // 4))
        if state["issued"] < last:
            state["issued"] += 1
        return scales

    def fetch(step, slot, pair_slot):
        for w in range(word_ops):
            mem.read(("W", slot, w), ("W", step))
        for o in range(a_ops):
            mem.read(("A", pair_slot, o), ("A", step // 2))
        if step % 2 == 0 and step + 1 <= last:                  # the pair's second step reads the slot again
            mem.expect(("A", pair_slot, 0), ("A", step // 2))

    slot_in = 0
    for d in range(depth - 1):
        issue(slot_in, d % 2 == 0)
        slot_in = (slot_in + 1) % depth
    mem.wait(wait_odd)
    fetch(0, 0, 0)
    slot_rd, pair_rd, scales_in_flight = 1, 0, False
    for s in range(0, steps, unroll):
        for u in range(unroll):
            scales = issue(slot_in, (u + depth - 1) % 2 == 0)
            slot_in = (slot_in + 1) % depth
            if group and u == 1:
                scales_in_flight = scales
            one_more = group and u in (1, 2) and scales_in_flight
            mem.wait((wait_odd if u % 2 else wait_even) + (1 if one_more else 0))
            if u % 2:
                pair_rd = (pair_rd + 1) % pair_slots
            if s + u + 1 <= last:
                fetch(s + u + 1, slot_rd, pair_rd)
            else:                                                # the look-ahead past the end reads a refetched last step
                mem.pending_reads.clear()
            slot_rd = (slot_rd + 1) % depth
        if group:
            mem.read(("S", (s // 4) % 2), ("S", s // 4))
    mem.wait(0)


@pytest.mark.parametrize("arows", [4, 16])
def test_decode_loop(arows):
    for steps in (4, 8, 12, 16, 40):
        run_m16(steps, 4, arows, fp6=False, group=True)
    for steps in (2, 4, 6, 10, 32):
        run_m16(steps, 4, arows, fp6=False, group=False)
        run_m16(steps, 3, arows, fp6=True, group=False)


def test_decode_loop_notices_a_lenient_wait(monkeypatch):
    """The replay is sharp: one load more allowed in flight, and a read comes too early."""
    import sys
    me = sys.modules[__name__]
    real = me.newer_step_ops
    monkeypatch.setattr(me, "newer_step_ops", lambda *a: real(*a) + 1)
    with pytest.raises(AssertionError, match="before its load completed"):
        run_m16(16, 4, 16, fp6=False, group=True)


def run_mb_ring(steps, depth, mb, fp6, group):
    """gemm_mb.h stream_tile_mb: one slot per step holds the words and MB blocks of A; the FP6 2-bit plane goes to one
    of two register sets; the load of group scales closes the fetch of every fourth step."""
    group = group and not fp6
    k_ops = 2 + mb + (2 if fp6 else 0)
    unroll = 4 if group else 2
    scale_u = (5 - depth) & 3
    mem = Memory()
    state = dict(issued=0)
    last = steps - 1

    def issue(slot, reg_set):
        step = state["issued"]
        for w in range(2):
            mem.load(("W", slot, w), ("W", step))
        for b in range(mb):
            mem.load(("A", slot, b), ("A", step))
        mem.expect(("W", slot, 0), ("W", step))
        mem.expect(("A", slot, 0), ("A", step))
        if fp6:
            for w in range(2):
                mem.load(("T", reg_set, w), ("T", step))
            mem.expect(("T", reg_set, 0), ("T", step))
        scales = group and step % 4 == 0
        if scales:
            mem.load(("S", (step // 4) % 2), ("S", step // 4))
            mem.expect(("S", (step // 4) % 2), ("S", step // 4))
        if state["issued"] < last:
            state["issued"] += 1
        return scales

    slot_in = 0
    for d in range(depth - 1):
        issue(slot_in, d & 1)
        slot_in = (slot_in + 1) % depth
    mem.wait(k_ops * (depth - 2))
    for w in range(2):
        mem.read(("W", 0, w), ("W", 0))
    mem.read(("A", 0, 0), ("A", 0))
    if fp6:
        mem.read(("T", 0, 0), ("T", 0))
    if group:
        mem.read(("S", 0), ("S", 0))
    slot_rd, scales_in_flight = 1, False
    for s in range(0, steps, unroll):
        for u in range(unroll):
            scales = issue(slot_in, u & 1)
            slot_in = (slot_in + 1) % depth
            if group and u == scale_u:
                scales_in_flight = scales
            more = group and scale_u <= u < scale_u + depth - 2 and scales_in_flight
            mem.wait(k_ops * (depth - 2) + (1 if more else 0))
            nxt = s + u + 1
            if nxt <= last:
                for w in range(2):
                    mem.read(("W", slot_rd, w), ("W", nxt))
                if group and u == unroll - 1:
                    mem.read(("S", (nxt // 4) % 2), ("S", nxt // 4))
                # this step's remaining A blocks and the first two of the next step are read while it multiplies; the
                # 2-bit plane of the next step is consumed by its dequantisation, also during this step
                for b in range(mb):
                    mem.read(("A", slot_rd, b), ("A", nxt))
                if fp6:
                    for w in range(2):
                        mem.read(("T", (u + 1) & 1, w), ("T", nxt))
            else:
                mem.pending_reads.clear()
            slot_rd = (slot_rd + 1) % depth
    mem.wait(0)


def test_ring_loop_of_the_row_block_kernel():
    for steps in (4, 8, 20):
        run_mb_ring(steps, 4, 2, fp6=False, group=True)
        run_mb_ring(steps, 3, 4, fp6=False, group=True)
    for steps in (2, 4, 6, 14):
        run_mb_ring(steps, 4, 2, fp6=False, group=False)
        run_mb_ring(steps, 3, 4, fp6=False, group=False)
        run_mb_ring(steps, 3, 2, fp6=True, group=False)
        run_mb_ring(steps, 3, 4, fp6=True, group=False)


def run_mb_paired(steps, group, mb=4):
    """gemm_mb.h stream_tile_mbp: A by pairs of steps into two pair slots, the words into two register sets."""
    w_ops, a_ops = 2, 2 * mb
    unroll = 4 if group else 2
    mem = Memory()
    state = dict(issued=0, pairs_issued=0, a_slot=0)
    last, last_pair = steps - 1, steps // 2 - 1

    def issue_a():
        pair = state["pairs_issued"]
        for q in range(a_ops):
            mem.load(("A", state["a_slot"], q), ("A", pair))
        mem.expect(("A", state["a_slot"], 0), ("A", pair))
        state["a_slot"] ^= 1
        if state["pairs_issued"] < last_pair:
            state["pairs_issued"] += 1

    def issue_w(reg_set):
        step = state["issued"]
        scales = group and step % 4 == 0
        if scales:
            mem.load(("S", (step // 4) % 2), ("S", step // 4))
            mem.expect(("S", (step // 4) % 2), ("S", step // 4))
        for w in range(w_ops):
            mem.load(("W", reg_set, w), ("W", step))
        mem.expect(("W", reg_set, 0), ("W", step))
        if state["issued"] < last:
            state["issued"] += 1
        return scales

    def read_a(step, blocks, slot):
        for b in blocks:
            for o in range(2):
                mem.read(("A", slot, 2 * b + o), ("A", step // 2))
        # the slot is needed again unless this was block mb - 1 of the pair's second step
        if not (step % 2 == 1 and blocks[-1] == mb - 1):
            mem.expect(("A", slot, 0), ("A", step // 2))

    issue_a()
    issue_w(0)
    issue_w(1)
    mem.wait(w_ops)
    cur = 0                                                       # pair slot of the step being multiplied
    read_a(0, [0, 1], cur)
    if group:
        mem.read(("S", 0), ("S", 0))
    for w in range(w_ops):                                        # the words of step 0 are dequantised up front
        mem.read(("W", 0, w), ("W", 0))
    for s in range(0, steps, unroll):
        for u in range(unroll):
            step = s + u
            scales = issue_w(u & 1)
            if u % 2 == 0:
                issue_a()
            mem.wait(a_ops + w_ops + (1 if (u % 2 == 0 and scales) else 0))
            nxt = step + 1
            if group and u == unroll - 1 and nxt <= last:
                mem.read(("S", (nxt // 4) % 2), ("S", nxt // 4))
            # blocks 2 .. mb-1 of this step, then (second step of a pair: after the wait in its middle) blocks 0, 1 of the next
            read_a(step, list(range(2, mb)), cur)
            if u % 2 == 1:
                mem.wait(w_ops)
            if nxt <= last:
                read_a(nxt, [0, 1], cur if u % 2 == 0 else cur ^ 1)
                for w in range(w_ops):                            # the next step's words, between this step's MFMAs
                    mem.read(("W", (u + 1) & 1, w), ("W", nxt))
            else:
                mem.pending_reads.clear()
            if u % 2 == 1:
                cur ^= 1
    mem.wait(0)


def test_paired_loop_of_the_row_block_kernel():
    for steps in (4, 8, 12, 36):
        run_mb_paired(steps, group=True)
    for steps in (2, 4, 6, 10, 30):
        run_mb_paired(steps, group=False)


def test_paired_loop_notices_a_missing_wait(monkeypatch):
    """Without the wait in the middle of a pair's second step the next pair is read while it may still be in flight."""
    real_wait = Memory.wait
    calls = itertools.count()

    def lenient(self, n):
        # drop the waits that allow only the words (the mid-step ones; the first is the prologue's)
        if n == 2 and next(calls) > 0:
            return
        real_wait(self, n)

    monkeypatch.setattr(Memory, "wait", lenient)
    with pytest.raises(AssertionError, match="before its load completed"):
        run_mb_paired(12, group=False)
