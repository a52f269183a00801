"""The continuous-batching scheduler (host logic, no GPU) against the scenarios and expected values of the
reference's own self-checks with scripted fake engines: ContinuousScheduler.selfCheck
(ContinuousBatch.swift:270-313), tokenBudgetSelfCheck (:383-470) and laneMemSelfCheck (:483-592)."""
import ctypes as C

import numpy as np
import pytest

from qwisp_amd import abi, lib


@pytest.fixture(scope="module")
def dll():
    return lib.get().dll


class Fake:
    """Scripted slots: first token = prompt[0] + 1, next token = last + 1.  Prefill advances in whole chunks of
    1024 (the final remainder completes the prompt), at least one per call whatever the budget (floor grant, as
    the reference's fake); every admit_step and every stepped slot is logged in order.  With budget_bytes set, a
    finished admit commits seq_budget 'bytes' and can_admit gates on the aggregate."""

    def __init__(self, slots=2, budget_bytes=None):
        self.n, self.chunk = slots, 1024
        self.pos, self.arena, self.log = [0] * slots, [0] * slots, []
        self.busy, self.max_busy = [False] * slots, 0
        self.budget_bytes = budget_bytes
        self.t = abi.BatchSlots()
        self.t.ctx, self.t.slot_count = None, slots
        self._keep = [abi.ADMIT_FN(self.admit_step), abi.SLOT_STEP_FN(self.step), abi.RELEASE_FN(self.release),
                      abi.CAN_ADMIT_FN(self.can_admit)]
        self.t.admit_step, self.t.step, self.t.release = self._keep[:3]
        if budget_bytes is not None:
            self.t.can_admit = self._keep[3]

    def admit_step(self, ctx, prompt, n, slot, budget, seq_budget, first, consumed):
        if not (0 <= slot < self.n) or n < 1:
            return -1
        first[0] = prompt[0] + 1
        remaining = n - self.pos[slot]
        if budget <= 0:                                    # atomic: the whole prompt, nothing logged
            took = remaining
        else:
            took = min(max(1, budget // self.chunk) * self.chunk, remaining)
            self.log.append(("admit", slot, budget, took, seq_budget))
        self.pos[slot] += took
        consumed[0] = took
        self.busy[slot] = True
        self.max_busy = max(self.max_busy, sum(self.busy))
        if self.pos[slot] >= n:
            self.arena[slot] = seq_budget
            return 0
        return 1

    def step(self, ctx, last, nxt):
        self.max_busy = max(self.max_busy, sum(self.busy))
        for s in range(self.n):
            if last[s] >= 0:
                self.log.append(("step", s))
                nxt[s] = last[s] + 1
            else:
                nxt[s] = -1
        return 0

    def release(self, ctx, slot):
        if 0 <= slot < self.n:
            self.pos[slot] = 0
            self.arena[slot] = 0
            self.busy[slot] = False

    def can_admit(self, ctx, prompt_len, seq_budget):
        return 1 if sum(self.arena) + seq_budget <= self.budget_bytes else 0


def run(dll, fake, token_budget, jobs):
    """jobs: (prompt list, max_tokens, stop list).  Returns per-job streams and the list of finished jobs."""
    streams, finished = [[] for _ in jobs], []
    tok = abi.TOKEN_FN(lambda user, job, t: streams[job].append(t))
    fin = abi.FINISH_FN(lambda user, job: finished.append(job))
    h = C.c_void_p()
    assert dll.sl_sched_create(C.byref(fake.t), token_budget, tok, fin, None, C.byref(h)) == abi.SL_OK
    for i, (prompt, max_tokens, stop) in enumerate(jobs):
        p = np.asarray(prompt, np.int32)
        s = np.asarray(stop, np.int32)
        jid = dll.sl_sched_submit(h, p.ctypes.data_as(C.c_void_p), len(p), max_tokens,
                                  s.ctypes.data_as(C.c_void_p) if len(s) else None, len(s))
        assert jid == i
    rounds = 0
    while True:
        left = dll.sl_sched_round(h)
        assert left >= 0
        rounds += 1
        assert rounds < 100000
        if left == 0:
            break
    dll.sl_sched_destroy(h)
    return streams, finished


def test_continuous_refill_streams_stop_and_slot_cap(dll):
    """ContinuousBatch.swift:289-312: five requests [100 i] x 4 tokens and one cut by a stop token, on two slots."""
    fake = Fake()
    jobs = [([100 * i], 4, []) for i in range(5)] + [([500], 100, [503])]
    streams, finished = run(dll, fake, 0, jobs)
    for i in range(5):
        assert streams[i] == [100 * i + 1, 100 * i + 2, 100 * i + 3, 100 * i + 4]      # streams_correct
    assert streams[5] == [501, 502]                                                    # stop_honored: 503 not emitted
    assert fake.max_busy == 2                                                          # concurrency_capped, slots_reused
    assert sorted(finished) == list(range(6))


def admits(log, slot):
    return [i for i, e in enumerate(log) if e[0] == "admit" and e[1] == slot]


def test_token_budget_no_starvation(dll):
    """ContinuousBatch.swift:416-430: a short decode job keeps stepping between the chunks of a long prefill."""
    f = Fake()
    out, _ = run(dll, f, 2048, [([7] * 1024, 8, []), ([9] * 6144, 2, [])])
    b1 = admits(f.log, 1)
    assert len(b1) >= 2 and out[0] == [8, 9, 10, 11, 12, 13, 14, 15]
    for k in range(1, len(b1)):
        assert ("step", 0) in f.log[b1[k - 1] + 1:b1[k]]


def test_token_budget_fifo_fairness(dll):
    """:432-442: two prompts that no single round can finish: the first submitted finishes prefill first."""
    f = Fake()
    out, _ = run(dll, f, 2048, [([3] * 4096, 1, []), ([5] * 4096, 1, [])])
    assert out == [[4], [6]]
    assert admits(f.log, 0)[-1] < admits(f.log, 1)[-1]


def test_token_budget_output_identical_to_atomic(dll):
    """:444-454: the same jobs under the atomic and the budgeted policy give the same streams."""
    jobs = [([7] * 2000, 4, []), ([21] * 3000, 3, [])]
    base, _ = run(dll, Fake(), 0, jobs)
    inter, _ = run(dll, Fake(), 1024, jobs)
    assert base == inter == [[8, 9, 10, 11], [22, 23, 24]]


def test_token_budget_pauses_only_at_chunk_boundaries(dll):
    """:456-470: a budget below one chunk still makes progress, in whole chunks or the final remainder."""
    f = Fake()
    plen = 3 * 1024 + 300
    run(dll, f, 512, [([1] * plen, 1, [])])
    took = [e[3] for e in f.log if e[0] == "admit" and e[1] == 0]
    assert took and sum(took) == plen
    cum = 0
    for c in took:
        cum += c
        assert c > 0 and (c % 1024 == 0 or cum == plen)


def test_memory_gate_head_of_line_wait(dll):
    """:556-569: budget 100 'bytes'; job0 = 71, jobX = 9 run together; job1 = 61 is the queue head and must wait for
    job0, and job2 = 12 never jumps ahead of it."""
    f = Fake(budget_bytes=100)
    run(dll, f, 2048, [([1] * 30, 40, []), ([2] * 5, 3, []), ([3] * 20, 40, []), ([4] * 7, 4, [])])
    assert [e[4] for e in f.log if e[0] == "admit"] == [71, 9, 61, 12]


def test_memory_gate_seq_budget_passthrough_and_default(dll):
    """:571-590: seq_budget = prompt + 1 + max_tokens reaches admit_step; a huge budget leaves scheduling as it was."""
    f = Fake(budget_bytes=1_000_000)
    run(dll, f, 2048, [([5] * 50, 10, [])])
    assert [e[4] for e in f.log if e[0] == "admit"] == [61]
    f = Fake(budget_bytes=1_000_000)
    out, _ = run(dll, f, 2048, [([7] * 1024, 8, []), ([9] * 6144, 2, [])])
    a1 = admits(f.log, 1)
    assert len(a1) >= 2 and out[0] == [8, 9, 10, 11, 12, 13, 14, 15]
    for k in range(1, len(a1)):
        assert ("step", 0) in f.log[a1[k - 1] + 1:a1[k]]


def test_edge_requests(dll):
    """Zero-token requests finish without output or a slot; a first token that is a stop token ends the request;
    a failing admit drops only that request."""
    f = Fake()
    out, fin = run(dll, f, 0, [([1], 0, []), ([10], 5, [11]), ([20], 2, [])])
    assert out == [[], [], [21, 22]] and sorted(fin) == [0, 1, 2]
    f = Fake()
    out, fin = run(dll, f, 2048, [([1], 0, []), ([10], 5, [11]), ([20], 2, [])])
    assert out == [[], [], [21, 22]] and sorted(fin) == [0, 1, 2] and f.max_busy <= 2
    assert dll.sl_sched_create(None, 0, abi.TOKEN_FN(0), abi.FINISH_FN(0), None, None) == abi.SL_ERR_ARG
