"""Host logic of Tell's SuffixSpec loop (no GPU): the suffix draft and the speculation gate.

Pins: the gate against the literal vectors of the reference's own self-check (Tell.specGateSelfCheck,
Tell.swift:60-78); the draft against hand-worked cases and against an independent brute-force statement of
the rule in Tell.swift:86-96 (all occurrences of the longest matching suffix vote token by token, ties to the
most recent occurrence, disagreeing occurrences drop out, length cap min(draftK, 4 * match length))."""
import ctypes as C

import numpy as np
import pytest

from qwisp_amd import abi, lib


@pytest.fixture(scope="module")
def dll():
    return lib.get().dll


def draft(dll, seq, max_match=32, draft_k=16, min_match=4):
    a = np.ascontiguousarray(seq, np.int32)
    out = np.full(max(draft_k, 1), -7, np.int32)
    n = dll.sl_suffix_draft(a.ctypes.data_as(C.c_void_p), len(a), max_match, draft_k, min_match, out.ctypes.data_as(C.c_void_p))
    assert n >= 0, n
    return out[:n].tolist()


def suspend(dll, window, hist_len):
    w = np.ascontiguousarray(window, np.int32)
    return dll.sl_spec_gate_should_suspend(w.ctypes.data_as(C.c_void_p), len(w), hist_len) == 1


def test_gate_matches_the_reference_self_check(dll):
    bad, good = [4] * 8, [20] * 8
    assert dll.sl_spec_gate_threshold(2000) == 4
    assert dll.sl_spec_gate_threshold(14000) == 8
    assert dll.sl_spec_gate_threshold(48000) == 20
    assert dll.sl_spec_gate_window_needed(0) == 8
    assert dll.sl_spec_gate_window_needed(14000) == 6
    assert dll.sl_spec_gate_window_needed(48000) == 1
    assert suspend(dll, [4], 48000)
    assert suspend(dll, bad, 48000)
    assert not suspend(dll, good, 48000)
    assert not suspend(dll, [24], 48000)
    assert not suspend(dll, bad, 0)            # 4 per attempt meets the threshold of 4
    assert not suspend(dll, [0], 0)            # a full window is needed at short context
    assert not suspend(dll, bad[4:] + [40, 40, 40, 40], 48000)


def test_suffix_draft_hand_cases(dll):
    # too short, or no earlier occurrence of the last 4 tokens
    assert draft(dll, [1, 2, 3, 4]) == []
    assert draft(dll, list(range(40))) == []
    # one earlier occurrence: its continuation up to the end of the sequence, capped at 4 * match length
    seq = [9, 1, 2, 3, 4, 5, 6, 7, 8, 1, 2, 3, 4]
    assert draft(dll, seq) == [5, 6, 7, 8, 1, 2, 3, 4]                  # match 4 -> cap 16, the source runs out after 8
    assert draft(dll, seq, draft_k=3) == [5, 6, 7]
    # the longest match decides: the suffix 2 3 4 5 6 (m = 5) occurs once, although 3 4 5 6 occurs twice
    seq = [3, 4, 5, 6, 70, 2, 3, 4, 5, 6, 80, 81, 2, 3, 4, 5, 6]
    assert draft(dll, seq)[:2] == [80, 81]
    # majority vote over occurrences, then the dissenting occurrence drops out
    a = [1, 2, 3, 4]
    seq = a + [50, 51] + a + [60, 61] + a + [50, 52] + a
    assert draft(dll, seq)[:2] == [50, 52]      # 50 wins 2:1; of the two left the more recent continues with 52
    # a tie goes to the most recent occurrence
    seq = a + [50] + a + [60] + a
    assert draft(dll, seq)[0] == 60
    # min_match is respected
    seq = [5, 1, 2, 7, 8, 1, 2]
    assert draft(dll, seq, min_match=4) == [] and draft(dll, seq, min_match=2) == [7, 8, 1, 2]


def brute_force_draft(seq, max_match, draft_k, min_match):
    n = len(seq)
    for m in range(min(max_match, n - 1), min_match - 1, -1):
        if m < 1:
            break
        starts = [i for i in range(n - m - 1, -1, -1) if seq[i:i + m] == seq[n - m:]]
        if not starts:
            continue
        out = []
        while len(out) < min(draft_k, 4 * m) and starts:
            prop = [(seq[i + m + len(out)] if i + m + len(out) < n else None) for i in starts]
            cands = [t for t in prop if t is not None]
            if not cands:
                break
            top = max(cands.count(t) for t in cands)
            best = next(t for t in prop if t is not None and cands.count(t) == top)
            out.append(best)
            starts = [i for i, t in zip(starts, prop) if t == best]
        return out
    return []


@pytest.mark.parametrize("seed", range(6))
def test_suffix_draft_equals_brute_force(dll, seed):
    rng = np.random.default_rng(seed)
    for _ in range(60):
        n = int(rng.integers(1, 120))
        vocab = int(rng.integers(2, 6))          # tiny alphabets: many repeats, many votes
        seq = rng.integers(0, vocab, n).tolist()
        mm, k, mn = int(rng.integers(1, 40)), int(rng.integers(0, 24)), int(rng.integers(1, 6))
        if mm < mn:
            mm = mn
        assert draft(dll, seq, mm, k, mn) == brute_force_draft(seq, mm, k, mn), (seq, mm, k, mn)


def test_argument_errors(dll):
    assert dll.sl_suffix_draft(None, 3, 32, 4, 4, None) == abi.SL_ERR_ARG
    assert dll.sl_spec_gate_should_suspend(None, 2, 0) == abi.SL_ERR_ARG
    assert dll.sl_spec_generate(None, None, 0, 0, None, None, None) == abi.SL_ERR_ARG


class FakeModel:
    """A deterministic stand-in for the engine behind the SpecBackend callbacks: the 'cache' is the list of tokens
    consumed so far and the next token is a function of the last three and, now and then, of the position
    (so that streams repeat, drafts get accepted, and some drafts are wrong)."""

    def __init__(self, vocab=7, max_rows=9, with_chain=True):
        self.vocab, self.cache, self.snap, self.calls = vocab, [], None, []
        self.b = abi.SpecBackend()
        self.b.ctx, self.b.max_rows = None, max_rows
        self._keep = [abi.STEP_FN(self.step), abi.CHAIN_FN(self.chain), abi.FORWARD_FN(self.forward),
                      abi.FIRST_FN(self.first), abi.VOID_FN(self.snapshot), abi.VOID_FN(self.rollback)]
        self.b.step_argmax, chain, self.b.forward_tokens, self.b.first_token, self.b.snapshot, self.b.rollback = self._keep
        if with_chain:
            self.b.chained_step_argmax = chain

    def nxt(self, hist):
        a, b, c = ([0, 0, 0] + hist)[-3:]
        bump = 1 if (len(hist) % 23) == 0 else 0
        return (3 * a + 5 * b + c * c + 1 + bump) % self.vocab

    def step(self, ctx, toks, m, out):
        self.calls.append(("step", m))
        for i in range(m):
            self.cache.append(toks[i])
            out[i] = self.nxt(self.cache)
        return 0

    def chain(self, ctx, first, k, out):
        self.calls.append(("chain", k))
        t = first
        for i in range(k):
            self.cache.append(t)
            t = out[i] = self.nxt(self.cache)
        return 0

    def forward(self, ctx, toks, m):
        self.calls.append(("forward", m))
        self.cache.extend(toks[i] for i in range(m))
        return 0

    def first(self, ctx, out):
        out[0] = self.nxt(self.cache)
        return 0

    def snapshot(self, ctx):
        self.snap = len(self.cache)
        return 0

    def rollback(self, ctx):
        assert self.snap is not None
        del self.cache[self.snap:]
        self.snap = None
        return 0

    def greedy(self, prompt, n):
        h = list(prompt)
        for _ in range(n):
            h.append(self.nxt(h))
        return h[len(prompt):]


@pytest.mark.parametrize("chain_k,gate,max_draft,with_chain", [(8, 0, 8, True), (0, 0, 8, True), (4, 1, 3, True), (8, 0, 16, False)])
def test_spec_loop_stream_equals_greedy_on_a_fake_backend(dll, chain_k, gate, max_draft, with_chain):
    """'spec stream == greedy stream' (the reference's lossless contract, TellRuntime.swift:735-738), with
    accepted drafts, rejected drafts (rollback + rebuild) and draftless chains all occurring; afterwards the
    backend's cache holds exactly prompt + stream up to its length, so no rejected row was left behind."""
    fm = FakeModel(with_chain=with_chain)
    prompt = np.array([1, 2, 3, 4, 5, 6, 1, 2, 3], np.int32)
    n_new = 300
    want = fm.greedy(prompt.tolist(), n_new + 40)
    out = np.zeros(n_new, np.int32)
    opt = abi.SpecOptions(max_draft, chain_k, 4, gate, 16, 0)
    st = abi.SpecStats()
    r = dll.sl_spec_generate_backend(C.byref(fm.b), prompt.ctypes.data_as(C.c_void_p), len(prompt), n_new, C.byref(opt),
                                     out.ctypes.data_as(C.c_void_p), C.byref(st))
    assert r == abi.SL_OK
    assert out.tolist() == want[:n_new]
    full = prompt.tolist() + want
    assert fm.cache == full[:len(fm.cache)] and len(fm.cache) >= len(prompt) + n_new - 1
    assert st.drafted > 0 and st.accepted > 0 and st.rejects > 0 and st.accepted <= st.drafted
    assert max(m for kind, m in fm.calls if kind == "step") <= fm.b.max_rows
    if chain_k and with_chain:
        assert st.chain_calls > 0 and ("chain", chain_k) in fm.calls
    else:
        assert st.chain_calls == 0 and not any(k == "chain" for k, _ in fm.calls)
    if gate:
        assert st.gate_suspensions >= 0
    # every reject was followed by a rebuild of the accepted rows
    assert sum(1 for k, _ in fm.calls if k == "forward") == -(-len(prompt) // fm.b.max_rows) + st.rejects


@pytest.mark.parametrize("chain_k,max_draft,max_rows,with_chain", [(8, 8, 40, True), (0, 8, 40, True), (4, 5, 9, True), (8, 16, 12, False)])
def test_pending_prefix_mode_stream_equals_greedy_on_a_fake_backend(dll, chain_k, max_draft, max_rows, with_chain):
    """The reference's opt-in A3 mode (TellRuntime.swift:792-845): after a reject nothing is rebuilt; the token and
    its accepted drafts wait and run as leading rows of the next step (draft p is checked against row pk + p of
    [pending] + [u] + drafts).  Same lossless contract; the backend's cache is a prefix of prompt + stream, behind
    it by at most the pending list; no step exceeds max_rows; a rebuild (forward after the prefill) only happens
    when the pending list reaches its cap."""
    fm = FakeModel(max_rows=max_rows, with_chain=with_chain)
    prompt = np.array([1, 2, 3, 4, 5, 6, 1, 2, 3], np.int32)
    n_new = 300
    want = fm.greedy(prompt.tolist(), n_new + 60)
    out = np.zeros(n_new, np.int32)
    opt = abi.SpecOptions(max_draft, chain_k, 4, 1, 16, 1)         # the gate flag is ignored in this mode
    st = abi.SpecStats()
    r = dll.sl_spec_generate_backend(C.byref(fm.b), prompt.ctypes.data_as(C.c_void_p), len(prompt), n_new, C.byref(opt),
                                     out.ctypes.data_as(C.c_void_p), C.byref(st))
    assert r == abi.SL_OK
    assert out.tolist() == want[:n_new]
    full = prompt.tolist() + want
    max_k = min(max_draft, max_rows - 2)
    cap = min(24, max_rows - 1 - max_k)
    assert fm.cache == full[:len(fm.cache)] and len(fm.cache) >= len(prompt) + n_new - 1 - (cap + max_k)
    assert st.drafted > 0 and st.accepted > 0 and st.rejects > 0 and st.gate_suspensions == 0
    assert max(m for kind, m in fm.calls if kind == "step") <= max_rows
    if cap > 1:
        assert st.rejects > st.pending_flushes            # rejects were not rebuilt at once: their tokens rode along later
    else:
        assert st.rejects == st.pending_flushes           # a list of one is flushed as soon as it exists
    forwards = [m for kind, m in fm.calls if kind == "forward"]
    assert len(forwards) == -(-len(prompt) // max_rows) + st.pending_flushes
    assert all(cap <= m <= max_rows for m in forwards[-st.pending_flushes:]) if st.pending_flushes else True
    if not (chain_k and with_chain):
        assert st.chain_calls == 0


def test_pending_prefix_mode_needs_three_rows(dll):
    fm = FakeModel(max_rows=2)
    prompt = np.array([1, 2, 3], np.int32)
    out = np.zeros(4, np.int32)
    opt = abi.SpecOptions(4, 0, 4, 0, 16, 1)
    assert dll.sl_spec_generate_backend(C.byref(fm.b), prompt.ctypes.data_as(C.c_void_p), 3, 4, C.byref(opt),
                                        out.ctypes.data_as(C.c_void_p), None) == abi.SL_ERR_ARG
