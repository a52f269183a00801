"""Host-side mirror of the reference's `SeedlessFusedForward` (SeedlessFusedVerify.swift:3111)
over the C ABI: same method names (snake_case), same argument meaning, and the reference's error
behaviour — a failed step returns None and poisons the engine (`gpu_fault` becomes non-None and
every later call returns None), argument errors return None without poisoning.

numpy arrays carry host data across the boundary; nothing here computes.
"""
import ctypes as C

import numpy as np

from . import abi, lib as _lib


def _p(a):
    return a.ctypes.data if a is not None else None


class SeedlessFusedForward:
    def __init__(self, cfg, tensors, max_m=8, max_seq_len=4096, location=None, library=None):
        """cfg: ModelConfig-like; tensors: dict name -> numpy array (host) or torch tensor (device)."""
        self.lib = library or _lib.get()
        self.cfg = cfg
        self.max_m, self.max_seq_len = max_m, max_seq_len
        if location is None:
            any_t = next(iter(tensors.values()))
            location = abi.SL_LOC_DEVICE if hasattr(any_t, "data_ptr") else abi.SL_LOC_HOST
        if location == abi.SL_LOC_HOST:
            tensors = {k: np.ascontiguousarray(v) for k, v in tensors.items()}
        desc, keep = abi.build_desc(cfg, tensors, location)
        h = C.c_void_p()
        status = self.lib.dll.sl_create(C.byref(desc), max_m, max_seq_len, C.byref(h))
        del keep
        self.h = h
        if status != abi.SL_OK:
            fault = self.lib.dll.sl_fault(self.h) if self.h else None
            if self.h:
                self.lib.dll.sl_destroy(self.h)
                self.h = None
            raise _lib.SeedlessError("sl_create", status, fault.decode() if fault else None)

    # -- lanes (SeedlessLaneBatch.swift:876): sequences that share this engine's weights ---------------
    def new_lane(self, max_m=1, max_seq_len=1024):
        """A further sequence on this engine's weights.  Close the lanes before this engine."""
        h = C.c_void_p()
        status = self.lib.dll.sl_lane_create(self.h, max_m, max_seq_len, C.byref(h))
        lane = object.__new__(type(self))
        lane.lib, lane.cfg, lane.h = self.lib, self.cfg, h
        lane.max_m, lane.max_seq_len = max_m, max_seq_len
        lane._base = self                      # the weights live in the base: keep it referenced while the lane exists
        if status != abi.SL_OK:
            fault = lane.gpu_fault if h else None
            lane.close()
            raise _lib.SeedlessError("sl_lane_create", status, fault)
        return lane

    @staticmethod
    def lane_step_argmax(lanes, tokens):
        """One token in, one out per lane; per lane identical to a solo step."""
        tok = np.ascontiguousarray(tokens, np.int32)
        assert len(tok) == len(lanes) > 0
        out = np.empty(len(tok), np.int32)
        arr = (C.c_void_p * len(lanes))(*[l.h for l in lanes])
        if lanes[0].lib.dll.sl_lane_step_argmax(arr, len(lanes), _p(tok), _p(out)) != abi.SL_OK:
            return None
        return out

    def step_sample_rows(self, tokens, temperature=1.0, top_p=1.0, seed=0):
        """Not built (greedy only): returns the status code, SL_ERR_UNSUPPORTED on a healthy engine."""
        tok = np.ascontiguousarray(tokens, np.int32)
        out = np.full(len(tok), -1, np.int32)
        return self.lib.dll.sl_step_sample_rows(self.h, _p(tok), len(tok), float(temperature), float(top_p), int(seed), _p(out)), out

    # -- lifetime ---------------------------------------------------------------------------------
    def close(self):
        if getattr(self, "h", None):
            self.lib.dll.sl_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- failure firewall (GPUFaultState, SeedlessFusedVerify.swift:388-401) -------------------------
    @property
    def gpu_fault(self):
        f = self.lib.dll.sl_fault(self.h)
        return f.decode() if f else None

    def inject_failure(self):
        self.lib.dll.sl_inject_failure(self.h)

    @property
    def position(self):
        return self.lib.dll.sl_position(self.h)

    @property
    def last_gpu_ms(self):
        return self.lib.dll.sl_last_gpu_ms(self.h)

    def set_hybrid(self, enable=True):
        """forwardRowsHybrid (SeedlessFusedVerify.swift:4247): prefill chunks of >= 16 rows on the matrix cores."""
        self.lib.check(self.lib.dll.sl_set_hybrid(self.h, 1 if enable else 0), "sl_set_hybrid", self.gpu_fault)

    def set_persistent(self, enable=True):
        return self.lib.dll.sl_set_persistent(self.h, int(enable)) == abi.SL_OK

    def profile_head(self, enable=True):
        return self.lib.dll.sl_profile_head(self.h, int(enable)) == abi.SL_OK

    def profile_head_read(self):
        ms, n = C.c_double(), C.c_int64()
        self.lib.dll.sl_profile_head_read(self.h, C.byref(ms), C.byref(n))
        return ms.value, n.value

    # -- steps --------------------------------------------------------------------------------------
    def step_argmax(self, tokens):
        tok = np.ascontiguousarray(tokens, np.int32)
        out = np.empty(len(tok), np.int32)
        if self.lib.dll.sl_step_argmax(self.h, _p(tok), len(tok), _p(out)) != abi.SL_OK:
            return None
        return out

    def chained_step_argmax(self, first_token, k):
        out = np.empty(max(k, 1), np.int32)
        if self.lib.dll.sl_chained_step_argmax(self.h, int(first_token), k, _p(out)) != abi.SL_OK:
            return None
        return out[:k]

    def forward_rows(self, x, final_norm=False):
        x = np.ascontiguousarray(x, np.float16).reshape(-1, abi.H)
        out = np.empty_like(x)
        if self.lib.dll.sl_forward_rows(self.h, _p(x), x.shape[0], int(final_norm), _p(out)) != abi.SL_OK:
            return None
        return out

    def forward_tokens(self, tokens, on_device=False):
        """Tell.SpecBackend.forward.  With on_device the rows stay on the GPU (True is returned); hidden_rows and
        head_argmax_rows read them afterwards."""
        tok = np.ascontiguousarray(tokens, np.int32)
        if on_device:
            return True if self.lib.dll.sl_forward_tokens(self.h, _p(tok), len(tok), None) == abi.SL_OK else None
        out = np.empty((len(tok), abi.H), np.float16)
        if self.lib.dll.sl_forward_tokens(self.h, _p(tok), len(tok), _p(out)) != abi.SL_OK:
            return None
        return out

    def hidden_rows(self, m):
        out = np.empty((m, abi.H), np.float16)
        if self.lib.dll.sl_hidden_rows(self.h, m, _p(out)) != abi.SL_OK:
            return None
        return out

    def logits_row(self, m):
        out = np.empty(self.cfg.vocab, np.float16)
        if self.lib.dll.sl_logits_row(self.h, m, _p(out)) != abi.SL_OK:
            return None
        return out

    def head_argmax(self, normed):
        x = np.ascontiguousarray(normed, np.float16).reshape(-1, abi.H)
        out = np.empty(x.shape[0], np.int32)
        if self.lib.dll.sl_head_argmax(self.h, _p(x), x.shape[0], _p(out)) != abi.SL_OK:
            return None
        return out

    def head_argmax_rows(self, first, m=1):
        """lm_head + arg-max over rows first .. first+m-1 of the normed rows the last forward left on the device."""
        out = np.empty(m, np.int32)
        if self.lib.dll.sl_head_argmax_rows(self.h, first, m, _p(out)) != abi.SL_OK:
            return None
        return out

    def greedy_generate(self, prompt, n_new, chain_k=8):
        pr = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(max(n_new, 1), np.int32)
        if self.lib.dll.sl_greedy_generate(self.h, _p(pr), len(pr), n_new, chain_k, _p(out)) != abi.SL_OK:
            return None
        return out[:n_new]

    def spec_generate(self, prompt, n_new, max_draft=16, chain_k=8, min_match=4, gate=True, gate_reprobe=256,
                      pending_prefix=False):
        """Tell.runSpecLoop (TellRuntime.swift:716): suffix drafts verified as rows of one step; pending_prefix = its
        opt-in A3 mode (accepted tokens of a rejected step wait as leading rows of the next).  Returns
        (tokens, stats dict) or None."""
        pr = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(max(n_new, 1), np.int32)
        opt = abi.SpecOptions(max_draft, chain_k, min_match, 1 if gate else 0, gate_reprobe, 1 if pending_prefix else 0)
        st = abi.SpecStats()
        if self.lib.dll.sl_spec_generate(self.h, _p(pr), len(pr), n_new, C.byref(opt), _p(out), C.byref(st)) != abi.SL_OK:
            return None
        return out[:n_new], {n: getattr(st, n) for n, _ in abi.SpecStats._fields_}

    # -- snapshots ------------------------------------------------------------------------------------
    def snapshot(self):
        s = abi.Snap()
        return s if self.lib.dll.sl_snapshot(self.h, C.byref(s)) == abi.SL_OK else None

    def rollback_one_step(self, snap):
        return self.lib.dll.sl_rollback_one_step(self.h, C.byref(snap)) == abi.SL_OK

    def full_snapshot(self):
        s = C.c_void_p()
        if self.lib.dll.sl_full_snapshot(self.h, C.byref(s)) != abi.SL_OK:
            if s:
                self.lib.dll.sl_full_snap_free(s)
            return None
        return _FullSnap(self.lib, s)

    def full_restore(self, snap):
        return self.lib.dll.sl_full_restore(self.h, snap.h) == abi.SL_OK

    def persistent_state_data(self):
        n = self.lib.dll.sl_persist_size(self.h)
        buf = np.empty(n, np.uint8)
        if self.lib.dll.sl_persist_write(self.h, _p(buf), n) != abi.SL_OK:
            return None
        return buf.tobytes()

    def restore_persistent_state(self, data):
        buf = np.frombuffer(data, np.uint8)
        return self.lib.dll.sl_persist_restore(self.h, _p(buf), len(buf)) == abi.SL_OK

    # -- test hooks -----------------------------------------------------------------------------------
    def read_layer_cache(self, layer):
        if self.cfg.is_linear(layer):
            a = np.empty((abi.CONV_K - 1, abi.CONV_DIM), np.float16)
            b = np.empty((abi.GDN_HV, abi.GDN_D, abi.GDN_D), np.float32)
        else:
            n = self.position
            a = np.empty((abi.ATT_KV, n, abi.ATT_D), np.float16)
            b = np.empty((abi.ATT_KV, n, abi.ATT_D), np.float16)
        if self.lib.dll.sl_read_layer_cache(self.h, layer, _p(a), _p(b)) != abi.SL_OK:
            return None, None
        return a, b

    def load_layer_cache(self, layer, a, b):
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        n = 0 if self.cfg.is_linear(layer) else a.shape[1]
        return self.lib.dll.sl_load_layer_cache(self.h, layer, _p(a), _p(b), n) == abi.SL_OK

    def read_route(self, layer, m):
        inds = np.empty((m, abi.TOPK), np.int32)
        sc = np.empty((m, abi.TOPK), np.float16)
        if self.lib.dll.sl_read_route(self.h, layer, m, _p(inds), _p(sc)) != abi.SL_OK:
            return None, None
        return inds, sc

    def debug_scratch(self, which, count):
        out = np.empty(count, np.float16)
        if self.lib.dll.sl_debug_scratch(self.h, which, _p(out), count) != abi.SL_OK:
            return None
        return out

    def _block(self, fn, layer, x):
        x = np.ascontiguousarray(x, np.float16).reshape(-1, abi.H)
        out = np.empty_like(x)
        if fn(self.h, layer, _p(x), x.shape[0], _p(out)) != abi.SL_OK:
            return None
        return out

    def moe_block_rows(self, layer, x):
        return self._block(self.lib.dll.sl_moe_block_rows, layer, x)

    def gdn_layer_rows(self, layer, x):
        return self._block(self.lib.dll.sl_gdn_layer_rows, layer, x)

    def attn_layer_rows(self, layer, x):
        return self._block(self.lib.dll.sl_attn_layer_rows, layer, x)


class _FullSnap:
    def __init__(self, lib, h):
        self.lib, self.h = lib, h

    def __del__(self):
        if self.h:
            self.lib.dll.sl_full_snap_free(self.h)
            self.h = None


class LaneScheduler:
    """ContinuousScheduler over LaneBatchSlots (ContinuousBatch.swift:95, LaneServe.swift:26): requests queue up,
    free slots admit, all active slots decode in one batched step per round.  Synchronous: `run()` drives rounds
    until every submitted request has finished and returns the token streams in submission order."""

    def __init__(self, base, slots, chunk_rows=8, max_seq_len=1024, token_budget=0, kv_budget_tokens=0):
        self.lib, self.base = base.lib, base
        self.streams, self.finished = [], []
        self._tok = abi.TOKEN_FN(lambda user, job, t: self.streams[job].append(t))
        self._fin = abi.FINISH_FN(lambda user, job: self.finished.append(job))
        self.table = abi.BatchSlots()
        self.slots = C.c_void_p()
        self.h = C.c_void_p()
        r = self.lib.dll.sl_lane_slots_create(base.h, slots, chunk_rows, max_seq_len, kv_budget_tokens, C.byref(self.slots),
                                              C.byref(self.table))
        if r != abi.SL_OK:
            self.close()
            raise _lib.SeedlessError("sl_lane_slots_create", r)
        r = self.lib.dll.sl_sched_create(C.byref(self.table), token_budget, self._tok, self._fin, None, C.byref(self.h))
        if r != abi.SL_OK:
            self.close()
            raise _lib.SeedlessError("sl_sched_create", r)

    def submit(self, prompt, max_tokens, stop=()):
        p = np.ascontiguousarray(prompt, np.int32)
        s = np.ascontiguousarray(list(stop), np.int32)
        jid = self.lib.dll.sl_sched_submit(self.h, _p(p), len(p), max_tokens, _p(s) if len(s) else None, len(s))
        if jid < 0:
            raise _lib.SeedlessError("sl_sched_submit", jid)
        self.streams.append([])
        return jid

    def round(self):
        return self.lib.dll.sl_sched_round(self.h)

    def run(self, max_rounds=1 << 20):
        for _ in range(max_rounds):
            left = self.round()
            if left < 0:
                return None
            if left == 0:
                return self.streams
        return None

    def close(self):
        if self.h:
            self.lib.dll.sl_sched_destroy(self.h)
            self.h = C.c_void_p()
        if self.slots:
            self.lib.dll.sl_lane_slots_destroy(self.slots)
            self.slots = C.c_void_p()
