"""Stage timeline of the single-launch batch-1 step, from the clock stamps of `sl_debug_stage_clock`.

Every workgroup of the stamping kernel variant records, per layer and stage, when it entered the stage, when the
stage's inputs had arrived, when its preparation and its arithmetic were done and when its results went to the
store (100 MHz clock, shared by all workgroups).  From the stamps of all 256 workgroups this module derives, per
stage, how long a hand-over takes (last producer's store -> consumers see the data), how long the consumers then
need, and how far the workgroups are spread; `table()` renders the averages per layer type.

The reference's counterpart is the per-layer GPU-timestamp profile of forwardRowsProfiled
(SeedlessFusedVerify.swift:4352) and the dispatch accounting of notes/09-phase2-token-feedback-spec.md:10-15.
"""
import numpy as np

KINDS = 8
STAGES = ("in-proj", "core", "merge", "out-proj", "moe A", "moe B", "moe C")
S_IN, S_CORE, S_MERGE, S_OUT, S_A, S_B, S_C = range(7)
TICK_US = 0.01


def _unwrap(raw):
    """u32 stamps -> int64 ticks relative to the earliest stamp (0 stays 'missing' = -1)."""
    raw = np.asarray(raw, np.uint32)
    nz = raw[raw != 0]
    if nz.size == 0:
        return np.full(raw.shape, -1, np.int64)
    ref = np.uint32(nz[0])
    d = (raw - ref).astype(np.int32).astype(np.int64)
    d0 = d[raw != 0].min()
    out = d - d0
    out[raw == 0] = -1
    return out


class Timeline:
    def __init__(self, stamps, n_layers, layer_is_linear, words):
        a = _unwrap(np.asarray(stamps).reshape(-1, words))
        self.t = a.reshape(a.shape[0], words // (8 * KINDS), 8, KINDS)     # [wg, layer, stage, kind]
        self.n_layers = n_layers
        self.lin = list(layer_is_linear)

    def _agg(self, layer, stage, kind, fn):
        v = self.t[:, layer, stage, kind]
        v = v[v >= 0]
        return float(fn(v)) * TICK_US if v.size else None

    def last(self, l, s, k): return self._agg(l, s, k, np.max)
    def first(self, l, s, k): return self._agg(l, s, k, np.min)
    def median(self, l, s, k): return self._agg(l, s, k, np.median)

    def producer(self, layer, stage):
        """(layer, stage) whose stores the given stage waits for."""
        if stage == S_IN:
            return (layer - 1, S_C) if layer > 0 else None
        if stage == S_CORE:
            return (layer, S_IN)
        if stage == S_OUT:
            return (layer, S_CORE)          # (attention: the merge publishes in between; its stamp is reported apart)
        if stage == S_A:
            return (layer, S_OUT)
        if stage == S_B:
            return (layer, S_A)
        if stage == S_C:
            return (layer, S_B)
        return None

    def stage_rows(self, layer):
        """Per stage of one layer: dict of the derived times in microseconds."""
        rows = []
        for s in (S_IN, S_CORE, S_OUT, S_A, S_B, S_C):
            prod = self.producer(layer, s)
            pub_prev = self.last(prod[0], prod[1], 4) if prod else None
            r = {"stage": STAGES[s]}
            pf, pl = self.first(layer, s, 1), self.last(layer, s, 1)
            r["handover_first"] = (pf - pub_prev) if (pf is not None and pub_prev is not None) else None
            r["handover_last"] = (pl - pub_prev) if (pl is not None and pub_prev is not None) else None
            pub_last, pub_first = self.last(layer, s, 4), self.first(layer, s, 4)
            r["work"] = (pub_last - pl) if (pub_last is not None and pl is not None) else None
            r["pub_spread"] = (pub_last - pub_first) if pub_last is not None else None
            r["total"] = (pub_last - pub_prev) if (pub_last is not None and pub_prev is not None) else None
            # inside a workgroup (median workgroup): entry -> polled -> prepared -> arithmetic -> stored
            e, p, q, d, w = (self.median(layer, s, k) for k in range(5))
            r["entry_to_polled"] = (p - e) if (p is not None and e is not None) else None
            r["polled_to_prep"] = (q - p) if (q is not None and p is not None) else None
            base = q if q is not None else p
            r["prep_to_done"] = (d - base) if (d is not None and base is not None) else None
            r["done_to_store"] = (w - d) if (w is not None and d is not None) else None
            rows.append(r)
        return rows

    def layer_time(self, layer):
        a = self.last(layer, S_C, 4)
        b = self.last(layer - 1, S_C, 4) if layer > 0 else self.first(layer, S_IN, 0)
        return (a - b) if (a is not None and b is not None) else None

    def head_time(self):
        nl = self.n_layers
        end = self.last(nl, 1, 4)
        start = self.last(nl - 1, S_C, 4)
        return (end - start) if (end is not None and start is not None) else None

    def table(self):
        keys = ("handover_first", "handover_last", "work", "pub_spread", "total", "entry_to_polled", "polled_to_prep",
                "prep_to_done", "done_to_store")
        out = []
        for name, want_lin in (("GDN layers", True), ("attention layers", False)):
            layers = [l for l in range(1, self.n_layers) if bool(self.lin[l]) == want_lin]
            if not layers:
                continue
            per = [self.stage_rows(l) for l in layers]
            lt = [self.layer_time(l) for l in layers]
            lt = [x for x in lt if x is not None]
            out.append(f"{name} (n={len(layers)}): {np.mean(lt):.2f} us per layer (min {np.min(lt):.2f}, max {np.max(lt):.2f})")
            out.append("  stage      | hand-over: last store -> first / last consumer | work: last consumer -> last store | store spread | stage total"
                       " || median workgroup: entry->inputs | ->prepared | ->arithmetic | ->store")
            for si in range(6):
                vals = {}
                for k in keys:
                    v = [p[si][k] for p in per if p[si][k] is not None]
                    vals[k] = np.mean(v) if v else float("nan")
                out.append(f"  {per[0][si]['stage']:10s} | {vals['handover_first']:6.2f} / {vals['handover_last']:6.2f}"
                           f" | {vals['work']:6.2f} | {vals['pub_spread']:6.2f} | {vals['total']:6.2f}"
                           f" || {vals['entry_to_polled']:6.2f} | {vals['polled_to_prep']:6.2f} | {vals['prep_to_done']:6.2f} | {vals['done_to_store']:6.2f}")
        ht = self.head_time()
        if ht is not None:
            out.append(f"head (final norm, lm_head, arg-max): {ht:.2f} us")
        tot = self.last(self.n_layers, 1, 4)
        t0 = self.first(0, S_IN, 0)
        if tot is not None and t0 is not None:
            out.append(f"step: {tot - t0:.1f} us")
        return "\n".join(out)


    def summary(self):
        """Averages per layer type in microseconds, for a report line."""
        out = {}
        for name, want_lin in (("gdn_layer", True), ("attention_layer", False)):
            layers = [l for l in range(1, self.n_layers) if bool(self.lin[l]) == want_lin]
            if not layers:
                continue
            per = [self.stage_rows(l) for l in layers]
            lt = [x for x in (self.layer_time(l) for l in layers) if x is not None]
            d = {"us": float(np.mean(lt)) if lt else None}
            for si in range(6):
                tot = [p[si]["total"] for p in per if p[si]["total"] is not None]
                ho = [p[si]["handover_last"] for p in per if p[si]["handover_last"] is not None]
                d[per[0][si]["stage"]] = {"total_us": float(np.mean(tot)) if tot else None,
                                          "handover_us": float(np.mean(ho)) if ho else None}
            mix = [sum(p[si]["total"] or 0.0 for si in (0, 1, 2)) for p in per]
            moe = [sum(p[si]["total"] or 0.0 for si in (3, 4, 5)) for p in per]
            d["mixer_us"], d["moe_block_us"] = float(np.mean(mix)), float(np.mean(moe))
            out[name] = d
        out["head_us"] = self.head_time()
        return out


def collect(engine):
    """Stamps of the engine's most recent stamped launch as a Timeline."""
    import ctypes as C
    dll = engine.lib.dll
    words = dll.sl_stage_clock_words()
    buf = np.zeros(256 * words, np.uint32)
    st = dll.sl_debug_stage_clock(engine.h, 1, buf.ctypes.data_as(C.c_void_p), buf.size)
    if st != 0:
        raise RuntimeError(f"sl_debug_stage_clock: {st}")
    cfg = engine.cfg
    return Timeline(buf, cfg.n_layers, [cfg.is_linear(i) for i in range(cfg.n_layers)], words)
