// Host side above the C ABI: the SuffixSpec decode loop of the reference's Tell runtime, written against the
// public entry points only (no device code, no access to the engine's internals).
//
//   * sl_suffix_draft      - Tell.suffixDraft (Tell.swift:104-175): training-free draft from the longest suffix
//                            of the sequence that occurred before, continued by majority vote.
//   * sl_spec_gate_*       - the mechanical speculation gate (Tell.swift:45-57).
//   * sl_spec_generate     - Tell.runSpecLoop (TellRuntime.swift:716-886):
//                            draft -> verify [u] + drafts as rows of one step -> accept the matching prefix;
//                            on a reject roll the step back and rebuild with the accepted rows - or, in the
//                            pending-prefix mode (the reference's opt-in "A3", TellRuntime.swift:792-845), keep
//                            the accepted tokens pending and run them as leading rows of the next step.  The loop
//                            itself (sl_spec_generate_backend) runs on a table of callbacks shaped like
//                            Tell.SpecBackend (TellRuntime.swift:83-111), so it is testable without a device.
//
// A step of M rows gives bit for bit what M single steps give here, so the token stream of the loop is the
// greedy stream exactly; the reference needs a margin test for near-ties (Tell.certTau) because its batched
// verify is not order-stable, this build does not.
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../include/seedless_hip.h"

namespace {

constexpr int SUFFIX_ALPHA = 4;     // draft length cap = alpha * match length (Tell.swift:19)
constexpr int GATE_WINDOW = 8;      // Tell.swift:45
constexpr int PENDING_CAP = 24;     // TellRuntime.swift:734

int gate_threshold(int hist_len) { return 4 + hist_len / 3000; }
int gate_window_needed(int hist_len) { const int w = GATE_WINDOW - hist_len / 6000; return w > 1 ? w : 1; }
bool gate_should_suspend(const int32_t* window, int n, int hist_len) {
  if (n < gate_window_needed(hist_len)) return false;
  long sum = 0;
  for (int i = 0; i < n; ++i) sum += window[i];
  return sum < (long)gate_threshold(hist_len) * n;
}

// Longest m in [min_match, max_match] whose suffix seq[n-m, n) also starts at an earlier position; all such
// positions vote, token by token, on the continuation.  Positions are kept most recent first: among tokens
// with equal votes the one proposed by the most recent position wins; positions that disagree with the
// chosen token drop out.
int suffix_draft(const int32_t* seq, int n, int max_match, int draft_k, int min_match, int32_t* draft) {
  if (n < min_match + 1 || draft_k < 1) return 0;
  std::vector<int> alive, kept, next;
  for (int m = max_match < n - 1 ? max_match : n - 1; m >= min_match && m >= 1; --m) {
    const int32_t* pat = seq + (n - m);
    alive.clear();
    for (int i = n - m - 1; i >= 0; --i)
      if (std::memcmp(seq + i, pat, (size_t)m * sizeof(int32_t)) == 0) alive.push_back(i);
    if (alive.empty()) continue;
    const int cap = draft_k < SUFFIX_ALPHA * m ? draft_k : SUFFIX_ALPHA * m;
    int len = 0;
    while (len < cap && !alive.empty()) {
      next.assign(alive.size(), -1);
      for (size_t k = 0; k < alive.size(); ++k) {
        const int idx = alive[k] + m + len;
        if (idx < n) next[k] = seq[idx];
      }
      int best = -1, best_votes = 0;
      for (size_t k = 0; k < alive.size(); ++k) {
        if (next[k] < 0) continue;
        int votes = 0;
        for (size_t j = 0; j < alive.size(); ++j) votes += next[j] == next[k];
        if (votes > best_votes) { best = next[k]; best_votes = votes; }   // strict: the more recent position keeps a tie
      }
      if (best < 0) break;                                                // every position ran into the end
      draft[len++] = best;
      kept.clear();
      for (size_t k = 0; k < alive.size(); ++k) if (next[k] == best) kept.push_back(alive[k]);
      alive.swap(kept);
    }
    return len;
  }
  return 0;
}

}  // namespace

extern "C" {

int sl_suffix_draft(const int32_t* seq, int n, int max_match, int draft_k, int min_match, int32_t* draft) {
  if (!seq || n < 0 || max_match < 1 || min_match < 1 || draft_k < 0 || (draft_k > 0 && !draft)) return SL_ERR_ARG;
  return suffix_draft(seq, n, max_match, draft_k, min_match, draft);
}
int sl_spec_gate_threshold(int hist_len) { return gate_threshold(hist_len); }
int sl_spec_gate_window_needed(int hist_len) { return gate_window_needed(hist_len); }
int sl_spec_gate_should_suspend(const int32_t* window, int n, int hist_len) {
  if (n < 0 || (n > 0 && !window)) return SL_ERR_ARG;
  return gate_should_suspend(window, n, hist_len) ? 1 : 0;
}

int sl_spec_generate_backend(const sl_spec_backend* b, const int32_t* prompt, int n_prompt, int n_new,
                             const sl_spec_options* opt, int32_t* out, sl_spec_stats* stats) {
  if (!b || !b->step_argmax || !b->forward_tokens || !b->first_token || !b->snapshot || !b->rollback ||
      !prompt || n_prompt < 1 || n_new < 0 || (n_new > 0 && !out) || !opt) return SL_ERR_ARG;
  const int max_rows = b->max_rows;
  if (max_rows < 1) return SL_ERR_ARG;
  int max_k = opt->max_draft < max_rows - 1 ? opt->max_draft : max_rows - 1;
  if (max_k < 0) max_k = 0;
  const int chain_k = !b->chained_step_argmax || opt->chain_k < 0 ? 0 : (opt->chain_k > 256 ? 256 : opt->chain_k);
  const int min_match = opt->min_match < 1 ? 4 : opt->min_match;
  const int reprobe = opt->gate_reprobe < 8 ? 8 : opt->gate_reprobe;
  // Pending-prefix mode: a verify step is [pending] + [u] + drafts, so the pending list is flushed once it has
  // pending_cap tokens (24 in the reference, TellRuntime.swift:734; less where max_rows is small).  The gate is
  // off in this mode (TellRuntime.swift:759).
  const bool pending_mode = opt->pending_prefix != 0;
  int pending_cap = 0;
  if (pending_mode) {
    if (max_rows < 3) return SL_ERR_ARG;
    if (max_k > max_rows - 2) max_k = max_rows - 2;
    pending_cap = max_rows - 1 - max_k < PENDING_CAP ? max_rows - 1 - max_k : PENDING_CAP;
  }
  const bool gate = opt->gate && !pending_mode;
  sl_spec_stats st;
  std::memset(&st, 0, sizeof(st));
  if (stats) *stats = st;

  // prefill in chunks of <= max_rows rows; first token from the last row (TellRuntime.swift:602, :724-727)
  int done = 0, r = 0;
  while (done < n_prompt) {
    const int m = n_prompt - done < max_rows ? n_prompt - done : max_rows;
    r = b->forward_tokens(b->ctx, prompt + done, m); if (r) return r;
    done += m;
  }
  if (n_new == 0) return SL_OK;
  int32_t u = 0;
  r = b->first_token(b->ctx, &u); if (r) return r;

  std::vector<int32_t> hist(prompt, prompt + n_prompt);   // prompt + emitted tokens; the draft source
  hist.reserve((size_t)n_prompt + n_new + 300);
  std::vector<int32_t> emitted;
  emitted.reserve((size_t)n_new + 300);
  std::vector<int32_t> drafts(max_k > 0 ? max_k : 1), rows((size_t)max_rows), evals((size_t)(max_rows > 256 ? max_rows : 256));
  std::vector<int32_t> window, pending;
  long suspended_until = -1;
  auto emit = [&](int32_t t) { emitted.push_back(t); hist.push_back(t); };

  while ((int)emitted.size() < n_new) {
    int D = 0;
    if (max_k > 0 && !(gate && (long)emitted.size() < suspended_until)) {
      hist.push_back(u);
      D = suffix_draft(hist.data(), (int)hist.size(), 32, max_k, min_match, drafts.data());
      hist.pop_back();
    }
    st.steps++; st.drafted += D; if (D == 0) st.draftless++;
    if (D == 0) {
      if (chain_k > 0 && pending.empty()) {
        // K greedy steps in one submission; the last result is the next pending token
        r = b->chained_step_argmax(b->ctx, u, chain_k, evals.data()); if (r) return r;
        st.chain_calls++;
        emit(u);
        int add = chain_k - 1;
        if (add > n_new - (int)emitted.size()) add = n_new - (int)emitted.size();
        for (int i = 0; i < add; ++i) emit(evals[i]);
        u = evals[chain_k - 1];
      } else if (!pending.empty()) {
        // one step over [pending] + [u] realises the pending rows; the last row's result follows u
        const int pk = (int)pending.size();
        std::memcpy(rows.data(), pending.data(), (size_t)pk * sizeof(int32_t));
        rows[pk] = u;
        r = b->step_argmax(b->ctx, rows.data(), pk + 1, evals.data()); if (r) return r;
        emit(u);
        u = evals[pk];
        pending.clear();
      } else {
        r = b->step_argmax(b->ctx, &u, 1, evals.data()); if (r) return r;
        emit(u);
        u = evals[0];
      }
      continue;
    }
    r = b->snapshot(b->ctx); if (r) return r;
    if (pending_mode) {
      // [pending] + [u] + drafts as one step; row pk is u's, so draft p is checked against the result of row pk + p
      const int pk = (int)pending.size();
      std::memcpy(rows.data(), pending.data(), (size_t)pk * sizeof(int32_t));
      rows[pk] = u;
      for (int i = 0; i < D; ++i) rows[pk + 1 + i] = drafts[i];
      r = b->step_argmax(b->ctx, rows.data(), pk + 1 + D, evals.data()); if (r) return r;
      int p = 0;
      while (p < D && drafts[p] == evals[pk + p]) ++p;
      st.accepted += p;
      if (p == D) {
        pending.clear();                               // the step has advanced the caches over every row
      } else {
        // reject: back to before the pending rows; u and the accepted drafts join them and wait for the next step
        st.rejects++;
        r = b->rollback(b->ctx); if (r) return r;
        pending.push_back(u);
        for (int i = 0; i < p; ++i) pending.push_back(drafts[i]);
        if ((int)pending.size() >= pending_cap) {
          r = b->forward_tokens(b->ctx, pending.data(), (int)pending.size()); if (r) return r;
          st.pending_flushes++;
          pending.clear();
        }
      }
      emit(u);
      for (int i = 0; i < p; ++i) emit(drafts[i]);
      u = evals[pk + p];
      continue;
    }
    rows[0] = u;
    for (int i = 0; i < D; ++i) rows[1 + i] = drafts[i];
    r = b->step_argmax(b->ctx, rows.data(), 1 + D, evals.data()); if (r) return r;
    int p = 0;
    while (p < D && drafts[p] == evals[p]) ++p;
    st.accepted += p;
    if (gate) {
      window.push_back(p);
      if ((int)window.size() > GATE_WINDOW) window.erase(window.begin());
      if (gate_should_suspend(window.data(), (int)window.size(), (int)hist.size())) {
        suspended_until = (long)emitted.size() + reprobe;
        st.gate_suspensions++;
      }
    }
    if (p < D) {
      // reject: undo the verify step, then run the accepted rows again so that the caches end after them
      st.rejects++;
      r = b->rollback(b->ctx); if (r) return r;
      r = b->forward_tokens(b->ctx, rows.data(), 1 + p); if (r) return r;
    }
    emit(u);
    for (int i = 0; i < p; ++i) emit(drafts[i]);
    u = evals[p];
  }
  std::memcpy(out, emitted.data(), (size_t)n_new * sizeof(int32_t));
  if (stats) *stats = st;
  return SL_OK;
}

}  // extern "C"

namespace {
// The engine behind the backend interface: each closure of Tell.SpecBackend is one entry point.
struct EngineCtx {
  sl_engine* e;
  sl_snap snap;
  int last_m;
};
int eng_step(void* c, const int32_t* t, int m, int32_t* out) { return sl_step_argmax(((EngineCtx*)c)->e, t, m, out); }
int eng_chain(void* c, int32_t first, int k, int32_t* out) { return sl_chained_step_argmax(((EngineCtx*)c)->e, first, k, out); }
int eng_forward(void* c, const int32_t* t, int m) {
  EngineCtx* x = (EngineCtx*)c;
  x->last_m = m;
  return sl_forward_tokens(x->e, t, m, nullptr);          // the rows stay on the device
}
int eng_first(void* c, int32_t* out) {
  EngineCtx* x = (EngineCtx*)c;
  return sl_head_argmax_rows(x->e, x->last_m - 1, 1, out);
}
int eng_snapshot(void* c) { EngineCtx* x = (EngineCtx*)c; return sl_snapshot(x->e, &x->snap); }
int eng_rollback(void* c) { EngineCtx* x = (EngineCtx*)c; return sl_rollback_one_step(x->e, &x->snap); }
}  // namespace

extern "C" int sl_spec_generate(sl_engine* e, const int32_t* prompt, int n_prompt, int n_new, const sl_spec_options* opt,
                                int32_t* out, sl_spec_stats* stats) {
  if (!e) return SL_ERR_ARG;
  const int max_rows = sl_max_rows(e);
  if (max_rows < 1) return SL_ERR_ARG;
  EngineCtx x{e, {}, 1};
  sl_spec_backend b;
  b.ctx = &x; b.max_rows = max_rows;
  b.step_argmax = eng_step; b.chained_step_argmax = eng_chain; b.forward_tokens = eng_forward; b.first_token = eng_first;
  b.snapshot = eng_snapshot; b.rollback = eng_rollback;
  return sl_spec_generate_backend(&b, prompt, n_prompt, n_new, opt, out, stats);
}
