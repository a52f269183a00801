// Host side above the C ABI: the continuous-batching scheduler seam of the reference
// (ContinuousBatch.swift:38-266) and a slot engine that backs it with lanes of this library.
//
//   * sl_batch_slots       - the BatchSlots protocol (ContinuousBatch.swift:38-66) as a table of callbacks.
//   * sl_sched_*           - ContinuousScheduler: requests queue up, free slots admit without a wave barrier,
//                            every round decodes all active slots in one batched step.  token_budget = 0 is the
//                            atomic policy (a prompt is prefilled whole when it gets a slot); token_budget > 0 is
//                            the budgeted policy: the running slots' one token each is reserved first, the rest
//                            of the budget drains waiting prefill in submission order through resumable
//                            admit_step calls (at least one chunk per call), behind the aggregate memory gate
//                            can_admit with head-of-line waiting (ContinuousBatch.swift:193-266).
//   * sl_lane_slots_*      - LaneBatchSlots (LaneServe.swift:26): slot = lane on shared weights, resumable
//                            prefill in chunks of max_m rows, batched step through sl_lane_step_argmax,
//                            a KV budget in tokens for can_admit.
//
// The scheduler is pure logic and reaches a device only through the callbacks; it runs synchronously on the
// caller's thread (one round per call), so a server drives it from its decode thread and guards submissions
// with its own lock.
#include <climits>
#include <cstdint>
#include <cstring>
#include <deque>
#include <vector>

#include "../../include/seedless_hip.h"

namespace {

struct Job {
  std::vector<int32_t> prompt, stop;
  int max_tokens = 0;
  bool stops_at(int32_t t) const { for (int32_t s : stop) if (s == t) return true; return false; }
};
struct Running { int job = -1; int produced = 0; int32_t last = 0; };

}  // namespace

struct sl_sched {
  sl_batch_slots slots;
  int token_budget = 0;
  sl_token_fn on_token = nullptr;
  sl_finish_fn on_finish = nullptr;
  void* user = nullptr;
  std::vector<Job> jobs;
  std::deque<int> queue;            // submitted, no slot yet
  std::vector<int> pending;         // slots that own a job still prefilling, in the order they were reserved
  std::vector<int> pending_job;     // per slot: that job, or -1
  std::vector<Running> active;      // per slot
  std::vector<int32_t> last, next;

  void yield(int job, int32_t t) { if (on_token) on_token(user, job, t); }
  void finish(int job) { if (on_finish) on_finish(user, job); }
  bool any_active() const { for (const Running& r : active) if (r.job >= 0) return true; return false; }
  int load() const {
    int n = (int)queue.size() + (int)pending.size();
    for (const Running& r : active) n += r.job >= 0;
    return n;
  }
  // first token of a freshly admitted job: stop -> finished without output; else emitted, and the slot runs on
  void activate(int slot, int job, int32_t first) {
    const Job& j = jobs[job];
    if (j.stops_at(first)) { finish(job); slots.release(slots.ctx, slot); return; }
    yield(job, first);
    if (j.max_tokens == 1) { finish(job); slots.release(slots.ctx, slot); return; }
    active[slot].job = job; active[slot].produced = 1; active[slot].last = first;
  }
  // one batched decode step over the active slots
  int decode_round() {
    if (!any_active()) return SL_OK;
    const int B = slots.slot_count;
    for (int b = 0; b < B; ++b) { last[b] = active[b].job >= 0 ? active[b].last : -1; next[b] = -1; }
    const int r = slots.step(slots.ctx, last.data(), next.data());
    if (r) return r;
    for (int b = 0; b < B; ++b) {
      Running& a = active[b];
      if (a.job < 0 || next[b] < 0) continue;
      const Job& j = jobs[a.job];
      if (j.stops_at(next[b])) { finish(a.job); a.job = -1; slots.release(slots.ctx, b); continue; }   // not emitted
      yield(a.job, next[b]);
      a.produced += 1; a.last = next[b];
      if (a.produced >= j.max_tokens) { finish(a.job); a.job = -1; slots.release(slots.ctx, b); }
    }
    return SL_OK;
  }
  int round_atomic() {
    const int B = slots.slot_count;
    for (int b = 0; b < B && !queue.empty(); ++b) {
      if (active[b].job >= 0) continue;
      const int job = queue.front(); queue.pop_front();
      const Job& j = jobs[job];
      int32_t first = 0, consumed = 0;
      if (j.max_tokens <= 0 ||
          slots.admit_step(slots.ctx, j.prompt.data(), (int)j.prompt.size(), b, 0, 0, &first, &consumed) != 0) {
        finish(job); slots.release(slots.ctx, b);       // empty budget or engine error
        continue;
      }
      activate(b, job, first);
    }
    return decode_round();
  }
  int round_budgeted() {
    const int B = slots.slot_count;
    for (int b = 0; b < B && !queue.empty(); ++b) {
      if (active[b].job >= 0 || pending_job[b] >= 0) continue;
      // the head of the queue waits until it fits; nothing behind it is admitted ahead of it
      const Job& head = jobs[queue.front()];
      const int seq_budget = (int)head.prompt.size() + 1 + head.max_tokens;
      if (slots.can_admit && !slots.can_admit(slots.ctx, (int)head.prompt.size(), seq_budget)) break;
      const int job = queue.front(); queue.pop_front();
      if (head.max_tokens <= 0) { finish(job); --b; continue; }     // nothing to produce: no slot taken
      pending.push_back(b); pending_job[b] = job;
    }
    int running = 0;
    for (const Running& r : active) running += r.job >= 0;
    int pool = token_budget - running;
    std::vector<int> still;
    std::vector<int32_t> first_of(B, 0);
    std::vector<int> ready;
    for (int b : pending) {
      if (pool <= 0) { still.push_back(b); continue; }
      const int job = pending_job[b];
      const Job& j = jobs[job];
      int32_t first = 0, consumed = 0;
      const int r = slots.admit_step(slots.ctx, j.prompt.data(), (int)j.prompt.size(), b, pool,
                                     (int)j.prompt.size() + 1 + j.max_tokens, &first, &consumed);
      if (r < 0) { pending_job[b] = -1; finish(job); slots.release(slots.ctx, b); continue; }
      pool -= consumed;                                   // only the work of this call is charged
      if (r > 0) { still.push_back(b); continue; }
      first_of[b] = first; ready.push_back(b);
    }
    pending.swap(still);
    for (int b : ready) { const int job = pending_job[b]; pending_job[b] = -1; activate(b, job, first_of[b]); }
    return decode_round();
  }
};

extern "C" {

int sl_sched_create(const sl_batch_slots* slots, int token_budget, sl_token_fn on_token, sl_finish_fn on_finish, void* user,
                    sl_sched** out) {
  if (!slots || !out || slots->slot_count < 1 || !slots->admit_step || !slots->step || !slots->release) return SL_ERR_ARG;
  sl_sched* s = new sl_sched();
  s->slots = *slots; s->token_budget = token_budget < 0 ? 0 : token_budget;
  s->on_token = on_token; s->on_finish = on_finish; s->user = user;
  const int B = slots->slot_count;
  s->pending_job.assign(B, -1); s->active.assign(B, Running()); s->last.assign(B, -1); s->next.assign(B, -1);
  *out = s;
  return SL_OK;
}
void sl_sched_destroy(sl_sched* s) { delete s; }

int sl_sched_submit(sl_sched* s, const int32_t* prompt, int n_prompt, int max_tokens, const int32_t* stop, int n_stop) {
  if (!s || !prompt || n_prompt < 1 || n_stop < 0 || (n_stop > 0 && !stop)) return SL_ERR_ARG;
  Job j;
  j.prompt.assign(prompt, prompt + n_prompt);
  if (n_stop) j.stop.assign(stop, stop + n_stop);
  j.max_tokens = max_tokens < 0 ? 0 : max_tokens;
  s->jobs.push_back(std::move(j));
  s->queue.push_back((int)s->jobs.size() - 1);
  return (int)s->jobs.size() - 1;
}

int sl_sched_round(sl_sched* s) {
  if (!s) return SL_ERR_ARG;
  if (s->load() == 0) return 0;
  const int r = s->token_budget > 0 ? s->round_budgeted() : s->round_atomic();
  if (r) return r < 0 ? r : SL_ERR_DEVICE;
  return s->load();
}

// ---- slots backed by lanes -------------------------------------------------------------------------------

}  // extern "C"

struct sl_lane_slots {
  std::vector<sl_engine*> lanes;
  std::vector<int> pos;             // resumable prefill: prompt tokens consumed per slot
  std::vector<int> reserved;        // tokens of KV budget a slot holds (0 = free)
  std::vector<sl_engine*> group;
  std::vector<int32_t> toks, outs;
  int chunk = 1, max_seq = 0;
  long kv_budget_tokens = 0;
};

namespace {

int lane_admit_step(void* ctx, const int32_t* prompt, int n_prompt, int slot, int token_budget, int seq_budget,
                    int32_t* first, int32_t* consumed) {
  sl_lane_slots* L = (sl_lane_slots*)ctx;
  *consumed = 0;
  if (slot < 0 || slot >= (int)L->lanes.size() || n_prompt < 1) return -1;
  if (seq_budget > L->max_seq || n_prompt + 1 > L->max_seq) return -1;      // would overflow the lane's KV arena
  sl_engine* e = L->lanes[slot];
  if (L->pos[slot] == 0) {
    if (sl_reset(e) != SL_OK) return -1;
    L->reserved[slot] = seq_budget > 0 ? seq_budget : L->max_seq;
  }
  // at least one chunk per call, and whole chunks only (the last one ends with the prompt)
  long grant = token_budget <= 0 ? LONG_MAX : ((long)(token_budget + L->chunk - 1) / L->chunk) * (long)L->chunk;
  int last_m = 0;
  while (L->pos[slot] < n_prompt && grant > 0) {
    const int m = n_prompt - L->pos[slot] < L->chunk ? n_prompt - L->pos[slot] : L->chunk;
    if (sl_forward_tokens(e, prompt + L->pos[slot], m, nullptr) != SL_OK) return -1;   // the rows stay on the device
    L->pos[slot] += m; *consumed += m; grant -= L->chunk; last_m = m;
  }
  if (L->pos[slot] < n_prompt) return 1;
  if (last_m == 0) return -1;                       // called again after completion
  return sl_head_argmax_rows(e, last_m - 1, 1, first) == SL_OK ? 0 : -1;
}
int lane_step(void* ctx, const int32_t* last, int32_t* next) {
  sl_lane_slots* L = (sl_lane_slots*)ctx;
  L->group.clear(); L->toks.clear();
  for (size_t b = 0; b < L->lanes.size(); ++b)
    if (last[b] >= 0) { L->group.push_back(L->lanes[b]); L->toks.push_back(last[b]); }
  if (L->group.empty()) return 0;
  L->outs.assign(L->group.size(), -1);
  const int r = sl_lane_step_argmax(L->group.data(), (int)L->group.size(), L->toks.data(), L->outs.data());
  if (r) return r;
  size_t k = 0;
  for (size_t b = 0; b < L->lanes.size(); ++b) next[b] = last[b] >= 0 ? L->outs[k++] : -1;
  return 0;
}
void lane_release(void* ctx, int slot) {
  sl_lane_slots* L = (sl_lane_slots*)ctx;
  if (slot < 0 || slot >= (int)L->lanes.size()) return;
  L->pos[slot] = 0; L->reserved[slot] = 0;
}
int lane_can_admit(void* ctx, int prompt_len, int seq_budget) {
  sl_lane_slots* L = (sl_lane_slots*)ctx;
  (void)prompt_len;
  long held = 0;
  for (int r : L->reserved) held += r;
  return held + seq_budget <= L->kv_budget_tokens ? 1 : 0;
}

}  // namespace

extern "C" {

int sl_lane_slots_create(const sl_engine* base, int n_slots, int chunk_rows, int max_seq_len, long kv_budget_tokens,
                         sl_lane_slots** out, sl_batch_slots* table) {
  if (!base || !out || !table || n_slots < 1 || chunk_rows < 1 || max_seq_len < 2) return SL_ERR_ARG;
  sl_lane_slots* L = new sl_lane_slots();
  *out = L;
  const int rows = chunk_rows > n_slots ? chunk_rows : n_slots;   // lanes[0] lends its scratch rows to the batched step
  for (int i = 0; i < n_slots; ++i) {
    sl_engine* e = nullptr;
    const int r = sl_lane_create(base, rows, max_seq_len, &e);
    if (e) L->lanes.push_back(e);
    if (r) return r;
  }
  L->pos.assign(n_slots, 0); L->reserved.assign(n_slots, 0);
  L->chunk = chunk_rows; L->max_seq = max_seq_len;
  L->kv_budget_tokens = kv_budget_tokens > 0 ? kv_budget_tokens : (long)n_slots * max_seq_len;
  table->ctx = L; table->slot_count = n_slots;
  table->admit_step = lane_admit_step; table->step = lane_step; table->release = lane_release; table->can_admit = lane_can_admit;
  return SL_OK;
}
void sl_lane_slots_destroy(sl_lane_slots* L) {
  if (!L) return;
  for (sl_engine* e : L->lanes) sl_destroy(e);
  delete L;
}

}  // extern "C"
