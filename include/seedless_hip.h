/*
 * seedless_hip.h — C ABI of libseedless_hip.so, an MI355X (gfx950) implementation of the
 * Seedless fused decode engine of penta2himajin/qwisp.
 *
 * Every entry point below replaces one public member of the reference's
 * `SeedlessFusedVerify.SeedlessFusedForward` (swift/Sources/QwispCore/SeedlessFusedVerify.swift,
 * abbreviated SFV) — the object that `Tell.SpecBackend` (TellRuntime.swift:83-111) is populated
 * from — or one of the static per-block functions its tests call.  Plain pointers and sizes only.
 *
 * Conventions
 *  - fp16 data crosses the boundary as uint16_t bit patterns.
 *  - All functions returning int return SL_OK (0) or a negative sl_status.  The first failure
 *    of an engine is sticky: sl_fault() returns its message and every later call on that engine
 *    returns SL_ERR_POISONED without touching its outputs (SFV:388-401, TellRuntime.swift:193).
 *  - One process per GPU, and one call at work on it at a time (the reference serialises callers with a semaphore,
 *    LLMBackend.swift:129, and treats the GPU as exclusive, AGENTS.md:95).  Engines and lanes may be created, driven
 *    and destroyed from different threads: every entry point that submits work holds one process-wide lock until its
 *    results are back, because a batch-1 step occupies every compute unit with one launch and must not share them.
 *    sl_head_argmax_noalloc only enqueues on the caller's stream and is outside that lock: its caller keeps it from
 *    overlapping other calls on the same GPU.  A second process on the same GPU is not supported.
 *  - After sl_destroy(e) returns, e is invalid for every call, sl_fault included, also when lanes created from e
 *    keep its weights alive for a while; no lane can be created from an engine that has been destroyed.
 *  - Weights are MLX-affine 4-bit, group 64 along K: w = scale*q + bias, q packed 8 per
 *    little-endian uint32, nibble j of a word is (word >> 4*j) & 15 (SeedlessMetalForward.swift
 *    :171-174); scales/biases are fp16 [N, K/64].
 */
#ifndef SEEDLESS_HIP_H
#define SEEDLESS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fixed per-layer geometry (SeedlessEngine.swift:13-16, QwispModel.swift:108-118) ---- */
#define SL_H            2048   /* hidden size */
#define SL_MOE_I        512    /* routed and shared expert intermediate size */
#define SL_TOPK         8
#define SL_MAX_EXPERTS  256
#define SL_ATT_HEADS    16
#define SL_ATT_KV       2
#define SL_ATT_D        256
#define SL_ROPE_DIM     64
#define SL_GDN_HK       16
#define SL_GDN_HV       32
#define SL_GDN_D        128    /* d_k = d_v */
#define SL_CONV_K       4
#define SL_CONV_DIM     8192   /* 2*HK*D + HV*D */
#define SL_GDN_IN_N     12352  /* qkv 8192 + z 4096 + b 32 + a 32 */
#define SL_ATT_QKV_N    9216   /* q(+gate) 16*512 + k 512 + v 512 */

typedef enum {
  SL_OK = 0,
  SL_ERR_ARG = -1,        /* bad argument (M > maxM, sequence overflow, null pointer, bad shape) */
  SL_ERR_POISONED = -2,   /* engine has a sticky fault */
  SL_ERR_DEVICE = -3,     /* a HIP call failed; message in sl_fault() */
  SL_ERR_UNSUPPORTED = -4,
  SL_ERR_FORMAT = -5,     /* persisted-state blob does not match this engine */
  SL_ERR_TOO_LARGE = -6   /* the request exceeds a fixed capacity of the entry point (sl_head_argmax_noalloc) */
} sl_status;

/* Where the tensors named by a model description live. */
#define SL_LOC_HOST   0
#define SL_LOC_DEVICE 1

/* One quantized matrix [n, k] in the checkpoint layout. */
typedef struct {
  const uint32_t* w;        /* [n, k/8]  */
  const uint16_t* scales;   /* [n, k/64] fp16 */
  const uint16_t* biases;   /* [n, k/64] fp16 */
  int32_t n, k;
} sl_q4;

/* Gated-DeltaNet mixer weights; tensor names as in SeedlessEngine.swift:47-66. */
typedef struct {
  sl_q4 in_proj_qkv;        /* [8192, 2048] */
  sl_q4 in_proj_z;          /* [4096, 2048] */
  sl_q4 in_proj_b;          /* [32, 2048]   */
  sl_q4 in_proj_a;          /* [32, 2048]   */
  sl_q4 out_proj;           /* [2048, 4096] */
  const float*    conv1d_w; /* [8192, 4] fp32, tap 3 multiplies the newest sample */
  const uint16_t* norm_w;   /* [128] fp16 */
  const float*    a_log;    /* [32] */
  const float*    dt_bias;  /* [32] */
  /* linear_attn.norm.weight stored in fp32: used instead of norm_w when non-NULL.  The gated norm then forms
   * w * (y * inv) in fp32 without the two half roundings of the fp16 case (the reference's "promote" variant,
   * SeedlessFusedVerify.swift:2815 and :811). */
  const float*    norm_w_f32; /* [128] */
} sl_gdn_w;

/* Full-attention mixer weights; names as in SeedlessEngine.swift:69-84. */
typedef struct {
  sl_q4 q_proj;             /* [16*512, 2048], per head [q 256 | gate 256] */
  sl_q4 k_proj;             /* [512, 2048] */
  sl_q4 v_proj;             /* [512, 2048] */
  sl_q4 o_proj;             /* [2048, 4096] */
  const uint16_t* q_norm;   /* [256] fp16 */
  const uint16_t* k_norm;   /* [256] fp16 */
} sl_attn_w;

/* Sparse MoE block weights; names as in SeedlessEngine.swift:97-121. */
typedef struct {
  const uint16_t* router_w;      /* [E, 2048] fp16 gate */
  const uint16_t* shared_gate_w; /* [2048] fp16 shared_expert_gate row */
  /* The two gates as the released checkpoint stores them: MLX affine 8-bit, group 64, 4 values per little-endian
   * word (mlp.gate and mlp.shared_expert_gate, SeedlessEngine.swift:93-106; kernel qmm8, SeedlessMetalForward.swift:384).
   * Used when router_w / shared_gate_w are NULL: w [n, 512], scales and biases [n, 32]; n = E and n = 1. */
  sl_q4 router_q8;
  sl_q4 shared_gate_q8;
  sl_q4 sw_gate;                 /* [E*512, 2048]  switch_mlp.gate_proj, expert-major */
  sl_q4 sw_up;                   /* [E*512, 2048]  */
  sl_q4 sw_down;                 /* [E*2048, 512]  */
  sl_q4 sh_gate;                 /* [512, 2048] shared expert */
  sl_q4 sh_up;                   /* [512, 2048] */
  sl_q4 sh_down;                 /* [2048, 512] */
} sl_moe_w;

typedef struct {
  int32_t is_linear;             /* 1 = Gated-DeltaNet mixer, 0 = full attention (SeedlessEngine.swift:29) */
  const uint16_t* input_ln;      /* [2048] fp16 */
  const uint16_t* post_ln;       /* [2048] fp16 */
  sl_gdn_w  gdn;                 /* valid when is_linear */
  sl_attn_w attn;                /* valid when !is_linear */
  sl_moe_w  moe;
} sl_layer_desc;

typedef struct {
  int32_t n_layers;
  int32_t n_experts;             /* multiple of 8, 8..256 */
  int32_t vocab;                 /* multiple of 16 */
  int32_t location;              /* SL_LOC_HOST or SL_LOC_DEVICE, applies to every pointer below */
  const sl_layer_desc* layers;   /* [n_layers], host memory */
  sl_q4 embed;                   /* [vocab, 2048]; all-null = engine without a head */
  sl_q4 lm_head;                 /* [vocab, 2048] */
  const uint16_t* final_norm;    /* [2048] fp16 */
} sl_model_desc;

typedef struct sl_engine sl_engine;
typedef struct sl_full_snap sl_full_snap;

/* Per-layer KV lengths captured before one forward (SFV:4039 `Snapshot`). */
typedef struct { int32_t kv_len; int32_t reserved; } sl_snap;

/* SeedlessFusedForward.init (SFV:3368) + attachHead (SFV:3799).  Copies every tensor into
 * device memory in the engine's own layout; the caller may free its tensors afterwards.
 * Caches start cold: conv history zero, recurrent state zero, KV length 0
 * (SeedlessEngine.swift:149-161). */
int sl_create(const sl_model_desc* desc, int max_m, int max_seq_len, sl_engine** out);
void sl_destroy(sl_engine* e);

/* gpuFault.fault (SFV:388-401): NULL while healthy. */
const char* sl_fault(const sl_engine* e);
/* injectCBFailure (SFV:404): makes the next device submission report failure (test hook; no
 * kernel is made to fault). */
void sl_inject_failure(sl_engine* e);

/* stepArgmax (SFV:3832): M <= max_m token ids in, M greedy next-token ids out; row m attends
 * to the KV prefix base+m+1; all caches advance by M. */
int sl_step_argmax(sl_engine* e, const int32_t* tokens, int m, int32_t* out);
/* chainedStepArgmax (SFV:4413): equals K successive sl_step_argmax of one token each, the
 * output of step k feeding step k+1 on the device. */
int sl_chained_step_argmax(sl_engine* e, int32_t first_token, int k, int32_t* out);
/* stepSampleRows (SFV:3954): sampling is outside this build (greedy only).  Always returns
 * SL_ERR_UNSUPPORTED without touching `out`; Tell then samples on its own side (TellRuntime.swift:424). */
int sl_step_sample_rows(sl_engine* e, const int32_t* tokens, int m, float temperature, float top_p,
                        uint64_t seed, int32_t* out);
/* A further sequence on the weights of `base` (reference: the lanes of SeedlessLaneBatch share one weight
 * set, SeedlessLaneBatch.swift:876): own caches, scratch and stream; `base` keeps the weights.  A base destroyed
 * before its lanes stops answering calls (sticky fault) and its memory is released with the last lane.  The lane is a
 * full engine: every entry point works on it. */
int sl_lane_create(const sl_engine* base, int max_m, int max_seq_len, sl_engine** out);
/* SeedlessLaneBatch.stepArgmaxBatch (SeedlessLaneBatch.swift:876): one token in and one out per lane, per
 * lane identical (bit for bit) to a solo sl_step_argmax of that lane.  With 2 <= b <= max_m of lanes[0], and
 * lanes of one base and one max_seq_len, the lanes go through the layers together as b rows in the scratch of
 * lanes[0]: every projection, expert and lm_head kernel is launched once for all lanes, the recurrence and
 * attention kernels take each row to its lane's caches and position.  From 32 lanes on the batch is stepped as two
 * halves side by side (lanes of even index, lanes of odd index), the second in the scratch and on the stream of its
 * own first lane (lanes[1], which must have max_m >= b / 2; otherwise one group), queued by a helper thread of the call.  Otherwise the lanes'
 * single-launch steps run back to back.  After a batched step sl_logits_row(lane, 0) and sl_hidden_rows(lane, 1) give that
 * lane's row.  A device failure poisons every lane of the call. */
int sl_lane_step_argmax(sl_engine** lanes, int b, const int32_t* tokens, int32_t* out);
/* forwardRows (SFV:3641): hidden rows in, hidden rows (final_norm=0) or final-normed rows out. */
int sl_forward_rows(sl_engine* e, const uint16_t* x_f16, int m, int final_norm, uint16_t* out_f16);
/* Tell.SpecBackend.forward (TellRuntime.swift:84): embed + forwardRows with final norm.  out_f16 may be NULL: the rows
 * then stay on the device, as the reference's forward leaves them in a device array (a prefill only looks at the last
 * row of its last chunk, TellRuntime.swift:724); sl_hidden_rows and sl_head_argmax_rows read them afterwards. */
int sl_forward_tokens(sl_engine* e, const int32_t* tokens, int m, uint16_t* out_f16);
/* hiddenRows (SFV:4392): the normed rows the last step left behind (volatile). */
int sl_hidden_rows(sl_engine* e, int m, uint16_t* out_f16);
/* Logits of row m of the last sl_step_argmax (the reference keeps them in HeadBufs.logits, SFV:3783). */
int sl_logits_row(sl_engine* e, int m, uint16_t* out_f16 /* [vocab] */);
/* engine.logits (SeedlessEngine.swift:180): lm_head + argmax over already-normed rows; used for
 * the first token after prefill (TellRuntime.swift:724-727). */
int sl_head_argmax(sl_engine* e, const uint16_t* normed_f16, int m, int32_t* out);
/* The same over rows first .. first + m - 1 of the final-normed rows that the last sl_forward_tokens / sl_forward_rows
 * left on the device (engine.logits on a slice of forward's result, TellRuntime.swift:724-727): the first token after
 * a prefill without the rows' trip to the host and back.  SL_ERR_ARG when those rows are gone (a step ran since). */
int sl_head_argmax_rows(sl_engine* e, int first, int m, int32_t* out);

/* No counterpart in the reference.  sl_head_argmax for callers that cannot allocate device memory or synchronise:
 * code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  `normed_dev` [m, 2048] fp16
 * and `out_dev` [m] are device pointers, the kernels are queued on `stream` (a hipStream_t; NULL = the default
 * stream) and the call returns without waiting.  It allocates nothing, copies nothing and frees nothing: logits and
 * arg-max candidates go to a fixed 5 MiB array inside the library's device image (one copy per GPU, held until
 * the process ends).  Limits: m <= 8 rows and a vocabulary of at most 262144, beyond that SL_ERR_TOO_LARGE.  All
 * calls on one GPU share that array, so calls that overlap on a GPU (different streams or engines) race; calls
 * queued on one stream are safe.  Results equal sl_head_argmax's. */
int sl_head_argmax_noalloc(sl_engine* e, const uint16_t* normed_dev, int m, int32_t* out_dev, void* stream);

/* snapshot / rollbackOneStep (SFV:4039-4047): undo exactly one forward made after the snapshot. */
int sl_snapshot(sl_engine* e, sl_snap* s);
int sl_rollback_one_step(sl_engine* e, const sl_snap* s);
/* fullSnapshot / fullRestore (SFV:4053-4068): arbitrary rewind; KV by length, GDN deep copy. */
int sl_full_snapshot(sl_engine* e, sl_full_snap** out);
int sl_full_restore(sl_engine* e, const sl_full_snap* s);
void sl_full_snap_free(sl_full_snap* s);
/* persistentStateData / restorePersistentState (SFV:4084-4154): "QWS1" little-endian blob. */
size_t sl_persist_size(sl_engine* e);
int sl_persist_write(sl_engine* e, void* dst, size_t cap);
int sl_persist_restore(sl_engine* e, const void* src, size_t len);

/* readLayerCache (SFV:4381).  GDN layer: a = conv history [3, 8192] fp16 (oldest first),
 * b = recurrent state [32, 128, 128] fp32 ([hv][dv][dk]).  Attention layer: a = K [2, len, 256]
 * fp16 (post-RoPE), b = V [2, len, 256] fp16.  Either pointer may be NULL. */
int sl_read_layer_cache(sl_engine* e, int layer, void* a, void* b);
/* Preloaded caches (the `caches:` argument of SFV:3368).  For attention layers `len` keys are
 * written and the engine's sequence position becomes `len` (all attention layers share it). */
int sl_load_layer_cache(sl_engine* e, int layer, const void* a, const void* b, int len);
int sl_position(const sl_engine* e);

/* indsCaptureHook (SFV:3366): routing of the last forward, layer `layer`: [m, 8] each. */
int sl_read_route(sl_engine* e, int layer, int m, int32_t* inds, uint16_t* scores_f16);

/* Per-block entry points used by the reference's block-level tests and by the single-block
 * workloads: fusedMoEBlockRows (SFV:1986), fusedGdnLayerRows (SFV:3065), fusedAttnLayerRows
 * (SFV:2460).  x is the already-normed input [m, 2048]; out is the block output before the
 * residual add.  They run on layer `layer` of the engine and advance only that layer's caches
 * (an attention block call advances the engine position by m).  A single row (m = 1) takes one launch: the
 * stages of the single-launch step for that block alone (unless sl_set_persistent(e, 0)); more rows take the
 * kernel-per-stage sequence.  Same bits either way. */
int sl_moe_block_rows(sl_engine* e, int layer, const uint16_t* x_f16, int m, uint16_t* out_f16);
int sl_gdn_layer_rows(sl_engine* e, int layer, const uint16_t* x_f16, int m, uint16_t* out_f16);
int sl_attn_layer_rows(sl_engine* e, int layer, const uint16_t* x_f16, int m, uint16_t* out_f16);

/* Test hook in the spirit of the reference's diagnostic buffers (diagRouteBufs, SFV:3486): copies
 * `count` fp16 elements of an internal scratch buffer left by the last launch sequence.
 * which: 0 projection rows (stride 12352), 1 GDN core output / gated attention output (stride 4096),
 * 2 rotated queries, 3 mixer output, 4 post-normed rows, 5 routed activations, 6 shared activations,
 * 7 router logits (stride 256), 8 MoE output.  After a block entry point that ran as a single launch (one
 * row) only 3, 7 and 8 exist (one row each, taken from the launch's exchange buffers); the others answer
 * SL_ERR_UNSUPPORTED. */
int sl_debug_scratch(sl_engine* e, int which, uint16_t* out_f16, size_t count);

/* Greedy loop standing in for Tell.runSpecLoop without drafts (TellRuntime.swift:716-802):
 * prefill the prompt in chunks of <= max_m rows through sl_forward_tokens, first token = argmax
 * of lm_head on the last normed row, then sl_chained_step_argmax in chains of `chain_k`. */
int sl_greedy_generate(sl_engine* e, const int32_t* prompt, int n_prompt, int n_new, int chain_k,
                       int32_t* out);

/* ---- Tell's SuffixSpec loop (host logic above the entry points; no device code of its own) -------------
 * Tell.suffixDraft (Tell.swift:104-175): the longest suffix of seq[0, n) of length min_match..max_match that
 * also occurs earlier; every earlier occurrence votes token by token on the continuation (ties go to the
 * most recent occurrence, occurrences that disagree drop out).  At most min(draft_k, 4 * match length)
 * tokens are written to `draft`; returns their number (0 = no draft) or SL_ERR_ARG. */
int sl_suffix_draft(const int32_t* seq, int n, int max_match, int draft_k, int min_match, int32_t* draft);
/* The mechanical speculation gate (Tell.swift:45-57): break-even threshold of accepted tokens per attempt,
 * attempts needed before suspending, and the decision on a rolling window of accepted counts (1 / 0). */
int sl_spec_gate_threshold(int hist_len);
int sl_spec_gate_window_needed(int hist_len);
int sl_spec_gate_should_suspend(const int32_t* window, int n, int hist_len);

typedef struct {
  int32_t max_draft;     /* cap on draft length (maxK); verify rows = 1 + drafts <= max_m */
  int32_t chain_k;       /* draftless spans run as chains of this many steps (0 = single steps); Tell default 8 */
  int32_t min_match;     /* QWISP_SUFFIX_MINMATCH, default 4 */
  int32_t gate;          /* 1 = speculation gate on (QWISP_SPEC_GATE) */
  int32_t gate_reprobe;  /* emitted tokens before drafting is tried again (QWISP_SPEC_REPROBE, default 256, >= 8) */
  int32_t pending_prefix; /* 1 = the reference's opt-in "A3" mode (QWISP_RAW_A3, TellRuntime.swift:792-845): after a reject
                           * the accepted tokens are not run again at once but kept pending and verified as leading rows of
                           * the next step: rows = [pending] + [u] + drafts <= max_m; the list is flushed with
                           * sl_forward_tokens at min(24, max_m - 1 - max_draft) tokens; no gate; needs max_m >= 3 */
} sl_spec_options;
typedef struct {
  int32_t steps, drafted, accepted, draftless, rejects, chain_calls, gate_suspensions, pending_flushes;
} sl_spec_stats;
/* Tell.runSpecLoop (TellRuntime.swift:716-886): prefill, then per step a suffix draft, one sl_step_argmax over
 * [next token] + drafts, acceptance of the matching prefix; a reject is undone with sl_rollback_one_step and the
 * accepted rows are run again with sl_forward_tokens (or kept pending, see pending_prefix; the caches then end
 * before any tokens still pending when the loop returns).  The n_new tokens written to `out` are those of
 * sl_greedy_generate.  max_seq_len must cover n_prompt + n_new + max_draft + chain_k. */
int sl_spec_generate(sl_engine* e, const int32_t* prompt, int n_prompt, int n_new, const sl_spec_options* opt,
                     int32_t* out, sl_spec_stats* stats);
/* The same loop on a table of callbacks shaped like Tell.SpecBackend (TellRuntime.swift:83-111); every
 * callback returns 0 or an error that ends the loop.  first_token = argmax of the head on the last row of
 * the most recent forward_tokens; rollback undoes the one step made since the last snapshot;
 * chained_step_argmax may be NULL (then draftless spans run as single steps). */
typedef struct {
  void* ctx;
  int32_t max_rows;
  int (*step_argmax)(void* ctx, const int32_t* tokens, int m, int32_t* out);
  int (*chained_step_argmax)(void* ctx, int32_t first, int k, int32_t* out);
  int (*forward_tokens)(void* ctx, const int32_t* tokens, int m);
  int (*first_token)(void* ctx, int32_t* out);
  int (*snapshot)(void* ctx);
  int (*rollback)(void* ctx);
} sl_spec_backend;
int sl_spec_generate_backend(const sl_spec_backend* b, const int32_t* prompt, int n_prompt, int n_new,
                             const sl_spec_options* opt, int32_t* out, sl_spec_stats* stats);
/* ---- continuous batching: the scheduler seam (host logic; a device is reached only through the callbacks) ----
 * BatchSlots (ContinuousBatch.swift:38-66) as a table of callbacks.
 *   admit_step: advance the prefill of `prompt` in `slot` by at most token_budget tokens but at least one
 *     chunk (token_budget <= 0: the whole prompt).  The full prompt is passed every call, the slot keeps its own
 *     resume position.  seq_budget = prompt + 1 + max_tokens, the arena the request needs (0 = unknown).
 *     Returns 0 when the prompt is done (*first = greedy first token), 1 when paused at a chunk boundary,
 *     < 0 on failure; *consumed = tokens processed in this call.
 *   step: one batched decode step; last[b] = token to feed slot b or -1 for an idle slot; next[b] likewise.
 *   release: the slot's request is over.   can_admit (may be NULL = always): the aggregate memory gate. */
typedef struct {
  void* ctx;
  int32_t slot_count;
  int (*admit_step)(void* ctx, const int32_t* prompt, int n_prompt, int slot, int token_budget, int seq_budget,
                    int32_t* first, int32_t* consumed);
  int (*step)(void* ctx, const int32_t* last, int32_t* next);
  void (*release)(void* ctx, int slot);
  int (*can_admit)(void* ctx, int prompt_len, int seq_budget);
} sl_batch_slots;
typedef void (*sl_token_fn)(void* user, int job, int32_t token);
typedef void (*sl_finish_fn)(void* user, int job);
typedef struct sl_sched sl_sched;
/* ContinuousScheduler (ContinuousBatch.swift:95-266).  token_budget 0: a request is prefilled whole when a slot
 * frees up, then all active slots step together; token_budget > 0: per round the running slots' tokens are
 * reserved first and the rest of the budget drains waiting prefill in submission order, so decode is never
 * starved by a long prompt.  Stop tokens are not emitted; a request ends at max_tokens.  Runs on the caller's
 * thread: sl_sched_submit returns the job id (>= 0) reported to the callbacks, sl_sched_round does one
 * scheduling round and returns the number of requests still queued, prefilling or running (0 = idle) or an
 * error.  The caller serialises submit and round. */
int sl_sched_create(const sl_batch_slots* slots, int token_budget, sl_token_fn on_token, sl_finish_fn on_finish,
                    void* user, sl_sched** out);
void sl_sched_destroy(sl_sched* s);
int sl_sched_submit(sl_sched* s, const int32_t* prompt, int n_prompt, int max_tokens, const int32_t* stop, int n_stop);
int sl_sched_round(sl_sched* s);
/* LaneBatchSlots (LaneServe.swift:26): n_slots lanes on the weights of `base`; prefill in chunks of chunk_rows
 * rows, resumable at chunk boundaries (a budget grants whole chunks, rounded up, at least one); decode through
 * sl_lane_step_argmax; can_admit holds the sum of the admitted requests' seq_budget within kv_budget_tokens
 * (<= 0: n_slots * max_seq_len).  Fills `table` for sl_sched_create; destroy after the scheduler, before `base`. */
typedef struct sl_lane_slots sl_lane_slots;
int sl_lane_slots_create(const sl_engine* base, int n_slots, int chunk_rows, int max_seq_len, long kv_budget_tokens,
                         sl_lane_slots** out, sl_batch_slots* table);
void sl_lane_slots_destroy(sl_lane_slots* slots);
/* Back to the cold state of a new engine: position 0, conv history and recurrent state zero (release of a slot). */
int sl_reset(sl_engine* e);
/* max_m of the engine (rows per call). */
int sl_max_rows(const sl_engine* e);

/* Timing of the most recent step on the engine's stream, measured with HIP events
 * (profLastGPUMs, SFV:3137). */
float sl_last_gpu_ms(const sl_engine* e);
/* The HIP stream (hipStream_t) the engine launches on. */
void* sl_stream(sl_engine* e);
/* Batch-1 steps run as one persistent kernel launch per token when the device has at least 256
 * compute units (the reference's counterpart is the one-command-buffer step, SFV:3881-3890);
 * 0 switches to the kernel-per-stage sequence used for M > 1.  Both give identical results. */
int sl_set_persistent(sl_engine* e, int enable);
/* forwardRowsHybrid (SeedlessFusedVerify.swift:4240-4247): while enabled, calls with 16 <= m <= 2048 rows of one
 * sequence (prefill chunks) compute the dense mixer projections (GDN in/out, attention q|k|v and o) on the matrix
 * cores, the routed experts grouped by expert (steelMoEGather, SeedlessFusedVerify.swift:4174) with weights
 * dequantised to half, the attention tile pass (scores, probabilities in half, values) and, when the router and
 * shared-gate rows are fp16, their logits as one fp16 GEMM (with 8-bit gates they stay on the exact rows): an expert
 * whose logit is within fp16 noise of the eighth largest may then be chosen differently from the exact path.
 * Like the reference's matrix-unit prefill this is not bit-identical to
 * the GEMV order (tolerance-level agreement) but deterministic.  Calls whose row count and start position are multiples
 * of 64 also run the recurrence of the GDN layers block-wise on the matrix cores (the chunked form of the delta rule);
 * a prompt's rows do not depend on how it is cut into such calls, nor on how it is cut into other calls, but the two
 * kinds agree to tolerance only.
 * Enabled on the engine that drives a lane batch (lanes[0] of sl_lane_step_argmax), batches of 16 or more lanes take
 * the same projections and lm_head to the matrix cores (the experts too from 64 lanes on); recurrent state, caches
 * and attention stay on the exact kernels.  Decode steps and steps of fewer than 16 rows are unaffected. */
int sl_set_hybrid(sl_engine* e, int enable);

/* Diagnostic in the manner of forwardRowsProfiled (SFV:4352), at the grain of one stage of the single-launch step:
 * while enabled, batch-1 steps run a variant of that kernel in which every workgroup records 100 MHz clock stamps of
 * the last step of a launch (kept on chip until the launch ends, so they do not disturb what they time).  The call
 * copies the stamps of the most recent launch out, then sets the mode:
 * out[wg * sl_stage_clock_words() + (layer * 8 + stage) * 8 + kind], 0 = not reached; stage 0 in-projection, 1 recurrence
 * or attention tiles, 2 attention merge, 3 K = 4096 projection, 4 router and shared gate/up, 5 routed gate/up, 6 down and
 * combine; layer n_layers = head (stage 0 lm_head, 1 final arg-max); kind 0 stage entered, 1 inputs arrived,
 * 2 preparation done, 3 arithmetic done, 4 results stored.  A launch whose waits gave up copies its stamps out as
 * well, and reading them (enable = 0, out != NULL) is the one call a poisoned engine still answers: the stamps show
 * where every workgroup stood; the fault text names the wait that gave up first. */
int sl_debug_stage_clock(sl_engine* e, int enable, uint32_t* out, int cap_words);
int sl_stage_clock_words(void);
/* Test hook beside injectCBFailure (SFV:404) for the single-launch step's own failure path: after `rounds` unanswered
 * polling rounds a workgroup stops waiting and raises an abort word, every other workgroup leaves at its next wait,
 * the kernel ends normally and the step returns SL_ERR_DEVICE (sticky).  The engine's default is 2^19 rounds, about
 * half a second; 0 makes the first unanswered poll give up.  No kernel is made to fault or hang. */
int sl_debug_set_spin_limit(sl_engine* e, unsigned rounds);
/* Test hooks for the tags of the single-launch step (no counterpart in the reference, whose stages are separated by
 * command-buffer order).  Values exchanged between workgroups carry a counter of stage instances, 8 * (layers + 1) per
 * step; before a launch that would take it past 0x7ff00000 the library clears its exchange buffers and restarts the
 * counter, so an engine can step indefinitely.  sl_debug_set_flow_counter moves the counter (to step an engine across
 * that point in a test); sl_debug_flow_tags evaluates, without a device, the 16-bit and 32-bit tags of (layer, stage)
 * at counter value `base` and returns 1 if a launch of `steps` steps from `base` is preceded by a restart, else 0. */
int sl_debug_set_flow_counter(sl_engine* e, uint32_t value);
int sl_debug_flow_tags(uint32_t base, int layer, int stage, int steps, int n_layers, uint32_t* tag16, uint32_t* tag32);

/* Micro-benchmarks of the machine limits that bound the kernels (measurement hooks; no counterpart in the reference).
 * Each runs on the current device's default stream, allocates and frees its own buffers and returns one figure.
 *  sl_ubench_exchange: a chain of `rounds` dependent hand-overs between the 256 resident workgroups of a persistent
 *    launch (every wait bounded), microseconds per round.  mode 0: all-gather of 2048 tagged words, eight waves poll,
 *    one barrier per polling round; 1: the same with one barrier per hand-over; 2: every thread polls the two words it
 *    owns, one barrier per hand-over (the step kernel's form); 3: 256 words among the 32 workgroups of one XCD;
 *    4: 256 words among 32 workgroups spread over the XCDs.  SL_ERR_UNSUPPORTED on a part with fewer than 256 CUs.
 *  sl_ubench_gemv_stream: 2.4 GB of 4-bit rows (K = 2048) streamed through `grid` workgroups of 16 waves, TB/s.
 *    mode 0: loads only; 1: with the step kernel's dot; 2: with the dot and the 64-lane reduction per row.
 *  sl_ubench_mfma_issue: v_mfma_f32_32x32x16_f16 with `valu_steps` (0..8) unpacking steps of three vector instructions
 *    and optionally one 16-byte LDS operand read per matrix instruction, 1 or 2 waves per SIMD: TFLOP/s of the whole
 *    chip and nanoseconds per matrix instruction and SIMD. */
int sl_ubench_exchange(int mode, int rounds, float* us_per_round);
int sl_ubench_gemv_stream(int mode, int grid, float* tb_per_s);
int sl_ubench_mfma_issue(int valu_steps, int lds_read, int waves_per_simd, float* tflops, float* ns_per_mfma);

/* Per-kernel timing in the manner of forwardRowsProfiled (SFV:4352): while enabled, every launch of
 * the dominant kernel (the persistent step kernel, or lm_head in the kernel-per-stage sequence) is bracketed by HIP events on the engine's stream; the read call returns the
 * summed duration and the number of launches since it was enabled. */
int sl_profile_head(sl_engine* e, int enable);
int sl_profile_head_read(sl_engine* e, double* ms_sum, int64_t* launches);

/* ---- synthetic checkpoints (seeded, no file I/O) --------------------------------------------
 * Fills device tensors with N(0, sigma) weights quantized by the MLX affine rule, group 64.
 * Element (row, col) of tensor `seed` is a pure function of (seed, row*k + col), so any slice can
 * be regenerated independently and a host implementation of the same rule gives the same bytes. */
int sl_synth_q4(uint32_t* w_dev, uint16_t* scales_dev, uint16_t* biases_dev,
                int64_t n, int32_t k, uint64_t seed, float sigma, void* stream);
/* fp16 tensor: value = mean + sigma * normal. */
int sl_synth_f16(uint16_t* dst_dev, int64_t count, uint64_t seed, float mean, float sigma, void* stream);
/* fp32 tensor: value = mean + sigma * normal. */
int sl_synth_f32(float* dst_dev, int64_t count, uint64_t seed, float mean, float sigma, void* stream);

/* Self-test of the device arithmetic: y[i] = op(x[i]) evaluated on the GPU (host arrays in/out).
 * op: 0 exp, 1 log, 2 sigmoid (fp32), 3 sigmoid (half), 4 softplus, 5 round-to-half,
 * 6 1/sqrt(x/128 + 1e-6), 7 half(x*sigmoid(x)), 8 normal quantile. */
int sl_selftest_math(int op, const float* x_host, float* y_host, int64_t n);
/* Self-test of the matrix-core GEMM of the hybrid prefill (host arrays in and out): y[m, n] = half(sum_k x[m, k] *
 * half(s*q + b)) for 4-bit group-64 weights [n, k]; m <= 512, n % 32 == 0, k % 64 == 0. */
int sl_selftest_qmm4(const uint16_t* x_host, int m, const uint32_t* w_host, const uint16_t* scales_host,
                     const uint16_t* biases_host, int n, int k, uint16_t* y_host);

#ifdef __cplusplus
}
#endif
#endif /* SEEDLESS_HIP_H */
