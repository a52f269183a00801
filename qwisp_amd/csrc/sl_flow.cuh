// Single-launch batch-1 decode step for gfx950: 256 workgroups x 1024 threads follow one token through all
// layers, the final norm, lm_head and the arg-max.  There are no grid barriers.
//
// Every value a stage hands to the next one travels with a tag that names the stage instance that
// produced it (layer, stage, launch): fp16 activations as 32-bit words {half, tag16}, fp32 attention
// partials and arg-max candidates as 16-byte chunks {v0, v1, tag, tag}.  A consumer loads the words it
// needs (sc1, coherent across XCDs) and retries until all tags are the expected ones; producers never wait.
// Buffers are reused every layer; this is safe because between the last reader of a buffer and its next
// writer there is always a stage to which every workgroup contributes (in-proj, routed gate/up, down-proj),
// and a writer only runs after it has consumed that stage's complete output.
//
// The residual stream is not exchanged: every workgroup computes all of it (thread t keeps elements 2t, 2t+1
// in registers), only projection outputs travel.
//
// Arithmetic and reduction order are those of sl_kernels.cuh (shared helpers in sl_device.cuh).
#pragma once
#include <type_traits>
#include "sl_decode.cuh"

namespace sl {

struct FlowP {
  DecodeP d;
  uint32_t *tproj;      // projection output               [12352]
  uint32_t *tycore;     // GDN core out / gated attn out   [4096]
  uint32_t *tmix;       // mixer output                    [2048]
  uint32_t *trlog;      // router logits                   [256]
  uint32_t *tsg;        // shared-gate logit               [4]
  uint32_t *tsh;        // shared expert activations       [512]
  uint32_t *tact;       // routed activations              [8*512]
  uint32_t *tmoe;       // MoE output                      [2048]
  uint4 *tml;           // attention {max, sum, tag, tag}  [16][max_tiles]
  uint4 *tpo;           // attention {o[2c], o[2c+1], tag, tag}  [16][max_tiles][128]
  uint4 *tcand;         // {value, index, tag, tag}        [256]
  uint4 *ttok;          // {token, token, tag, tag}: the token a step of a multi-step launch hands to the next [1]
  int sdpa_round;       // long contexts: (tile, kv head) units a workgroup scores before it turns to their values
  unsigned spin_limit;  // polling rounds after which a workgroup gives up and raises the abort word (FLOW_SPIN_LIMIT; tests: 0)
  const uint16_t* xin;  // single-block launches (k_block_flow): the block's input row, plain halves [2048]
};

// Parameters live in LDS for the whole launch.  Reading them there (ds_read + readfirstlane) does not
// pass through the vector-memory return queue, so fetching a pointer never waits behind the weight
// loads that are in flight, and the scalar cache is not asked for a new line every stage.
constexpr int FLOW_MAX_LAYERS = 64;
struct FlowLds {
  FlowP F;
  LayerP layers[FLOW_MAX_LAYERS];
  unsigned long long parity;      // bit l = which copy of layer l's recurrent state / history is current
  unsigned long long linmask;     // bit l = layer l is a linear-attention layer (its parity flips every step)
  int pos;
  uint32_t base;
  int tok;                        // token of the current step when it came from the step before in the same launch
};
__shared__ FlowLds g_K;

template <typename T>
SL_DEV T uni(const T& r) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "parameter fields are 4 or 8 bytes");
  if constexpr (sizeof(T) == 4) {
    const uint32_t v = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const uint32_t*>(&r));
    return __builtin_bit_cast(T, v);
  } else {
    const uint2 v = *reinterpret_cast<const uint2*>(&r);
    const unsigned long long u = (unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane(v.x) |
                                 ((unsigned long long)(uint32_t)__builtin_amdgcn_readfirstlane(v.y) << 32);
    if constexpr (std::is_pointer<T>::value) {
      // Every pointer parameter is device memory.  Saying so keeps accesses through it on the vector-memory
      // counter only; a generic ("flat") access would also count as an LDS operation, and the next parameter
      // read from LDS would then wait for it to come back from HBM.
      typedef typename std::remove_pointer<T>::type E;
      return (T)(E __attribute__((address_space(1)))*)u;
    } else {
      return __builtin_bit_cast(T, u);
    }
  }
}

// Thread and workgroup ids pass through an empty volatile asm in every stage: index arithmetic derived
// from them is then recomputed where it is used instead of being hoisted out of the layer loop, kept live
// across all stages and spilled (a spill reload is a vector-memory load and would queue behind the weight
// prefetch).
SL_DEV int fresh_v(int x) { asm volatile("" : "+v"(x)); return x; }
SL_DEV int fresh_s(int x) { asm volatile("" : "+s"(x)); return x; }

enum { FS_IN = 0, FS_CORE = 1, FS_MERGE = 2, FS_OUT = 3, FS_A = 4, FS_B = 5, FS_C = 6 };
constexpr unsigned FLOW_SPIN_LIMIT = 1u << 19;

// `base` counts stage instances over all launches (advanced by 8*(layers+1) per step).  The 16-bit tags keep 15 bits
// of it: every slot that carries one is rewritten by the stage instance that a consumer expects before that consumer
// polls it, at most one step (8*(layers+1) < 2^15 instances) after its previous writer, so an equal tag always means
// the expected writer.  The 32-bit tags keep 31 bits, and their slots may stay untouched for any number of steps; the
// host therefore never lets the counter reach 2^31: before the launch that would, it clears every exchange buffer and
// restarts the counter at 0 (launch_decode in sl_engine.hip).
#define SL_HD __host__ __device__ __forceinline__
SL_HD uint32_t flow_tag(uint32_t base, int layer, int stage) { return 0x8000u | ((base + (uint32_t)(layer * 8 + stage)) & 0x7fffu); }
// 16-byte chunks carry the whole counter: their slots are not rewritten every layer (a key tile beyond
// the current position keeps what an earlier, longer sequence left there).
SL_HD uint32_t flow_tag32(uint32_t base, int layer, int stage) { return 0x80000000u | (base + (uint32_t)(layer * 8 + stage)); }
SL_DEV uint32_t tagged(float v, uint32_t tag) { return (uint32_t)f2h(v) | (tag << 16); }
SL_DEV bool tag_ok(uint32_t w, uint32_t tag) { return (w >> 16) == tag; }

// Loads of words that other workgroups publish.  To the optimiser a buffer-load intrinsic only reads memory, so in a
// loop that polls with it and stores nothing the load is loop-invariant: it gets hoisted, and the loop spins on its
// first look until its bound (the volatile bit of the intrinsic only acts at instruction selection).  Every loop that
// polls therefore starts its trips with SL_FRESH_LOOK(), an empty asm with a memory clobber that no load moves across.
// (One per trip: in front of every load it cost 0.45 % of the step, and an opaque offset operand per load 2 %.)
#define SL_FRESH_LOOK() asm volatile("" ::: "memory")
SL_DEV uint32_t ldw1(rsrc_t r, int idx) { return __builtin_amdgcn_raw_buffer_load_b32(r, idx * 4, 0, CO_SC1); }
SL_DEV uint2 ldw2(rsrc_t r, int idx) { const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, idx * 4, 0, CO_SC1); return make_uint2(v.x, v.y); }
SL_DEV uint4 ldw4(rsrc_t r, int idx) { const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, idx * 4, 0, CO_SC1); return make_uint4(v.x, v.y, v.z, v.w); }
// (the same with a wave-uniform part of the index in the instruction's scalar offset: no vector register per address)
SL_DEV uint4 ldw4s(rsrc_t r, int idx, int uniform_idx) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, idx * 4, uniform_idx * 4, CO_SC1);
  return make_uint4(v.x, v.y, v.z, v.w);
}
SL_DEV void stw1(rsrc_t r, int idx, uint32_t w) { __builtin_amdgcn_raw_buffer_store_b32(w, r, idx * 4, 0, CO_SC1); }
SL_DEV void stw2(rsrc_t r, int idx, uint32_t a, uint32_t b) {
  u32x2_t v; v.x = a; v.y = b;
  __builtin_amdgcn_raw_buffer_store_b64(v, r, idx * 4, 0, CO_SC1);
}
SL_DEV void stw4(rsrc_t r, int idx, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4_t v; v.x = a; v.y = b; v.z = c; v.w = d;
  __builtin_amdgcn_raw_buffer_store_b128(v, r, idx * 4, 0, CO_SC1);
}

// Diagnostic stage clock (kernel variant ST only): every workgroup keeps 100 MHz clock stamps of the last step
// it ran in LDS, word (layer * 8 + stage) * STAMP_KINDS + kind, and copies them out when the launch ends.  Nothing
// is stored to memory while the step runs, so the stamps do not disturb the polls they time.
//   kind 0 stage entered, 1 poll satisfied, 2 prologue / preparation done, 3 arithmetic done (wave 0),
//   4 results handed to the publishing wave's store, 5..7 stage specific.
constexpr int STAMP_KINDS = 8;
constexpr int STAMP_LAYERS = 41;                      // 40 layers and the head
constexpr int STAMP_WORDS = STAMP_LAYERS * 8 * STAMP_KINDS;
__shared__ uint32_t g_stamps[STAMP_WORDS];
template <bool ST>
SL_DEV void fstamp(int layer, int stage, int kind, bool who) {
  if constexpr (ST) {
    if (who && layer < STAMP_LAYERS) g_stamps[(layer * 8 + stage) * STAMP_KINDS + kind] = (uint32_t)wall_clock64();
  }
}
// One polling round's outcome for the whole workgroup: 1 = all tags present, 0 = retry, -1 = give up (spin
// limit reached here, or another workgroup raised the abort word).  One barrier per round: a wave with a
// missing tag marks slot (round % 3) in LDS before the barrier, everybody reads it after, and thread 0 then
// clears the slot of the round before (nobody can still be reading that one), so a successful round leaves
// all three slots clear for the next stage.
SL_DEV int flow_round(bool ok, unsigned& spins, unsigned* abort_word, unsigned code = 1u) {
  const unsigned slot = spins % 3u;
  if (!__all(ok ? 1 : 0) && (threadIdx.x & 63) == 0) g_L.pf[slot] = 1;
  if (threadIdx.x == 0 && (spins > g_K.F.spin_limit || ((spins & 63u) == 63u && ld_co32(abort_word) != 0))) {
    if (ld_co32(abort_word) == 0u) st_co32(abort_word, code);        // (the first to give up names its wait)
    g_L.pf[3] = 1;
  }
  lds_barrier();
  const int failed = g_L.pf[slot], dead = g_L.pf[3];
  if (threadIdx.x == 0) g_L.pf[(spins + 2u) % 3u] = 0;
  if (dead) return -1;
  if (!failed) return 1;
  ++spins;
  __builtin_amdgcn_s_sleep(1);
  return 0;
}

// The same wait with one barrier in all: every polling wave repeats its own attempt until all its lanes have their
// words, and the workgroup meets once at the end.  With a barrier per round every wave waits for the slowest wave's
// round trip again and again (all-gather of 8 KB between 256 workgroups: 2.0 against 2.2 us per dependent round).
// `attempt()` fetches what the lane still misses and returns whether the lane is complete; `polls` is uniform per
// wave.  Bounded like flow_round: a wave that gives up raises the abort word, and false comes back to everybody.
template <bool MEET = true, typename Attempt>
SL_DEV bool flow_poll(bool polls, Attempt attempt, unsigned* abort_word, unsigned code = 1u) {
  if (polls) {
    for (unsigned spins = 0;; ++spins) {
      SL_FRESH_LOOK();
      const bool ok = attempt();
      if (__all(ok ? 1 : 0)) break;
      if (spins > g_K.F.spin_limit || ((spins & 63u) == 63u && ld_co32(abort_word) != 0)) {
        if ((threadIdx.x & 63) == 0) { if (ld_co32(abort_word) == 0u) st_co32(abort_word, code); g_L.pf[3] = 1; }
        break;
      }
    }                                                   // (no back-off between attempts: a sleep of 64 clocks measured 0.3 % slower)
  }
  if constexpr (!MEET) return true;                     // the caller's next barrier is the meeting point; it looks at the give-up flag there
  lds_barrier();
  return g_L.pf[3] == 0;
}

// Prologue on the whole workgroup: thread t owns elements 2t, 2t+1 of the hidden row and keeps them in
// registers from stage to stage (every workgroup follows the whole residual stream, so it is never exchanged).
//   h' = half(h + r) (returned in h0, h1); x = w * half(h' * inv_rms(h')) -> packed into LDS with the share sums.
// Sum of squares in the canonical order (a balanced tree over the 1024 pair terms): every wave reduces its 64 pair
// terms, the 16 wave sums meet in LDS, and every wave adds them up for itself, so one barrier is enough.
SL_DEV void flow_prologue(float& h0, float& h1, bool has_r, float r0, float r1, uint32_t lnw_pair, uint16_t* xn_plain) {
  const int tid = fresh_v(threadIdx.x), lane = tid & 63, wave = tid >> 6;
  if (has_r) { h0 = f16r(h0 + r0); h1 = f16r(h1 + r1); }
  const float ws = tree_sum<64>(fmaf(h1, h1, h0 * h0));
  if (lane == 0) g_L.red[wave] = ws;
  lds_barrier();
  const float ss = tree_sum<16>(g_L.red[lane & 15]);
  const float inv = 1.0f / sqrtf(ss / 2048.0f + EPS);
  const float y0 = f16r(lo_h(lnw_pair) * f16r(h0 * inv)), y1 = f16r(hi_h(lnw_pair) * f16r(h1 * inv));
  g_L.xs[(tid & 15) * 64 + (tid >> 4)] = pack2(y0, y1);
  // a share of 32 elements = the pairs of 16 consecutive threads: balanced tree over the pair sums
  const float s = tree_sum<16>(y0 + y1);
  if ((tid & 15) == 0) g_L.sxs[tid >> 4] = s;
  if (xn_plain) *reinterpret_cast<uint32_t*>(xn_plain + 2 * tid) = pack2(y0, y1);
  lds_barrier();
}

// The same hand-over to the dot products for a row that is used as it is (the input of a single block: no residual,
// no norm): packed pairs and share sums into LDS.
SL_DEV void flow_plain_x(const uint16_t* x) {
  const int tid = fresh_v(threadIdx.x);
  const uint32_t w = *reinterpret_cast<const uint32_t*>(x + 2 * tid);
  g_L.xs[(tid & 15) * 64 + (tid >> 4)] = w;
  const float s = tree_sum<16>(lo_h(w) + hi_h(w));
  if ((tid & 15) == 0) g_L.sxs[tid >> 4] = s;
  lds_barrier();
}

// Stores of a wave are acknowledged in order with its loads, so a wave that has just published results cannot
// finish a poll before the write has travelled to memory and back.  All tagged results of a stage are therefore
// gathered in LDS and written by one wave, wave 15 (full 64-byte lines), so that only that wave's polls of the next
// stage return behind a store.  (It does poll where every thread fetches its own share of a vector: handing its
// share to another wave through LDS measured slower than the late return.)
constexpr int PUB_WAVE = DEC_WAVES - 1;
constexpr int DENSE_WAVE0 = 128 * DEC_WAVES;     // first wave of the router rows (workgroup 128)
constexpr int PAIR_WAVE0 = 160 * DEC_WAVES;      // first wave of the shared gate/up pairs (workgroups 160..191)

// ---- weight rows parked in LDS ahead of their stage ------------------------------------------------------------
// A stage that requests its weight rows when it starts has them in flight while it polls for its inputs: the polls
// of a wave return behind its own loads, and a burst of 14 MB from all workgroups at once takes 2.5 us to arrive, so
// the hand-over ends with the burst however early the inputs were published.  The rows that do not depend on the
// routing and whose stage starts with a long hand-over therefore travel one to three stages ahead, straight into LDS
// (global_load_lds_dwordx4: no registers are held meanwhile): the in-projection rows of layer l+1 are requested when
// a workgroup is through with the K = 4096 projection of layer l (the upper half of the grid has no rows there and
// starts at once), a GDN layer's out-projection rows when its recurrence stage begins (by the waves that do not poll
// there).  The ring lies in the dynamic
// LDS behind stage C's activation rows; only attention's tile stage uses that space otherwise, and no row is parked
// across it.  A wave reads back rows it requested itself after waiting for its own loads (vmcnt); rows requested by
// another wave after that wave's wait and a barrier.
constexpr int WR_OFF = 12288;                    // bytes into g_vt (stage C's rows take 9 * 16 * XC_STRIDE words = 11520 bytes)
constexpr int WR_SLOTS = DEC_WAVES * 3 + 1;      // three rows of 1 KB per wave, and the b / a row of a GDN in-projection
SL_DEV void wr_request(int slot, const uint32_t* row_words, int lane) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* glb_ptr;
  __builtin_amdgcn_global_load_lds((glb_ptr)(row_words + 4 * lane), (lds_ptr)(reinterpret_cast<unsigned char*>(g_vt) + WR_OFF + slot * 1024), 16, 0, 0);
}
SL_DEV uint4 wr_read(int slot, int lane) {
  return *reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned char*>(g_vt) + WR_OFF + slot * 1024 + 16 * lane);
}
// The rows' {scale, bias} words travel with them: 32 words per row of 2048 weights, lane l < 32 fetches word l.
constexpr int SBR_OFF = WR_OFF + WR_SLOTS * 1024;
SL_DEV void sbr_request(int slot, const uint32_t* sb_words, int lane) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* glb_ptr;
  if (lane < 32)
    __builtin_amdgcn_global_load_lds((glb_ptr)(sb_words + lane), (lds_ptr)(reinterpret_cast<unsigned char*>(g_vt) + SBR_OFF + slot * 128), 4, 0, 0);
}
SL_DEV uint32_t sbr_read(int slot, int lane) {
  return *reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned char*>(g_vt) + SBR_OFF + slot * 128 + 4 * (lane >> 1));
}
// A GDN layer's conv taps and the history rows of the channels a workgroup's recurrence unit needs (threads 0..271:
// five waves) are parked the same way while the in-projection runs: [wave][64 lanes] conv weights (16 bytes), then
// three rows of [wave][64 lanes] history words (the word that holds the channel's half).
constexpr int CVW_OFF = SBR_OFF + WR_SLOTS * 128, CVH_OFF = CVW_OFF + 5 * 1024, CV_END = CVH_OFF + 3 * 5 * 256;
static_assert(CV_END <= DEC_DYN_LDS, "the parked rows fit the dynamic LDS");
// Before a wave reads rows it requested: its loads have landed (the compiler does not know that they write LDS).
SL_DEV void wr_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

#define FLOW_IDS const int tid = fresh_v(threadIdx.x), lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); \
                 const int wg = fresh_s(blockIdx.x), G = fresh_s(gridDim.x), NW = G * DEC_WAVES, gw = wg * DEC_WAVES + wave; \
                 (void)tid; (void)lane; (void)wave; (void)wg; (void)G; (void)NW; (void)gw

// Every thread polls the two tagged words of the pair it owns of a 2048-long vector.
template <bool ST>
SL_DEV bool poll_vec2048(const DecodeP& P, const uint32_t* vec, uint32_t tag, float& r0, float& r1, int sl, int ss) {
  const int tid = fresh_v(threadIdx.x);
  const rsrc_t rr = co_rsrc(vec);
  bool ok = false;
  uint2 b = make_uint2(0u, 0u);
  if (!flow_poll(true, [&]() {
        if (!ok) {
          b = ldw2(rr, 2 * tid);
          ok = tag_ok(b.x, tag) && tag_ok(b.y, tag);
        }
        return ok;
      }, uni(P.bar) + 32, 2u)) return false;
  fstamp<ST>(sl, ss, 1, tid == 0);
  r0 = lo_h(b.x); r1 = lo_h(b.y);
  return true;
}

// ---- stage 1: input norm + in-projection ------------------------------------------------------------
// The rows of the in-projection are not equally urgent.  What the next stage waits for (GDN: q, k, v and the
// two gate logits rows, 8256 of 12352; attention: the query halves, k and v, 5120 of 9216) is computed and
// published first; the rows that are only read a stage later (GDN: z; attention: the output gates; 4096 either
// way, one per wave) follow while the first batch is on its way to its consumers, and their weights are only
// requested once this stage's own inputs have arrived, so they stream during the arithmetic.
//   GDN: workgroup wg owns the block of 32 rows gdn_row_block(wg) (wave w: two of them) and eight workgroups of
//        every XCD one of the 64 b / a rows (wave 0); deferred row 8192 + 16 wg + w.
//   attention: urgent index c = 20 wg + slot, slot = 2w, 2w + 1 on waves 0..3 and 4 + w on the others;
//        c < 4096 is query element c % 256 of head c / 256, then k and v; deferred: gate element of the same numbering.
// GDN layers, who computes what: workgroup n runs on XCD n % 8, and an exchange between workgroups of one XCD goes
// through that XCD's L2 (1.1 against 1.5 us for a few hundred words).  XCD x therefore owns the value heads 4x .. 4x+3
// with their two key heads 2x, 2x+1 in both stages: its 32 workgroups compute those heads' q, k, v rows and gate rows
// of the in-projection (8 + 8 + 16 blocks of 32 rows, eight of them one b / a row more) and then their 32 units (value
// head, 16 of its 128 value dims) of the recurrence.
SL_DEV int gdn_row_block(int wg) {              // first of the workgroup's 32 urgent in-projection rows, / 32
  const int x = wg & 7, j = wg >> 3;
  if (j < 8) return (2 * x + (j >> 2)) * 4 + (j & 3);                    // q rows of key head 2x + j/4
  if (j < 16) return 64 + (2 * x + ((j - 8) >> 2)) * 4 + (j & 3);        // k rows
  return 128 + (4 * x + ((j - 16) >> 2)) * 4 + (j & 3);                  // v rows of value head 4x + (j-16)/4
}
SL_DEV int gdn_extra_row(int wg) {              // the workgroup's b (j < 4) or a (j < 8) row, -1: none
  const int x = wg & 7, j = wg >> 3;
  return j < 4 ? 12288 + 4 * x + j : (j < 8 ? 12320 + 4 * x + (j - 4) : -1);
}
SL_DEV int gdn_unit_head(int wg) { return 4 * (wg & 7) + (wg >> 6); }   // value head of the workgroup's recurrence unit
SL_DEV int gdn_unit_dvb(int wg) { return (wg >> 3) & 7; }               // its block of 16 value dims
struct InRows { int crit[3]; int ncrit; int def; };
SL_DEV int attn_urgent_row(int c) { return c < 4096 ? ((c >> 8) * 512 + (c & 255)) : (8192 + (c - 4096)); }
SL_DEV int attn_gate_row(int zi) { return (zi >> 8) * 512 + 256 + (zi & 255); }
SL_DEV InRows in_rows(bool lin, int wg, int wave) {
  InRows r;
  if (lin) {
    const int xr = gdn_extra_row(wg);
    const bool extra = wave == 0 && xr >= 0;
    r.crit[0] = gdn_row_block(wg) * 32 + wave * 2; r.crit[1] = r.crit[0] + 1; r.crit[2] = extra ? xr : 0;
    r.ncrit = extra ? 3 : 2;
    r.def = 8192 + wg * 16 + wave;
  } else {
    const int c0 = wg * 20 + (wave < 4 ? 2 * wave : 4 + wave);
    r.ncrit = wave < 4 ? 2 : 1;
    r.crit[0] = attn_urgent_row(c0); r.crit[1] = wave < 4 ? attn_urgent_row(c0 + 1) : 0; r.crit[2] = 0;
    r.def = attn_gate_row(wg * 16 + wave);
  }
  return r;
}
// The channel a thread of a GDN recurrence unit looks after (threads 0..271: 128 query, 128 key, 16 value channels).
SL_DEV int gdn_unit_channel(int wg, int tid) {
  const int hv = gdn_unit_head(wg), dvb = gdn_unit_dvb(wg), hk = hv >> 1;
  return tid < 128 ? hk * 128 + tid : (tid < 256 ? 2048 + hk * 128 + (tid - 128) : 4096 + hv * 128 + dvb * 16 + (tid - 256));
}
SL_DEV void flow_request_conv(const LayerP& Y, int li) {
  FLOW_IDS;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* glb_ptr;
  if (wave < 5) {
    const int ch = gdn_unit_channel(wg, min(tid, 271));
    unsigned char* const lds = reinterpret_cast<unsigned char*>(g_vt);
    const uint16_t* hin = uni(Y.hist[(int)((uni(g_K.parity) >> li) & 1ull)]);
    __builtin_amdgcn_global_load_lds((glb_ptr)(uni(Y.conv_w) + ch * 4), (lds_ptr)(lds + CVW_OFF + wave * 1024), 16, 0, 0);
#pragma unroll
    for (int k = 0; k < 3; ++k)
      __builtin_amdgcn_global_load_lds((glb_ptr)(hin + k * SL_CONV_DIM + (ch & ~1)), (lds_ptr)(lds + CVH_OFF + (k * 5 + wave) * 256), 4, 0, 0);
  }
}
template <bool ST, bool PLAIN = false>
SL_DEV bool flow_in(const FlowP& F, const LayerP& Y, int li, int pos, uint32_t base, float& h0, float& h1, int step) {
  FLOW_IDS;
  fstamp<ST>(li, FS_IN, 0, tid == 0);
  const DecodeP& P = F.d;
  const bool lin = uni(Y.is_linear) != 0;
  const InRows rows = in_rows(lin, wg, wave);
  WRegs<1, 3> wr;
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    // (the rows and their scales were requested into LDS stages ago, flow_request_in: read back after the prologue)
    wr.w[j][0] = make_uint4(0, 0, 0, 0);
    wr.sb[j][0] = 0u;
  }
  const uint32_t lnw = *reinterpret_cast<const uint32_t*>(uni(Y.input_ln) + 2 * tid);
  float r0 = 0.0f, r1 = 0.0f;
  if constexpr (PLAIN) {
    // (a single block: its input row is given)
  } else if (li == 0) {
    // the token's embedding row, dequantised in half arithmetic: half(half(s * q) + b) (embed_rows_q4,
    // SeedlessFusedVerify.swift:556-569); thread t owns elements 2t, 2t+1
    if (step > 0) {
      // the token comes from the step before of this launch: workgroup 0 published it with this step's tag
      const uint32_t ttag = flow_tag32(base, 0, 7);
      const rsrc_t rt = co_rsrc(uni(F.ttok));
      unsigned spins = 0;
      for (;;) {
        bool ok = true;
        if (wave == 1) {                 // not wave 0: in workgroup 0 that one has just stored the step's results
          const uint4 c = ldw4(rt, 0);
          ok = c.z == ttag && c.w == ttag;
          if (ok && lane == 0) g_K.tok = (int)c.x;
        }
        const int v = flow_round(ok, spins, uni(P.bar) + 32, 3u);
        if (v > 0) break;
        if (v < 0) return false;
      }
    }
    const size_t tok = (size_t)(step > 0 ? uni(g_K.tok) : uni(P.tok_in)[0]);
    const uint32_t w = uni(P.emb_w)[tok * 256 + (tid >> 2)];
    const uint32_t sb = uni(P.emb_sb)[tok * 32 + (tid >> 5)];
    const float q0 = (float)((w >> (8 * (tid & 3))) & 15u), q1 = (float)((w >> (8 * (tid & 3) + 4)) & 15u);
    h0 = f16r(f16r(lo_h(sb) * q0) + hi_h(sb));
    h1 = f16r(f16r(lo_h(sb) * q1) + hi_h(sb));
  } else {
    if (!poll_vec2048<ST>(P, uni(F.tmoe), flow_tag(base, li - 1, FS_C), r0, r1, li, FS_IN)) return false;
  }
  // the deferred row (no branch around the load: the waits that follow stay exact)
  uint4 wd; uint32_t sbd;
  wd = make_uint4(0, 0, 0, 0);
  sbd = 0u;
  if (lin) flow_request_conv(Y, li);             // behind the poll, to arrive while this stage computes
  const uint32_t tin = flow_tag(base, li, FS_IN);
  if constexpr (PLAIN) { (void)lnw; flow_plain_x(uni(F.xin)); }
  else flow_prologue(h0, h1, li > 0, r0, r1, lnw, nullptr);
  fstamp<ST>(li, FS_IN, 2, tid == 0);
  uint32_t x[16]; float sx;
  lds_get_x(0, lane, x, sx);
  wr_wait();
  wr.w[0][0] = wr_read(wave * 3, lane); wr.sb[0][0] = sbr_read(wave * 3, lane);
  if (rows.ncrit >= 2) { wr.w[1][0] = wr_read(wave * 3 + 1, lane); wr.sb[1][0] = sbr_read(wave * 3 + 1, lane); }
  if (rows.ncrit >= 3) { wr.w[2][0] = wr_read(DEC_WAVES * 3, lane); wr.sb[2][0] = sbr_read(DEC_WAVES * 3, lane); }
  wd = wr_read(wave * 3 + 2, lane); sbd = sbr_read(wave * 3 + 2, lane);
  {
    // urgent rows: slot of row j = first slot of the wave + j (the extra b / a row: slot 32)
    const int slot0 = lin ? 2 * wave : (wave < 4 ? 2 * wave : 4 + wave);
    const float o0 = tree_sum<64>(share_term(wr.w[0][0], wr.sb[0][0], x, sx));
    if (lane == 0) g_L.pub[slot0] = tagged(o0, tin);
    if (rows.ncrit >= 2) {                // wave-uniform
      const float o1 = tree_sum<64>(share_term(wr.w[1][0], wr.sb[1][0], x, sx));
      if (lane == 0) g_L.pub[slot0 + 1] = tagged(o1, tin);
    }
    if (rows.ncrit >= 3) {
      const float o2 = tree_sum<64>(share_term(wr.w[2][0], wr.sb[2][0], x, sx));
      if (lane == 0) g_L.pub[32] = tagged(o2, tin);
    }
  }
  fstamp<ST>(li, FS_IN, 3, tid == 0);
  lds_barrier();
  if (wave == PUB_WAVE) {
    const rsrc_t rp = co_rsrc(uni(F.tproj));
    if (lin) {
      if (lane < 32) stw1(rp, gdn_row_block(wg) * 32 + lane, g_L.pub[lane]);
      else if (lane == 32 && gdn_extra_row(wg) >= 0) stw1(rp, gdn_extra_row(wg), g_L.pub[32]);
    } else if (lane < 20) {
      stw1(rp, attn_urgent_row(wg * 20 + lane), g_L.pub[lane]);
    }
  }
  fstamp<ST>(li, FS_IN, 4, tid == PUB_WAVE * 64);
  {
    const float od = tree_sum<64>(share_term(wd, sbd, x, sx));
    if (lane == 0) g_L.pub[40 + wave] = tagged(od, tin);
  }
  lds_barrier();
  if (wave == PUB_WAVE && lane < 16) {
    const int zi = wg * 16 + lane;
    stw1(co_rsrc(uni(F.tproj)), lin ? 8192 + zi : attn_gate_row(zi), g_L.pub[40 + lane]);
  }
  fstamp<ST>(li, FS_IN, 5, tid == PUB_WAVE * 64);
  return true;
}
// Requests the in-projection rows of layer Y for this wave into the ring (the rows in_rows() deals out).
SL_DEV void flow_request_in(const LayerP& Y) {
  FLOW_IDS;
  const InRows rows = in_rows(uni(Y.is_linear) != 0, wg, wave);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // whatever this wave last read from its places is in registers
  const uint32_t* W = uni(Y.in_w);
  const uint32_t* SB = uni(Y.in_sb);
  wr_request(wave * 3, W + (size_t)rows.crit[0] * 256, lane); sbr_request(wave * 3, SB + (size_t)rows.crit[0] * 32, lane);
  if (rows.ncrit >= 2) { wr_request(wave * 3 + 1, W + (size_t)rows.crit[1] * 256, lane); sbr_request(wave * 3 + 1, SB + (size_t)rows.crit[1] * 32, lane); }
  if (rows.ncrit >= 3) { wr_request(DEC_WAVES * 3, W + (size_t)rows.crit[2] * 256, lane); sbr_request(DEC_WAVES * 3, SB + (size_t)rows.crit[2] * 32, lane); }
  wr_request(wave * 3 + 2, W + (size_t)rows.def * 256, lane); sbr_request(wave * 3 + 2, SB + (size_t)rows.def * 32, lane);
}

// ---- GDN stage 2: conv + prep + gated delta rule ------------------------------------------------------
// New conv-history samples of a thread's channel; written to memory by the next stage once its poll is over
// (a store issued here would hold up that poll until it is acknowledged).
struct GdnHist { uint32_t t12; uint32_t tnew; };
constexpr int BETA_TID = 5 * 64, DECAY_TID = 6 * 64;
template <bool ST>
SL_DEV bool flow_gdn(const FlowP& F, const LayerP& Y, int li, uint32_t base, GdnHist& gh) {
  FLOW_IDS;
  fstamp<ST>(li, FS_CORE, 0, tid == 0);
  const DecodeP& P = F.d;
  Lds& L = g_L;
  if (wg >= 256) return true;
  const int par = (int)((uni(g_K.parity) >> li) & 1ull);
  const int hv = gdn_unit_head(wg), dvb = gdn_unit_dvb(wg), hk = hv >> 1;
  const int half = lane >> 5, l32 = lane & 31;
  // waves 8..15 hold the recurrent state (they take no part in this stage's poll)
  float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (wave >= 8) {
    const int dv = dvb * 16 + (wave - 8) * 2 + half;
    const float4 v4 = *reinterpret_cast<const float4*>(uni(Y.state[par]) + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
    s[0] = v4.x; s[1] = v4.y; s[2] = v4.z; s[3] = v4.w;
    // The workgroup's rows of the K = 4096 projection (2 KB per wave) set out for LDS now, into the places of the
    // in-projection rows.  The state waves request them, their own and those of the wave eight below: they take no
    // part in this stage's poll, which would otherwise return behind the rows.
    if (wg * DEC_WAVES < H) {
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        const int w = wave - 8 * o;
        const size_t row = (size_t)(wg * DEC_WAVES + w);
        wr_request(w * 3, uni(Y.out_w) + row * 512, lane);
        wr_request(w * 3 + 1, uni(Y.out_w) + row * 512 + 256, lane);
        sbr_request(w * 3, uni(Y.out_sb) + row * 64, lane);
        sbr_request(w * 3 + 1, uni(Y.out_sb) + row * 64 + 32, lane);
      }
    }
  }
  int ch = -1;
  if (tid < 128) ch = hk * 128 + tid;
  else if (tid < 256) ch = 2048 + hk * 128 + (tid - 128);
  else if (tid < 272) ch = 4096 + hv * 128 + dvb * 16 + (tid - 256);
  // the two gate logits sit on the first lanes of waves 5 and 6, which have nothing else to do here: on wave 4, next
  // to the value channels, the three branches ran one after the other and the decay's chain of exponentials and a
  // logarithm (1 us) held the whole workgroup at the barrier
  else if (tid == BETA_TID) ch = 12288 + hv;  // beta logit
  else if (tid == DECAY_TID) ch = 12320 + hv; // decay logit
  // the decay's constants of this head do not depend on the projection: fetched and exponentiated ahead of the wait
  float decay_rate = 0.0f, dt_bias = 0.0f;
  if (tid == DECAY_TID) { decay_rate = exp_c(uni(Y.a_log)[hv]); dt_bias = uni(Y.dt_bias)[hv]; }
  // history taps and conv weights were parked in LDS while the in-projection ran (flow_request_conv): read after the poll
  uint16_t traw[3] = {0, 0, 0};
  float cw[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  float newest = 0.0f;
  {
    const uint32_t tin = flow_tag(base, li, FS_IN);
    const rsrc_t rp = co_rsrc(uni(F.tproj));
    bool got = ch < 0;
    if (!flow_poll(wave < 7, [&]() {                 // channels sit on threads 0..271 and on the two gate threads
          if (!got) { const uint32_t w = ldw1(rp, ch); got = tag_ok(w, tin); newest = lo_h(w); }
          return got;
        }, uni(P.bar) + 32, 4u)) return false;
    fstamp<ST>(li, FS_CORE, 1, tid == 0);
  }
  if (tid < 272) {
    wr_wait();
    const unsigned char* const lds = reinterpret_cast<const unsigned char*>(g_vt);
    const float4 c4 = *reinterpret_cast<const float4*>(lds + CVW_OFF + wave * 1024 + 16 * lane);
    cw[0] = c4.x; cw[1] = c4.y; cw[2] = c4.z; cw[3] = c4.w;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint32_t hw = *reinterpret_cast<const uint32_t*>(lds + CVH_OFF + (k * 5 + wave) * 256 + 4 * lane);
      traw[k] = (uint16_t)((ch & 1) ? (hw >> 16) : (hw & 0xffffu));
    }
  }
  const float tap[3] = {h2f(traw[0]), h2f(traw[1]), h2f(traw[2])};
  if (tid < 272) {
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 3; ++k) acc = fmaf(tap[k], cw[k], acc);
    acc = fmaf(newest, cw[3], acc);
    const float c = f16r(acc * sigmoid32(acc));
    if (tid < 128) L.q[tid] = c; else if (tid < 256) L.k[tid - 128] = c; else L.v[tid - 256] = c;
  }
  lds_barrier();
  // between the two barriers: waves 0 and 1 norm q and k, and the gate threads form beta and the decay meanwhile
  // (neither is needed before the recurrence)
  if (tid == BETA_TID) L.gb[1] = sigmoid16(newest);
  else if (tid == DECAY_TID) L.gb[0] = exp_c(-(decay_rate * softplus_c(newest + dt_bias)));
  if (wave < 2) {
    float* buf = wave ? L.k : L.q;
    const float x0 = buf[2 * lane], x1 = buf[2 * lane + 1];
    float ss = fmaf(x1, x1, fmaf(x0, x0, 0.0f));
    ss = tree_sum<64>(ss);
    const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
    const float sc = wave ? f16r(0.08838834764831845f) : f16r(0.0078125f);
    const float y0 = f16r(sc * f16r(x0 * inv)), y1 = f16r(sc * f16r(x1 * inv));
    buf[2 * lane] = y0; buf[2 * lane + 1] = y1;
  }
  lds_barrier();
  fstamp<ST>(li, FS_CORE, 2, tid == 0);
  if (wave >= 8) {
    const float g = L.gb[0], beta = L.gb[1];
    const int dvl = (wave - 8) * 2 + half;
    float kk[4], qq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { kk[i] = L.k[4 * l32 + i]; qq[i] = L.q[4 * l32 + i]; }
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) { s[i] = s[i] * g; acc = fmaf(s[i], kk[i], acc); }
    const float kv = tree_sum<32>(acc);
    const float delta = (L.v[dvl] - kv) * beta;
    acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) { s[i] = fmaf(kk[i], delta, s[i]); acc = fmaf(s[i], qq[i], acc); }
    const float y = tree_sum<32>(acc);
    const int dv = dvb * 16 + dvl;
    if (l32 == 0) L.pub[dvl] = tagged(y, flow_tag(base, li, FS_CORE));
    *reinterpret_cast<float4*>(uni(Y.state[par ^ 1]) + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[0], s[1], s[2], s[3]);
  }
  gh.t12 = (uint32_t)traw[1] | ((uint32_t)traw[2] << 16);
  gh.tnew = f2h(newest);
  fstamp<ST>(li, FS_CORE, 3, tid == 8 * 64);
  lds_barrier();
  if (wave == PUB_WAVE && lane < 16) stw1(co_rsrc(uni(F.tycore)), hv * 128 + dvb * 16 + lane, L.pub[lane]);
  fstamp<ST>(li, FS_CORE, 4, tid == PUB_WAVE * 64);
  return true;
}

// ---- attention stage 2: q/k prep, KV append, tile pass ---------------------------------------------------
// A unit is (key tile of 64 positions, kv head); the workgroups take their units in two passes: scores, softmax
// weights (kept in LDS) and the published {max, sum} of every unit first, then the weighted value sums in the same
// order.  With several units per workgroup (contexts beyond about 7000 tokens) the merge knows the global maximum
// after the first pass and adds the tiles up while the second pass runs.
#ifndef SL_MERGE_WGS
#define SL_MERGE_WGS 32
#endif
constexpr int FLOW_MERGE_WGS = SL_MERGE_WGS;     // workgroups that merge the attention tiles: two or four per query head
// Contexts of 13 to 1024 key tiles (from 800 tokens to 64K): every workgroup merges a sixteenth of a query head after
// the tile units (flow_merge_wide), and beyond 32 tiles every workgroup takes tile units as well.  Up to 12 tiles the 32
// merging workgroups get everything in one round trip, from workgroups of their own XCD (0.2 % faster there than the
// wide merge); above 1024 tiles the parked partial sums no longer fit the LDS.
constexpr int WIDE_MERGE_MAX_TILES = 1024;
SL_DEV bool sdpa_wide_merge(int nt) { return nt > 12 && nt <= WIDE_MERGE_MAX_TILES; }
template <bool ST>
SL_DEV bool flow_sdpa(const FlowP& F, const LayerP& Y, int li, int pos, uint32_t base) {
  FLOW_IDS;
  fstamp<ST>(li, FS_CORE, 0, tid == 0);
  const DecodeP& P = F.d;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  const int N = pos + 1, nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  const uint32_t tin = flow_tag(base, li, FS_IN), tcore = flow_tag32(base, li, FS_CORE);
  // The workgroups that merge the tiles take no units: they start polling at once, see every tile's maximum after
  // the first pass below and add up the tiles' value sums while the second pass is still producing them.
  const int GU = (G > 2 * FLOW_MERGE_WGS && !sdpa_wide_merge(nt)) ? G - FLOW_MERGE_WGS : G;
  if (wg >= GU) return true;
  const int U = nt * SL_ATT_KV, RND = uni(F.sdpa_round);
  float* const ps = reinterpret_cast<float*>(g_vt + SDPA_TILE * 256);      // [SDPA_ROUND][8 heads][64 keys]
  float* const sp = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(g_vt) + SPART_OFF);   // [8 heads][8 chains][64 keys]
  uint32_t* const vn = reinterpret_cast<uint32_t*>(L.vnew);                // [kv head][128 words]: the new value row
  // The queries of the kv head's group and the new key and value row are the same for every unit of a workgroup
  // (with an even count of unit workgroups a workgroup stays with one kv head): polled, normed and rotated for its
  // first unit only.
  uint4 w4 = make_uint4(0, 0, 0, 0);
  int prep_kvh = -1;
  const int hp = wave >> 2, kh = (wave >> 1) & 1, dh = wave & 1;        // second pass: pair of heads, half of the keys, of the dims
  float pend_m = 0.0f, pend_l = 0.0f, po[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};     // results waiting to be published
  int pend_slot = -1;
  // A thread stages two 16-byte pieces of a unit's key and value tiles: rows srow and srow + 32.  The tiles travel
  // through registers one unit ahead of their use, so the loads of the next unit are in flight while this one is
  // scored or summed.  (Rows beyond the context repeat its last row and the row of the new position is fetched like
  // any other: neither is stored to LDS, the new row comes from this step's projection instead.)
  const int srow = tid >> 5, c8 = (tid & 31) * 8;
  uint4 kq[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)}, vq[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  auto fetch = [&](bool keys, bool values, int u) {
    const int j0 = (u >> 1) * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
    const size_t off = ((size_t)(u & 1) * uni(P.max_seq) + j0) * 256 + c8;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int row = min(it * 32 + srow, nk - 1);
      if (keys) kq[it] = ld16(uni(Y.kcache) + off + (size_t)row * 256);
      if (values) vq[it] = ld16(uni(Y.vcache) + off + (size_t)row * 256);
    }
  };
  auto put = [&](bool keys, bool values, int u) {
    const int j0 = (u >> 1) * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int row = it * 32 + srow;
      if (row < nk && j0 + row != pos) {
        if (keys) st16(&L.kt[row * KT_STRIDE + c8], kq[it]);
        if (values) st16(&g_vt[row * 256 + c8], vq[it]);
      } else if (row >= nk && values) {
        st16(&g_vt[row * 256 + c8], make_uint4(0, 0, 0, 0));       // weight 0 times value 0 leaves a sum as it is
      }
    }
  };
  if (wg < U) fetch(true, true, wg);
  for (int ub = wg; ub < U; ub += GU * RND) {
    const int nr = min(RND, (U - ub + GU - 1) / GU);       // units of this round
    // pass 1, keys: scores and softmax weights of every unit of the round; maxima and sums published per tile.
    // The value tile of the round's first unit is staged here as well (its space is free during this pass).
    for (int r = 0; r < nr; ++r) {
      const int u = ub + r * GU;
      const int tile = u >> 1, kvh = u & 1;
      const int j0 = tile * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
      const bool has_new = (pos >= j0) && (pos < j0 + SDPA_TILE);
      lds_barrier();                    // the key tile aliases the activation vector the in-projection just read
      // (the tile travelling in registers is parked behind the poll below: parked first, the poll would only start
      // once the tile has arrived)
      // waves 0..7: query heads of the group; wave 8: new key; wave 9: new value -- 4 tagged words per lane
      const int src = wave < 8 ? (kvh * 8 + wave) * 512 : (wave == 8 ? 8192 + kvh * 256 : 8192 + 512 + kvh * 256);
      if (kvh != prep_kvh) {
        prep_kvh = kvh;
        {
          const rsrc_t rp = co_rsrc(uni(F.tproj));
          if (!flow_poll(wave < 10, [&]() {
                w4 = ldw4(rp, src + 4 * lane);
                return tag_ok(w4.x, tin) && tag_ok(w4.y, tin) && tag_ok(w4.z, tin) && tag_ok(w4.w, tin);
              }, uni(P.bar) + 32, 5u)) return false;
          fstamp<ST>(li, FS_CORE, 1, tid == 0);
        }
        if (wave < 9) {
          const bool isq = wave < 8;
          const uint16_t* nwp = isq ? uni(Y.q_norm) : uni(Y.k_norm);
          const float xv[4] = {lo_h(w4.x), lo_h(w4.y), lo_h(w4.z), lo_h(w4.w)};
          float wv[4];
          const uint2 wraw = *reinterpret_cast<const uint2*>(nwp + 4 * lane);
          wv[0] = lo_h(wraw.x); wv[1] = hi_h(wraw.x); wv[2] = lo_h(wraw.y); wv[3] = hi_h(wraw.y);
          const float ss = tree_sum<64>(fmaf(xv[1], xv[1], xv[0] * xv[0]) + fmaf(xv[3], xv[3], xv[2] * xv[2]));
          const float inv = 1.0f / sqrtf(ss / 256.0f + EPS);
          float* dst = isq ? &L.sq[wave * 256] : L.knew;
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[4 * lane + i] = f16r(wv[i] * f16r(xv[i] * inv));
          float o[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = dst[4 * lane + i];
          if (lane < 16) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int d = 4 * lane + i, ii = d & 31;
              const float c = uni(P.rope_cos)[(size_t)pos * 32 + ii], sn = uni(P.rope_sin)[(size_t)pos * 32 + ii];
              const float x0 = dst[ii], x1 = dst[ii + 32];
              o[i] = (d < 32) ? f16r(fmaf(-x1, sn, x0 * c)) : f16r(fmaf(x1, c, x0 * sn));
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[4 * lane + i] = isq ? 0.0625f * o[i] : o[i];
        } else if (wave == 9) {             // the new value row waits in LDS for the second pass
          vn[kvh * 128 + 2 * lane] = (w4.x & 0xffffu) | (w4.y << 16);
          vn[kvh * 128 + 2 * lane + 1] = (w4.z & 0xffffu) | (w4.w << 16);
        }
      }
      put(true, r == 0, u);
      if (has_new && wave == 8) {         // the unit whose tile holds the new position: its key row
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = L.knew[4 * lane + i];
        st_co_h4(co_rsrc(uni(Y.kcache) + ((size_t)kvh * uni(P.max_seq) + pos) * 256), 4 * lane, o);
        *reinterpret_cast<uint2*>(&L.kt[(pos - j0) * KT_STRIDE + 4 * lane]) = make_uint2(pack2(o[0], o[1]), pack2(o[2], o[3]));
      }
      // next in line (requested behind the poll above, which must not wait for it): the keys of the round's next
      // unit, or after the last one the values of its second unit (those of the first are staged already)
      if (r + 1 < nr) fetch(true, false, u + GU);
      else if (nr > 1) fetch(false, true, ub + GU);
      // the previous unit's {max, sum} go out here: a store right before the wait for a tile would make that wait last
      // until the store is acknowledged (loads and stores share one counter and may finish in either order)
      if (pend_slot >= 0 && wave < 8 && lane == 0) stw4(co_rsrc(uni(F.tml)), pend_slot * 4, __float_as_uint(pend_m), __float_as_uint(pend_l), tcore, tcore);
      pend_slot = -1;
      lds_barrier();
      if (ub == wg && r == 0) fstamp<ST>(li, FS_CORE, 2, tid == 0);     // first unit: queries prepared, key tile parked
      {
        // scores: wave (chain ch of 32 dims, four of the eight heads), lane j is key j: a key's 32 dims are read once
        // for four heads; the queries come as LDS broadcasts (one 16-byte read per four multiply-adds)
        const int ch = wave & 7, hg = wave >> 3;
        const uint16_t* kr = &L.kt[(lane < nk ? lane : 0) * KT_STRIDE + 32 * ch];
        uint32_t kw[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint4 t = *reinterpret_cast<const uint4*>(kr + 8 * i);
          kw[4 * i] = t.x; kw[4 * i + 1] = t.y; kw[4 * i + 2] = t.z; kw[4 * i + 3] = t.w;
        }
        float c[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int d4 = 0; d4 < 8; ++d4) {
          const h2_t k01 = as_h2(kw[2 * d4]), k23 = as_h2(kw[2 * d4 + 1]);
#pragma unroll
          for (int hh = 0; hh < 4; ++hh) {
            const float4 q4 = *reinterpret_cast<const float4*>(&L.sq[(4 * hg + hh) * 256 + 32 * ch + 4 * d4]);
            c[hh] = fmaf(q4.x, (float)k01.x, c[hh]);
            c[hh] = fmaf(q4.y, (float)k01.y, c[hh]);
            c[hh] = fmaf(q4.z, (float)k23.x, c[hh]);
            c[hh] = fmaf(q4.w, (float)k23.y, c[hh]);
          }
        }
#pragma unroll
        for (int hh = 0; hh < 4; ++hh) sp[((4 * hg + hh) * 8 + ch) * 64 + lane] = c[hh];
      }
      lds_barrier();
      if (wave < 8) {
        const int h = wave;
        float pr[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) pr[i] = sp[(h * 8 + i) * 64 + lane];
        const float dotv = ((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]));
        const float sc = (lane < nk) ? dotv : NEG;
        const float mx = tree_max<64>(sc);
        const float p = (lane < nk) ? exp_c(sc - mx) : 0.0f;
        const float l = tree_sum<64>(p);
        ps[(r * 8 + h) * 64 + lane] = p;
        pend_m = mx; pend_l = l;
        pend_slot = (kvh * 8 + h) * uni(P.max_tiles) + tile;
      }
    }
    if (pend_slot >= 0 && wave < 8 && lane == 0) stw4(co_rsrc(uni(F.tml)), pend_slot * 4, __float_as_uint(pend_m), __float_as_uint(pend_l), tcore, tcore);
    pend_slot = -1;
    if (ub == wg) fstamp<ST>(li, FS_CORE, 3, tid == 0);                 // first round: scores and softmax weights of its units done
    // pass 2, values: the weighted value sums of the same units, in the same order
    for (int r = 0; r < nr; ++r) {
      const int u = ub + r * GU;
      const int tile = u >> 1, kvh = u & 1;
      const int j0 = tile * SDPA_TILE;
      const bool has_new = (pos >= j0) && (pos < j0 + SDPA_TILE);
      lds_barrier();                    // the previous unit's value tile has been read; the weights are in place
      if (r > 0) {
        put(false, true, u);
        if (r + 1 < nr) fetch(false, true, u + GU);
      }
      if (r + 1 == nr && ub + GU * RND < U) fetch(true, true, ub + GU * RND);   // the next round's first unit
      if (pend_slot >= 0 && kh == 0) {                     // the previous unit's sums (behind the wait for this unit's tile)
#pragma unroll
        for (int e = 0; e < 2; ++e)
          stw4(co_rsrc(uni(F.tpo)), ((pend_slot + e * uni(P.max_tiles)) * 128 + 64 * dh + lane) * 4, __float_as_uint(po[e][0]), __float_as_uint(po[e][1]), tcore, tcore);
      }
      pend_slot = -1;
      if (has_new && wave == 9) {
        const uint32_t a = vn[kvh * 128 + 2 * lane], b = vn[kvh * 128 + 2 * lane + 1];
        stw2(co_rsrc(uni(Y.vcache) + ((size_t)kvh * uni(P.max_seq) + pos) * 256), 2 * lane, a, b);
        *reinterpret_cast<uint2*>(&g_vt[(pos - j0) * 256 + 4 * lane]) = make_uint2(a, b);
      }
      lds_barrier();
      // wave (pair of heads, half of the keys, half of the dims), two dims per lane: a value is read once for two heads.
      // The two chains over the keys, 0..31 and 32..63, run on different waves and meet through LDS; all 64 keys are
      // walked (beyond the context the weight and the staged value are zero).  The weights come as LDS broadcasts,
      // four keys per read.
      float o[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
      const uint16_t* vt = &g_vt[(32 * kh) * 256 + 128 * dh + 2 * lane];
      const float* pw = &ps[(r * 8 + 2 * hp) * 64 + 32 * kh];
#pragma unroll
      for (int j = 0; j < 32; j += 4) {
        uint32_t va[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) va[i] = *reinterpret_cast<const uint32_t*>(vt + (j + i) * 256);
        const float4 pa = *reinterpret_cast<const float4*>(pw + j), pb = *reinterpret_cast<const float4*>(pw + 64 + j);
        const float pav[4] = {pa.x, pa.y, pa.z, pa.w}, pbv[4] = {pb.x, pb.y, pb.z, pb.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const h2_t a01 = as_h2(va[i]);
          o[0][0] = fmaf(pav[i], (float)a01.x, o[0][0]); o[0][1] = fmaf(pav[i], (float)a01.y, o[0][1]);
          o[1][0] = fmaf(pbv[i], (float)a01.x, o[1][0]); o[1][1] = fmaf(pbv[i], (float)a01.y, o[1][1]);
        }
      }
      float4* const xo = reinterpret_cast<float4*>(sp) + (hp * 2 + dh) * 64 + lane;
      if (kh == 1) *xo = make_float4(o[0][0], o[0][1], o[1][0], o[1][1]);
      lds_barrier();
      if (kh == 0) {
        const float4 ob = *xo;
        po[0][0] = o[0][0] + ob.x; po[0][1] = o[0][1] + ob.y; po[1][0] = o[1][0] + ob.z; po[1][1] = o[1][1] + ob.w;
        pend_slot = (kvh * 8 + 2 * hp) * uni(P.max_tiles) + tile;
      }
    }
    if (pend_slot >= 0 && kh == 0) {
#pragma unroll
      for (int e = 0; e < 2; ++e)
        stw4(co_rsrc(uni(F.tpo)), ((pend_slot + e * uni(P.max_tiles)) * 128 + 64 * dh + lane) * 4, __float_as_uint(po[e][0]), __float_as_uint(po[e][1]), tcore, tcore);
    }
    pend_slot = -1;
    lds_barrier();
  }
  fstamp<ST>(li, FS_CORE, 4, tid == 0);
  return true;
}

// The same stage at contexts of up to G/8 key tiles: a unit is (tile, kv head, quarter of the group's 8 query
// heads), so four times as many workgroups share the work and a unit's arithmetic is a quarter.  Wave (head of
// the pair, slice of 32 dims) scores its slice; waves 0..3 = (head, half of the dims) accumulate the values, two dims per
// lane.  The partial sums meet in the order of the undivided stage: 32-dim groups pairwise up to the halves of
// the 256 dims, keys in sequence.  Only quarter 0 writes the new key and value rows to the cache.
template <bool ST>
SL_DEV bool flow_sdpa4(const FlowP& F, const LayerP& Y, int li, int pos, uint32_t base) {
  FLOW_IDS;
  fstamp<ST>(li, FS_CORE, 0, tid == 0);
  const DecodeP& P = F.d;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  const int N = pos + 1, nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  const uint32_t tin = flow_tag(base, li, FS_IN), tcore = flow_tag32(base, li, FS_CORE);
  if (wg >= nt * SL_ATT_KV * 4) return true;
  const int tile = wg >> 3, kvh = (wg >> 2) & 1, hq = wg & 3;
  const int j0 = tile * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
  const bool has_new = (pos >= j0) && (pos < j0 + SDPA_TILE);
  const uint16_t* kbase = uni(Y.kcache) + ((size_t)kvh * uni(P.max_seq) + j0) * 256;
  const uint16_t* vbase = uni(Y.vcache) + ((size_t)kvh * uni(P.max_seq) + j0) * 256;
  // The unit's key and value tile: requested now, parked in LDS once the poll below is over.  (Parked first, the
  // poll would only start when the tile has arrived, and the stage would pay the tile's latency and then the poll's.)
  uint4 kq[2], vq[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int row = min(it * 32 + (tid >> 5), nk - 1), c8 = (tid & 31) * 8;       // (rows beyond the context repeat its last row: not stored)
    kq[it] = ld16(kbase + (size_t)row * 256 + c8);
    vq[it] = ld16(vbase + (size_t)row * 256 + c8);
  }
  // waves 0,1: the unit's two query heads; wave 8: new key; wave 9: new value -- 4 tagged words per lane
  const bool fetches = wave < 2 || wave == 8 || wave == 9;
  const int src = wave < 2 ? (kvh * 8 + hq * 2 + wave) * 512 : (wave == 8 ? 8192 + kvh * 256 : 8192 + 512 + kvh * 256);
  uint4 w4 = make_uint4(0, 0, 0, 0);
  // norm weights and the rope row of this position do not depend on the projection: fetched ahead of the poll
  uint2 wraw = make_uint2(0, 0);
  float rc[4] = {1.0f, 1.0f, 1.0f, 1.0f}, rsn[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (wave < 2 || wave == 8) {
    wraw = *reinterpret_cast<const uint2*>((wave < 2 ? uni(Y.q_norm) : uni(Y.k_norm)) + 4 * lane);
    if (lane < 16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ii = (4 * lane + i) & 31;
        rc[i] = uni(P.rope_cos)[(size_t)pos * 32 + ii]; rsn[i] = uni(P.rope_sin)[(size_t)pos * 32 + ii];
      }
    }
  }
  {
    const rsrc_t rp = co_rsrc(uni(F.tproj));
    if (!flow_poll(fetches, [&]() {
          w4 = ldw4(rp, src + 4 * lane);
          return tag_ok(w4.x, tin) && tag_ok(w4.y, tin) && tag_ok(w4.z, tin) && tag_ok(w4.w, tin);
        }, uni(P.bar) + 32, 6u)) return false;
    fstamp<ST>(li, FS_CORE, 1, tid == 0);
  }
  // (the poll's barrier is behind us: the key tile aliases the activation vector the in-projection read)
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int row = it * 32 + (tid >> 5), c8 = (tid & 31) * 8;
    if (row < nk && j0 + row != pos) {
      st16(&L.kt[row * KT_STRIDE + c8], kq[it]);
      st16(&g_vt[row * 256 + c8], vq[it]);
    } else if (row >= nk) {
      st16(&g_vt[row * 256 + c8], make_uint4(0, 0, 0, 0));         // weight 0 times value 0 leaves a sum as it is
    }
  }
  if (wave < 2 || wave == 8) {
    const bool isq = wave < 2;
    const float xv[4] = {lo_h(w4.x), lo_h(w4.y), lo_h(w4.z), lo_h(w4.w)};
    float wv[4];
    wv[0] = lo_h(wraw.x); wv[1] = hi_h(wraw.x); wv[2] = lo_h(wraw.y); wv[3] = hi_h(wraw.y);
    const float ss = tree_sum<64>(fmaf(xv[1], xv[1], xv[0] * xv[0]) + fmaf(xv[3], xv[3], xv[2] * xv[2]));
    const float inv = 1.0f / sqrtf(ss / 256.0f + EPS);
    float* dst = isq ? &L.sq[wave * 256] : L.knew;
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[4 * lane + i] = f16r(wv[i] * f16r(xv[i] * inv));
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = dst[4 * lane + i];
    if (lane < 16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 4 * lane + i, ii = d & 31;
        const float c = rc[i], sn = rsn[i];
        const float x0 = dst[ii], x1 = dst[ii + 32];
        o[i] = (d < 32) ? f16r(fmaf(-x1, sn, x0 * c)) : f16r(fmaf(x1, c, x0 * sn));
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[4 * lane + i] = isq ? 0.0625f * o[i] : o[i];
    if (!isq && has_new) {
      if (hq == 0) st_co_h4(co_rsrc(uni(Y.kcache) + ((size_t)kvh * uni(P.max_seq) + pos) * 256), 4 * lane, o);
      *reinterpret_cast<uint2*>(&L.kt[(pos - j0) * KT_STRIDE + 4 * lane]) = make_uint2(pack2(o[0], o[1]), pack2(o[2], o[3]));
    }
  } else if (wave == 9 && has_new) {
    const uint32_t a = (w4.x & 0xffffu) | (w4.y << 16), b = (w4.z & 0xffffu) | (w4.w << 16);
    if (hq == 0) stw2(co_rsrc(uni(Y.vcache) + ((size_t)kvh * uni(P.max_seq) + pos) * 256), 2 * lane, a, b);
    *reinterpret_cast<uint2*>(&g_vt[(pos - j0) * 256 + 4 * lane]) = make_uint2(a, b);
  }
  lds_barrier();
  {
    // scores: wave (head, slice) takes one of the eight chains of 32 dims, lane j is key j; the queries come as LDS
    // broadcasts
    const int hh = wave >> 3, sl = wave & 7;
    const uint16_t* kr = &L.kt[(lane < nk ? lane : 0) * KT_STRIDE + 32 * sl];
    const float* qs = &L.sq[hh * 256 + 32 * sl];
    float ch = 0.0f;
#pragma unroll
    for (int l = 0; l < 8; ++l) {
      const uint2 kraw = *reinterpret_cast<const uint2*>(kr + 4 * l);
      const h2_t k01 = as_h2(kraw.x), k23 = as_h2(kraw.y);
      const float4 q4 = *reinterpret_cast<const float4*>(qs + 4 * l);
      ch = fmaf(q4.x, (float)k01.x, ch);
      ch = fmaf(q4.y, (float)k01.y, ch);
      ch = fmaf(q4.z, (float)k23.x, ch);
      ch = fmaf(q4.w, (float)k23.y, ch);
    }
    L.part[wave * 64 + lane] = ch;
  }
  lds_barrier();
  if ((wave & 7) == 0) {
    const int hh = wave >> 3;
    const float* pp = &L.part[hh * 512 + lane];
    const float lo = (pp[0] + pp[64]) + (pp[128] + pp[192]), hi = (pp[256] + pp[320]) + (pp[384] + pp[448]);
    const float sc = (lane < nk) ? lo + hi : NEG;
    const float mx = tree_max<64>(sc);
    const float p = (lane < nk) ? exp_c(sc - mx) : 0.0f;
    const float l = tree_sum<64>(p);
    L.sm[hh * 64 + lane] = p;
    const int head = kvh * 8 + hq * 2 + hh;
    if (lane == 0) stw4(co_rsrc(uni(F.tml)), (head * uni(P.max_tiles) + tile) * 4, __float_as_uint(mx), __float_as_uint(l), tcore, tcore);
  }
  lds_barrier();
  if (wave < 4) {
    // values: wave (head, half of the dims), two dims per lane (one LDS word per key); two chains over the keys,
    // 0..31 and 32..63, added at the end; all 64 keys are walked (beyond the context the weight and the staged value are
    // zero).  The weights come as LDS broadcasts, four keys per read.
    const int hh = wave >> 1, half = wave & 1;
    float oa0 = 0.0f, oa1 = 0.0f, ob0 = 0.0f, ob1 = 0.0f;
    const uint16_t* vt = &g_vt[128 * half + 2 * lane];
    const float* pw = &L.sm[hh * 64];
#pragma unroll
    for (int j = 0; j < 32; j += 4) {
      uint32_t va[4], vb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        va[i] = *reinterpret_cast<const uint32_t*>(vt + (j + i) * 256);
        vb[i] = *reinterpret_cast<const uint32_t*>(vt + (32 + j + i) * 256);
      }
      const float4 pa = *reinterpret_cast<const float4*>(pw + j), pb = *reinterpret_cast<const float4*>(pw + 32 + j);
      const float pav[4] = {pa.x, pa.y, pa.z, pa.w}, pbv[4] = {pb.x, pb.y, pb.z, pb.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const h2_t a01 = as_h2(va[i]), b01 = as_h2(vb[i]);
        oa0 = fmaf(pav[i], (float)a01.x, oa0); oa1 = fmaf(pav[i], (float)a01.y, oa1);
        ob0 = fmaf(pbv[i], (float)b01.x, ob0); ob1 = fmaf(pbv[i], (float)b01.y, ob1);
      }
    }
    const float o0 = oa0 + ob0, o1 = oa1 + ob1;
    const int head = kvh * 8 + hq * 2 + hh;
    stw4(co_rsrc(uni(F.tpo)), ((head * uni(P.max_tiles) + tile) * 128 + 64 * half + lane) * 4, __float_as_uint(o0), __float_as_uint(o1),
         tcore, tcore);
  }
  fstamp<ST>(li, FS_CORE, 4, tid == 0);
  lds_barrier();
  return true;
}

// History shift of a linear-attention layer: rows 1,2 of the old history and the new sample (each channel is
// written by one workgroup).
SL_DEV void store_hist(const LayerP& Y, int li, const GdnHist& gh) {
  const int tid = fresh_v(threadIdx.x), wg = fresh_s(blockIdx.x);
  if (tid < 272) {
    const int hv = gdn_unit_head(wg), dvb = gdn_unit_dvb(wg), hk = hv >> 1;
    const int ch = tid < 128 ? hk * 128 + tid : (tid < 256 ? 2048 + hk * 128 + (tid - 128) : 4096 + hv * 128 + dvb * 16 + (tid - 256));
    if (tid >= 256 || ((hv & 1) == 0 && dvb == 0)) {
      uint16_t* hout = uni(Y.hist[(int)(((uni(g_K.parity) >> li) & 1ull) ^ 1ull)]);
      hout[ch] = (uint16_t)(gh.t12 & 0xffffu);
      hout[SL_CONV_DIM + ch] = (uint16_t)(gh.t12 >> 16);
      hout[2 * SL_CONV_DIM + ch] = (uint16_t)gh.tnew;
    }
  }
}

// ---- attention merge on all workgroups ------------------------------------------------------------------------
// Workgroup n merges dims 16 (n % 16) .. + 15 of query head n / 16: eight 16-byte chunks per key tile.  What bounds a
// merge on few workgroups is how fast those can pull the published chunks (16 MB per layer at 32K tokens through 32
// compute units); spread over the whole grid every thread fetches at most eight chunks, all in one round trip, parks
// them in LDS, and the sums are formed from LDS.  The order is the canonical one: per block of 64 tiles a chain from
// zero in tile order (one lane per (block, dim); the tiles' sums likewise, one lane per block), the blocks' chains
// added in block order.
template <bool ST>
SL_DEV bool flow_merge_wide(const FlowP& F, const LayerP& Y, int li, int nt, uint32_t base) {
  FLOW_IDS;
  const DecodeP& P = F.d;
  const float NEG = -__int_as_float(0x7f800000);
  const uint32_t tin = flow_tag(base, li, FS_IN), tmerge = flow_tag(base, li, FS_MERGE), tcore32 = flow_tag32(base, li, FS_CORE);
  const int h = wg >> 4, c0 = 8 * (wg & 15), slot0 = h * uni(P.max_tiles);
  const rsrc_t rml = co_rsrc(uni(F.tml)), rpo = co_rsrc(uni(F.tpo)), rp = co_rsrc(uni(F.tproj));
  unsigned char* const dyn = reinterpret_cast<unsigned char*>(g_vt);
  float* const ll = reinterpret_cast<float*>(dyn);                       // [1024] tile sums
  float* const fl = reinterpret_cast<float*>(dyn + 4096);                // [1024] tile scales exp(max - global max)
  uint2* const park = reinterpret_cast<uint2*>(dyn + 12288);             // [tile][8 chunks] {o0, o1}
  static_assert(12288 + WIDE_MERGE_MAX_TILES * 8 * 8 <= DEC_DYN_LDS && WIDE_MERGE_MAX_TILES <= DEC_THREADS, "parked sums fit; a thread per tile");
  lds_barrier();                                                         // the tile units are through with the dynamic LDS
  // One round trip for everything: every tile's {max, sum} (thread t: tile t), the slice's output gate (lanes 0..15 of
  // wave 0) and the partial sums -- item i = tid + 1024 j is chunk i % 8 of tile i / 8.  All requests of an attempt
  // first, then the looks at them; what has arrived is parked and not asked for again.
  float m = NEG;
  {
    const bool mine = tid < nt, gmine = tid < 16;
    bool mdone = !mine, gdone = !gmine;
    const int items = 8 * nt;
    uint4 v[8];
    unsigned have = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) if (tid + DEC_THREADS * j >= items) have |= 1u << j;
    if (!flow_poll(true, [&]() {
          const bool want_m = !mdone, want_g = !gdone;
          const unsigned missing = ~have;
          uint4 q = make_uint4(0u, 0u, 0u, 0u);
          uint32_t g = 0;
          if (want_m) q = ldw4(rml, (slot0 + tid) * 4);
          if (want_g) g = ldw1(rp, h * 512 + 256 + 2 * c0 + tid);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int i = tid + DEC_THREADS * j;
            if (missing & (1u << j)) v[j] = ldw4(rpo, ((slot0 + (i >> 3)) * 128 + c0 + (i & 7)) * 4);
          }
          if (want_m && q.z == tcore32 && q.w == tcore32) { mdone = true; m = __uint_as_float(q.x); ll[tid] = __uint_as_float(q.y); }
          if (want_g && tag_ok(g, tin)) { gdone = true; g_L.red[32 + tid] = sigmoid16(lo_h(g)); }
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if ((missing & (1u << j)) && v[j].z == tcore32 && v[j].w == tcore32) {
              have |= 1u << j;
              park[tid + DEC_THREADS * j] = make_uint2(v[j].x, v[j].y);
            }
          return mdone && gdone && (have & 0xffu) == 0xffu;
        }, uni(P.bar) + 32, 25u)) return false;
    const float wm = tree_max<64>(m);
    if (lane == 0) g_L.red[wave] = wm;
  }
  lds_barrier();
  fstamp<ST>(li, FS_MERGE, 1, tid == 0);
  // (tiles up to the next multiple of 16 count as tiles of scale 0 and sums 0, so the chains below walk whole batches
  // without a test per tile: a multiply-add of zeros leaves a sum as it is)
  const int nt16 = (nt + 15) & ~15;
  {
    const float Mx = tree_max<64>(g_L.red[lane & 15]);
    if (tid < nt) fl[tid] = exp_c(m - Mx);
    else if (tid < nt16) { fl[tid] = 0.0f; ll[tid] = 0.0f; }
    for (int i = 8 * nt + tid; i < 8 * nt16; i += DEC_THREADS) park[i] = make_uint2(0u, 0u);
  }
  lds_barrier();
  fstamp<ST>(li, FS_MERGE, 2, tid == 0);
  const int nb = (nt + 63) / 64;                               // at most 16
  float* const blk = g_L.part;                                 // [block][8 chunks][2], then [block] sums at 256
  // One lane per (block, one of the 16 dims): a single wave issues an instruction every eight clocks or so, so what a
  // chain costs is its instruction count -- sixteen tiles per batch, their values and scales read with constant
  // offsets ahead of the sixteen multiply-adds.
  if (tid < 16 * nb) {
    const int b = tid >> 4, c2 = tid & 15;
    const int t1 = min(64 * b + 64, nt16);
    const float* const parkf = reinterpret_cast<const float*>(park);
    float B = 0.0f;
    for (int t0 = 64 * b; t0 < t1; t0 += 16) {
      const float* const pp = parkf + t0 * 16 + c2;
      const float4* const fp = reinterpret_cast<const float4*>(fl + t0);
      float pv[16];
      float4 f4[4];
#pragma unroll
      for (int i = 0; i < 16; ++i) pv[i] = pp[16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) f4[j] = fp[j];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        B = fmaf(pv[4 * j], f4[j].x, B); B = fmaf(pv[4 * j + 1], f4[j].y, B);
        B = fmaf(pv[4 * j + 2], f4[j].z, B); B = fmaf(pv[4 * j + 3], f4[j].w, B);
      }
    }
    blk[tid] = B;
  } else if (wave == 4 && lane < nb) {
    const int t1 = min(64 * lane + 64, nt16);
    float Lb = 0.0f;
    for (int t0 = 64 * lane; t0 < t1; t0 += 16) {
      const float4* const lp = reinterpret_cast<const float4*>(ll + t0);
      const float4* const fp = reinterpret_cast<const float4*>(fl + t0);
      float4 l4[4], f4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) { l4[j] = lp[j]; f4[j] = fp[j]; }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Lb = fmaf(l4[j].x, f4[j].x, Lb); Lb = fmaf(l4[j].y, f4[j].y, Lb);
        Lb = fmaf(l4[j].z, f4[j].z, Lb); Lb = fmaf(l4[j].w, f4[j].w, Lb);
      }
    }
    blk[256 + lane] = Lb;
  }
  lds_barrier();
  fstamp<ST>(li, FS_MERGE, 3, tid == 0);
  if (wave == PUB_WAVE && lane < 8) {
    float O0 = blk[2 * lane], O1 = blk[2 * lane + 1], Ls = blk[256];
    for (int b = 1; b < nb; ++b) { O0 = O0 + blk[2 * (8 * b + lane)]; O1 = O1 + blk[2 * (8 * b + lane) + 1]; Ls = Ls + blk[256 + b]; }
    const uint32_t r0 = tagged(f16r(f16r(O0 / Ls) * g_L.red[32 + 2 * lane]), tmerge);
    const uint32_t r1 = tagged(f16r(f16r(O1 / Ls) * g_L.red[32 + 2 * lane + 1]), tmerge);
    stw2(co_rsrc(uni(F.tycore)), h * 256 + 2 * (c0 + lane), r0, r1);
  }
  fstamp<ST>(li, FS_MERGE, 4, tid == PUB_WAVE * 64);
  (void)Y;
  return true;
}

// ---- K = 4096 projection (GDN out_proj with gated rmsnorm prologue / attention merge + o_proj) ---------
template <bool ST>
SL_DEV bool flow_out(const FlowP& F, const LayerP& Y, int li, int nt, uint32_t base, const GdnHist& gh) {
  FLOW_IDS;
  fstamp<ST>(li, FS_OUT, 0, tid == 0);
  const DecodeP& P = F.d;
  const bool lin = uni(Y.is_linear) != 0;
  const float NEG = -__int_as_float(0x7f800000);
  WRegs<2, 1> wr;
  const bool valid = gw < H;
  if (lin) {           // the row was requested into LDS when the in-projection ended; its scales and biases come now
    wr.w[0][0] = wr.w[0][1] = make_uint4(0, 0, 0, 0);
    wr.sb[0][0] = wr.sb[0][1] = 0u;
  } else
  wload_row<2>(wr.w[0], wr.sb[0], uni(Y.out_w), uni(Y.out_sb), (size_t)(valid ? gw : 0), valid, lane);
  const uint32_t tin = flow_tag(base, li, FS_IN), tcore = flow_tag(base, li, FS_CORE), tmerge = flow_tag(base, li, FS_MERGE);
  const uint32_t tcore32 = flow_tag32(base, li, FS_CORE);
  if (!lin && sdpa_wide_merge(nt)) {
    if (!flow_merge_wide<ST>(F, Y, li, nt, base)) return false;
  } else if (!lin && wg >= G - FLOW_MERGE_WGS) {
    // Merge the attention tiles in order with the global max: the last 32 workgroups take half a head each (they own
    // no tile units, so their waves have no stores of their own to wait for and poll from the start of the
    // stage).  Wave 0 is the merging wave: a lane owns one 16-byte chunk (2 dims) of its 128 dims.
    // First round trip: {max, sum} of the first 64 tiles (lane i fetches tile i), the partials of the first MB tiles
    // and the output gate (it sits in the q projection of this step) are polled together, each piece until it has
    // arrived; at contexts of up to MB tiles that is everything the merge needs.  (From there to 1024 tiles every
    // workgroup merges a slice, flow_merge_wide; beyond, the waves of these workgroups share the blocks of 64 tiles,
    // below.)  The accumulation always runs in tile order.
    constexpr int MPH = FLOW_MERGE_WGS / SL_ATT_HEADS, LPW = 128 / MPH;      // workgroups per head, chunks (lanes) per workgroup
    // Workgroup n runs on XCD n % 8, and at short contexts the tile units of heads 2x, 2x+1 run on XCD x (flow_sdpa4:
    // workgroup % 8 = kv head * 4 + head pair): the workgroups that merge those two heads are taken from the same XCD,
    // so the partial sums change hands through that XCD's L2 (1.1 against 1.5 us for a small exchange).
    static_assert(FLOW_MERGE_WGS % 8 == 0 && FLOW_MERGE_WGS / 8 == 2 * MPH, "two heads per XCD");
    const int mi = wg - (G - FLOW_MERGE_WGS);
    const int xcd = mi & 7, kx = mi >> 3;                 // (G - FLOW_MERGE_WGS is a multiple of 8 on the full machine)
    const int h = 2 * xcd + kx / MPH, slot0 = h * uni(P.max_tiles);
    const bool act = lane < LPW;
    const int chunk = LPW * (kx % MPH) + (act ? lane : 0);      // (idle lanes of a narrower workgroup fetch and store nothing)
    const rsrc_t rml = co_rsrc(uni(F.tml)), rpo = co_rsrc(uni(F.tpo)), rp = co_rsrc(uni(F.tproj));
    int fail = 0;
    float Mx = NEG, Ls = 0.0f, O0 = 0.0f, O1 = 0.0f;
    uint4 m0 = make_uint4(0, 0, 0, 0);
    uint2 g2 = make_uint2(0u, 0u);
    // {max, sum} of every tile, kept in LDS once they have been seen (the key tile's space: merging workgroups stage none)
    uint2* const mls = reinterpret_cast<uint2*>(g_L.kt);
    constexpr int MB = 12;                                  // tiles of the first round trip
    if (nt > MB) {                                          // the hand-over words of the long merge (below), before any wave uses them
      if (tid < 128) reinterpret_cast<volatile uint32_t*>(reinterpret_cast<unsigned char*>(g_vt) + (DEC_WAVES - 2) * 8 * 64 * 8)[tid] = 0u;
      lds_barrier();
    }
    float sg0 = 0.0f, sg1 = 0.0f;                          // sigmoids of the lane's two gate values
    if (wave == 0) {
      uint4 a[MB];
      // maxima of the tiles beyond the first 64, eight blocks per round trip: they are published after the first pass
      // over the keys, well before the first partial sums, so this wait is over when those arrive
      for (int t0 = 64; t0 < nt && !fail; t0 += 512) {
        float pm[8];
        unsigned have = 0, spins = 0;
        for (;;) {
          SL_FRESH_LOOK();
          uint4 mq[8];
          const unsigned missing = ~have;
#pragma unroll
          for (int j = 0; j < 8; ++j) {                    // all requests of an attempt first, then the looks at them
            const int t = t0 + 64 * j + lane;
            mq[j] = make_uint4(0u, 0u, tcore32, tcore32);
            if ((missing & (1u << j)) && t < nt) mq[j] = ldw4(rml, (slot0 + t) * 4);
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            if (!(missing & (1u << j))) continue;
            const int t = t0 + 64 * j + lane;
            pm[j] = t < nt ? __uint_as_float(mq[j].x) : NEG;
            if (__all((mq[j].z == tcore32 && mq[j].w == tcore32) ? 1 : 0)) {
              have |= 1u << j;
              if (t < nt) mls[t] = make_uint2(mq[j].x, mq[j].y);      // kept for the blocks' additions below
            }
          }
          if (have == 0xffu) break;
          if (++spins > uni(F.spin_limit)) { fail = 17; break; }
        }
        if (!fail) {
#pragma unroll
          for (int j = 0; j < 8; ++j) Mx = fmaxf(Mx, tree_max<64>(pm[j]));
        }
      }
      {
        const bool mine = lane < nt;
        const int cnt0 = min(MB, nt);
        bool mdone = false, gdone = false;
        unsigned have = 0, spins = 0;
        for (;;) {
          SL_FRESH_LOOK();
          // every piece still missing is requested first and looked at afterwards: with a look behind each request the
          // round trips of an attempt would follow one another (up to fourteen of them)
          const bool want_m = !mdone, want_g = !gdone;
          const unsigned missing = ~have;
          if (want_m && mine) m0 = ldw4(rml, (slot0 + lane) * 4);
          if (want_g && act) g2 = ldw2(rp, h * 512 + 256 + 2 * chunk);
#pragma unroll
          for (int u = 0; u < MB; ++u)
            if (u < cnt0 && (missing & (1u << u)) && act) a[u] = ldw4(rpo, ((slot0 + u) * 128 + chunk) * 4);
          if (want_m) mdone = __all((!mine || (m0.z == tcore32 && m0.w == tcore32)) ? 1 : 0) != 0;
          if (want_g) {
            gdone = __all((!act || (tag_ok(g2.x, tin) && tag_ok(g2.y, tin))) ? 1 : 0) != 0;
            // the gate was published a stage earlier: its sigmoids are formed while the tiles are still on their way
            if (gdone) { sg0 = sigmoid16(lo_h(g2.x)); sg1 = sigmoid16(lo_h(g2.y)); }
          }
#pragma unroll
          for (int u = 0; u < MB; ++u)
            if (u < cnt0 && (missing & (1u << u)) && __all((!act || (a[u].z == tcore32 && a[u].w == tcore32)) ? 1 : 0)) have |= 1u << u;
          if (mdone && gdone && have == (1u << cnt0) - 1u) break;
          if (++spins > uni(F.spin_limit)) { fail = 18; break; }
        }
        Mx = fmaxf(Mx, tree_max<64>(mine ? __uint_as_float(m0.x) : NEG));
        if (mine) mls[lane] = make_uint2(m0.x, m0.y);
        fstamp<ST>(li, FS_MERGE, 1, lane == 0);
      }
      if (!fail) {                                          // the first batch is already here
        float fl = 0.0f, pl = 0.0f;
        if (lane < nt) { fl = exp_c(__uint_as_float(m0.x) - Mx); pl = __uint_as_float(m0.y); }
        // the tiles' scales and sums as scalars, read out in batches ahead of their use (a scalar written by the
        // vector unit takes tens of clocks to become readable)
        static_assert(MB <= 16, "two batches of eight lane reads");
        float f[16], l[16];
        lanes8(fl, 0, reinterpret_cast<float(&)[8]>(f[0])); lanes8(fl, 8, reinterpret_cast<float(&)[8]>(f[8]));
        lanes8(pl, 0, reinterpret_cast<float(&)[8]>(l[0])); lanes8(pl, 8, reinterpret_cast<float(&)[8]>(l[8]));
#pragma unroll
        for (int u = 0; u < MB; ++u) {
          if (u < nt) {
            Ls = fmaf(l[u], f[u], Ls);
            O0 = fmaf(__uint_as_float(a[u].x), f[u], O0); O1 = fmaf(__uint_as_float(a[u].y), f[u], O1);
          }
        }
        fstamp<ST>(li, FS_MERGE, 3, lane == 0);
      }
    }
    const int nb = (nt + 63) / 64;                          // blocks of 64 tiles: a chain each, the chains added in block order
    if (nt > MB) {
      // (More than 1024 tiles -- up to there every workgroup merges, flow_merge_wide.)  The blocks' chains run side by side.  Wave 2 + w takes blocks w, w + 14, ...: it polls
      // sixteen tiles at a time (one 16-byte chunk per lane and tile; the tile index sits in the load's scalar offset,
      // so sixteen requests in flight cost no address registers) -- from the start of the stage, while the maxima are
      // still on their way -- and, once wave 0 has left the global maximum, adds them up in tile order (block 0 goes
      // on from wave 0's chain over the first tiles) and leaves the block's chain in LDS.  Wave 1 carries the chains
      // of the tiles' sums, which need no partial sums.  After one barrier wave 0 adds the blocks' chains in block
      // order.  The waves meet through LDS words only; every wait is bounded, and a wave that gives up raises the
      // abort word, which ends the others' waits.  (What bounds this stage is the rate at which 32 workgroups pull
      // 16 MB of published chunks past their caches, about 1 TB/s at 32K tokens: a block's quarters dealt out to four
      // waves with the chain handed on through LDS only added polls, 46.9 against 41.0 us.)
      uint2* const blk_o = reinterpret_cast<uint2*>(g_vt);                        // [block][64 lanes] {o0, o1}
      constexpr int RW_OFF = (DEC_WAVES - 2) * 8 * 64 * 8, MAX_BLOCKS = (SDPA_TILE * KT_STRIDE * 2 / 8 + 63) / 64;
      static_assert(MAX_BLOCKS * 512 <= RW_OFF && MAX_BLOCKS + 2 <= 128, "a chain and a word per block of the longest context");
      volatile uint32_t* const rw = reinterpret_cast<volatile uint32_t*>(reinterpret_cast<unsigned char*>(g_vt) + RW_OFF);
      // rw[0]: wave 0 has left the maximum, its sum and its chains; rw[1]: abort.
      // (Cleared at the top of the stage.)
      const unsigned limit = uni(F.spin_limit);
      if (wave == 0) {
        if (lane == 0) { g_L.red[0] = Mx; g_L.red[1] = Ls; }
        blk_o[lane] = make_uint2(__float_as_uint(O0), __float_as_uint(O1));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) rw[0] = 1u;
      } else if (wave == 1) {
        unsigned spins = 0;
        while (rw[0] == 0u) {
          if (++spins > limit || rw[1] != 0u) { fail = 20; break; }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (!fail) {
          Mx = g_L.red[0];
          float Lb = g_L.red[1], La = 0.0f;               // the block's chain (block 0: from wave 0's), the blocks before
          for (int b = 0; b < nb; ++b) {
            const int t0 = 64 * b;
            const uint2 cur = mls[min(t0 + lane, nt - 1)];
            float fl = 0.0f, pl = 0.0f;
            if (t0 + lane < nt) { fl = exp_c(__uint_as_float(cur.x) - Mx); pl = __uint_as_float(cur.y); }
            const int lo = b == 0 ? MB : 0, hi = min(64, nt - t0);
            for (int u0 = lo & ~7; u0 < hi; u0 += 8) {
              float f[8], l[8];
              lanes8(fl, u0, f);
              lanes8(pl, u0, l);
#pragma unroll
              for (int i = 0; i < 8; ++i) if (u0 + i >= lo && u0 + i < hi) Lb = fmaf(l[i], f[i], Lb);
            }
            La = b == 0 ? Lb : La + Lb;
            Lb = 0.0f;
          }
          if (lane == 0) g_L.red[2] = La;
        } else if (lane == 0) rw[1] = 1u;
      } else {
        constexpr int WB = 16;                            // tiles per round trip (a multiple of 8)
        unsigned spins = 0;
        bool have_max = false;
        for (int b = wave - 2; b < nb && !fail; b += DEC_WAVES - 2) {
          const int tlo = b == 0 ? MB : 64 * b, thi = min(64 * b + 64, nt);
          float B0 = 0.0f, B1 = 0.0f, fl = 0.0f;
          for (int tb = tlo; tb < thi && !fail; tb += WB) {
            uint4 v[WB];
            auto request = [&]() {
#pragma unroll
              for (int j = 0; j < WB; ++j) v[j] = ldw4s(rpo, chunk * 4, (slot0 + min(tb + j, nt - 1)) * 512);
            };
            request();
            for (;;) {
              bool ok = true;
#pragma unroll
              for (int j = 0; j < WB; ++j) ok = ok && (tb + j >= thi || !act || (v[j].z == tcore32 && v[j].w == tcore32));
              if (__all(ok ? 1 : 0)) break;
              if (++spins > limit || rw[1] != 0u) { fail = 21; break; }
              SL_FRESH_LOOK();
              request();
            }
            if (fail) break;
            if (!have_max) {
              while (rw[0] == 0u) {
                if (++spins > limit || rw[1] != 0u) { fail = 22; break; }
              }
              if (fail) break;
              __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
              Mx = g_L.red[0];
              have_max = true;
            }
            if (tb == tlo) {                               // lane i: the scale of tile i of the block
              const int t = 64 * b + lane;
              fl = t < nt ? exp_c(__uint_as_float(mls[min(t, nt - 1)].x) - Mx) : 0.0f;
              if (b == 0) { const uint2 c0 = blk_o[lane]; B0 = __uint_as_float(c0.x); B1 = __uint_as_float(c0.y); }
            }
            float f[WB];
#pragma unroll
            for (int k = 0; k < WB; k += 8) lanes8(fl, tb - 64 * b + k, reinterpret_cast<float(&)[8]>(f[k]));   // (lanes beyond 63 belong to tiles beyond the block: unused)
            if (tb + WB <= thi) {
#pragma unroll
              for (int i = 0; i < WB; ++i) { B0 = fmaf(__uint_as_float(v[i].x), f[i], B0); B1 = fmaf(__uint_as_float(v[i].y), f[i], B1); }
            } else {
#pragma unroll
              for (int i = 0; i < WB; ++i) {
                if (tb + i < thi) { B0 = fmaf(__uint_as_float(v[i].x), f[i], B0); B1 = fmaf(__uint_as_float(v[i].y), f[i], B1); }
              }
            }
          }
          if (!fail) blk_o[b * 64 + lane] = make_uint2(__float_as_uint(B0), __float_as_uint(B1));
        }
        if (fail && lane == 0) rw[1] = 1u;
      }
      lds_barrier();
      if (rw[1] != 0u) fail = 24;
      if (wave == 0 && !fail) {
        Ls = g_L.red[2];
        const uint2 c0 = blk_o[lane];
        O0 = __uint_as_float(c0.x); O1 = __uint_as_float(c0.y);
        for (int b = 1; b < nb; ++b) {
          const uint2 c = blk_o[b * 64 + lane];
          O0 = O0 + __uint_as_float(c.x); O1 = O1 + __uint_as_float(c.y);
        }
      }
    }
    if (fail && ld_co32(uni(P.bar) + 32) == 0u) st_co32(uni(P.bar) + 32, (uint32_t)fail);
    if (wave == 0 && !fail && act) {
      const uint32_t r0 = tagged(f16r(f16r(O0 / Ls) * sg0), tmerge);
      const uint32_t r1 = tagged(f16r(f16r(O1 / Ls) * sg1), tmerge);
      stw2(co_rsrc(uni(F.tycore)), h * 256 + 2 * chunk, r0, r1);
    }
    fstamp<ST>(li, FS_MERGE, 4, tid == 0);
  }
  if (wg * DEC_WAVES >= H) {                       // no output row here (uniform per workgroup): nothing to fetch
    if (lin) store_hist(Y, li, gh);
    return true;
  }
  // every thread prepares 4 consecutive elements of the 4096-long activation and polls them itself
  const int e0 = 256 * wave + 4 * lane;
  float out[4], sz[4] = {0.0f, 0.0f, 0.0f, 0.0f};            // sz: z * sigmoid(z) of the gate values
  // the gated norm's weights do not depend on the hand-over: requested ahead of the poll, which outlasts them
  float4 wraw = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (lin) wraw = *reinterpret_cast<const float4*>(uni(Y.gdn_norm_w) + (e0 & 127));
  {
    const uint32_t ty = lin ? tcore : tmerge;
    const rsrc_t ry = co_rsrc(uni(F.tycore)), rz = co_rsrc(uni(F.tproj));
    uint4 a = make_uint4(0, 0, 0, 0);
    bool zdone = false, ydone = false;                    // what has arrived is not fetched again
    if (!flow_poll(true, [&]() {
          // (both requests first, then the looks at them: one round trip per attempt)
          const bool want_y = !ydone, want_z = lin && !zdone;
          uint4 b = make_uint4(0, 0, 0, 0);
          if (want_y) a = ldw4(ry, e0);
          if (want_z) b = ldw4(rz, 8192 + e0);
          if (want_y) ydone = tag_ok(a.x, ty) && tag_ok(a.y, ty) && tag_ok(a.z, ty) && tag_ok(a.w, ty);
          bool ok = ydone;
          if (want_z) {                             // the gate values were published a stage earlier: fetched once
            zdone = tag_ok(b.x, tin) && tag_ok(b.y, tin) && tag_ok(b.z, tin) && tag_ok(b.w, tin);
            ok = ok && zdone;
            if (zdone) {
              // z * sigmoid(z) does not need the core output: formed while that is still on its way
              const float z1[4] = {lo_h(b.x), lo_h(b.y), lo_h(b.z), lo_h(b.w)};
#pragma unroll
              for (int i = 0; i < 4; ++i) sz[i] = z1[i] * sigmoid32(z1[i]);
            }
          }
          return ok;
        }, uni(P.bar) + 32, 7u)) return false;
    fstamp<ST>(li, FS_OUT, 1, tid == 0);
    if (lin) store_hist(Y, li, gh);
    out[0] = lo_h(a.x); out[1] = lo_h(a.y); out[2] = lo_h(a.z); out[3] = lo_h(a.w);
  }
  if (lin) {
    const float nw[4] = {wraw.x, wraw.y, wraw.z, wraw.w};
    const bool nf32 = uni(Y.gdn_norm_f32) != 0;
    const float la = fmaf(out[1], out[1], fmaf(out[0], out[0], 0.0f));
    const float lb = fmaf(out[3], out[3], fmaf(out[2], out[2], 0.0f));
    const float ss = tree_sum<32>(la + lb);
    const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float nrm = nf32 ? nw[i] * (out[i] * inv) : f16r(nw[i] * f16r(out[i] * inv));
      out[i] = f16r(sz[i] * nrm);
    }
  }
  {
    const int b = e0 >> 11, r = e0 & 2047, lo = r >> 5, i0 = r & 31;
    g_L.xs[(16 * b + (i0 >> 1)) * 64 + lo] = pack2(out[0], out[1]);
    g_L.xs[(16 * b + (i0 >> 1) + 1) * 64 + lo] = pack2(out[2], out[3]);
    // a share of 32 elements sits on eight neighbouring lanes: balanced tree over its 16 pair sums
    const float ssum = tree_sum<8>((out[0] + out[1]) + (out[2] + out[3]));
    if ((lane & 7) == 0) g_L.sxs[64 * b + lo] = ssum;
  }
  if (lin) wr_wait();          // the rows this wave requested for the workgroup have landed (the barrier hands them on)
  lds_barrier();
  fstamp<ST>(li, FS_OUT, 2, tid == 0);
  if (lin) {
    wr.w[0][0] = wr_read(wave * 3, lane); wr.w[0][1] = wr_read(wave * 3 + 1, lane);
    wr.sb[0][0] = sbr_read(wave * 3, lane); wr.sb[0][1] = sbr_read(wave * 3 + 1, lane);
  }
  const float o = dot_2x1(wr);
  fstamp<ST>(li, FS_OUT, 3, tid == 0);
  if (wg * DEC_WAVES < H) {                       // uniform per workgroup
    if (lane == 0) g_L.pub[wave] = tagged(o, flow_tag(base, li, FS_OUT));
    lds_barrier();
    if (wave == PUB_WAVE && lane < 16) stw1(co_rsrc(uni(F.tmix)), wg * DEC_WAVES + lane, g_L.pub[lane]);
    fstamp<ST>(li, FS_OUT, 4, tid == PUB_WAVE * 64);
  }
  return true;
}

// ---- MoE stage A -------------------------------------------------------------------------------------
// GATE8: the router and shared-gate rows are 8-bit affine rows instead of fp16 (a compile-time variant, so that
// the fp16 configuration carries none of its registers or branches).
template <bool GATE8, bool ST, bool PLAIN = false>
SL_DEV bool flow_moe_a(const FlowP& F, const LayerP& Y, int li, uint32_t base, float& h0, float& h1) {
  FLOW_IDS;
  fstamp<ST>(li, FS_A, 0, tid == 0);
  const DecodeP& P = F.d;
  // The router rows, the shared-gate row and the shared gate/up pairs sit on workgroups of the upper half
  // of the grid: those have no row of the K = 4096 projection, reach this stage early and so have their
  // rows in registers long before the hand-over arrives (the router logits are what stage B waits for).
  const int gd = gw - DENSE_WAVE0, gp = gw - PAIR_WAVE0;
  const bool is_dense = gd >= 0 && gd <= uni(P.E);
  const bool is_pair = gp >= 0 && gp < 512;
  uint4 dwr[4] = {};                      // dense fp16 row, kept packed until the wait is over
  WRegs<1, 2> wr;
  const size_t prow = is_pair ? (size_t)gp : 0;
  wload_row<1>(wr.w[0], wr.sb[0], uni(Y.shg_w), uni(Y.shg_sb), prow, is_pair, lane);
  wload_row<1>(wr.w[1], wr.sb[1], uni(Y.shu_w), uni(Y.shu_sb), prow, is_pair, lane);
  constexpr bool gate8 = GATE8;
  uint32_t dsb = 0;                       // 8-bit gates: {scale, bias} of this lane's half group
  if (is_dense && !gate8) {
    const uint16_t* drow = (gd < uni(P.E) ? uni(Y.router_w) + (size_t)gd * H : uni(Y.sgate_w)) + 32 * lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) dwr[j] = ld16(drow + 8 * j);
  } else if (is_dense) {
    const uint32_t* drow = reinterpret_cast<const uint32_t*>(uni(Y.router_w)) + (size_t)gd * 512 + 8 * lane;
    dwr[0] = ld16(drow); dwr[1] = ld16(drow + 4);
    dsb = reinterpret_cast<const uint32_t*>(uni(Y.sgate_w))[(size_t)gd * 32 + (lane >> 1)];
  }
  const uint32_t lnw = *reinterpret_cast<const uint32_t*>(uni(Y.post_ln) + 2 * tid);
  const uint32_t ta = flow_tag(base, li, FS_A);
  if constexpr (PLAIN) {
    (void)lnw;
    flow_plain_x(uni(F.xin));
  } else {
    float r0, r1;
    if (!poll_vec2048<ST>(P, uni(F.tmix), flow_tag(base, li, FS_OUT), r0, r1, li, FS_A)) return false;
    flow_prologue(h0, h1, true, r0, r1, lnw, nullptr);
  }
  fstamp<ST>(li, FS_A, 2, tid == 0);
  if (is_dense) {
    uint32_t xp[16]; float sx;
    lds_get_x(0, lane, xp, sx);
    const uint32_t dww[16] = {dwr[0].x, dwr[0].y, dwr[0].z, dwr[0].w, dwr[1].x, dwr[1].y, dwr[1].z, dwr[1].w,
                              dwr[2].x, dwr[2].y, dwr[2].z, dwr[2].w, dwr[3].x, dwr[3].y, dwr[3].z, dwr[3].w};
    float acc = 0.0f;
    if (!gate8) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {               // (half operands straight into the mixed-precision multiply-add)
        const h2_t xv = as_h2(xp[i]), wv = as_h2(dww[i]);
        acc = fmaf((float)xv.x, (float)wv.x, acc);
        acc = fmaf((float)xv.y, (float)wv.y, acc);
      }
    } else {
      float xf[32];
#pragma unroll
      for (int i = 0; i < 16; ++i) { xf[2 * i] = lo_h(xp[i]); xf[2 * i + 1] = hi_h(xp[i]); }
      acc = q8_lane(dww, dsb, xf);
    }
    acc = tree_sum<64>(acc);
    if (lane == 0) g_L.pub[wave] = tagged(acc, ta);
  }
  if (is_pair) {
    const F2 gu = dot_1x2(wr);
    if (lane == 0) g_L.pub[wave] = tagged(swiglu16(f16r(gu.v[0]), f16r(gu.v[1])), ta);
  }
  {
    const int d0 = wg * DEC_WAVES - DENSE_WAVE0, p0 = wg * DEC_WAVES - PAIR_WAVE0, E = uni(P.E);
    if ((d0 >= 0 && d0 <= E) || (p0 >= 0 && p0 < 512)) {     // uniform per workgroup: it holds router rows, the gate row or pairs
      lds_barrier();
      if (wave == PUB_WAVE && lane < 16) {
        if (d0 >= 0 && d0 <= E) {
          const int g = d0 + lane;
          if (g < E) stw1(co_rsrc(uni(F.trlog)), g, g_L.pub[lane]);
          else if (g == E) stw1(co_rsrc(uni(F.tsg)), 0, g_L.pub[lane]);
        } else {
          stw1(co_rsrc(uni(F.tsh)), p0 + lane, g_L.pub[lane]);
        }
      }
      fstamp<ST>(li, FS_A, 4, tid == PUB_WAVE * 64);
    }
  }
  return true;
}

// ---- MoE stage B: routing + routed gate/up + SwiGLU -------------------------------------------------------
// Order key of a router logit: larger logit first, lower expert index first on ties (+0 and -0 tie).
SL_DEV uint32_t route_key(uint32_t hbits, int e) {
  uint32_t u = hbits & 0xffffu;
  if ((u & 0x7fffu) == 0) u = 0;
  u = (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
  return (u << 8) | (uint32_t)(255 - e);
}
// Rounds [r0, r1) of the top-8 selection on one wave: k holds the lane's keys not yet chosen, in falling order.
SL_DEV void route_rounds(uint32_t (&k)[4], int r0, int r1, int E, int lane) {
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    if (r < r0 || r >= r1) continue;                      // (uniform)
    // (the wave-wide maximum stays in vector registers: a value read out to a scalar register takes tens of clocks
    // to become usable, eight times in a row)
    const uint32_t M = wave_max_u32(k[0]);
    const bool won = k[0] == M;
    k[0] = won ? k[1] : k[0]; k[1] = won ? k[2] : k[1]; k[2] = won ? k[3] : k[2]; k[3] = won ? 0u : k[3];
    if (lane == 0) g_L.inds[r] = min(255 - (int)(M & 255u), E - 1);
  }
}
template <bool ST>
SL_DEV bool flow_moe_b(const FlowP& F, const LayerP& Y, int li, uint32_t base) {
  FLOW_IDS;
  fstamp<ST>(li, FS_B, 0, tid == 0);
  const DecodeP& P = F.d;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  float* ex = L.part + 256;                             // [256] exp(logit - max)
  // A workgroup's routed gate/up rows belong to one of the eight chosen experts (slot = workgroup / 32): wave 0 runs the
  // max-and-remove rounds only up to that slot, the workgroup meets and requests its rows, and wave 0 finds the
  // remaining indices (needed from the next stage on) while the rows are on their way.
  const int myslot = (wg >> 5) & 7;
  uint32_t rk[4] = {0u, 0u, 0u, 0u};
  // Waves 0 and 1 each poll all the logits (four per lane, 1 KB) and go straight on: wave 0 picks the 8 largest keys
  // in order (max, remove, repeat), wave 1 forms the softmax sums.  The workgroup meets once, when the indices are
  // known (a hop of the logits through LDS and a barrier ahead of the routing measured 0.1 % slower).
  if (wave < 2) {
    const uint32_t ta = flow_tag(base, li, FS_A);
    const rsrc_t rl = co_rsrc(uni(F.trlog));
    const int E = uni(P.E);
    uint4 w4 = make_uint4(0u, 0u, 0u, 0u);
    const bool mine = 4 * lane < E;                        // (words of experts beyond E are ignored)
    flow_poll<false>(true, [&]() {
      if (mine) w4 = ldw4(rl, 4 * lane);
      const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
      bool ok = true;
#pragma unroll
      for (int i = 0; i < 4; ++i) ok = ok && (4 * lane + i >= E || tag_ok(w[i], ta));
      return ok;
    }, uni(P.bar) + 32, 8u);
    fstamp<ST>(li, FS_B, 1, tid == 0);
    const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
    if (wave == 0) {
      uint32_t k[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) k[i] = 4 * lane + i < E ? route_key(w[i], 4 * lane + i) : 0u;
      // a lane's four keys in falling order first (keys are distinct: the index rides in the low byte), so that a round
      // is the wave-wide maximum of the lanes' first keys and a shift of the winner's list
      auto order = [](uint32_t& a, uint32_t& b) { const uint32_t hi = max(a, b), lo = min(a, b); a = hi; b = lo; };
      order(k[0], k[1]); order(k[2], k[3]); order(k[0], k[2]); order(k[1], k[3]); order(k[1], k[2]);
      rk[0] = k[0]; rk[1] = k[1]; rk[2] = k[2]; rk[3] = k[3];
      route_rounds(rk, 0, myslot + 1, E, lane);
    } else {
      float v[4], x4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = 4 * lane + i < E ? lo_h(w[i]) : NEG;
      const float mx = tree_max<64>(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
#pragma unroll
      for (int i = 0; i < 4; ++i) { x4[i] = (4 * lane + i < E) ? exp_c(v[i] - mx) : 0.0f; ex[4 * lane + i] = x4[i]; }
      const float Z = tree_sum<64>(((x4[0] + x4[1]) + x4[2]) + x4[3]);
      if (lane == 0) L.gb[0] = Z;
    }
  }
  lds_barrier();
  if (g_L.pf[3] != 0) return false;
  fstamp<ST>(li, FS_B, 2, tid == 0);
  // (the renormalised scores are only needed by the combine of the next stage and are formed there, off this
  // stage's path: exp values, sum and indices stay in LDS)
  // this wave's gate/up pair, requested as soon as the indices are known
  const int p = gw;
  WRegs<1, 2> wr;
  int k = 0, i = 0;
  const bool active = p < 8 * 512;
  if (active) {
    k = p >> 9; i = p & 511;
    const size_t row = (size_t)L.inds[k] * 512 + i;
    wload_row<1>(wr.w[0], wr.sb[0], uni(Y.swg_w), uni(Y.swg_sb), row, true, lane);
    wload_row<1>(wr.w[1], wr.sb[1], uni(Y.swu_w), uni(Y.swu_sb), row, true, lane);
  }
  if (wave == 0) route_rounds(rk, myslot + 1, 8, uni(P.E), lane);
  if (active) {
    const F2 gu = dot_1x2(wr);
    fstamp<ST>(li, FS_B, 3, tid == 0);
    if (lane == 0) L.pub[wave] = tagged(swiglu16(f16r(gu.v[0]), f16r(gu.v[1])), flow_tag(base, li, FS_B));
  }
  lds_barrier();
  if (wave == PUB_WAVE && lane < 16 && wg * DEC_WAVES + lane < 8 * 512) stw1(co_rsrc(uni(F.tact)), wg * DEC_WAVES + lane, L.pub[lane]);
  fstamp<ST>(li, FS_B, 4, tid == PUB_WAVE * 64);
  return true;
}

// ---- MoE stage C: down-projections, half combine, gated shared add ---------------------------------------
// Units (quad of 4 outputs, slot): slots 0..7 routed experts, slot 8 shared; 2 quads per workgroup.  The nine
// activation rows are fetched once per workgroup into LDS (packed pairs, 20-word stride per 32 elements, the
// share's sum in word 16 of its slot).
constexpr int XC_STRIDE = 20;
template <bool ST>
SL_DEV bool flow_moe_c(const FlowP& F, const LayerP& Y, int li, uint32_t base) {
  FLOW_IDS;
  fstamp<ST>(li, FS_C, 0, tid == 0);
  const DecodeP& P = F.d;
  Lds& L = g_L;
  uint32_t* xc = reinterpret_cast<uint32_t*>(g_vt);      // [9][16][XC_STRIDE]
  const int sub = lane >> 4, li16 = lane & 15;
  const uint32_t ta = flow_tag(base, li, FS_A), tb = flow_tag(base, li, FS_B);
  // Waves 6..14 own the 18 units (two each) and fetch their down-projection rows now; every wave polls a share of the
  // activation rows (one chunk per thread: with six polling waves of three chunks the step measured 0.5 % slower,
  // although the unit waves' polls return behind their weight rows); wave 15 combines and publishes.
  const bool unit_wave = wave >= 6 && wave < 15;
  uint4 wv[2]; uint32_t sbv[2];
#pragma unroll
  for (int qq = 0; qq < 2; ++qq) {
    const int un = (wave - 6) * 2 + qq, ql = un / 9, slot = un % 9;
    wv[qq] = make_uint4(0, 0, 0, 0); sbv[qq] = 0;
    if (unit_wave) {
      const size_t row = (slot < 8 ? (size_t)L.inds[slot] * 2048 : 0) + (size_t)(wg * 2 + ql) * 4 + sub;
      const uint32_t* W = slot < 8 ? uni(Y.swd_w) : uni(Y.shd_w);
      const uint32_t* SB = slot < 8 ? uni(Y.swd_sb) : uni(Y.shd_sb);
      wv[qq] = ld16(W + row * 64 + 4 * li16);
      sbv[qq] = SB[row * 8 + (li16 >> 1)];
    }
  }
  if (tid == PUB_WAVE * 64) {
    // scores of the routing done in the stage before: gates = half(exp / Z) of the selected, renormalised in half
    // (the publisher wave neither polls nor owns a unit, so this costs the stage nothing)
    const float* ex = L.part + 256;
    float sc[8], ss = 0.0f;
    const float Z = L.gb[0];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) { sc[kk] = f16r(ex[L.inds[kk]] / Z); ss = f16r(ss + sc[kk]); }
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) L.scores[kk] = f16r(sc[kk] / ss);
    if (wg == 0) for (int kk = 0; kk < 8; ++kk) { uni(Y.route_inds)[kk] = L.inds[kk]; uni(Y.route_scores)[kk] = f2h(L.scores[kk]); }
  }
  {
    // the nine activation rows (8 x 512 routed + 512 shared) are 1152 chunks of 4 tagged words: one per thread, two on
    // the first 128
    const rsrc_t ra = co_rsrc(uni(F.tact)), rs = co_rsrc(uni(F.tsh)), rg = co_rsrc(uni(F.tsg));
    bool have[2] = {false, tid >= 128};           // a chunk that has arrived is not fetched again
    float psum[2] = {0.0f, 0.0f};                 // sum of the chunk's two pair sums
    flow_poll<false>(true, [&]() {
      bool ok = true;
      // (the requests of an attempt first, then the looks at them: one round trip per attempt)
      const bool want[2] = {!have[0], !have[1]};
      uint4 q4[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
      uint32_t gw1 = 0;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int t = tid + 1024 * c, slot = t >> 7;
        if (want[c]) q4[c] = (slot < 8) ? ldw4(ra, 4 * t) : ldw4(rs, 4 * (t & 127));
      }
      if (tid == 0) gw1 = ldw1(rg, 0);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        if (!want[c]) continue;
        // chunk t holds elements 4(t%128).. of slot t/128 (slot 8 = shared): packed pairs 2(t%128), 2(t%128)+1
        const int t = tid + 1024 * c, slot = t >> 7, pi = 2 * (t & 127);
        const uint4 a4 = q4[c];
        const uint32_t tx = (slot < 8) ? tb : ta;
        have[c] = tag_ok(a4.x, tx) && tag_ok(a4.y, tx) && tag_ok(a4.z, tx) && tag_ok(a4.w, tx);
        ok = ok && have[c];
        psum[c] = (lo_h(a4.x) + lo_h(a4.y)) + (lo_h(a4.z) + lo_h(a4.w));
        *reinterpret_cast<uint2*>(&xc[(slot * 16 + (pi >> 4)) * XC_STRIDE + (pi & 15)]) =
            make_uint2((a4.x & 0xffffu) | (a4.y << 16), (a4.z & 0xffffu) | (a4.w << 16));
      }
      if (tid == 0) { ok = ok && tag_ok(gw1, ta); L.gb[1] = lo_h(gw1); }
      return ok;
    }, uni(P.bar) + 32, 9u);
    // a share of 32 activations = the chunks of eight neighbouring threads: its sum (the balanced tree over the 16 pair
    // sums) goes into the padding word behind the share's packed pairs
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (c == 1 && wave >= 2) break;               // second chunks sit on threads 0..127 (wave-uniform)
      const int t = tid + 1024 * c;
      const float ssum = tree_sum<8>(psum[c]);
      if ((tid & 7) == 0) xc[((t >> 7) * 16 + ((t & 127) >> 3)) * XC_STRIDE + 16] = __float_as_uint(ssum);
    }
    lds_barrier();
    if (g_L.pf[3] != 0) return false;
    fstamp<ST>(li, FS_C, 1, tid == 0);
  }
  // the shared expert's gate came with the poll: its sigmoid is formed by the publishing wave while the units run
  float sgs = 0.0f;
  if (wave == PUB_WAVE) sgs = sigmoid16(L.gb[1]);
#pragma unroll
  for (int qq = 0; qq < 2; ++qq) {
    const int un = (wave - 6) * 2 + qq, ql = un / 9, slot = un % 9;
    if (unit_wave) {
      uint32_t xp[16];
      const uint4* src = reinterpret_cast<const uint4*>(&xc[(slot * 16 + li16) * XC_STRIDE]);
#pragma unroll
      for (int j = 0; j < 4; ++j) { const uint4 q = src[j]; xp[4 * j] = q.x; xp[4 * j + 1] = q.y; xp[4 * j + 2] = q.z; xp[4 * j + 3] = q.w; }
      const float d = tree_sum<16>(share_term(wv[qq], sbv[qq], xp, __uint_as_float(xc[(slot * 16 + li16) * XC_STRIDE + 16])));
      if (li16 == 0) L.dbuf[(ql * 9 + slot) * 4 + sub] = f16r(d);
    }
  }
  fstamp<ST>(li, FS_C, 3, tid == 6 * 64);
  lds_barrier();
  if (wave == PUB_WAVE && lane < 8) {
    const int ql = lane >> 2, sb4 = lane & 3;
    const int quad = wg * 2 + ql;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) acc = f16r(acc + f16r(L.dbuf[(ql * 9 + k) * 4 + sb4] * L.scores[k]));
    stw1(co_rsrc(uni(F.tmoe)), quad * 4 + sb4, tagged(f16r(acc + f16r(sgs * L.dbuf[(ql * 9 + 8) * 4 + sb4])), flow_tag(base, li, FS_C)));
  }
  fstamp<ST>(li, FS_C, 4, tid == PUB_WAVE * 64);
  lds_barrier();
  return true;
}

// ---- head -------------------------------------------------------------------------------------------
template <bool ST>
SL_DEV bool flow_head(const FlowP& F, int pos, int out_off, int feed, uint32_t base, float h0, float h1, bool hand_on) {
  FLOW_IDS;
  const DecodeP& P = F.d;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  const int nl = uni(P.n_layers);
  float bv = NEG; int bi = 0x7fffffff;
  // The vocabulary in groups of four rows, dealt out evenly: wave gw takes groups gw, gw + NW, ... and the groups left
  // over go one each to waves 0, 1, ... of every workgroup in turn, so that the four waves of a SIMD (which share its
  // issue slot: the stage ends when the last of them is through) differ by at most one group anywhere on the chip.
  // A wave meets its groups in rising order, so its first maximum is the one of the lowest index.
  const int NG = (uni(P.vocab) + 3) / 4, per = NG / NW, ex = wave * G + wg;
  const int mine = per + (ex < NG - per * NW ? 1 : 0);
  auto group_of = [&](int k) { return k < per ? gw + k * NW : per * NW + ex; };
  WRegs<1, 4> cur, nxt;
  auto load_group = [&](WRegs<1, 4>& r, int k) {
    const long g = group_of(k);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long row = g * 4 + j;
      const bool v = k < mine && row < uni(P.vocab);
      wload_row<1>(r.w[j], r.sb[j], uni(P.lm_w), uni(P.lm_sb), (size_t)(v ? row : 0), v, lane);
    }
  };
  load_group(cur, 0);
  const uint32_t lnw = *reinterpret_cast<const uint32_t*>(uni(P.final_norm) + 2 * tid);
  float r0, r1;
  fstamp<ST>(nl, 0, 0, tid == 0);
  if (!poll_vec2048<ST>(P, uni(F.tmoe), flow_tag(base, nl - 1, FS_C), r0, r1, nl, 0)) return false;
  const uint32_t thd32 = flow_tag32(base, nl, 0);
  flow_prologue(h0, h1, true, r0, r1, lnw, wg == 0 ? uni(P.normed) : nullptr);
  // the activation row stays in registers for all groups; the two weight sets swap roles from group to group (a copy
  // would cost twenty moves per group in a stage that is bound by its instruction count)
  uint32_t x[16]; float sx;
  lds_get_x(0, lane, x, sx);
  // The four row sums of a group are reduced together.  After the first two levels of the reduction tree (lane
  // pairs, then quads) the four lanes of a quad hold the same value, so one register can carry all four rows, lane l
  // the row rho(l) = l % 4 in the lower quad of every eight lanes and 3 - l % 4 in the upper one: the partners of the
  // remaining levels (mirror within 8, mirror within 16, the other row of 16, the other half) then hold the same row,
  // and every addition has the operands it has in tree_sum.  A lane follows the maximum of its own row class; the
  // four classes meet when the stage ends (lowest index on ties, as everywhere).
  const int rho = (lane & 4) ? 3 - (lane & 3) : (lane & 3);
  auto group_step = [&](const WRegs<1, 4>& a, WRegs<1, 4>& b, int k) {
    load_group(b, k + 1);
    float q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = tree_sum<4>(share_term(a.w[j][0], a.sb[j][0], x, sx));
    float f = rho == 0 ? q[0] : (rho == 1 ? q[1] : (rho == 2 ? q[2] : q[3]));
    f = f + dpp_f<DPP_HALF_MIRROR>(f);
    f = f + dpp_f<DPP_MIRROR>(f);
    f = swap32_sum(swap16_sum(f));
    const long row = (long)group_of(k) * 4 + rho;
    if (row < uni(P.vocab)) {
      const float v = f16r(f);
      if (v > bv) { bv = v; bi = (int)row; }
      if (lane < 4) uni(P.logits)[row] = f2h(f);
    }
  };
#pragma unroll 1
  for (int k = 0; k < mine; k += 2) {
    group_step(cur, nxt, k);
    if (k + 1 < mine) group_step(nxt, cur, k + 1);
  }
  fstamp<ST>(nl, 0, 3, tid == 0);
#pragma unroll
  for (int msk = 1; msk < 4; msk <<= 1) {               // lanes 0..3: the four row classes
    const float ov = __shfl_xor(bv, msk, 64); const int oi = __shfl_xor(bi, msk, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (lane == 0) { L.red[wave] = bv; L.ired[wave] = bi; }
  lds_barrier();
  if (wave == PUB_WAVE && lane == 0) {
    bv = L.red[0]; bi = L.ired[0];
    for (int w = 1; w < DEC_WAVES; ++w)
      if (L.red[w] > bv || (L.red[w] == bv && L.ired[w] < bi)) { bv = L.red[w]; bi = L.ired[w]; }
    stw4(co_rsrc(uni(F.tcand)), wg * 4, __float_as_uint(bv), (uint32_t)bi, thd32, thd32);
  }
  if (wg != 0) return true;
  float v = NEG; int i = 0x7fffffff;
  {
    const rsrc_t rc = co_rsrc(uni(F.tcand));
    unsigned spins = 0;
    for (;;) {
      bool ok = true;
      if (tid < G) { const uint4 c = ldw4(rc, tid * 4); ok = c.z == thd32 && c.w == thd32; v = __uint_as_float(c.x); i = (int)c.y; }
      const int r = flow_round(ok, spins, uni(P.bar) + 32, 10u);
      if (r > 0) break;
      if (r < 0) return false;
    }
    fstamp<ST>(nl, 1, 1, tid == 0);
  }
#pragma unroll
  for (int msk = 1; msk < 64; msk <<= 1) {
    const float ov = __shfl_xor(v, msk, 64); const int oi = __shfl_xor(i, msk, 64);
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
  }
  lds_barrier();
  if (lane == 0) { L.red[wave] = v; L.ired[wave] = i; }
  lds_barrier();
  if (tid == 0) {
    for (int w = 1; w < DEC_WAVES; ++w)
      if (L.red[w] > v || (L.red[w] == v && L.ired[w] < i)) { v = L.red[w]; i = L.ired[w]; }
    uni(P.tok_out)[out_off] = i;
    if (feed) uni(P.tok_in)[0] = i;
    uni(P.st)[0] = pos + 1;
    const uint32_t nbase = base + (uint32_t)(nl + 1) * 8u;
    st_co32(uni(P.bar) + 16, nbase);
    if (hand_on) { const uint32_t ttag = flow_tag32(nbase, 0, 7); stw4(co_rsrc(uni(F.ttok)), 0, (uint32_t)i, (uint32_t)i, ttag, ttag); }
    fstamp<ST>(nl, 1, 4, true);
  }
  for (int l = tid; l < nl; l += DEC_THREADS) uni(P.st)[1 + l] ^= 1;
  return true;
}

// ---- the kernel: hA already holds the embedded token row (k_embed) --------------------------------------
// `steps` tokens per launch (a chain feeds each token back on the device): between two steps workgroup 0 hands the
// new token to everybody as a tagged word, which costs one hand-over instead of a kernel boundary.
template <bool GATE8, bool ST>
__global__ __launch_bounds__(DEC_THREADS) void k_decode_flow(const FlowP* __restrict__ Fp, int out_off, int feed, int steps) {
  {
    const int tid = threadIdx.x;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(Fp);
    uint32_t* dst = reinterpret_cast<uint32_t*>(&g_K.F);
    for (int i = tid; i < (int)(sizeof(FlowP) / 4); i += DEC_THREADS) dst[i] = src[i];
    const int nl = Fp->d.n_layers;
    const uint32_t* lsrc = reinterpret_cast<const uint32_t*>(Fp->d.layers);
    uint32_t* ldst = reinterpret_cast<uint32_t*>(g_K.layers);
    for (int i = tid; i < nl * (int)(sizeof(LayerP) / 4); i += DEC_THREADS) ldst[i] = lsrc[i];
    if (tid < 64) {
      const int bit = (tid < nl) ? (Fp->d.st[1 + tid] & 1) : 0;
      const unsigned long long m = __ballot(bit);
      const unsigned long long lm = __ballot((tid < nl) ? (Fp->d.layers[tid].is_linear != 0) : 0);
      if (tid == 0) { g_K.parity = m; g_K.linmask = lm; g_K.pos = Fp->d.st[0]; g_K.base = ld_co32(Fp->d.bar + 16); g_K.tok = 0; }
      if (tid < 4) g_L.pf[tid] = 0;
    }
    if constexpr (ST) for (int i = tid; i < STAMP_WORDS; i += DEC_THREADS) g_stamps[i] = 0;
    __syncthreads();
  }
  const FlowP& F = g_K.F;
  const DecodeP& P = F.d;
  const int nl = uni(P.n_layers);
  // A workgroup that leaves (a wait gave up, or the launch is over) first lets its outstanding loads land: rows on
  // their way into LDS must not arrive after the LDS has passed to another workgroup.
#define FLOW_TRY(call) do { if (!(call)) goto flow_exit; } while (0)
  flow_request_in(g_K.layers[0]);
  for (int step = 0; step < steps; ++step) {
    const uint32_t base = uni(g_K.base);
    const int pos = uni(g_K.pos);
    float h0 = 0.0f, h1 = 0.0f;          // this thread's two elements of the residual stream
    for (int li = 0; li < nl; ++li) {
      const LayerP& Y = g_K.layers[li];
      const int is_linear = uni(Y.is_linear);
      FLOW_TRY(flow_in<ST>(F, Y, li, pos, base, h0, h1, step));
      GdnHist gh = {0u, 0u};
      if (is_linear) {
        FLOW_TRY(flow_gdn<ST>(F, Y, li, base, gh));
        FLOW_TRY(flow_out<ST>(F, Y, li, 0, base, gh));
      } else {
        if (((pos + SDPA_TILE) / SDPA_TILE) * SL_ATT_KV * 4 <= (int)gridDim.x) FLOW_TRY(flow_sdpa4<ST>(F, Y, li, pos, base));
        else FLOW_TRY(flow_sdpa<ST>(F, Y, li, pos, base));
        FLOW_TRY(flow_out<ST>(F, Y, li, (pos + SDPA_TILE) / SDPA_TILE, base, gh));
      }
      // through with the K = 4096 projection (the upper half of the grid has no rows there and is here at once): the
      // in-projection rows of the next layer, or of the next step's first layer, set out for LDS
      const LayerP* const Ynext = li + 1 < nl ? &g_K.layers[li + 1] : (step + 1 < steps ? &g_K.layers[0] : nullptr);
      if (Ynext) flow_request_in(*Ynext);
      FLOW_TRY((flow_moe_a<GATE8, ST>(F, Y, li, base, h0, h1)));
      FLOW_TRY(flow_moe_b<ST>(F, Y, li, base));
      FLOW_TRY(flow_moe_c<ST>(F, Y, li, base));
    }
    FLOW_TRY(flow_head<ST>(F, pos, out_off + step, feed, base, h0, h1, step + 1 < steps));
    if (step + 1 < steps) {
      lds_barrier();                     // everybody has read this step's position, tag base and parities
      if (threadIdx.x == 0) { g_K.pos = pos + 1; g_K.base = base + (uint32_t)(nl + 1) * 8u; g_K.parity ^= g_K.linmask; }
      lds_barrier();
    }
  }
#undef FLOW_TRY
flow_exit:
  wr_wait();
  if constexpr (ST) {                                  // (also after a wait that gave up: the stamps show where every workgroup stood)
    __syncthreads();
    uint32_t* dst = uni(P.tstamp) + (size_t)blockIdx.x * STAMP_WORDS;
    for (int i = threadIdx.x; i < STAMP_WORDS; i += DEC_THREADS) dst[i] = g_stamps[i];
  }
}

// ---- a single block in one launch ---------------------------------------------------------------------------------
// One layer's mixer (mode 0: in-projection, recurrence or attention, out-projection) or its MoE block (mode 1: router,
// shared and routed experts, combine) on the row F.xin, taken as it is (no residual, no norm): the stages of the step
// kernel, handed over the same way, so the arithmetic is that of a decode step.  The result stays in its exchange
// buffer (tmix / tmoe: halves with the tags of this launch), from where the host takes it; position, parities and caches
// are read as they stand and the host moves them on.
template <bool GATE8>
__global__ __launch_bounds__(DEC_THREADS) void k_block_flow(const FlowP* __restrict__ Fp, const LayerP* __restrict__ layers,
                                                            const int32_t* __restrict__ st, const unsigned* bar, int nl, int li, int mode) {
  {
    // (the layer's parameters, the position and the tag counter come through pointers passed as arguments, so their
    // loads leave together with those of the parameter block instead of after it; only layer li is copied)
    const int tid = threadIdx.x;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(Fp);
    uint32_t* dst = reinterpret_cast<uint32_t*>(&g_K.F);
    for (int i = tid; i < (int)(sizeof(FlowP) / 4); i += DEC_THREADS) dst[i] = src[i];
    const uint32_t* lsrc = reinterpret_cast<const uint32_t*>(layers + li);
    uint32_t* ldst = reinterpret_cast<uint32_t*>(g_K.layers + li);
    for (int i = tid; i < (int)(sizeof(LayerP) / 4); i += DEC_THREADS) ldst[i] = lsrc[i];
    if (tid < 64) {
      const int bit = (tid < nl) ? (st[1 + tid] & 1) : 0;
      const unsigned long long m = __ballot(bit);
      if (tid == 0) { g_K.parity = m; g_K.linmask = 0ull; g_K.pos = st[0]; g_K.base = ld_co32(bar + 16); g_K.tok = 0; }
      if (tid < 4) g_L.pf[tid] = 0;
    }
    __syncthreads();
  }
  const FlowP& F = g_K.F;
  const DecodeP& P = F.d;
  const LayerP& Y = g_K.layers[li];
  const uint32_t base = uni(g_K.base);
  const int pos = uni(g_K.pos);
  float h0 = 0.0f, h1 = 0.0f;
  bool ok = true;
  if (mode == 0) {
    flow_request_in(Y);
    ok = flow_in<false, true>(F, Y, li, pos, base, h0, h1, 0);
    GdnHist gh = {0u, 0u};
    if (ok) {
      if (uni(Y.is_linear)) {
        ok = flow_gdn<false>(F, Y, li, base, gh);
        if (ok) ok = flow_out<false>(F, Y, li, 0, base, gh);
      } else {
        if (((pos + SDPA_TILE) / SDPA_TILE) * SL_ATT_KV * 4 <= (int)gridDim.x) ok = flow_sdpa4<false>(F, Y, li, pos, base);
        else ok = flow_sdpa<false>(F, Y, li, pos, base);
        if (ok) ok = flow_out<false>(F, Y, li, (pos + SDPA_TILE) / SDPA_TILE, base, gh);
      }
    }
  } else {
    ok = flow_moe_a<GATE8, false, true>(F, Y, li, base, h0, h1);
    if (ok) ok = flow_moe_b<false>(F, Y, li, base);
    if (ok) ok = flow_moe_c<false>(F, Y, li, base);
  }
  wr_wait();
  // the next launch's tags.  (Every workgroup has read `base` by now: workgroup 0's last stage consumed results to
  // which, directly or through the stages before, every workgroup of the grid contributed.)
  if (blockIdx.x == 0 && threadIdx.x == 0) st_co32(uni(P.bar) + 16, base + (uint32_t)(uni(P.n_layers) + 1) * 8u);
}

}  // namespace sl
