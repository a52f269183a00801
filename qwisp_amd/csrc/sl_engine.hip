// Host side of libseedless_hip.so: persistent device buffers, the per-step launch sequence and
// the C ABI declared in include/seedless_hip.h.  Mirrors SeedlessFusedForward
// (SeedlessFusedVerify.swift:3111-4470 in the reference): weights, caches and scratch are
// allocated once at creation; a step enqueues its kernels on one stream and reads back int32
// token ids.  No CPU fallback exists: without a GPU every entry point fails.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <system_error>
#include <thread>
#include <vector>

#include "sl_flow.cuh"
#include "sl_mfma.cuh"
#include "sl_gdn_chunk.cuh"

using namespace sl;

namespace {

struct DevQ4 {
  uint32_t* w = nullptr;    // [n, k/8]
  uint32_t* sb = nullptr;   // [n, k/64] {scale, bias}
  int n = 0, k = 0;
};

struct LayerDev {
  int is_linear = 0;
  uint16_t *input_ln = nullptr, *post_ln = nullptr;
  // Gated-DeltaNet
  DevQ4 in_proj, out_proj;
  float *conv_w = nullptr, *a_log = nullptr, *dt_bias = nullptr;
  float* gdn_norm_w = nullptr;     // [128] fp32; norm_f32: it came as fp32 (gated norm without the half roundings)
  int norm_f32 = 0;
  uint16_t* hist[2] = {nullptr, nullptr};
  float* state[2] = {nullptr, nullptr};
  // attention
  DevQ4 qkv, o_proj;
  uint16_t *q_norm = nullptr, *k_norm = nullptr, *kcache = nullptr, *vcache = nullptr;
  // MoE
  uint16_t *router_w = nullptr, *sgate_w = nullptr;
  uint16_t* router_pad = nullptr;   // fp16 gates as one matrix [288, 2048] for the matrix-core router of hybrid chunks: rows 0..E-1, row 256 = shared gate
  uint32_t *gate8_w = nullptr, *gate8_sb = nullptr;   // 8-bit gates instead: [E+1, 512] words and [E+1, 32] {scale, bias}; row E = shared gate
  DevQ4 sw_gate, sw_up, sw_down, sh_gate, sh_up, sh_down;
  int32_t* route_inds = nullptr;
  uint16_t* route_scores = nullptr;
};

constexpr size_t HIST_ELEMS = (size_t)(SL_CONV_K - 1) * SL_CONV_DIM;
constexpr size_t STATE_ELEMS = (size_t)SL_GDN_HV * SL_GDN_D * SL_GDN_D;
constexpr int MAX_CHAIN = 256;
#ifndef SL_MERGE_BLOCKS_ROWS
#define SL_MERGE_BLOCKS_ROWS 8
#endif
constexpr int MERGE_BLOCKS_ROWS = SL_MERGE_BLOCKS_ROWS;   // steps of up to this many rows: the blocks' chains side by side, a workgroup per quarter head
constexpr int MERGE_LONG_ROWS = 64;      // steps of up to this many rows merge their attention tiles with the 16-wave kernel
constexpr int ROUTER_PAD_ROWS = 288;

// The single-launch step is a grid of workgroups that wait for each other's results without a grid barrier: it
// only makes progress when all of them are resident at once, so nothing else of this process may occupy compute
// units while it runs (another engine's step, a lane batch, a prefill chunk).  Every entry point that submits work
// and waits for it holds this process-wide lock from its first launch to its read-back; it is recursive because the
// lane entry points fall back to the single-engine ones.  (sl_head_argmax_noalloc, which only enqueues on the
// caller's stream, is outside it: its caller keeps it apart from single-launch steps.)
std::recursive_mutex g_gpu_mutex;
#define SL_ENTER(e) std::lock_guard<std::recursive_mutex> gpu_lock_(g_gpu_mutex); int r = guard(e); if (r) return r
std::atomic<uint64_t> g_engine_uid{1};

// ---- scratch of the entry point that allocates nothing (sl_head_argmax_noalloc) --------------------------------
// lm_head + arg-max needs room for the logits rows and for one (value, index) candidate per 16 vocabulary rows and
// activation row.  For callers that must not allocate, that room is a fixed array in the library's device image:
// every GPU the library runs on holds its own copy at its own address until the process ends.  The array's name is
// only a host-side handle; the address kernels can use comes from hipGetSymbolAddress, once per device.
constexpr int NA_MAX_ROWS = 8;
constexpr int NA_MAX_VOCAB = 262144;
constexpr size_t NA_LOGITS_BYTES = (size_t)NA_MAX_ROWS * NA_MAX_VOCAB * sizeof(uint16_t);          // 4 MiB
constexpr size_t NA_CAND = (size_t)NA_MAX_ROWS * (NA_MAX_VOCAB / 16);                               // 131072 candidates
constexpr size_t NA_SCRATCH_BYTES = NA_LOGITS_BYTES + NA_CAND * (sizeof(float) + sizeof(int32_t));  // 5 MiB
static __device__ __align__(256) unsigned char scratch[NA_SCRATCH_BYTES];
constexpr int NA_MAX_DEVICES = 64;
void* g_scratch_ptr[NA_MAX_DEVICES] = {};
std::mutex g_scratch_mutex;
// Address of this device's copy of `scratch`; resolved on the first call per device (with that device current).
hipError_t scratch_address(int device, void** out) {
  if (device < 0 || device >= NA_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    const hipError_t r = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (r != hipSuccess) return r;
    g_scratch_ptr[device] = p;
  }
  *out = g_scratch_ptr[device];
  return hipSuccess;
}

}  // namespace

struct sl_full_snap {
  int pos = 0;
  std::vector<uint16_t*> hist;   // device copies, null for attention layers
  std::vector<float*> state;
};

struct sl_engine {
  uint64_t uid = g_engine_uid.fetch_add(1);   // never reused: identifies an engine in another engine's lane table
  // lanes keep their base alive: a base destroyed while lanes exist is only marked, and goes with its last lane
  sl_engine* base_of = nullptr;
  std::atomic<int> lane_refs{0};
  bool destroy_pending = false;
  int n_layers = 0, n_experts = 0, vocab = 0, max_m = 0, max_seq = 0, max_tiles = 0;
  int normed_rows = 0;             // final-normed rows of the last forward still held in `normed` (0 after a step)
  bool has_attn = false, has_head = false;
  int device = 0;                  // the device that was current when the engine was created
  void* na_scratch = nullptr;      // this device's copy of the no-allocation scratch array
  bool gate8 = false;              // router / shared gate are 8-bit rows (all layers alike)
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  hipStream_t side = nullptr;      // hybrid MoE: the shared expert's kernels run here, beside routing and the routed experts
  hipEvent_t side_fork = nullptr, side_join = nullptr;
  std::vector<void*> allocs;
  std::vector<LayerDev> layers;
  DevQ4 embed, lm_head;
  uint16_t* final_norm = nullptr;
  float *rope_cos = nullptr, *rope_sin = nullptr;
  // scratch
  uint16_t *hA = nullptr, *hB = nullptr, *proj = nullptr, *ycore = nullptr, *qrot = nullptr, *mix = nullptr, *xn = nullptr;
  float* xsum = nullptr;           // [max_m, 64] share sums of the rows in xn (steps of two or more rows)
  float* ysum = nullptr;           // [max_m, 128] share sums of the rows in ycore (gated mixer outputs) for the exact K = 4096 projection
  uint16_t *rlogits = nullptr, *sgate = nullptr, *sh_act = nullptr, *act = nullptr, *moe_out = nullptr, *normed = nullptr;
  uint16_t *logits = nullptr, *rows_out = nullptr;
  float *pm = nullptr, *pl = nullptr, *po = nullptr, *cand_v = nullptr;
  uint16_t *gdn_qn = nullptr, *gdn_kn = nullptr, *gdn_vc = nullptr;   // per-row inputs of the GDN scan (M >= 2 rows)
  float* gdn_gb = nullptr;
  int32_t *cand_i = nullptr, *tok_in = nullptr, *tok_out = nullptr, *st = nullptr;
  int n_cand = 0;
  // persistent single-token kernel
  uint32_t* dec_tstamp = nullptr;  // stage clock stamps [dec_grid][STAMP_WORDS], written by the stamping kernel variant
  bool stage_clock = false;
  unsigned* dec_bar = nullptr;
  int dec_grid = 0;                // 0 = not available (fewer than 256 compute units)
  FlowP* flow_params = nullptr;    // device copy of the single-launch step's parameters
  FlowP flow_host;
  uint32_t flow_base = 0;                                   // host mirror of the device's stage-instance counter
  std::vector<std::pair<void*, size_t>> flow_tagged;        // the tagged exchange buffers (cleared when the counter is rebased)
  void* pinned = nullptr;        // host staging
  size_t pinned_bytes = 0;
  // host mirrors of the device step state
  int pos = 0;
  std::vector<int> parity;
  float last_ms = 0.0f;
  // optional HIP-event timing of the lm_head kernel, one event pair per step of a chain
  bool profile_head = false;
  std::vector<hipEvent_t> head_ev;      // 2 * MAX_CHAIN
  int head_pending = 0;
  double head_ms_sum = 0.0;
  long head_launches = 0;
  bool use_persistent = true;
  bool last_block_flow = false;    // the last block entry point ran as a single launch: its intermediate rows are in the exchange buffers
  bool hybrid = false;             // prefill chunks: dense projections and grouped experts on the matrix cores (not bit-identical to the GEMV order)
  // scratch of the hybrid MoE (allocated when hybrid is first enabled): routed gate / up / down results per pair,
  // shared gate / up / down rows, pairs listed per expert
  uint16_t *hy_d = nullptr, *hy_sg = nullptr, *hy_su = nullptr, *hy_sy = nullptr, *hy_lists = nullptr;
  int32_t* hy_counts = nullptr;
  unsigned char* gc_scratch = nullptr;   // chunked gated-delta scan of hybrid chunks: [max_m / 64][32][GC_UNIT_BYTES]
  bool inject_failure = false;
  // lane batch driven from this engine's scratch: device table [n_layers][max_m] of the lanes last stepped together
  LaneRef* lane_tab = nullptr;
  std::vector<uint64_t> lane_set;              // uids of the lanes the table was built for
  // where the logits / normed rows of the most recent step live (a lane-batched step leaves them in the driver's rows)
  const uint16_t* logits_view = nullptr;
  const uint16_t* normed_view = nullptr;
  std::string fault;
};

namespace {

bool ok(sl_engine* e, hipError_t r, const char* what) {
  if (r == hipSuccess) return true;
  if (e->fault.empty()) e->fault = std::string(what) + ": " + hipGetErrorString(r);
  return false;
}
#define SL_TRY(e, call) do { if (!ok((e), (call), #call)) return SL_ERR_DEVICE; } while (0)

template <typename T>
T* dalloc(sl_engine* e, size_t count, bool zero = false) {
  void* p = nullptr;
  if (!ok(e, hipMalloc(&p, count * sizeof(T) > 0 ? count * sizeof(T) : 16), "hipMalloc")) return nullptr;
  e->allocs.push_back(p);
  if (zero && !ok(e, hipMemsetAsync(p, 0, count * sizeof(T), e->stream), "hipMemsetAsync")) return nullptr;
  return (T*)p;
}
bool copy_in(sl_engine* e, void* dst, const void* src, size_t bytes, int loc) {
  return ok(e, hipMemcpyAsync(dst, src, bytes, loc == SL_LOC_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice, e->stream),
            "hipMemcpyAsync(weights)") &&
         (loc != SL_LOC_HOST || ok(e, hipStreamSynchronize(e->stream), "hipStreamSynchronize"));
}
template <typename T>
T* upload(sl_engine* e, const void* src, size_t count, int loc) {
  if (!src) { if (e->fault.empty()) e->fault = "null tensor in model description"; return nullptr; }
  T* d = dalloc<T>(e, count);
  if (!d || !copy_in(e, d, src, count * sizeof(T), loc)) return nullptr;
  return d;
}
bool alloc_q4(sl_engine* e, DevQ4& d, int n, int k) {
  d.n = n; d.k = k;
  d.w = dalloc<uint32_t>(e, (size_t)n * (k / 8));
  d.sb = dalloc<uint32_t>(e, (size_t)n * (k / 64));
  return d.w && d.sb;
}
// Copies rows of `src` into rows [row_off, row_off + src.n) of `dst`, interleaving scale/bias.
bool fill_q4(sl_engine* e, DevQ4& dst, int row_off, const sl_q4& src, int n, int k, int loc) {
  if (!src.w || !src.scales || !src.biases || src.n != n || src.k != k || dst.k != k || row_off + n > dst.n) {
    if (e->fault.empty()) e->fault = "quantized tensor missing or of the wrong shape";
    return false;
  }
  const size_t wcount = (size_t)n * (k / 8), gcount = (size_t)n * (k / 64);
  if (!copy_in(e, dst.w + (size_t)row_off * (k / 8), src.w, wcount * 4, loc)) return false;
  uint32_t* out = dst.sb + (size_t)row_off * (k / 64);
  if (loc == SL_LOC_HOST) {
    std::vector<uint32_t> tmp(gcount);
    for (size_t i = 0; i < gcount; ++i) tmp[i] = (uint32_t)src.scales[i] | ((uint32_t)src.biases[i] << 16);
    return copy_in(e, out, tmp.data(), gcount * 4, SL_LOC_HOST);
  }
  hipLaunchKernelGGL(k_pack_sb, dim3((unsigned)((gcount + 255) / 256)), dim3(256), 0, e->stream, src.scales, src.biases, out, gcount);
  return ok(e, hipGetLastError(), "k_pack_sb");
}
// Rows of an 8-bit matrix (k = 2048: 512 words and 32 groups per row) into rows [row_off, row_off + src.n).
bool fill_q8(sl_engine* e, uint32_t* dw, uint32_t* dsb, int row_off, const sl_q4& src, int loc) {
  const size_t wcount = (size_t)src.n * (H / 4), gcount = (size_t)src.n * (H / 64);
  if (!copy_in(e, dw + (size_t)row_off * (H / 4), src.w, wcount * 4, loc)) return false;
  uint32_t* out = dsb + (size_t)row_off * (H / 64);
  if (loc == SL_LOC_HOST) {
    std::vector<uint32_t> tmp(gcount);
    for (size_t i = 0; i < gcount; ++i) tmp[i] = (uint32_t)src.scales[i] | ((uint32_t)src.biases[i] << 16);
    return copy_in(e, out, tmp.data(), gcount * 4, SL_LOC_HOST);
  }
  hipLaunchKernelGGL(k_pack_sb, dim3((unsigned)((gcount + 255) / 256)), dim3(256), 0, e->stream, src.scales, src.biases, out, gcount);
  return ok(e, hipGetLastError(), "k_pack_sb");
}
bool upload_q4(sl_engine* e, DevQ4& d, const sl_q4& src, int n, int k, int loc) {
  return alloc_q4(e, d, n, k) && fill_q4(e, d, 0, src, n, k, loc);
}

float half_bits_to_float(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
void build_rope(std::vector<float>& c, std::vector<float>& s, int max_seq) {
  c.resize((size_t)max_seq * 32); s.resize((size_t)max_seq * 32);
  for (int i = 0; i < 32; ++i) {
    // freq = theta^(-2i/64), theta = 1e7; the angle is formed in fp32 as in attn_q_prep_rows
    // (SeedlessFusedVerify.swift:1240-1242), its cosine and sine are taken in double.
    const float freq = (float)std::exp(-2.0 * (double)i / (double)SL_ROPE_DIM * std::log(1e7));
    for (int p = 0; p < max_seq; ++p) {
      const float ang = (float)p * freq;
      c[(size_t)p * 32 + i] = (float)std::cos((double)ang);
      s[(size_t)p * 32 + i] = (float)std::sin((double)ang);
    }
  }
}

int push_state(sl_engine* e, int layer_parity_only = -1) {
  (void)layer_parity_only;
  std::vector<int32_t> h(1 + e->n_layers);
  h[0] = e->pos;
  for (int i = 0; i < e->n_layers; ++i) h[1 + i] = e->parity[i];
  std::memcpy(e->pinned, h.data(), h.size() * 4);
  SL_TRY(e, hipMemcpyAsync(e->st, e->pinned, h.size() * 4, hipMemcpyHostToDevice, e->stream));
  SL_TRY(e, hipStreamSynchronize(e->stream));
  return SL_OK;
}

int guard(sl_engine* e) {
  if (!e) return SL_ERR_ARG;
  if (!e->fault.empty()) return SL_ERR_POISONED;
  return SL_OK;
}
int check_rows(sl_engine* e, int m) {
  if (m < 1 || m > e->max_m) return SL_ERR_ARG;
  if (e->has_attn && e->pos + m > e->max_seq) return SL_ERR_ARG;
  return SL_OK;
}
// Waits for the stream; the injected failure stands in for a failed submission.
int finish(sl_engine* e, const char* what) {
  hipError_t r = hipStreamSynchronize(e->stream);
  if (r == hipSuccess) r = hipGetLastError();
  if (e->inject_failure) {
    e->inject_failure = false;
    e->fault = std::string(what) + ": injected device failure";
    return SL_ERR_DEVICE;
  }
  if (!ok(e, r, what)) return SL_ERR_DEVICE;
  return SL_OK;
}

// ---- launch sequences -------------------------------------------------------------------------------
// Hybrid prefill: the shared expert and the routed experts, grouped by expert, go to the matrix cores.  So do the
// router and shared-gate logits when the gates are fp16 rows (one fp16 GEMM, k_router_mfma: another accumulation
// order than the exact rows, so an expert whose logit is within fp16 noise of the eighth may be chosen differently);
// 8-bit gates keep the exact rows of k_moe_a.
void launch_moe_hybrid(sl_engine* e, LayerDev& L, int M, const HiddenArgs& ha) {
  const int E = e->n_experts;
  MoeAArgs a{};
  a.ha = ha;
  a.router_w = L.router_w; a.sgate_w = L.sgate_w; a.g8_w = L.gate8_w; a.g8_sb = L.gate8_sb; a.E = E; a.skip_shared = 1;
  a.sh_act = e->sh_act; a.rlogits = e->rlogits; a.sgate = e->sgate;
  const int router_blocks = (E + 1 + 15) / 16;
  hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, ha);     // residual + norm once per row
  a.xn_in = ha.xn_out;
  // The shared expert needs nothing of the routing: its three kernels go to a second stream and run beside the router,
  // the routing and the grouping (a small GEMM, a kernel of one wave per row and one of a single workgroup, which
  // leave the device nearly idle for 40 us per layer) and the routed experts; the combine waits for both.
  hipStream_t shs = e->side ? e->side : e->stream;
  if (e->side) {
    (void)hipEventRecord(e->side_fork, e->stream);
    (void)hipStreamWaitEvent(e->side, e->side_fork, 0);
  }
  launch_qmm4_mfma(QmmArgs{e->xn, H, L.sh_gate.w, L.sh_gate.sb, M, SL_MOE_I, H, e->hy_sg, SL_MOE_I, L.sh_up.w, L.sh_up.sb, e->hy_su}, shs);
  hipLaunchKernelGGL(k_swiglu_rows, dim3((M * SL_MOE_I + 255) / 256), dim3(256), 0, shs, e->hy_sg, e->hy_su, e->sh_act, M * SL_MOE_I);
  launch_qmm4_mfma(QmmArgs{e->sh_act, SL_MOE_I, L.sh_down.w, L.sh_down.sb, M, H, SL_MOE_I, e->hy_sy, H}, shs);
  if (e->side) (void)hipEventRecord(e->side_join, e->side);
  if (L.router_pad)      // fp16 gates: router and shared-gate logits of all rows as one small GEMM on the matrix cores
    hipLaunchKernelGGL(k_router_mfma, dim3((ROUTER_PAD_ROWS / 32 + 3) / 4, (M + 31) / 32), dim3(256), 0, e->stream,
                       RouterMmArgs{ha.xn_out, L.router_pad, M, ROUTER_PAD_ROWS, e->rlogits, e->sgate});
  else
    hipLaunchKernelGGL(k_moe_a, dim3(router_blocks, M), dim3(256), 0, e->stream, a);
  hipLaunchKernelGGL(k_route_rows, dim3(M), dim3(64), 0, e->stream, e->rlogits, E, L.route_inds, L.route_scores);
  hipLaunchKernelGGL(k_group_pairs, dim3(1), dim3(1024), 0, e->stream, L.route_inds, M, E, e->hy_lists, e->hy_counts, e->hy_counts + SL_MAX_EXPERTS);
  // routed gate and up by expert in one pass with SwiGLU, then routed down by expert
  QmmGroupArgs g{e->xn, H, 0, L.sw_gate.w, L.sw_gate.sb, L.sw_up.w, L.sw_up.sb, SL_MOE_I, H, e->hy_lists, e->hy_counts, e->hy_counts + SL_MAX_EXPERTS, e->act, SL_MOE_I};
  hipLaunchKernelGGL(k_qmm4_mfma_grouped<true>, dim3(SL_MOE_I / 128, E), dim3(256), 0, e->stream, g);
  QmmGroupArgs d{e->act, SL_MOE_I, 1, L.sw_down.w, L.sw_down.sb, nullptr, nullptr, H, SL_MOE_I, e->hy_lists, e->hy_counts, e->hy_counts + SL_MAX_EXPERTS, e->hy_d, H};
  hipLaunchKernelGGL(k_qmm4_mfma_grouped<false>, dim3(H / 128, E), dim3(256), 0, e->stream, d);
  if (e->side) (void)hipStreamWaitEvent(e->stream, e->side_join, 0);
  hipLaunchKernelGGL(k_moe_combine_rows, dim3(H / 256, M), dim3(256), 0, e->stream, e->hy_d, L.route_scores, e->sgate, e->hy_sy, e->moe_out);
}
constexpr int HIDDEN_TILE_MAX_ROWS = 4;  // up to here the in-projection's waves do residual + norm of a row each
constexpr int MOE_PROLOGUE_MAX_ROWS = 8;  // up to here stage A's waves do residual + norm themselves
constexpr int MOE_GROUP_MIN_ROWS = 128;   // below, most experts are chosen by one row and the extra launches cost more
void launch_moe(sl_engine* e, LayerDev& L, int M, const HiddenArgs& ha) {
  MoeAArgs a{};
  a.ha = ha;
  a.shg_w = L.sh_gate.w; a.shg_sb = L.sh_gate.sb; a.shu_w = L.sh_up.w; a.shu_sb = L.sh_up.sb;
  a.router_w = L.router_w; a.sgate_w = L.sgate_w; a.g8_w = L.gate8_w; a.g8_sb = L.gate8_sb; a.E = e->n_experts;
  a.sh_act = e->sh_act; a.rlogits = e->rlogits; a.sgate = e->sgate;
  const int router_blocks = (e->n_experts + 1 + 15) / 16;
  // residual + norm once per row (k_final_rows) instead of once per wave of stage A; for a few rows (a verify step)
  // the waves' own prologue costs less than the launch
  const bool rows_first = M > MOE_PROLOGUE_MAX_ROWS;
  if (rows_first) {
    HiddenArgs hs = ha;
    hs.xs_out = e->xsum;                                // and the row's word sums for the routed experts' dots
    hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, hs);
    a.xn_in = ha.xn_out;
  }
  const bool grouped = M >= MOE_GROUP_MIN_ROWS && M <= GROUP_CAP;   // the shared expert then rides with the routed ones, by expert
  a.skip_shared = grouped ? 1 : 0;
  hipLaunchKernelGGL(k_moe_a, dim3((grouped ? 0 : MOE_A_SHARED_BLOCKS) + router_blocks, M), dim3(256), 0, e->stream, a);
  const bool route_in_b = !rows_first;                  // a few rows: stage B's waves route for themselves, one launch less
  if (!route_in_b) hipLaunchKernelGGL(k_route_rows, dim3(M), dim3(64), 0, e->stream, e->rlogits, e->n_experts, L.route_inds, L.route_scores);
  MoeBArgs b{};
  b.xn = e->xn; b.g_w = L.sw_gate.w; b.g_sb = L.sw_gate.sb; b.u_w = L.sw_up.w; b.u_sb = L.sw_up.sb;
  b.act = e->act; b.inds = L.route_inds; b.xsum = rows_first ? e->xsum : nullptr;
  if (route_in_b) { b.rlogits = e->rlogits; b.E = e->n_experts; b.inds_out = L.route_inds; b.scores_out = L.route_scores; }
  if (grouped) {                                        // weights of an expert fetched once for all rows that chose it
    hipLaunchKernelGGL(k_group_pairs, dim3(1), dim3(1024), 0, e->stream, L.route_inds, M, e->n_experts, e->hy_lists, e->hy_counts, e->hy_counts + SL_MAX_EXPERTS);
    MoeBGroupArgs g{e->xn, b.g_w, b.g_sb, b.u_w, b.u_sb, e->act, e->hy_lists, e->hy_counts, e->xsum, e->hy_counts + SL_MAX_EXPERTS,
                    L.sh_gate.w, L.sh_gate.sb, L.sh_up.w, L.sh_up.sb, e->sh_act, M};
    hipLaunchKernelGGL(k_moe_b_grouped, dim3(64, (M + 63) / 64 + e->n_experts), dim3(256), 0, e->stream, g);
  } else {
    if (route_in_b) hipLaunchKernelGGL(k_moe_b<true>, dim3(256, M), dim3(256), 0, e->stream, b);
    else hipLaunchKernelGGL(k_moe_b<false>, dim3(256, M), dim3(256), 0, e->stream, b);
  }
  if (M >= MOE_GROUP_MIN_ROWS && M <= GROUP_CAP && e->hy_d && e->hy_sy) {   // the down stage by expert as well, then the combine
    MoeCGroupArgs cg{e->act, e->sh_act, L.sw_down.w, L.sw_down.sb, L.sh_down.w, L.sh_down.sb, e->hy_lists, e->hy_counts,
                     e->hy_counts + SL_MAX_EXPERTS, e->hy_d, e->hy_sy, M, e->n_experts};
    hipLaunchKernelGGL(k_moe_c_grouped, dim3(64, (M + 63) / 64 + e->n_experts), dim3(256), 0, e->stream, cg);
    hipLaunchKernelGGL(k_moe_combine_rows, dim3(H / 256, M), dim3(256), 0, e->stream, e->hy_d, L.route_scores, e->sgate, e->hy_sy, e->moe_out);
    return;
  }
  MoeCArgs c{};
  c.act = e->act; c.sh_act = e->sh_act; c.inds = L.route_inds; c.scores = L.route_scores; c.sgate = e->sgate;
  c.d_w = L.sw_down.w; c.d_sb = L.sw_down.sb; c.shd_w = L.sh_down.w; c.shd_sb = L.sh_down.sb; c.out = e->moe_out;
  hipLaunchKernelGGL(k_moe_c, dim3(128, M), dim3(256), 0, e->stream, c);
}
// In-projection of M >= 2 rows: residual + norm once per row (beyond four rows), then the row-tiled projection into e->proj.  Workgroups
// of 16 weight rows, three to a compute unit: when the count is just over a multiple of the machine's 768 places the
// surplus rows go one each to the first workgroups instead of opening another round.
void launch_hidden_tile(sl_engine* e, const HiddenArgs& ha, const uint32_t* w, const uint32_t* sb, int N, int M) {
  constexpr int PLACES = 768;
  int G = N / 16;
  const int over = G % PLACES;
  if (G > PLACES && over <= 16) G -= over;
  if (G * 16 + G < N) G = (N + 15) / 16;          // (not with the shapes of this model)
  if (M <= HIDDEN_TILE_MAX_ROWS) {
    // a few rows (a verify step): the waves of every workgroup do residual + norm of a row each, one launch less
    hipLaunchKernelGGL((k_qmv_tile<1, 4, 8, true>), dim3(G, (M + 7) / 8), dim3(256), 0, e->stream, ha, (const uint16_t*)nullptr, 0,
                       w, sb, N, e->proj, PROJ_STRIDE, M);
    return;
  }
  HiddenArgs hn = ha;
  hn.xn_out = e->xn;
  hn.xs_out = e->xsum;
  hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, hn);
  hipLaunchKernelGGL((k_qmv_tile<1, 4, 8, false>), dim3(G, (M + 7) / 8), dim3(256), 0, e->stream, HiddenArgs{}, e->xn, H,
                     w, sb, N, e->proj, PROJ_STRIDE, M, (float*)nullptr, (int32_t*)nullptr, e->xsum);
}
// Hybrid mode: steps of at least 16 rows (prefill chunks, lane batches) take the dense projections to the matrix cores.
// (Rows of one sequence or one row each of a batch of lanes: the projections and the experts do not care.)
// The K = 4096 projections have 2048 outputs = 16 workgroups per 32-row tile on the matrix cores: a lane batch of
// fewer than 64 rows keeps the row-tiled exact kernel for them (256 workgroups per 4 rows; 32 rows: 21 against 28 us).
// Prefill chunks do not switch, so that a row's result does not depend on the chunking.
constexpr int MM_OUT_ROWS = 64;
constexpr int GDN_PREP_LONG = 512;    // from here on a wave of the GDN preparation walks 16 rows, below 4
bool use_matrix_cores(const sl_engine* e, int M, const LaneRef* lanes) { (void)lanes; return e->hybrid && M >= 16 && M <= GROUP_CAP; }
// `lanes` (null for rows of one sequence) = this layer's row of the lane table: row b of the batch is lane b's next token.
void launch_gdn_mixer(sl_engine* e, LayerDev& L, int li, int M, const HiddenArgs& ha, const LaneRef* lanes) {
  const bool mm = use_matrix_cores(e, M, lanes);
  if (mm) {
    HiddenArgs hn = ha; hn.xn_out = e->xn;      // residual + norm rows on their own, then the GEMM
    hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, hn);
    launch_qmm4_mfma(QmmArgs{e->xn, H, L.in_proj.w, L.in_proj.sb, M, SL_GDN_IN_N, H, e->proj, PROJ_STRIDE}, e->stream);
  } else if (M >= 2) {
    launch_hidden_tile(e, ha, L.in_proj.w, L.in_proj.sb, SL_GDN_IN_N, M);
  } else {
    hipLaunchKernelGGL(k_qmv_hidden<4>, dim3(SL_GDN_IN_N / 16, M), dim3(256), 0, e->stream, ha, L.in_proj.w, L.in_proj.sb,
                       SL_GDN_IN_N, e->proj, PROJ_STRIDE);
  }
  GdnArgs g{};
  g.proj = e->proj; g.conv_w = L.conv_w; g.a_log = L.a_log; g.dt_bias = L.dt_bias;
  g.hist[0] = L.hist[0]; g.hist[1] = L.hist[1]; g.state[0] = L.state[0]; g.state[1] = L.state[1];
  g.st = e->st + li;       // st[1] of this view = parity of layer li
  g.ycore = e->ycore; g.M = M; g.lanes = lanes; g.layer = li;
  const bool few = !lanes && !mm && M >= 2 && M <= GDN_FEW_ROWS;
  if (few) {
    // a verify step: conv, norms, recurrence and gated norm of a value head in one workgroup, one launch instead of three
    hipLaunchKernelGGL(k_gdn_few_rows, dim3(SL_GDN_HV), dim3(1024), 0, e->stream, g, L.gdn_norm_w, L.norm_f32, e->ysum);
  } else if (!lanes && M >= 2) {
    // rows of one sequence: the state-independent part for all rows at once, then the scan without barriers
    GdnPrepArgs pa{g, e->gdn_qn, e->gdn_kn, e->gdn_vc, e->gdn_gb};
    if (M >= GDN_PREP_LONG) hipLaunchKernelGGL(k_gdn_prep_rows<16>, dim3(65, (M + 15) / 16), dim3(64), 0, e->stream, pa);
    else hipLaunchKernelGGL(k_gdn_prep_rows<4>, dim3(65, (M + 3) / 4), dim3(64), 0, e->stream, pa);
    if (mm && e->gc_scratch && M % GC == 0 && e->pos % GC == 0) {
      // hybrid chunks cut at multiples of 64 rows: the delta rule in its chunked form on the matrix cores
      GdnChunkArgs ca{e->gdn_qn, e->gdn_kn, e->gdn_vc, e->gdn_gb, e->gc_scratch, {L.state[0], L.state[1]}, {L.hist[0], L.hist[1]},
                      e->proj, e->st + li, e->ycore, M};
      hipLaunchKernelGGL(k_gdn_chunk_prep, dim3(M / GC, SL_GDN_HV), dim3(256), 0, e->stream, ca);
      hipLaunchKernelGGL(k_gdn_chunk_scan, dim3(SL_GDN_HV), dim3(256), GC_SCAN_LDS, e->stream, ca);
    } else {
      hipLaunchKernelGGL(k_gdn_scan_rows, dim3(512), dim3(256), 0, e->stream, pa);
    }
  } else {
    if (lanes) hipLaunchKernelGGL(k_gdn_core<4>, dim3(128, M), dim3(256), 0, e->stream, g);
    else hipLaunchKernelGGL(k_gdn_core<2>, dim3(256, 1), dim3(256), 0, e->stream, g);
  }
  if (mm && !(lanes && M < MM_OUT_ROWS)) {
    hipLaunchKernelGGL(k_gdn_gate_rows, dim3(SL_GDN_HV, M), dim3(64), 0, e->stream, e->ycore, e->proj, L.gdn_norm_w, L.norm_f32);
    launch_qmm4_mfma(QmmArgs{e->ycore, 4096, L.out_proj.w, L.out_proj.sb, M, H, 4096, e->mix, H}, e->stream);
  } else if (M >= 2) {
    // the gated norm once per row, then the row-tiled projection (same bits as the fused kernel below)
    if (!few) hipLaunchKernelGGL(k_gdn_gate_rows, dim3(SL_GDN_HV, M), dim3(64), 0, e->stream, e->ycore, e->proj, L.gdn_norm_w, L.norm_f32, e->ysum);
    hipLaunchKernelGGL((k_qmv_tile<2, 2, 4, false>), dim3(H / 8, (M + 3) / 4), dim3(256), 0, e->stream, HiddenArgs{}, e->ycore, 4096,
                       L.out_proj.w, L.out_proj.sb, H, e->mix, H, M, (float*)nullptr, (int32_t*)nullptr, e->ysum);
  } else {
    hipLaunchKernelGGL(k_qmv_gdn_out<2>, dim3(H / 8, M), dim3(256), 0, e->stream, e->ycore, e->proj, L.gdn_norm_w, L.norm_f32,
                       L.out_proj.w, L.out_proj.sb, H, e->mix);
  }
}
void launch_attn_mixer(sl_engine* e, LayerDev& L, int M, const HiddenArgs& ha, const LaneRef* lanes, int lane_tiles) {
  const bool mm = use_matrix_cores(e, M, lanes);
  if (mm) {
    HiddenArgs hn = ha; hn.xn_out = e->xn;
    hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, hn);
    launch_qmm4_mfma(QmmArgs{e->xn, H, L.qkv.w, L.qkv.sb, M, SL_ATT_QKV_N, H, e->proj, PROJ_STRIDE}, e->stream);
  } else if (M >= 2) {
    launch_hidden_tile(e, ha, L.qkv.w, L.qkv.sb, SL_ATT_QKV_N, M);
  } else {
    hipLaunchKernelGGL(k_qmv_hidden<4>, dim3(SL_ATT_QKV_N / 16, M), dim3(256), 0, e->stream, ha, L.qkv.w, L.qkv.sb,
                       SL_ATT_QKV_N, e->proj, PROJ_STRIDE);
  }
  AttnPrepArgs p{};
  p.proj = e->proj; p.q_norm = L.q_norm; p.k_norm = L.k_norm; p.rope_cos = e->rope_cos; p.rope_sin = e->rope_sin;
  p.st = e->st; p.qrot = e->qrot; p.kcache = L.kcache; p.vcache = L.vcache; p.maxSeq = e->max_seq; p.lanes = lanes;
  hipLaunchKernelGGL(k_attn_prep, dim3(18, M), dim3(64), 0, e->stream, p);
  const int tiles = lanes ? lane_tiles : (e->pos + M + SDPA_TILE - 1) / SDPA_TILE;
  SdpaArgs s{};
  s.qrot = e->qrot; s.kcache = L.kcache; s.vcache = L.vcache; s.st = e->st; s.maxSeq = e->max_seq; s.maxTiles = e->max_tiles;
  s.pm = e->pm; s.pl = e->pl; s.po = e->po; s.lanes = lanes;
  if (mm && lanes) {
    const int T = tiles >= 32 ? 4 : (tiles >= 8 ? 2 : 1);
    hipLaunchKernelGGL(k_sdpa_lane_mfma, dim3((tiles + T - 1) / T, SL_ATT_KV, M), dim3(256), 0, e->stream, SdpaLaneArgs{s, T});
  }
  int tiles_per_part = 0;
  if (mm && !lanes) {
    // parts of SDPA_FLASH_TILES key tiles at fixed positions: a row's tiles are then added up in the same grouping
    // whatever the chunking of the prompt, so the result of a row does not depend on it
    const int row_blocks = (M + 31) / 32;
    tiles_per_part = SDPA_FLASH_TILES;
    const int parts = (tiles + tiles_per_part - 1) / tiles_per_part;
    hipLaunchKernelGGL(k_sdpa_flash_mfma, dim3(parts, SL_ATT_KV, row_blocks), dim3(512), 0, e->stream, SdpaFlashArgs{s, M, tiles_per_part});
  }
  else if (!mm) hipLaunchKernelGGL(k_sdpa_tile, dim3(tiles, SL_ATT_KV, M), dim3(256), 0, e->stream, s);
  SdpaMergeArgs g{};
  g.pm = e->pm; g.pl = e->pl; g.po = e->po; g.proj = e->proj; g.st = e->st; g.maxTiles = e->max_tiles; g.gated = e->ycore; g.lanes = lanes;
  g.group = tiles_per_part;
  g.gsum = mm ? nullptr : e->ysum;                       // the exact merge leaves the gated rows' word sums for the projection
  if (mm && lanes) hipLaunchKernelGGL(k_sdpa_merge_par<16>, dim3(SL_ATT_HEADS, M), dim3(1024), 0, e->stream, g);
  else if (mm) hipLaunchKernelGGL(k_sdpa_merge_par<4>, dim3(SL_ATT_HEADS, M), dim3(256), 0, e->stream, g);
  else if (M <= MERGE_BLOCKS_ROWS) hipLaunchKernelGGL(k_sdpa_merge_blocks, dim3(SL_ATT_HEADS, M, 4), dim3(64 * MERGE_BLOCKS_WAVES), 0, e->stream, g);
  else if (M <= MERGE_LONG_ROWS) hipLaunchKernelGGL(k_sdpa_merge_long, dim3(SL_ATT_HEADS, M), dim3(1024), MERGE_DYN_LDS, e->stream, g);
  else hipLaunchKernelGGL(k_sdpa_merge, dim3(SL_ATT_HEADS, M), dim3(64), 0, e->stream, g);
  if (mm && !(lanes && M < MM_OUT_ROWS)) launch_qmm4_mfma(QmmArgs{e->ycore, 4096, L.o_proj.w, L.o_proj.sb, M, H, 4096, e->mix, H}, e->stream);
  else if (M >= 2) hipLaunchKernelGGL((k_qmv_tile<2, 2, 4, false>), dim3(H / 8, (M + 3) / 4), dim3(256), 0, e->stream, HiddenArgs{}, e->ycore, 4096,
                                      L.o_proj.w, L.o_proj.sb, H, e->mix, H, M, (float*)nullptr, (int32_t*)nullptr, mm ? (float*)nullptr : e->ysum);
  else hipLaunchKernelGGL((k_qmv_plain<2, 2>), dim3(H / 8, M), dim3(256), 0, e->stream, e->ycore, 4096, L.o_proj.w, L.o_proj.sb,
                          H, e->mix, H);
}
// All layers over M rows held in hA.  On return the hidden state is hA + moe_out (residual pending).
// With `lane_tab` the M rows are one token each of M lanes (caches and positions from the table, the longest
// lane needing `lane_tiles` key tiles); without, M consecutive rows of this engine's own sequence.
void launch_layer(sl_engine* e, int li, int M, const LaneRef* lane_tab = nullptr, int lane_tiles = 0) {
  e->last_block_flow = false;
  LayerDev& L = e->layers[li];
  const LaneRef* lanes = lane_tab ? lane_tab + (size_t)li * e->max_m : nullptr;
  HiddenArgs ha{e->hA, li > 0 ? e->moe_out : nullptr, L.input_ln, e->hB, nullptr};
  if (L.is_linear) launch_gdn_mixer(e, L, li, M, ha, lanes);
  else launch_attn_mixer(e, L, M, ha, lanes, lane_tiles);
  HiddenArgs hb{e->hB, e->mix, L.post_ln, e->hA, e->xn};
  // grouping by expert pays once an expert sees several rows; a batch of fewer than 64 lanes leaves most experts
  // with one row or none, and the per-row expert kernels stream the same weights with less overhead (rows of one
  // sequence always take the grouped path, so that a row's result does not depend on the size of its chunk)
  if (use_matrix_cores(e, M, lanes) && (!lanes || M >= 64)) launch_moe_hybrid(e, L, M, hb);
  else launch_moe(e, L, M, hb);
}
void launch_layers(sl_engine* e, int M, const LaneRef* lane_tab = nullptr, int lane_tiles = 0) {
  for (int li = 0; li < e->n_layers; ++li) launch_layer(e, li, M, lane_tab, lane_tiles);
}
void advance(sl_engine* e, int M) {
  hipLaunchKernelGGL(k_advance, dim3(1), dim3(64), 0, e->stream, e->st, M, e->n_layers);
  e->pos += M;
  for (int i = 0; i < e->n_layers; ++i) if (e->layers[i].is_linear) e->parity[i] ^= 1;
}
void launch_head(sl_engine* e, int M, const HiddenArgs& ha, int out_off, bool feed) {
  const bool prof = e->profile_head && e->head_pending < MAX_CHAIN;
  if (prof) (void)hipEventRecord(e->head_ev[2 * e->head_pending], e->stream);
  bool have_tokens = false;
  if (M >= 2) {
    // residual + final norm once per row, then the row-tiled lm_head (weights streamed once per 8 rows)
    const uint16_t* xin = ha.h_in;
    if (ha.r_in || ha.lnw) {
      HiddenArgs hn = ha;
      if (!hn.xn_out) hn.xn_out = e->xn;
      hipLaunchKernelGGL(k_final_rows, dim3(M), dim3(64), 0, e->stream, hn);
      xin = hn.xn_out;
    }
    if (use_matrix_cores(e, M, nullptr) && e->vocab % 32 == 0) {
      // hybrid mode: lm_head on the matrix cores, arg-max of the rounded logits rows
      launch_qmm4_mfma(QmmArgs{xin, H, e->lm_head.w, e->lm_head.sb, M, e->vocab, H, e->logits, e->vocab}, e->stream);
      hipLaunchKernelGGL(k_argmax_logits, dim3(M), dim3(1024), 0, e->stream, e->logits, e->vocab, e->tok_out, out_off);
      have_tokens = true;
    } else {
      hipLaunchKernelGGL((k_qmv_tile<1, 4, 8, false, true>), dim3(e->n_cand, (M + 7) / 8), dim3(256), 0, e->stream, HiddenArgs{}, xin, H,
                         e->lm_head.w, e->lm_head.sb, e->vocab, e->logits, e->vocab, M, e->cand_v, e->cand_i);
    }
  } else {
    hipLaunchKernelGGL(k_head, dim3(e->n_cand, M), dim3(256), 0, e->stream, ha, e->lm_head.w, e->lm_head.sb, e->vocab,
                       e->logits, e->cand_v, e->cand_i);
  }
  if (prof) { (void)hipEventRecord(e->head_ev[2 * e->head_pending + 1], e->stream); e->head_pending++; }
  if (!have_tokens)
    hipLaunchKernelGGL(k_argmax_final, dim3(M), dim3(256), 0, e->stream, e->cand_v, e->cand_i, e->n_cand, e->tok_out, out_off,
                       feed ? e->tok_in : (int32_t*)nullptr);
}
// `steps` batch-1 steps in a single persistent launch (each token fed back on the device); host mirrors advance
// as the kernel's own update does.
// The step kernel tags what it exchanges with a counter of stage instances that it advances by 8 * (layers + 1) per
// step (sl_flow.cuh).  Attention partials carry 31 bits of it and their slots are not rewritten every step, so the
// counter must never wrap while a stale slot could still hold the equal tag of 2^31 instances earlier.  It does not
// get there: before a launch that would take the counter past FLOW_BASE_LIMIT the host clears every tagged buffer
// (tag 0 is never expected: expected tags have their top bit set) and starts the counter again at 0.
constexpr uint32_t FLOW_BASE_LIMIT = 0x7ff00000u;
bool flow_rebase_needed(uint32_t base, int steps, int n_layers) {
  return (uint64_t)base + (uint64_t)(steps + 1) * (uint64_t)(n_layers + 1) * 8u > (uint64_t)FLOW_BASE_LIMIT;
}
// Moves the host's mirror of the tag counter on by `steps` step-sized strides, restarting it first where it would wrap.
void flow_advance_base(sl_engine* e, int steps) {
  if (flow_rebase_needed(e->flow_base, steps, e->n_layers)) {
    for (const auto& b : e->flow_tagged) (void)hipMemsetAsync(b.first, 0, b.second, e->stream);
    (void)hipMemsetAsync(e->dec_bar + 16, 0, 4, e->stream);
    e->flow_base = 0;
  }
  e->flow_base += (uint32_t)steps * (uint32_t)(e->n_layers + 1) * 8u;
}
// One block of one layer (mode 0: the mixer, 1: the MoE block) on the row in e->xn, in a single launch of the step
// kernel's stages; the result is left in the stage's exchange buffer (tmix / tmoe: halves with the tags of this launch).
bool block_flow_ready(const sl_engine* e, int m) { return m == 1 && e->dec_grid > 0 && e->use_persistent && e->flow_params; }
void launch_block_flow(sl_engine* e, int layer, int mode) {
  e->last_block_flow = true;
  flow_advance_base(e, 1);
  auto kern = e->gate8 ? k_block_flow<true> : k_block_flow<false>;
  hipLaunchKernelGGL(kern, dim3(e->dec_grid), dim3(DEC_THREADS), DEC_DYN_LDS, e->stream, e->flow_params, e->flow_host.d.layers,
                     (const int32_t*)e->st, (const unsigned*)e->dec_bar, e->n_layers, layer, mode);
}
void launch_decode(sl_engine* e, int out_off, bool feed, int steps) {
  flow_advance_base(e, steps);
  const bool prof = e->profile_head && e->head_pending < MAX_CHAIN;
  if (prof) (void)hipEventRecord(e->head_ev[2 * e->head_pending], e->stream);
  auto kern = e->gate8 ? (e->stage_clock ? k_decode_flow<true, true> : k_decode_flow<true, false>)
                       : (e->stage_clock ? k_decode_flow<false, true> : k_decode_flow<false, false>);
  hipLaunchKernelGGL(kern, dim3(e->dec_grid), dim3(DEC_THREADS), DEC_DYN_LDS, e->stream, e->flow_params, out_off, feed ? 1 : 0, steps);
  if (prof) { (void)hipEventRecord(e->head_ev[2 * e->head_pending + 1], e->stream); e->head_pending++; }
  e->pos += steps;
  if (steps & 1) for (int i = 0; i < e->n_layers; ++i) if (e->layers[i].is_linear) e->parity[i] ^= 1;
}
int to_device(sl_engine* e, void* dst, const void* src, size_t bytes) {
  if (bytes > e->pinned_bytes) return SL_ERR_ARG;
  std::memcpy(e->pinned, src, bytes);
  SL_TRY(e, hipMemcpyAsync(dst, e->pinned, bytes, hipMemcpyHostToDevice, e->stream));
  return SL_OK;
}
// Large transfers (caches, snapshots) go straight between the caller's memory and the device.
int copy_sync(sl_engine* e, void* dst, const void* src, size_t bytes, hipMemcpyKind kind) {
  SL_TRY(e, hipMemcpyAsync(dst, src, bytes, kind, e->stream));
  SL_TRY(e, hipStreamSynchronize(e->stream));
  return SL_OK;
}

bool shape_ok(const sl_q4& q, int n, int k) { return q.w && q.scales && q.biases && q.n == n && q.k == k; }

}  // namespace

extern "C" {

namespace {
// Per-sequence storage of one layer: conv history and recurrent state (ping-pong), or the KV arena; routing read-back.
int alloc_layer_state(sl_engine* e, LayerDev& L) {
  if (L.is_linear) {
    for (int p = 0; p < 2; ++p) {
      L.hist[p] = dalloc<uint16_t>(e, HIST_ELEMS, true);
      L.state[p] = dalloc<float>(e, STATE_ELEMS, true);
    }
    if (!L.hist[1] || !L.state[1]) return SL_ERR_DEVICE;
  } else {
    e->has_attn = true;
    L.kcache = dalloc<uint16_t>(e, (size_t)SL_ATT_KV * e->max_seq * SL_ATT_D, true);
    L.vcache = dalloc<uint16_t>(e, (size_t)SL_ATT_KV * e->max_seq * SL_ATT_D, true);
    if (!L.kcache || !L.vcache) return SL_ERR_DEVICE;
  }
  L.route_inds = dalloc<int32_t>(e, (size_t)e->max_m * 8, true);
  L.route_scores = dalloc<uint16_t>(e, (size_t)e->max_m * 8, true);
  if (!L.route_inds || !L.route_scores) return SL_ERR_DEVICE;
  return SL_OK;
}
int alloc_runtime(sl_engine* e);
}  // namespace
static int read_back(sl_engine* e, void* dst, const void* dev, size_t bytes, const char* what, bool abort_word = false);
static void time_end(sl_engine* e);
static int read_back_tagged(sl_engine* e, uint16_t* out, const uint32_t* words, uint32_t tag, const char* what);

int sl_create(const sl_model_desc* d, int max_m, int max_seq_len, sl_engine** out) {
  if (!d || !out || max_m < 1 || max_seq_len < 1 || d->n_layers < 1 || !d->layers) return SL_ERR_ARG;
  if (d->n_experts < 8 || d->n_experts > SL_MAX_EXPERTS || (d->n_experts % 8) != 0) return SL_ERR_ARG;
  if (d->location != SL_LOC_HOST && d->location != SL_LOC_DEVICE) return SL_ERR_ARG;
  const bool has_head = d->embed.w != nullptr;
  if (has_head && (d->vocab < 16 || (d->vocab % 16) != 0 || !shape_ok(d->embed, d->vocab, H) ||
                   !shape_ok(d->lm_head, d->vocab, H) || !d->final_norm)) return SL_ERR_ARG;
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) return SL_ERR_DEVICE;

  sl_engine* e = new sl_engine();
  *out = e;   // returned even on failure so the caller can read sl_fault() and must sl_destroy()
  e->n_layers = d->n_layers; e->n_experts = d->n_experts; e->vocab = has_head ? d->vocab : 0;
  e->max_m = max_m; e->max_seq = max_seq_len; e->max_tiles = (max_seq_len + SDPA_TILE - 1) / SDPA_TILE;
  e->has_head = has_head;
  e->parity.assign(d->n_layers, 0);
  SL_TRY(e, hipGetDevice(&e->device));
  SL_TRY(e, scratch_address(e->device, &e->na_scratch));
  SL_TRY(e, hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
  SL_TRY(e, hipEventCreate(&e->ev0));
  SL_TRY(e, hipEventCreate(&e->ev1));
  const int loc = d->location, E = d->n_experts;
  e->layers.resize(d->n_layers);
  for (int i = 0; i < d->n_layers; ++i) {
    const sl_layer_desc& s = d->layers[i];
    LayerDev& L = e->layers[i];
    L.is_linear = s.is_linear;
    L.input_ln = upload<uint16_t>(e, s.input_ln, H, loc);
    L.post_ln = upload<uint16_t>(e, s.post_ln, H, loc);
    if (!L.input_ln || !L.post_ln) return SL_ERR_DEVICE;
    if (s.is_linear) {
      const sl_gdn_w& g = s.gdn;
      if (!alloc_q4(e, L.in_proj, SL_GDN_IN_N, H)) return SL_ERR_DEVICE;
      if (!fill_q4(e, L.in_proj, 0, g.in_proj_qkv, SL_CONV_DIM, H, loc) ||
          !fill_q4(e, L.in_proj, SL_CONV_DIM, g.in_proj_z, 4096, H, loc) ||
          !fill_q4(e, L.in_proj, SL_CONV_DIM + 4096, g.in_proj_b, SL_GDN_HV, H, loc) ||
          !fill_q4(e, L.in_proj, SL_CONV_DIM + 4096 + SL_GDN_HV, g.in_proj_a, SL_GDN_HV, H, loc) ||
          !upload_q4(e, L.out_proj, g.out_proj, H, 4096, loc)) return SL_ERR_ARG;
      L.conv_w = upload<float>(e, g.conv1d_w, (size_t)SL_CONV_DIM * SL_CONV_K, loc);
      L.a_log = upload<float>(e, g.a_log, SL_GDN_HV, loc);
      L.dt_bias = upload<float>(e, g.dt_bias, SL_GDN_HV, loc);
      if (g.norm_w_f32) {
        L.gdn_norm_w = upload<float>(e, g.norm_w_f32, SL_GDN_D, loc);
        L.norm_f32 = 1;
      } else if (g.norm_w) {
        // fp16 weight, kept as fp32 on the device (exact); a device-resident source comes through the host
        uint16_t hw[SL_GDN_D];
        float fw[SL_GDN_D];
        if (loc == SL_LOC_HOST) std::memcpy(hw, g.norm_w, sizeof(hw));
        else SL_TRY(e, hipMemcpy(hw, g.norm_w, sizeof(hw), hipMemcpyDeviceToHost));
        for (int j = 0; j < SL_GDN_D; ++j) fw[j] = half_bits_to_float(hw[j]);
        L.gdn_norm_w = upload<float>(e, fw, SL_GDN_D, SL_LOC_HOST);
      }
      if (!L.conv_w || !L.a_log || !L.dt_bias || !L.gdn_norm_w) return SL_ERR_DEVICE;
    } else {
      const sl_attn_w& a = s.attn;
      if (!alloc_q4(e, L.qkv, SL_ATT_QKV_N, H)) return SL_ERR_DEVICE;
      if (!fill_q4(e, L.qkv, 0, a.q_proj, 8192, H, loc) || !fill_q4(e, L.qkv, 8192, a.k_proj, 512, H, loc) ||
          !fill_q4(e, L.qkv, 8192 + 512, a.v_proj, 512, H, loc) || !upload_q4(e, L.o_proj, a.o_proj, H, 4096, loc))
        return SL_ERR_ARG;
      L.q_norm = upload<uint16_t>(e, a.q_norm, SL_ATT_D, loc);
      L.k_norm = upload<uint16_t>(e, a.k_norm, SL_ATT_D, loc);
      if (!L.q_norm || !L.k_norm) return SL_ERR_DEVICE;
    }
    const sl_moe_w& w = s.moe;
    if (w.router_w || w.shared_gate_w) {
      L.router_w = upload<uint16_t>(e, w.router_w, (size_t)E * H, loc);
      L.sgate_w = upload<uint16_t>(e, w.shared_gate_w, H, loc);
      L.router_pad = dalloc<uint16_t>(e, (size_t)ROUTER_PAD_ROWS * H, true);
      if (!L.router_w || !L.sgate_w || !L.router_pad) return SL_ERR_DEVICE;
      SL_TRY(e, hipMemcpyAsync(L.router_pad, L.router_w, (size_t)E * H * 2, hipMemcpyDeviceToDevice, e->stream));
      SL_TRY(e, hipMemcpyAsync(L.router_pad + (size_t)256 * H, L.sgate_w, (size_t)H * 2, hipMemcpyDeviceToDevice, e->stream));
    } else {
      // 8-bit gates: router rows and the shared-gate row in one matrix of E + 1 rows
      if (!shape_ok(w.router_q8, E, H) || !shape_ok(w.shared_gate_q8, 1, H)) {
        e->fault = "router / shared gate: neither fp16 rows nor 8-bit tensors of the right shape";
        return SL_ERR_ARG;
      }
      L.gate8_w = dalloc<uint32_t>(e, (size_t)(E + 1) * (H / 4));
      L.gate8_sb = dalloc<uint32_t>(e, (size_t)(E + 1) * (H / 64));
      if (!L.gate8_w || !L.gate8_sb) return SL_ERR_DEVICE;
      if (!fill_q8(e, L.gate8_w, L.gate8_sb, 0, w.router_q8, loc) || !fill_q8(e, L.gate8_w, L.gate8_sb, E, w.shared_gate_q8, loc))
        return SL_ERR_DEVICE;
    }
    if (i == 0) e->gate8 = L.gate8_w != nullptr;
    else if (e->gate8 != (L.gate8_w != nullptr)) { e->fault = "fp16 and 8-bit gates mixed across layers"; return SL_ERR_ARG; }
    if (!upload_q4(e, L.sw_gate, w.sw_gate, E * SL_MOE_I, H, loc) || !upload_q4(e, L.sw_up, w.sw_up, E * SL_MOE_I, H, loc) ||
        !upload_q4(e, L.sw_down, w.sw_down, E * H, SL_MOE_I, loc) || !upload_q4(e, L.sh_gate, w.sh_gate, SL_MOE_I, H, loc) ||
        !upload_q4(e, L.sh_up, w.sh_up, SL_MOE_I, H, loc) || !upload_q4(e, L.sh_down, w.sh_down, H, SL_MOE_I, loc))
      return SL_ERR_ARG;
    { const int r = alloc_layer_state(e, L); if (r) return r; }
  }
  if (has_head) {
    if (!upload_q4(e, e->embed, d->embed, d->vocab, H, loc) || !upload_q4(e, e->lm_head, d->lm_head, d->vocab, H, loc))
      return SL_ERR_ARG;
    e->final_norm = upload<uint16_t>(e, d->final_norm, H, loc);
    if (!e->final_norm) return SL_ERR_DEVICE;
  }
  return alloc_runtime(e);
}

namespace {
// Everything an engine needs besides weights and per-layer caches: scratch rows, head buffers, rope table,
// step state, the single-launch step's parameter blocks, pinned staging.
int alloc_runtime(sl_engine* e) {
  const int max_m = e->max_m, max_seq_len = e->max_seq, E = e->n_experts;
  const bool has_head = e->has_head;
  struct { int n_layers, vocab; } dd = {e->n_layers, e->vocab};
  const auto* d = &dd;
  SL_TRY(e, hipFuncSetAttribute((const void*)k_sdpa_merge_long, hipFuncAttributeMaxDynamicSharedMemorySize, MERGE_DYN_LDS));
  if (has_head) {
    e->n_cand = d->vocab / 16;
    e->logits = dalloc<uint16_t>(e, (size_t)max_m * d->vocab);
    e->cand_v = dalloc<float>(e, (size_t)max_m * e->n_cand + 1024);
    e->cand_i = dalloc<int32_t>(e, (size_t)max_m * e->n_cand + 1024);
    if (!e->logits || !e->cand_v || !e->cand_i) return SL_ERR_DEVICE;
  }
  if (e->has_attn) {
    std::vector<float> c, s;
    build_rope(c, s, max_seq_len);
    e->rope_cos = upload<float>(e, c.data(), c.size(), SL_LOC_HOST);
    e->rope_sin = upload<float>(e, s.data(), s.size(), SL_LOC_HOST);
    e->pm = dalloc<float>(e, (size_t)max_m * 16 * e->max_tiles);
    e->pl = dalloc<float>(e, (size_t)max_m * 16 * e->max_tiles);
    e->po = dalloc<float>(e, (size_t)max_m * 16 * e->max_tiles * 256);
    e->qrot = dalloc<uint16_t>(e, (size_t)max_m * 16 * 256);
    if (!e->rope_cos || !e->rope_sin || !e->pm || !e->pl || !e->po || !e->qrot) return SL_ERR_DEVICE;
  }
  const size_t MH = (size_t)max_m * H;
  e->hA = dalloc<uint16_t>(e, MH, true); e->hB = dalloc<uint16_t>(e, MH, true);
  e->proj = dalloc<uint16_t>(e, (size_t)max_m * PROJ_STRIDE, true);
  e->ycore = dalloc<uint16_t>(e, (size_t)max_m * 4096, true);
  e->mix = dalloc<uint16_t>(e, MH, true); e->xn = dalloc<uint16_t>(e, MH, true); e->xsum = dalloc<float>(e, (size_t)max_m * 64, true); e->ysum = dalloc<float>(e, (size_t)max_m * 128, true);
  if (max_m >= MOE_GROUP_MIN_ROWS) {               // exact steps of many rows run the experts' down stage by expert: results by pair, then the combine
    const size_t rows = (size_t)(max_m < GROUP_CAP ? max_m : GROUP_CAP);
    e->hy_d = dalloc<uint16_t>(e, rows * 8 * H); e->hy_sy = dalloc<uint16_t>(e, rows * H);
    if (!e->hy_d || !e->hy_sy) return SL_ERR_DEVICE;
  }
  e->rlogits = dalloc<uint16_t>(e, (size_t)max_m * 256, true); e->sgate = dalloc<uint16_t>(e, max_m, true);
  e->sh_act = dalloc<uint16_t>(e, (size_t)max_m * 512, true); e->act = dalloc<uint16_t>(e, (size_t)max_m * 8 * 512, true);
  e->hy_lists = dalloc<uint16_t>(e, (size_t)SL_MAX_EXPERTS * GROUP_CAP, true);
  e->hy_counts = dalloc<int32_t>(e, 2 * SL_MAX_EXPERTS, true);    // counts, then the experts ordered by falling count
  e->moe_out = dalloc<uint16_t>(e, MH, true); e->normed = dalloc<uint16_t>(e, MH, true);
  e->rows_out = dalloc<uint16_t>(e, MH, true);
  e->gdn_qn = dalloc<uint16_t>(e, MH, true); e->gdn_kn = dalloc<uint16_t>(e, MH, true);
  e->gdn_vc = dalloc<uint16_t>(e, (size_t)max_m * 4096, true); e->gdn_gb = dalloc<float>(e, (size_t)max_m * 64, true);
  if (!e->gdn_qn || !e->gdn_kn || !e->gdn_vc || !e->gdn_gb) return SL_ERR_DEVICE;
  e->tok_in = dalloc<int32_t>(e, max_m, true);
  e->tok_out = dalloc<int32_t>(e, max_m > MAX_CHAIN ? max_m : MAX_CHAIN, true);
  e->st = dalloc<int32_t>(e, 1 + d->n_layers, true);
  if (!e->hA || !e->hB || !e->proj || !e->ycore || !e->mix || !e->xn || !e->xsum || !e->ysum || !e->rlogits || !e->sgate || !e->sh_act || !e->act || !e->hy_lists || !e->hy_counts ||
      !e->moe_out || !e->normed || !e->rows_out || !e->tok_in || !e->tok_out || !e->st) return SL_ERR_DEVICE;
  {                                // (also for engines without a head: their block entry points use the single-launch stages)
    int ncu = 0;
    SL_TRY(e, hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, 0));
    if (ncu >= 256 && d->n_layers <= FLOW_MAX_LAYERS) {
      std::vector<LayerP> lp(d->n_layers);
      for (int i = 0; i < d->n_layers; ++i) {
        const LayerDev& L = e->layers[i];
        LayerP& q = lp[i];
        std::memset(&q, 0, sizeof(q));
        q.is_linear = L.is_linear; q.input_ln = L.input_ln; q.post_ln = L.post_ln;
        if (L.is_linear) {
          q.in_w = L.in_proj.w; q.in_sb = L.in_proj.sb; q.out_w = L.out_proj.w; q.out_sb = L.out_proj.sb;
          q.conv_w = L.conv_w; q.a_log = L.a_log; q.dt_bias = L.dt_bias; q.gdn_norm_w = L.gdn_norm_w; q.gdn_norm_f32 = L.norm_f32;
          q.hist[0] = L.hist[0]; q.hist[1] = L.hist[1]; q.state[0] = L.state[0]; q.state[1] = L.state[1];
        } else {
          q.in_w = L.qkv.w; q.in_sb = L.qkv.sb; q.out_w = L.o_proj.w; q.out_sb = L.o_proj.sb;
          q.q_norm = L.q_norm; q.k_norm = L.k_norm; q.kcache = L.kcache; q.vcache = L.vcache;
        }
        q.router_w = L.router_w; q.sgate_w = L.sgate_w;
        if (L.gate8_w) { q.router_w = reinterpret_cast<const uint16_t*>(L.gate8_w); q.sgate_w = reinterpret_cast<const uint16_t*>(L.gate8_sb); }
        q.swg_w = L.sw_gate.w; q.swg_sb = L.sw_gate.sb; q.swu_w = L.sw_up.w; q.swu_sb = L.sw_up.sb;
        q.swd_w = L.sw_down.w; q.swd_sb = L.sw_down.sb; q.shg_w = L.sh_gate.w; q.shg_sb = L.sh_gate.sb;
        q.shu_w = L.sh_up.w; q.shu_sb = L.sh_up.sb; q.shd_w = L.sh_down.w; q.shd_sb = L.sh_down.sb;
        q.route_inds = L.route_inds; q.route_scores = L.route_scores;
      }
      LayerP* dl = upload<LayerP>(e, lp.data(), lp.size(), SL_LOC_HOST);
      e->dec_bar = dalloc<unsigned>(e, 4096, true);
      if (!dl || !e->dec_bar) return SL_ERR_DEVICE;
      DecodeP P;
      std::memset(&P, 0, sizeof(P));
      P.n_layers = d->n_layers; P.E = E; P.vocab = d->vocab; P.max_seq = max_seq_len; P.max_tiles = e->max_tiles;
      P.layers = dl; P.lm_w = e->lm_head.w; P.lm_sb = e->lm_head.sb; P.emb_w = e->embed.w; P.emb_sb = e->embed.sb;
      P.final_norm = e->final_norm; P.rope_cos = e->rope_cos; P.rope_sin = e->rope_sin;
      P.hA = e->hA; P.normed = e->normed; P.logits = e->logits;
      P.tok_in = e->tok_in; P.tok_out = e->tok_out; P.st = e->st; P.bar = e->dec_bar;
      e->dec_tstamp = dalloc<uint32_t>(e, (size_t)256 * STAMP_WORDS, true);
      if (!e->dec_tstamp) return SL_ERR_DEVICE;
      P.tstamp = e->dec_tstamp;
      {
        FlowP F;
        std::memset(&F, 0, sizeof(F));
        F.d = P;
        auto tagged_words = [&](size_t n) {
          uint32_t* p = dalloc<uint32_t>(e, n, true);
          e->flow_tagged.emplace_back(p, n * sizeof(uint32_t));
          return p;
        };
        auto tagged_chunks = [&](size_t n) { return reinterpret_cast<uint4*>(tagged_words(4 * n)); };
        F.tproj = tagged_words(PROJ_STRIDE); F.tycore = tagged_words(4096);
        F.tmix = tagged_words(H); F.trlog = tagged_words(256); F.tsg = tagged_words(4);
        F.tsh = tagged_words(512); F.tact = tagged_words(8 * 512); F.tmoe = tagged_words(H);
        F.tml = tagged_chunks((size_t)SL_ATT_HEADS * e->max_tiles);
        F.tpo = tagged_chunks((size_t)SL_ATT_HEADS * e->max_tiles * 128);
        F.tcand = tagged_chunks(256);
        F.ttok = tagged_chunks(4);
        F.sdpa_round = SDPA_ROUND;
        F.spin_limit = FLOW_SPIN_LIMIT;
        F.xin = e->xn;
        if (const char* s = std::getenv("QWISP_SDPA_ROUND")) {      // smaller rounds, for tests of the round loop
          const int v = std::atoi(s);
          if (v >= 1 && v <= SDPA_ROUND) F.sdpa_round = v;
        }
        if (!F.tproj || !F.tycore || !F.tmix || !F.trlog || !F.tsg || !F.tsh || !F.tact || !F.tmoe ||
            !F.tml || !F.tpo || !F.tcand || !F.ttok) return SL_ERR_DEVICE;
        e->flow_host = F;
        e->flow_params = upload<FlowP>(e, &F, 1, SL_LOC_HOST);
        if (!e->flow_params) return SL_ERR_DEVICE;
        SL_TRY(e, hipFuncSetAttribute((const void*)k_decode_flow<false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
        SL_TRY(e, hipFuncSetAttribute((const void*)k_decode_flow<true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
        SL_TRY(e, hipFuncSetAttribute((const void*)k_decode_flow<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
        SL_TRY(e, hipFuncSetAttribute((const void*)k_decode_flow<true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
        SL_TRY(e, hipFuncSetAttribute((const void*)k_block_flow<false>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
        SL_TRY(e, hipFuncSetAttribute((const void*)k_block_flow<true>, hipFuncAttributeMaxDynamicSharedMemorySize, DEC_DYN_LDS));
      }
      // every workgroup of the grid must be resident at once: one per compute unit
      int per_cu = 0;
      SL_TRY(e, hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k_decode_flow<false, false>, DEC_THREADS, DEC_DYN_LDS));
      // (the merging workgroups keep every tile's {max, sum} in the key tile's LDS space: 4224 tiles = 270336 tokens;
      // beyond that the kernel-per-stage sequence runs)
      if (per_cu >= 1 && e->max_tiles <= SDPA_TILE * KT_STRIDE * 2 / 8) e->dec_grid = 256;
    }
  }
  e->pinned_bytes = MH * 2 + 4096 + (size_t)d->n_layers * 4 + (size_t)MAX_CHAIN * 4 + 64;
  SL_TRY(e, hipHostMalloc(&e->pinned, e->pinned_bytes, hipHostMallocDefault));
  SL_TRY(e, hipStreamSynchronize(e->stream));
  return SL_OK;
}
}  // namespace

// A further sequence ("lane") on the weights of `base`: own caches, scratch and stream; the weight pointers are
// shared and stay owned by `base`, which must outlive its lanes.
int sl_lane_create(const sl_engine* base, int max_m, int max_seq_len, sl_engine** out) {
  if (!base || !out || max_m < 1 || max_seq_len < 1) return SL_ERR_ARG;
  if (!base->fault.empty()) return SL_ERR_POISONED;
  {
    const sl_engine* root = base->base_of ? base->base_of : base;       // (a lane of a lane hangs on the root's weights)
    if (root->destroy_pending || !root->fault.empty()) return SL_ERR_POISONED;
  }
  std::lock_guard<std::recursive_mutex> gpu_lock_(g_gpu_mutex);
  sl_engine* e = new sl_engine();
  *out = e;
  e->n_layers = base->n_layers; e->n_experts = base->n_experts; e->vocab = base->vocab;
  e->max_m = max_m; e->max_seq = max_seq_len; e->max_tiles = (max_seq_len + SDPA_TILE - 1) / SDPA_TILE;
  e->has_head = base->has_head;
  e->parity.assign(e->n_layers, 0);
  e->device = base->device; e->na_scratch = base->na_scratch;
  SL_TRY(e, hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
  SL_TRY(e, hipEventCreate(&e->ev0));
  SL_TRY(e, hipEventCreate(&e->ev1));
  e->layers = base->layers;                       // weight pointers; the per-sequence ones are replaced below
  for (LayerDev& L : e->layers) {
    L.hist[0] = L.hist[1] = nullptr; L.state[0] = L.state[1] = nullptr;
    L.kcache = L.vcache = nullptr; L.route_inds = nullptr; L.route_scores = nullptr;
    const int r = alloc_layer_state(e, L); if (r) return r;
  }
  e->embed = base->embed; e->lm_head = base->lm_head; e->final_norm = base->final_norm; e->gate8 = base->gate8;
  sl_engine* root = const_cast<sl_engine*>(base->base_of ? base->base_of : base);   // a lane of a lane shares the root's weights
  e->base_of = root;
  root->lane_refs += 1;
  return alloc_runtime(e);
}

namespace {
// Lanes can be stepped as one batch of rows when they share weights and shapes with the driver (lanes[0]),
// whose scratch rows they then use.
bool lanes_batchable(sl_engine** lanes, int b) {
  sl_engine* d = lanes[0];
  if (b < 2 || b > d->max_m || !d->has_head) return false;
  for (int i = 0; i < b; ++i) {
    const sl_engine* l = lanes[i];
    if (l->n_layers != d->n_layers || l->max_seq != d->max_seq || l->lm_head.w != d->lm_head.w ||
        l->layers[0].router_w != d->layers[0].router_w || l->layers[0].gate8_w != d->layers[0].gate8_w) return false;
  }
  return true;
}
// Into how many groups a batch of lanes is dealt (lane i to group i % groups) that are stepped side by side
// (sl_lane_step_argmax); a group's first lane lends scratch rows and stream.  Two groups from 32 lanes on, so that a group
// keeps the 16 rows that the matrix-core kernels of hybrid mode want.  (Measured at 32 lanes of 1K-16K tokens: one group
// 9.83 ms per step of exact rows and 8.0 ms hybrid, two groups 9.1 and 7.8, four groups of 8 rows 14.9: kernels of
// 8 rows are too small to share the device, and there are 2000 of them.)
constexpr int LANE_GROUPS_MAX = 2, LANE_GROUP_ROWS = 16;
int lane_groups(sl_engine** lanes, int b) {
  if (b < 2 * LANE_GROUP_ROWS) return 1;
  // the second group's first lane (lanes[1]) must be able to drive its half
  const sl_engine* d1 = lanes[1];
  if (b / 2 > d1->max_m || !d1->has_head || d1->max_seq != lanes[0]->max_seq) return 1;
  return 2;
}
// Device table of the lanes' caches, [n_layers][max_m] in the driver; rebuilt when the set of lanes changes.
int bind_lanes(sl_engine* d, sl_engine** lanes, int b) {
  if ((int)d->lane_set.size() == b &&
      std::equal(d->lane_set.begin(), d->lane_set.end(), lanes, [](uint64_t u, const sl_engine* l) { return u == l->uid; })) return SL_OK;
  if (!d->lane_tab) {
    d->lane_tab = dalloc<LaneRef>(d, (size_t)d->n_layers * d->max_m, true);
    if (!d->lane_tab) return SL_ERR_DEVICE;
  }
  std::vector<LaneRef> tab((size_t)d->n_layers * d->max_m);
  std::memset(tab.data(), 0, tab.size() * sizeof(LaneRef));
  for (int li = 0; li < d->n_layers; ++li)
    for (int i = 0; i < b; ++i) {
      const LayerDev& L = lanes[i]->layers[li];
      LaneRef& r = tab[(size_t)li * d->max_m + i];
      r.hist[0] = L.hist[0]; r.hist[1] = L.hist[1]; r.state[0] = L.state[0]; r.state[1] = L.state[1];
      r.kcache = L.kcache; r.vcache = L.vcache; r.st = lanes[i]->st; r.max_seq = lanes[i]->max_seq;
    }
  int r = copy_sync(d, d->lane_tab, tab.data(), tab.size() * sizeof(LaneRef), hipMemcpyHostToDevice); if (r) return r;
  d->lane_set.clear();
  for (int i = 0; i < b; ++i) d->lane_set.push_back(lanes[i]->uid);
  return SL_OK;
}
}  // namespace

// One token per lane (reference: SeedlessLaneBatch.stepArgmaxBatch, SeedlessLaneBatch.swift:876).  When the lanes
// fit the scratch rows of lanes[0] (b <= its max_m, same weights and max_seq_len) the step runs as b rows through the
// kernel-per-stage path: every projection, expert and lm_head kernel sees all lanes in one launch, and only the
// recurrence and attention kernels go to each lane's own caches and position.  The arithmetic per row is that of
// a solo step, so per lane the result is bit-identical to stepping it alone.  Otherwise the lanes' single-launch
// steps are queued back to back.
int sl_lane_step_argmax(sl_engine** lanes, int b, const int32_t* tokens, int32_t* out) {
  if (!lanes || b < 1 || !tokens || !out) return SL_ERR_ARG;
  std::lock_guard<std::recursive_mutex> gpu_lock_(g_gpu_mutex);
  for (int i = 0; i < b; ++i) {
    if (!lanes[i]) return SL_ERR_ARG;
    for (int j = 0; j < i; ++j) if (lanes[j] == lanes[i]) return SL_ERR_ARG;
  }
  for (int i = 0; i < b; ++i) lanes[i]->normed_rows = 0;
  if (!lanes_batchable(lanes, b)) {
    for (int i = 0; i < b; ++i) { const int r = sl_step_argmax(lanes[i], tokens + i, 1, out + i); if (r) return r; }
    return SL_OK;
  }
  sl_engine* d = lanes[0];
  for (int i = 0; i < b; ++i) {
    int r = guard(lanes[i]); if (r) return r;
    if (tokens[i] < 0 || tokens[i] >= d->vocab) return SL_ERR_ARG;
    if (lanes[i]->has_attn && lanes[i]->pos + 1 > lanes[i]->max_seq) return SL_ERR_ARG;
  }
  // Two groups of lanes, each on the scratch rows and the stream of its first lane: the two launch sequences run
  // side by side on the device, so the short kernels of one group (norms, routing,
  // gates: a third of a step's launches, a few microseconds each and bound by nothing but their start and end) and the
  // ends of its large ones are covered by the other group's kernels.  The dense weights are streamed once per group
  // instead of once per step (5 % of a 32-lane step's bytes); what a lane computes does not change.
  // (Lane i goes to group i % 2: whatever order the caller keeps its lanes in, neighbours are dealt to both groups,
  // so a batch sorted by context length does not end up as a short group and a long one.)
  const int ng = lane_groups(lanes, b);
  std::vector<sl_engine*> grp[LANE_GROUPS_MAX];
  std::vector<int32_t> gtok[LANE_GROUPS_MAX];
  for (int i = 0; i < b; ++i) { grp[i % ng].push_back(lanes[i]); gtok[i % ng].push_back(tokens[i]); }
  int tiles[LANE_GROUPS_MAX];
  for (int g = 0; g < ng; ++g) {
    sl_engine* dg = grp[g][0];
    if (g > 0 && d->hybrid != dg->hybrid) { const int r = sl_set_hybrid(dg, d->hybrid ? 1 : 0); if (r) return r; }
    int max_pos = 0;
    for (const sl_engine* l : grp[g]) if (l->pos > max_pos) max_pos = l->pos;
    tiles[g] = (max_pos + 1 + SDPA_TILE - 1) / SDPA_TILE;
    const int r = bind_lanes(dg, grp[g].data(), (int)grp[g].size()); if (r) return r;
  }
  // work queued on the other lanes' own streams (none after a completed call) must not overlap this step
  for (int i = 1; i < b; ++i) SL_TRY(lanes[i], hipStreamSynchronize(lanes[i]->stream));
  SL_TRY(d, hipEventRecord(d->ev0, d->stream));
  for (int g = 0; g < ng; ++g) {
    sl_engine* dg = grp[g][0];
    const int n = (int)grp[g].size();
    const int r = to_device(dg, dg->tok_in, gtok[g].data(), (size_t)n * 4); if (r) return r;
    if (g > 0) SL_TRY(dg, hipStreamWaitEvent(dg->stream, d->ev0, 0));      // (the step's time is measured on the first group's stream)
    hipLaunchKernelGGL(k_embed, dim3(H / 256, n), dim3(256), 0, dg->stream, dg->tok_in, dg->embed.w, dg->embed.sb, dg->hA);
  }
  // (a host thread per further group: queueing a group's 500 launches takes 1.4 ms of host time, so both sequences
  // are on the device early in the step)
  hipError_t queued[LANE_GROUPS_MAX];
  auto queue_group = [&](int g) {
    sl_engine* dg = grp[g][0];
    const int n = (int)grp[g].size();
    if (g > 0) { (void)hipSetDevice(dg->device); (void)hipGetLastError(); }
    launch_layers(dg, n, dg->lane_tab, tiles[g]);
    HiddenArgs ha{dg->hA, dg->moe_out, dg->final_norm, dg->hB, dg->normed};
    launch_head(dg, n, ha, 0, false);
    hipLaunchKernelGGL(k_lane_advance, dim3(n), dim3(64), 0, dg->stream, dg->lane_tab, dg->n_layers);
    queued[g] = g > 0 ? hipGetLastError() : hipSuccess;   // (a helper's launch errors are its thread's: handed back here)
  };
  {
    std::vector<std::thread> helpers;
    int started = 1;
    try {
      for (int g = 1; g < ng; ++g) { helpers.emplace_back(queue_group, g); started = g + 1; }
    } catch (const std::system_error&) {
      // no thread to be had: the groups not handed to one are queued from this thread, after its own
    }
    queue_group(0);
    for (int g = started; g < ng; ++g) queue_group(g);
    for (auto& t : helpers) t.join();
  }
  for (int g = 1; g < ng; ++g)
    if (!ok(d, queued[g], "stepArgmaxBatch (second group)")) {
      for (int h = 0; h < ng; ++h) (void)hipStreamSynchronize(grp[h][0]->stream);
      for (int i = 1; i < b; ++i) if (lanes[i]->fault.empty()) lanes[i]->fault = d->fault;
      return SL_ERR_DEVICE;
    }
  for (int g = 1; g < ng; ++g) {                         // the first group's stream ends the step: it waits for the others
    sl_engine* dg = grp[g][0];
    SL_TRY(dg, hipEventRecord(dg->ev1, dg->stream));
    SL_TRY(d, hipStreamWaitEvent(d->stream, dg->ev1, 0));
  }
  SL_TRY(d, hipEventRecord(d->ev1, d->stream));
  int r = SL_OK;
  for (int g = 0; g < ng && !r; ++g) {
    sl_engine* dg = grp[g][0];
    r = read_back(dg, gtok[g].data(), dg->tok_out, grp[g].size() * 4, "stepArgmaxBatch");
    if (r && d->fault.empty()) d->fault = dg->fault;
  }
  if (r) {   // the lanes' caches were written by the failed step: all of them are unusable
    for (int g = 1; g < ng; ++g) (void)hipStreamSynchronize(grp[g][0]->stream);
    for (int i = 1; i < b; ++i) if (lanes[i]->fault.empty()) lanes[i]->fault = d->fault;
    return r;
  }
  time_end(d);
  for (int i = 0; i < b; ++i) {
    sl_engine* l = lanes[i];
    sl_engine* dg = grp[i % ng][0];
    const int row = i / ng;
    out[i] = gtok[i % ng][row];
    l->pos += 1;
    for (int j = 0; j < l->n_layers; ++j) if (l->layers[j].is_linear) l->parity[j] ^= 1;
    l->logits_view = dg->logits + (size_t)row * dg->vocab;
    l->normed_view = dg->normed + (size_t)row * H;
    l->last_ms = d->last_ms;
  }
  return SL_OK;
}

// Sampling is outside this build (greedy only); Tell falls back to its own sampler on "unsupported".
int sl_step_sample_rows(sl_engine* e, const int32_t* tokens, int m, float temperature, float top_p, uint64_t seed, int32_t* out) {
  (void)tokens; (void)m; (void)temperature; (void)top_p; (void)seed; (void)out;
  SL_ENTER(e);
  return SL_ERR_UNSUPPORTED;
}

void sl_destroy(sl_engine* e) {
  if (!e) return;
  std::lock_guard<std::recursive_mutex> gpu_lock_(g_gpu_mutex);
  if (e->lane_refs > 0) {            // lanes still read these weights: the memory goes with the last of them
    if (e->stream) (void)hipStreamSynchronize(e->stream);
    e->destroy_pending = true;
    if (e->fault.empty()) e->fault = "engine destroyed (kept alive by its lanes)";
    return;
  }
  sl_engine* root = e->base_of;
  if (e->stream) (void)hipStreamSynchronize(e->stream);
  for (void* p : e->allocs) (void)hipFree(p);
  if (e->pinned) (void)hipHostFree(e->pinned);
  for (hipEvent_t ev : e->head_ev) (void)hipEventDestroy(ev);
  if (e->side_fork) (void)hipEventDestroy(e->side_fork);
  if (e->side_join) (void)hipEventDestroy(e->side_join);
  if (e->side) { (void)hipStreamSynchronize(e->side); (void)hipStreamDestroy(e->side); }
  if (e->ev0) (void)hipEventDestroy(e->ev0);
  if (e->ev1) (void)hipEventDestroy(e->ev1);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  delete e;
  if (root && --root->lane_refs == 0 && root->destroy_pending) sl_destroy(root);
}

const char* sl_fault(const sl_engine* e) { return (e && !e->fault.empty()) ? e->fault.c_str() : nullptr; }
void sl_inject_failure(sl_engine* e) { if (e) e->inject_failure = true; }
int sl_position(const sl_engine* e) { return e ? e->pos : -1; }
int sl_max_rows(const sl_engine* e) { return e ? e->max_m : -1; }
float sl_last_gpu_ms(const sl_engine* e) { return e ? e->last_ms : 0.0f; }
void* sl_stream(sl_engine* e) { return e ? (void*)e->stream : nullptr; }
int sl_set_hybrid(sl_engine* e, int enable) {
  SL_ENTER(e);
  if (enable && !e->hy_sg) {
    const size_t rows = (size_t)(e->max_m < GROUP_CAP ? e->max_m : GROUP_CAP);
    if (!e->hy_d) e->hy_d = dalloc<uint16_t>(e, rows * 8 * H);        // (engines of 128 rows or more have these two already)
    e->hy_sg = dalloc<uint16_t>(e, rows * SL_MOE_I); e->hy_su = dalloc<uint16_t>(e, rows * SL_MOE_I);
    if (!e->hy_sy) e->hy_sy = dalloc<uint16_t>(e, rows * H);
    if (!e->hy_d || !e->hy_sg || !e->hy_su || !e->hy_sy) return SL_ERR_DEVICE;
    if (rows >= GC) {
      e->gc_scratch = dalloc<unsigned char>(e, (rows / GC) * SL_GDN_HV * GC_UNIT_BYTES);
      if (!e->gc_scratch) return SL_ERR_DEVICE;
      SL_TRY(e, hipFuncSetAttribute((const void*)k_gdn_chunk_scan, hipFuncAttributeMaxDynamicSharedMemorySize, GC_SCAN_LDS));
    }
    SL_TRY(e, hipStreamSynchronize(e->stream));
  }
  if (enable && !e->side) {
    SL_TRY(e, hipStreamCreateWithFlags(&e->side, hipStreamNonBlocking));
    SL_TRY(e, hipEventCreateWithFlags(&e->side_fork, hipEventDisableTiming));
    SL_TRY(e, hipEventCreateWithFlags(&e->side_join, hipEventDisableTiming));
  }
  e->hybrid = enable != 0;
  return SL_OK;
}
int sl_set_persistent(sl_engine* e, int enable) {
  SL_ENTER(e);
  e->use_persistent = enable != 0;
  return SL_OK;
}
// Diagnostic hook: while enabled, batch-1 steps run the stamping variant of the single-launch kernel, in which every
// workgroup records 100 MHz clock stamps of the last step of a launch; the call copies them out,
// out[wg * sl_stage_clock_words() + (layer * 8 + stage) * 8 + kind] (0 = not reached).
int sl_debug_stage_clock(sl_engine* e, int enable, uint32_t* out, int cap_words) {
  // (reading the stamps is allowed on an engine whose last launch gave up: they show where every workgroup stood)
  std::lock_guard<std::recursive_mutex> gpu_lock_(g_gpu_mutex);
  if (!e) return SL_ERR_ARG;
  if (!e->fault.empty() && (enable || !out)) return SL_ERR_POISONED;
  int r = SL_OK;
  if (!e->flow_params) return SL_ERR_UNSUPPORTED;
  if (out && cap_words > 0) {
    const size_t n = std::min<size_t>((size_t)cap_words, (size_t)e->dec_grid * STAMP_WORDS);
    r = copy_sync(e, out, e->dec_tstamp, n * 4, hipMemcpyDeviceToHost); if (r) return r;
  }
  e->stage_clock = enable != 0;
  return SL_OK;
}
int sl_stage_clock_words(void) { return STAMP_WORDS; }
// Test hook in the manner of injectCBFailure (SFV:404): the number of polling rounds after which a workgroup of the
// single-launch step stops waiting, raises the abort word and leaves (every workgroup then does the same at its next
// wait, so the kernel ends normally).  0 makes the first unanswered poll give up.
int sl_debug_set_spin_limit(sl_engine* e, unsigned rounds) {
  SL_ENTER(e);
  if (!e->flow_params) return SL_ERR_UNSUPPORTED;
  e->flow_host.spin_limit = rounds;
  return copy_sync(e, e->flow_params, &e->flow_host, sizeof(FlowP), hipMemcpyHostToDevice);
}
// Test hook: moves the stage-instance counter (device word and host mirror) so that a test can step an engine across
// the point where the counter is rebased without running millions of steps first.
int sl_debug_set_flow_counter(sl_engine* e, uint32_t value) {
  SL_ENTER(e);
  if (!e->flow_params) return SL_ERR_UNSUPPORTED;
  e->flow_base = value;
  return copy_sync(e, e->dec_bar + 16, &value, 4, hipMemcpyHostToDevice);
}
// The tags of stage instance (layer, stage) at counter value `base`, and whether a launch of `steps` steps from there
// is preceded by a rebase: pure functions of their arguments (no device needed).
int sl_debug_flow_tags(uint32_t base, int layer, int stage, int steps, int n_layers, uint32_t* tag16, uint32_t* tag32) {
  if (tag16) *tag16 = flow_tag(base, layer, stage);
  if (tag32) *tag32 = flow_tag32(base, layer, stage);
  return flow_rebase_needed(base, steps, n_layers) ? 1 : 0;
}
int sl_profile_head(sl_engine* e, int enable) {
  SL_ENTER(e);
  if (enable && e->head_ev.empty()) {
    e->head_ev.resize(2 * MAX_CHAIN, nullptr);
    for (auto& ev : e->head_ev) SL_TRY(e, hipEventCreate(&ev));
  }
  e->profile_head = enable != 0;
  e->head_pending = 0; e->head_ms_sum = 0.0; e->head_launches = 0;
  return SL_OK;
}
int sl_profile_head_read(sl_engine* e, double* ms_sum, int64_t* launches) {
  if (!e || !ms_sum || !launches) return SL_ERR_ARG;
  *ms_sum = e->head_ms_sum; *launches = e->head_launches;
  return SL_OK;
}

// abort_word: after a persistent step, the word a workgroup that gave up waiting leaves set comes back with the same
// synchronisation (the last 64 bytes of the pinned buffer are kept for it).
static int read_back(sl_engine* e, void* dst, const void* dev, size_t bytes, const char* what, bool abort_word) {
  if (bytes > e->pinned_bytes - 64) return SL_ERR_ARG;
  unsigned char* flag_at = (unsigned char*)e->pinned + e->pinned_bytes - 64;
  SL_TRY(e, hipMemcpyAsync(e->pinned, dev, bytes, hipMemcpyDeviceToHost, e->stream));
  if (abort_word) SL_TRY(e, hipMemcpyAsync(flag_at, e->dec_bar + 32, 4, hipMemcpyDeviceToHost, e->stream));
  int r = finish(e, what);
  if (r) return r;
  if (abort_word) {
    unsigned flag = 0;
    std::memcpy(&flag, flag_at, 4);
    if (flag) {      // (the word names the wait that gave up first: 1 = a stage's hand-over, 16 + n = wait n of the attention merge)
      if (e->fault.empty()) e->fault = "persistent decode kernel: grid barrier timed out (wait " + std::to_string(flag) + ")";
      return SL_ERR_DEVICE;
    }
  }
  std::memcpy(dst, e->pinned, bytes);
  return SL_OK;
}
// The 2048-long result of a single-block launch: halves with their 16-bit tags, checked and stripped here.
static int read_back_tagged(sl_engine* e, uint16_t* out, const uint32_t* words, uint32_t tag, const char* what) {
  std::vector<uint32_t> w(H);
  const int r = read_back(e, w.data(), words, (size_t)H * 4, what, true);
  if (r) return r;
  for (int i = 0; i < H; ++i) {
    if ((w[i] >> 16) != tag) {
      if (e->fault.empty()) e->fault = std::string(what) + ": single-block launch left an incomplete result";
      return SL_ERR_DEVICE;
    }
    out[i] = (uint16_t)(w[i] & 0xffffu);
  }
  return SL_OK;
}
static void time_end(sl_engine* e) {
  float ms = 0.0f;
  if (hipEventElapsedTime(&ms, e->ev0, e->ev1) == hipSuccess) e->last_ms = ms;
  for (int i = 0; i < e->head_pending; ++i)
    if (hipEventElapsedTime(&ms, e->head_ev[2 * i], e->head_ev[2 * i + 1]) == hipSuccess) { e->head_ms_sum += ms; e->head_launches += 1; }
  e->head_pending = 0;
}

int sl_step_argmax(sl_engine* e, const int32_t* tokens, int m, int32_t* out) {
  SL_ENTER(e);
  e->normed_rows = 0;
  e->logits_view = e->normed_view = nullptr;
  if (!tokens || !out || !e->has_head) return SL_ERR_ARG;
  r = check_rows(e, m); if (r) return r;
  for (int i = 0; i < m; ++i) if (tokens[i] < 0 || tokens[i] >= e->vocab) return SL_ERR_ARG;
  r = to_device(e, e->tok_in, tokens, (size_t)m * 4); if (r) return r;
  const bool persistent = (m == 1 && e->dec_grid > 0 && e->use_persistent);
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  if (persistent) {
    launch_decode(e, 0, false, 1);
  } else {
    hipLaunchKernelGGL(k_embed, dim3(H / 256, m), dim3(256), 0, e->stream, e->tok_in, e->embed.w, e->embed.sb, e->hA);
    launch_layers(e, m);
    HiddenArgs ha{e->hA, e->moe_out, e->final_norm, e->hB, e->normed};
    launch_head(e, m, ha, 0, false);
    advance(e, m);
  }
  SL_TRY(e, hipEventRecord(e->ev1, e->stream));
  r = read_back(e, out, e->tok_out, (size_t)m * 4, "stepArgmax", persistent); if (r) return r;
  time_end(e);
  return SL_OK;
}

int sl_chained_step_argmax(sl_engine* e, int32_t first, int k, int32_t* out) {
  SL_ENTER(e);
  e->normed_rows = 0;
  e->logits_view = e->normed_view = nullptr;
  if (!out || !e->has_head || k < 1 || k > MAX_CHAIN || first < 0 || first >= e->vocab) return SL_ERR_ARG;
  if (e->has_attn && e->pos + k > e->max_seq) return SL_ERR_ARG;
  r = to_device(e, e->tok_in, &first, 4); if (r) return r;
  const bool persistent = (e->dec_grid > 0 && e->use_persistent);
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  if (persistent) launch_decode(e, 0, true, k);        // the whole chain in one launch
  for (int s = 0; s < k && !persistent; ++s) {
    hipLaunchKernelGGL(k_embed, dim3(H / 256, 1), dim3(256), 0, e->stream, e->tok_in, e->embed.w, e->embed.sb, e->hA);
    launch_layers(e, 1);
    HiddenArgs ha{e->hA, e->moe_out, e->final_norm, e->hB, e->normed};
    launch_head(e, 1, ha, s, true);
    advance(e, 1);
  }
  SL_TRY(e, hipEventRecord(e->ev1, e->stream));
  r = read_back(e, out, e->tok_out, (size_t)k * 4, "chainedStepArgmax", persistent); if (r) return r;
  time_end(e);
  return SL_OK;
}

static int forward_common(sl_engine* e, int m, int final_norm, uint16_t* out, const char* what) {
  e->logits_view = e->normed_view = nullptr;
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  launch_layers(e, m);
  HiddenArgs ha{e->hA, e->moe_out, final_norm ? e->final_norm : nullptr, final_norm ? e->hB : e->rows_out,
                final_norm ? e->normed : nullptr};
  hipLaunchKernelGGL(k_final_rows, dim3(m), dim3(64), 0, e->stream, ha);
  advance(e, m);
  SL_TRY(e, hipEventRecord(e->ev1, e->stream));
  // out == nullptr: the rows stay on the device (the reference's forward returns a device array, and a prefill only
  // ever looks at the last row of the last chunk); sl_hidden_rows / sl_head_argmax_rows read them later
  int r = out ? read_back(e, out, final_norm ? e->normed : e->rows_out, (size_t)m * H * 2, what) : finish(e, what);
  if (r) return r;
  e->normed_rows = final_norm ? m : 0;
  time_end(e);
  return SL_OK;
}
int sl_forward_rows(sl_engine* e, const uint16_t* x, int m, int final_norm, uint16_t* out) {
  SL_ENTER(e);
  if (!x || !out || (final_norm && !e->final_norm)) return SL_ERR_ARG;
  r = check_rows(e, m); if (r) return r;
  r = to_device(e, e->hA, x, (size_t)m * H * 2); if (r) return r;
  return forward_common(e, m, final_norm, out, "forwardRows");
}
int sl_forward_tokens(sl_engine* e, const int32_t* tokens, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!tokens || !e->has_head) return SL_ERR_ARG;
  r = check_rows(e, m); if (r) return r;
  for (int i = 0; i < m; ++i) if (tokens[i] < 0 || tokens[i] >= e->vocab) return SL_ERR_ARG;
  r = to_device(e, e->tok_in, tokens, (size_t)m * 4); if (r) return r;
  hipLaunchKernelGGL(k_embed, dim3(H / 256, m), dim3(256), 0, e->stream, e->tok_in, e->embed.w, e->embed.sb, e->hA);
  return forward_common(e, m, 1, out, "forward");
}
int sl_hidden_rows(sl_engine* e, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!out || m < 1 || m > e->max_m) return SL_ERR_ARG;
  if (e->normed_view) {   // after a lane-batched step: this lane's one row, held by the driver
    if (m != 1) return SL_ERR_ARG;
    return read_back(e, out, e->normed_view, (size_t)H * 2, "hiddenRows");
  }
  return read_back(e, out, e->normed, (size_t)m * H * 2, "hiddenRows");
}
int sl_logits_row(sl_engine* e, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!out || !e->has_head || m < 0 || m >= e->max_m) return SL_ERR_ARG;
  if (e->logits_view && m != 0) return SL_ERR_ARG;   // after a lane-batched step a lane has one row
  const uint16_t* src = e->logits_view ? e->logits_view : e->logits + (size_t)m * e->vocab;
  r = copy_sync(e, out, src, (size_t)e->vocab * 2, hipMemcpyDeviceToHost);
  return r;
}
int sl_head_argmax(sl_engine* e, const uint16_t* normed, int m, int32_t* out) {
  SL_ENTER(e);
  if (!normed || !out || !e->has_head || m < 1 || m > e->max_m) return SL_ERR_ARG;
  e->logits_view = e->normed_view = nullptr;      // the logits this call leaves are the engine's own rows
  r = to_device(e, e->xn, normed, (size_t)m * H * 2); if (r) return r;
  HiddenArgs ha{e->xn, nullptr, nullptr, nullptr, nullptr};
  launch_head(e, m, ha, 0, false);
  return read_back(e, out, e->tok_out, (size_t)m * 4, "headArgmax");
}

// lm_head + arg-max of rows first .. first + m - 1 of the normed rows that the last sl_forward_tokens / sl_forward_rows
// (with final norm) left on the device: the first token after a prefill without the rows' trip to the host and back.
int sl_head_argmax_rows(sl_engine* e, int first, int m, int32_t* out) {
  SL_ENTER(e);
  if (!out || !e->has_head || m < 1 || first < 0 || first + m > e->normed_rows) return SL_ERR_ARG;
  e->logits_view = e->normed_view = nullptr;
  HiddenArgs ha{e->normed + (size_t)first * H, nullptr, nullptr, nullptr, nullptr};
  launch_head(e, m, ha, 0, false);
  return read_back(e, out, e->tok_out, (size_t)m * 4, "headArgmaxRows");
}

// lm_head + arg-max for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that
// forbid it): device pointers in and out, the caller's stream, no allocation, copy or synchronisation.  The logits
// rows and arg-max candidates live in this device's copy of the fixed `scratch` array, which every call on the
// device shares: calls that overlap on one GPU race.  Every word the reduction reads is written by the same call,
// so nothing has to be cleared.
int sl_head_argmax_noalloc(sl_engine* e, const uint16_t* normed_dev, int m, int32_t* out_dev, void* stream) {
  int r = guard(e); if (r) return r;
  if (!normed_dev || !out_dev || !e->has_head || m < 1) return SL_ERR_ARG;
  if (m > NA_MAX_ROWS || e->vocab > NA_MAX_VOCAB) return SL_ERR_TOO_LARGE;
  if (!e->na_scratch) return SL_ERR_DEVICE;
  hipStream_t st = (hipStream_t)stream;
  (void)hipGetLastError();            // an error an unrelated earlier call of this thread left behind is not this call's
  uint16_t* logits = reinterpret_cast<uint16_t*>(e->na_scratch);
  float* cand_v = reinterpret_cast<float*>(static_cast<unsigned char*>(e->na_scratch) + NA_LOGITS_BYTES);
  int32_t* cand_i = reinterpret_cast<int32_t*>(cand_v + NA_CAND);
  const int n_cand = e->vocab / 16;
  if (m >= 2) {
    hipLaunchKernelGGL((k_qmv_tile<1, 4, 8, false, true>), dim3(n_cand, (m + 7) / 8), dim3(256), 0, st, HiddenArgs{}, normed_dev, H,
                       e->lm_head.w, e->lm_head.sb, e->vocab, logits, e->vocab, m, cand_v, cand_i);
  } else {
    HiddenArgs ha{normed_dev, nullptr, nullptr, nullptr, nullptr};
    hipLaunchKernelGGL(k_head, dim3(n_cand, 1), dim3(256), 0, st, ha, e->lm_head.w, e->lm_head.sb, e->vocab, logits, cand_v, cand_i);
  }
  hipLaunchKernelGGL(k_argmax_final, dim3(m), dim3(256), 0, st, cand_v, cand_i, n_cand, out_dev, 0, (int32_t*)nullptr);
  return hipGetLastError() == hipSuccess ? SL_OK : SL_ERR_DEVICE;
}

int sl_snapshot(sl_engine* e, sl_snap* s) {
  SL_ENTER(e);
  if (!s) return SL_ERR_ARG;
  s->kv_len = e->pos; s->reserved = 0;
  return SL_OK;
}
int sl_rollback_one_step(sl_engine* e, const sl_snap* s) {
  SL_ENTER(e);
  if (!s || s->kv_len < 0 || s->kv_len > e->pos) return SL_ERR_ARG;
  e->pos = s->kv_len;
  for (int i = 0; i < e->n_layers; ++i) if (e->layers[i].is_linear) e->parity[i] ^= 1;
  return push_state(e);
}
int sl_reset(sl_engine* e) {
  SL_ENTER(e);
  for (LayerDev& L : e->layers) {
    if (!L.is_linear) continue;
    for (int p = 0; p < 2; ++p) {
      SL_TRY(e, hipMemsetAsync(L.hist[p], 0, HIST_ELEMS * sizeof(uint16_t), e->stream));
      SL_TRY(e, hipMemsetAsync(L.state[p], 0, STATE_ELEMS * sizeof(float), e->stream));
    }
  }
  e->pos = 0;
  e->parity.assign(e->n_layers, 0);
  e->logits_view = e->normed_view = nullptr;
  return push_state(e);
}
int sl_full_snapshot(sl_engine* e, sl_full_snap** out) {
  SL_ENTER(e);
  if (!out) return SL_ERR_ARG;
  sl_full_snap* s = new sl_full_snap();
  s->pos = e->pos;
  s->hist.assign(e->n_layers, nullptr); s->state.assign(e->n_layers, nullptr);
  *out = s;
  for (int i = 0; i < e->n_layers; ++i) {
    LayerDev& L = e->layers[i];
    if (!L.is_linear) continue;
    SL_TRY(e, hipMalloc((void**)&s->hist[i], HIST_ELEMS * 2));
    SL_TRY(e, hipMalloc((void**)&s->state[i], STATE_ELEMS * 4));
    SL_TRY(e, hipMemcpyAsync(s->hist[i], L.hist[e->parity[i]], HIST_ELEMS * 2, hipMemcpyDeviceToDevice, e->stream));
    SL_TRY(e, hipMemcpyAsync(s->state[i], L.state[e->parity[i]], STATE_ELEMS * 4, hipMemcpyDeviceToDevice, e->stream));
  }
  SL_TRY(e, hipStreamSynchronize(e->stream));
  return SL_OK;
}
int sl_full_restore(sl_engine* e, const sl_full_snap* s) {
  SL_ENTER(e);
  if (!s || (int)s->hist.size() != e->n_layers) return SL_ERR_ARG;
  for (int i = 0; i < e->n_layers; ++i) {
    LayerDev& L = e->layers[i];
    if (!L.is_linear) continue;
    if (!s->hist[i] || !s->state[i]) return SL_ERR_ARG;
    SL_TRY(e, hipMemcpyAsync(L.hist[e->parity[i]], s->hist[i], HIST_ELEMS * 2, hipMemcpyDeviceToDevice, e->stream));
    SL_TRY(e, hipMemcpyAsync(L.state[e->parity[i]], s->state[i], STATE_ELEMS * 4, hipMemcpyDeviceToDevice, e->stream));
  }
  e->pos = s->pos;
  return push_state(e);
}
void sl_full_snap_free(sl_full_snap* s) {
  if (!s) return;
  for (auto p : s->hist) if (p) (void)hipFree(p);
  for (auto p : s->state) if (p) (void)hipFree(p);
  delete s;
}

// "QWS1" blob, little-endian (layout of persistentStateData, SeedlessFusedVerify.swift:4077-4111):
// magic, format, nLayers, then per layer: flags (bit0 KV, bit1 GDN); KV: u32 KV, D, len, K bytes
// (per head the used rows), V bytes; GDN: u32 convCount, stateCount, history bytes, state bytes.
static const uint32_t PERSIST_MAGIC = 0x31535751u, PERSIST_FORMAT = 1u;
size_t sl_persist_size(sl_engine* e) {
  if (!e) return 0;
  size_t n = 12;
  for (auto& L : e->layers) {
    n += 4;
    if (L.is_linear) n += 8 + HIST_ELEMS * 2 + STATE_ELEMS * 4;
    else n += 12 + 2 * (size_t)SL_ATT_KV * e->pos * SL_ATT_D * 2;
  }
  return n;
}
int sl_persist_write(sl_engine* e, void* dst, size_t cap) {
  SL_ENTER(e);
  if (!dst || cap < sl_persist_size(e)) return SL_ERR_ARG;
  uint8_t* p = (uint8_t*)dst;
  auto u32 = [&](uint32_t v) { std::memcpy(p, &v, 4); p += 4; };
  u32(PERSIST_MAGIC); u32(PERSIST_FORMAT); u32((uint32_t)e->n_layers);
  for (int i = 0; i < e->n_layers; ++i) {
    LayerDev& L = e->layers[i];
    u32(L.is_linear ? 2u : 1u);
    if (!L.is_linear) {
      u32(SL_ATT_KV); u32(SL_ATT_D); u32((uint32_t)e->pos);
      const size_t rb = (size_t)e->pos * SL_ATT_D * 2;
      for (uint16_t* buf : {L.kcache, L.vcache})
        for (int h = 0; h < SL_ATT_KV; ++h) {
          if (rb) { r = copy_sync(e, p, buf + (size_t)h * e->max_seq * SL_ATT_D, rb, hipMemcpyDeviceToHost); if (r) return r; }
          p += rb;
        }
    } else {
      u32((uint32_t)HIST_ELEMS); u32((uint32_t)STATE_ELEMS);
      r = copy_sync(e, p, L.hist[e->parity[i]], HIST_ELEMS * 2, hipMemcpyDeviceToHost); if (r) return r;
      p += HIST_ELEMS * 2;
      r = copy_sync(e, p, L.state[e->parity[i]], STATE_ELEMS * 4, hipMemcpyDeviceToHost); if (r) return r;
      p += STATE_ELEMS * 4;
    }
  }
  return SL_OK;
}
int sl_persist_restore(sl_engine* e, const void* src, size_t len) {
  SL_ENTER(e);
  if (!src) return SL_ERR_ARG;
  const uint8_t* p = (const uint8_t*)src;
  const uint8_t* end = p + len;
  auto u32 = [&](uint32_t& v) { if (end - p < 4) return false; std::memcpy(&v, p, 4); p += 4; return true; };
  uint32_t v = 0;
  if (!u32(v) || v != PERSIST_MAGIC || !u32(v) || v != PERSIST_FORMAT || !u32(v) || v != (uint32_t)e->n_layers) return SL_ERR_FORMAT;
  int new_pos = e->has_attn ? -1 : e->pos;
  for (int i = 0; i < e->n_layers; ++i) {
    LayerDev& L = e->layers[i];
    if (!u32(v) || v != (L.is_linear ? 2u : 1u)) return SL_ERR_FORMAT;
    if (!L.is_linear) {
      uint32_t kv = 0, dd = 0, ln = 0;
      if (!u32(kv) || kv != SL_ATT_KV || !u32(dd) || dd != SL_ATT_D || !u32(ln) || ln > (uint32_t)e->max_seq) return SL_ERR_FORMAT;
      if (new_pos >= 0 && (uint32_t)new_pos != ln) return SL_ERR_FORMAT;
      new_pos = (int)ln;
      const size_t rb = (size_t)ln * SL_ATT_D * 2;
      for (uint16_t* buf : {L.kcache, L.vcache})
        for (int h = 0; h < SL_ATT_KV; ++h) {
          if ((size_t)(end - p) < rb) return SL_ERR_FORMAT;
          if (rb) { r = copy_sync(e, buf + (size_t)h * e->max_seq * SL_ATT_D, p, rb, hipMemcpyHostToDevice); if (r) return r; }
          p += rb;
        }
    } else {
      uint32_t cc = 0, sc = 0;
      if (!u32(cc) || cc != HIST_ELEMS || !u32(sc) || sc != STATE_ELEMS) return SL_ERR_FORMAT;
      if ((size_t)(end - p) < HIST_ELEMS * 2 + STATE_ELEMS * 4) return SL_ERR_FORMAT;
      r = copy_sync(e, L.hist[e->parity[i]], p, HIST_ELEMS * 2, hipMemcpyHostToDevice); if (r) return r;
      p += HIST_ELEMS * 2;
      r = copy_sync(e, L.state[e->parity[i]], p, STATE_ELEMS * 4, hipMemcpyHostToDevice); if (r) return r;
      p += STATE_ELEMS * 4;
    }
  }
  if (p != end) return SL_ERR_FORMAT;
  if (new_pos >= 0) e->pos = new_pos;
  return push_state(e);
}

int sl_read_layer_cache(sl_engine* e, int layer, void* a, void* b) {
  SL_ENTER(e);
  if (layer < 0 || layer >= e->n_layers) return SL_ERR_ARG;
  LayerDev& L = e->layers[layer];
  if (L.is_linear) {
    if (a) { r = copy_sync(e, a, L.hist[e->parity[layer]], HIST_ELEMS * 2, hipMemcpyDeviceToHost); if (r) return r; }
    if (b) { r = copy_sync(e, b, L.state[e->parity[layer]], STATE_ELEMS * 4, hipMemcpyDeviceToHost); if (r) return r; }
  } else {
    const size_t rb = (size_t)e->pos * SL_ATT_D * 2;
    for (int h = 0; h < SL_ATT_KV && rb; ++h) {
      if (a) { r = copy_sync(e, (uint8_t*)a + h * rb, L.kcache + (size_t)h * e->max_seq * SL_ATT_D, rb, hipMemcpyDeviceToHost); if (r) return r; }
      if (b) { r = copy_sync(e, (uint8_t*)b + h * rb, L.vcache + (size_t)h * e->max_seq * SL_ATT_D, rb, hipMemcpyDeviceToHost); if (r) return r; }
    }
  }
  return SL_OK;
}
int sl_load_layer_cache(sl_engine* e, int layer, const void* a, const void* b, int len) {
  SL_ENTER(e);
  if (layer < 0 || layer >= e->n_layers) return SL_ERR_ARG;
  LayerDev& L = e->layers[layer];
  if (L.is_linear) {
    if (a) { r = copy_sync(e, L.hist[e->parity[layer]], a, HIST_ELEMS * 2, hipMemcpyHostToDevice); if (r) return r; }
    if (b) { r = copy_sync(e, L.state[e->parity[layer]], b, STATE_ELEMS * 4, hipMemcpyHostToDevice); if (r) return r; }
    return SL_OK;
  }
  if (len < 0 || len > e->max_seq) return SL_ERR_ARG;
  const size_t rb = (size_t)len * SL_ATT_D * 2;
  for (int h = 0; h < SL_ATT_KV && rb; ++h) {
    if (a) { r = copy_sync(e, L.kcache + (size_t)h * e->max_seq * SL_ATT_D, (const uint8_t*)a + h * rb, rb, hipMemcpyHostToDevice); if (r) return r; }
    if (b) { r = copy_sync(e, L.vcache + (size_t)h * e->max_seq * SL_ATT_D, (const uint8_t*)b + h * rb, rb, hipMemcpyHostToDevice); if (r) return r; }
  }
  e->pos = len;
  return push_state(e);
}

int sl_read_route(sl_engine* e, int layer, int m, int32_t* inds, uint16_t* scores) {
  SL_ENTER(e);
  if (layer < 0 || layer >= e->n_layers || m < 1 || m > e->max_m) return SL_ERR_ARG;
  if (inds) { r = copy_sync(e, inds, e->layers[layer].route_inds, (size_t)m * 32, hipMemcpyDeviceToHost); if (r) return r; }
  if (scores) { r = copy_sync(e, scores, e->layers[layer].route_scores, (size_t)m * 16, hipMemcpyDeviceToHost); if (r) return r; }
  return SL_OK;
}

// ---- per-block entry points -----------------------------------------------------------------------
int sl_moe_block_rows(sl_engine* e, int layer, const uint16_t* x, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!x || !out || layer < 0 || layer >= e->n_layers || m < 1 || m > e->max_m) return SL_ERR_ARG;
  r = to_device(e, e->xn, x, (size_t)m * H * 2); if (r) return r;
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  if (block_flow_ready(e, m)) {                  // a single row: the stages of the step kernel in one launch, same bits
    launch_block_flow(e, layer, 1);
    SL_TRY(e, hipEventRecord(e->ev1, e->stream));
    const uint32_t tag = flow_tag(e->flow_base - (uint32_t)(e->n_layers + 1) * 8u, layer, FS_C);
    r = read_back_tagged(e, out, e->flow_host.tmoe, tag, "moeBlockRows"); if (r) return r;
    time_end(e);
    return SL_OK;
  }
  HiddenArgs ha{e->xn, nullptr, nullptr, nullptr, nullptr};
  e->last_block_flow = false;
  launch_moe(e, e->layers[layer], m, ha);
  SL_TRY(e, hipEventRecord(e->ev1, e->stream));
  r = read_back(e, out, e->moe_out, (size_t)m * H * 2, "moeBlockRows"); if (r) return r;
  time_end(e);
  return SL_OK;
}
int sl_gdn_layer_rows(sl_engine* e, int layer, const uint16_t* x, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!x || !out || layer < 0 || layer >= e->n_layers || m < 1 || m > e->max_m || !e->layers[layer].is_linear) return SL_ERR_ARG;
  r = to_device(e, e->xn, x, (size_t)m * H * 2); if (r) return r;
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  if (block_flow_ready(e, m)) {
    launch_block_flow(e, layer, 0);
    SL_TRY(e, hipEventRecord(e->ev1, e->stream));
    const uint32_t tag = flow_tag(e->flow_base - (uint32_t)(e->n_layers + 1) * 8u, layer, FS_OUT);
    r = read_back_tagged(e, out, e->flow_host.tmix, tag, "gdnLayerRows"); if (r) return r;
  } else {
    HiddenArgs ha{e->xn, nullptr, nullptr, nullptr, nullptr};
    e->last_block_flow = false;
    launch_gdn_mixer(e, e->layers[layer], layer, m, ha, nullptr);
    SL_TRY(e, hipEventRecord(e->ev1, e->stream));
    r = read_back(e, out, e->mix, (size_t)m * H * 2, "gdnLayerRows"); if (r) return r;
  }
  time_end(e);
  e->parity[layer] ^= 1;
  return push_state(e);
}
int sl_attn_layer_rows(sl_engine* e, int layer, const uint16_t* x, int m, uint16_t* out) {
  SL_ENTER(e);
  if (!x || !out || layer < 0 || layer >= e->n_layers || e->layers[layer].is_linear) return SL_ERR_ARG;
  r = check_rows(e, m); if (r) return r;
  r = to_device(e, e->xn, x, (size_t)m * H * 2); if (r) return r;
  SL_TRY(e, hipEventRecord(e->ev0, e->stream));
  if (block_flow_ready(e, m)) {
    launch_block_flow(e, layer, 0);
    SL_TRY(e, hipEventRecord(e->ev1, e->stream));
    const uint32_t tag = flow_tag(e->flow_base - (uint32_t)(e->n_layers + 1) * 8u, layer, FS_OUT);
    r = read_back_tagged(e, out, e->flow_host.tmix, tag, "attnLayerRows"); if (r) return r;
  } else {
    HiddenArgs ha{e->xn, nullptr, nullptr, nullptr, nullptr};
    e->last_block_flow = false;
    launch_attn_mixer(e, e->layers[layer], m, ha, nullptr, 0);
    SL_TRY(e, hipEventRecord(e->ev1, e->stream));
    r = read_back(e, out, e->mix, (size_t)m * H * 2, "attnLayerRows"); if (r) return r;
  }
  time_end(e);
  e->pos += m;
  return push_state(e);
}

// Test hook: copy `count` fp16 elements of one internal scratch buffer of the last launch sequence.
int sl_debug_scratch(sl_engine* e, int which, uint16_t* out, size_t count) {
  SL_ENTER(e);
  const uint16_t* src = nullptr;
  switch (which) {
    case 0: src = e->proj; break;
    case 1: src = e->ycore; break;
    case 2: src = e->qrot; break;
    case 3: src = e->mix; break;
    case 4: src = e->xn; break;
    case 5: src = e->act; break;
    case 6: src = e->sh_act; break;
    case 7: src = e->rlogits; break;
    case 8: src = e->moe_out; break;
    default: return SL_ERR_ARG;
  }
  if (!src || !out) return SL_ERR_ARG;
  if (e->last_block_flow) {
    // a single-launch block keeps its rows in the step kernel's exchange buffers (halves with tags): router logits,
    // mixer output and MoE output can be read from there, the other scratch rows were not written
    const uint32_t* words = which == 7 ? e->flow_host.trlog : (which == 3 ? e->flow_host.tmix : (which == 8 ? e->flow_host.tmoe : nullptr));
    const size_t cap = which == 7 ? 256 : (size_t)H;
    if (!words || count > cap) return SL_ERR_UNSUPPORTED;
    std::vector<uint32_t> w(count);
    r = copy_sync(e, w.data(), words, count * 4, hipMemcpyDeviceToHost); if (r) return r;
    for (size_t i = 0; i < count; ++i) out[i] = (uint16_t)(w[i] & 0xffffu);
    return SL_OK;
  }
  return copy_sync(e, out, src, count * 2, hipMemcpyDeviceToHost);
}

int sl_greedy_generate(sl_engine* e, const int32_t* prompt, int n_prompt, int n_new, int chain_k, int32_t* out) {
  SL_ENTER(e);
  if (!prompt || n_prompt < 1 || n_new < 0 || (n_new > 0 && !out) || !e->has_head) return SL_ERR_ARG;
  if (chain_k < 1) chain_k = 1;
  if (chain_k > MAX_CHAIN) chain_k = MAX_CHAIN;
  int done = 0, last_m = 0;
  while (done < n_prompt) {                    // the rows of a chunk stay on the device: only the last row of the last chunk is used
    last_m = n_prompt - done < e->max_m ? n_prompt - done : e->max_m;
    r = sl_forward_tokens(e, prompt + done, last_m, nullptr); if (r) return r;
    done += last_m;
  }
  if (n_new == 0) return SL_OK;
  r = sl_head_argmax_rows(e, last_m - 1, 1, &out[0]); if (r) return r;
  int have = 1;
  while (have < n_new) {
    const int k = n_new - have < chain_k ? n_new - have : chain_k;
    r = sl_chained_step_argmax(e, out[have - 1], k, out + have); if (r) return r;
    have += k;
  }
  return SL_OK;
}

}  // extern "C"

// Self-test of the matrix-core GEMM (sl_mfma.cuh): host arrays in and out, temporary device buffers.
extern "C" int sl_selftest_qmm4(const uint16_t* x_host, int m, const uint32_t* w_host, const uint16_t* s_host,
                                const uint16_t* b_host, int n, int k, uint16_t* y_host) {
  if (!x_host || !w_host || !s_host || !b_host || !y_host || m < 1 || m > 512 || n < 32 || (n % 32) || k < 64 || (k % 64))
    return SL_ERR_ARG;
  const size_t xb = (size_t)m * k * 2, wb = (size_t)n * (k / 8) * 4, gb = (size_t)n * (k / 64) * 4, yb = (size_t)m * n * 2;
  std::vector<uint32_t> sb((size_t)n * (k / 64));
  for (size_t i = 0; i < sb.size(); ++i) sb[i] = (uint32_t)s_host[i] | ((uint32_t)b_host[i] << 16);
  uint16_t *dx = nullptr, *dy = nullptr;
  uint32_t *dw = nullptr, *dsb = nullptr;
  int rc = SL_ERR_DEVICE;
  if (hipMalloc((void**)&dx, xb) == hipSuccess && hipMalloc((void**)&dw, wb) == hipSuccess &&
      hipMalloc((void**)&dsb, gb) == hipSuccess && hipMalloc((void**)&dy, yb) == hipSuccess &&
      hipMemcpy(dx, x_host, xb, hipMemcpyHostToDevice) == hipSuccess && hipMemcpy(dw, w_host, wb, hipMemcpyHostToDevice) == hipSuccess &&
      hipMemcpy(dsb, sb.data(), gb, hipMemcpyHostToDevice) == hipSuccess) {
    QmmArgs a{dx, k, dw, dsb, m, n, k, dy, n};
    launch_qmm4_mfma(a, nullptr);
    if (hipGetLastError() == hipSuccess && hipDeviceSynchronize() == hipSuccess &&
        hipMemcpy(y_host, dy, yb, hipMemcpyDeviceToHost) == hipSuccess) rc = SL_OK;
  }
  (void)hipFree(dx); (void)hipFree(dw); (void)hipFree(dsb); (void)hipFree(dy);
  return rc;
}
