// The whole-path entry point and the library's housekeeping calls.
#include <atomic>
#include <mutex>
#include "moe_common.h"
#include "moe_layout.h"
#include "act_quant.h"
#include "../../include/moe_hip.h"

namespace moe {

int permute_launch(hipStream_t st, const int32_t *ids, int T, int K, int E, int tile_m, int32_t *sorted_slot,
                   int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &ws, uint16_t *zero_rows = nullptr,
                   int row_len = 0, bool counted = false, const QuantJob *ride = nullptr);
int permute_quant_small_launch(hipStream_t st, const int32_t *ids, int T, int K, int E, int tile_m, int32_t *sorted_slot,
                               int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &ws, uint16_t *zero_rows,
                               int row_len, const uint16_t *x, int H, uint8_t *xq, float *xs);
int gemm1_launch(hipStream_t st, const uint8_t *xq, const float *xs, int T, int H, const uint8_t *w13,
                 const float *w13s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint8_t *hq, float *hs, const uint8_t *sh_w13,
                 const float *sh_w13s, uint8_t *sh_hq, float *sh_hs, int numerics = kNumericsFp8);
int gemm2_launch(hipStream_t st, const uint8_t *hq, const float *hs, int rows_a, int T, int H, const uint8_t *w2,
                 const float *w2s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint16_t *y, const uint8_t *sh_hq, const float *sh_hs,
                 int sh_rows, const uint8_t *sh_w2, const float *sh_w2s, uint16_t *sh_y, int numerics = kNumericsFp8);

int decode_prep_launch(hipStream_t st, const uint16_t *x, int T, int H, const uint16_t *wr, const float *bias, int E, int K,
                       int mode, int n_groups, int topk_groups, int renorm, float scale, uint16_t *logits, float *weights,
                       int32_t *ids, int *arrivals, uint8_t *xq, float *xs, int tile_m, int32_t *sorted_slot,
                       int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &pw);

int weighted_reduce_launch(hipStream_t st, const uint16_t *y, const void *w, const uint16_t *shared_y,
                           const int32_t *slot_to_row, int T, int K, int H, uint16_t *out, int w_bf16 = 0);
size_t router_front_partial_bytes(int T, int H, int E);
int router_front_launch(hipStream_t st, const void *x, int T, int H, const void *wr, int E, float *partial, int *n_slices_out,
                        int32_t *zero = nullptr, int n_zero = 0);
int sum_slices_launch(hipStream_t st, const float *partial, int n_slices, int T, int E, uint16_t *logits);
int route_from_partials_launch(hipStream_t st, const float *partial, int n_slices, const float *bias, int T, int E, int K,
                               int mode, int n_groups, int topk_groups, int renorm, float scale, float *weights_out,
                               int32_t *ids_out, const uint16_t *x, int H, uint8_t *xq, float *xs,
                               int32_t *chunk_counts = nullptr);

size_t dense_small_partial_bytes(int M, int K, int N, bool keep_partial);
int dense_small_launch(hipStream_t st, const uint8_t *xq, const float *xs, int M, int K, const uint8_t *w, const float *ws,
                       int N, uint16_t *out, float *partial, int *n_splits_out);
int swiglu_quant_reduce_launch(hipStream_t st, const float *partial, int n_splits, int M, int I, uint8_t *hq, float *hs);
constexpr int kDenseSmallRows = 128;        // up to this many rows the gated MLP uses the per-wavefront dense kernel
// A single product of few rows: the per-wavefront kernel slices the reduction over the chip, which is what a narrow
// layer with a long reduction needs (16384 -> 1024 at 64 rows: 28 us against 67 us for the grouped kernel's 16 strips).
// A wide layer gives the grouped kernel's 64-column strips enough workgroups by itself, and they stream through the
// deeper LDS ring (7168 -> 36864 at 32 / 64 / 128 rows: 57 / 71 / 59 us against 61 / 88 / 129 us; the boundary lies
// between 7168 and 12288 columns for reductions of 4096 and 7168), and under a short reduction both are a couple of
// launch latencies, of which the grouped path has one fewer (no slices to add).  A layer of at most 2048 columns keeps
// the sliced kernel up to 384 rows, one of at most 1024 up to 512: the grouped kernel has a handful of strips there
// (7168 -> 1536 at 129 / 256 / 384 rows: 24 / 27 / 29 us against 34 / 35 / 36 us; 16384 -> 1024: 27 / 31 / 40 against
// 67 / 69 / 70 us; 4096 -> 4096 is already the grouped kernel's).
static inline bool mm_uses_small_kernel(int M, int K, int N) {
  if (K <= 2048) return false;
  if (M <= 128) return N < 12288;
  return (M <= 384 && N <= 2048) || (M <= 512 && N <= 1024);
}

// Carves the caller's workspace.  Every piece starts on a 256-byte boundary.
struct FusedWs {
  void *permute;
  int32_t *sorted_slot, *expert_offsets, *slot_to_row;
  uint8_t *xq;
  float *xs;
  uint8_t *hq;
  float *hs;
  uint16_t *y;
  uint8_t *sh_hq;
  float *sh_hs;
  uint16_t *sh_y;
  size_t bytes;
};

static FusedWs fused_layout(void *base, int T, int H, int I, int E, int K, int I_sh) {
  FusedWs w{};
  size_t off = 0;
  auto take = [&](size_t n) {
    void *p = base ? (void *)((uint8_t *)base + off) : nullptr;
    off += align_up(n ? n : 1, 256);
    return p;
  };
  const size_t TK = (size_t)T * K;
  w.permute = take(permute_ws_bytes(T, K, E));
  w.sorted_slot = (int32_t *)take(TK * 4);
  w.expert_offsets = (int32_t *)take((size_t)(E + 1) * 4);
  w.slot_to_row = (int32_t *)take(TK * 4);
  w.xq = (uint8_t *)take((size_t)T * H);
  w.xs = (float *)take((size_t)T * scale_pitch(H / kBlock) * 4);
  w.hq = (uint8_t *)take(TK * I);
  w.hs = (float *)take(TK * scale_pitch(I / kBlock) * 4);
  w.y = (uint16_t *)take(TK * H * 2);
  if (I_sh > 0) {
    w.sh_hq = (uint8_t *)take((size_t)T * I_sh);
    w.sh_hs = (float *)take((size_t)T * scale_pitch(I_sh / kBlock) * 4);
    w.sh_y = (uint16_t *)take((size_t)T * H * 2);
  }
  w.bytes = off;
  return w;
}

// ---- the shared expert's first GEMM beside the front end ----
// The shared expert's first GEMM needs the quantised activations and nothing of the routing.  The router product,
// the routing and the permutation launches are short chains that leave most of the chip idle, so for batches
// beyond the decode size moe_layer_fp8 runs the quantisation and that GEMM on a stream of its own while the caller's
// stream goes through the front end: an event on the caller's stream lets the side stream start, the caller's stream
// waits for the quantised activations before the first grouped GEMM and for the shared expert's first GEMM before
// the second (which carries the shared expert's tiles as before).  The router product comes first on the caller's
// stream: its workgroups need most of a compute unit's LDS, which a GEMM workgroup would not leave them.
// To the caller the call is still work on its one stream.  One side stream and three events per (device,
// caller's stream), created at the first call that uses them and kept until the process ends; streams of the default
// priority, no implicit synchronisation with the null stream.  Not used while the caller's stream is being captured
// into a graph, nor by the entry point that allocates nothing.
struct SideLane {
  int device;
  hipStream_t main, side;
  hipEvent_t fork, quantised, join;
};
constexpr int kMaxSideLanes = 32;
static std::mutex g_side_mutex;
static SideLane g_side[kMaxSideLanes];
static int g_n_side = 0;
static std::atomic<int> g_overlap_enabled{1};
constexpr int kOverlapMinTokens = 512;       // below, the front end is too short to hide anything behind

static const SideLane *side_lane(hipStream_t st) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_side_mutex);
  for (int i = 0; i < g_n_side; i++)
    if (g_side[i].device == dev && g_side[i].main == st) return &g_side[i];
  if (g_n_side == kMaxSideLanes) return nullptr;       // more caller streams than lanes: those go without
  SideLane l{dev, st, nullptr, nullptr, nullptr, nullptr};
  if (hipStreamCreateWithFlags(&l.side, hipStreamNonBlocking) != hipSuccess) return nullptr;
  if (hipEventCreateWithFlags(&l.fork, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&l.quantised, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&l.join, hipEventDisableTiming) != hipSuccess) {
    if (l.fork) (void)hipEventDestroy(l.fork);
    if (l.quantised) (void)hipEventDestroy(l.quantised);
    (void)hipStreamDestroy(l.side);
    return nullptr;
  }
  g_side[g_n_side] = l;
  return &g_side[g_n_side++];
}

// The grouped GEMMs and the weighted sum, once the permutation and the quantised activations are in the workspace.
// join: the shared expert's first GEMM has been launched elsewhere and this event marks its end.
static int run_experts(void *stream, const FusedWs &w, const PermuteWs &pw, int T, int H, const uint8_t *w13,
                       const float *w13_scale, const uint8_t *w2, const float *w2_scale, int I, int E, int K,
                       const void *routing_weights, const uint8_t *shared_w13, const float *shared_w13_scale,
                       const uint8_t *shared_w2, const float *shared_w2_scale, int I_sh, void *out_bf16, int out_mode,
                       hipEvent_t join = nullptr, int weights_bf16 = 0) {
  hipStream_t st = (hipStream_t)stream;
  const bool has_shared = shared_w13 != nullptr;
  // a shared expert of the routed experts' width rides in the routed launches (its tiles fill the
  // machine together with theirs); any other width gets launches of its own
  const bool fuse_shared = has_shared && I_sh == I;
  int rc = gemm1_launch(st, w.xq, w.xs, T, H, w13, w13_scale, I, E, K, w.sorted_slot, w.expert_offsets, &pw, -1, w.hq, w.hs,
                        fuse_shared && !join ? shared_w13 : nullptr, shared_w13_scale, w.sh_hq, w.sh_hs);
  if (join) {
    // also after a failed launch: nothing of this call may outlive the caller's stream on the side stream
    const int rc_wait = (int)hipStreamWaitEvent(st, join, 0);
    if (rc == MOE_OK) rc = rc_wait;
  }
  if (rc) return rc;
  uint16_t *y = out_mode == 0 ? (uint16_t *)out_bf16 : w.y;
  rc = gemm2_launch(st, w.hq, w.hs, T * K, T, H, w2, w2_scale, I, E, K, w.sorted_slot, w.expert_offsets, &pw, -1, y,
                    w.sh_hq, w.sh_hs, T, fuse_shared ? shared_w2 : nullptr, shared_w2_scale, w.sh_y);
  if (rc) return rc;
  // slots whose expert id lies outside [0, E) have no row: zero rows in the per-slot form (cleared by the permutation
  // launch), no term in the sum
  if (out_mode == 0) return MOE_OK;
  if (has_shared && !fuse_shared) {
    rc = gemm1_launch(st, w.xq, w.xs, T, H, shared_w13, shared_w13_scale, I_sh, 1, 1, nullptr, nullptr, nullptr, 0,
                      w.sh_hq, w.sh_hs, nullptr, nullptr, nullptr, nullptr);
    if (rc) return rc;
    rc = gemm2_launch(st, w.sh_hq, w.sh_hs, T, T, H, shared_w2, shared_w2_scale, I_sh, 1, 1, nullptr, nullptr, nullptr,
                      0, w.sh_y, nullptr, nullptr, 0, nullptr, nullptr, nullptr);
    if (rc) return rc;
  }
  return weighted_reduce_launch(st, y, routing_weights, has_shared ? w.sh_y : nullptr, w.slot_to_row, T, K, H,
                                (uint16_t *)out_bf16, weights_bf16);
}

// moe_layer_fp8: the fused-experts workspace followed by the router's own pieces
struct LayerWs {
  FusedWs fused;
  uint16_t *logits;
  float *weights;
  int32_t *ids;
  int *arrivals;
  float *partial;      // batches beyond the decode size: partial sums of the router product
  size_t bytes;
};

// the two-launch decode front end: up to kChunk slots (T * K), which one workgroup can permute, and up to 256 experts,
// which one workgroup can rank; every other problem takes the matrix-core router product, routing and permutation launches
static bool decode_size(int T, int K, int E) { return (long)T * K <= kChunk && E <= 256; }

static LayerWs layer_layout(void *base, int T, int H, int I, int E, int K, int I_sh) {
  LayerWs d{};
  d.fused = fused_layout(base, T, H, I, E, K, I_sh);
  size_t off = d.fused.bytes;
  auto take = [&](size_t n) {
    void *p = base ? (void *)((uint8_t *)base + off) : nullptr;
    off += align_up(n ? n : 1, 256);
    return p;
  };
  d.logits = (uint16_t *)take((size_t)T * E * 2);
  d.weights = (float *)take((size_t)T * K * 4);
  d.ids = (int32_t *)take((size_t)T * K * 4);
  d.arrivals = (int *)take(4);
  if (!decode_size(T, K, E)) d.partial = (float *)take(router_front_partial_bytes(T, H, E));
  d.bytes = off;
  return d;
}

// The grouped GEMMs keep one weight-block scale per 128 columns of the reduction in LDS (at most 256 of them) and
// address their operands with 32-bit per-lane offsets: reduction lengths up to 32768, activation tensors below 2 GiB.
static bool dims_in_range(int T, int H, int I, int K) {
  if (H > 32768 || I > 32768) return false;
  return (double)T * H < 2147483648.0 && (double)T * K * I < 2147483648.0;
}

}  // namespace moe

// 200: the GEMM entry points read their weights tile-blocked (moe_pack_weights); 100 read them row-major
extern "C" int moe_hip_version(void) { return 200; }
extern "C" const char *moe_hip_arch(void) { return "gfx950"; }

extern "C" const char *moe_hip_strerror(int code) {
  switch (code) {
    case MOE_OK: return "ok";
    case MOE_E_NULL: return "a required pointer is NULL";
    case MOE_E_SHAPE: return "a dimension is out of the supported range";
    case MOE_E_ALIGN: return "H or I is not a multiple of 128, or a pointer is misaligned";
    case MOE_E_WORKSPACE: return "workspace too small";
    case MOE_E_MODE: return "unknown mode or dtype selector";
    case MOE_E_STATIC_SCRATCH: return "the problem needs more scratch than the library's built-in array holds (MOE_STATIC_SCRATCH_BYTES)";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
  }
}

extern "C" size_t moe_fused_experts_workspace_bytes(int T, int H, int I, int E, int K, int I_shared) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || K < 1 || I_shared < 0) return 0;
  return moe::fused_layout(nullptr, T, H, I, E, K, I_shared).bytes;
}

extern "C" int moe_fused_experts_fp8(void *stream, const void *x_bf16, int T, int H, const uint8_t *w13,
                                     const float *w13_scale, const uint8_t *w2, const float *w2_scale, int I, int E,
                                     const int32_t *ids, const float *routing_weights, int K,
                                     const uint8_t *shared_w13, const float *shared_w13_scale,
                                     const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                                     void *out_bf16, int out_mode, void *workspace, size_t workspace_bytes) {
  return moe_fused_experts_fp8_rw(stream, x_bf16, T, H, w13, w13_scale, w2, w2_scale, I, E, ids, routing_weights,
                                  MOE_DTYPE_F32, K, shared_w13, shared_w13_scale, shared_w2, shared_w2_scale, I_shared,
                                  out_bf16, out_mode, workspace, workspace_bytes);
}

extern "C" int moe_fused_experts_fp8_rw(void *stream, const void *x_bf16, int T, int H, const uint8_t *w13,
                                        const float *w13_scale, const uint8_t *w2, const float *w2_scale, int I, int E,
                                        const int32_t *ids, const void *routing_weights, int routing_weights_dtype,
                                        int K, const uint8_t *shared_w13, const float *shared_w13_scale,
                                        const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared,
                                        void *out_bf16, int out_mode, void *workspace, size_t workspace_bytes) {
  using namespace moe;
  if (routing_weights_dtype != MOE_DTYPE_F32 && routing_weights_dtype != MOE_DTYPE_BF16) return MOE_E_MODE;
  // per-token pointers may be NULL for an empty batch (T == 0): nothing is read or written through them
  if (!w13 || !w13_scale || !w2 || !w2_scale || !workspace) return MOE_E_NULL;
  if (T != 0 && (!x_bf16 || !ids || !out_bf16)) return MOE_E_NULL;
  if (out_mode != 0 && out_mode != 1) return MOE_E_MODE;
  if (T != 0 && out_mode == 1 && !routing_weights) return MOE_E_NULL;
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK || K > E) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30)) return MOE_E_SHAPE;
  if (!dims_in_range(T, H, I, K)) return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  const bool has_shared = shared_w13 != nullptr;
  if (has_shared) {
    if (out_mode != 1) return MOE_E_MODE;
    if (!shared_w13_scale || !shared_w2 || !shared_w2_scale) return MOE_E_NULL;
    if (I_shared < 1 || !dims_in_range(T, H, I_shared, 1)) return MOE_E_SHAPE;
    if (I_shared % kBlock) return MOE_E_ALIGN;
  }
  const int I_sh = has_shared ? I_shared : 0;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) ||
      ((uintptr_t)w13 % 16) || ((uintptr_t)w2 % 16))
    return MOE_E_ALIGN;
  FusedWs w = fused_layout(workspace, T, H, I, E, K, I_sh);
  if (workspace_bytes < w.bytes) return MOE_E_WORKSPACE;
  if (T == 0) return MOE_OK;

  hipStream_t st = (hipStream_t)stream;
  PermuteWs pw = permute_ws_layout(w.permute, T, K, E);
  // per-slot output form: the rows of slots without an expert are cleared by the permutation (nothing else writes them)
  uint16_t *const zero_rows = out_mode == 0 ? (uint16_t *)out_bf16 : nullptr;
  int rc;
  if ((long)T * K <= kChunk) {
    // decode sizes: permutation and activation quantisation share one launch
    rc = permute_quant_small_launch(st, ids, T, K, E, choose_tile_m(T, K, E), w.sorted_slot, w.expert_offsets,
                                    w.slot_to_row, pw, zero_rows, H, (const uint16_t *)x_bf16, H, w.xq, w.xs);
    if (rc) return rc;
  } else {
    // the activations are quantised by extra workgroups of the permutation's scan launch
    const QuantJob job{(const uint16_t *)x_bf16, w.xq, w.xs, (size_t)T * (H / kBlock), H / kBlock, scale_pitch(H / kBlock)};
    rc = permute_launch(st, ids, T, K, E, choose_tile_m(T, K, E), w.sorted_slot, w.expert_offsets, w.slot_to_row, pw,
                        zero_rows, H, false, &job);
    if (rc) return rc;
  }
  return run_experts(stream, w, pw, T, H, w13, w13_scale, w2, w2_scale, I, E, K, routing_weights, shared_w13,
                     shared_w13_scale, shared_w2, shared_w2_scale, I_sh, out_bf16, out_mode, nullptr,
                     routing_weights_dtype == MOE_DTYPE_BF16);
}

extern "C" size_t moe_layer_fp8_workspace_bytes(int T, int H, int I, int E, int K, int I_shared) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || I_shared < 0 || H % moe::kBlock) return 0;
  return moe::layer_layout(nullptr, T, H, I, E, K, I_shared).bytes;
}

namespace moe {
static int layer_fp8_run(void *stream, const void *x_bf16, int T, int H, const void *router_w_bf16,
                         const float *router_bias, int E, int K, int mode, int n_groups, int topk_groups,
                         int renorm, float scale, const uint8_t *w13, const float *w13_scale, const uint8_t *w2,
                         const float *w2_scale, int I, const uint8_t *shared_w13, const float *shared_w13_scale,
                         const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared, void *out_bf16,
                         void *logits_out_bf16, float *weights_out, int32_t *ids_out, void *workspace,
                         size_t workspace_bytes, bool may_use_side_stream) {
  if (!router_w_bf16 || !w13 || !w13_scale || !w2 || !w2_scale || !workspace) return MOE_E_NULL;
  if (T != 0 && (!x_bf16 || !out_bf16)) return MOE_E_NULL;
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK || K > E) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30)) return MOE_E_SHAPE;
  if (!dims_in_range(T, H, I, K)) return MOE_E_SHAPE;
  if (mode != MOE_ROUTE_SOFTMAX && mode != MOE_ROUTE_SIGMOID && mode != MOE_ROUTE_SOFTMAX_LOGIT_BIAS) return MOE_E_MODE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  const bool has_shared = shared_w13 != nullptr;
  if (has_shared) {
    if (!shared_w13_scale || !shared_w2 || !shared_w2_scale) return MOE_E_NULL;
    if (I_shared < 1 || !dims_in_range(T, H, I_shared, 1)) return MOE_E_SHAPE;
    if (I_shared % kBlock) return MOE_E_ALIGN;
  }
  const int I_sh = has_shared ? I_shared : 0;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) ||
      ((uintptr_t)router_w_bf16 % 16) || ((uintptr_t)w13 % 16) || ((uintptr_t)w2 % 16))
    return MOE_E_ALIGN;
  LayerWs d = layer_layout(workspace, T, H, I, E, K, I_sh);
  if (workspace_bytes < d.bytes) return MOE_E_WORKSPACE;
  if (T == 0) return MOE_OK;
  hipStream_t st = (hipStream_t)stream;
  const FusedWs &w = d.fused;
  PermuteWs pw = permute_ws_layout(w.permute, T, K, E);
  float *weights = weights_out ? weights_out : d.weights;
  int32_t *ids = ids_out ? ids_out : d.ids;
  int rc;
  hipEvent_t join = nullptr;
  if (decode_size(T, K, E)) {
    // two launches: router logits + activation quantisation, then routing + permutation
    rc = decode_prep_launch(st, (const uint16_t *)x_bf16, T, H, (const uint16_t *)router_w_bf16, router_bias, E, K, mode,
                            n_groups, topk_groups, renorm, scale, logits_out_bf16 ? (uint16_t *)logits_out_bf16 : d.logits,
                            weights, ids, d.arrivals, w.xq, w.xs, choose_tile_m(T, K, E), w.sorted_slot, w.expert_offsets,
                            w.slot_to_row, pw);
    if (rc) return rc;
  } else {
    // a shared expert of the routed experts' width: its first GEMM runs beside the front end
    const SideLane *lane = nullptr;
    if (may_use_side_stream && has_shared && I_sh == I && T >= kOverlapMinTokens && g_overlap_enabled.load())
      lane = side_lane(st);
    // the router product on the matrix cores, its reduction cut into slices; the routing kernel adds the slices.
    // More than kChunk slots: the routing kernel also counts the slots per (chunk, expert) - the permutation's first
    // pass - into a table the router product's launch has cleared (table, per-expert totals and arrival counter are
    // one run of integers).
    int n_slices = 0;
    const bool counted = (long)T * K > kChunk && (size_t)pw.n_chunks * E < ((size_t)1 << 30);
    int32_t *const zero = counted ? pw.chunk_counts : nullptr;
    const int n_zero = counted ? (int)(pw.arrivals + 1 - pw.chunk_counts) : 0;
    if (lane) {
      rc = (int)hipEventRecord(lane->fork, st);
      if (rc) return rc;
      rc = router_front_launch(st, x_bf16, T, H, router_w_bf16, E, d.partial, &n_slices, zero, n_zero);
      if (rc) return rc;
      rc = (int)hipStreamWaitEvent(lane->side, lane->fork, 0);
      if (rc) return rc;
      rc = moe_act_quant(lane->side, x_bf16, T, H, w.xq, w.xs);
      if (rc == MOE_OK) rc = (int)hipEventRecord(lane->quantised, lane->side);
      if (rc == MOE_OK)
        rc = gemm1_launch(lane->side, w.xq, w.xs, T, H, shared_w13, shared_w13_scale, I_sh, 1, 1, nullptr, nullptr,
                          nullptr, 0, w.sh_hq, w.sh_hs, nullptr, nullptr, nullptr, nullptr);
      // whatever the launches returned, the caller's stream waits for the side stream: nothing of this call may still
      // run there when the caller's stream has finished
      const int rc_join = (int)hipEventRecord(lane->join, lane->side);
      if (rc_join) return rc_join;
      join = lane->join;
      if (rc) {
        (void)hipStreamWaitEvent(st, join, 0);
        return rc;
      }
    } else {
      rc = router_front_launch(st, x_bf16, T, H, router_w_bf16, E, d.partial, &n_slices, zero, n_zero);
    }
    if (rc == MOE_OK && logits_out_bf16) rc = sum_slices_launch(st, d.partial, n_slices, T, E, (uint16_t *)logits_out_bf16);
    // Unless the side stream quantises the activations, extra workgroups do: of the permutation's scan launch (a
    // few dozen workgroups of its own), or - up to kChunk slots, where the permutation is one workgroup - of the
    // routing launch.
    const bool ride_in_scan = !lane && (long)T * K > kChunk;
    if (rc == MOE_OK)
      rc = route_from_partials_launch(st, d.partial, n_slices, router_bias, T, E, K, mode, n_groups, topk_groups, renorm,
                                      scale, weights, ids, lane || ride_in_scan ? nullptr : (const uint16_t *)x_bf16, H,
                                      w.xq, w.xs, zero);
    const QuantJob job{(const uint16_t *)x_bf16, w.xq, w.xs, (size_t)T * (H / kBlock), H / kBlock, scale_pitch(H / kBlock)};
    if (rc == MOE_OK)
      rc = permute_launch(st, ids, T, K, E, choose_tile_m(T, K, E), w.sorted_slot, w.expert_offsets, w.slot_to_row, pw,
                          nullptr, 0, counted, ride_in_scan ? &job : nullptr);
    if (rc == MOE_OK && lane) rc = (int)hipStreamWaitEvent(st, lane->quantised, 0);
    if (rc) {
      if (join) (void)hipStreamWaitEvent(st, join, 0);
      return rc;
    }
  }
  return run_experts(stream, w, pw, T, H, w13, w13_scale, w2, w2_scale, I, E, K, weights, shared_w13, shared_w13_scale,
                     shared_w2, shared_w2_scale, I_sh, out_bf16, 1, join);
}
}  // namespace moe

extern "C" int moe_layer_fp8(void *stream, const void *x_bf16, int T, int H, const void *router_w_bf16,
                             const float *router_bias, int E, int K, int mode, int n_groups, int topk_groups,
                             int renorm, float scale, const uint8_t *w13, const float *w13_scale, const uint8_t *w2,
                             const float *w2_scale, int I, const uint8_t *shared_w13, const float *shared_w13_scale,
                             const uint8_t *shared_w2, const float *shared_w2_scale, int I_shared, void *out_bf16,
                             void *logits_out_bf16, float *weights_out, int32_t *ids_out, void *workspace,
                             size_t workspace_bytes) {
  return moe::layer_fp8_run(stream, x_bf16, T, H, router_w_bf16, router_bias, E, K, mode, n_groups, topk_groups, renorm,
                            scale, w13, w13_scale, w2, w2_scale, I, shared_w13, shared_w13_scale, shared_w2,
                            shared_w2_scale, I_shared, out_bf16, logits_out_bf16, weights_out, ids_out, workspace,
                            workspace_bytes, true);
}

extern "C" int moe_set_shared_overlap(int enabled) { return moe::g_overlap_enabled.exchange(enabled ? 1 : 0); }

// ---- the same call for callers that cannot allocate: the workspace is an array that lives in the library ----
//
// One copy of `scratch` exists per GPU, at an address of its own; the array's name means nothing to host code, so
// the device address is looked up once per device (with that device current) and that pointer is what the
// kernels get, exactly as they get the caller's workspace in moe_layer_fp8.  Nothing in the layer's kernels
// needs the workspace to start at zero (the one counter in it is cleared by the first launch of every call), so
// the previous call's contents may stay.
static __device__ __align__(256) unsigned char scratch[MOE_STATIC_SCRATCH_BYTES];

namespace moe {
constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device; the lookup runs once per device
static int static_scratch(void **out) {
  int dev = -1;
  hipError_t rc = hipGetDevice(&dev);
  if (rc != hipSuccess) return (int)rc;
  if (dev < 0 || dev >= kMaxDevices) return MOE_E_SHAPE;
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess) return (int)rc;
    if (!p || ((uintptr_t)p % 256)) return MOE_E_ALIGN;
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // two threads racing here store the same address
  }
  *out = p;
  return MOE_OK;
}
}  // namespace moe

extern "C" int moe_hip_init(void) {
  void *p = nullptr;
  return moe::static_scratch(&p);
}

extern "C" int moe_static_scratch_address(void **address) {
  if (!address) return MOE_E_NULL;
  return moe::static_scratch(address);
}

extern "C" int moe_layer_fp8_static(void *stream, const void *x_bf16, int T, int H, const void *router_w_bf16,
                                    const float *router_bias, int E, int K, int mode, int n_groups, int topk_groups,
                                    int renorm, float scale, const uint8_t *w13, const float *w13_scale,
                                    const uint8_t *w2, const float *w2_scale, int I, const uint8_t *shared_w13,
                                    const float *shared_w13_scale, const uint8_t *shared_w2,
                                    const float *shared_w2_scale, int I_shared, void *out_bf16, void *logits_out_bf16,
                                    float *weights_out, int32_t *ids_out) {
  using namespace moe;
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK || K > E || I_shared < 0)
    return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  const int I_sh = shared_w13 ? I_shared : 0;
  // the problem must fit the array: refused here, before anything is launched
  if (layer_layout(nullptr, T, H, I, E, K, I_sh).bytes > (size_t)MOE_STATIC_SCRATCH_BYTES) return MOE_E_STATIC_SCRATCH;
  void *ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  return layer_fp8_run(stream, x_bf16, T, H, router_w_bf16, router_bias, E, K, mode, n_groups, topk_groups, renorm, scale,
                       w13, w13_scale, w2, w2_scale, I, shared_w13, shared_w13_scale, shared_w2, shared_w2_scale, I_shared,
                       out_bf16, logits_out_bf16, weights_out, ids_out, ws, (size_t)MOE_STATIC_SCRATCH_BYTES, false);
}

// The router product on its own: logits [T, E] bf16 = x [T, H] . Wr [E, H]^T (fp32 sums, rounded once).
extern "C" size_t moe_router_logits_workspace_bytes(int T, int H, int E) {
  if (T < 0 || H < 1 || E < 1 || E > MOE_MAX_EXPERTS || H % moe::kBlock) return 0;
  return moe::align_up(moe::router_front_partial_bytes(T, H, E) + 1, 256);
}

extern "C" int moe_router_logits(void *stream, const void *x_bf16, int T, int H, const void *router_w_bf16, int E,
                                 void *logits_bf16, void *workspace, size_t workspace_bytes) {
  using namespace moe;
  if (!router_w_bf16 || !workspace) return MOE_E_NULL;
  if (T != 0 && (!x_bf16 || !logits_bf16)) return MOE_E_NULL;
  if (T < 0 || H < 1 || E < 1 || E > MOE_MAX_EXPERTS) return MOE_E_SHAPE;
  if (H % kBlock) return MOE_E_ALIGN;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)router_w_bf16 % 16)) return MOE_E_ALIGN;
  if (workspace_bytes < moe_router_logits_workspace_bytes(T, H, E)) return MOE_E_WORKSPACE;
  if (T == 0) return MOE_OK;
  int n_slices = 0;
  int rc = router_front_launch((hipStream_t)stream, x_bf16, T, H, router_w_bf16, E, (float *)workspace, &n_slices);
  if (rc) return rc;
  return sum_slices_launch((hipStream_t)stream, (const float *)workspace, n_slices, T, E, (uint16_t *)logits_bf16);
}

// ---- dense block-scaled FP8 linear layers: the grouped kernels with one "expert" that owns every row ----

namespace moe {
struct DenseWs {
  uint8_t *xq;
  float *xs;
  uint8_t *hq;
  float *hs;
  float *partial;     // slices of the (only or second) product
  float *partial1;    // MLP: slices of the first product
  size_t bytes;
};
static DenseWs dense_layout(void *base, int M, int K, int I, int N = 0) {
  DenseWs w{};
  size_t off = 0;
  auto take = [&](size_t n) {
    void *p = base ? (void *)((uint8_t *)base + off) : nullptr;
    off += align_up(n ? n : 1, 256);
    return p;
  };
  w.xq = (uint8_t *)take((size_t)M * K);
  w.xs = (float *)take((size_t)M * scale_pitch(K / kBlock) * 4);
  if (I > 0) {
    w.hq = (uint8_t *)take((size_t)M * I);
    w.hs = (float *)take((size_t)M * scale_pitch(I / kBlock) * 4);
  }
  if (N > 0 && (I > 0 ? M <= kDenseSmallRows : mm_uses_small_kernel(M, K, N))) {
    if (I > 0) {      // MLP: K = H, N = H; first product [M, 2I] over H, second [M, H] over I
      w.partial1 = (float *)take(dense_small_partial_bytes(M, K, 2 * I, true));
      w.partial = (float *)take(dense_small_partial_bytes(M, I, N, false));
    } else {
      w.partial = (float *)take(dense_small_partial_bytes(M, K, N, false));
    }
  }
  w.bytes = off;
  return w;
}
}  // namespace moe

extern "C" size_t moe_mm_fp8_workspace_bytes(int M, int K, int N) {
  if (M < 0 || K < 1 || N < 16 || K % moe::kBlock || N % 16) return 0;
  return moe::dense_layout(nullptr, M, K, 0, N).bytes;
}

extern "C" int moe_mm_fp8(void *stream, const void *x_bf16, int M, int K, const uint8_t *w, const float *w_scale,
                          int N, void *out_bf16, void *workspace, size_t workspace_bytes) {
  using namespace moe;
  if (!w || !w_scale || !workspace) return MOE_E_NULL;
  if (M != 0 && (!x_bf16 || !out_bf16)) return MOE_E_NULL;
  if (M < 0 || K < 1 || N < 16 || K > 32768 || N > (1 << 20)) return MOE_E_SHAPE;
  if (K % kBlock || N % 16) return MOE_E_ALIGN;
  if ((double)M * K >= 2147483648.0 || (double)M * N >= 2147483648.0 || (double)N * K >= 4294967296.0) return MOE_E_SHAPE;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) || ((uintptr_t)w % 16))
    return MOE_E_ALIGN;
  DenseWs d = dense_layout(workspace, M, K, 0, N);
  if (workspace_bytes < d.bytes) return MOE_E_WORKSPACE;
  if (M == 0) return MOE_OK;
  int rc = moe_act_quant(stream, x_bf16, M, K, d.xq, d.xs);
  if (rc) return rc;
  if (mm_uses_small_kernel(M, K, N))
    return dense_small_launch((hipStream_t)stream, d.xq, d.xs, M, K, w, w_scale, N, (uint16_t *)out_bf16, d.partial, nullptr);
  return gemm2_launch((hipStream_t)stream, d.xq, d.xs, M, M, N, w, w_scale, K, 1, 1, nullptr, nullptr, nullptr, 0,
                      (uint16_t *)out_bf16, nullptr, nullptr, 0, nullptr, nullptr, nullptr);
}

extern "C" int moe_mm_bf16(void *stream, const void *x_bf16, int M, int K, const void *w_bf16, int N, void *out_bf16) {
  using namespace moe;
  if (!w_bf16) return MOE_E_NULL;
  if (M != 0 && (!x_bf16 || !out_bf16)) return MOE_E_NULL;
  if (M < 0 || K < 1 || N < 16 || K > 16384 || N > (1 << 20)) return MOE_E_SHAPE;
  if (K % 64 || N % 16) return MOE_E_ALIGN;                 // a 128-byte step is 64 elements
  if ((double)M * K * 2 >= 2147483648.0 || (double)M * N >= 2147483648.0 || (double)N * K * 2 >= 4294967296.0)
    return MOE_E_SHAPE;
  if (((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) || ((uintptr_t)w_bf16 % 16)) return MOE_E_ALIGN;
  if (M == 0) return MOE_OK;
  return gemm2_launch((hipStream_t)stream, (const uint8_t *)x_bf16, nullptr, M, M, N, (const uint8_t *)w_bf16, nullptr, K,
                      1, 1, nullptr, nullptr, nullptr, 0, (uint16_t *)out_bf16, nullptr, nullptr, 0, nullptr, nullptr,
                      nullptr, kNumericsBf16);
}

// The same product in the reference's own arithmetic: bf16 activations against FP8 weights de-quantised in registers
extern "C" int moe_mm_w8a16(void *stream, const void *x_bf16, int M, int K, const uint8_t *w, const float *w_scale, int N,
                            void *out_bf16) {
  using namespace moe;
  if (!w || !w_scale) return MOE_E_NULL;
  if (M != 0 && (!x_bf16 || !out_bf16)) return MOE_E_NULL;
  if (M < 0 || K < 1 || N < 16 || K > 16384 || N > (1 << 20)) return MOE_E_SHAPE;
  if (K % kBlock || N % 16) return MOE_E_ALIGN;
  if ((double)M * K * 2 >= 2147483648.0 || (double)M * N >= 2147483648.0 || (double)N * K >= 4294967296.0) return MOE_E_SHAPE;
  if (((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) || ((uintptr_t)w % 16)) return MOE_E_ALIGN;
  if (M == 0) return MOE_OK;
  return gemm2_launch((hipStream_t)stream, (const uint8_t *)x_bf16, nullptr, M, M, N, w, w_scale, K, 1, 1, nullptr, nullptr,
                      nullptr, 0, (uint16_t *)out_bf16, nullptr, nullptr, 0, nullptr, nullptr, nullptr, kNumericsW8A16);
}

extern "C" size_t moe_mlp_fp8_workspace_bytes(int M, int H, int I) {
  if (M < 0 || H < 1 || I < 1) return 0;
  return moe::dense_layout(nullptr, M, H, I, H).bytes;
}

extern "C" int moe_mlp_fp8(void *stream, const void *x_bf16, int M, int H, const uint8_t *w13, const float *w13_scale,
                           const uint8_t *w2, const float *w2_scale, int I, void *out_bf16, void *workspace,
                           size_t workspace_bytes) {
  using namespace moe;
  if (!w13 || !w13_scale || !w2 || !w2_scale || !workspace) return MOE_E_NULL;
  if (M != 0 && (!x_bf16 || !out_bf16)) return MOE_E_NULL;
  if (M < 0 || H < 1 || I < 1 || H > 32768 || I > 32768) return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  if ((double)M * H >= 2147483648.0 || (double)M * I >= 2147483648.0) return MOE_E_SHAPE;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) || ((uintptr_t)w13 % 16) ||
      ((uintptr_t)w2 % 16))
    return MOE_E_ALIGN;
  DenseWs d = dense_layout(workspace, M, H, I, H);
  if (workspace_bytes < d.bytes) return MOE_E_WORKSPACE;
  if (M == 0) return MOE_OK;
  hipStream_t st = (hipStream_t)stream;
  int rc = moe_act_quant(stream, x_bf16, M, H, d.xq, d.xs);
  if (rc) return rc;
  if (M <= kDenseSmallRows) {
    int n1 = 0;
    rc = dense_small_launch(st, d.xq, d.xs, M, H, w13, w13_scale, 2 * I, nullptr, d.partial1, &n1);
    if (rc) return rc;
    rc = swiglu_quant_reduce_launch(st, d.partial1, n1, M, I, d.hq, d.hs);
    if (rc) return rc;
    return dense_small_launch(st, d.hq, d.hs, M, I, w2, w2_scale, H, (uint16_t *)out_bf16, d.partial, nullptr);
  }
  rc = gemm1_launch(st, d.xq, d.xs, M, H, w13, w13_scale, I, 1, 1, nullptr, nullptr, nullptr, 0, d.hq, d.hs, nullptr,
                    nullptr, nullptr, nullptr);
  if (rc) return rc;
  return gemm2_launch(st, d.hq, d.hs, M, M, H, w2, w2_scale, I, 1, 1, nullptr, nullptr, nullptr, 0, (uint16_t *)out_bf16,
                      nullptr, nullptr, 0, nullptr, nullptr, nullptr);
}

// ---- un-quantised experts: bf16 weights, bf16 activations, no scales ----

namespace moe {
struct Bf16Ws {
  void *permute;
  int32_t *sorted_slot, *expert_offsets, *slot_to_row;
  uint16_t *h, *y;
  size_t bytes;
};
static Bf16Ws bf16_layout(void *base, int T, int H, int I, int E, int K) {
  Bf16Ws w{};
  size_t off = 0;
  auto take = [&](size_t n) {
    void *p = base ? (void *)((uint8_t *)base + off) : nullptr;
    off += align_up(n ? n : 1, 256);
    return p;
  };
  const size_t TK = (size_t)T * K;
  w.permute = take(permute_ws_bytes(T, K, E));
  w.sorted_slot = (int32_t *)take(TK * 4);
  w.expert_offsets = (int32_t *)take((size_t)(E + 1) * 4);
  w.slot_to_row = (int32_t *)take(TK * 4);
  w.h = (uint16_t *)take(TK * I * 2);
  w.y = (uint16_t *)take(TK * H * 2);
  w.bytes = off;
  return w;
}
}  // namespace moe

extern "C" size_t moe_fused_experts_bf16_workspace_bytes(int T, int H, int I, int E, int K) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || K < 1) return 0;
  return moe::bf16_layout(nullptr, T, H, I, E, K).bytes;
}

namespace moe {
// bf16 activations against bf16 weights (scales NULL) or against FP8 weights de-quantised in registers
static int experts_a16_run(void *stream, const void *x_bf16, int T, int H, const void *w13, const float *w13_scale,
                           const void *w2, const float *w2_scale, int I, int E, const int32_t *ids,
                           const float *routing_weights, int K, void *out_bf16, int out_mode, void *workspace,
                           size_t workspace_bytes, int numerics) {
  if (!w13 || !w2 || !workspace) return MOE_E_NULL;
  if (numerics == kNumericsW8A16 && (!w13_scale || !w2_scale)) return MOE_E_NULL;
  if (T != 0 && (!x_bf16 || !ids || !out_bf16)) return MOE_E_NULL;
  if (out_mode != 0 && out_mode != 1) return MOE_E_MODE;
  if (T != 0 && out_mode == 1 && !routing_weights) return MOE_E_NULL;
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK || K > E) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30) || H > 16384 || I > 16384) return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  if ((double)T * H * 2 >= 2147483648.0 || (double)T * K * I * 2 >= 2147483648.0) return MOE_E_SHAPE;
  if (((uintptr_t)workspace % 256) || ((uintptr_t)x_bf16 % 16) || ((uintptr_t)out_bf16 % 16) ||
      ((uintptr_t)w13 % 16) || ((uintptr_t)w2 % 16))
    return MOE_E_ALIGN;
  Bf16Ws w = bf16_layout(workspace, T, H, I, E, K);
  if (workspace_bytes < w.bytes) return MOE_E_WORKSPACE;
  if (T == 0) return MOE_OK;
  hipStream_t st = (hipStream_t)stream;
  PermuteWs pw = permute_ws_layout(w.permute, T, K, E);
  int rc = permute_launch(st, ids, T, K, E, choose_tile_m(T, K, E), w.sorted_slot, w.expert_offsets, w.slot_to_row, pw,
                          out_mode == 0 ? (uint16_t *)out_bf16 : nullptr, H);
  if (rc) return rc;
  rc = gemm1_launch(st, (const uint8_t *)x_bf16, nullptr, T, H, (const uint8_t *)w13, w13_scale, I, E, K, w.sorted_slot,
                    w.expert_offsets, &pw, -1, (uint8_t *)w.h, nullptr, nullptr, nullptr, nullptr, nullptr, numerics);
  if (rc) return rc;
  uint16_t *y = out_mode == 0 ? (uint16_t *)out_bf16 : w.y;
  rc = gemm2_launch(st, (const uint8_t *)w.h, nullptr, T * K, T, H, (const uint8_t *)w2, w2_scale, I, E, K,
                    w.sorted_slot, w.expert_offsets, &pw, -1, y, nullptr, nullptr, 0, nullptr, nullptr, nullptr, numerics);
  if (rc) return rc;
  if (out_mode == 0) return MOE_OK;        // the rows of slots without an expert were cleared by the permutation launch
  return weighted_reduce_launch(st, y, routing_weights, nullptr, w.slot_to_row, T, K, H, (uint16_t *)out_bf16);
}
}  // namespace moe

extern "C" int moe_fused_experts_bf16(void *stream, const void *x_bf16, int T, int H, const void *w13_bf16,
                                      const void *w2_bf16, int I, int E, const int32_t *ids,
                                      const float *routing_weights, int K, void *out_bf16, int out_mode,
                                      void *workspace, size_t workspace_bytes) {
  return moe::experts_a16_run(stream, x_bf16, T, H, w13_bf16, nullptr, w2_bf16, nullptr, I, E, ids, routing_weights, K,
                              out_bf16, out_mode, workspace, workspace_bytes, moe::kNumericsBf16);
}

extern "C" int moe_fused_experts_w8a16(void *stream, const void *x_bf16, int T, int H, const uint8_t *w13,
                                       const float *w13_scale, const uint8_t *w2, const float *w2_scale, int I, int E,
                                       const int32_t *ids, const float *routing_weights, int K, void *out_bf16,
                                       int out_mode, void *workspace, size_t workspace_bytes) {
  return moe::experts_a16_run(stream, x_bf16, T, H, w13, w13_scale, w2, w2_scale, I, E, ids, routing_weights, K, out_bf16,
                              out_mode, workspace, workspace_bytes, moe::kNumericsW8A16);
}
