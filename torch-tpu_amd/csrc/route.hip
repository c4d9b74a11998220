// Router selection kernels: one 64-lane wavefront owns one token's row of scores.
//
// A row of E <= 1024 scores lives in registers, element e in lane e % 64, register e / 64
// (coalesced loads).  Every arg-max is a butterfly over the wave on (value, index) pairs with
// "greater value, then lower index" as the order, so equal scores resolve to the lower index
// on every lane identically and the K picks come out in descending order.  (value, index) travels as one
// 64-bit key, so a comparison is one instruction.
#include "moe_common.h"
#include "moe_layout.h"
#include "act_quant.h"
#include "route_block.h"
#include "../../include/moe_hip.h"

namespace moe {


// A candidate is one 64-bit key: the score's bits mapped monotonically onto unsigned integers in the upper half
// (-0 counts as +0, NaN sorts below -inf: it never wins), the complement of the element index in the lower half.
// "Greater value, then lower index" is then a single unsigned comparison, candidates of one row never compare equal,
// and 0 - below every real candidate - stands for "no candidate".
typedef unsigned long long cand_t;

__device__ __forceinline__ uint32_t ordered_bits(float x) {
  uint32_t b = __float_as_uint(x);
  if (x == 0.f) b = 0;
  uint32_t u = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  if (x != x) u = 1;
  return u;
}
__device__ __forceinline__ cand_t make_cand(float v, int index) {
  return ((cand_t)ordered_bits(v) << 32) | (uint32_t)~index;
}
__device__ __forceinline__ int cand_index(cand_t c) { return (int)~(uint32_t)c; }       // c != 0
__device__ __forceinline__ float cand_value(cand_t c) {                                 // c != 0
  const uint32_t u = (uint32_t)(c >> 32);
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// Arg-max over the wavefront with data-parallel-primitive moves (no LDS round trips): an inclusive
// scan inside each row of 16 lanes (row_shr 1, 2, 4, 8), then row 0 -> 1 and 2 -> 3 (row_bcast:15),
// then rows 0-1 -> 2-3 (row_bcast:31); lane 63 ends up with the winner, which is broadcast.
// Lanes that have no source in a move see "no candidate".
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void argmax_step(cand_t &c) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)c, CTRL, ROW_MASK, 0xf, false);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(c >> 32), CTRL, ROW_MASK, 0xf, false);
  const cand_t o = ((cand_t)hi << 32) | lo;
  c = o > c ? o : c;
}

__device__ __forceinline__ cand_t read_cand(cand_t c, int src_lane) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)c, src_lane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(c >> 32), src_lane);
  return ((cand_t)hi << 32) | lo;
}

__device__ __forceinline__ cand_t wave_argmax(cand_t c) {
  argmax_step<0x111, 0xf>(c);   // row_shr:1
  argmax_step<0x112, 0xf>(c);   // row_shr:2
  argmax_step<0x114, 0xf>(c);   // row_shr:4
  argmax_step<0x118, 0xf>(c);   // row_shr:8
  argmax_step<0x142, 0xa>(c);   // row_bcast:15 into rows 1 and 3
  argmax_step<0x143, 0xc>(c);   // row_bcast:31 into rows 2 and 3
  return read_cand(c, 63);
}

// Arg-max inside each half of the wavefront (lanes 0-31 and 32-63 separately); every lane ends up with
// the winner of its own half.
__device__ __forceinline__ cand_t half_argmax(cand_t c, int lane) {
  argmax_step<0x111, 0xf>(c);   // row_shr:1
  argmax_step<0x112, 0xf>(c);   // row_shr:2
  argmax_step<0x114, 0xf>(c);   // row_shr:4
  argmax_step<0x118, 0xf>(c);   // row_shr:8
  argmax_step<0x142, 0xa>(c);   // row_bcast:15 into rows 1 and 3: lanes 31 and 63 hold the halves' winners
  const cand_t lo = read_cand(c, 31), hi = read_cand(c, 63);
  return lane < 32 ? lo : hi;
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// p[0] + p[stride] + ... (n terms, n <= 8) added in that order; all terms are asked for before the first is used
__device__ __forceinline__ float sum_slices_in_order(const float *__restrict__ p, size_t stride, int n) {
  float v[8];
#pragma unroll
  for (int k = 0; k < 8; k++) v[k] = k < n ? p[(size_t)k * stride] : 0.f;
  float acc = v[0];
#pragma unroll
  for (int k = 1; k < 8; k++)
    if (k < n) acc += v[k];
  return acc;
}

// Select top_k of one row.  v[j] holds element lane + 64*j (only j < per_lane are used,
// elements >= E must be pre-marked dead).  dead bit j set = element is not a candidate.
// Group limiting (n_groups > 1): group score = top1 + top2 of the group (fp32 add, rounded to
// bf16 when round_bf16), keep the topk_groups best groups, the rest get value -inf but stay
// candidates, exactly as a masked_fill(-inf) followed by top-k would leave them.
template <int PER_LANE>
__device__ __forceinline__ void select_row(float (&v)[PER_LANE], int E, int lane, int n_groups, int topk_groups,
                                           int top_k, bool round_bf16, float &my_value, int &my_index) {
  uint32_t dead = 0;
#pragma unroll
  for (int j = 0; j < PER_LANE; j++)
    if (lane + 64 * j >= E) dead |= 1u << j;

  if (n_groups > 1) {
    const int per = E / n_groups;
    float gscore = 0.f;          // lane g keeps the score of group g (n_groups <= 64)
    if (per == 32 && E == 64 * PER_LANE) {
      // Groups of 32 (the DeepSeek-V3 shape): register j of lanes 0-31 is group 2j, of lanes 32-63
      // group 2j+1, so both halves reduce at once and no range scan is needed.
#pragma unroll
      for (int j = 0; j < PER_LANE; j++) {
        const cand_t mine = make_cand(v[j], lane + 64 * j);
        const cand_t b1 = half_argmax(mine, lane);
        const cand_t b2 = half_argmax(mine == b1 ? 0 : mine, lane);
        float sum = cand_value(b1) + (b2 != 0 ? cand_value(b2) : 0.f);
        if (round_bf16) sum = round_to_bf16(sum);
        const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sum), 0));
        const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sum), 32));
        if (lane == 2 * j) gscore = lo;
        if (lane == 2 * j + 1) gscore = hi;
      }
    } else {
      for (int g = 0; g < n_groups; g++) {
        const int lo = g * per, hi = lo + per;
        float sum = 0.f;
        cand_t first = 0;
        for (int pass = 0; pass < 2; pass++) {
          cand_t b = 0;
#pragma unroll
          for (int j = 0; j < PER_LANE; j++) {
            const int e = lane + 64 * j;
            const cand_t c = make_cand(v[j], e);
            if (e >= lo && e < hi && c != first && !(dead >> j & 1) && c > b) b = c;
          }
          b = wave_argmax(b);
          if (b != 0) sum = (pass == 0) ? cand_value(b) : sum + cand_value(b);
          first = b;
        }
        if (round_bf16) sum = round_to_bf16(sum);
        if (lane == g) gscore = sum;
      }
    }
    // the topk_groups best groups: lane g counts the groups that come before its own in
    // "greater score, then lower index" order
    int rank = 0;
    for (int g = 0; g < n_groups; g++) {
      const float s = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gscore), g));
      rank += (s > gscore || (s == gscore && g < lane)) ? 1 : 0;
    }
    const uint64_t keep = __ballot(lane < n_groups && rank < topk_groups);
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) {
      int e = lane + 64 * j;
      if (e < E && !(keep >> (e / per) & 1)) v[j] = -INFINITY;
    }
  }

  my_value = 0.f;
  my_index = -1;
  cand_t cand[PER_LANE];          // 0 once picked (and for elements beyond E)
#pragma unroll
  for (int j = 0; j < PER_LANE; j++) cand[j] = (dead >> j & 1) ? 0 : make_cand(v[j], lane + 64 * j);
  for (int s = 0; s < top_k; s++) {
    cand_t b = 0;
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) b = cand[j] > b ? cand[j] : b;
    b = wave_argmax(b);
    if (b == 0) break;                      // fewer than top_k elements: cannot happen (K <= E)
#pragma unroll
    for (int j = 0; j < PER_LANE; j++)
      if (cand[j] == b) cand[j] = 0;
    if (lane == s) my_index = cand_index(b);
  }
  // the value of pick `lane` as its owner holds it (element i lives in lane i % 64, register i / 64)
#pragma unroll
  for (int j = 0; j < PER_LANE; j++) {
    const float held = __shfl(v[j], my_index >= 0 ? (my_index & 63) : 0, 64);
    if (my_index >= 0 && (my_index >> 6) == j) my_value = held;
  }
}

template <int PER_LANE, bool BF16>
__global__ __launch_bounds__(256) void noaux_tc_topk_kernel(const void *__restrict__ scores, int T, int E, int n_groups,
                                                             int topk_groups, int top_k, void *__restrict__ values_out,
                                                             int32_t *__restrict__ indices_out) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= T) return;
  float v[PER_LANE];
#pragma unroll
  for (int j = 0; j < PER_LANE; j++) {
    int e = lane + 64 * j;
    float x = -INFINITY;
    if (e < E) {
      if (BF16) x = bf16_to_f32(((const uint16_t *)scores)[(size_t)t * E + e]);
      else x = ((const float *)scores)[(size_t)t * E + e];
    }
    v[j] = x;
  }
  float val;
  int idx;
  select_row<PER_LANE>(v, E, lane, n_groups, topk_groups, top_k, BF16, val, idx);
  if (lane < top_k) {
    if (BF16) ((uint16_t *)values_out)[(size_t)t * top_k + lane] = f32_to_bf16(val);
    else ((float *)values_out)[(size_t)t * top_k + lane] = val;
    indices_out[(size_t)t * top_k + lane] = idx;
  }
}

// Activation quantisation riding in the routing launch: the workgroups from `first_block` on quantise x (eight lanes
// per 128-column group) instead of routing.  Routing is a chain of cross-lane steps per token and leaves the memory
// system idle; the quantiser is pure streaming, so the two share the chip instead of following one another.
struct QuantRide {
  const uint16_t *x;      // null: nobody rides
  uint8_t *q;
  float *s;
  size_t n_groups;
  int groups_per_row;
  int pitch;
  int first_block;
};

template <int PER_LANE>
__global__ __launch_bounds__(256) void route_topk_kernel(const void *__restrict__ logits, int logits_bf16,
                                                          const float *__restrict__ bias, int T, int E, int K, int mode,
                                                          int n_groups, int topk_groups, int renorm, float scale,
                                                          float *__restrict__ weights_out, int32_t *__restrict__ ids_out,
                                                          float *__restrict__ scores_out, int n_slices = 0,
                                                          const QuantRide ride = QuantRide{},
                                                          int32_t *__restrict__ chunk_counts = nullptr) {
  if (ride.x != nullptr && (int)blockIdx.x >= ride.first_block) {
    act_quant_thread(ride.x, ride.n_groups, ride.groups_per_row, ride.pitch, ride.q, ride.s,
                     (size_t)(blockIdx.x - ride.first_block) * 256 + threadIdx.x);
    return;
  }
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= T) return;
  const bool logit_bias = mode == MOE_ROUTE_SOFTMAX_LOGIT_BIAS;
  if (logit_bias) mode = MOE_ROUTE_SOFTMAX;
  float raw[PER_LANE];   // score used for the weight (before the bias)
  float v[PER_LANE];     // score used for the selection
  float row_max = -INFINITY;
#pragma unroll
  for (int j = 0; j < PER_LANE; j++) {
    int e = lane + 64 * j;
    float x = -INFINITY;
    if (e < E) {
      if (n_slices > 0) {
        // the logits arrive as fp32 partial sums over slices of the reduction [n_slices][T][E]: added in slice
        // order and rounded to bf16, which is what a bf16 matrix product would have left
        x = round_to_bf16(sum_slices_in_order((const float *)logits + (size_t)t * E + e, (size_t)T * E, n_slices));
      } else if (logits_bf16) x = bf16_to_f32(((const uint16_t *)logits)[(size_t)t * E + e]);
      else x = ((const float *)logits)[(size_t)t * E + e];
    }
    if (mode == MOE_ROUTE_SIGMOID && e < E) x = 1.0f / (1.0f + expf(-x));
    if (logit_bias && bias != nullptr && e < E) x += bias[e];      // the bias is part of the logits
    raw[j] = x;
    row_max = fmaxf(row_max, x);
    v[j] = (!logit_bias && bias != nullptr && e < E) ? x + bias[e] : x;
    if (scores_out != nullptr && e < E && mode != MOE_ROUTE_SOFTMAX) scores_out[(size_t)t * E + e] = x;
  }
  float denom_all = 0.f;
  if (mode == MOE_ROUTE_SOFTMAX) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) row_max = fmaxf(row_max, __shfl_xor(row_max, off, 64));
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) {
      int e = lane + 64 * j;
      float p = (e < E) ? expf(raw[j] - row_max) : 0.f;
      raw[j] = p;     // un-normalised softmax numerator becomes the weight source
      denom_all += p;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) denom_all += __shfl_xor(denom_all, off, 64);
    if (scores_out != nullptr) {
#pragma unroll
      for (int j = 0; j < PER_LANE; j++) {
        int e = lane + 64 * j;
        if (e < E) scores_out[(size_t)t * E + e] = raw[j] / denom_all;
      }
    }
  }
  float val;
  int idx;
  select_row<PER_LANE>(v, E, lane, n_groups, topk_groups, K, false, val, idx);
  // weight of pick `lane`: fetch the un-biased score of element idx from its owner lane
  float w = 0.f;
#pragma unroll
  for (int j = 0; j < PER_LANE; j++) {
    // element idx lives in lane idx % 64, register idx / 64
    float cand = __shfl(raw[j], idx >= 0 ? (idx & 63) : 0, 64);
    if (idx >= 0 && (idx >> 6) == j) w = cand;
  }
  if (mode == MOE_ROUTE_SOFTMAX && !renorm) w = w / denom_all;
  if (renorm) {
    float s = (lane < K) ? w : 0.f;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    w = w / s;
  }
  if (lane < K) {
    weights_out[(size_t)t * K + lane] = w * scale;
    ids_out[(size_t)t * K + lane] = idx;
    // the permutation's first pass on the way: slots per (chunk of kChunk slots, expert); the table starts at zero
    if (chunk_counts != nullptr) atomicAdd(&chunk_counts[(size_t)((t * K + lane) / kChunk) * E + idx], 1);
  }
}

template <int PER_LANE>
static int launch_noaux(hipStream_t st, const void *scores, int dtype, int T, int E, int n_groups, int topk_groups,
                        int top_k, void *values, int32_t *indices) {
  dim3 grid((T + 3) / 4), block(256);
  if (dtype == MOE_DTYPE_BF16)
    noaux_tc_topk_kernel<PER_LANE, true><<<grid, block, 0, st>>>(scores, T, E, n_groups, topk_groups, top_k, values, indices);
  else
    noaux_tc_topk_kernel<PER_LANE, false><<<grid, block, 0, st>>>(scores, T, E, n_groups, topk_groups, top_k, values, indices);
  return (int)hipGetLastError();
}

// One workgroup per token: the short-chain form for batches of a few tokens (route_block.h).
__global__ __launch_bounds__(kRouteBlock) void route_block_kernel(const void *__restrict__ logits, int logits_bf16,
                                                                  const float *__restrict__ bias, int E, int K, int mode,
                                                                  int n_groups, int topk_groups, int renorm, float scale,
                                                                  float *__restrict__ weights_out,
                                                                  int32_t *__restrict__ ids_out,
                                                                  float *__restrict__ scores_out) {
  __shared__ __attribute__((aligned(16))) RouteBlockSmem sm;
  const size_t t = blockIdx.x;
  const void *row = logits_bf16 ? (const void *)((const uint16_t *)logits + t * E) : (const void *)((const float *)logits + t * E);
  route_block(sm, row, logits_bf16, bias, E, K, mode, n_groups, topk_groups, renorm, scale, weights_out + t * K,
              ids_out + t * K, scores_out ? scores_out + t * E : nullptr);
}

constexpr int kRouteBlockMaxTokens = 64;   // up to here a launch is latency-bound and the workgroup-per-token form wins

int check_route_shape(int T, int E, int K, int n_groups, int topk_groups) {
  if (T < 0 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > E || K > MOE_MAX_TOPK) return MOE_E_SHAPE;
  if (n_groups > 1) {
    if (n_groups > 64 || E % n_groups != 0 || topk_groups < 1 || topk_groups > n_groups) return MOE_E_SHAPE;
    if (E / n_groups < 2) return MOE_E_SHAPE;
    if ((long)topk_groups * (E / n_groups) < K) return MOE_E_SHAPE;
  }
  return MOE_OK;
}

// partial sums [n_slices][T][E] -> bf16 logits [T][E], slices added in order (the same sum the routing kernel forms)
__global__ __launch_bounds__(256) void sum_slices_kernel(const float *__restrict__ partial, int n_slices, size_t n,
                                                         uint16_t *__restrict__ logits) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  logits[i] = f32_to_bf16(sum_slices_in_order(partial + i, n, n_slices));
}

int sum_slices_launch(hipStream_t st, const float *partial, int n_slices, int T, int E, uint16_t *logits) {
  const size_t n = (size_t)T * E;
  sum_slices_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(partial, n_slices, n, logits);
  return (int)hipGetLastError();
}

// routing straight from the partial sums of the router product
// x / H / xq / xs: the activations [T, H] bf16 are quantised in the same launch (xq e4m3fn [T, H], xs fp32 with
// pitch scale_pitch(H / 128)); x null: routing only.
// chunk_counts (may be null): [ceil(T K / kChunk)][E], zero on entry; every slot is counted under its chunk and
// expert, which is the first pass of the permutation.
int route_from_partials_launch(hipStream_t st, const float *partial, int n_slices, const float *bias, int T, int E, int K,
                               int mode, int n_groups, int topk_groups, int renorm, float scale, float *weights_out,
                               int32_t *ids_out, const uint16_t *x, int H, uint8_t *xq, float *xs,
                               int32_t *chunk_counts) {
  if (n_slices < 1 || n_slices > 8) return MOE_E_SHAPE;
  if (mode != MOE_ROUTE_SOFTMAX && mode != MOE_ROUTE_SIGMOID && mode != MOE_ROUTE_SOFTMAX_LOGIT_BIAS) return MOE_E_MODE;
  const int rc = check_route_shape(T, E, K, n_groups, topk_groups);
  if (rc) return rc;
  const int route_blocks = (T + 3) / 4;
  QuantRide ride{};
  long blocks = route_blocks;
  if (x != nullptr) {
    if (H % kBlock) return MOE_E_ALIGN;
    ride.x = x; ride.q = xq; ride.s = xs;
    ride.n_groups = (size_t)T * (H / kBlock);
    ride.groups_per_row = H / kBlock;
    ride.pitch = scale_pitch(H / kBlock);
    ride.first_block = route_blocks;
    blocks += (long)((quant_threads(ride.n_groups) + 255) / 256);
  }
  if (blocks > 0x7fffffffl) return MOE_E_SHAPE;
  dim3 grid((unsigned)blocks), block(256);
#define MOE_LAUNCH_ROUTE_PARTIALS(P)                                                                               \
  route_topk_kernel<P><<<grid, block, 0, st>>>(partial, 0, bias, T, E, K, mode, n_groups, topk_groups, renorm, scale, \
                                               weights_out, ids_out, nullptr, n_slices, ride, chunk_counts)
  if (E <= 64) MOE_LAUNCH_ROUTE_PARTIALS(1);
  else if (E <= 128) MOE_LAUNCH_ROUTE_PARTIALS(2);
  else if (E <= 256) MOE_LAUNCH_ROUTE_PARTIALS(4);
  else if (E <= 512) MOE_LAUNCH_ROUTE_PARTIALS(8);
  else MOE_LAUNCH_ROUTE_PARTIALS(16);
#undef MOE_LAUNCH_ROUTE_PARTIALS
  return (int)hipGetLastError();
}

}  // namespace moe

extern "C" int moe_noaux_tc_topk(void *stream, const void *scores, int scores_dtype, int T, int E, int n_groups,
                                 int topk_groups, int top_k, void *values_out, int32_t *indices_out) {
  using namespace moe;
  if (T != 0 && (!scores || !values_out || !indices_out)) return MOE_E_NULL;
  if (scores_dtype != MOE_DTYPE_F32 && scores_dtype != MOE_DTYPE_BF16) return MOE_E_MODE;
  int rc = check_route_shape(T, E, top_k, n_groups, topk_groups);
  if (rc) return rc;
  if (T == 0) return MOE_OK;
  hipStream_t st = (hipStream_t)stream;
  if (E <= 64) return launch_noaux<1>(st, scores, scores_dtype, T, E, n_groups, topk_groups, top_k, values_out, indices_out);
  if (E <= 128) return launch_noaux<2>(st, scores, scores_dtype, T, E, n_groups, topk_groups, top_k, values_out, indices_out);
  if (E <= 256) return launch_noaux<4>(st, scores, scores_dtype, T, E, n_groups, topk_groups, top_k, values_out, indices_out);
  if (E <= 512) return launch_noaux<8>(st, scores, scores_dtype, T, E, n_groups, topk_groups, top_k, values_out, indices_out);
  return launch_noaux<16>(st, scores, scores_dtype, T, E, n_groups, topk_groups, top_k, values_out, indices_out);
}

extern "C" int moe_route_topk(void *stream, const void *logits, int logits_dtype, const float *bias, int T, int E,
                              int K, int mode, int n_groups, int topk_groups, int renorm, float scale,
                              float *weights_out, int32_t *ids_out, float *scores_out) {
  using namespace moe;
  if (T != 0 && (!logits || !weights_out || !ids_out)) return MOE_E_NULL;
  if (logits_dtype != MOE_DTYPE_F32 && logits_dtype != MOE_DTYPE_BF16) return MOE_E_MODE;
  if (mode != MOE_ROUTE_SOFTMAX && mode != MOE_ROUTE_SIGMOID && mode != MOE_ROUTE_SCORES && mode != MOE_ROUTE_SOFTMAX_LOGIT_BIAS)
    return MOE_E_MODE;
  int rc = check_route_shape(T, E, K, n_groups, topk_groups);
  if (rc) return rc;
  if (T == 0) return MOE_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((T + 3) / 4), block(256);
  const int bf = logits_dtype == MOE_DTYPE_BF16;
  if (T <= kRouteBlockMaxTokens && E <= kRouteBlock) {
    route_block_kernel<<<T, kRouteBlock, 0, st>>>(logits, bf, bias, E, K, mode, n_groups, topk_groups, renorm, scale,
                                                  weights_out, ids_out, scores_out);
    return (int)hipGetLastError();
  }
#define MOE_LAUNCH_ROUTE(P)                                                                                          \
  route_topk_kernel<P><<<grid, block, 0, st>>>(logits, bf, bias, T, E, K, mode, n_groups, topk_groups, renorm, scale, \
                                               weights_out, ids_out, scores_out)
  if (E <= 64) MOE_LAUNCH_ROUTE(1);
  else if (E <= 128) MOE_LAUNCH_ROUTE(2);
  else if (E <= 256) MOE_LAUNCH_ROUTE(4);
  else if (E <= 512) MOE_LAUNCH_ROUTE(8);
  else MOE_LAUNCH_ROUTE(16);
#undef MOE_LAUNCH_ROUTE
  return (int)hipGetLastError();
}
