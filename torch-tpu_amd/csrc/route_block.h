// Routing of ONE token by a whole 256-thread workgroup (E <= 256), for batches so small that the
// time of a launch is the length of its longest dependent chain, not its instruction count.
//
// Thread e owns expert e.  Instead of K arg-max rounds in sequence, every thread counts the
// experts that come before its own in "greater score, then lower index" order: that count is the
// expert's position in the sorted row, so the K picks are the threads whose count is below K, and
// they come out in descending order.  The order is one unsigned 64-bit compare per pair: the
// score mapped to an unsigned integer of the same order in the high half, "lower index first" in
// the low half (compare masks combined on the scalar side cost several times as much).  The group limit works the same way: position inside the
// group (0 and 1 make the group's score), then position of the group among the groups.  All reads
// of the score table are LDS broadcasts.  Orders, sums and divisions are those of the
// one-wavefront-per-token kernel, so both give the same ids and the same weights, bit for bit.
#pragma once
#include "moe_common.h"
#include "../../include/moe_hip.h"

namespace moe {

constexpr int kRouteBlock = 256;

struct RouteBlockSmem {
  uint64_t key[kRouteBlock];   // order key of every expert's selection score (0 beyond E: after everything)
  float raw[kRouteBlock];      // softmax numerators
  float gtop[64][2];           // best two selection scores of every group
  uint64_t gkey[64];           // order key of every group's score
  float wmax[kRouteBlock / 64];
  float wsel[64];              // weight source of pick k
  int isel[64];                // expert of pick k
};

// (score a, index ai) comes before (b, bi) - greater score, then lower index - exactly when
// order_key(a, ai) > order_key(b, bi).  Adding +0 first makes -0 and +0 the same key, as they compare equal.
__device__ __forceinline__ uint64_t order_key(float v, int idx) {
  uint32_t u = __float_as_uint(v + 0.0f);
  u = (u >> 31) ? ~u : (u | 0x80000000u);
  return ((uint64_t)u << 32) | (uint32_t)(0x7fffffff - idx);
}

__device__ __forceinline__ void route_block(RouteBlockSmem &sm, const void *logits_row, int logits_bf16,
                                            const float *__restrict__ bias, int E, int K, int mode, int n_groups,
                                            int topk_groups, int renorm, float scale, float *weights_row,
                                            int32_t *ids_row, float *scores_row) {
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6;
  const bool live = e < E;
  float x = -INFINITY;
  if (live) x = logits_bf16 ? bf16_to_f32(((const uint16_t *)logits_row)[e]) : ((const float *)logits_row)[e];
  if (mode == MOE_ROUTE_SIGMOID && live) x = 1.0f / (1.0f + expf(-x));
  const bool logit_bias = mode == MOE_ROUTE_SOFTMAX_LOGIT_BIAS;     // the bias is part of the logits
  if (logit_bias) {
    mode = MOE_ROUTE_SOFTMAX;
    if (bias != nullptr && live) x += bias[e];
    bias = nullptr;
  }
  float raw = x;                                          // what the weight is made of (no bias)
  float v = (bias != nullptr && live) ? x + bias[e] : x;  // what the selection looks at
  if (scores_row != nullptr && live && mode != MOE_ROUTE_SOFTMAX) scores_row[e] = x;
  if (e < 64) { sm.isel[e] = -1; sm.wsel[e] = 0.f; }
  float denom_all = 0.f;
  if (mode == MOE_ROUTE_SOFTMAX) {
    float m = x;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) sm.wmax[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sm.wmax[0], sm.wmax[1]), fmaxf(sm.wmax[2], sm.wmax[3]));
    raw = live ? expf(x - m) : 0.f;
    sm.raw[e] = raw;
    __syncthreads();
    // the sum in the order the per-wavefront kernel uses: lane l adds elements l, l+64, l+128, l+192, then a butterfly
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < kRouteBlock / 64; j++) part += sm.raw[lane + 64 * j];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) part += __shfl_xor(part, off, 64);
    denom_all = part;
    if (scores_row != nullptr && live) scores_row[e] = raw / denom_all;
  }
  uint64_t key = live ? order_key(v, e) : 0;
  sm.key[e] = key;
  __syncthreads();

  if (n_groups > 1) {
    const int per = E / n_groups, g = live ? e / per : 0;
    if (live) {
      int r = 0;
#pragma unroll 8
      for (int j = g * per; j < g * per + per; j++) r += sm.key[j] > key;
      if (r < 2) sm.gtop[g][r] = v;
    }
    __syncthreads();
    if (e < n_groups) sm.gkey[e] = order_key(sm.gtop[e][0] + sm.gtop[e][1], e);
    __syncthreads();
    if (live) {
      const uint64_t gk = sm.gkey[g];
      int r = 0;
#pragma unroll 8
      for (int h = 0; h < n_groups; h++) r += sm.gkey[h] > gk;
      if (r >= topk_groups) {     // dropped groups stay candidates with -inf, as a masked_fill would leave them
        v = -INFINITY;
        key = order_key(v, e);
      }
    }
    sm.key[e] = key;        // every read of the unmasked table happened before the barrier above
    __syncthreads();
  }

  if (live) {
    int r = 0;
#pragma unroll 16
    for (int j = 0; j < kRouteBlock; j++) r += sm.key[j] > key;     // the whole table, so that the reads pipeline
    if (r < K) { sm.isel[r] = e; sm.wsel[r] = raw; }
  }
  __syncthreads();
  if (wave == 0) {
    float w = lane < K ? sm.wsel[lane] : 0.f;
    const int idx = lane < K ? sm.isel[lane] : -1;
    if (mode == MOE_ROUTE_SOFTMAX && !renorm) w = w / denom_all;
    if (renorm) {
      float s = w;
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
      w = w / s;
    }
    if (lane < K) {
      weights_row[lane] = w * scale;
      ids_row[lane] = idx;
    }
  }
}

}  // namespace moe
