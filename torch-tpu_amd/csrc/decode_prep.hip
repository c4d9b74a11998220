// Everything in front of the grouped GEMMs for a decode-size batch (T*K <= 256 slots, E <= 256), in two launches
// instead of five.  At this size every stage is one dependent chain long, so what counts is the number of launches
// and the length of each chain, not the instruction count.
//
//   router_logits_quant   workgroup (e, token block): the dot products of router row e with up to 8 tokens, the
//                         reduction dimension split over the four wavefronts (every load of a wavefront is in
//                         flight at once), fp32 sums rounded to bf16 as a bf16 matmul would leave them.
//                         The workgroups after those quantise the activations (the stage the GEMMs need next to
//                         the routing), and the first one clears the arrival counter of the second launch.
//   route_permute_small   workgroup t routes token t (route_block.h).  The workgroup that arrives last - an atomic
//                         counter, no waiting - sees every token's picks and builds the permutation and the tile list.
#include "moe_common.h"
#include "moe_layout.h"
#include "act_quant.h"
#include "permute_small.h"
#include "route_block.h"
#include "../../include/moe_hip.h"

namespace moe {

constexpr int kLogitTokens = 8;      // tokens per workgroup of the logits kernel
constexpr int kLogitSpan = 2048;     // reduction elements one workgroup pass covers: 256 lanes x 8 bf16

__device__ __forceinline__ void unpack8(const v4i raw, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t w = (uint32_t)raw[i];
    f[2 * i] = __uint_as_float(w << 16);
    f[2 * i + 1] = __uint_as_float(w & 0xffff0000u);
  }
}

template <int PASSES>
__device__ __forceinline__ void dot_rows(const uint16_t *__restrict__ wrow, const uint16_t *__restrict__ x, int H, int T,
                                         int t0, int c0, float (&acc)[kLogitTokens]) {
  v4i wv[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; p++) {
    const int c = c0 + p * kLogitSpan;
    wv[p] = c < H ? *(const v4i *)(wrow + c) : (v4i){0, 0, 0, 0};
  }
#pragma unroll
  for (int i = 0; i < kLogitTokens; i++) {
    if (t0 + i >= T) break;
    const uint16_t *xrow = x + (size_t)(t0 + i) * H;
    v4i xv[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
      const int c = c0 + p * kLogitSpan;
      xv[p] = c < H ? *(const v4i *)(xrow + c) : (v4i){0, 0, 0, 0};
    }
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
      float wf[8], xf[8];
      unpack8(wv[p], wf);
      unpack8(xv[p], xf);
#pragma unroll
      for (int j = 0; j < 8; j++) acc[i] = fmaf(wf[j], xf[j], acc[i]);
    }
  }
}

__global__ __launch_bounds__(256) void router_logits_quant_kernel(const uint16_t *__restrict__ x,
                                                                  const uint16_t *__restrict__ wr, int T, int H, int E,
                                                                  uint16_t *__restrict__ logits, int n_logit_blocks,
                                                                  size_t n_groups, int groups_per_row, int pitch,
                                                                  uint8_t *__restrict__ xq, float *__restrict__ xs,
                                                                  int *__restrict__ arrivals) {
  if ((int)blockIdx.x >= n_logit_blocks) {
    act_quant_thread(x, n_groups, groups_per_row, pitch, xq, xs, (size_t)(blockIdx.x - n_logit_blocks) * 256 + threadIdx.x);
    return;
  }
  __shared__ float part[4][kLogitTokens];
  if (blockIdx.x == 0 && threadIdx.x == 0) *arrivals = 0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = blockIdx.x % E, t0 = (blockIdx.x / E) * kLogitTokens;
  const uint16_t *wrow = wr + (size_t)e * H;
  float acc[kLogitTokens];
#pragma unroll
  for (int i = 0; i < kLogitTokens; i++) acc[i] = 0.f;
  for (int c0 = threadIdx.x * 8; c0 < H; c0 += 4 * kLogitSpan) dot_rows<4>(wrow, x, H, T, t0, c0, acc);
#pragma unroll
  for (int i = 0; i < kLogitTokens; i++) {
    float s = acc[i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) part[wave][i] = s;
  }
  __syncthreads();
  if (threadIdx.x < kLogitTokens && t0 + (int)threadIdx.x < T) {
    const int i = threadIdx.x;
    const float s = ((part[0][i] + part[1][i]) + part[2][i]) + part[3][i];
    logits[(size_t)(t0 + i) * E + e] = f32_to_bf16(s);
  }
}

__global__ __launch_bounds__(kRouteBlock) void route_permute_small_kernel(
    const uint16_t *__restrict__ logits, const float *__restrict__ bias, int T, int E, int K, int mode, int n_groups,
    int topk_groups, int renorm, float scale, float *__restrict__ weights, int32_t *__restrict__ ids,
    int *__restrict__ arrivals, int tile_m, int max_tiles, int32_t *__restrict__ sorted_slot,
    int32_t *__restrict__ expert_offsets, int32_t *__restrict__ slot_to_row, int32_t *__restrict__ tile_prefix,
    int32_t *__restrict__ tile_expert, int32_t *__restrict__ tile_desc) {
  static_assert(kRouteBlock == kChunk, "the last workgroup permutes with the threads it routed with");
  __shared__ __attribute__((aligned(16))) RouteBlockSmem rs;
  __shared__ PermuteSmallSmem ps;
  __shared__ int is_last;
  const int t = blockIdx.x;
  route_block(rs, logits + (size_t)t * E, 1, bias, E, K, mode, n_groups, topk_groups, renorm, scale,
              weights + (size_t)t * K, ids + (size_t)t * K, nullptr);
  const int s = threadIdx.x, TK = T * K;
  int v;
  if (gridDim.x == 1) {
    v = s < TK ? rs.isel[s] : -1;       // one token: its picks are still in LDS
  } else {
    // this token's picks are visible device-wide before the arrival is counted: one fence per workgroup, by the
    // thread that counts, after the barrier that orders the other wavefronts' stores before it
    __syncthreads();
    if (threadIdx.x == 0) {
      __threadfence();
      is_last = atomicAdd(arrivals, 1) == (int)gridDim.x - 1;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();
    v = s < TK ? __hip_atomic_load(ids + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : -1;
  }
  permute_small_block(ps, v, TK, E, tile_m, max_tiles, sorted_slot, expert_offsets, slot_to_row, tile_prefix, tile_expert,
                      tile_desc);
}

int check_route_shape(int T, int E, int K, int n_groups, int topk_groups);

// x [T,H] bf16, wr [E,H] bf16 -> logits [T,E] bf16, weights [T,K], ids [T,K], the quantised activations and
// the permutation.  The caller has checked pointers and alignment.
int decode_prep_launch(hipStream_t st, const uint16_t *x, int T, int H, const uint16_t *wr, const float *bias, int E, int K,
                       int mode, int n_groups, int topk_groups, int renorm, float scale, uint16_t *logits, float *weights,
                       int32_t *ids, int *arrivals, uint8_t *xq, float *xs, int tile_m, int32_t *sorted_slot,
                       int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &pw) {
  if (T < 1 || (long)T * K > kChunk || E > kRouteBlock || H % kBlock) return MOE_E_SHAPE;
  if (mode != MOE_ROUTE_SOFTMAX && mode != MOE_ROUTE_SIGMOID && mode != MOE_ROUTE_SOFTMAX_LOGIT_BIAS) return MOE_E_MODE;
  const int rc = check_route_shape(T, E, K, n_groups, topk_groups);
  if (rc) return rc;
  const int n_logit_blocks = E * ((T + kLogitTokens - 1) / kLogitTokens);
  const size_t groups = (size_t)T * (H / kBlock);
  const int quant_blocks = (int)((quant_threads(groups) + 255) / 256);
  router_logits_quant_kernel<<<n_logit_blocks + quant_blocks, 256, 0, st>>>(x, wr, T, H, E, logits, n_logit_blocks, groups,
                                                                           H / kBlock, scale_pitch(H / kBlock), xq, xs,
                                                                           arrivals);
  route_permute_small_kernel<<<T, kRouteBlock, 0, st>>>(logits, bias, T, E, K, mode, n_groups, topk_groups, renorm, scale,
                                                        weights, ids, arrivals, tile_m, pw.max_tiles, sorted_slot,
                                                        expert_offsets, slot_to_row, pw.tile_prefix, pw.tile_expert,
                                                        pw.tile_desc);
  return (int)hipGetLastError();
}

}  // namespace moe
