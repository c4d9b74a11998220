// The bandwidth-bound elementwise stages around the grouped GEMMs:
//   act_quant        bf16 [R, C] -> e4m3fn [R, C] + fp32 scale per row per 128 columns
//   weighted_reduce  bf16 [T, K, H] per-slot results -> bf16 [T, H], fp32 weighted sum
//   repack_weights   weight bytes row-major <-> tile-blocked (once, when a checkpoint is loaded)
// All move 16 bytes per lane per access; rows are contiguous so every access is coalesced.
#include "moe_common.h"
#include "moe_layout.h"
#include "act_quant.h"
#include "../../include/moe_hip.h"

namespace moe {

__global__ __launch_bounds__(256) void act_quant_kernel(const uint16_t *__restrict__ x, size_t n_groups,
                                                        int groups_per_row, int pitch, uint8_t *__restrict__ q,
                                                        float *__restrict__ s) {
  act_quant_thread(x, n_groups, groups_per_row, pitch, q, s, (size_t)blockIdx.x * 256 + threadIdx.x);
}

// One lane produces 8 consecutive columns of one token.  STREAM: the per-slot rows are more than the last-level cache
// holds and are read exactly once - loaded (and the result stored) with the non-temporal hint, which reads 10-12 %
// faster there; a small batch, whose rows the second GEMM has just left in the cache, keeps the plain loads.
template <bool STREAM>
__global__ __launch_bounds__(256) void weighted_reduce_kernel(const uint16_t *__restrict__ y,
                                                              const void *__restrict__ w, int w_bf16,
                                                              const uint16_t *__restrict__ shared_y,
                                                              const int32_t *__restrict__ slot_to_row, int T, int K,
                                                              int H, uint16_t *__restrict__ out) {
  const int hv = H >> 3;   // 16-byte vectors per row
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)T * hv) return;
  const int t = (int)(idx / hv), c = (int)(idx % hv) * 8;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = 0.f;
  // eight slots at a time, every load of a group asked for before the first is used.  A slot whose expert id was
  // outside [0, E) has no row (slot_to_row < 0): nothing was computed for it and it adds nothing.
  for (int k0 = 0; k0 < K; k0 += 8) {
    v4i raw[8];
    float wk[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const size_t slot = (size_t)t * K + min(k0 + i, K - 1);
      const bool live = k0 + i < K && (slot_to_row == nullptr || slot_to_row[slot] >= 0);
      // weights kept in bf16 by the caller are widened here (exact), fp32 ones taken as they are
      wk[i] = !live ? 0.f : w_bf16 ? bf16_to_f32(((const uint16_t *)w)[slot]) : ((const float *)w)[slot];
      raw[i] = STREAM ? __builtin_nontemporal_load((const v4i *)(y + slot * H + c)) : *(const v4i *)(y + slot * H + c);
      if (!live) raw[i] = (v4i){0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t u = (uint32_t)raw[i][j];
        acc[2 * j] += wk[i] * bf16_to_f32((uint16_t)(u & 0xffff));
        acc[2 * j + 1] += wk[i] * bf16_to_f32((uint16_t)(u >> 16));
      }
    }
  }
  if (shared_y != nullptr) {
    v4i raw = *(const v4i *)(shared_y + (size_t)t * H + c);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t u = (uint32_t)raw[i];
      acc[2 * i] += bf16_to_f32((uint16_t)(u & 0xffff));
      acc[2 * i + 1] += bf16_to_f32((uint16_t)(u >> 16));
    }
  }
  v4i o;
#pragma unroll
  for (int i = 0; i < 4; i++)
    o[i] = (int)((uint32_t)f32_to_bf16(acc[2 * i]) | ((uint32_t)f32_to_bf16(acc[2 * i + 1]) << 16));
  if (STREAM) __builtin_nontemporal_store(o, (v4i *)(out + (size_t)t * H + c));
  else *(v4i *)(out + (size_t)t * H + c) = o;
}

// Weight bytes between row-major order and the tile-blocked order the GEMMs read.  Tile-blocked: the matrix is cut
// into tiles of 16 rows and steps of 128 bytes; the 2 KB of a (tile, step) pair are contiguous, tiles in row order,
// a tile's steps one after the other, and inside the 2 KB: half h (0/1), then lane l (0..63), 16 bytes each =
// row l % 16 of the tile, bytes 16 * (l / 16 + 4 h) .. + 15 of the step - a wavefront's operand of the 16x16x128
// matrix instruction, so that a load instruction reads 1 KB of consecutive memory.  One thread moves 16 bytes;
// the tile-blocked side is the coalesced one.
__global__ __launch_bounds__(256) void repack_weights_kernel(const v4i *__restrict__ src, v4i *__restrict__ dst,
                                                             size_t n_units, int nkb, int row_units, bool to_blocked) {
  const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;      // 16-byte unit in tile-blocked order
  if (o >= n_units) return;
  const size_t block = o >> 7;
  const int u = (int)(o & 127), h = u >> 6, l = u & 63, r = l & 15, g = l >> 4;
  const size_t tile = block / nkb;
  const int kb = (int)(block % nkb);
  const size_t rm = (tile * 16 + r) * (size_t)row_units + (size_t)kb * 8 + g + 4 * h;   // the same unit in row-major order
  if (to_blocked) dst[o] = src[rm];
  else dst[rm] = src[o];
}

static int repack_launch(hipStream_t st, const void *src, int64_t rows, int row_bytes, void *dst, bool to_blocked) {
  if (rows < 0 || row_bytes < 1) return MOE_E_SHAPE;
  if (rows % 16 || row_bytes % kBlock) return MOE_E_ALIGN;
  if (rows == 0) return MOE_OK;
  if (!src || !dst) return MOE_E_NULL;
  if (src == dst) return MOE_E_MODE;                             // not an in-place operation
  if (((uintptr_t)src % 16) || ((uintptr_t)dst % 16)) return MOE_E_ALIGN;
  const size_t n_units = (size_t)rows * (row_bytes / 16);
  const size_t blocks = (n_units + 255) / 256;
  if (blocks > 0x7fffffffull) return MOE_E_SHAPE;
  repack_weights_kernel<<<(unsigned)blocks, 256, 0, st>>>((const v4i *)src, (v4i *)dst, n_units, row_bytes / kBlock,
                                                          row_bytes / 16, to_blocked);
  return (int)hipGetLastError();
}

// slot_to_row (may be null): slots with a negative entry are left out of the sum; w: [T, K] fp32, or bf16 with w_bf16
int weighted_reduce_launch(hipStream_t st, const uint16_t *y, const void *w, const uint16_t *shared_y,
                           const int32_t *slot_to_row, int T, int K, int H, uint16_t *out, int w_bf16) {
  const size_t n = (size_t)T * (H / 8);
  if (n == 0) return MOE_OK;
  const size_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffull) return MOE_E_SHAPE;
  // 256 MB of last-level cache on this GPU
  if ((size_t)T * K * H * 2 > ((size_t)256 << 20))
    weighted_reduce_kernel<true><<<(unsigned)blocks, 256, 0, st>>>(y, w, w_bf16, shared_y, slot_to_row, T, K, H, out);
  else
    weighted_reduce_kernel<false><<<(unsigned)blocks, 256, 0, st>>>(y, w, w_bf16, shared_y, slot_to_row, T, K, H, out);
  return (int)hipGetLastError();
}

}  // namespace moe

extern "C" int moe_pack_weights(void *stream, const void *w_rowmajor, int64_t rows, int row_bytes, void *w_blocked) {
  return moe::repack_launch((hipStream_t)stream, w_rowmajor, rows, row_bytes, w_blocked, true);
}

extern "C" int moe_unpack_weights(void *stream, const void *w_blocked, int64_t rows, int row_bytes, void *w_rowmajor) {
  return moe::repack_launch((hipStream_t)stream, w_blocked, rows, row_bytes, w_rowmajor, false);
}

extern "C" int moe_scale_pitch(int n_groups) { return n_groups < 0 ? 0 : moe::scale_pitch(n_groups); }

extern "C" int moe_act_quant(void *stream, const void *x_bf16, int R, int C, uint8_t *q, float *s) {
  using namespace moe;
  if (R != 0 && (!x_bf16 || !q || !s)) return MOE_E_NULL;
  if (R < 0 || C < 1) return MOE_E_SHAPE;
  if (C % kBlock) return MOE_E_ALIGN;
  if (((uintptr_t)x_bf16 % 16) || ((uintptr_t)q % 16) || ((uintptr_t)s % 64)) return MOE_E_ALIGN;
  const size_t groups = (size_t)R * (C / kBlock);
  if (groups == 0) return MOE_OK;
  const size_t blocks = (quant_threads(groups) + 255) / 256;
  if (blocks > 0x7fffffffull) return MOE_E_SHAPE;
  act_quant_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint16_t *)x_bf16, groups, C / kBlock,
                                                                      scale_pitch(C / kBlock), q, s);
  return (int)hipGetLastError();
}

extern "C" int moe_weighted_reduce(void *stream, const void *y_bf16, const float *routing_weights,
                                   const void *shared_y_bf16, int T, int K, int H, void *out_bf16) {
  using namespace moe;
  if (T != 0 && (!y_bf16 || !routing_weights || !out_bf16)) return MOE_E_NULL;
  if (T < 0 || K < 1 || H < 1) return MOE_E_SHAPE;
  if (H % 8) return MOE_E_ALIGN;
  if (((uintptr_t)y_bf16 % 16) || ((uintptr_t)out_bf16 % 16) || (shared_y_bf16 && ((uintptr_t)shared_y_bf16 % 16)))
    return MOE_E_ALIGN;
  return weighted_reduce_launch((hipStream_t)stream, (const uint16_t *)y_bf16, routing_weights,
                                (const uint16_t *)shared_y_bf16, nullptr, T, K, H, (uint16_t *)out_bf16, 0);
}
