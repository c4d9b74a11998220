// Activation quantisation of one 128-column group by a few neighbouring lanes, as a device function:
// shared by the stand-alone kernel and by the decode-size kernel that also computes the router logits.
#pragma once
#include "moe_common.h"

namespace moe {

// A group is quantised by kQuantLanes neighbouring lanes, 16 bf16 (32 bytes) per lane: a wavefront reads 2 KB and
// writes 1 KB of consecutive memory.
constexpr int kQuantLanes = 8;
// threads of a flat launch that quantises n_groups groups
__host__ __device__ inline size_t quant_threads(size_t n_groups) { return n_groups * kQuantLanes; }

// Thread `index` of such a launch.  Every lane of a wavefront must call it (the maximum is taken with cross-lane
// moves); lanes past the end do nothing.
__device__ __forceinline__ void act_quant_thread(const uint16_t *__restrict__ x, size_t n_groups, int groups_per_row,
                                                 int pitch, uint8_t *__restrict__ q, float *__restrict__ s,
                                                 size_t index) {
  const size_t g = index / kQuantLanes;
  const int sub = (int)(index % kQuantLanes);
  const bool live = g < n_groups;
  float f[16];
  float amax = 0.f;
  if (live) {
    const v4i *src = (const v4i *)(x + g * kBlock + sub * 16);
    const v4i raw[2] = {src[0], src[1]};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      uint32_t w = (uint32_t)raw[i >> 2][i & 3];
      f[2 * i] = bf16_to_f32((uint16_t)(w & 0xffff));
      f[2 * i + 1] = bf16_to_f32((uint16_t)(w >> 16));
    }
#pragma unroll
    for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(f[i]));
  }
  amax = max_over_row8(amax);
  if (!live) return;
  const float sc = group_scale(amax);
  const ScaleRecip r = scale_recip(sc);
  v4i out;
#pragma unroll
  for (int i = 0; i < 4; i++)
    out[i] = (int)pack4_fp8(div_by_scale(f[4 * i], r), div_by_scale(f[4 * i + 1], r), div_by_scale(f[4 * i + 2], r),
                            div_by_scale(f[4 * i + 3], r));
  *(v4i *)(q + g * kBlock + sub * 16) = out;
  if (sub == 0) s[(g / groups_per_row) * pitch + g % groups_per_row] = sc;
}

// A quantisation job that rides in another kernel's launch as extra workgroups of 256 threads (x null: none).
struct QuantJob {
  const uint16_t *x;      // [rows, groups_per_row * 128] bf16
  uint8_t *q;             // e4m3fn, same shape
  float *s;               // [rows, pitch] fp32
  size_t n_groups;
  int groups_per_row;
  int pitch;
  __host__ __device__ unsigned blocks() const { return x ? (unsigned)((quant_threads(n_groups) + 255) / 256) : 0u; }
};

}  // namespace moe
