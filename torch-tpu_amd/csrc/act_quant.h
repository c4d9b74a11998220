// Activation quantisation of one 128-column group by 16 neighbouring lanes, as a device function:
// shared by the stand-alone kernel and by the decode-size kernel that also computes the router logits.
#pragma once
#include "moe_common.h"

namespace moe {

// Thread `index` of a flat launch: group index / 16, 8 bf16 (16 bytes) per lane.  Every lane of a
// wavefront must call it (the maximum is taken with cross-lane moves); lanes past the end do nothing.
__device__ __forceinline__ void act_quant_thread(const uint16_t *__restrict__ x, size_t n_groups, int groups_per_row,
                                                 int pitch, uint8_t *__restrict__ q, float *__restrict__ s,
                                                 size_t index) {
  const size_t g = index >> 4;
  const int sub = (int)(index & 15);
  const bool live = g < n_groups;
  float f[8];
  float amax = 0.f;
  if (live) {
    v4i raw = *(const v4i *)(x + g * kBlock + sub * 8);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t w = (uint32_t)raw[i];
      f[2 * i] = bf16_to_f32((uint16_t)(w & 0xffff));
      f[2 * i + 1] = bf16_to_f32((uint16_t)(w >> 16));
    }
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(f[i]));
  }
  amax = max_over_row16(amax);
  if (!live) return;
  const float sc = group_scale(amax);
  v2i out;
  out[0] = (int)pack4_fp8(f[0] / sc, f[1] / sc, f[2] / sc, f[3] / sc);
  out[1] = (int)pack4_fp8(f[4] / sc, f[5] / sc, f[6] / sc, f[7] / sc);
  *(v2i *)(q + g * kBlock + sub * 8) = out;
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
  __host__ __device__ unsigned blocks() const { return x ? (unsigned)((n_groups * 16 + 255) / 256) : 0u; }
};

}  // namespace moe
