// Shared device helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moe {

constexpr int kWave = 64;
constexpr int kBlock = 128;          // quantisation block edge / activation group width
constexpr float kFp8Max = 448.0f;
constexpr float kActEps = 1e-10f;

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float clamp_fp8(float v) { return fminf(fmaxf(v, -kFp8Max), kFp8Max); }

// four fp32 -> four e4m3fn bytes packed little-endian (element 0 in the low byte)
__device__ __forceinline__ uint32_t pack4_fp8(float a, float b, float c, float d) {
  int p = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_fp8(a), clamp_fp8(b), 0, false);
  p = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_fp8(c), clamp_fp8(d), p, true);
  return (uint32_t)p;
}

// scale of one 128-wide activation group from its absolute maximum
__device__ __forceinline__ float group_scale(float amax) { return fmaxf(amax, kActEps) / kFp8Max; }

// x / sc for the activation quantiser without the IEEE division sequence (ten-odd instructions per element): the
// reciprocal of the scale, refined once, serves all elements of the group; a quotient costs a multiply and one
// correction (remainder by fused multiply-add, then folded in).  The quantiser's whole domain is small - x any bf16
// value, sc the scale of any bf16 amax >= |x| - and over all of it the e4m3fn code of this quotient equals the code
// of the IEEE quotient (checked pair by pair on the device by the tests).
struct ScaleRecip {
  float sc, y;
};
__device__ __forceinline__ ScaleRecip scale_recip(float sc) {
  const float y = __builtin_amdgcn_rcpf(sc);
  return {sc, fmaf(fmaf(-sc, y, 1.0f), y, y)};
}
__device__ __forceinline__ float div_by_scale(float x, const ScaleRecip r) {
  const float q = x * r.y;
  return __builtin_copysignf(fmaf(fmaf(-q, r.sc, x), r.y, q), x);      // (the correction would turn -0 into +0)
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

// silu on the hardware's exp2 and reciprocal (a few ulp; two instructions instead of a division sequence)
__device__ __forceinline__ float silu_fast(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }

// two fp32 -> two bf16 (round to nearest even) in one instruction, first value in the low half
typedef float v2f_t __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f_t){lo, hi}, v2bf_t));
}

// max over the lanes that share (lane % 16): butterflies over lane bits 4 and 5
__device__ __forceinline__ float max_over_lane_groups(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// max over the 16 lanes of a row (lane bits 0..3)
__device__ __forceinline__ float max_over_row16(float v) {
  v = fmaxf(v, __shfl_xor(v, 1, 64));
  v = fmaxf(v, __shfl_xor(v, 2, 64));
  v = fmaxf(v, __shfl_xor(v, 4, 64));
  v = fmaxf(v, __shfl_xor(v, 8, 64));
  return v;
}

// max over 8 neighbouring lanes (lane bits 0..2)
__device__ __forceinline__ float max_over_row8(float v) {
  v = fmaxf(v, __shfl_xor(v, 1, 64));
  v = fmaxf(v, __shfl_xor(v, 2, 64));
  v = fmaxf(v, __shfl_xor(v, 4, 64));
  return v;
}

}  // namespace moe
