// A measuring aid of the benchmark, NOT part of the product library: built into a library of its own
// (libmoe_bench_probe.so) that only bench.py loads, and declared in no public header.  What a pure read of device
// memory reaches on this GPU, with the decomposition the grouped GEMMs use for their weights - one workgroup of
// eight wavefronts streams one contiguous piece, 16 bytes per lane and load, eight loads of a lane in flight.
// bench.py reports it next to the nominal HBM peak so that a kernel's fraction of the peak can be read against what
// a kernel that does nothing else reaches.  Returns 0, a negative argument error, or a positive hipError_t.
#include "moe_common.h"

namespace moe {

__global__ __launch_bounds__(512) void hbm_read_probe_kernel(const v4i *__restrict__ p, size_t n_vec, size_t vec_per_wg,
                                                             int *__restrict__ sink) {
  const size_t lo = (size_t)blockIdx.x * vec_per_wg;
  const size_t hi = lo + vec_per_wg < n_vec ? lo + vec_per_wg : n_vec;
  v4i acc = {0, 0, 0, 0};
  constexpr int U = 8;
  size_t i = lo + threadIdx.x;
  for (; i + (size_t)(U - 1) * 512 < hi; i += (size_t)U * 512) {
    v4i v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = p[i + (size_t)u * 512];
#pragma unroll
    for (int u = 0; u < U; u++) acc ^= v[u];
  }
  for (; i < hi; i += 512) acc ^= p[i];
  // the loads must not be optimised away; the store itself practically never happens
  if ((acc[0] ^ acc[1]) == 0x5eed1234 && (acc[2] ^ acc[3]) == 0x4321deed) *sink = acc[0];
}

// The other yardstick: nothing but FP8 matrix instructions (v_mfma_f32_16x16x128_f8f6f4 on pseudo-random e4m3 operands
// that stay in registers, eight independent accumulators per wavefront, two wavefronts per SIMD).  What this reaches -
// and the package power and shader clock it reaches it at - is the matrix roof of the GPU at hand under its power cap.
__global__ __launch_bounds__(512) void mfma_probe_kernel(int iters, float *__restrict__ out) {
  v8i a, b;
  uint32_t h = (uint32_t)(blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    h = h * 1664525u + 1013904223u;
    a[i] = (int)(h & 0xfefefefeu);                  // no byte is the NaN code: bit 0 of every code is clear
    h = h * 1664525u + 1013904223u;
    b[i] = (int)(h & 0xfefefefeu);
  }
  v4f acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[i], 0, 0, 0, 0, 0, 0);
  }
  v4f s = acc[0];
#pragma unroll
  for (int i = 1; i < 8; i++) s += acc[i];
  out[(size_t)blockIdx.x * 512 + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

}  // namespace moe

// `workgroups` x 8 wavefronts x `iters` x 8 matrix instructions of 2 * 16 * 16 * 128 operations each.
// out: workgroups * 512 floats (written once, so that the work cannot be dropped).
extern "C" int bench_mfma_probe(void *stream, int workgroups, int iters, float *out) {
  if (!out) return -1;
  if (workgroups < 1 || workgroups > (1 << 20) || iters < 1) return -2;
  moe::mfma_probe_kernel<<<(unsigned)workgroups, 512, 0, (hipStream_t)stream>>>(iters, out);
  return (int)hipGetLastError();
}

extern "C" int bench_hbm_read_probe(void *stream, const void *buf, size_t bytes, size_t bytes_per_workgroup, void *sink) {
  using namespace moe;
  if (!buf || !sink) return -1;
  if (((uintptr_t)buf % 16) || ((uintptr_t)sink % 4)) return -3;
  if (bytes < 16 || bytes % 16 || bytes_per_workgroup < 16 || bytes_per_workgroup % 16) return -2;
  const size_t n_vec = bytes / 16, per = bytes_per_workgroup / 16;
  const size_t blocks = (n_vec + per - 1) / per;
  if (blocks > 0x7fffffffull) return -2;
  hbm_read_probe_kernel<<<(unsigned)blocks, 512, 0, (hipStream_t)stream>>>((const v4i *)buf, n_vec, per, (int *)sink);
  return (int)hipGetLastError();
}
