// Router logits for batches beyond the decode size (and for any batch of a layer with more than 256 experts):
// logits[T, E] = x[T, H] . Wr[E, H]^T in bf16 on the matrix cores, E <= 1024 in blocks of 256 experts.
//
// The product is short and wide (a few thousand tokens by at most 256 experts over a long reduction), so the
// reduction is cut into slices: workgroup (block of 128 tokens, slice) leaves its fp32 partial sums, and the routing
// kernel that follows adds the slices in a fixed order, rounds to bf16 (what a bf16 matmul leaves) and routes.
// Eight wavefronts, two per SIMD, so that one's LDS reads and barrier waits hide behind the other's matrix
// instructions: wavefront (token half, expert quarter) owns 64 tokens x 64 experts of the workgroup's 128 tokens x
// block of 256 experts (4 x 4 tiles of 16 x 16; with fewer tokens per workgroup the router rows, re-read by every
// token block, saturate the L2 -> LDS path before the matrix pipe).  A step is 64 reduction elements = 128 bytes of a
// row = two v_mfma_f32_16x16x32_bf16 per tile pair.  Both operands travel L2 -> LDS with direct loads, two steps
// ahead, through three stages, one barrier per step.
#include "moe_common.h"
#include "moe_layout.h"
#include "../../include/moe_hip.h"

namespace moe {

typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));

constexpr int kRfTokens = 128;                // tokens per workgroup
constexpr int kRfMT = kRfTokens / 16;
constexpr int kRfXStages = 3, kRfWStages = 3;

template <int EB>
struct RfSmem {
  alignas(1024) uint8_t x[kRfXStages][kRfTokens * 128];   // [row][16-byte chunk, XOR-swizzled by row % 8]
  alignas(1024) uint8_t w[kRfWStages][EB * 128];
};

typedef __attribute__((address_space(3))) uint8_t rf_lds_byte;
__device__ __forceinline__ uint32_t rf_lds_offset(const void *p) { return (uint32_t)(uintptr_t)(rf_lds_byte *)p; }

constexpr int kRfThreads = 512;

// EB: experts per workgroup (256; 128 or 64 for a layer with no more experts than that, so that nothing is loaded or
// multiplied for rows that do not exist); a wavefront owns EB / 4 of them
template <int EB>
__global__ __launch_bounds__(kRfThreads) void router_logits_splitk_kernel(const uint8_t *__restrict__ x,
                                                                   const uint8_t *__restrict__ wr, int T, int H, int E,
                                                                   int n_slices, int blocks_per_slice, int n_eblocks,
                                                                   float *__restrict__ partial,
                                                                   int32_t *__restrict__ zero, int n_zero) {
  constexpr int EQ = EB / 4;                              // experts of a wavefront
  constexpr int NJ = EQ / 16;                             // its expert tiles
  __shared__ RfSmem<EB> sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // the counters of the permutation that follows start at zero (the routing kernel adds to them)
  for (int i = blockIdx.x * kRfThreads + tid; i < n_zero; i += gridDim.x * kRfThreads) zero[i] = 0;
  const int li = lane & 15, lg = lane >> 4;
  const int wm = wave & 1, wn = wave >> 1;                // token half, expert quarter
  // workgroup id = ((token block) * n_eblocks + expert block) * n_slices + slice: the workgroups that share a token
  // block, and then an expert block, are neighbours in launch order
  const int slice = blockIdx.x % n_slices, eb = (blockIdx.x / n_slices) % n_eblocks, e0 = eb * EB;
  const int m0 = (blockIdx.x / (n_slices * n_eblocks)) * kRfTokens;
  const int nblk = H >> 7;
  const int b0 = slice * blocks_per_slice, b1 = min(nblk, b0 + blocks_per_slice);
  const int n_steps = 2 * (b1 - b0);                      // steps of 64 elements
  if (n_steps <= 0) return;
  const size_t row_bytes = (size_t)H * 2;
  const uint8_t *const xbase = x + (size_t)b0 * 256;      // first byte of the slice in a row
  const uint8_t *const wbase = wr + (size_t)b0 * 256;

  // direct-to-LDS loads: one instruction moves 8 rows x 128 bytes; lane l fetches row l/8 and the chunk that
  // belongs at position l%8 of the swizzled row
  const int sub = lane >> 3, chunk = (lane & 7) ^ sub;
  constexpr int NX = kRfTokens / 64, NWR = (EB / 8 + 7) / 8;   // token-tile and router-row instructions per wavefront and step
  uint32_t x_src[NX], w_src[NWR];
#pragma unroll
  for (int u = 0; u < NX; u++) x_src[u] = (uint32_t)min(m0 + 8 * (NX * wave + u) + sub, T - 1) * (uint32_t)row_bytes + chunk * 16;
#pragma unroll
  for (int u = 0; u < NWR; u++)      // (64 experts: eight pieces, one per wavefront)
    w_src[u] = (uint32_t)min(e0 + 8 * min(NWR * wave + u, EB / 8 - 1) + sub, E - 1) * (uint32_t)row_bytes + chunk * 16;
  const uint32_t x_lds = __builtin_amdgcn_readfirstlane(rf_lds_offset(&sm.x[0][0])) + (NX * wave) * 1024;
  const uint32_t w_lds = __builtin_amdgcn_readfirstlane(rf_lds_offset(&sm.w[0][0])) + min(NWR * wave, EB / 8 - 1) * 1024;
  auto request = [&](int step) {
    const uint8_t *xb = xbase + (size_t)step * 128, *wb = wbase + (size_t)step * 128;
    const uint32_t xm = x_lds + (step % kRfXStages) * (kRfTokens * 128), wst = w_lds + (step % kRfWStages) * (EB * 128);
#pragma unroll
    for (int u = 0; u < NX; u++)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(xm + u * 1024), "v"(x_src[u]), "s"(xb) : "memory", "m0");
#pragma unroll
    for (int u = 0; u < NWR; u++)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(wst + u * 1024), "v"(w_src[u]), "s"(wb) : "memory", "m0");
  };
  constexpr int kLoadsPerStep = NX + NWR;
  constexpr int kWaveMT = kRfMT / 2;              // row tiles of a wavefront

  v4f acc[kWaveMT][NJ];
#pragma unroll
  for (int i = 0; i < kWaveMT; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int last = n_steps - 1;
  request(0);
  request(min(1, last));
  const int o0 = (lg ^ (li & 7)) << 4, o1 = ((lg + 4) ^ (li & 7)) << 4;
  for (int t = 0; t < n_steps; t++) {
    // step t has landed (step t + 1 may still be in flight); everybody has left step t - 1, whose stages the
    // request below overwrites
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerStep) : "memory");
    __syncthreads();
    request(min(t + 2, last));          // past the end: the last step again, so that the count in flight stays the same
    const uint8_t *xs = sm.x[t % kRfXStages] + (64 * wm + li) * 128;
    const uint8_t *ws = sm.w[t % kRfWStages] + (EQ * wn + li) * 128;
    v4i xa[kWaveMT][2], wb[NJ][2];
#pragma unroll
    for (int i = 0; i < NJ; i++) {
      wb[i][0] = *(const v4i *)(ws + i * 2048 + o0);
      wb[i][1] = *(const v4i *)(ws + i * 2048 + o1);
    }
#pragma unroll
    for (int i = 0; i < kWaveMT; i++) {
      xa[i][0] = *(const v4i *)(xs + i * 2048 + o0);
      xa[i][1] = *(const v4i *)(xs + i * 2048 + o1);
    }
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int i = 0; i < kWaveMT; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, xa[i][h]),
                                                              __builtin_bit_cast(v8bf_t, wb[j][h]), acc[i][j], 0, 0, 0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // c[r] of tile (i, j): token m0 + 64 wm + 16 i + 4 (l / 16) + r, expert e0 + EQ wn + 16 j + l % 16
  float *const out = partial + (size_t)slice * T * E;
#pragma unroll
  for (int i = 0; i < kWaveMT; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int tok = m0 + 64 * wm + 16 * i + 4 * lg + r;
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        const int e = e0 + EQ * wn + 16 * j + li;
        if (tok < T && e < E) out[(size_t)tok * E + e] = acc[i][j][r];
      }
    }
}

// how the reduction is cut: a workgroup for every compute unit (144 KB of LDS: one fits), slices of whole 128-column
// blocks.  Two rounds of shorter workgroups lose to one round of longer ones, and every slice is another 4 T E bytes
// for the routing kernel to read (Qwen3 shape, T=16384: router product 29.9 -> 24.6 us, routing 43.9 -> 41.6 us with
// two slices instead of four; one slice, half the units busy: 36 us)
void router_front_plan(int T, int H, int E, int *n_slices, int *blocks_per_slice) {
  const int mblocks = (T + kRfTokens - 1) / kRfTokens * ((E + 255) / 256), nblk = H / kBlock;
  int s = (256 + mblocks - 1) / mblocks;                  // one workgroup per compute unit
  if (s < 1) s = 1;
  if (s > 8) s = 8;
  if (s > nblk) s = nblk;
  const int per = (nblk + s - 1) / s;
  *blocks_per_slice = per;
  *n_slices = (nblk + per - 1) / per;
}

size_t router_front_partial_bytes(int T, int H, int E) {
  int s, per;
  if (T < 1) return 0;
  router_front_plan(T, H, E, &s, &per);
  return (size_t)s * T * E * 4;
}

// x [T, H] bf16, wr [E, H] bf16 -> partial [n_slices][T][E] fp32.  The caller has checked pointers and alignment.
// zero / n_zero: integers the launch clears on the way (may be null / 0).
int router_front_launch(hipStream_t st, const void *x, int T, int H, const void *wr, int E, float *partial, int *n_slices_out,
                        int32_t *zero, int n_zero) {
  if (T < 1 || E < 1 || E > MOE_MAX_EXPERTS || H % kBlock) return MOE_E_SHAPE;
  // per-lane source offsets are 32-bit
  if ((double)T * H * 2 >= 2147483648.0 || (double)E * H * 2 >= 2147483648.0) return MOE_E_SHAPE;
  int s, per;
  router_front_plan(T, H, E, &s, &per);
  const int n_eblocks = (E + 255) / 256;
  const long blocks = (long)((T + kRfTokens - 1) / kRfTokens) * n_eblocks * s;
  if (blocks > 0x7fffffffl) return MOE_E_SHAPE;
#define MOE_ROUTER_PRODUCT(EB)                                                                                         \
  router_logits_splitk_kernel<EB><<<(unsigned)blocks, kRfThreads, 0, st>>>((const uint8_t *)x, (const uint8_t *)wr, T, H, E, \
                                                                           s, per, n_eblocks, partial, zero, n_zero)
  if (E <= 64) MOE_ROUTER_PRODUCT(64);
  else if (E <= 128) MOE_ROUTER_PRODUCT(128);
  else MOE_ROUTER_PRODUCT(256);
#undef MOE_ROUTER_PRODUCT
  *n_slices_out = s;
  return (int)hipGetLastError();
}

}  // namespace moe
