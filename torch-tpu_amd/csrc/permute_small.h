// The permutation of at most kChunk slots by one workgroup, as a device function: shared by the
// stand-alone permutation kernel and by the decode-size kernel that routes and permutes in one launch.
#pragma once
#include "moe_common.h"
#include "moe_layout.h"
#include "../../include/moe_hip.h"

namespace moe {

// every row tile of expert e gets the expert's whole description: the GEMM workgroups, which only know
// "some tile of my expert", find their tile, rows and neighbours from one 32-byte record
__device__ __forceinline__ void write_tiles(int e, int count, int first_row, int first_tile, int tile_m,
                                            int32_t *tile_expert, int32_t *tile_desc, int max_tiles) {
  int nt = (count + tile_m - 1) / tile_m;
  for (int j = 0; j < nt; j++)
    if (first_tile + j < max_tiles) {
      tile_expert[first_tile + j] = e;
      v4i *d = (v4i *)(tile_desc + (size_t)(first_tile + j) * 8);
      d[0] = (v4i){e, first_tile, nt, first_row};
      d[1] = (v4i){count, 0, 0, 0};
    }
}

struct __attribute__((aligned(16))) PermuteSmallSmem {
  int sid[kChunk];
  int hist[MOE_MAX_EXPERTS];
  int offs[MOE_MAX_EXPERTS];
  int wave_sums[2][kChunk / 64];
};

// Whole permutation of at most kChunk slots by one workgroup of kChunk threads, one slot per thread
// (`v` = the thread's expert id, anything outside [0, E) for "no slot"): the rank of a slot inside its
// expert is the number of earlier slots with the same id (every thread walks the id list in LDS in
// step, so each read is a broadcast), the expert offsets are a block scan of the histogram.
// `sm` must sit on a 16-byte boundary.
__device__ __forceinline__ void permute_small_block(PermuteSmallSmem &sm, int v, int TK, int E, int tile_m, int max_tiles,
                                                    int32_t *__restrict__ sorted_slot,
                                                    int32_t *__restrict__ expert_offsets,
                                                    int32_t *__restrict__ slot_to_row,
                                                    int32_t *__restrict__ tile_prefix,
                                                    int32_t *__restrict__ tile_expert,
                                                    int32_t *__restrict__ tile_desc) {
  const int s = threadIdx.x;
  for (int e = s; e < E; e += kChunk) sm.hist[e] = 0;
  const bool valid = s < TK && v >= 0 && v < E;
  if (!valid) v = -1;
  // (expert, slot) as one integer: the slots of expert v that precede slot s are the entries in [v * kChunk, own)
  const uint32_t own = valid ? (uint32_t)v * kChunk + s : 0x7fffffffu, lo = (uint32_t)v * kChunk;
  sm.sid[s] = (int)own;
  __syncthreads();
  if (valid) atomicAdd(&sm.hist[v], 1);
  // every thread walks the same (TK + 3) / 4 vectors, so the trip count is uniform and the reads pipeline
  int rank = 0;
  const v4i *sid4 = (const v4i *)sm.sid;
#pragma unroll 8
  for (int j4 = 0; j4 < (TK + 3) / 4; j4++) {
    const v4i q = sid4[j4];
    rank += ((uint32_t)q[0] - lo < own - lo) + ((uint32_t)q[1] - lo < own - lo) + ((uint32_t)q[2] - lo < own - lo) +
            ((uint32_t)q[3] - lo < own - lo);
  }
  __syncthreads();
  // exclusive scans of the counts and of the tile counts over the experts, kChunk experts per pass
  int carry = 0, tcarry = 0;
  for (int e0 = 0; e0 < E; e0 += kChunk) {
    const int e = e0 + s;
    const int c = e < E ? sm.hist[e] : 0;
    const int t = (c + tile_m - 1) / tile_m;
    int inc = c, tinc = t;
    const int lane = s & 63, wave = s >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int y = __shfl_up(inc, off, 64), ty = __shfl_up(tinc, off, 64);
      if (lane >= off) { inc += y; tinc += ty; }
    }
    if (lane == 63) { sm.wave_sums[0][wave] = inc; sm.wave_sums[1][wave] = tinc; }
    __syncthreads();
    int base = carry, tbase = tcarry, tot = 0, ttot = 0;
    for (int w = 0; w < kChunk / 64; w++) {
      if (w < wave) { base += sm.wave_sums[0][w]; tbase += sm.wave_sums[1][w]; }
      tot += sm.wave_sums[0][w]; ttot += sm.wave_sums[1][w];
    }
    if (e < E) {
      sm.offs[e] = base + inc - c;
      expert_offsets[e] = base + inc - c;
      tile_prefix[e] = tbase + tinc - t;
      write_tiles(e, c, base + inc - c, tbase + tinc - t, tile_m, tile_expert, tile_desc, max_tiles);
    }
    carry += tot; tcarry += ttot;
    __syncthreads();
  }
  if (s == 0) { expert_offsets[E] = carry; tile_prefix[E] = tcarry; }
  if (s < TK) {
    const int row = valid ? sm.offs[v] + rank : -1;
    if (valid && row < TK) sorted_slot[row] = s;
    slot_to_row[s] = row;
  }
}

}  // namespace moe
