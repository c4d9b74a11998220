// Token permutation: a stable counting sort of the flattened [T*K] expert ids.
//
// Three small kernels, no host round trip (the grouped GEMMs that follow read the expert
// offsets and the tile list from device memory):
//   count    one wavefront per chunk of kChunk consecutive slots: per-chunk histogram in LDS.
//   scan     one wavefront per expert: running sum over the chunks (turns the histogram into
//            the chunk's starting rank inside its expert); the workgroup that finishes last adds
//            an exclusive scan over the experts -> expert_offsets, and the list of row tiles the
//            GEMMs walk.
//   scatter  one workgroup per chunk, one wavefront per 64 slots: ranks its slots in slot order
//            with a ballot "match-any" loop, so equal experts keep their original order (stable),
//            and writes sorted_slot / slot_to_row.
// A problem of at most kChunk slots is done by one workgroup in a single launch.
#include "moe_common.h"
#include "moe_layout.h"
#include "permute_small.h"
#include "act_quant.h"
#include "../../include/moe_hip.h"

namespace moe {

// rank of each lane among the lanes holding the same expert id, in lane order; also the
// size of that set and whether the lane is the last of it.
__device__ __forceinline__ void match_rank(int v, bool valid, int lane, int &rank, int &cnt, bool &is_last) {
  uint64_t todo = __ballot(valid);
  rank = 0; cnt = 0; is_last = false;
  const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  while (todo) {
    int leader = __ffsll((unsigned long long)todo) - 1;
    int lv = __shfl(v, leader, 64);
    uint64_t m = __ballot(valid && v == lv);
    if (valid && v == lv) {
      rank = __popcll(m & lt);
      cnt = __popcll(m);
      is_last = (lane == 63 - __clzll((long long)m));
    }
    todo &= ~m;
  }
}

// The per-slot output row of a slot without an expert is zero: its one thread clears it (such slots are rare - a rank of
// an expert-parallel group sees them for the experts it does not hold).  rows null: nothing to clear.
__device__ __forceinline__ void zero_slot_row(uint16_t *__restrict__ rows, int row_len, int slot) {
  if (rows == nullptr) return;
  v4i *row = (v4i *)(rows + (size_t)slot * row_len);
  for (int i = 0; i < row_len / 8; i++) row[i] = (v4i){0, 0, 0, 0};
}

__global__ __launch_bounds__(64) void permute_count_kernel(const int32_t *__restrict__ ids, int TK, int E,
                                                           int32_t *__restrict__ chunk_counts,
                                                           int32_t *__restrict__ arrivals) {
  __shared__ int hist[MOE_MAX_EXPERTS];
  const int lane = threadIdx.x, c = blockIdx.x;
  if (c == 0 && lane == 0) *arrivals = 0;               // the scan kernel counts its workgroups here
  for (int e = lane; e < E; e += 64) hist[e] = 0;
  __syncthreads();
  const int lo = c * kChunk;
  for (int s = lo + lane; s < min(lo + kChunk, TK); s += 64) {
    int v = ids[s];
    if (v >= 0 && v < E) atomicAdd(&hist[v], 1);
  }
  __syncthreads();
  for (int e = lane; e < E; e += 64) chunk_counts[(size_t)c * E + e] = hist[e];
}

// exclusive scan of one value per thread over a 1024-thread workgroup
__device__ __forceinline__ int block_exclusive_scan(int x, int *lds_wave_sums, int &total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = x;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int y = __shfl_up(inc, off, 64);
    if (lane >= off) inc += y;
  }
  if (lane == 63) lds_wave_sums[wave] = inc;
  __syncthreads();
  int base = 0, tot = 0;
  for (int w = 0; w < (int)(blockDim.x >> 6); w++) {
    int s = lds_wave_sums[w];
    if (w < wave) base += s;
    tot += s;
  }
  __syncthreads();
  total = tot;
  return base + inc - x;
}

// Scan.  First half, one wavefront per expert: a running sum over the chunks turns each chunk's histogram entry into
// the rank of the chunk's first slot inside the expert (64 lanes x 8 chunks at a time: every load of a round is
// independent of the others), and leaves the expert's total.  Second half, by the workgroup that arrives last (a
// counter the count kernel cleared): exclusive scan over the experts -> expert_offsets, and the list of row tiles the
// GEMMs walk.  Workgroups of four wavefronts with a few registers each find room on a compute unit whatever else runs
// there.
constexpr int kScanWaves = 4;
__global__ __launch_bounds__(64 * kScanWaves) void permute_scan_kernel(int32_t *__restrict__ chunk_counts, int n_chunks,
                                                                       int E, int tile_m, int max_tiles,
                                                                       int32_t *__restrict__ expert_offsets,
                                                                       int32_t *__restrict__ tile_prefix,
                                                                       int32_t *__restrict__ tile_expert,
                                                                       int32_t *__restrict__ tile_desc,
                                                                       int32_t *__restrict__ expert_count,
                                                                       int32_t *__restrict__ arrivals, int n_scan,
                                                                       const QuantJob ride) {
  // The scan is a few dozen workgroups and a chain of latencies; workgroups past its own quantise the activations
  // (pure streaming, needed only by the GEMM after the permutation) in the shadow of it.
  if ((int)blockIdx.x >= n_scan) {
    act_quant_thread(ride.x, ride.n_groups, ride.groups_per_row, ride.pitch, ride.q, ride.s,
                     (size_t)(blockIdx.x - n_scan) * (64 * kScanWaves) + threadIdx.x);
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e_mine = blockIdx.x * kScanWaves + wave;
  if (e_mine < E) {
    constexpr int B = 8;
    int running = 0;
    for (int c0 = 0; c0 < n_chunks; c0 += 64 * B) {
      const int c = c0 + lane * B;
      int x[B];
#pragma unroll
      for (int i = 0; i < B; i++) x[i] = c + i < n_chunks ? chunk_counts[(size_t)(c + i) * E + e_mine] : 0;
      int sum = 0;
#pragma unroll
      for (int i = 0; i < B; i++) sum += x[i];
      int inc = sum;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int y = __shfl_up(inc, off, 64);
        if (lane >= off) inc += y;
      }
      int rank = running + inc - sum;
#pragma unroll
      for (int i = 0; i < B; i++) {
        if (c + i < n_chunks) chunk_counts[(size_t)(c + i) * E + e_mine] = rank;
        rank += x[i];
      }
      running += __shfl(inc, 63, 64);
    }
    if (lane == 0) expert_count[e_mine] = running;
  }
  __shared__ int is_last;
  // This workgroup's totals are visible device-wide before its arrival is counted.  One fence per workgroup, by the
  // thread that counts, after the barrier that orders the other wavefronts' stores before it: on this chip a
  // device-scope fence writes back and invalidates the whole L2 of its XCD, so they are worth counting.
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    is_last = atomicAdd(arrivals, 1) == n_scan - 1;
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();

  __shared__ int wave_sums[16];
  __shared__ int t_first[MOE_MAX_EXPERTS + 1], t_count[MOE_MAX_EXPERTS], t_off[MOE_MAX_EXPERTS];
  // thread t owns experts 4 t .. 4 t + 3 (MOE_MAX_EXPERTS = 4 x 256 threads)
  static_assert(MOE_MAX_EXPERTS <= 4 * 64 * kScanWaves, "four experts per thread");
  int count[4], tiles[4], rows_mine = 0, tiles_mine = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int e = 4 * threadIdx.x + j;
    count[j] = e < E ? __hip_atomic_load(expert_count + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
    tiles[j] = (count[j] + tile_m - 1) / tile_m;
    rows_mine += count[j];
    tiles_mine += tiles[j];
  }
  int total, total_tiles;
  int off = block_exclusive_scan(rows_mine, wave_sums, total);
  int first_tile = block_exclusive_scan(tiles_mine, wave_sums, total_tiles);
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int e = 4 * threadIdx.x + j;
    if (e < E) {
      expert_offsets[e] = off;
      tile_prefix[e] = first_tile;
    }
    if (e < MOE_MAX_EXPERTS) {
      t_first[e] = e < E ? first_tile : total_tiles;
      t_count[e] = count[j];
      t_off[e] = off;
    }
    off += count[j];
    first_tile += tiles[j];
  }
  if (threadIdx.x == 0) {
    expert_offsets[E] = total;
    tile_prefix[E] = total_tiles;
    t_first[MOE_MAX_EXPERTS] = total_tiles;
  }
  __syncthreads();
  // The tile list, one thread per tile: under a skewed load one expert holds hundreds of row tiles, and a loop over
  // them in that expert's thread would be the longest chain of the kernel.  A tile finds its expert by bisection of
  // the first-tile table (experts without a tile share their successor's entry and are never the answer).
  const int n_tiles = min(total_tiles, max_tiles);
  for (int j = threadIdx.x; j < n_tiles; j += 64 * kScanWaves) {
    int lo = 0, hi = E;                                 // t_first[lo] <= j < t_first[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (t_first[mid] <= j) lo = mid; else hi = mid;
    }
    const int c = t_count[lo];
    tile_expert[j] = lo;
    v4i *d = (v4i *)(tile_desc + (size_t)j * 8);
    d[0] = (v4i){lo, t_first[lo], (c + tile_m - 1) / tile_m, t_off[lo]};
    d[1] = (v4i){c, 0, 0, 0};
  }
}

// One workgroup per chunk, one wavefront per 64 consecutive slots of it: every wavefront ranks its
// slots among themselves, leaves its per-expert counts in LDS, and adds the counts of the
// wavefronts before it - all slots of the chunk are placed in one round.
__global__ __launch_bounds__(kChunk) void permute_scatter_kernel(const int32_t *__restrict__ ids, int TK, int E,
                                                                 const int32_t *__restrict__ chunk_counts,
                                                                 const int32_t *__restrict__ expert_offsets,
                                                                 int32_t *__restrict__ sorted_slot,
                                                                 int32_t *__restrict__ slot_to_row,
                                                                 uint16_t *__restrict__ zero_rows, int row_len) {
  constexpr int NWV = kChunk / 64;
  __shared__ int base[MOE_MAX_EXPERTS];
  __shared__ int wcount[NWV][MOE_MAX_EXPERTS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = blockIdx.x;
  for (int e = tid; e < E; e += kChunk) {
    base[e] = expert_offsets[e] + chunk_counts[(size_t)c * E + e];
#pragma unroll
    for (int w = 0; w < NWV; w++) wcount[w][e] = 0;
  }
  const int s = c * kChunk + tid;
  const int v = s < TK ? ids[s] : -1;
  const bool valid = s < TK && v >= 0 && v < E;
  int rank, cnt;
  bool is_last;
  match_rank(v, valid, lane, rank, cnt, is_last);
  __syncthreads();
  if (valid && is_last) wcount[wave][v] = cnt;
  __syncthreads();
  int row = -1;
  if (valid) {
    row = base[v] + rank;
    for (int w = 0; w < wave; w++) row += wcount[w][v];
  }
  if (valid && row < TK) sorted_slot[row] = s;
  if (s < TK) slot_to_row[s] = row;
  if (s < TK && row < 0) zero_slot_row(zero_rows, row_len, s);
}

__global__ __launch_bounds__(kChunk) void permute_small_kernel(const int32_t *__restrict__ ids, int TK, int E, int tile_m,
                                                              int max_tiles, int32_t *__restrict__ sorted_slot,
                                                              int32_t *__restrict__ expert_offsets,
                                                              int32_t *__restrict__ slot_to_row,
                                                              int32_t *__restrict__ tile_prefix,
                                                              int32_t *__restrict__ tile_expert,
                                                              int32_t *__restrict__ tile_desc,
                                                              uint16_t *__restrict__ zero_rows, int row_len) {
  __shared__ PermuteSmallSmem sm;
  const int s = threadIdx.x;
  const int v = (s < TK) ? ids[s] : -1;
  permute_small_block(sm, v, TK, E, tile_m, max_tiles, sorted_slot, expert_offsets, slot_to_row, tile_prefix, tile_expert,
                      tile_desc);
  if (s < TK && (v < 0 || v >= E)) zero_slot_row(zero_rows, row_len, s);
}

// The same with the activation quantisation in the launch: workgroup 0 permutes, the workgroups after it quantise x
// (eight lanes per 128-column group).  At this size either is one short dependent chain; side by side they cost one launch.
__global__ __launch_bounds__(kChunk) void permute_small_quant_kernel(
    const int32_t *__restrict__ ids, int TK, int E, int tile_m, int max_tiles, int32_t *__restrict__ sorted_slot,
    int32_t *__restrict__ expert_offsets, int32_t *__restrict__ slot_to_row, int32_t *__restrict__ tile_prefix,
    int32_t *__restrict__ tile_expert, int32_t *__restrict__ tile_desc, uint16_t *__restrict__ zero_rows, int row_len,
    const uint16_t *__restrict__ x, size_t n_groups, int groups_per_row, int pitch, uint8_t *__restrict__ xq,
    float *__restrict__ xs) {
  if (blockIdx.x > 0) {
    act_quant_thread(x, n_groups, groups_per_row, pitch, xq, xs, (size_t)(blockIdx.x - 1) * kChunk + threadIdx.x);
    return;
  }
  __shared__ PermuteSmallSmem sm;
  const int s = threadIdx.x;
  const int v = (s < TK) ? ids[s] : -1;
  permute_small_block(sm, v, TK, E, tile_m, max_tiles, sorted_slot, expert_offsets, slot_to_row, tile_prefix, tile_expert,
                      tile_desc);
  if (s < TK && (v < 0 || v >= E)) zero_slot_row(zero_rows, row_len, s);
}

// Permutation of at most kChunk slots and quantisation of x [T, H] bf16 -> xq e4m3fn [T, H], xs fp32 (pitch
// scale_pitch(H / 128)) in one launch.  The caller has checked T * K <= kChunk, H % 128 == 0 and the pointers.
int permute_quant_small_launch(hipStream_t st, const int32_t *ids, int T, int K, int E, int tile_m, int32_t *sorted_slot,
                               int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &ws, uint16_t *zero_rows,
                               int row_len, const uint16_t *x, int H, uint8_t *xq, float *xs) {
  const size_t groups = (size_t)T * (H / kBlock);
  const unsigned quant_blocks = (unsigned)((quant_threads(groups) + kChunk - 1) / kChunk);
  permute_small_quant_kernel<<<1 + quant_blocks, kChunk, 0, st>>>(ids, T * K, E, tile_m, ws.max_tiles, sorted_slot,
                                                                  expert_offsets, slot_to_row, ws.tile_prefix,
                                                                  ws.tile_expert, ws.tile_desc, zero_rows, row_len, x,
                                                                  groups, H / kBlock, scale_pitch(H / kBlock), xq, xs);
  return (int)hipGetLastError();
}

// zero_rows (may be null): a [T*K, row_len] bf16 tensor in slot order whose rows of slots WITHOUT an expert (id outside
// [0, E)) are cleared here - the per-slot output form: nothing else ever writes those rows
// counted: the routing launch has filled ws.chunk_counts and ws.arrivals is zero (more than kChunk slots only)
// ride (may be null; more than kChunk slots only): activations quantised by extra workgroups of the scan launch
int permute_launch(hipStream_t st, const int32_t *ids, int T, int K, int E, int tile_m, int32_t *sorted_slot,
                   int32_t *expert_offsets, int32_t *slot_to_row, const PermuteWs &ws, uint16_t *zero_rows, int row_len,
                   bool counted, const QuantJob *ride) {
  const int TK = T * K;
  if (TK <= kChunk) {
    permute_small_kernel<<<1, kChunk, 0, st>>>(ids, TK, E, tile_m, ws.max_tiles, sorted_slot, expert_offsets, slot_to_row,
                                           ws.tile_prefix, ws.tile_expert, ws.tile_desc, zero_rows, row_len);
    return (int)hipGetLastError();
  }
  if (!counted) permute_count_kernel<<<ws.n_chunks, 64, 0, st>>>(ids, TK, E, ws.chunk_counts, ws.arrivals);
  static_assert(64 * kScanWaves == 256, "a quantising workgroup has 256 threads");
  const int n_scan = (E + kScanWaves - 1) / kScanWaves;
  const QuantJob job = ride ? *ride : QuantJob{};
  permute_scan_kernel<<<n_scan + job.blocks(), 64 * kScanWaves, 0, st>>>(
      ws.chunk_counts, ws.n_chunks, E, tile_m, ws.max_tiles, expert_offsets, ws.tile_prefix, ws.tile_expert, ws.tile_desc,
      ws.expert_count, ws.arrivals, n_scan, job);
  permute_scatter_kernel<<<ws.n_chunks, kChunk, 0, st>>>(ids, TK, E, ws.chunk_counts, expert_offsets, sorted_slot,
                                                     slot_to_row, zero_rows, row_len);
  return (int)hipGetLastError();
}

}  // namespace moe

extern "C" size_t moe_permute_workspace_bytes(int T, int K, int E) {
  if (T < 0 || K < 1 || E < 1) return 0;
  return moe::permute_ws_bytes(T, K, E);
}

extern "C" int moe_tile_rows(int T, int K, int E) { return moe::choose_tile_m(T, K, E); }

extern "C" int moe_permute(void *stream, const int32_t *ids, int T, int K, int E, int32_t *sorted_slot,
                           int32_t *expert_offsets, int32_t *slot_to_row, void *workspace, size_t workspace_bytes) {
  using namespace moe;
  if (!expert_offsets || !workspace) return MOE_E_NULL;
  if (T != 0 && (!ids || !sorted_slot || !slot_to_row)) return MOE_E_NULL;   // an empty batch still gets its (all zero) offsets
  if (T < 0 || K < 1 || K > MOE_MAX_TOPK || E < 1 || E > MOE_MAX_EXPERTS) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30)) return MOE_E_SHAPE;
  if (workspace_bytes < permute_ws_bytes(T, K, E)) return MOE_E_WORKSPACE;
  if ((uintptr_t)workspace % 4) return MOE_E_ALIGN;
  PermuteWs ws = permute_ws_layout(workspace, T, K, E);
  return permute_launch((hipStream_t)stream, ids, T, K, E, choose_tile_m(T, K, E), sorted_slot, expert_offsets,
                        slot_to_row, ws, nullptr, 0, false, nullptr);
}
