// Host-side layout of the caller-provided workspaces (shared by the launchers).
#pragma once
#include <cmath>
#include <stddef.h>
#include <stdint.h>

namespace moe {

constexpr int kChunk = 256;   // slots ranked by one wavefront in the permutation kernels

// What the grouped GEMMs multiply: FP8 activations x FP8 weights with scales (the path proper), bf16 x bf16
// (un-quantised experts), or bf16 activations x FP8 weights de-quantised to bf16 in registers (the reference's arithmetic)
enum { kNumericsFp8 = 0, kNumericsBf16 = 1, kNumericsW8A16 = 2 };

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Rows of an activation-scale tensor are padded to whole 64-byte pieces: the grouped GEMMs fetch
// the scales of 16 reduction steps of a row with one aligned 64-byte read.
static inline int scale_pitch(int n_groups) { return (n_groups + 15) & ~15; }

// Rows of one expert that a grouped-GEMM workgroup owns.  A pure function of the problem
// shape so that the permutation (which builds the tile list) and the GEMM launchers agree
// without passing it around.  A token's K experts are distinct, so no expert ever holds
// more than T rows: small T gets small tiles.
static inline int choose_tile_m(int T, int K, int E) {
  if (T <= 16) return 16;
  if (T <= 32) return 32;
  if (T <= 64) return 64;
  // Balanced routing puts T*K/E rows on an expert, give or take a few standard deviations.  A
  // second, nearly empty tile costs as much weight traffic as a full one, so prefer the tile
  // that holds a typical expert whole.
  // Measured (step in ms with 64 / 128 / 192 rows forced; the 64-row kernel streams its weights into LDS with the
  // non-temporal hint when an expert's rows fit one tile, which the large tiles' register loads do not profit from):
  // DeepSeek-V3 shape, T=512 (16 rows per expert on average) 1.827 / 1.999 / -, T=768 1.877 / 2.033, T=1024 1.925 / 2.062,
  // T=1280 (40 rows) 2.000 / 2.114, T=1536 (48 rows) 2.120 / 2.149, T=2048 (64 rows) 2.412 / 2.227 / 2.252,
  // T=3072 2.993 / 2.404 / 2.410, T=4096 (128 rows) 3.627 / 2.924 / 2.651; Mixtral shape, T=96 (24 rows) 0.252 / 0.290 / 0.298,
  // T=192 (48 rows) 0.297 / 0.312 / 0.319, T=256 (64 rows) 0.338 / 0.319 / 0.325; Qwen3 shape under a skewed load, T=512
  // (32 rows) 0.130 / 0.140, T=768 (48 rows) 0.148 / 0.144, T=1024 0.172 / 0.156.
  // The rule those crossovers follow: under balanced routing an expert's row count is binomial (T*K draws, 1/E each);
  // take the smallest tile that holds mean + 2.4 standard deviations - an expert's rows with about 99 % probability.
  // That puts the 64 | 128 boundary at 47 rows per expert on average and the 128 | 192 boundary at 103.
  const double mean = (double)T * K / E;
  const double reach = mean + 2.4 * std::sqrt(mean * (1.0 - 1.0 / E));
  if (reach <= 64.0) return 64;
  return reach <= 128.0 ? 128 : 192;
}

// Row tile of the dense layers (one "expert" owns every row; M > 128 rows, `items_per_row_tile` strips of the output,
// `steps` 128-steps of the reduction).  Nothing is read from HBM more than once here and the matrix fits the caches,
// so what counts is how the work items fill the 256 compute units and what one item costs: a model instead of a
// table - rounds of work items x (steps x (cost of a step, which grows with the tile's m-tiles) + the item's fixed
// start and end).  Shader cycles measured with the operands coming from L2: a step costs about 300 + 150 per m-tile,
// start and end of an item about 20 000; the 96-row kernel runs two workgroups per unit (512 items per round), one
// hiding the other's start and end, which pays while the reduction is short (kHalfTileMaxSteps).
// Example: 4096 x 7168 -> 1536 (6 strips of 256 columns): 192 rows = 132 items, half the units idle, 56 steps x 2100
// cycles; 128 rows = 192 items x 56 x 1500, a third less.
constexpr int kHalfTileMaxSteps = 20;
static inline int choose_dense_tile_m(long rows, int items_per_row_tile, int steps) {
  int best = 192;
  double best_cost = 0.0;
  const int tiles[4] = {192, 128, 96, 64};
  for (int i = 0; i < 4; i++) {
    const int tm = tiles[i];
    if (tm == 96 && steps > kHalfTileMaxSteps) continue;
    const long items = (rows + tm - 1) / tm * (long)items_per_row_tile;
    const long per_round = tm == 96 ? 512 : 256;
    const long rounds = (items + per_round - 1) / per_round;
    const double item = (double)steps * (300.0 + 150.0 * (tm / 16)) + (tm == 96 ? 10000.0 : 20000.0);
    const double cost = (double)rounds * item * (tm == 96 ? 2.0 : 1.0);      // two resident workgroups share a unit
    if (i == 0 || cost < best_cost * 0.97) { best = tm; best_cost = cost; }     // near-ties go to the taller tile
  }
  return best;
}

struct PermuteWs {
  int32_t *chunk_counts;   // [n_chunks, E]
  int32_t *tile_prefix;    // [E + 1] first tile of each expert; [E] = number of tiles
  int32_t *tile_expert;    // [max_tiles]
  int32_t *tile_desc;      // [max_tiles][8]: expert, its first tile, its tiles, its first row, its rows, 0, 0, 0
  int32_t *expert_count;   // [E] slots per expert (between the two halves of the scan kernel)
  int32_t *arrivals;       // [1] workgroups of the scan kernel that have finished their first half
  int n_chunks;
  int max_tiles;
};

static inline int permute_max_tiles(int T, int K, int E) {
  const int tm = choose_tile_m(T, K, E);
  long tk = (long)T * K;
  long a = tk / tm + E;           // sum_e ceil(n_e / tm) <= TK/tm + (#non-empty experts)
  long b = tk;                    // and never more than one tile per row
  long m = a < b ? a : b;
  return (int)(m < 1 ? 1 : m);
}

static inline size_t permute_ws_bytes(int T, int K, int E) {
  long tk = (long)T * K;
  size_t n_chunks = (size_t)((tk + kChunk - 1) / kChunk);
  if (n_chunks == 0) n_chunks = 1;
  size_t ints = n_chunks * (size_t)E + 2 * (size_t)(E + 1) + 9 * (size_t)permute_max_tiles(T, K, E) + 8;
  return align_up(ints * 4, 256);
}

static inline PermuteWs permute_ws_layout(void *ws, int T, int K, int E) {
  PermuteWs p;
  long tk = (long)T * K;
  p.n_chunks = (int)((tk + kChunk - 1) / kChunk);
  if (p.n_chunks == 0) p.n_chunks = 1;
  p.max_tiles = permute_max_tiles(T, K, E);
  p.chunk_counts = (int32_t *)ws;
  p.expert_count = p.chunk_counts + (size_t)p.n_chunks * E;
  p.arrivals = p.expert_count + E;
  p.tile_prefix = p.arrivals + 1;
  p.tile_expert = p.tile_prefix + (E + 1);
  // 32-byte aligned: one descriptor is fetched with a single scalar load
  p.tile_desc = (int32_t *)(((uintptr_t)(p.tile_expert + p.max_tiles) + 31) & ~(uintptr_t)31);
  return p;
}

}  // namespace moe
