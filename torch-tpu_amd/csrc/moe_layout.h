// Host-side layout of the caller-provided workspaces (shared by the launchers).
#pragma once
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
  const double mean = (double)T * K / E;
  if (mean <= 40.0) return 64;
  return mean > 104.0 ? 192 : 128;
}

struct PermuteWs {
  int32_t *chunk_counts;   // [n_chunks, E]
  int32_t *tile_prefix;    // [E + 1] first tile of each expert; [E] = number of tiles
  int32_t *tile_expert;    // [max_tiles]
  int32_t *tile_desc;      // [max_tiles][8]: expert, its first tile, its tiles, its first row, its rows, 0, 0, 0
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
  size_t ints = n_chunks * (size_t)E + (size_t)(E + 1) + 9 * (size_t)permute_max_tiles(T, K, E) + 8;
  return align_up(ints * 4, 256);
}

static inline PermuteWs permute_ws_layout(void *ws, int T, int K, int E) {
  PermuteWs p;
  long tk = (long)T * K;
  p.n_chunks = (int)((tk + kChunk - 1) / kChunk);
  if (p.n_chunks == 0) p.n_chunks = 1;
  p.max_tiles = permute_max_tiles(T, K, E);
  p.chunk_counts = (int32_t *)ws;
  p.tile_prefix = p.chunk_counts + (size_t)p.n_chunks * E;
  p.tile_expert = p.tile_prefix + (E + 1);
  // 32-byte aligned: one descriptor is fetched with a single scalar load
  p.tile_desc = (int32_t *)(((uintptr_t)(p.tile_expert + p.max_tiles) + 31) & ~(uintptr_t)31);
  return p;
}

}  // namespace moe
