// Host-side arithmetic of the library (workspace layout, tile heights, bounds on the tile list) exercised on its own,
// so that it can be built with -fsanitize=address,undefined and run on a machine without a GPU
// (tests/test_capi_cpu.py builds and runs it).  Exits 0 when every check holds.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../torch-tpu_amd/csrc/moe_layout.h"

using namespace moe;

static int failures = 0;
#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      failures++;                                                          \
    }                                                                      \
  } while (0)

int main() {
  const int Ts[] = {0, 1, 2, 7, 16, 17, 32, 33, 64, 65, 100, 512, 1280, 1281, 4096, 16384, 100000};
  const int Ks[] = {1, 2, 6, 8, 32};
  const int Es[] = {1, 2, 8, 37, 128, 256, 1000, 1024};
  for (int T : Ts)
    for (int K : Ks)
      for (int E : Es) {
        if (K > E) continue;
        const int tm = choose_tile_m(T, K, E);
        CHECK(tm == 16 || tm == 32 || tm == 64 || tm == 128 || tm == 192);
        const long tk = (long)T * K;
        const int mt = permute_max_tiles(T, K, E);
        CHECK(mt >= 1);
        // the bound holds for the two extreme loads: everything on as few experts as the distinctness of a token's
        // experts allows (K experts with T rows each), and one row on as many experts as there are slots
        long worst_packed = (long)K * ((T + tm - 1) / tm);
        long worst_spread = tk < E ? tk : (long)E + (tk - E + tm - 1) / tm;
        CHECK(worst_packed <= mt || T == 0);
        CHECK(worst_spread <= mt + (long)E || T == 0);
        // the workspace: pieces in order, inside the size that is announced, the descriptor table 32-byte aligned
        const size_t bytes = permute_ws_bytes(T, K, E);
        std::vector<unsigned char> buf(bytes + 64);
        unsigned char *base = buf.data() + (32 - (uintptr_t)buf.data() % 32) % 32;
        PermuteWs p = permute_ws_layout(base, T, K, E);
        CHECK((unsigned char *)p.chunk_counts == base);
        // the table, the per-expert totals and the arrival counter are one run of integers (cleared in one go)
        CHECK(p.expert_count == p.chunk_counts + (size_t)p.n_chunks * E);
        CHECK(p.arrivals == p.expert_count + E);
        CHECK(p.tile_prefix == p.arrivals + 1);
        CHECK(p.tile_expert == p.tile_prefix + E + 1);
        CHECK((uintptr_t)p.tile_desc % 32 == 0 && p.tile_desc >= p.tile_expert + p.max_tiles);
        CHECK((unsigned char *)(p.tile_desc + (size_t)8 * p.max_tiles) <= base + bytes);
        CHECK(p.max_tiles == mt);
        // touch every byte the layout hands out (the sanitizer watches the vector's bounds)
        for (int i = 0; i < p.n_chunks * E; i++) p.chunk_counts[i] = i;
        for (int i = 0; i < E; i++) p.expert_count[i] = i;
        *p.arrivals = 0;
        for (int i = 0; i <= E; i++) p.tile_prefix[i] = i;
        for (int i = 0; i < p.max_tiles; i++) p.tile_expert[i] = i;
        for (long i = 0; i < 8l * p.max_tiles; i++) p.tile_desc[i] = (int)i;
      }
  for (int g = 0; g <= 300; g++) {
    const int pitch = scale_pitch(g);
    CHECK(pitch >= g && pitch % 16 == 0 && pitch < g + 16);
  }
  // the dense layers' tile model: a legal height, monotone in nothing, but never a half tile for a long reduction
  for (long rows : {129l, 192l, 1000l, 4096l, 1l << 20})
    for (int strips : {1, 6, 28, 144, 4096})
      for (int steps : {1, 6, 16, 20, 21, 56, 256}) {
        const int tm = choose_dense_tile_m(rows, strips, steps);
        CHECK(tm == 64 || tm == 96 || tm == 128 || tm == 192);
        CHECK(tm != 96 || steps <= kHalfTileMaxSteps);
      }
  CHECK(choose_dense_tile_m(4096, 6, 56) == 128);       // 132 items of 192 rows leave half the units idle
  CHECK(choose_dense_tile_m(4096, 144, 56) == 192);
  CHECK(align_up(0, 256) == 0 && align_up(1, 256) == 256 && align_up(256, 256) == 256);
  if (failures) return 1;
  std::printf("host layout checks passed\n");
  return 0;
}
