// Grouped block-scaled FP8 GEMMs of the expert MLP on gfx950 matrix cores.
//
// One workgroup of NW = 8 wavefronts owns a tile of one expert: BM = 16*MT permuted rows
// (tokens) by a strip of that expert's weight rows (output columns).  The reduction runs in
// steps of 128 = one quantisation block = one v_mfma_f32_16x16x128_f8f6f4, so every matrix
// instruction yields the un-scaled partial sum of exactly one (activation group, weight block)
// pair and the two fp32 scales are applied in registers right after it:
//     acc += partial * (act_scale[row, kb] * weight_scale[n_block, kb]).
//
// Operand roles: the WEIGHT tile is the MFMA "A" operand (its 16 rows become the rows of the
// 16x16 result) and the TOKEN tile is the "B" operand (its 16 rows become the columns).  A
// lane then holds 4 consecutive output columns of ONE token, which makes the activation scale
// a single value per lane and instruction, and lets the epilogue pack 4 outputs at a time.
//   lane l of an operand: row (l % 16), reduction bytes 16g..16g+15 and 64+16g..64+16g+15 of the
//                         128-step, g = l / 16 (the instruction only needs both operands to agree;
//                         this split makes the 128-bit LDS reads of the token tile conflict-free)
//   lane l of the result: c[r] = (weight row 4*(l / 16) + r, token l % 16)
//
// Data movement per step: the token tile is shared by all wavefronts and goes L2 -> LDS with
// direct-to-LDS loads (no registers held while in flight, XOR swizzle applied on the source
// side); each wavefront's WT = 16 / NW weight tiles are used by nobody else and go HBM ->
// registers in operand layout through a two-step register ring (WREG, row tiles of 128 / 192)
// or, for small row tiles, -> LDS the same way as the tokens.  Activation scales come sixteen
// steps at a time into a double-buffered LDS table.  Requests run ahead of the matrix work and
// are waited for with hand-placed s_waitcnt; one barrier per step.  The large-tile loop is one
// software pipeline over all m-tiles of all steps (see the loop itself).
//
// BF16 = true: the same tiles and pipelines on un-quantised operands (no scales, two
// v_mfma_f32_16x16x32_bf16 per 128-byte step accumulating in place, bf16 intermediate).
// DQ = true (with BF16): bf16 activations against FP8 weights that are de-quantised on the way into the
// matrix instruction - bf16(float(code) * block scale), the arithmetic of the reference's own kernel
// (fusedMoE.pl:217-269) - at the FP8 weights' byte count.  A step is still 128 bytes of a token row = 64
// elements; its weights are one 1 KB half of a tile-blocked (16 rows x 128 codes) block: the halves of a
// block are reduction elements 0..63 and 64..127, a lane holding codes 16g..16g+15 of its row in either,
// which become its operands of the step's two matrix instructions.
//
// GATED = true  (first GEMM): the strip is 128 gate columns plus the 128 matching up columns of
//   W13; wavefront w owns gate columns 16w..16w+15 and the same up columns.  Epilogue:
//   h = silu(gate) * up, per-token amax over the strip's 128 columns (registers -> lane
//   butterflies -> LDS across the wavefronts), scale = max(amax, 1e-10) / 448, h * (1 / scale) -> e4m3fn.
// GATED = false (second GEMM): the strip is 256 output columns, wavefront w owns 32 of them (with small
//   row tiles: 64 output columns, four wavefronts with 16 each - more, smaller workgroups, same sums);
//   the bf16 result row is written at its slot (t*K + k), which undoes the permutation.
// Both epilogues lay the output tile down in LDS and store it in whole rows.
#include <cstddef>
#include <type_traits>
#include "moe_common.h"
#include "moe_layout.h"
#include "../../include/moe_hip.h"

namespace moe {

struct GemmArgs {
  const uint8_t *aq;            // activations fp8 [rows_a, Kd]
  const float *as;              // activation scales [rows_a, as_pitch] (Kd/128 used columns)
  const uint8_t *w;             // weights fp8 [E, n_rows_w, Kd]
  const float *ws;              // weight scales [E, n_rows_w/128, Kd/128]
  const int32_t *sorted_slot;   // [TK]
  const int32_t *expert_offsets;
  const int32_t *tile_prefix;
  const int32_t *tile_expert;
  const int32_t *tile_desc;     // [tiles][8], see the permutation
  uint8_t *hq;                  // GATED: [TK, N] fp8
  float *hs;                    // GATED: [TK, N/128]
  uint16_t *y;                  // !GATED: [TK, N] bf16 in slot order
  int as_pitch;                 // floats per row of as / sh_as: scale_pitch(Kd/128)
  int hs_pitch;                 // GATED: floats per row of hs / sh_hs: scale_pitch(N/128)
  int Kd;                       // reduction length (multiple of 128)
  int N;                        // GATED: I (gate columns); !GATED: H
  int n_rows_w;                 // GATED: 2*I; !GATED: H
  int rows_a;                   // T (GATED) or TK (!GATED): bound for gathered row ids
  int topk;                     // K
  int n_strips;                 // strips along N
  int total_blocks;             // launched workgroups (multiple of 8)
  int E;                        // experts (tile_prefix[E] = number of row tiles)
  int fixed_expert;             // >= 0: dense mode, every row belongs to this expert and A row p = p
  int max_mtiles;               // entries allocated in tile_expert (row tiles of the list's height)
  int split;                    // row tiles of this kernel per row tile of the list (1, or 2: half tiles)
  // optional shared expert riding in the same launch (same N / Kd as the routed experts): its
  // row tiles follow the routed ones; rows are the tokens in order
  const uint8_t *sh_aq;         // its activations ([sh_rows, Kd]; the token tensor for the first GEMM)
  const float *sh_as;
  const uint8_t *sh_w;
  const float *sh_ws;
  uint8_t *sh_hq;
  float *sh_hs;
  uint16_t *sh_y;
  int sh_rows;                  // 0 = no shared expert in this launch
};

constexpr int kMaxKB = 256;                 // reduction length limit: 256 * 128 = 32768

template <int MT, int NW, int STAGES, int WSTAGES, int WTILE = 2048, int TPS = 16>
struct GemmSmem {
  static constexpr int BM = 16 * MT;
  alignas(1024) uint8_t wt[WSTAGES][TPS * WTILE];   // weight tiles: [tile][row][swizzled 16-byte chunk], read by their owner
  alignas(1024) uint8_t tok[STAGES][BM * 128];   // token tiles, XOR-swizzled 16-byte chunks
  alignas(1024) float sac[2][MT * 256];          // activation scales, 16 steps at a time: [m-tile][4-step part][row][4]
  int arow[BM];                                  // source row in aq / as for each tile row
  int oslot[BM];                                 // second GEMM: output row of each tile row
  float amax[NW][BM];                            // GATED epilogue: per-wavefront partial amax
  float2 fsc[4][BM];                             // large tiles: scale products of four steps, one pair per tile row
  float sb[2][kMaxKB + 4];                       // weight-block scales of the strip for every 128-step, then zeros
};

typedef __attribute__((address_space(3))) uint8_t lds_byte;
// byte offset of a __shared__ object inside the workgroup's LDS allocation (what M0 wants)
__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(uintptr_t)(lds_byte *)p; }

__device__ __forceinline__ v8i load_w_frag(const uint8_t *p) {
  v4i lo = *(const v4i *)p;
  v4i hi = *(const v4i *)(p + 16);
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

__device__ __forceinline__ v8i concat8(v4i lo, v4i hi) {
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// 16 e4m3fn codes (reduction elements in byte order) -> 16 bf16 = bf16(float(code) * s), the reference's
// weight_dequant (fusedMoE.pl:11-34; python/regression/test_llm/test_moe.py:10-50), element b in half b % 2 of dword b / 2
__device__ __forceinline__ v8i dequant16(v4i raw, float s) {
  v8i r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const v2f_t a = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], false);
    const v2f_t b = __builtin_amdgcn_cvt_pk_f32_fp8(raw[i], true);
    r[2 * i] = (int)pack2_bf16(a[0] * s, a[1] * s);
    r[2 * i + 1] = (int)pack2_bf16(b[0] * s, b[1] * s);
  }
  return r;
}

// bf16 operands: the two 16-byte chunks a lane holds of a 128-byte step are the lane's share of two
// 32-element matrix instructions; all first halves are issued before the second halves so that an
// accumulator is not needed again right away
template <int WT>
__device__ __forceinline__ void mma_bf16(v4f (&acc)[WT], const v8i (&w)[WT], const v8i &x) {
  const v4i xl = {x[0], x[1], x[2], x[3]}, xh = {x[4], x[5], x[6], x[7]};
#pragma unroll
  for (int j = 0; j < WT; j++) {
    const v4i wl = {w[j][0], w[j][1], w[j][2], w[j][3]};
    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wl), __builtin_bit_cast(v8bf, xl), acc[j], 0, 0, 0);
  }
#pragma unroll
  for (int j = 0; j < WT; j++) {
    const v4i wh = {w[j][4], w[j][5], w[j][6], w[j][7]};
    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wh), __builtin_bit_cast(v8bf, xh), acc[j], 0, 0, 0);
  }
}

// MT     token m-tiles (of 16 rows) per workgroup
// NW     wavefronts per workgroup (4 or 8); each owns WT = TPS / NW of the strip's weight tiles
// TPS    weight tiles (of 16 rows) per strip: 16, or 4 for the second GEMM of a batch that would leave most
//        of the chip without a strip (narrow strips of 64 output columns; every sum keeps its order)
// DEPTH  128-steps of weights kept in flight per wavefront (register ring)
// DQ     BF16 arithmetic on FP8 weights with block scales, de-quantised in registers (a.Kd counts the token row's bytes)
// BF16   un-quantised mode: both operands are bf16 (a 128-byte step is 64 elements = two
//        v_mfma_f32_16x16x32_bf16 accumulating in place), no scales, bf16 intermediate
template <int MT, int NW, int DEPTH, bool GATED, bool WREG, bool BF16 = false, int TPS = 16, bool DQ = false>
// Four wavefronts with the weights in registers: two such workgroups share a compute unit (256 registers a lane each)
__global__ __launch_bounds__(64 * NW, (WREG && NW == 4) ? 2 : 1) void grouped_gemm_kernel(const GemmArgs a) {
  static_assert(!DQ || BF16, "de-quantised weights feed the bf16 matrix instructions");
  static_assert(TPS % NW == 0 && (TPS == 16 || (!GATED && !WREG && TPS <= 8)), "narrow strips: second GEMM, operands through LDS");
  constexpr int BM = 16 * MT;
  constexpr int NT = 64 * NW;                         // threads
  constexpr int WT = TPS / NW;                        // weight tiles per wavefront
  constexpr int STAGES = WREG ? 4 : DEPTH + 1;        // token tiles staged in LDS
  using Smem = GemmSmem<MT, NW, STAGES, WREG ? 1 : STAGES, WREG ? 64 : 2048, TPS>;
  static_assert(sizeof(Smem) <= 160 * 1024, "one workgroup's LDS");
  __shared__ Smem sm;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lg = lane >> 4;

  // ---- which tile -------------------------------------------------------------------------
  // Workgroup ids are dealt round-robin to the 8 XCDs (id % 8).  Remap so that each XCD, which
  // has its own L2, works on a contiguous range of the real tiles (their number is only known
  // on the device): neighbours in that range share the token tile and, for experts with more
  // than one row tile, the weight strip.
  // The tile list may be coarser than this kernel's row tile (a.split of its tiles per list entry, 192 = 2 x 96): an
  // entry's tiles follow one another, the ones past the expert's last row exit right away.
  const int n_routed = a.fixed_expert >= 0 ? (a.rows_a + BM - 1) / BM : min(a.tile_prefix[a.E], a.max_mtiles) * a.split;
  const int n_mtiles = n_routed + (a.sh_rows + BM - 1) / BM;
  // Each XCD takes an equal share of the shared expert's work items (full tiles: the heaviest, so
  // they go first) and then an equal, contiguous share of the routed ones.
  const int n_routed_work = n_routed * a.n_strips, n_shared_work = (n_mtiles - n_routed) * a.n_strips;
  const int per_xcd_r = (n_routed_work + 7) >> 3, per_xcd_s = (n_shared_work + 7) >> 3;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int my_shared = min(max(n_shared_work - xcd * per_xcd_s, 0), per_xcd_s);
  int logical;
  if (idx < my_shared) {
    logical = n_routed_work + xcd * per_xcd_s + idx;
  } else {
    const int j = idx - my_shared;
    if (j >= per_xcd_r) return;
    logical = xcd * per_xcd_r + j;
    if (logical >= n_routed_work) return;
  }
  // Inside one expert the (row tile, strip) pairs are walked in blocks of up to kBlockM row tiles x
  // kBlockS strips, so that the ~32 workgroups an XCD runs at a time share a few token tiles and a few
  // weight strips through its L2 instead of streaming 32 different strips.
  constexpr int kBlockM = 6, kBlockS = 5;
  const int g0 = logical / a.n_strips;                // some row tile of the expert this work item is in
  int e, first_mtile, n_mt, e_row0 = 0, e_rows = 0;   // expert, its first row tile, its row tiles, first row, rows
  const bool shared = g0 >= n_routed;                 // a tile of the shared expert
  const bool direct = shared || a.fixed_expert >= 0;  // rows are taken in order, no permutation
  if (shared) {
    e = 0; first_mtile = n_routed; n_mt = n_mtiles - n_routed;
  } else if (a.fixed_expert >= 0) {
    e = a.fixed_expert; first_mtile = 0; n_mt = n_routed;
  } else {
    // one 32-byte record holds everything about the expert this tile belongs to
    const v4i d0 = *(const v4i *)(a.tile_desc + (size_t)(g0 / a.split) * 8);
    const v4i d1 = *(const v4i *)(a.tile_desc + (size_t)(g0 / a.split) * 8 + 4);
    e = d0[0];
    if (e < 0 || e >= a.E) return;
    first_mtile = d0[1] * a.split;
    n_mt = (min(d0[1] + d0[2], a.max_mtiles) - d0[1]) * a.split;
    e_row0 = d0[3];
    e_rows = d1[0];
  }
  int mtile, strip;
  {
    const int local = logical - first_mtile * a.n_strips;
    const int mb = local / (kBlockM * a.n_strips);
    const int r1 = local - mb * kBlockM * a.n_strips;
    const int hm = min(kBlockM, n_mt - kBlockM * mb);
    if (hm <= 0) return;
    const int sb = r1 / (hm * kBlockS);
    const int r2 = r1 - sb * hm * kBlockS;
    const int w = min(kBlockS, a.n_strips - kBlockS * sb);
    mtile = first_mtile + kBlockM * mb + r2 / w;
    strip = kBlockS * sb + r2 % w;
  }
  int row0, rows;                                     // first permuted row, rows in tile
  if (shared) {
    row0 = (mtile - n_routed) * BM;
    rows = min(BM, a.sh_rows - row0);
  } else if (a.fixed_expert >= 0) {
    row0 = mtile * BM;
    rows = min(BM, a.rows_a - row0);
  } else {
    row0 = e_row0 + (mtile - first_mtile) * BM;
    rows = min(BM, e_row0 + e_rows - row0);
  }
  const uint8_t *const aq = shared ? a.sh_aq : a.aq;
  const float *const as = shared ? a.sh_as : a.as;
  const uint8_t *const wq = shared ? a.sh_w : a.w;
  const float *const ws = shared ? a.sh_ws : a.ws;
  const int rows_a = shared ? a.sh_rows : a.rows_a;
  if (rows <= 0) return;
  const int mt_live = (rows + 15) >> 4;               // m-tiles that hold at least one row
  const bool stream_weights = n_mt == 1;              // the expert's rows fit this one row tile

  const int NKB = a.Kd >> 7;
  const int n_wblk = (a.n_rows_w + 127) >> 7;         // weight-scale rows per expert

  // ---- per-lane source addresses ------------------------------------------------------------
  // GATED: tiles 0..WT/2-1 are gate columns, WT/2..WT-1 the matching up columns.
  // Every global address of the loop is "uniform 64-bit base in SGPRs + 32-bit per-lane offset":
  // one VGPR per address instead of two and no vector address arithmetic per step.
  const uint8_t *wtile[WT];                            // uniform: first row of the wavefront's tile j
#pragma unroll
  for (int j = 0; j < WT; j++) {
    int wrow;
    if (GATED) wrow = (j < WT / 2 ? 0 : a.N) + strip * 128 + wave * (8 * WT) + (j % (WT / 2)) * 16;
    else wrow = strip * (16 * TPS) + wave * (16 * WT) + j * 16;
    wrow = min(wrow, a.n_rows_w - 16);                 // tiles past the matrix re-read its last rows
    wtile[j] = wq + ((size_t)e * a.n_rows_w + wrow) * (DQ ? a.Kd >> 1 : a.Kd);
  }
  // Weights are stored tile-blocked: the 2 KB a (16-row tile, 128-byte step) pair needs are contiguous and already
  // in operand order - two 1 KB halves of [lane][16 bytes] - so every load instruction of a wavefront reads 1 KB of
  // consecutive memory (whole cache lines, nothing to shuffle), and a tile's steps follow one another in memory.
  const uint32_t woff = (uint32_t)lane * 16u;
  // The strip's weight-block scales for all steps go to LDS once (two rows: gate/up blocks for
  // the gated GEMM, the strip's two 128-column blocks otherwise): uniform values re-read per
  // step from LDS instead of through the vector-memory queue.  They are asked for together with
  // the rows' sources, before either is waited for.
  constexpr int NSB = (2 * kMaxKB + NT - 1) / NT;
  float sbv[NSB];
  // DQ: a step is half a 128-block of the reduction (64 elements), two steps share a block scale
  const int NKBW = DQ ? NKB >> 1 : NKB;
  if constexpr (!BF16 || DQ) {
    // second GEMM: the 128-row blocks the strip's first and ninth tile lie in (a narrow strip lies in one)
    const int blk0 = GATED ? strip : min(strip * TPS / 8, n_wblk - 1);
    const int blk1 = GATED ? (a.N >> 7) + strip : min(strip * TPS / 8 + 1, n_wblk - 1);
#pragma unroll
    for (int u = 0; u < NSB; u++) {
      const int i = tid + u * NT, r = i >= NKB, kb = i - r * NKB;
      sbv[u] = i < 2 * NKB ? ws[((size_t)e * n_wblk + (r ? blk1 : blk0)) * NKBW + (DQ ? kb >> 1 : kb)] : 0.f;
    }
  }
  for (int i = tid; i < BM; i += NT) {
    const int p = row0 + min(i, rows - 1);
    int src = p;
    if (GATED && !direct) src = a.sorted_slot[p] / a.topk;
    sm.arow[i] = min(max(src, 0), rows_a - 1);
    if (!GATED) sm.oslot[i] = direct ? p : a.sorted_slot[p];      // output row (slot) of each tile row
  }
  if constexpr (!BF16 || DQ) {
#pragma unroll
    for (int u = 0; u < NSB; u++) {
      const int i = tid + u * NT, r = i >= NKB, kb = i - r * NKB;
      if (i < 2 * NKB) sm.sb[r][kb] = sbv[u];
    }
    if (tid < 8) sm.sb[tid >> 2][NKB + (tid & 3)] = 0.f;
  }
  __syncthreads();
  const int sb_row0 = GATED ? 0 : (wave * WT) / 8;      // which of the two rows this wavefront's tiles use
  const int sb_row1 = GATED ? 1 : sb_row0;
  // Token tile -> LDS by direct loads: one instruction moves 64 x 16 bytes = 8 rows x 128 bytes to
  // LDS bytes [M0 + 16*lane); the XOR swizzle is applied on the source side (lane l fetches the
  // chunk that belongs at position l).  NTOK instructions per wavefront and step; wavefronts past
  // the tile's end repeat its last eight rows (same bytes to the same place).
  constexpr int NROW8 = BM / 8;                        // 1 KB row-groups in the tile
  constexpr int NTOK = (NROW8 + NW - 1) / NW;
  uint32_t tok_src[NTOK];
  uint32_t tok_m0[NTOK];
#pragma unroll
  for (int u = 0; u < NTOK; u++) {
    const int t = min(wave * NTOK + u, NROW8 - 1);
    const int row = 8 * t + (lane >> 3);
    const int c = (lane & 7) ^ (lane >> 3);
    // row-groups past the tile's last row are never read by a matrix instruction that matters:
    // every lane fetches the same 16 bytes there, which costs one cache line instead of eight
    tok_src[u] = 8 * t < rows ? (uint32_t)sm.arow[row] * (uint32_t)a.Kd + c * 16 : (uint32_t)sm.arow[0] * (uint32_t)a.Kd;
    tok_m0[u] = t * 1024;
  }
  // Activation scales travel 16 steps (64 bytes of a row) at a time: one instruction moves the 16
  // rows of an m-tile, lane (part, row) fetching 16 bytes = 4 steps, into [part][row][4] order, which
  // the 16 lanes that later read one step of 16 rows hit in 16 different banks.  Two buffers; the
  // chunk after the current one is requested when the current one starts.
  constexpr int NSC = (MT + NW - 1) / NW;              // scale instructions per wavefront and chunk
  uint32_t sac_src[NSC];
  uint32_t sac_m0[NSC];
#pragma unroll
  for (int u = 0; u < NSC; u++) {
    const int mt = min(wave + u * NW, MT - 1);
    sac_src[u] = (uint32_t)sm.arow[mt * 16 + li] * (uint32_t)a.as_pitch * 4u + lg * 16;   // bytes
    sac_m0[u] = mt * 1024;
  }
  const uint32_t wt_base = __builtin_amdgcn_readfirstlane(lds_offset(&sm.wt[0][0])) + wave * (WT * 2048);
  constexpr uint32_t kWtStage = TPS * 2048;
  const uint32_t tok_base = __builtin_amdgcn_readfirstlane(lds_offset(&sm.tok[0][0]));
  const uint32_t sac_base = __builtin_amdgcn_readfirstlane(lds_offset(&sm.sac[0][0]));
  constexpr uint32_t kTokStage = BM * 128, kSacBuf = MT * 1024;
  const int n_chunks = (NKB + 15) >> 4;

  v4f acc[MT][WT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int j = 0; j < WT; j++) acc[mt][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  // ---- operand pipelines ----------------------------------------------------------------------
  // Both operands travel HBM/L2 -> LDS by direct loads (no registers held while in flight), DEPTH
  // steps ahead, through STAGES = DEPTH + 1 LDS stages.  The loads are inline assembly waited for
  // by hand: the memory counter retires loads in issue order and every wavefront issues the same
  // sequence each step (token tile pieces, token scales, its own weight fragments), so "how many
  // younger loads may still be in flight" is a compile-time constant.
  //   weights: the wavefront's WT tiles, each as two 1 KB halves laid out [lane][16 bytes] - the
  //            owner reads them back with two linear 128-bit LDS reads per tile;
  //   tokens:  1 KB pieces = 8 rows x 128 bytes, swizzled on the source side.
  constexpr int LPT = DQ ? 1 : 2;                      // load instructions per weight tile and step (1 KB each)
  constexpr int WSTEP = 1024 * LPT;                    // bytes of a tile's step in memory
  constexpr int L_STEP = NTOK + LPT * WT;              // loads per wavefront and step (scale chunks come on top)
  v4i wlo[WREG ? DEPTH : 1][WT], whi[WREG ? DEPTH : 1][WT];   // WREG: weight fragments ride in a register ring
  auto request_weights_reg = [&](int kb, v4i(&lo)[WT], v4i(&hi)[WT]) {
#pragma unroll
    for (int j = 0; j < WT; j++) {
      const uint8_t *base = wtile[j] + (size_t)kb * WSTEP;
      if constexpr (DQ)
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(lo[j]) : "v"(woff), "s"(base) : "memory");
      else
        asm volatile("global_load_dwordx4 %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:1024"
                     : "=&v"(lo[j]), "=&v"(hi[j]) : "v"(woff), "s"(base) : "memory");
    }
  };
  auto arrived_weights = [&](v4i(&lo)[WT], v4i(&hi)[WT]) {
#pragma unroll
    for (int j = 0; j < WT; j++) {
      if constexpr (DQ) asm volatile("" : "+v"(lo[j]));
      else asm volatile("" : "+v"(lo[j]), "+v"(hi[j]));
    }
  };
  auto request_scales = [&](int chunk) {
    if constexpr (BF16) return;
#pragma unroll
    for (int u = 0; u < NSC; u++) {
      const float *base = as + chunk * 16;
      const uint32_t m0 = sac_base + (chunk & 1) * kSacBuf + sac_m0[u];
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0), "v"(sac_src[u]), "s"(base) : "memory", "m0");
    }
  };
  auto request_tok = [&](int kb, int stage, int u) {
    const uint8_t *base = aq + (size_t)kb * 128;
    const uint32_t m0 = tok_base + stage * kTokStage + tok_m0[u];
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0), "v"(tok_src[u]), "s"(base) : "memory", "m0");
  };
  auto request = [&](int kb, int stage) {
#pragma unroll
    for (int u = 0; u < NTOK; u++) request_tok(kb, stage, u);
    // weight tiles through LDS: an instruction copies one 1 KB half of a tile's step as it lies in memory (the
    // instruction offset advances the memory address and the LDS address alike).  With the non-temporal hint when the
    // expert's rows fit this one row tile - every weight byte is then read exactly once, and hinted loads stream 6-9 %
    // faster; an expert with several row tiles keeps plain loads, its later tiles find the strip in L2.
    if (!WREG) {
      if (stream_weights) {
#pragma unroll
        for (int j = 0; j < WT; j++) {
          const uint8_t *base = wtile[j] + (size_t)kb * WSTEP;
          const uint32_t m0 = wt_base + stage * kWtStage + j * 2048;
          if constexpr (DQ)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0), "v"(woff), "s"(base) : "memory", "m0");
          else
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\t"
                         "global_load_lds_dwordx4 %1, %2 offset:1024 nt"
                         ::"s"(m0), "v"(woff), "s"(base) : "memory", "m0");
        }
      } else {
#pragma unroll
        for (int j = 0; j < WT; j++) {
          const uint8_t *base = wtile[j] + (size_t)kb * WSTEP;
          const uint32_t m0 = wt_base + stage * kWtStage + j * 2048;
          if constexpr (DQ)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0), "v"(woff), "s"(base) : "memory", "m0");
          else
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                         "global_load_lds_dwordx4 %1, %2 offset:1024"
                         ::"s"(m0), "v"(woff), "s"(base) : "memory", "m0");
        }
      }
    }
  };

  // Which two 16-byte chunks of a token row's 128-byte step a lane reads (positions XOR-swizzled by the row).  FP8 and
  // bf16 operands: chunks g and g + 4, conflict-free for 128-bit LDS reads, and the weights are stored to match.  DQ:
  // the lane's 16 weight codes are reduction elements 16g..16g+15 of the step, bytes 32g..32g+31 of the token row.
  auto tok_chunk0 = [](int g, int i) { return ((DQ ? 2 * g : g) ^ (i & 7)) << 4; };
  auto tok_chunk1 = [](int g, int i) { return ((DQ ? 2 * g + 1 : g + 4) ^ (i & 7)) << 4; };
  // m-tiles are processed in groups of up to four; a group is skipped when it holds no row.  A
  // group first issues all of its LDS reads (one exposed LDS latency per group, not per tile),
  // then its matrix instructions back to back, each tile's scale multiply-adds trailing the
  // matrix instruction that feeds them.
  constexpr int MG = MT < 4 ? MT : (MT % 4 == 0 && MT <= 8 ? 4 : (DEPTH >= 3 ? 2 : 3));
  auto compute = [&](int stage, int kb, const v4i(&lo)[WT], const v4i(&hi)[WT]) {
    v8i wc[WT];
    const uint8_t *wbase = sm.wt[WREG ? 0 : stage] + wave * (WT * 2048) + lane * 16;
    const float s0 = BF16 && !DQ ? 0.f : sm.sb[sb_row0][kb], s1 = BF16 && !DQ ? 0.f : sm.sb[sb_row1][kb];
#pragma unroll
    for (int j = 0; j < WT; j++) {
      if constexpr (DQ) wc[j] = dequant16(WREG ? lo[j] : *(const v4i *)(wbase + j * 2048), (GATED && j >= WT / 2) ? s1 : s0);
      else if (WREG) wc[j] = concat8(lo[j], hi[j]);
      else wc[j] = concat8(*(const v4i *)(wbase + j * 2048), *(const v4i *)(wbase + j * 2048 + 1024));
    }
    const uint8_t *tbase = sm.tok[stage] + li * 128;
    const int o0 = tok_chunk0(lg, li), o1 = tok_chunk1(lg, li);
    const float *sap = sm.sac[(kb >> 4) & 1] + ((kb & 12) << 4) + li * 4 + (kb & 3);
#pragma unroll
    for (int mg = 0; mg < MT / MG; mg++) {
      if (mg == 0 || mg * MG < mt_live) {
        v8i x[MG];
        float sa_[MG];
        // m-tiles of the group that hold no row (the first of a group always does) are left out one by one
#pragma unroll
        for (int mi = 0; mi < MG; mi++) {
          const int mt = mg * MG + mi;
          if (mi == 0 || mt < mt_live) {
            x[mi] = concat8(*(const v4i *)(tbase + mt * 2048 + o0), *(const v4i *)(tbase + mt * 2048 + o1));
            sa_[mi] = BF16 ? 0.f : sap[mt * 256];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (BF16) {
#pragma unroll
          for (int mi = 0; mi < MG; mi++)
            if (mi == 0 || mg * MG + mi < mt_live) mma_bf16<WT>(acc[mg * MG + mi], wc, x[mi]);
          __builtin_amdgcn_sched_barrier(0);
          continue;
        }
        v4f p[MG][WT];
#pragma unroll
        for (int mi = 0; mi < MG; mi++) {
          if (mi == 0 || mg * MG + mi < mt_live) {
#pragma unroll
            for (int j = 0; j < WT; j++) {
              const v4f zero = {0.f, 0.f, 0.f, 0.f};
              p[mi][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wc[j], x[mi], zero, 0, 0, 0, 0, 0, 0);
            }
          }
        }
#pragma unroll
        for (int mi = 0; mi < MG; mi++) {
          const int mt = mg * MG + mi;
          if (mi == 0 || mt < mt_live) {
            const float f0 = sa_[mi] * s0, f1 = sa_[mi] * s1;
#pragma unroll
            for (int j = 0; j < WT; j++) {
              const float f = (GATED && j >= WT / 2) ? f1 : f0;
#pragma unroll
              for (int r = 0; r < 4; r++) acc[mt][j][r] = fmaf(p[mi][j][r], f, acc[mt][j][r]);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // ---- main loop -----------------------------------------------------------------------------
  // Step kb: wait until this wavefront's requests for step kb have landed | barrier: everybody's
  // share of the token tile is there and everybody is done reading the stage that is reused next |
  // request step kb+DEPTH into that stage | matrix work on stage kb % STAGES.
  // DEPTH-1 whole steps stay in flight across the wait, DEPTH during the matrix work.
  // Scale chunk c+1 is requested right after the barrier of step 16c: every wavefront has then left
  // step 16c-1, the last reader of the buffer it goes to, and any later step's wait covers it (a wait
  // leaves only the (DEPTH-1) youngest steps' loads outstanding, so extra loads make it stricter).
  request_scales(0);
  if constexpr (!WREG) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) request(min(d, NKB - 1), d);
    int kb = 0, stage = 0, stage_req = DEPTH;
    for (; kb + DEPTH < NKB; kb++) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * L_STEP) : "memory");
      __syncthreads();
      if ((kb & 15) == 0 && (kb >> 4) + 1 < n_chunks) request_scales((kb >> 4) + 1);
      request(kb + DEPTH, stage_req);
      compute(stage, kb, wlo[0], whi[0]);
      stage = stage + 1 == STAGES ? 0 : stage + 1;
      stage_req = stage_req + 1 == STAGES ? 0 : stage_req + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (; kb < NKB; kb++) {
      __syncthreads();
      compute(stage, kb, wlo[0], whi[0]);
      stage = stage + 1 == STAGES ? 0 : stage + 1;
    }
  } else {
    // Large tiles: weights in a register ring of two steps, token tiles three steps ahead through
    // four LDS stages, and ONE software pipeline over all m-tiles of all steps: the LDS reads of
    // m-tile g+2 and the scale multiply-adds of m-tile g-1 are issued around the matrix
    // instructions of m-tile g, across step boundaries.  For that the token tile of step s+1 is
    // made visible (wait + barrier) one step early, at the top of step s.  Per step and wavefront
    // the loads go out in a fixed order - token tile of step s+3 at the top, weights of step s+2
    // at the end - so the wait at the top of step s+1 leaves exactly those two requests in flight.
    // Requests past the last step re-read it (cheap cache hits) instead of branching; a step past
    // an odd count multiplies by the zero weight scale stored behind the table.  The loop body is
    // instantiated per number of live m-tiles, so there is no branch between matrix instructions.
    static_assert(DEPTH == 2, "the register ring holds two steps");
    constexpr int R = DEPTH;                             // ring slots = steps per pass of the unrolled loop
    constexpr int XB = 4;                                // token operand buffers; R * LIVE is a multiple of it
    constexpr int L_WAIT = NTOK + LPT * WT * (R - 1);    // loads younger than the ones a step boundary needs
    const int last = NKB - 1;
    const int o0 = tok_chunk0(lg, li), o1 = tok_chunk1(lg, li);
    auto run = [&](auto live_c) {
      constexpr int LIVE = decltype(live_c)::value;
      static_assert(LIVE % 2 == 0 && LIVE >= 2 && LIVE <= MT, "live m-tiles come in pairs");
      constexpr int PD = 2;                              // m-tiles between an LDS read and its use
      const bool top_empty = mt_live < LIVE;             // uniform: the top m-tile of the top pair holds no row
      // the first requests go out inside the instantiation: no branch may sit between a register
      // load's request and its wait (the compiler would copy the registers while the load is in flight)
      request(0, 0);
      request(min(1, last), 1);
      request_weights_reg(0, wlo[0], whi[0]);
      request(min(2, last), 2);
#pragma unroll
      for (int d = 1; d < R; d++) request_weights_reg(min(d, last), wlo[d], whi[d]);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(L_WAIT) : "memory");
      arrived_weights(wlo[0], whi[0]);
      __syncthreads();
      if (n_chunks > 1) request_scales(1);
      // Scale products: what a lane multiplies a matrix-instruction result with is (activation scale
      // of its token and step) x (weight-block scale of its tile and step).  One thread per tile row
      // forms both products of a step once, two steps ahead, instead of every wavefront forming them
      // for every m-tile (one multiply less per matrix instruction on the shared issue port).
      auto produce_f = [&](int k) {
        if constexpr (BF16) return;
        if (tid < BM) {
          const int kc = min(k, last);                   // past the end: a finite scale times the zero behind the table
          const float sa = sm.sac[(kc >> 4) & 1][(tid >> 4) * 256 + ((kc & 12) << 4) + (tid & 15) * 4 + (kc & 3)];
          sm.fsc[k & 3][tid] = make_float2(sa * sm.sb[0][k], sa * sm.sb[1][k]);
        }
      };
      produce_f(0);
      produce_f(1);
      produce_f(2);
      __syncthreads();
      auto read_x = [&](int kb, int mt) {
        const uint8_t *t = sm.tok[kb & 3] + li * 128 + mt * 2048;
        return concat8(*(const v4i *)(t + o0), *(const v4i *)(t + o1));
      };
      // GATED: both products (gate tiles use .x, up tiles .y); second GEMM: the one of this wavefront's column block
      auto read_f = [&](int kb, int mt) {
        if (BF16) return make_float2(0.f, 0.f);
        if (GATED) return sm.fsc[kb & 3][mt * 16 + li];
        const float f = ((const float *)&sm.fsc[kb & 3][mt * 16 + li])[sb_row0];
        return make_float2(f, f);
      };
      v8i x[XB];
      float2 fb[XB];
      v4f p[2][WT];
#pragma unroll
      for (int q = 0; q < PD; q++) {
        const int qq = q < LIVE ? q : q - LIVE, kk = q < LIVE ? 0 : 1;
        x[q] = read_x(kk, LIVE - 1 - qq); fb[q] = read_f(kk, LIVE - 1 - qq);
      }
      // the multiply-add slot of the very first m-tile adds zero
#pragma unroll
      for (int j = 0; j < WT; j++) p[1][j] = (v4f){0.f, 0.f, 0.f, 0.f};
      fb[XB - 1] = make_float2(0.f, 0.f);
      for (int s0 = 0; s0 < NKB; s0 += R) {
#pragma unroll
        for (int h = 0; h < R; h++) {
          const int kb = s0 + h;
          v8i wc[WT];
#pragma unroll
          for (int j = 0; j < WT; j++) {
            if constexpr (DQ) wc[j] = dequant16(wlo[h][j], sm.sb[(GATED && j >= WT / 2) ? sb_row1 : sb_row0][kb]);
            else wc[j] = concat8(wlo[h][j], whi[h][j]);
          }
          // one m-tile: LDS reads two m-tiles ahead, its matrix instructions, then the multiply-adds
          // of the m-tile before it (tp), whose products are complete by now
          // m-tiles are walked from the last live one down to 0 so that the m-tile whose products are
          // still pending at a step boundary is m-tile 0 whatever the number of live m-tiles
          auto tile = [&](int q, int tp) {
            const int g = h * LIVE + q;                  // position in the R-step pattern
            {
              const int qq = q + PD < LIVE ? q + PD : q + PD - LIVE;
              const int kk = q + PD < LIVE ? kb : kb + 1;
              if (qq != 0 || !top_empty) {               // nothing to read for a top m-tile without a row
                x[(g + PD) % XB] = read_x(kk, LIVE - 1 - qq);
                fb[(g + PD) % XB] = read_f(kk, LIVE - 1 - qq);
              }
            }
            // the token tile of step kb + 3 goes into the stage that step kb - 1 used, one piece with each of a few
            // m-tiles: all wavefronts asking for everything at the step boundary queued up behind one another
#pragma unroll
            for (int u = 0; u < NTOK; u++)
              if (u * LIVE / NTOK == q) request_tok(min(kb + 3, last), (kb + 3) & 3, u);
            // the scale products of step kb + 3 take the slot step kb - 1 read from: formed in the middle of a step, where
            // the matrix pipe has work, instead of at the boundary, where every wavefront stands still
            if (q == LIVE / 2) produce_f(kb + 3);
            if constexpr (BF16) {                        // accumulates in place: nothing is pending afterwards
              if (q != 0 || !top_empty) mma_bf16<WT>(acc[LIVE - 1 - q], wc, x[g % XB]);
              __builtin_amdgcn_sched_barrier(0);
              return;
            }
            // Live m-tiles come in pairs; when the rows end in the lower one of the top pair, the top m-tile (the
            // first of the walk) has no row: its matrix instructions are left out, like its operand reads and the
            // multiply-adds that would fold its products in; the epilogue never looks at its accumulator.
            if (q != 0 || !top_empty) {
#pragma unroll
              for (int j = 0; j < WT; j++) {
                const v4f zero = {0.f, 0.f, 0.f, 0.f};
                p[g & 1][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wc[j], x[g % XB], zero, 0, 0, 0, 0, 0, 0);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (q != 1 || !top_empty) {                  // the m-tile before this one was the empty top one: no products
#pragma unroll
              for (int j = 0; j < WT; j++) {
                const float f = (GATED && j >= WT / 2) ? fb[(g + XB - 1) % XB].y : fb[(g + XB - 1) % XB].x;
#pragma unroll
                for (int r = 0; r < 4; r++) acc[tp][j][r] = fmaf(p[(g + 1) & 1][j][r], f, acc[tp][j][r]);
                // pins the multiply-adds here: without it they are sunk below the whole step's matrix
                // instructions, whose results then all stay live
                asm volatile("" : "+v"(acc[tp][j]));
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          };
          tile(0, 0);
#pragma unroll
          for (int q = 1; q < LIVE; q++) tile(q, LIVE - q);
          // top of step kb + 1
          request_weights_reg(min(kb + R, last), wlo[h], whi[h]);
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(L_WAIT) : "memory");
          arrived_weights(wlo[(h + 1) % R], whi[(h + 1) % R]);
          __syncthreads();
          if (((kb + 1) & 15) == 0 && ((kb + 1) >> 4) + 1 < n_chunks) request_scales(((kb + 1) >> 4) + 1);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // the requests past the last step are still in flight: they land before anything else happens
      // (their registers and LDS stages must not be reused under them)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int d = 0; d < R; d++) arrived_weights(wlo[d], whi[d]);
      // m-tile 0 of the last step is still pending
#pragma unroll
      for (int j = 0; j < WT; j++) {
        const float f = (GATED && j >= WT / 2) ? fb[XB - 1].y : fb[XB - 1].x;
#pragma unroll
        for (int r = 0; r < 4; r++) acc[0][j][r] = fmaf(p[1][j][r], f, acc[0][j][r]);
      }
    };
    auto pick = [&](auto self, auto live_c) -> void {
      constexpr int LIVE = decltype(live_c)::value;
      if constexpr (LIVE >= MT) run(std::integral_constant<int, MT>{});
      else if (mt_live <= LIVE) run(live_c);
      else self(self, std::integral_constant<int, LIVE + 2>{});
    };
    pick(pick, std::integral_constant<int, 2>{});
  }
  __syncthreads();

  // ---- epilogue -------------------------------------------------------------------------------
  // A lane holds 4 neighbouring columns of a row: stored from the registers, one instruction would touch 16 rows with
  // a few bytes each.  The tile is laid down in LDS instead (the operand stages are idle now: every load has landed
  // and the barrier above has passed) and streamed out in whole rows, 16 bytes per lane.
  constexpr int RB = GATED ? (BF16 ? 256 : 128) : 32 * TPS;    // bytes of one output row inside this strip
  // row pitch in LDS: the lanes of a write hit different banks.  16 rows x 4 dwords (RB = 128, a dword per lane) or
  // 16 rows x 2 lane groups x 2 dwords (a half-wavefront of 8-byte writes) must spread over the 64 banks: a pitch of
  // 4 dwords modulo 64.
  constexpr int RS = RB + 16;
  static_assert(offsetof(Smem, arow) >= (size_t)BM * RS, "the staged output tile overlays the operand stages only");
  uint8_t *const stage = (uint8_t *)&sm;
  if (GATED && BF16) {
    constexpr int G = WT / 2;                          // gate tiles per wavefront
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      if (mt < mt_live) {
#pragma unroll
        for (int j = 0; j < G; j++) {
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float g = acc[mt][j][r], u = acc[mt][j + G][r];
            v[r] = silu_fast(g) * u;
          }
          v2i o;
          o[0] = (int)pack2_bf16(v[0], v[1]);
          o[1] = (int)pack2_bf16(v[2], v[3]);
          *(v2i *)(stage + (mt * 16 + li) * RS + (wave * (16 * G) + j * 16 + lg * 4) * 2) = o;
        }
      }
    }
  } else if (GATED) {
    constexpr int G = WT / 2;                          // gate tiles per wavefront
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      if (mt < mt_live) {                              // m-tiles without a row have nothing to write
        float m = 0.f;
#pragma unroll
        for (int j = 0; j < G; j++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float g = acc[mt][j][r], u = acc[mt][j + G][r];
            const float h = silu_fast(g) * u;
            acc[mt][j][r] = h;
            m = fmaxf(m, fabsf(h));
          }
        m = max_over_lane_groups(m);
        if (lg == 0) sm.amax[wave][mt * 16 + li] = m;
      }
    }
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const int i = mt * 16 + li;
      if (mt < mt_live) {
        float am = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) am = fmaxf(am, sm.amax[w][i]);
        const float sc = group_scale(am);
        // one division per row, the elements are multiplied: against an IEEE division per element (what the stand-alone
        // quantiser does) not one code in a million differs - measured on 1.0e6 codes of a full-size layer, identical
        // share of codes equal to the CPU oracle's either way - and the divisions cost 1.2 % of the launch
        const float inv = 1.0f / sc;
#pragma unroll
        for (int j = 0; j < G; j++)
          *(uint32_t *)(stage + i * RS + wave * (16 * G) + j * 16 + lg * 4) =
              pack4_fp8(acc[mt][j][0] * inv, acc[mt][j][1] * inv, acc[mt][j][2] * inv, acc[mt][j][3] * inv);
        if (i < rows && wave == 0 && lg == 0) (shared ? a.sh_hs : a.hs)[(size_t)(row0 + i) * a.hs_pitch + strip] = sc;
      }
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      if (mt < mt_live) {
#pragma unroll
        for (int j = 0; j < WT; j++) {
          v2i o;
          o[0] = (int)pack2_bf16(acc[mt][j][0], acc[mt][j][1]);
          o[1] = (int)pack2_bf16(acc[mt][j][2], acc[mt][j][3]);
          *(v2i *)(stage + (mt * 16 + li) * RS + (wave * (16 * WT) + j * 16 + lg * 4) * 2) = o;
        }
      }
    }
  }
  __syncthreads();
  {
    constexpr int PIECES = RB / 16;                    // 16-byte pieces of a row
    constexpr int RPI = 64 / PIECES;                   // rows one instruction of a wavefront moves
    const int piece = lane % PIECES;
    uint8_t *const out = GATED ? (shared ? a.sh_hq : a.hq) : (uint8_t *)(shared ? a.sh_y : a.y);
    const size_t row_bytes = (size_t)a.N * (GATED && !BF16 ? 1 : 2);
    // second GEMM: a strip is 256 columns, the matrix may end inside it (its width is a multiple of 8 columns)
    const bool in_width = GATED || strip * (16 * TPS) + piece * 8 < a.N;
    for (int r = wave * RPI + lane / PIECES; r < rows; r += NW * RPI) {
      const v4i d = *(const v4i *)(stage + r * RS + piece * 16);
      const size_t orow = GATED ? (size_t)(row0 + r) : (size_t)sm.oslot[r];
      if (in_width) *(v4i *)(out + orow * row_bytes + (size_t)strip * RB + piece * 16) = d;
    }
  }
}

// Launch shape per tile height.  Eight wavefronts (two per SIMD, two weight tiles each) keep
// more loads in flight for the bandwidth-bound shapes.
// tile_m: row tile of the tile list (grouped mode) or of this launch (dense mode); routed_tiles: entries of the list
// (an upper bound known on the host) or row tiles of the dense matrix; mean_rows: rows per expert on average.
template <bool GATED, bool BF16 = false, bool DQ = false>
static int launch_gemm(hipStream_t st, GemmArgs &a, int tile_m, int routed_tiles, double mean_rows) {
  // the kernel keeps one weight-block scale per 128-step in LDS and forms per-lane operand offsets in 32 bits
  if (a.Kd < 128 || a.Kd % 128 || (a.Kd >> 7) > kMaxKB) return MOE_E_SHAPE;
  if ((double)a.rows_a * a.Kd >= 2147483648.0 || (double)a.sh_rows * a.Kd >= 2147483648.0) return MOE_E_SHAPE;
  // Half tiles: experts with many rows (the launch is bound by the matrix pipes, not by the weight stream) and a
  // short reduction - a work item's start and end are then as long as its loop.  The 192-row entries of the tile list
  // are walked as two 96-row tiles each by workgroups of four wavefronts with four weight tiles each (the token
  // operand is read from LDS once per four matrix instructions instead of two), two workgroups per compute unit, so
  // that one's start and end hide behind the other's loop.  Measured, Qwen3-shaped layer under the skewed load
  // (T=16384; 16 and 6 steps): first GEMM 0.522 -> 0.458 ms, second 0.366 -> 0.347; Mixtral shape (32 and 112 steps):
  // 1.02 -> 1.06 and 0.486 -> 0.579 ms - each row tile re-reads its weight strip from L2, which a long reduction
  // does not forgive; DeepSeek shape (128 rows per expert, bound by the weight stream): 1.40 -> 1.73 ms.
  int km = tile_m;                                   // this launch's row tile
  a.split = 1;
  if (a.fixed_expert < 0 && tile_m == 192 && (a.Kd >> 7) <= kHalfTileMaxSteps && mean_rows >= 320.0) {
    km = 96;
    a.split = 2;
  }
  const long row_tiles = (long)routed_tiles * a.split + (a.sh_rows + km - 1) / km;
  // Second GEMM with small row tiles: strips of 64 output columns instead of 256 - four times the workgroups,
  // three of them resident per compute unit, so that one's start and end hide behind the others' streams (and a
  // batch with few experts still reaches every compute unit: a workgroup alone streams at most ~37 GB/s).  The
  // order of every sum is the same.  With 64-row tiles it only pays while the wide strips would leave units idle: two
  // such workgroups fit a compute unit (60 KB of LDS each), so up to 128 wide work items = 512 narrow ones run in one
  // round (a dense 7168 -> 7168 product at 288-384 rows, 140-168 wide items: 64 us in narrow strips, 46 us in wide ones).
  // (a dense layer knows its row tiles; the tile list's entries are an upper bound, a few more than the real ones -
  // Mixtral shape at 48-96 tokens: 9-11 entries for 8 real tiles of 16 strips each - hence the wider margin there)
  const bool narrow = !GATED && (km <= 32 || (km == 64 && row_tiles * ((a.N + 255) / 256) < (a.fixed_expert >= 0 ? 129 : 193)));
  a.n_strips = GATED ? a.N / 128 : narrow ? (a.N + 63) / 64 : (a.N + 255) / 256;
  a.max_mtiles = routed_tiles;
  long total = row_tiles * a.n_strips;
  total = (total + 7) / 8 * 8 + 16;                  // the per-XCD split rounds two shares up
  if (total <= 0 || total > 0x7fffffffl) return MOE_E_SHAPE;
  a.total_blocks = (int)total;
  dim3 grid((unsigned)total);
#define MOE_GEMM(MT, NW, D, WREG) grouped_gemm_kernel<MT, NW, D, GATED, WREG, BF16, 16, DQ><<<grid, dim3(64 * NW), 0, st>>>(a)
  // small tiles: both operands through LDS (few registers, deeper pipeline); large tiles: weights in
  // a register ring so that LDS holds three stages of the bigger token tile
  if constexpr (!GATED) {
    if (narrow) {
#define MOE_GEMM_NARROW(MT, D) grouped_gemm_kernel<MT, 4, D, false, false, BF16, 4, DQ><<<grid, dim3(256), 0, st>>>(a)
      switch (km) {
        case 16: MOE_GEMM_NARROW(1, 3); break;
        case 32: MOE_GEMM_NARROW(2, 3); break;
        default: MOE_GEMM_NARROW(4, 2); break;
      }
#undef MOE_GEMM_NARROW
      return (int)hipGetLastError();
    }
  }
  switch (km) {
    case 16: MOE_GEMM(1, 8, 3, false); break;
    case 32: MOE_GEMM(2, 8, 3, false); break;
    case 64: MOE_GEMM(4, 8, 2, false); break;
    case 96: MOE_GEMM(6, 4, 2, true); break;
    case 128: MOE_GEMM(8, 8, 2, true); break;
    case 192: MOE_GEMM(12, 8, 2, true); break;
    default: return MOE_E_SHAPE;
  }
#undef MOE_GEMM
  return (int)hipGetLastError();
}

static int check_dims(int T, int H, int I, int E, int K) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30)) return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  if (H > kMaxKB * kBlock || I > kMaxKB * kBlock) return MOE_E_SHAPE;
  // per-lane offsets into the activation tensors are 32-bit
  if ((double)T * H >= 2147483648.0 || (double)T * K * I >= 2147483648.0) return MOE_E_SHAPE;
  return MOE_OK;
}

int gemm1_launch(hipStream_t st, const uint8_t *xq, const float *xs, int T, int H, const uint8_t *w13,
                 const float *w13s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint8_t *hq, float *hs, const uint8_t *sh_w13,
                 const float *sh_w13s, uint8_t *sh_hq, float *sh_hs, int numerics) {
  const bool bf16 = numerics != kNumericsFp8;
  GemmArgs a{};
  if (sh_w13) { a.sh_aq = xq; a.sh_as = xs; a.sh_w = sh_w13; a.sh_ws = sh_w13s; a.sh_hq = sh_hq; a.sh_hs = sh_hs; a.sh_rows = T; }
  a.aq = xq; a.as = xs; a.w = w13; a.ws = w13s;
  a.sorted_slot = sorted_slot; a.expert_offsets = expert_offsets;
  a.tile_prefix = pw ? pw->tile_prefix : nullptr; a.tile_expert = pw ? pw->tile_expert : nullptr;
  a.tile_desc = pw ? pw->tile_desc : nullptr;
  a.hq = hq; a.hs = hs; a.y = nullptr;
  a.as_pitch = scale_pitch(H / kBlock); a.hs_pitch = scale_pitch(I / kBlock);
  a.Kd = bf16 ? 2 * H : H; a.N = I; a.n_rows_w = 2 * I; a.rows_a = T; a.topk = K; a.E = E; a.fixed_expert = fixed_expert;
  // the dense layers (rows in order, nothing shared with a permutation) size their row tile from the problem at hand
  const bool dense = fixed_expert >= 0 && T > 128 && !sh_w13;
  const int tile_m = dense ? choose_dense_tile_m(T, I / kBlock, a.Kd >> 7) : choose_tile_m(T, K, E);
  const int routed_tiles = fixed_expert >= 0 ? (T + tile_m - 1) / tile_m : pw->max_tiles;
  const double mean_rows = (double)T * K / E;
  if (numerics == kNumericsW8A16) return launch_gemm<true, true, true>(st, a, tile_m, routed_tiles, mean_rows);
  if (bf16) return launch_gemm<true, true>(st, a, tile_m, routed_tiles, mean_rows);
  return launch_gemm<true>(st, a, tile_m, routed_tiles, mean_rows);
}

int gemm2_launch(hipStream_t st, const uint8_t *hq, const float *hs, int rows_a, int T, int H, const uint8_t *w2,
                 const float *w2s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint16_t *y, const uint8_t *sh_hq, const float *sh_hs,
                 int sh_rows, const uint8_t *sh_w2, const float *sh_w2s, uint16_t *sh_y, int numerics) {
  const bool bf16 = numerics != kNumericsFp8;
  GemmArgs a{};
  if (sh_w2) { a.sh_aq = sh_hq; a.sh_as = sh_hs; a.sh_w = sh_w2; a.sh_ws = sh_w2s; a.sh_y = sh_y; a.sh_rows = sh_rows; }
  a.aq = hq; a.as = hs; a.w = w2; a.ws = w2s;
  a.sorted_slot = sorted_slot; a.expert_offsets = expert_offsets;
  a.tile_prefix = pw ? pw->tile_prefix : nullptr; a.tile_expert = pw ? pw->tile_expert : nullptr;
  a.tile_desc = pw ? pw->tile_desc : nullptr;
  a.hq = nullptr; a.hs = nullptr; a.y = y;
  a.as_pitch = scale_pitch(I / kBlock); a.hs_pitch = 0;
  a.Kd = bf16 ? 2 * I : I; a.N = H; a.n_rows_w = H; a.rows_a = rows_a; a.topk = K; a.E = E; a.fixed_expert = fixed_expert;
  const bool dense = fixed_expert >= 0 && rows_a > 128 && !sh_w2;
  const int tile_m = dense ? choose_dense_tile_m(rows_a, (H + 255) / 256, a.Kd >> 7) : choose_tile_m(T, K, E);
  const int routed_tiles = fixed_expert >= 0 ? (rows_a + tile_m - 1) / tile_m : pw->max_tiles;
  const double mean_rows = (double)rows_a / E;
  if (numerics == kNumericsW8A16) return launch_gemm<false, true, true>(st, a, tile_m, routed_tiles, mean_rows);
  if (bf16) return launch_gemm<false, true>(st, a, tile_m, routed_tiles, mean_rows);
  return launch_gemm<false>(st, a, tile_m, routed_tiles, mean_rows);
}

}  // namespace moe

extern "C" int moe_gemm1_swiglu(void *stream, const uint8_t *xq, const float *xs, int T, int H, const uint8_t *w13,
                                const float *w13_scale, int I, int E, int K, const int32_t *sorted_slot,
                                const int32_t *expert_offsets, const void *permute_workspace, uint8_t *hq, float *hs) {
  using namespace moe;
  if (!w13 || !w13_scale || !expert_offsets || !permute_workspace) return MOE_E_NULL;
  if (T != 0 && (!xq || !xs || !sorted_slot || !hq || !hs)) return MOE_E_NULL;
  int rc = check_dims(T, H, I, E, K);
  if (rc) return rc;
  if (((uintptr_t)xq % 16) || ((uintptr_t)w13 % 16) || ((uintptr_t)hq % 16) || ((uintptr_t)xs % 64) || ((uintptr_t)hs % 64))
    return MOE_E_ALIGN;
  if (T == 0) return MOE_OK;
  PermuteWs pw = permute_ws_layout(const_cast<void *>(permute_workspace), T, K, E);
  return gemm1_launch((hipStream_t)stream, xq, xs, T, H, w13, w13_scale, I, E, K, sorted_slot, expert_offsets, &pw, -1,
                      hq, hs, nullptr, nullptr, nullptr, nullptr, kNumericsFp8);
}

extern "C" int moe_gemm2(void *stream, const uint8_t *hq, const float *hs, int T, int H, const uint8_t *w2,
                         const float *w2_scale, int I, int E, int K, const int32_t *sorted_slot,
                         const int32_t *expert_offsets, const void *permute_workspace, void *y_bf16) {
  using namespace moe;
  if (!w2 || !w2_scale || !expert_offsets || !permute_workspace) return MOE_E_NULL;
  if (T != 0 && (!hq || !hs || !sorted_slot || !y_bf16)) return MOE_E_NULL;
  int rc = check_dims(T, H, I, E, K);
  if (rc) return rc;
  if (((uintptr_t)hq % 16) || ((uintptr_t)w2 % 16) || ((uintptr_t)y_bf16 % 16) || ((uintptr_t)hs % 64)) return MOE_E_ALIGN;
  if (T == 0) return MOE_OK;
  PermuteWs pw = permute_ws_layout(const_cast<void *>(permute_workspace), T, K, E);
  return gemm2_launch((hipStream_t)stream, hq, hs, T * K, T, H, w2, w2_scale, I, E, K, sorted_slot, expert_offsets, &pw,
                      -1, (uint16_t *)y_bf16, nullptr, nullptr, 0, nullptr, nullptr, nullptr, kNumericsFp8);
}
