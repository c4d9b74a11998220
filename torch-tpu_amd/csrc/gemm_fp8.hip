// Grouped block-scaled FP8 GEMMs of the expert MLP on gfx950 matrix cores.
//
// One workgroup (4 wavefronts) owns a tile of one expert: BM = 16*MT permuted rows (tokens)
// by a strip of that expert's weight rows (output columns).  The reduction runs in steps of
// 128 = one quantisation block = one v_mfma_f32_16x16x128_f8f6f4, so every matrix
// instruction yields the un-scaled partial sum of exactly one (activation group, weight block)
// pair and the two fp32 scales are applied in registers right after it:
//     acc += partial * (act_scale[row, kb] * weight_scale[n_block, kb]).
//
// Operand roles: the WEIGHT tile is the MFMA "A" operand (its 16 rows become the rows of the
// 16x16 result) and the TOKEN tile is the "B" operand (its 16 rows become the columns).  A
// lane then holds 4 consecutive output columns of ONE token, which makes the activation scale
// a single value per lane and instruction, and lets the epilogue pack 4 outputs per store.
//   lane l of an operand: row (l % 16), reduction bytes 32*(l / 16) .. +31 of the 128-step
//   lane l of the result: c[r] = (weight row 4*(l / 16) + r, token l % 16)
//
// Data movement per step: weights stream HBM -> registers directly in operand layout (each
// weight byte is used by one wavefront only, so LDS would add nothing); the token tile is
// shared by the four wavefronts and goes HBM/L2 -> registers -> LDS (XOR-swizzled 16-byte
// chunks, conflict-free 128-bit reads), double buffered, one barrier per step.  Loads for
// step kb+1 are issued before the matrix work of step kb.
//
// GATED = true  (first GEMM): the strip is 128 gate columns plus the 128 matching up columns of
//   W13; wavefront w owns gate columns 32w..32w+31 and the same up columns.  Epilogue:
//   h = silu(gate) * up, per-token amax over the strip's 128 columns (registers -> lane
//   butterflies -> LDS across the four wavefronts), scale = max(amax, 1e-10) / 448, h / scale -> e4m3fn.
// GATED = false (second GEMM): the strip is 256 output columns, wavefront w owns 64 of them;
//   the bf16 result row is written at its slot (t*K + k), which undoes the permutation.
#include "moe_common.h"
#include "moe_layout.h"
#include "../../include/moe_hip.h"

namespace moe {

struct GemmArgs {
  const uint8_t *aq;            // activations fp8 [rows_a, Kd]
  const float *as;              // activation scales [rows_a, Kd/128]
  const uint8_t *w;             // weights fp8 [E, n_rows_w, Kd]
  const float *ws;              // weight scales [E, n_rows_w/128, Kd/128]
  const int32_t *sorted_slot;   // [TK]
  const int32_t *expert_offsets;
  const int32_t *tile_prefix;
  const int32_t *tile_expert;
  uint8_t *hq;                  // GATED: [TK, N] fp8
  float *hs;                    // GATED: [TK, N/128]
  uint16_t *y;                  // !GATED: [TK, N] bf16 in slot order
  int Kd;                       // reduction length (multiple of 128)
  int N;                        // GATED: I (gate columns); !GATED: H
  int n_rows_w;                 // GATED: 2*I; !GATED: H
  int rows_a;                   // T (GATED) or TK (!GATED): bound for gathered row ids
  int topk;                     // K
  int n_strips;                 // strips along N
  int total_blocks;             // launched workgroups (multiple of 8)
  int E;                        // experts (tile_prefix[E] = number of row tiles)
  int fixed_expert;             // >= 0: dense mode, every row belongs to this expert and A row p = p
  int max_mtiles;               // entries allocated in tile_expert
};

template <int MT>
struct GemmSmem {
  static constexpr int BM = 16 * MT;
  alignas(16) uint8_t tok[2][BM * 128];   // token tile, two stages, swizzled 16-byte chunks
  float sa[2][BM];              // activation scales of the step
  int arow[BM];                 // source row in aq / as for each tile row
  float amax[4][BM];            // GATED epilogue: per-wavefront partial amax
};

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

template <int MT, bool GATED>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(const GemmArgs a) {
  constexpr int BM = 16 * MT;
  constexpr int NCHUNK = BM * 8;                      // 16-byte chunks of one token-tile stage
  constexpr int NLOAD = (NCHUNK + 255) / 256;         // chunks per thread
  __shared__ GemmSmem<MT> sm;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lg = lane >> 4;

  // ---- which tile -------------------------------------------------------------------------
  // Workgroup ids are dealt round-robin to the 8 XCDs; remap so that each XCD (own L2) gets a
  // contiguous range of logical tiles: neighbours share the token tile.
  const int per_xcd = a.total_blocks >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int mtile = logical / a.n_strips;
  const int strip = logical - mtile * a.n_strips;
  int e, row0, rows;                                  // expert, first permuted row, rows in tile
  if (a.fixed_expert >= 0) {
    e = a.fixed_expert;
    row0 = mtile * BM;
    rows = min(BM, a.rows_a - row0);
  } else {
    if (mtile >= min(a.tile_prefix[a.E], a.max_mtiles)) return;
    e = a.tile_expert[mtile];
    if (e < 0 || e >= a.E) return;
    row0 = a.expert_offsets[e] + (mtile - a.tile_prefix[e]) * BM;
    rows = min(BM, a.expert_offsets[e + 1] - row0);
  }
  if (rows <= 0) return;

  for (int i = tid; i < BM; i += 256) {
    const int p = row0 + min(i, rows - 1);
    int src = p;
    if (GATED && a.fixed_expert < 0) src = a.sorted_slot[p] / a.topk;
    sm.arow[i] = min(max(src, 0), a.rows_a - 1);
  }
  __syncthreads();

  const int NKB = a.Kd >> 7;
  const int n_wblk = a.n_rows_w >> 7;                 // weight-scale rows per expert

  // ---- per-lane source addresses ------------------------------------------------------------
  const uint8_t *wptr[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    int wrow;
    if (GATED) wrow = (j < 2 ? 0 : a.N) + strip * 128 + wave * 32 + (j & 1) * 16 + li;
    else wrow = strip * 256 + wave * 64 + j * 16 + li;
    wrow = min(wrow, a.n_rows_w - 1);
    wptr[j] = a.w + ((size_t)e * a.n_rows_w + wrow) * a.Kd + lg * 32;
  }
  const float *sb0_ptr, *sb1_ptr;
  if (GATED) {
    sb0_ptr = a.ws + ((size_t)e * n_wblk + strip) * NKB;
    sb1_ptr = a.ws + ((size_t)e * n_wblk + (a.N >> 7) + strip) * NKB;
  } else {
    const int nblk = min(strip * 2 + (wave >> 1), n_wblk - 1);
    sb0_ptr = a.ws + ((size_t)e * n_wblk + nblk) * NKB;
    sb1_ptr = sb0_ptr;
  }
  size_t tok_src[NLOAD];
  int tok_dst[NLOAD];
#pragma unroll
  for (int u = 0; u < NLOAD; u++) {
    const int q = min(tid + 256 * u, NCHUNK - 1);
    const int row = q >> 3, c = q & 7;
    tok_src[u] = (size_t)sm.arow[row] * a.Kd + c * 16;
    tok_dst[u] = row * 128 + ((c ^ (row & 7)) << 4);
  }
  const size_t sa_src = (size_t)sm.arow[min(tid, BM - 1)] * NKB;

  v4f acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[mt][j] = (v4f){0.f, 0.f, 0.f, 0.f};

  v8i w0[4], w1[4];
  v4i treg[NLOAD];
  float sareg = 0.f, sbA0, sbA1, sbB0 = 0.f, sbB1 = 0.f;

  auto issue_loads = [&](int kb, v8i(&wn)[4], float &s0, float &s1) {
#pragma unroll
    for (int j = 0; j < 4; j++) wn[j] = load_w_frag(wptr[j] + (size_t)kb * 128);
#pragma unroll
    for (int u = 0; u < NLOAD; u++) treg[u] = *(const v4i *)(a.aq + tok_src[u] + (size_t)kb * 128);
    if (tid < BM) sareg = a.as[sa_src + kb];
    s0 = sb0_ptr[kb];
    s1 = sb1_ptr[kb];
  };
  auto stage_store = [&](int stage) {
#pragma unroll
    for (int u = 0; u < NLOAD; u++)
      if (tid + 256 * u < NCHUNK) *(v4i *)(sm.tok[stage] + tok_dst[u]) = treg[u];
    if (tid < BM) sm.sa[stage][tid] = sareg;
  };
  auto compute = [&](const v8i(&wc)[4], int stage, float s0, float s1) {
    const int sw = li & 7;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const uint8_t *base = sm.tok[stage] + (mt * 16 + li) * 128;
      const v4i x0 = *(const v4i *)(base + (((2 * lg) ^ sw) << 4));
      const v4i x1 = *(const v4i *)(base + (((2 * lg + 1) ^ sw) << 4));
      const v8i x = concat8(x0, x1);
      const float s_a = sm.sa[stage][mt * 16 + li];
      const float f0 = s_a * s0, f1 = s_a * s1;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const v4f zero = {0.f, 0.f, 0.f, 0.f};
        const v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wc[j], x, zero, 0, 0, 0, 0, 0, 0);
        const float f = (GATED && j >= 2) ? f1 : f0;
#pragma unroll
        for (int r = 0; r < 4; r++) acc[mt][j][r] = fmaf(p[r], f, acc[mt][j][r]);
      }
    }
  };

  // ---- main loop: two 128-steps per trip so the weight registers ping-pong without copies -----
  issue_loads(0, w0, sbA0, sbA1);
  stage_store(0);
  __syncthreads();
  for (int kb = 0; kb < NKB; kb += 2) {
    const bool more1 = kb + 1 < NKB;
    if (more1) issue_loads(kb + 1, w1, sbB0, sbB1);
    compute(w0, 0, sbA0, sbA1);
    if (more1) stage_store(1);
    __syncthreads();
    if (!more1) break;
    const bool more2 = kb + 2 < NKB;
    if (more2) issue_loads(kb + 2, w0, sbA0, sbA1);
    compute(w1, 1, sbB0, sbB1);
    if (more2) stage_store(0);
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------------------------
  if (GATED) {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      float m = 0.f;
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float g = acc[mt][j][r], u = acc[mt][j + 2][r];
          const float h = (g / (1.0f + expf(-g))) * u;
          acc[mt][j][r] = h;
          m = fmaxf(m, fabsf(h));
        }
      m = max_over_lane_groups(m);
      if (lg == 0) sm.amax[wave][mt * 16 + li] = m;
    }
    __syncthreads();
    const int n_grp = a.N >> 7;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const int i = mt * 16 + li;
      const bool valid = i < rows;
      const float am = fmaxf(fmaxf(sm.amax[0][i], sm.amax[1][i]), fmaxf(sm.amax[2][i], sm.amax[3][i]));
      const float sc = group_scale(am);
      const size_t orow = (size_t)(row0 + i);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const uint32_t packed = pack4_fp8(acc[mt][j][0] / sc, acc[mt][j][1] / sc, acc[mt][j][2] / sc, acc[mt][j][3] / sc);
        if (valid) *(uint32_t *)(a.hq + orow * a.N + strip * 128 + wave * 32 + j * 16 + lg * 4) = packed;
      }
      if (valid && wave == 0 && lg == 0) a.hs[orow * n_grp + strip] = sc;
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const int i = mt * 16 + li;
      const bool valid = i < rows;
      int slot = row0 + min(i, rows - 1);
      if (a.fixed_expert < 0) slot = a.sorted_slot[slot];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int col = strip * 256 + wave * 64 + j * 16 + lg * 4;
        if (valid && col < a.N) {
          v2i o;
          o[0] = (int)((uint32_t)f32_to_bf16(acc[mt][j][0]) | ((uint32_t)f32_to_bf16(acc[mt][j][1]) << 16));
          o[1] = (int)((uint32_t)f32_to_bf16(acc[mt][j][2]) | ((uint32_t)f32_to_bf16(acc[mt][j][3]) << 16));
          *(v2i *)(a.y + (size_t)slot * a.N + col) = o;
        }
      }
    }
  }
}

template <bool GATED>
static int launch_gemm(hipStream_t st, GemmArgs &a, int tile_m, int max_mtiles) {
  a.n_strips = GATED ? a.N / 128 : (a.N + 255) / 256;
  a.max_mtiles = max_mtiles;
  long total = (long)max_mtiles * a.n_strips;
  total = (total + 7) / 8 * 8;
  if (total <= 0 || total > 0x7fffffffl) return MOE_E_SHAPE;
  a.total_blocks = (int)total;
  dim3 grid((unsigned)total), block(256);
  switch (tile_m) {
    case 16: grouped_gemm_kernel<1, GATED><<<grid, block, 0, st>>>(a); break;
    case 32: grouped_gemm_kernel<2, GATED><<<grid, block, 0, st>>>(a); break;
    case 64: grouped_gemm_kernel<4, GATED><<<grid, block, 0, st>>>(a); break;
    case 128: grouped_gemm_kernel<8, GATED><<<grid, block, 0, st>>>(a); break;
    default: return MOE_E_SHAPE;
  }
  return (int)hipGetLastError();
}

static int check_dims(int T, int H, int I, int E, int K) {
  if (T < 0 || H < 1 || I < 1 || E < 1 || E > MOE_MAX_EXPERTS || K < 1 || K > MOE_MAX_TOPK) return MOE_E_SHAPE;
  if ((long)T * K > (1l << 30)) return MOE_E_SHAPE;
  if (H % kBlock || I % kBlock) return MOE_E_ALIGN;
  return MOE_OK;
}

int gemm1_launch(hipStream_t st, const uint8_t *xq, const float *xs, int T, int H, const uint8_t *w13,
                 const float *w13s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint8_t *hq, float *hs) {
  GemmArgs a{};
  a.aq = xq; a.as = xs; a.w = w13; a.ws = w13s;
  a.sorted_slot = sorted_slot; a.expert_offsets = expert_offsets;
  a.tile_prefix = pw ? pw->tile_prefix : nullptr; a.tile_expert = pw ? pw->tile_expert : nullptr;
  a.hq = hq; a.hs = hs; a.y = nullptr;
  a.Kd = H; a.N = I; a.n_rows_w = 2 * I; a.rows_a = T; a.topk = K; a.E = E; a.fixed_expert = fixed_expert;
  const int tile_m = choose_tile_m(T, K, E);
  const int max_mtiles = fixed_expert >= 0 ? (T + tile_m - 1) / tile_m : pw->max_tiles;
  return launch_gemm<true>(st, a, tile_m, max_mtiles);
}

int gemm2_launch(hipStream_t st, const uint8_t *hq, const float *hs, int rows_a, int T, int H, const uint8_t *w2,
                 const float *w2s, int I, int E, int K, const int32_t *sorted_slot, const int32_t *expert_offsets,
                 const PermuteWs *pw, int fixed_expert, uint16_t *y) {
  GemmArgs a{};
  a.aq = hq; a.as = hs; a.w = w2; a.ws = w2s;
  a.sorted_slot = sorted_slot; a.expert_offsets = expert_offsets;
  a.tile_prefix = pw ? pw->tile_prefix : nullptr; a.tile_expert = pw ? pw->tile_expert : nullptr;
  a.hq = nullptr; a.hs = nullptr; a.y = y;
  a.Kd = I; a.N = H; a.n_rows_w = H; a.rows_a = rows_a; a.topk = K; a.E = E; a.fixed_expert = fixed_expert;
  const int tile_m = choose_tile_m(T, K, E);
  const int max_mtiles = fixed_expert >= 0 ? (rows_a + tile_m - 1) / tile_m : pw->max_tiles;
  return launch_gemm<false>(st, a, tile_m, max_mtiles);
}

}  // namespace moe

extern "C" int moe_gemm1_swiglu(void *stream, const uint8_t *xq, const float *xs, int T, int H, const uint8_t *w13,
                                const float *w13_scale, int I, int E, int K, const int32_t *sorted_slot,
                                const int32_t *expert_offsets, const void *permute_workspace, uint8_t *hq, float *hs) {
  using namespace moe;
  if (!xq || !xs || !w13 || !w13_scale || !sorted_slot || !expert_offsets || !permute_workspace || !hq || !hs)
    return MOE_E_NULL;
  int rc = check_dims(T, H, I, E, K);
  if (rc) return rc;
  if (((uintptr_t)xq % 16) || ((uintptr_t)w13 % 16) || ((uintptr_t)hq % 4)) return MOE_E_ALIGN;
  if (T == 0) return MOE_OK;
  PermuteWs pw = permute_ws_layout(const_cast<void *>(permute_workspace), T, K, E);
  return gemm1_launch((hipStream_t)stream, xq, xs, T, H, w13, w13_scale, I, E, K, sorted_slot, expert_offsets, &pw, -1,
                      hq, hs);
}

extern "C" int moe_gemm2(void *stream, const uint8_t *hq, const float *hs, int T, int H, const uint8_t *w2,
                         const float *w2_scale, int I, int E, int K, const int32_t *sorted_slot,
                         const int32_t *expert_offsets, const void *permute_workspace, void *y_bf16) {
  using namespace moe;
  if (!hq || !hs || !w2 || !w2_scale || !sorted_slot || !expert_offsets || !permute_workspace || !y_bf16)
    return MOE_E_NULL;
  int rc = check_dims(T, H, I, E, K);
  if (rc) return rc;
  if (((uintptr_t)hq % 16) || ((uintptr_t)w2 % 16) || ((uintptr_t)y_bf16 % 8)) return MOE_E_ALIGN;
  if (T == 0) return MOE_OK;
  PermuteWs pw = permute_ws_layout(const_cast<void *>(permute_workspace), T, K, E);
  return gemm2_launch((hipStream_t)stream, hq, hs, T * K, T, H, w2, w2_scale, I, E, K, sorted_slot, expert_offsets, &pw,
                      -1, (uint16_t *)y_bf16);
}
