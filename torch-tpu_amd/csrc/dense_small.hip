// Dense block-scaled FP8 linear layer at decode batch sizes (M <= 128): out [M, N] = x [M, K] . w [N, K]^T.
//
// With so few rows the work is streaming the weights once, and the grouped kernel's 256-column
// strips leave most of the chip idle (N = 1536 gives six workgroups).  Here one WAVEFRONT is the
// unit: it owns one 16-row weight tile for a slice of the reduction and up to 64 token rows, keeps
// everything in registers (no LDS, no barrier, operands loaded straight into matrix-instruction
// layout), and several wavefronts per SIMD hide each other's load latency.  Slices of the
// reduction are summed by a second, tiny kernel in a fixed order, so results are reproducible.
#include <type_traits>
#include "moe_common.h"
#include "moe_layout.h"
#include "../../include/moe_hip.h"

namespace moe {

struct SmallArgs {
  const uint8_t *xq;     // [M, K] fp8
  const float *xs;       // [M, xs_pitch] fp32
  const uint8_t *w;      // [N, K] fp8
  const float *ws;       // [ceil(N/128), K/128] fp32
  float *partial;        // [n_splits, M, N] fp32 (n_splits > 1)
  uint16_t *out;         // [M, N] bf16 (n_splits == 1)
  int xs_pitch, M, K, N, NKB;
  int split_len;         // reduction steps per slice
  int n_splits, n_mchunks;
  int keep_partial;      // write fp32 slices even when there is only one (a fused reduction follows)
};

__device__ __forceinline__ v8i cat8(v4i a, v4i b) {
  v8i r;
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
  r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
  return r;
}

// MT   m-tiles of 16 token rows per work item
// NTW  weight tiles of 16 rows per work item: every token operand loaded from L2 serves NTW matrix
//      instructions (wide layers), or 1 to get the most work items out of a narrow layer
// STREAM  the weights are read once and are too many for the caches: non-temporal loads
// a workgroup is one wavefront: the dispatcher then spreads the work items over the compute units one by one (with
// four per workgroup a 7168 x 36864 layer put 8 wavefronts on some units and 12 on others, and ran 6 % longer)
constexpr int kDsWaves = 1;
template <int MT, int NTW, bool STREAM>
__global__ __launch_bounds__(64 * kDsWaves) void dense_small_kernel(const SmallArgs a) {
  constexpr int U = NTW == 1 ? 4 : 1;                    // reduction steps of one load batch
  constexpr int NB = NTW == 1 ? 1 : 2;                   // batches held in registers
  const int lane = threadIdx.x & 63, li = lane & 15, lg = lane >> 4;
  const int n_tiles = a.N / (16 * NTW);
  long item = (long)blockIdx.x * kDsWaves + (threadIdx.x >> 6);  // (row chunk, slice, weight tile group), the last fastest
  const int nt = (int)(item % n_tiles);
  item /= n_tiles;
  const int sp = (int)(item % a.n_splits);
  const int mc = (int)(item / a.n_splits);
  if (mc >= a.n_mchunks) return;
  const int kb0 = sp * a.split_len, kb1 = min(kb0 + a.split_len, a.NKB);
  if (kb0 >= kb1) return;
  // lane (li, lg) holds row li of an operand tile and 16-byte reduction chunks lg and lg + 4.  The weights are
  // stored tile-blocked: a (tile, step) pair is 2 KB in operand order, two halves of [lane][16 bytes]
  const uint8_t *wp = a.w + (size_t)(nt * 16 * NTW) * a.K + lane * 16;
  const size_t wtile = (size_t)16 * a.K;                 // bytes between consecutive weight tiles
  const float *wsp = a.ws + (size_t)((nt * NTW) >> 3) * a.NKB;   // a group of tiles lies inside one 128-row block
  const uint8_t *xp[MT];
  const float *sap[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int row = min(mc * 16 * MT + mt * 16 + li, a.M - 1);
    xp[mt] = a.xq + (size_t)row * a.K + lg * 16;
    sap[mt] = a.xs + (size_t)row * a.xs_pitch;
  }
  v4f acc[NTW][MT];
#pragma unroll
  for (int j = 0; j < NTW; j++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[j][mt] = (v4f){0.f, 0.f, 0.f, 0.f};
  // Wide layers (NTW = 4): two batches of one step in registers; the loads of the next batch are issued before the
  // matrix work of the current one, so a wavefront always has a batch in flight (with one batch, loaded and then
  // consumed, only the other wavefronts of the SIMD cover its load latency: the weight stream of a 7168 x 36864 layer
  // ran at 3.9 TB/s, now 5 TB/s).  Narrow layers (NTW = 1): slices of a few steps, one batch of four steps per pass -
  // most items are a single round trip to memory.  The sums are formed in the same order either way.
  v4i wl[NB][U][NTW], wh[NB][U][NTW], xl[NB][U][MT], xh[NB][U][MT];
  float f[NB][U][MT];
  auto load = [&](auto buf_c, int kb) {
    constexpr int B = decltype(buf_c)::value;
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int kk = min(kb + u, kb1 - 1);               // past the slice: the last step again, times zero
      const float sb = kb + u < kb1 ? wsp[kk] : 0.f;
#pragma unroll
      for (int j = 0; j < NTW; j++) {
        const v4i *lo = (const v4i *)(wp + j * wtile + (size_t)kk * 2048), *hi = lo + 64;
        // a large matrix whose rows fit one work item per weight tile is read once, every byte: streamed with the
        // non-temporal hint (7 % faster on a 7168 x 18432 gated MLP at 32 rows)
        if (STREAM) { wl[B][u][j] = __builtin_nontemporal_load(lo); wh[B][u][j] = __builtin_nontemporal_load(hi); }
        else { wl[B][u][j] = *lo; wh[B][u][j] = *hi; }
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        xl[B][u][mt] = *(const v4i *)(xp[mt] + (size_t)kk * 128);
        xh[B][u][mt] = *(const v4i *)(xp[mt] + (size_t)kk * 128 + 64);
        f[B][u][mt] = sap[mt][kk] * sb;
      }
    }
  };
  auto compute = [&](auto buf_c) {
    constexpr int B = decltype(buf_c)::value;
#pragma unroll
    for (int u = 0; u < U; u++) {
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const v8i xc = cat8(xl[B][u][mt], xh[B][u][mt]);
#pragma unroll
        for (int j = 0; j < NTW; j++) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
          const v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(cat8(wl[B][u][j], wh[B][u][j]), xc, zero, 0, 0, 0, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; r++) acc[j][mt][r] = fmaf(p[r], f[B][u][mt], acc[j][mt][r]);
        }
      }
    }
  };
  using buf0 = std::integral_constant<int, 0>;
  if constexpr (NB == 1) {
    for (int kb = kb0; kb < kb1; kb += U) {
      load(buf0{}, kb);
      compute(buf0{});
    }
  } else {
    load(buf0{}, kb0);
    for (int kb = kb0; kb < kb1; kb += 2 * U) {
      // a batch past the end of the slice is the last step again with factor zero: loaded (from cache), never computed
      load(std::integral_constant<int, NB - 1>{}, kb + U);
      compute(buf0{});
      if (kb + U >= kb1) break;
      load(buf0{}, kb + 2 * U);
      compute(std::integral_constant<int, NB - 1>{});
    }
  }
  // a lane holds output columns (tile)*16 + 4*lg .. +3 of token row li of each m-tile
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int row = mc * 16 * MT + mt * 16 + li;
    if (row >= a.M) continue;
#pragma unroll
    for (int j = 0; j < NTW; j++) {
      const size_t o = (size_t)row * a.N + (nt * NTW + j) * 16 + lg * 4;
      if (a.n_splits == 1 && !a.keep_partial) {
        v2i v;
        v[0] = (int)((uint32_t)f32_to_bf16(acc[j][mt][0]) | ((uint32_t)f32_to_bf16(acc[j][mt][1]) << 16));
        v[1] = (int)((uint32_t)f32_to_bf16(acc[j][mt][2]) | ((uint32_t)f32_to_bf16(acc[j][mt][3]) << 16));
        *(v2i *)(a.out + o) = v;
      } else {
        *(v4f *)(a.partial + (size_t)sp * a.M * a.N + o) = acc[j][mt];
      }
    }
  }
}

// out[m, n] = bf16(sum over slices in slice order), four columns per lane
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial, int n_splits, size_t mn,
                                                           uint16_t *__restrict__ out) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= mn) return;
  v4f s = *(const v4f *)(partial + i);
  for (int k = 1; k < n_splits; k++) {
    const v4f t = *(const v4f *)(partial + (size_t)k * mn + i);
    s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
  }
  v2i v;
  v[0] = (int)((uint32_t)f32_to_bf16(s[0]) | ((uint32_t)f32_to_bf16(s[1]) << 16));
  v[1] = (int)((uint32_t)f32_to_bf16(s[2]) | ((uint32_t)f32_to_bf16(s[3]) << 16));
  *(v2i *)(out + i) = v;
}

// Gated-MLP middle stage on the slices of the first product [n_splits, M, 2I] (gate columns, then up
// columns): h = silu(sum gate) * (sum up), re-quantised per row and 128 columns.  Sixteen lanes share
// one (row, 128-column group), eight columns each.
__global__ __launch_bounds__(256) void swiglu_quant_reduce_kernel(const float *__restrict__ partial, int n_splits, int M,
                                                                 int I, int hs_pitch, uint8_t *__restrict__ hq,
                                                                 float *__restrict__ hs) {
  const size_t grp = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  const int groups_per_row = I / kBlock;
  const bool live = grp < (size_t)M * groups_per_row;
  float h[8];
  float amax = 0.f;
  size_t row = 0;
  int col = 0;
  if (live) {
    row = grp / groups_per_row;
    col = (int)(grp % groups_per_row) * kBlock + sub * 8;
    float g[8], u[8];
#pragma unroll
    for (int i = 0; i < 8; i++) g[i] = u[i] = 0.f;
    const size_t mn = (size_t)M * 2 * I;
    for (int k = 0; k < n_splits; k++) {
      const float *p = partial + (size_t)k * mn + row * 2 * I + col;
      const v4f g0 = *(const v4f *)p, g1 = *(const v4f *)(p + 4), u0 = *(const v4f *)(p + I), u1 = *(const v4f *)(p + I + 4);
#pragma unroll
      for (int i = 0; i < 4; i++) { g[i] += g0[i]; g[4 + i] += g1[i]; u[i] += u0[i]; u[4 + i] += u1[i]; }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      h[i] = (g[i] / (1.0f + expf(-g[i]))) * u[i];
      amax = fmaxf(amax, fabsf(h[i]));
    }
  }
  amax = max_over_row16(amax);
  if (!live) return;
  const float sc = group_scale(amax);
  v2i o;
  o[0] = (int)pack4_fp8(h[0] / sc, h[1] / sc, h[2] / sc, h[3] / sc);
  o[1] = (int)pack4_fp8(h[4] / sc, h[5] / sc, h[6] / sc, h[7] / sc);
  *(v2i *)(hq + row * I + col) = o;
  if (sub == 0) hs[row * hs_pitch + col / kBlock] = sc;
}

// How the reduction is sliced: enough wavefront-sized work items to fill the chip (the reference's
// launcher weighs the same split-N against split-K trade-off on the host, MmW8A16Dq.cpp:94-142).
void dense_small_plan(int M, int K, int N, int *n_splits, int *split_len, int *rows_per_item, int *n_mchunks,
                      int *tiles_per_item) {
  const int NKB = K / kBlock;
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int chunks = M > 0 ? (M + 16 * mt - 1) / (16 * mt) : 1;        // an empty batch plans like one row
  // four weight tiles per item when the layer is wide enough to still fill the chip with short slices
  // (with two or four m-tiles per item a lone weight tile would have the item load 2 to 4 token tiles per matrix
  // instruction: 7168 x 7168 at 64 rows 49.5 -> 26.4 us, 4096 x 14336 52.0 -> 30.3 us with four tiles from 128 such items on)
  const int ntw = (N % 64 == 0 && (long)(N / 64) * chunks * (NKB / 8) >= (mt == 1 ? 1024 : 128)) ? 4 : 1;
  *tiles_per_item = ntw;
  const long tiles = (long)(N / (16 * ntw)) * chunks;
  // wavefront-sized work items: about two per SIMD for a narrow layer; fewer and longer for a wide one, whose items keep
  // a load batch in flight on their own.  Measured on 7168 x 36864, product alone, 4096 / 2048 / 1536 / 1024 / 576
  // items wanted: 32 rows - / 62 / 62 / 60 / - us (gated MLP 18432: 0.118 / 0.101 / - / 0.096 / 0.125 ms), 128 rows
  // - / 159 / 159 / 129 us; up to 16 rows (little matrix work between the loads) 1 row 46.8 / 46.2 / 50.3 us,
  // 16 rows 51.7 / 50.3 / 48.3 us
  const int target = ntw == 1 ? 2048 : (mt == 1 ? 1536 : 1024);
  long want = (target + tiles - 1) / tiles;
  if (want < 1) want = 1;
  int len = (int)((NKB + want - 1) / want);
  len = (len + 3) / 4 * 4;                               // whole load batches
  if (len > NKB) len = NKB;
  *split_len = len;
  *n_splits = (NKB + len - 1) / len;
  *rows_per_item = 16 * mt;
  *n_mchunks = chunks;
}

size_t dense_small_partial_bytes(int M, int K, int N, bool keep_partial) {
  int s, l, r, c, t;
  dense_small_plan(M, K, N, &s, &l, &r, &c, &t);
  return (s > 1 || keep_partial) ? (size_t)s * M * N * 4 : 0;
}

// out != nullptr: bf16 result (slices added by a second kernel); out == nullptr: the fp32 slices stay in
// `partial` for the caller's own reduction, their number is returned through n_splits_out.
int dense_small_launch(hipStream_t st, const uint8_t *xq, const float *xs, int M, int K, const uint8_t *w, const float *ws,
                       int N, uint16_t *out, float *partial, int *n_splits_out) {
  SmallArgs a{};
  a.keep_partial = out == nullptr;
  int rows, ntw;
  dense_small_plan(M, K, N, &a.n_splits, &a.split_len, &rows, &a.n_mchunks, &ntw);
  a.xq = xq; a.xs = xs; a.xs_pitch = scale_pitch(K / kBlock); a.w = w; a.ws = ws; a.partial = partial; a.out = out;
  a.M = M; a.K = K; a.N = N; a.NKB = K / kBlock;
  const bool stream_w = a.n_mchunks == 1 && (size_t)N * K >= ((size_t)64 << 20);
  const long items = (long)(N / (16 * ntw)) * a.n_splits * a.n_mchunks;
  const long blocks = (items + kDsWaves - 1) / kDsWaves;
  if (blocks > 0x7fffffffl) return MOE_E_SHAPE;
  const unsigned g = (unsigned)blocks;
#define MOE_DENSE_SMALL(MT, NTW)                                                          \
  do {                                                                                    \
    if (stream_w) dense_small_kernel<MT, NTW, true><<<g, 64 * kDsWaves, 0, st>>>(a);                 \
    else dense_small_kernel<MT, NTW, false><<<g, 64 * kDsWaves, 0, st>>>(a);                         \
  } while (0)
  if (ntw == 1) {
    if (rows == 16) MOE_DENSE_SMALL(1, 1);
    else if (rows == 32) MOE_DENSE_SMALL(2, 1);
    else MOE_DENSE_SMALL(4, 1);
  } else {
    if (rows == 16) MOE_DENSE_SMALL(1, 4);
    else if (rows == 32) MOE_DENSE_SMALL(2, 4);
    else MOE_DENSE_SMALL(4, 4);
  }
#undef MOE_DENSE_SMALL
  if (n_splits_out) *n_splits_out = a.n_splits;
  if (a.n_splits > 1 && out != nullptr) {
    const size_t mn = (size_t)M * N;
    splitk_reduce_kernel<<<(unsigned)((mn / 4 + 255) / 256), 256, 0, st>>>(partial, a.n_splits, mn, out);
  }
  return (int)hipGetLastError();
}

int swiglu_quant_reduce_launch(hipStream_t st, const float *partial, int n_splits, int M, int I, uint8_t *hq, float *hs) {
  const size_t lanes = (size_t)M * (I / kBlock) * 16;
  swiglu_quant_reduce_kernel<<<(unsigned)((lanes + 255) / 256), 256, 0, st>>>(partial, n_splits, M, I,
                                                                             scale_pitch(I / kBlock), hq, hs);
  return (int)hipGetLastError();
}

}  // namespace moe
