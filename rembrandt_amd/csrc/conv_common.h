// Host-side helpers shared by the three convolution passes.
#pragma once
#include <stdlib.h>

#include "gemm_core.h"

namespace rh {

inline int conv_out_dim(int in, int size, int stride, int pad) {
  int t = in + 2 * pad - size + stride;
  if (t < 0) t = 0;
  return t / stride;
}

inline size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

// Contraction tables are padded to a multiple of this many entries (>= every BK in use).
constexpr int kTabPad = 64;
// Readable bytes kept after an operand that LoadRow4 reads: its last group of four rows may begin at the last valid row.
constexpr size_t kRow4Slack = 16;

struct ConvDims {
  int N, C, H, W, K, R, S, st, pad, P, Q;
  long long x_elems, w_elems, y_elems;
};

inline int conv_dims(const rh_conv_geom* g, ConvDims* d) {
  if (!g) return RH_E_INVALID;
  if (g->N <= 0 || g->C <= 0 || g->H <= 0 || g->W <= 0 || g->K <= 0 || g->R <= 0 || g->S <= 0 ||
      g->stride <= 0 || g->pad < 0)
    return RH_E_INVALID;
  d->N = g->N; d->C = g->C; d->H = g->H; d->W = g->W; d->K = g->K; d->R = g->R; d->S = g->S;
  d->st = g->stride; d->pad = g->pad;
  d->P = conv_out_dim(g->H, g->R, g->stride, g->pad);
  d->Q = conv_out_dim(g->W, g->S, g->stride, g->pad);
  d->x_elems = (long long)g->N * g->C * g->H * g->W;
  d->w_elems = (long long)g->K * g->C * g->R * g->S;
  d->y_elems = (long long)g->N * g->K * d->P * d->Q;
  if ((size_t)d->x_elems * 4 > kMaxBufferBytes || (size_t)d->y_elems * 4 > kMaxBufferBytes ||
      (size_t)d->w_elems * 4 > kMaxBufferBytes)
    return RH_E_LIMIT;
  return 0;
}

// Row-tile height with the least zero padding for `rows` result rows; ties go to the taller tile.
inline int pick_bm(int rows) {
  const int cand[4] = {128, 96, 64, 32};
  int best = 128;
  long long best_pad = -1;
  for (int i = 0; i < 4; ++i) {
    const long long padded = (long long)round_up(rows, cand[i]);
    if (best_pad < 0 || padded < best_pad) { best_pad = padded; best = cand[i]; }
  }
  return best;
}

template <class T, class AL, class BL, bool NCHW, class PASS>
inline int launch_mfma_gemm(const typename AL::Params& ap, const typename BL::Params& bp,
                            const EpiParams& ep, int K, int splits, int* splits_used,
                            hipStream_t stream, const char* tag, int k_algorithmic = 0) {
  const int tiles_m = cdiv(ep.rows, T::BM), tiles_n = cdiv(ep.cols, T::BN);
  const int k_chunks = cdiv(K, T::BK);
  if (ep.tail_tiles > 0) splits = ep.tail_splits;  // tail form: the slices apply to the last tail_tiles tiles only
  if (splits < 1) splits = 1;
  const int cps = cdiv(k_chunks, splits) > 0 ? cdiv(k_chunks, splits) : 1;
  const int used = cdiv(k_chunks, cps) > 0 ? cdiv(k_chunks, cps) : 1;
  if (splits_used) *splits_used = used;
  dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)used);
  if (ep.tail_tiles > 0) {
    if (used != ep.tail_splits || ep.full_tiles + ep.tail_tiles != tiles_m * tiles_n) return RH_E_INVALID;
    grid = dim3((unsigned)(ep.full_tiles + ep.tail_tiles * ep.tail_splits), 1u);
  }
  constexpr size_t lds_bytes = sizeof(float) * 2 * T::BK * (AL::LD + BL::LD);
  static_assert(lds_bytes <= 160 * 1024, "tile does not fit the 160 KB LDS of a CU");
  if (lds_bytes > 48 * 1024) {
    // opt in to more than the default dynamic LDS limit, once per kernel instantiation
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&mfma_gemm_kernel<T, AL, BL, NCHW, PASS>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr != hipSuccess) return (int)attr;
  }
  ProfScope prof(tag, 2.0 * (double)ep.rows * (double)ep.cols * (double)(k_algorithmic > 0 ? k_algorithmic : K), stream);
  hipLaunchKernelGGL((mfma_gemm_kernel<T, AL, BL, NCHW, PASS>), grid, dim3(T::NT), lds_bytes, stream, ap, bp, ep,
                     tiles_m, k_chunks, cps);
  return launch_status();
}

// Same grid and split logic for the bf16-operand kernel.  FLOPs are counted as for fp32.
template <class T, class AL, class BL, bool NCHW, class PASS, bool PK = false>
inline int launch_mfma_gemm_bf16(const typename AL::Params& ap, const typename BL::Params& bp,
                                 const EpiParams& ep, int K, int splits, int* splits_used,
                                 hipStream_t stream, const char* tag, int k_algorithmic = 0,
                                 const PackedOut& pk = PackedOut()) {
  const int tiles_m = cdiv(ep.rows, T::BM), tiles_n = cdiv(ep.cols, T::BN);
  const int k_chunks = cdiv(K, T::BK);
  if (splits < 1) splits = 1;
  const int cps = cdiv(k_chunks, splits) > 0 ? cdiv(k_chunks, splits) : 1;
  const int used = cdiv(k_chunks, cps) > 0 ? cdiv(k_chunks, cps) : 1;
  if (splits_used) *splits_used = used;
  dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)used);
  constexpr size_t lds_bytes = 16 * 2 * (T::BK / 8) * (T::BM + T::BN);
  static_assert(lds_bytes <= 160 * 1024, "tile does not fit the 160 KB LDS of a CU");
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&mfma_gemm_bf16_kernel<T, AL, BL, NCHW, PASS, PK>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr != hipSuccess) return (int)attr;
  }
  ProfScope prof(tag, 2.0 * (double)ep.rows * (double)ep.cols * (double)(k_algorithmic > 0 ? k_algorithmic : K), stream);
  if (PK && (splits != 1 || !pk.ptr)) return RH_E_INVALID;
  hipLaunchKernelGGL((mfma_gemm_bf16_kernel<T, AL, BL, NCHW, PASS, PK>), grid, dim3(T::NT), lds_bytes, stream, ap, bp, ep,
                     tiles_m, k_chunks, cps, pk);
  return launch_status();
}

// The direct-to-LDS form for packed operands (ring of four LDS buffers, one pass over the whole contraction).
template <class T, bool A_LINEAR, bool B_LINEAR, bool NCHW, class PASS, bool PK = false, int R = 4>
inline int launch_mfma_gemm_bf16_dma(const RowV8Params& ap, const RowV8Params& bp, const EpiParams& ep, int K,
                                     hipStream_t stream, const char* tag, int k_algorithmic = 0,
                                     const PackedOut& pk = PackedOut()) {
  const int tiles_m = cdiv(ep.rows, T::BM), tiles_n = cdiv(ep.cols, T::BN);
  if (K <= 0 || K % T::BK != 0) return RH_E_INVALID;
  constexpr size_t lds_bytes = 16 * R * (T::BK / 8) * (T::BM + T::BN);
  static_assert(lds_bytes * T::OCC <= 160 * 1024, "the blocks meant to share a CU do not fit its 160 KB of LDS");
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&mfma_gemm_bf16_dma_kernel<T, A_LINEAR, B_LINEAR, NCHW, PASS, PK, R>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr != hipSuccess) return (int)attr;
  }
  ProfScope prof(tag, 2.0 * (double)ep.rows * (double)ep.cols * (double)(k_algorithmic > 0 ? k_algorithmic : K), stream);
  if (PK && !pk.ptr) return RH_E_INVALID;
  hipLaunchKernelGGL((mfma_gemm_bf16_dma_kernel<T, A_LINEAR, B_LINEAR, NCHW, PASS, PK, R>), dim3((unsigned)(tiles_m * tiles_n)),
                     dim3(T::NT), lds_bytes, stream, ap, bp, ep, tiles_m, K / T::BK, pk);
  return launch_status();
}

#ifndef RH_OCC_128
#define RH_OCC_128 4
#endif
// Tile shapes in use.  rows x cols x k, waves as WM x WN.
typedef Tile<128, 128, 16, 2, 2, RH_OCC_128> T128x128;
typedef Tile<96, 256, 16, 1, 4> T96x256;
typedef Tile<96, 128, 16, 1, 4, 4> T96x128;
typedef Tile<96, 96, 16, 1, 3, 4> T96x96;   // three waves: a 96 x 96 result (1x1 layer, 96 -> 96 channels) without a quarter of dead columns
#ifndef RH_BF16_BK
#define RH_BF16_BK 32
#endif
#ifndef RH_BF16_OCC
#define RH_BF16_OCC 3
#endif
// bf16-operand kernel: a deeper K step keeps more operand loads in flight per wave (its MFMAs are 16x shorter)
typedef Tile<128, 128, RH_BF16_BK, 2, 2, RH_BF16_OCC> T128x128bf;
// Tile of the direct-to-LDS bf16 kernel: eight waves of 128x64 each, one block per CU, four 32-k LDS buffers.
typedef Tile<256, 256, 32, 2, 4, 1> T256x256bf;
typedef Tile<256, 128, 32, 2, 2, 2> T256x128bf;   // direct-to-LDS form with a ring of three: two blocks of four waves share a CU
typedef Tile<128, 256, 32, 2, 2, 2> T128x256bf;   // the same for filter counts that would waste rows of a 256-row tile
typedef Tile<64, 256, 16, 1, 4, 3> T64x256;
typedef Tile<32, 256, 16, 1, 4, 3> T32x256;
// few result columns as well (a first layer's filter gradient: 20 x 25, 32 x 75): narrower tiles, fewer dead columns
typedef Tile<32, 128, 16, 1, 4, 4> T32x128;
typedef Tile<32, 64, 16, 1, 2, 4> T32x64;
typedef Tile<128, 64, 16, 2, 2, 4> T128x64;   // sliced forward contractions (small images late in a network)
typedef Tile<64, 128, 16, 1, 4, 4> T64x128;   // sliced forward / backward-data contractions of small layers
// Half the K step: 20 KB of LDS, so a CU holds 4 blocks instead of 3.  For grids that need a second round of
// blocks at 3 per CU but fit in one at 4 (e.g. 64 output channels over 64 x 56 x 56 pixels: 784 tiles).
typedef Tile<64, 256, 8, 1, 4, 4> T64x256k8;
inline bool prefer_k8_64(long long cols) {
  const long long tiles = cdiv<long long>(cols, 256);
  return cdiv<long long>(tiles, 1024) < cdiv<long long>(tiles, 768);
}

// Second pass of a split contraction: out[i*ld + j] = alpha * sum_s part[s][i*cols + j] + beta*out.
// A bias gradient that rides in a reduction's launch, in blocks of its own behind the reduction's (small layers are
// bound by the number of dependent launches): db[k] = alpha * sum over n and the plane of src[(n K + k) plane + i] +
// beta * db[k]; plane == 1: src is an [N][K] matrix (an affine layer's delta, or per-image plane sums).
struct BiasJob {
  const float* src = nullptr;
  float* db = nullptr;           // nullptr: no job
  int N = 0, K = 0, plane = 0;
  float alpha = 1.0f, beta = 0.0f;
  unsigned first = 0;            // the job's first block (filled in by the launcher)
  unsigned blocks() const { return !db ? 0u : plane == 1 ? (unsigned)((K + 63) / 64) : (unsigned)K; }
};
void launch_split_reduce(const float* part, int splits, long long split_stride, float* out, int rows, int cols,
                         int ld, float alpha, float beta, hipStream_t stream, const float* bias_col = nullptr, int relu = 0,
                         const BiasJob* bias_job = nullptr);

// Tail form of a forward / backward-data launch (see EpiParams): when the tile count is not close to a multiple of
// the 256 CUs, the column tiles beyond the last multiple are cut into `splits` slices so that every CU ends up with
// nearly the same work, whether the CUs hold all tiles at once or take them in rounds.  splits == 1: not worth it.
struct TailSplit {
  int full_tiles, tail_tiles, splits;
  long long col0;  // first column of the tail
};
inline TailSplit plan_tail_split(int rows, long long cols, int n_k, int bn_force = 0) {
  TailSplit t = {0, 0, 1, 0};
  const int bm = pick_bm(rows), bn = bn_force ? bn_force : bm >= 96 ? 128 : 256;
  const int tiles_m = cdiv(rows, bm);
  const long long tiles_n = cdiv<long long>(cols, bn), T = tiles_m * tiles_n;
  const bool k8 = bm == 64 && tiles_m == 1 && prefer_k8_64(cols);  // the 64x256 tile with the halved K step: 4 per CU
  const long long slots = 256 * (bm >= 96 || k8 ? 4 : 3);
  if (T * 3 <= slots) return t;  // the whole-result split applies
  const long long full_cols = (T / 256 * 256) / tiles_m, full = full_cols * tiles_m, tail = T - full;
  if (tail == 0 || full == 0) return t;
  // Busiest CU in units of one tile's time: whole tiles + its pieces + the partial-sum traffic of those pieces
  // (a tile alone on a CU at ~0.47 TFLOP/s; a piece's slab written and read at a CU's share of ~4 TB/s).
  const double tile_us = 2.0 * bm * bn * (double)n_k / 0.47e6, piece_us = 8.0 * bm * bn / 15.6e3;
  const int k_chunks = n_k / 16;
  double best = (double)cdiv<long long>(T, 256);
  // modelled gain asked for: 7 % when all tiles are resident at once, 2.5 % when the CUs take tiles in several rounds
  // (measured: 1568 tiles 0.511 -> 0.454 ms, 2916 tiles 1.94 -> 1.87 ms, 3136 tiles 0.505 -> 0.478 ms)
  const double need = (T > slots ? 0.975 : 0.93) * best;
  for (int S = 2; S <= 16 && S * 8 <= k_chunks; ++S) {
    if (k_chunks % S != 0) continue;  // equal slices, for the 16- and the 8-deep K step alike
    const long long pieces = cdiv<long long>(tail * S, 256);
    const double cost = (double)cdiv<long long>(full, 256) + (double)pieces / S + pieces * piece_us / tile_us;
    if (cost < best && cost <= need) { best = cost; t.splits = S; }
  }
  if (t.splits > 1) { t.full_tiles = (int)full; t.tail_tiles = (int)tail; t.col0 = full_cols * bn; }
  return t;
}
// First element of the NCHW result that a tail column can touch: the start of the image that holds column col0.
// The partial slabs of the tail form hold the result from there on.
inline long long tail_first_elem(const TailSplit& t, long long inner, long long rows) {
  return t.splits > 1 && inner > 0 ? (t.col0 / inner) * rows * inner : 0;
}

// Scratch layout of the scalar-offset forward / backward-data paths:
//   [k -> byte offset table : n_k ints][transposed filter : n_k x rows floats][padded image copy]
struct SoffPlan {
  int n_k;         // contraction length rounded up to kTabPad
  int Hp, Wp;      // padded image extent
  int halo;        // zeros added on each side
  size_t tab_bytes, wt_bytes, img_bytes;  // img_bytes == 0: the image is used in place
  int splits;      // > 1: the contraction is cut into this many slices, partial results in part_bytes of scratch
  TailSplit tail;  // tail.splits > 1: only the last tiles are cut (splits == 1 then)
  bool narrow128 = false;  // forward, 128-row tiles: the 128 x 64 tile, planned as such
  size_t part_bytes;
  bool ok;         // false: fall back to the per-element gather path
  size_t total() const { return tab_bytes + wt_bytes + img_bytes + part_bytes; }
};

// A forward / backward-data launch whose tiles would occupy under half of the block slots the GPU holds at a time
// (small images late in a network, small batches) cuts the contraction into slices so that the slots fill; every
// slice keeps at least 16 K steps.  Partial results go to scratch slabs shaped like the output and are added in a
// fixed order by split_reduce_nchw.  Returns the slice count (1: no split).
// How many slices the depth of a contraction allows: every slice keeps `normal_min` K steps, so that prologue and
// partial-sum traffic stay small next to it.  Where even that many slices leave three quarters of the block slots
// empty (the layers of a small network at a small batch) a block's chain of K steps, each a memory round trip, is
// what the kernel takes, and the slices go down to `small_min` steps.
inline long long slices_by_depth(long long k_steps, long long tiles, long long slots, int normal_min, int small_min) {
  long long by = k_steps / normal_min;
  if (by < 1) by = 1;
  if (tiles * by * 4 <= slots) by = k_steps / small_min;
  return by < 1 ? 1 : by;
}

inline int plan_k_split(int rows, long long cols, int n_k, int bn_force = 0) {
  const int bm = pick_bm(rows), bn = bn_force ? bn_force : bm >= 96 ? 128 : 256;
  const long long slots = 256 * (bm >= 96 ? 4 : 3);
  const long long tiles = (long long)cdiv(rows, bm) * cdiv<long long>(cols, bn);
  if (tiles * 2 > slots) return 1;
  long long want = slots / tiles;
  const long long by_depth = slices_by_depth(n_k / 16, tiles, slots, 16, 4);
  if (want > by_depth) want = by_depth;
  if (want > 16) want = tiles * 64 <= slots ? (want > 32 ? 32 : want) : 16;
  return want < 3 ? 1 : (int)want;   // two slices only trade one round of blocks for the partial-sum traffic
}

// out[i] = alpha * sum_s part[s*stride + i] + beta*out[i] (+ bias[channel], ReLU) over an NCHW tensor of `total`
// elements, channel = (i / inner) % rows; only elements whose column (image * inner + pixel) is >= col0.
void launch_split_reduce_nchw(const float* part, int splits, long long stride, float* out, long long total, int inner,
                              int rows, float alpha, float beta, const float* bias, int relu, hipStream_t stream,
                              long long col0 = 0, const float* mask = nullptr);


inline SoffPlan plan_soff_fwd(const ConvDims& d) {
  SoffPlan p;
  p.n_k = round_up(d.C * d.R * d.S, kTabPad);
  p.halo = d.pad;
  p.Hp = d.H + 2 * d.pad;
  p.Wp = d.W + 2 * d.pad;
  p.tab_bytes = align256(sizeof(int) * (size_t)p.n_k);
  p.wt_bytes = align256(sizeof(float) * (size_t)p.n_k * d.K + kRow4Slack);
  const size_t img = sizeof(float) * (size_t)d.N * d.C * p.Hp * p.Wp;
  p.img_bytes = d.pad > 0 ? align256(img) : 0;
  p.ok = img <= kMaxBufferBytes && d.P > 0 && d.Q > 0;
  p.splits = plan_k_split(d.K, (long long)d.N * d.P * d.Q, p.n_k);
  p.tail = plan_tail_split(d.K, (long long)d.N * d.P * d.Q, p.n_k);
  if (pick_bm(d.K) == 128 && p.splits > 1) {
    // Few 128 x 128 tiles (small images late in a network): the half-width tile, planned as such.  Twice the tiles often
    // need no slices any more, only a cut of the tiles past the last multiple of 256 (NIN's 1024-channel layers on
    // 6 x 6: 576 tiles = 512 + 64 in eight slices, instead of 288 x 3 with a reduction over the whole result).
    p.narrow128 = true;
    p.splits = plan_k_split(d.K, (long long)d.N * d.P * d.Q, p.n_k, 64);
    p.tail = plan_tail_split(d.K, (long long)d.N * d.P * d.Q, p.n_k, 64);
  }
  const size_t tail_elems_f = (size_t)(d.y_elems - tail_first_elem(p.tail, (long long)d.P * d.Q, d.K));
  p.part_bytes = p.splits > 1 ? align256(sizeof(float) * (size_t)p.splits * (size_t)d.y_elems)
               : p.tail.splits > 1 ? align256(sizeof(float) * (size_t)p.tail.splits * tail_elems_f) : 0;
  return p;
}

// Winograd F(2x2, 3x3) form of a 3x3 stride-1 layer (conv_wino.hip), written as a forward convolution: an input of
// (N, Ci, Hi, Wi) with `halo` zeros around it, Ko filters, a result of (N, Ko, P, Q).  Backward-data is the same over dy
// with halo 2 - pad.  Scratch: [U: transformed filter][V: transformed image patches].
constexpr int kWinoBM = 128, kWinoBN = 32, kWinoR = 3;
struct WinoGeom {
  int N, Ci, Hi, Wi, Ko, halo, P, Q, TP, TQ;
  int Cg;                     // groups of four input channels
  int rows_p;                 // Ko rounded up to whole row tiles
  long long tiles, tiles_p;   // 2x2 output tiles; rounded up to whole column tiles
  size_t u_bytes, v_bytes;
  bool ok;
  // Tail form (V made in the kernel only): the blocks past the last multiple of 256 are cut into tail_S slices of the
  // channel loop, tail_L stages each, whose untransformed-blend partial results go to slabs of scratch that hold the
  // result from element part_first on (the first image a tail block touches); tail_S == 1: not worth it.
  int full_tiles, tail_S, tail_L;
  long long part_first, slab_elems;
  size_t part_bytes;
  // 5x5 forward (wino_geom_fwd5): the filter, extended with zeros to 6x6, is four 3x3 filters at offsets (3 bi, 3 bj);
  // the layer is the sum of their four 3x3 layers over shifted inputs, added in the transform domain: the same 16
  // products over 4 C "channels" (channel 4 c + 2 bi + bj = input channel c read 3 bi rows and 3 bj columns further
  // on): 64 multiply-adds per 2x2 outputs, filter and channel instead of 100.  Ci = 4 C here; the input is read from a
  // zero-bordered copy of Hp x Wp a plane (pad zeros in front, the rest behind), made in img_bytes of scratch.
  int blk5 = 0, C5 = 0, H5 = 0, W5 = 0, pad5 = 0;
  size_t img_bytes = 0;
  size_t total() const { return u_bytes + v_bytes + img_bytes + part_bytes; }
};
WinoGeom wino_geom(int N, int Ci, int Hi, int Wi, int Ko, int halo, int blk5 = 0);
inline bool wino_shape(const ConvDims& d) { return d.R == 3 && d.S == 3 && d.st == 1 && d.pad <= 2; }
inline bool wino_shape5(const ConvDims& d) { return d.R == 5 && d.S == 5 && d.st == 1 && d.pad <= 4 && d.P > 0 && d.Q > 0; }
inline WinoGeom wino_geom_fwd5(const ConvDims& d) { return wino_geom(d.N, d.C, d.H, d.W, d.K, d.pad, 1); }
inline WinoGeom wino_geom_fwd(const ConvDims& d) { return wino_geom(d.N, d.C, d.H, d.W, d.K, d.pad); }
inline WinoGeom wino_geom_bwd_data(const ConvDims& d) { return wino_geom(d.N, d.K, d.P, d.Q, d.C, 2 - d.pad); }
// Where the library takes it by itself: enough channels on both sides for the 16 products to be worth their
// transforms, and a grid that fills the GPU.
inline bool wino_pays(const WinoGeom& g) {
  // (rows: 128-row tiles at least three quarters full: 64 filters in one would execute as much as the direct form)
  return g.ok && g.Ci >= 64 && g.Ko >= 64 && 4 * g.Ko >= 3 * g.rows_p &&
         (long long)(g.rows_p / kWinoBM) * (g.tiles_p / kWinoBN) >= 192;
}
// The 5x5 forward form executes 64 % of the direct form's multiply-adds (a little more where the 2x2 tiles overhang
// the result) at a lower rate than the direct kernels reach, 18 % less time on 96 -> 256 channels, 27 x 27, batch 256:
// taken for full row tiles, a channel loop long next to a block's prologue and epilogue, and several rounds of blocks.
inline bool wino_pays5(const WinoGeom& g) {
  return g.ok && g.blk5 && g.C5 >= 64 && g.Ko >= 64 && 8 * g.Ko >= 7 * g.rows_p &&
         (long long)(g.rows_p / kWinoBM) * (g.tiles_p / kWinoBN) >= 512;
}
// Filter gradient in the same form: zero-bordered copies of x and dy, S slices of the tiles, their partial sums.
struct WinoFilterPlan {
  bool ok;
  int TP, TQ, Kp, Cp, S, stages;   // S slices of `stages` tile groups (of four tiles) each
  long long tiles, TGs;            // tiles; tile groups over all slices
  size_t vt_bytes, dyt_bytes, part_bytes;
  size_t total() const { return vt_bytes + dyt_bytes + part_bytes; }
};
WinoFilterPlan plan_wino_bwd_filter(const ConvDims& d);
// Where the library takes it by itself: as for the other two passes, and few enough slices for their traffic not to matter.
inline bool wino_filter_pays(const ConvDims& d, const WinoFilterPlan& p) {
  return p.ok && d.C >= 64 && d.K >= 64 && 4 * d.K >= 3 * p.Kp && 4 * d.C >= 3 * p.Cp && p.tiles >= 4096 &&
         (long long)(p.Kp / kWinoBM) * (p.Cp / kWinoBN) * p.S >= 192;
}
int launch_conv_wino_bwd_filter(const ConvDims& d, const WinoFilterPlan& p, const float* x, const float* dy, float* dw, float alpha,
                                float beta, void* ws, hipStream_t stream);
int launch_conv_wino(const WinoGeom& g, bool bwd, const float* in, const float* w, float* out, float alpha, float beta,
                     const float* bias, int relu, const float* mask, void* ws, hipStream_t stream, const char* tag);

// Forward with packed bf16 operands (RH_MATH_BF16_MFMA_FP32ACC, input channels a multiple of 8): the contraction runs
// over k = (r, s, c) with c fastest, the image is copied once to bf16 as [n][hp][c/8][wp][8] with its zero border,
// the filter to bf16 as [k/8][ko][8] (zero past C*R*S), so that eight consecutive k of one row are 16 contiguous
// bytes of either operand and neighbouring rows are neighbouring 16-byte pieces.
// Scratch: table of byte offsets per group of eight k | filter copy | image copy.
struct Bf16FwdPlan {
  int n_k, Hp, Wp;
  int s_groups;  // 0: groups of eight channels; > 0: groups of eight filter columns, this many per filter row
  size_t tab_bytes, wt_bytes, img_bytes;
  bool ok;
  size_t total() const { return tab_bytes + wt_bytes + img_bytes; }
};

// Channel counts that are not a multiple of 8 (first layers: 3 channels) with an even stride group the contraction
// by filter columns instead: k = (c, r, s) with s padded to a multiple of 8, the image copied to bf16 in its own
// NCHW order with its zero border (rows widened by the padding of s, to an even width), so that the eight s of a
// group are 16 contiguous bytes starting at an even element (4-byte aligned, as a vector load needs) and
// neighbouring pixels are `stride` elements apart.  An 11x11 filter pads to 16 columns (1.45x the contraction; with
// channels padded 3 -> 8 it would be 2.7x), a 7x7 to 8.
inline Bf16FwdPlan plan_bf16_fwd(const ConvDims& d) {
  Bf16FwdPlan p;
  p.Hp = d.H + 2 * d.pad;
  if (d.C % 8 == 0) {
    p.s_groups = 0;
    p.n_k = round_up(d.C * d.R * d.S, kTabPad);
    p.Wp = d.W + 2 * d.pad;
  } else {
    p.s_groups = cdiv(d.S, 8);
    p.n_k = round_up(d.C * d.R * p.s_groups * 8, kTabPad);
    p.Wp = round_up(d.W + 2 * d.pad + p.s_groups * 8 - d.S, 2);
  }
  p.tab_bytes = align256(sizeof(int) * (size_t)(p.n_k / 8));
  p.wt_bytes = align256(2 * (size_t)p.n_k * d.K);
  const size_t img = 2 * (size_t)d.N * d.C * p.Hp * p.Wp;
  p.img_bytes = align256(img);
  p.ok = (d.C % 8 == 0 || d.st % 2 == 0) && img <= kMaxBufferBytes && d.P > 0 && d.Q > 0 &&
         (long long)p.Hp * p.Wp < (1ll << 31) / 64;
  return p;
}

// Backward-data with stride 1: dx[n,c,h,w] = sum dyp[n,ko,h+R-1-r,w+S-1-s] * w[ko,c,r,s] on dy padded
// by R-1-pad zeros per side.
// Backward-data as a stride-1 correlation of the flipped filter with dy.  For stride > 1 the padded copy of dy is
// also dilated (dy[p][q] lands on [halo + st*p][halo + st*q], zeros between): the contraction then multiplies
// (st^2 - 1)/st^2 zeros, but runs on the scalar-offset loaders; the copy is (H + R - 1) x (W + S - 1) per plane.
inline SoffPlan plan_soff_bwd_data(const ConvDims& d) {
  SoffPlan p;
  p.n_k = round_up(d.K * d.R * d.S, kTabPad);
  p.halo = d.R - 1 - d.pad;
  p.Hp = d.H + d.R - 1;   // = P + 2*halo when the stride is 1
  p.Wp = d.W + d.S - 1;
  p.tab_bytes = align256(sizeof(int) * (size_t)p.n_k);
  p.wt_bytes = align256(sizeof(float) * (size_t)p.n_k * d.C);
  const size_t img = p.halo >= 0 ? sizeof(float) * (size_t)d.N * d.K * p.Hp * p.Wp : 0;
  p.img_bytes = (p.halo > 0 || d.st > 1 || p.Hp != d.P || p.Wp != d.Q) ? align256(img) : 0;
  p.ok = p.halo >= 0 && d.R == d.S && img <= kMaxBufferBytes && d.P > 0 && d.Q > 0;
  p.splits = plan_k_split(d.C, (long long)d.N * d.H * d.W, p.n_k);
  p.tail = plan_tail_split(d.C, (long long)d.N * d.H * d.W, p.n_k);
  if (pick_bm(d.C) == 128 && p.splits > 1 && plan_k_split(d.C, (long long)d.N * d.H * d.W, p.n_k, 64) == 1) {
    // As in the forward pass, where 128 x 64 tiles need no slices (NIN's 1024-channel 1x1 layers: 0.120 -> 0.098 ms).
    // Where they would still be sliced the 128 x 128 tile stays (a 384-channel 3x3 layer on 6 x 6 lost 9 %).
    p.narrow128 = true;
    p.splits = 1;
    p.tail = plan_tail_split(d.C, (long long)d.N * d.H * d.W, p.n_k, 64);
  }
  if (d.st > 1) p.tail.splits = 1;  // the zero-dilated form is a fallback only
  const size_t tail_elems_b = (size_t)(d.x_elems - tail_first_elem(p.tail, (long long)d.H * d.W, d.C));
  p.part_bytes = p.splits > 1 ? align256(sizeof(float) * (size_t)p.splits * (size_t)d.x_elems)
               : p.tail.splits > 1 ? align256(sizeof(float) * (size_t)p.tail.splits * tail_elems_b) : 0;
  return p;
}

// Backward-data with stride st > 1, decomposed by the residue (a, b) of (h + pad, w + pad) modulo st: an input pixel
// with h + pad = st*u + a only meets the filter rows r = a + st*i, and then through dy row p = u - i.  Each of the
// st*st classes is therefore a stride-1 correlation of dy with the sub-filter w[ko][c][a + st*i][b + st*j] over the
// sub-grid (u, v) of that class, with no wasted products.  Scratch: one padded copy of dy shared by all classes
// (halo L = ceil(R/st) - 1 on top / left, zeros below / right up to the largest u any class reaches), the transposed
// sub-filter and offset table of the class at hand, and the dense per-class results, which one pass interleaves into dx.
constexpr int kMaxPhaseStride = 4;
struct PhaseGeom {
  int Ra, Sb;          // filter rows / columns of the class (0: the class receives nothing)
  int u0, U, v0, V;    // first u, v of the class inside the image and how many
  long long sub_off;   // where the class's dense [n][c][U][V] result starts in the scratch, in floats
  int splits;          // slices of the class's contraction (plan_k_split)
};
struct PhasePlan {
  bool ok;
  int L, Hp, Wp, n_k;  // n_k: the largest padded contraction length among the classes
  size_t tab_bytes, wt_bytes, img_bytes, sub_bytes, part_bytes;
  PhaseGeom ph[kMaxPhaseStride * kMaxPhaseStride];
  size_t total() const { return tab_bytes + wt_bytes + img_bytes + sub_bytes + part_bytes; }
};

inline void phase_axis(int a, int st, int pad, int extent, int taps, int* n_taps, int* first, int* count) {
  *n_taps = a < taps ? (taps - a + st - 1) / st : 0;
  const int lo = pad > a ? (pad - a + st - 1) / st : 0;
  const int top = extent - 1 + pad - a;
  const int hi = top >= 0 ? top / st + 1 : 0;
  *first = lo;
  *count = hi > lo ? hi - lo : 0;
}

inline PhasePlan plan_phase_bwd_data(const ConvDims& d) {
  PhasePlan p;
  p.ok = false;
  p.L = p.Hp = p.Wp = p.n_k = 0;
  p.tab_bytes = p.wt_bytes = p.img_bytes = p.sub_bytes = p.part_bytes = 0;
  if (d.st < 2 || d.st > kMaxPhaseStride || d.P <= 0 || d.Q <= 0) return p;
  const int st = d.st;
  p.L = (d.R > d.S ? d.R : d.S);
  p.L = (p.L + st - 1) / st - 1;
  const int umax = (d.H - 1 + d.pad) / st + 1, vmax = (d.W - 1 + d.pad) / st + 1;
  p.Hp = p.L + (d.P > umax ? d.P : umax);
  p.Wp = p.L + (d.Q > vmax ? d.Q : vmax);
  long long off = 0;
  int max_taps = 0;
  for (int a = 0; a < st; ++a)
    for (int b = 0; b < st; ++b) {
      PhaseGeom& g = p.ph[a * st + b];
      phase_axis(a, st, d.pad, d.H, d.R, &g.Ra, &g.u0, &g.U);
      phase_axis(b, st, d.pad, d.W, d.S, &g.Sb, &g.v0, &g.V);
      g.sub_off = off;
      const long long elems = (long long)d.N * d.C * g.U * g.V;
      off += elems;
      if (g.Ra * g.Sb > max_taps) max_taps = g.Ra * g.Sb;
      g.splits = 1;
      if (g.Ra * g.Sb > 0 && elems > 0) {
        g.splits = plan_k_split(d.C, (long long)d.N * g.U * g.V, round_up(d.K * g.Ra * g.Sb, kTabPad));
        const size_t part = g.splits > 1 ? align256(sizeof(float) * (size_t)g.splits * (size_t)elems) : 0;
        if (part > p.part_bytes) p.part_bytes = part;
      }
    }
  p.n_k = round_up(d.K * (max_taps > 0 ? max_taps : 1), kTabPad);
  p.tab_bytes = align256(sizeof(int) * (size_t)p.n_k);
  p.wt_bytes = align256(sizeof(float) * (size_t)p.n_k * d.C);
  const size_t img = sizeof(float) * (size_t)d.N * d.K * p.Hp * p.Wp;
  p.img_bytes = (p.L > 0 || p.Hp != d.P || p.Wp != d.Q) ? align256(img) : 0;
  p.sub_bytes = align256(sizeof(float) * (size_t)off);
  p.ok = img <= kMaxBufferBytes && (size_t)off * 4 <= kMaxBufferBytes;
  return p;
}

// 1x1 / stride 1 / no padding layers with at most this many channels on both sides run on the register-resident
// streaming kernel (conv1x1.hip) in forward and backward-data.
constexpr int kConv1x1MaxChannels = 128;
bool conv1x1_stream_applies(const ConvDims& d);
int launch_conv1x1_stream(const ConvDims& d, int pass, const float* w, const float* src, float* out, float alpha, float beta,
                          const float* bias, int relu, hipStream_t stream, const float* mask = nullptr);

// The same for packed bf16 activations on both sides (conv1x1_bf16.hip): channels in multiples of 32, at most 128.
bool conv1x1_bf16_stream_applies(const ConvDims& d);   // the layers it is chosen for
bool conv1x1_bf16_stream_runs(const ConvDims& d);      // the layers it can run (RH_ALGO_SCALAR_OFFSET forces it on those)
int launch_conv1x1_bf16_stream(const ConvDims& d, const void* xp, const void* wb, const float* bias, int relu,
                               const PackedOut& pk, hipStream_t stream);

// dst[n][c][halo + dil*h][halo + dil*w] = src[n][c][h][w], zeros elsewhere; dst is planes x Hp x Wp.
void launch_pad_image(const float* src, float* dst, long long planes, int H, int W, int Hp, int Wp, int halo,
                      hipStream_t stream, int dil = 1);

// Filter-side scratch of the scalar-offset paths: wT[k][row] and the byte-offset table soff[k] into the padded copy
// (bwd = 0: forward, k = (c,r,s), rows = output channels; bwd = 1: stride-1 backward-data, k = (ko,r,s) with the
// filter flipped, rows = input channels), alone or in one launch with the padded copy of the image (no dilation).
void launch_prep_soff(const float* w, float* wT, int* soff, int n_k, int k_true, int rows, int R, int S, int HpWp, int Wp,
                      int bwd, hipStream_t stream);
void launch_pad_image_prep_soff(const float* src, float* dst, long long planes, int H, int W, int Hp, int Wp, int halo,
                                const float* w, float* wT, int* soff, int n_k, int k_true, int rows, int R, int S, int bwd,
                                hipStream_t stream);

void launch_build_fwd_tab(int4* tab, int n_entries, int CRS, int R, int S, int HW, int W,
                          hipStream_t stream);

}  // namespace rh
