// 1x1 convolution, stride 1, no padding, few channels on both sides (<= 128): forward and backward-data.
//
//   y[n][row][pix] = alpha * sum_k A(row, k) * src[n][k][pix] + beta * y (+ bias[row], ReLU)
//   forward:        A(ko, c) = w[ko][c],  src = x,  rows = K, contraction = C
//   backward-data:  A(c, ko) = w[ko][c],  src = dy, rows = C, contraction = K
//
// Such a layer (NIN's "cccp" layers after the first convolution: 96 -> 96 on 54 x 54) sits on the ridge between the
// matrix pipe and HBM: 2*96 FLOPs per 8 bytes moved.  The block-tiled engine spends most of a tile's life in its
// prologue and epilogue there (six K steps per tile) and reloads the 36 KB filter for each of its thousands of tiles.
// Here a block copies the filter into LDS once, already in the operand layout of v_mfma_f32_32x32x2_f32
// (a = A[lane % 32][lane / 32]: one conflict-free ds_read_b32 per MFMA), and then every wave streams 32-pixel column
// tiles on its own: the other operand of that instruction, b = B[lane / 32][lane % 32], is for a pixel-contiguous
// source exactly one coalesced dword load per (k pair): lanes 0-31 read 32 consecutive pixels of channel 2s, lanes
// 32-63 those of channel 2s + 1, straight into the operand register.  One barrier in the life of a block; a wave
// refills its operand registers for the next tile as the current tile's MFMAs free them, and the waves of an XCD
// sweep that XCD's eighth of the tensor in address order.
//
// Measured on the 96 -> 96, 54 x 54, batch 128 layer (286 MB, 6.9 GFLOP; 46 us at the 6.2 TB/s a copy reaches, 44 us
// at the matrix peak): 96 us.  With parts removed: MFMAs and filter reads alone 65 us (the matrix pipe at the
// clock it gets, three or four tiles per wave, prologue), loads and stores alone 77 us (dword accesses: what a
// one-float-per-thread copy reaches), loads alone 40, stores alone 38.
#include <type_traits>

#include "conv_common.h"

namespace rh {

struct Conv1x1Params {
  const float* A;       // filter
  int a_row_stride, a_k_stride;
  const float* src;     // [N][Cin][PQ]
  uint32_t src_bytes;
  int rows, kdim;       // result rows (channels), contraction length (= Cin)
  int PQ;
  long long cols;       // N * PQ
  int tiles;            // ceil(cols / 32)
};

template <int TM_>
struct StreamTile {
  static constexpr int TM = TM_, TN = 1, BM = 32 * TM_, BN = 32;
};

// FAST: alpha == 1, beta == 0, rows == 32 * TM and the contraction == 2 * KH, so the loads need no channel guard
// and a column tile that lies inside one image is stored without per-element checks.
// Registers: 16 TM accumulators + KH operands + about seventy (the general epilogue of the non-FAST form needs more
// and runs two blocks per CU): as many blocks per CU (four waves each, one per SIMD) as fit 512 registers per lane,
// two to four; the filter's LDS copy (256 TM KH bytes) fits as often.
template <int TM, int KH, bool FAST>
constexpr int stream_blocks_per_cu() {
  const int regs = 16 * TM + KH + 72 + (TM == 4 ? 8 : 0);
  return !FAST || 512 / regs < 2 ? 2 : (512 / regs > 4 ? 4 : 512 / regs);
}

// The filter, once per block: sa[(s * TM + i) * 64 + lane] = A(32 i + lane % 32, 2 s + lane / 32), zero outside.
// Every thread first issues all its loads (KH TM / 4 of them, out-of-range ones read zero) and then writes LDS, so
// a block waits for memory once.  Which element a thread takes follows the filter's layout in memory: with the
// contraction index contiguous (forward) a wave reads eight rows by eight consecutive k (32-byte pieces; its LDS
// writes meet eight to a bank), with the row index contiguous (backward-data) a wave reads LDS order directly.
template <int TM, int KH>
__device__ __forceinline__ void stage_filter(const Conv1x1Params& p, float* __restrict__ sa) {
  constexpr int PER = KH * TM / 4;
  const __amdgpu_buffer_rsrc_t rflt = make_rsrc(p.A, (uint32_t)(sizeof(float) * (size_t)p.rows * p.kdim));
  const bool k_major = p.a_k_stride == 1;
  float tmp[PER];
  int pos[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = (int)threadIdx.x + 256 * j;
    int row, k;
    if (k_major) {
      const int rest = e >> 6, k_hi = rest % (KH / 4), r_hi = rest / (KH / 4);
      k = 8 * k_hi + (e & 7);
      row = 8 * r_hi + ((e >> 3) & 7);
      pos[j] = ((k >> 1) * TM + (row >> 5)) * 64 + (k & 1) * 32 + (row & 31);
    } else {
      const int l = e & 63, si = e >> 6;
      row = 32 * (si % TM) + (l & 31);
      k = 2 * (si / TM) + (l >> 5);
      pos[j] = e;
    }
    const uint32_t off = (row < p.rows && k < p.kdim) ? 4u * (uint32_t)(row * p.a_row_stride + k * p.a_k_stride) : 0x80000000u;
    tmp[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rflt, (int)off, 0, 0));
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) sa[pos[j]] = tmp[j];
}

// MASK: ep.mask (a tensor shaped like the result) zeroes the result where it is not > 0 (backward-data that applies
// the backward of the ReLU before this layer as it writes; sixteen more loads per row tile and column tile).
template <int TM, int KH, bool FAST, class PASS, bool MASK = false>
__global__ __launch_bounds__(256, (stream_blocks_per_cu<TM, KH, FAST && !MASK>())) void conv1x1_stream_kernel(Conv1x1Params p, EpiParams ep, FastDiv dPQ) {
  const int lane = threadIdx.x & 63;
  // Blocks go to the eight XCDs in turn (block b to XCD b % 8), each with an L2 of its own.  An XCD takes a
  // contiguous eighth of the column tiles and its waves sweep that eighth in address order, so the two halves of a
  // cache line that neighbouring tiles share (planes are not line-aligned) meet in one L2: read from memory once,
  // and written back as a whole line.  Grids that are no multiple of eight blocks sweep the whole range together.
  const bool by_xcd = (gridDim.x & 7) == 0;
  const int nwaves = by_xcd ? (int)(gridDim.x >> 3) * 4 : (int)gridDim.x * 4;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((by_xcd ? blockIdx.x >> 3 : blockIdx.x) * 4 + (threadIdx.x >> 6)));
  const int span = by_xcd ? (p.tiles + 7) >> 3 : p.tiles;            // column tiles per XCD
  const int first = by_xcd ? (int)(blockIdx.x & 7) * span : 0;
  const int last = min(first + span, p.tiles);                      // (one past) this XCD's range
  const int half = lane >> 5, l32 = lane & 31;

  extern __shared__ float sa[];
  stage_filter<TM, KH>(p, sa);
  __syncthreads();
  const float* const sal = sa + lane;

  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.src, p.src_bytes);
  const __amdgpu_buffer_rsrc_t rdst = make_rsrc(ep.out, (uint32_t)(sizeof(float) * (size_t)p.cols * p.rows));
  const __amdgpu_buffer_rsrc_t rmask = make_rsrc(MASK ? ep.mask : ep.out, (uint32_t)(sizeof(float) * (size_t)p.cols * p.rows));
  const int PQ4 = p.PQ * 4;
  const uint32_t img_bytes = (uint32_t)p.kdim * (uint32_t)PQ4;
  const uint32_t out_img_bytes = (uint32_t)p.rows * (uint32_t)PQ4;

  // Loads of one column tile: b[s] = src[img][2 s + half][pix]; lanes past the last column (and, unless FAST, channel
  // pairs past the contraction) read zero: offset 0x80000000 is out of range of the buffer.  The address advances in
  // a register from one channel pair to the next.  tile_addr gives a lane's first address and the step between
  // channel pairs (both "nowhere" for a tile past the range), load_part issues the loads of pairs [s0, s1).
  auto tile_addr = [&](int tile, uint32_t& v, uint32_t& step) __attribute__((always_inline)) {
    const long long col64 = (long long)tile * 32 + l32;   // tile may be up to nwaves past the range's last one
    v = 0x80000000u;
    step = 0u;
    if (tile < last && col64 < p.cols) {
      uint32_t img, pix;
      dPQ.divmod((uint32_t)col64, img, pix);
      v = img * img_bytes + pix * 4u + (uint32_t)(half * PQ4);
      step = (uint32_t)(2 * PQ4);
    }
  };
  auto load_part = [&](float (&b)[KH], uint32_t& v, uint32_t step, int s0, int s1) __attribute__((always_inline)) {
#pragma unroll
    for (int s = s0; s < s1; ++s) {
      const uint32_t vv = (FAST || 2 * s + half < p.kdim) ? v : 0x80000000u;
      b[s] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)vv, 0, 0));
      v += step;
    }
  };
  // One column tile: the MFMAs over the operand registers b, which are refilled for the tile `next` as they fall
  // free (first half of the channel pairs in the middle of the contraction, second half at its end), then the
  // epilogue and the stores.  A wave therefore holds one tile's operands, not two, four blocks fit a CU, and the waits
  // of one wave (for its loads, and for the write acknowledgements that the shared memory counter makes it sit out
  // too) are covered by the matrix work of the three others on its SIMD.
  auto compute_tile = [&](float (&b)[KH], int tile, int next) __attribute__((always_inline)) {
    uint32_t nv, nstep;
    tile_addr(next, nv, nstep);
    f32x16 acc[TM][1];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][0][v] = 0.0f;
    // where this tile goes, if it lies inside one image (then it is stored without per-element checks)
    const uint32_t col0 = (uint32_t)tile * 32u;
    uint32_t img0, pix0;
    dPQ.divmod(col0, img0, pix0);
    const bool inside = (long long)col0 + 31 < p.cols && pix0 + 31u < (uint32_t)p.PQ;   // uniform over the wave
    const uint32_t out_o = img0 * out_img_bytes + (pix0 + (uint32_t)l32) * 4u + (uint32_t)(4 * half * PQ4);
    float mreg[MASK ? TM : 1][16];
    const uint32_t mask_o = inside ? out_o : 0x80000000u, mask_step = inside ? (uint32_t)PQ4 : 0u;
    (void)mreg; (void)mask_o; (void)mask_step;
    // (opaque pointer: the filter reads must stay in the loop, one per MFMA, not be hoisted into KH * TM registers)
    // An LDS-space pointer: through a generic one these become flat loads, whose waits also cover the global loads.
    typedef const __attribute__((address_space(3))) float* lds_ptr;
    lds_ptr sl = (lds_ptr)sal;
    asm volatile("" : "+v"(sl));
    // pinned order per channel pair: [filter reads of the next pair] [MFMAs of this pair]; left alone the scheduler
    // issues every read of the tile first and spills
    float av[2][TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) av[0][i] = sl[i * 64];
#pragma unroll
    for (int s = 0; s < KH; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < KH) {
#pragma unroll
        for (int i = 0; i < TM; ++i) av[(s + 1) & 1][i] = sl[((s + 1) * TM + i) * 64];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s & 1][i], b[s], acc[i][0], 0, 0, 0);
      if (s == KH / 2 - 1) {
        __builtin_amdgcn_sched_barrier(0);
        load_part(b, nv, nstep, 0, KH / 2);
        if (FAST && MASK) {
          // this tile's mask values, in flight during the second half of the contraction (nothing for a tile that is
          // stored element by element: every offset out of range)
          uint32_t om = mask_o;
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                mreg[i][4 * q + e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rmask, (int)om, 0, 0));
                om += mask_step;
              }
              om += 4u * mask_step;
            }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    load_part(b, nv, nstep, KH / 2, KH);
    __builtin_amdgcn_sched_barrier(0);
    if (FAST) {
      if (ep.bias) {
        // added after the sum, as the separate bias pass of the reference does (same rounding).  Rows
        // 32 i + 8 (v / 4) + 4 half + v % 4: four consecutive rows per 16-byte load; the pointer is made opaque so
        // that these (cached) loads stay here instead of occupying 16 * TM registers for the life of the wave.
        typedef const __attribute__((address_space(1))) float* global_ptr;   // (a generic pointer would mean flat loads)
        global_ptr bias = (global_ptr)ep.bias;
        asm volatile("" : "+s"(bias));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            global_ptr bq = bias + 32 * i + 8 * q + 4 * half;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][0][4 * q + e] += bq[e];
          }
      }
      if (inside) {
        if (ep.relu) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][0][v] = acc[i][0][v] > 0.0f ? acc[i][0][v] : 0.0f;
        }
        uint32_t o = out_o;
        if (MASK) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][0][v] = mreg[i][v] > 0.0f ? acc[i][0][v] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float val = acc[i][0][4 * q + e];   // (bit-casting the vector element directly stored element 4q)
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), rdst, (int)o, 0, 0);
              o += (uint32_t)PQ4;
            }
            o += (uint32_t)(4 * PQ4);
          }
        return;
      }
      // A tile that straddles two images or ends ragged (one in PQ / 32): element by element.  The bias is already
      // added.  Everything here derives from an opaque copy of PQ so that none of it is computed (and kept
      // in registers) outside this branch.
      int inner = p.PQ;
      asm volatile("" : "+s"(inner));
      const long long col = (long long)col0 + l32;
      if (col < p.cols) {
        const int img = (int)(col / inner), pix = (int)(col - (long long)img * inner);
        float* dst = ep.out + ((size_t)img * p.rows + 4 * half) * inner + pix;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float val = acc[i][0][v];
            if (ep.relu) val = val > 0.0f ? val : 0.0f;
            const size_t at = (size_t)(32 * i + 8 * (v >> 2) + (v & 3)) * inner;
            if (MASK && !(ep.mask[(dst - ep.out) + at] > 0.0f)) val = 0.0f;
            dst[at] = val;
          }
      }
      return;
    }
    store_tile<StreamTile<TM>, true>(acc, ep, 0, tile * 32, 0, 0, lane, -1);
  };

  // The refill is unconditional (a tile past the end reads nothing: every lane's offset is out of range), so the
  // loop body is straight-line code.
  float b0[KH];
  int t = first + wave;
  if (t >= last) return;
  {
    uint32_t v, step;
    tile_addr(t, v, step);
    load_part(b0, v, step, 0, KH);
  }
  for (; t < last; t += nwaves) compute_tile(b0, t, t + nwaves);
}


// The same kernel for column counts per image that are a multiple of W (2 or 4), alpha == 1, beta == 0, full row tiles
// and a contraction of exactly 2 KH: a wave takes 32 W columns at a time and lane l holds the W consecutive pixels
// W l .. W l + W - 1 of each, so that every access to the source and to the result is W dwords wide (dword accesses top
// out near 3.8 TB/s on this GPU, 16-byte ones reach 6).  The W pixels of a lane are the same column of W different
// MFMA tiles (tile j = pixels W l + j over the 32 lanes: which 32 pixels make up a tile is free), and since both the
// count of columns and of pixels per image are multiples of W, a lane's pixels lie in one image and are either all
// inside the tensor or all outside: every lane computes its own image and pixel once per 32 W columns, no case
// distinction for a group of columns that straddles two images.  One filter read from LDS serves W MFMAs.
// The second half of the next group's operands is requested after the stores of this one, so that their registers are
// free for the mask values of the epilogue in between.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int W>
__device__ __forceinline__ void load_w(float (&d)[W], __amdgpu_buffer_rsrc_t r, uint32_t off) {
  if constexpr (W == 4) {
    const u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = __uint_as_float(q[j]);
  } else {
    const u32x2 q = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
    d[0] = __uint_as_float(q[0]); d[1] = __uint_as_float(q[1]);
  }
}
template <int W>
__device__ __forceinline__ void store_w(const float (&d)[W], __amdgpu_buffer_rsrc_t r, uint32_t off) {
  if constexpr (W == 4) {
    u32x4 q;
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = __float_as_uint(d[j]);
    __builtin_amdgcn_raw_buffer_store_b128(q, r, (int)off, 0, 0);
  } else {
    u32x2 q;
    q[0] = __float_as_uint(d[0]); q[1] = __float_as_uint(d[1]);
    __builtin_amdgcn_raw_buffer_store_b64(q, r, (int)off, 0, 0);
  }
}

template <int TM, int KH, int W>
constexpr int wide_blocks_per_cu() {
  return (16 * TM * W + KH * W + 64) <= 256 ? 2 : 1;
}

template <int TM, int KH, int W, class PASS, bool MASK>
__global__ __launch_bounds__(256, (wide_blocks_per_cu<TM, KH, W>())) void conv1x1_stream_wide_kernel(Conv1x1Params p, EpiParams ep, FastDiv dPQ) {
  const int lane = threadIdx.x & 63;
  const bool by_xcd = (gridDim.x & 7) == 0;   // (see conv1x1_stream_kernel: an XCD sweeps its eighth in address order)
  const int nwaves = by_xcd ? (int)(gridDim.x >> 3) * 4 : (int)gridDim.x * 4;
  const int wave = __builtin_amdgcn_readfirstlane(
      (int)((by_xcd ? blockIdx.x >> 3 : blockIdx.x) * 4 + (threadIdx.x >> 6)));
  const int span = by_xcd ? (p.tiles + 7) >> 3 : p.tiles;            // groups of 32 W columns per XCD
  const int first = by_xcd ? (int)(blockIdx.x & 7) * span : 0;
  const int last = min(first + span, p.tiles);
  const int half = lane >> 5, l32 = lane & 31;

  extern __shared__ float sa[];
  stage_filter<TM, KH>(p, sa);
  __syncthreads();
  const float* const sal = sa + lane;

  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.src, p.src_bytes);
  const __amdgpu_buffer_rsrc_t rdst = make_rsrc(ep.out, (uint32_t)(sizeof(float) * (size_t)p.cols * p.rows));
  const __amdgpu_buffer_rsrc_t rmask = make_rsrc(MASK ? ep.mask : ep.out, (uint32_t)(sizeof(float) * (size_t)p.cols * p.rows));
  const int PQ4 = p.PQ * 4;
  const uint32_t img_bytes = (uint32_t)p.kdim * (uint32_t)PQ4;
  const uint32_t out_img_bytes = (uint32_t)p.rows * (uint32_t)PQ4;

  // A lane's place in group g: image and pixel of its first column (W l32 columns into the group); "nowhere" (offset
  // 0x80000000: loads return 0, stores are dropped) past this XCD's range or the tensor's last column.
  auto place = [&](int g, uint32_t& img, uint32_t& pix) __attribute__((always_inline)) -> bool {
    const long long col64 = (long long)g * (32 * W) + W * l32;
    if (g >= last || col64 >= p.cols) return false;
    dPQ.divmod((uint32_t)col64, img, pix);
    return true;
  };
  auto src_addr = [&](int g, uint32_t& v, uint32_t& step) __attribute__((always_inline)) {
    uint32_t img, pix;
    v = 0x80000000u;
    step = 0u;
    if (place(g, img, pix)) {
      v = img * img_bytes + pix * 4u + (uint32_t)(half * PQ4);
      step = (uint32_t)(2 * PQ4);
    }
  };
  auto load_part = [&](float (&b)[KH][W], uint32_t& v, uint32_t step, int s0, int s1) __attribute__((always_inline)) {
#pragma unroll
    for (int s = s0; s < s1; ++s) {
      load_w<W>(b[s], rsrc, v);
      v += step;
    }
  };

  auto compute_group = [&](float (&b)[KH][W], int g, int next, uint32_t& nv, uint32_t& nstep) __attribute__((always_inline)) {
    // (nv, nstep): where the second half of this group's successor starts, left by the first-half request below
    f32x16 acc[TM][W];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    uint32_t out_o = 0x80000000u;
    {
      uint32_t img, pix;
      if (place(g, img, pix)) out_o = img * out_img_bytes + pix * 4u + (uint32_t)(4 * half * PQ4);
    }
    typedef const __attribute__((address_space(3))) float* lds_ptr;
    lds_ptr sl = (lds_ptr)sal;
    asm volatile("" : "+v"(sl));   // (the filter reads stay in the loop, one per row tile and channel pair)
    float av[2][TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) av[0][i] = sl[i * 64];
#pragma unroll
    for (int s = 0; s < KH; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < KH) {
#pragma unroll
        for (int i = 0; i < TM; ++i) av[(s + 1) & 1][i] = sl[((s + 1) * TM + i) * 64];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < W; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s & 1][i], b[s][j], acc[i][j], 0, 0, 0);
      if (s == KH / 2 - 1) {
        __builtin_amdgcn_sched_barrier(0);
        src_addr(next, nv, nstep);
        load_part(b, nv, nstep, 0, KH / 2);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (ep.bias) {
      // rows 32 i + 8 q + 4 half + e: added after the sum, as the separate bias pass of the reference does
      typedef const __attribute__((address_space(1))) float* global_ptr;
      global_ptr bias = (global_ptr)ep.bias;
      asm volatile("" : "+s"(bias));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          global_ptr bq = bias + 32 * i + 8 * q + 4 * half;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float bv = bq[e];
#pragma unroll
            for (int j = 0; j < W; ++j) acc[i][j][4 * q + e] += bv;
          }
        }
    }
    if (ep.relu) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < W; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] = acc[i][j][v] > 0.0f ? acc[i][j][v] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float m[MASK ? 16 : 1][W];
      (void)m;
      if (MASK) {   // one row tile's mask values at a time: sixteen loads in flight, then its stores
        uint32_t om = out_o + (uint32_t)(32 * i) * (uint32_t)PQ4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            load_w<W>(m[4 * q + e], rmask, om);
            om += (uint32_t)PQ4;
          }
          om += (uint32_t)(4 * PQ4);
        }
      }
      uint32_t o = out_o + (uint32_t)(32 * i) * (uint32_t)PQ4;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float val[W];
#pragma unroll
          for (int j = 0; j < W; ++j) {
            val[j] = acc[i][j][4 * q + e];
            if (MASK) val[j] = m[4 * q + e][j] > 0.0f ? val[j] : 0.0f;
          }
          store_w<W>(val, rdst, o);
          o += (uint32_t)PQ4;
        }
        o += (uint32_t)(4 * PQ4);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    load_part(b, nv, nstep, KH / 2, KH);
  };

  float b0[KH][W];
  int g = first + wave;
  if (g >= last) return;
  {
    uint32_t v, step;
    src_addr(g, v, step);
    load_part(b0, v, step, 0, KH);
  }
  uint32_t nv = 0x80000000u, nstep = 0u;
  for (; g < last; g += nwaves) compute_group(b0, g, g + nwaves, nv, nstep);
}

// ------------------------------------------------------------------------------------------------------------------
// The same layer with every global access 16 bytes wide, no wave ever waiting for a store, the epilogue of one tile
// issued in the shadow of the next tile's MFMAs, and two tiles of loads in flight per wave: the image's way through
// LDS, the filter in registers.  (Dword accesses top out near 3.8 TB/s on this GPU whatever is done around them; a wave
// that waits for loads behind its own fresh stores sits out their acknowledgements, since the memory counter retires
// in order; an epilogue that a wave runs between two tiles costs it 1.8 us per tile, a fifth of the tile's matrix
// time; and with one tile of loads in flight per wave, 48 KB per CU, the memory system delivers 3.5 TB/s.)
// One block of four waves per CU, one per SIMD, each wave on column tiles of its own with private LDS: three source
// buffers of 32 pixels by the contraction and a 4 KB result buffer (160 KB per CU for a contraction of 96).
//   * The filter is staged through LDS once (before the buffers are in use) into registers: a lane holds its
//     A(32 i + lane % 32, 2 s + lane / 32) for every row tile i and channel pair s, TM * KH values.
//   * A tile of the source arrives by direct global -> LDS loads (buffer_load_dwordx4 ... lds: eight channel rows of
//     32 pixels per instruction, no registers), requested two tiles ahead: loads(j+2) go out at the top of tile j,
//     into the buffer tile j-1 was multiplied from.
//   * The MFMAs read the image operand from LDS, one conflict-free ds_read_b32 per channel pair.
//   * Two sets of accumulators: while tile j is multiplied into one, the other (tile j-1) is drained, one element per
//     K step (bias, ReLU, into the result buffer as Y[row][32 pixels]); after each row tile of 32 rows the buffer is read
//     back as eight rows of 128 bytes per instruction and stored with 16 bytes per lane.
// Memory instructions of a wave in program order: loads(j+2), then the stores of tile j-1 spread over tile j; the wait
// for loads(j) at the top of tile j allows the two younger tiles' loads and the two younger tiles' stores to be in flight.
// Column tiles are cut per image (the last one of an image is ragged), so a tile never straddles two images.  No
// block-wide barrier once the filter is in registers.
// ------------------------------------------------------------------------------------------------------------------
template <int TM, int KH>
constexpr size_t lds_kernel_bytes() {
  const size_t bufs = sizeof(float) * 4 * (3 * 32 * (size_t)(2 * KH) + 1024);
  const size_t stage = sizeof(float) * ((size_t)TM * KH * 64 + 32 * TM);
  return bufs > stage ? bufs : stage;
}
template <int TM, int KH>
constexpr bool lds_kernel_fits() {
  return KH % 4 == 0 && KH >= 16 * TM && TM * KH <= 160 && lds_kernel_bytes<TM, KH>() <= 160 * 1024;
}

template <int TM, int KH, bool RELU, class PASS>
__global__ __launch_bounds__(256, 1) void conv1x1_lds_kernel(Conv1x1Params p, EpiParams ep, FastDiv dTpi) {
  constexpr int KD = 2 * KH, ROWS = 32 * TM;
  constexpr int XBUF = 32 * KD;               // floats per source buffer
  constexpr int LD = KD / 8, ST = ROWS / 8;   // load / store instructions per tile
  static_assert(KH >= 16 * TM, "one K step per drained accumulator element");
  static_assert(2 * LD + 2 * ST <= 63, "the memory counter counts to 63");
  const int lane = threadIdx.x & 63;
  const int wib = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const bool by_xcd = (gridDim.x & 7) == 0;   // (see conv1x1_stream_kernel: an XCD sweeps its eighth in address order)
  const int nwaves = by_xcd ? (int)(gridDim.x >> 3) * 4 : (int)gridDim.x * 4;
  const int wave = __builtin_amdgcn_readfirstlane((int)((by_xcd ? blockIdx.x >> 3 : blockIdx.x) * 4) + wib);
  const int span = by_xcd ? (p.tiles + 7) >> 3 : p.tiles;
  const int first = by_xcd ? (int)(blockIdx.x & 7) * span : 0;
  const int last = min(first + span, p.tiles);
  const int half = lane >> 5, l32 = lane & 31;

  extern __shared__ float sa[];
  // filter and bias: through LDS into registers, in accumulator / operand order, for the life of the wave
  float areg[KH][TM], breg[16 * TM];
  {
    float* const sbias = sa + TM * KH * 64;
    stage_filter<TM, KH>(p, sa);
    if (threadIdx.x < ROWS) sbias[threadIdx.x] = ep.bias ? ep.bias[threadIdx.x] : 0.0f;
    __syncthreads();
#pragma unroll
    for (int s = 0; s < KH; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i) areg[s][i] = sa[(s * TM + i) * 64 + lane];
#pragma unroll
    for (int u = 0; u < 16 * TM; ++u) breg[u] = sbias[32 * (u >> 4) + 8 * ((u & 15) >> 2) + 4 * half + (u & 3)];
    __syncthreads();   // the staging area becomes the waves' buffers
  }
  float* const xbuf = sa + wib * (3 * XBUF + 1024);   // this wave's three source buffers ...
  float* const ybuf = xbuf + 3 * XBUF;                // ... and its result buffer (32 rows x 32 pixels)

  const int PQ4 = p.PQ * 4;
  const uint32_t img_bytes = (uint32_t)p.kdim * (uint32_t)PQ4;
  const uint32_t out_img_bytes = (uint32_t)p.rows * (uint32_t)PQ4;
  u32x4 rsrc;
  {
    const uint64_t a = reinterpret_cast<uint64_t>(p.src);
    rsrc.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
    rsrc.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    rsrc.z = __builtin_amdgcn_readfirstlane(p.src_bytes);
    rsrc.w = 0x00020000u;
  }
  const __amdgpu_buffer_rsrc_t rdst = make_rsrc(ep.out, (uint32_t)(sizeof(float) * (size_t)p.cols * p.rows));
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)xbuf;
  const int row8 = lane >> 3, px4 = (lane & 7) * 4;   // this lane's place in a 16-byte access: row within eight, first pixel

  // tile -> image and first pixel (wave-uniform)
  auto where = [&](int t, uint32_t& img, uint32_t& pix0) __attribute__((always_inline)) {
    uint32_t ti;
    dTpi.divmod((uint32_t)t, img, ti);
    pix0 = ti * 32u;
  };
  auto issue_loads = [&](int t, int buf) __attribute__((always_inline)) {
    uint32_t img, pix0;
    where(t, img, pix0);
    const uint32_t px = pix0 + (uint32_t)px4;
    const uint32_t voff = px < (uint32_t)p.PQ ? img * img_bytes + (uint32_t)(row8 * PQ4) + px * 4u : 0x80000000u;
    const uint32_t dst = lds0 + (uint32_t)(buf * XBUF * 4);
#pragma unroll
    for (int g = 0; g < LD; ++g) dma_load16(rsrc, dst + (uint32_t)(g * 1024), voff, (uint32_t)(g * 8 * PQ4));
  };
  // the memory counter may stand at `loads` tiles of loads plus `stores` tiles of stores (each 0, 1 or 2)
  auto wait_for_tile = [&](int loads, int stores) __attribute__((always_inline)) {
    switch (loads * 3 + stores) {
      case 0: wait_vmcnt<0>(); break;
      case 1: wait_vmcnt<ST>(); break;
      case 2: wait_vmcnt<2 * ST>(); break;
      case 3: wait_vmcnt<LD>(); break;
      case 4: wait_vmcnt<LD + ST>(); break;
      case 5: wait_vmcnt<LD + 2 * ST>(); break;
      case 6: wait_vmcnt<2 * LD>(); break;
      case 7: wait_vmcnt<2 * LD + ST>(); break;
      default: wait_vmcnt<2 * LD + 2 * ST>(); break;
    }
  };
  typedef const __attribute__((address_space(3))) float* lds_ptr;

  // Where a drained tile's rows go (per lane: the 16-byte access of row 8 r + row8) and the stores of one row tile.
  struct Dest { uint32_t o0, ow; int nvalid; };
  auto dest_of = [&](int t) __attribute__((always_inline)) -> Dest {
    uint32_t img, pix0;
    where(t, img, pix0);
    const uint32_t px = pix0 + (uint32_t)px4;
    Dest d;
    d.o0 = img * out_img_bytes + (uint32_t)(row8 * PQ4) + px * 4u;
    d.ow = px + 3u < (uint32_t)p.PQ ? d.o0 : 0x80000000u;   // lanes whose four pixels lie inside the image
    d.nvalid = px < (uint32_t)p.PQ && px + 3u >= (uint32_t)p.PQ ? p.PQ - (int)px : 0;   // the image's ragged end
    return d;
  };
  // Row tile i of a drained tile is complete in the result buffer (32 rows x 128 bytes): read_rows fetches it, four
  // instructions of eight rows, and store_rows, a K step later, stores it the same way.
  auto read_rows = [&](float4 (&yv)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 4; ++r) yv[r] = *reinterpret_cast<const float4*>(ybuf + (8 * r + row8) * 32 + px4);
  };
  auto store_rows = [&](const Dest& d, const float4 (&yv)[4], int i) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4 q;
      q[0] = __float_as_uint(yv[r].x); q[1] = __float_as_uint(yv[r].y); q[2] = __float_as_uint(yv[r].z); q[3] = __float_as_uint(yv[r].w);
      __builtin_amdgcn_raw_buffer_store_b128(q, rdst, (int)d.ow, (4 * i + r) * 8 * PQ4, 0);
    }
    if (d.nvalid) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float vals[4] = {yv[r].x, yv[r].y, yv[r].z, yv[r].w};
#pragma unroll
        for (int e = 0; e < 3; ++e)
          if (e < d.nvalid)
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(vals[e]), rdst, (int)(d.o0 + 4u * e), (4 * i + r) * 8 * PQ4, 0);
      }
    }
  };
  // element u (0 .. 16 TM - 1) of a drained accumulator set: row 32 i + 8 q + 4 half + e of this lane's pixel
  auto drain_one = [&](const f32x16 (&acc)[TM], int u) __attribute__((always_inline)) {
    const int i = u >> 4, v = u & 15;
    float val = acc[i][v] + breg[u];   // added after the sum, as the reference's bias pass
    if (RELU) val = val > 0.0f ? val : 0.0f;
    ybuf[(8 * (v >> 2) + 4 * half + (v & 3)) * 32 + l32] = val;
  };
  auto drain_all = [&](const f32x16 (&acc)[TM], const Dest& d) __attribute__((always_inline)) {
    float4 yv[4];
#pragma unroll
    for (int u = 0; u < 16 * TM; ++u) {
      drain_one(acc, u);
      if ((u & 15) == 15) { read_rows(yv); store_rows(d, yv, u >> 4); }
    }
  };

  // One tile: the contraction from source buffer `cur` into `acc`; with DRAIN, the tile before (accumulators `old`,
  // destination `od`) leaves through the result buffer meanwhile, one element per K step.
  auto tile = [&](f32x16 (&acc)[TM], const f32x16 (&old)[TM], const Dest& od, int cur, auto drain_tag, int next_t, int next_buf) __attribute__((always_inline)) {
    constexpr bool DRAIN = decltype(drain_tag)::value;
    // the loads of the tile after next, one instruction per K step (next_t < 0: none)
    uint32_t nvoff = 0x80000000u, ndst = 0;
    if (next_t >= 0) {
      uint32_t img, pix0;
      where(next_t, img, pix0);
      const uint32_t px = pix0 + (uint32_t)px4;
      nvoff = px < (uint32_t)p.PQ ? img * img_bytes + (uint32_t)(row8 * PQ4) + px * 4u : 0x80000000u;
      ndst = lds0 + (uint32_t)(next_buf * XBUF * 4);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
    lds_ptr bl = (lds_ptr)(xbuf + cur * XBUF + half * 32 + l32);
    asm volatile("" : "+v"(bl));
    float bv[2];
    float4 yv[4];
    bv[0] = bl[0];
#pragma unroll
    for (int s = 0; s < KH; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if (DRAIN) {
        // the row tile read back in the step before leaves (its reads were issued ahead of that step's operand read,
        // which this step's MFMAs waited for)
        if (s > 0 && (s & 15) == 0 && s <= 16 * TM) store_rows(od, yv, (s >> 4) - 1);
      }
      if (s + 1 < KH) bv[(s + 1) & 1] = bl[(s + 1) * 64];
      if (s < LD && next_t >= 0) dma_load16(rsrc, ndst + (uint32_t)(s * 1024), nvoff, (uint32_t)(s * 8 * PQ4));
      if (DRAIN) {
        if (s < 16 * TM) drain_one(old, s);
        if (s < 16 * TM && (s & 15) == 15) read_rows(yv);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s][i], bv[s & 1], acc[i], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (DRAIN && KH == 16 * TM) store_rows(od, yv, TM - 1);
  };

  int t = first + wave;
  if (t >= last) return;
  // tile j of this wave: t + j * nwaves, in source buffer j % 3; loads two tiles ahead
  const int n = (last - t + nwaves - 1) / nwaves;
  f32x16 accA[TM], accB[TM];
  Dest dA, dB = {0x80000000u, 0x80000000u, 0};
  issue_loads(t, 0);
  if (n > 1) issue_loads(t + nwaves, 1);
  int cur = 0;
  for (int j = 0; j < n; j += 2) {
    // even tile into A while B (tile j-1) drains
    {
      wait_for_tile((j + 1 < n), j >= 3 ? 2 : j >= 2 ? 1 : 0);
      dA = dest_of(t + j * nwaves);
      const int nt = j + 2 < n ? t + (j + 2) * nwaves : -1, nb = cur == 0 ? 2 : cur - 1;
      if (j == 0) tile(accA, accB, dB, cur, std::false_type(), nt, nb);
      else        tile(accA, accB, dB, cur, std::true_type(), nt, nb);
      cur = cur == 2 ? 0 : cur + 1;
    }
    if (j + 1 >= n) {   // the even tile was the last one
      drain_all(accA, dA);
      return;
    }
    // odd tile into B while A drains
    {
      const int k = j + 1;
      wait_for_tile((k + 1 < n), k >= 3 ? 2 : k >= 2 ? 1 : 0);
      dB = dest_of(t + k * nwaves);
      tile(accB, accA, dA, cur, std::true_type(), k + 2 < n ? t + (k + 2) * nwaves : -1, cur == 0 ? 2 : cur - 1);
      cur = cur == 2 ? 0 : cur + 1;
    }
  }
  drain_all(accB, dB);
}

template <int TM, int KH, class PASS>
static int launch_lds_kernel(Conv1x1Params p, const EpiParams& ep, hipStream_t stream) {
  constexpr size_t lds = lds_kernel_bytes<TM, KH>();
  static const hipError_t a1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_lds_kernel<TM, KH, true, PASS>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  static const hipError_t a2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_lds_kernel<TM, KH, false, PASS>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (a1 != hipSuccess) return (int)a1;
  if (a2 != hipSuccess) return (int)a2;
  const int tpi = cdiv(p.PQ, 32);
  p.tiles = (int)(p.cols / p.PQ) * tpi;   // per-image tiles
  if (ep.relu)
    hipLaunchKernelGGL((conv1x1_lds_kernel<TM, KH, true, PASS>), dim3(256u), dim3(256), lds, stream, p, ep, FastDiv((uint32_t)tpi));
  else
    hipLaunchKernelGGL((conv1x1_lds_kernel<TM, KH, false, PASS>), dim3(256u), dim3(256), lds, stream, p, ep, FastDiv((uint32_t)tpi));
  return launch_status();
}

template <int TM, int KH, int W>
constexpr bool wide_fits() { return TM * W <= 12 && 16 * TM * W + KH * W + 80 <= 512; }

template <int TM, int KH, int W, class PASS, bool MASK>
static int launch_stream_wide_one(Conv1x1Params p, const EpiParams& ep, const FastDiv& dPQ, size_t lds, hipStream_t stream) {
  if (lds > 48 * 1024) {
    static const hipError_t a = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_stream_wide_kernel<TM, KH, W, PASS, MASK>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (a != hipSuccess) return (int)a;
  }
  p.tiles = (int)cdiv<long long>(p.cols, 32 * W);   // groups of 32 W columns
  const int full = 256 * wide_blocks_per_cu<TM, KH, W>();
  const int blocks = p.tiles >= 4 * full ? full : (p.tiles >= 256 ? 8 * cdiv(cdiv(p.tiles, 8), 4) : cdiv(p.tiles, 4));
  hipLaunchKernelGGL((conv1x1_stream_wide_kernel<TM, KH, W, PASS, MASK>), dim3((unsigned)blocks), dim3(256), lds, stream, p, ep, dPQ);
  return launch_status();
}

template <int TM, int KH, int W, class PASS>
static int launch_stream_wide(const Conv1x1Params& p, const EpiParams& ep, const FastDiv& dPQ, size_t lds, hipStream_t stream) {
  if constexpr (std::is_same<PASS, PassConvBwdData>::value && W == 2) {   // (the masked form exists for two pixels per lane)
    if (ep.mask) return launch_stream_wide_one<TM, KH, W, PASS, true>(p, ep, dPQ, lds, stream);
  }
  return launch_stream_wide_one<TM, KH, W, PASS, false>(p, ep, dPQ, lds, stream);
}

template <int TM, int KH, class PASS>
static int launch_stream(const Conv1x1Params& p, const EpiParams& ep, hipStream_t stream) {
  const FastDiv dPQ((uint32_t)p.PQ);
  constexpr size_t lds = sizeof(float) * KH * TM * 64;
  if (lds > 48 * 1024) {
    static const hipError_t a1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_stream_kernel<TM, KH, true, PASS>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    static const hipError_t a2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_stream_kernel<TM, KH, false, PASS>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (a1 != hipSuccess) return (int)a1;
    if (a2 != hipSuccess) return (int)a2;
  }
  const bool fast = ep.alpha == 1.0f && ep.beta == 0.0f && p.rows == 32 * TM && p.kdim == 2 * KH &&
                    (!ep.bias || (reinterpret_cast<uintptr_t>(ep.bias) & 15) == 0);
  // Long contractions (96 channels and more) with a pixel count per image that allows it take the form that moves
  // two or four pixels per lane (measured on 96 -> 96, 54 x 54, batch 128: forward 97 -> 92 us with two, backward-data
  // 97 -> 88 with four, backward-data with the mask 132 -> 117 with two; on 128 -> 128, 28 x 28 the masked form
  // 86 -> 31).  Short ones lose there (32 -> 64 on 56 x 56: 27 -> 29-32 us: less matrix work per group of columns to
  // cover the epilogue of a wave that has its SIMD to itself or shares it with one other).
  // Large layers without a mask: the image through LDS with 16-byte accesses on both sides (conv1x1_lds_kernel).
  // Measured with the library's events on 96 -> 96 at batch 128: forward with bias and ReLU 101 -> 94 us on 54 x 54,
  // 115 -> 104 us on 55 x 55 (no even pixel count: the register form falls back to dword accesses there); backward-data
  // 97 -> 94 and 107 -> 103; 64 -> 64 on 56 x 56 at batch 256 forward 101 -> 91, backward-data 87 -> 90, which therefore
  // stays with four pixels per lane where the pixel count is a multiple of four.
  if constexpr (lds_kernel_fits<TM, KH>()) {
    constexpr bool bwd = std::is_same<PASS, PassConvBwdData>::value;
    if (fast && !ep.mask && p.cols / p.PQ * (long long)cdiv(p.PQ, 32) >= 4096 && !(bwd && KH < 48 && p.PQ % 4 == 0))
      return launch_lds_kernel<TM, KH, PASS>(p, ep, stream);
  }
  if constexpr (KH >= 48) {
    if (fast && p.PQ % 2 == 0) {
      constexpr bool bwd = std::is_same<PASS, PassConvBwdData>::value;
      if constexpr (bwd && wide_fits<TM, KH, 4>()) {
        if (!ep.mask && p.PQ % 4 == 0) return launch_stream_wide<TM, KH, 4, PASS>(p, ep, dPQ, lds, stream);
      }
      return launch_stream_wide<TM, KH, 2, PASS>(p, ep, dPQ, lds, stream);
    }
  }
  // every block slot of the GPU; smaller problems: a wave per tile, in whole blocks per XCD when there are enough tiles
  const int full = 256 * (fast && !ep.mask ? stream_blocks_per_cu<TM, KH, true>() : stream_blocks_per_cu<TM, KH, false>());
  const int blocks = p.tiles >= 4 * full ? full : (p.tiles >= 256 ? 8 * cdiv(cdiv(p.tiles, 8), 4) : cdiv(p.tiles, 4));
  if constexpr (std::is_same<PASS, PassConvBwdData>::value) {
    if (ep.mask) {   // (the forward pass has no masked form)
      if (lds > 48 * 1024) {
        static const hipError_t a3 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_stream_kernel<TM, KH, true, PASS, true>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        static const hipError_t a4 = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_stream_kernel<TM, KH, false, PASS, true>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (a3 != hipSuccess) return (int)a3;
        if (a4 != hipSuccess) return (int)a4;
      }
      if (fast)
        hipLaunchKernelGGL((conv1x1_stream_kernel<TM, KH, true, PASS, true>), dim3((unsigned)blocks), dim3(256), lds, stream, p, ep, dPQ);
      else
        hipLaunchKernelGGL((conv1x1_stream_kernel<TM, KH, false, PASS, true>), dim3((unsigned)blocks), dim3(256), lds, stream, p, ep, dPQ);
      return launch_status();
    }
  }
  if (fast)
    hipLaunchKernelGGL((conv1x1_stream_kernel<TM, KH, true, PASS>), dim3((unsigned)blocks), dim3(256), lds, stream, p, ep, dPQ);
  else
    hipLaunchKernelGGL((conv1x1_stream_kernel<TM, KH, false, PASS>), dim3((unsigned)blocks), dim3(256), lds, stream, p, ep, dPQ);
  return launch_status();
}

template <int TM, class PASS>
static int pick_kh(const Conv1x1Params& p, const EpiParams& ep, hipStream_t stream) {
  const int kh = cdiv(p.kdim, 2);
  if (kh <= 16) return launch_stream<TM, 16, PASS>(p, ep, stream);
  if (kh <= 32) return launch_stream<TM, 32, PASS>(p, ep, stream);
  if (kh <= 48) return launch_stream<TM, 48, PASS>(p, ep, stream);
  return launch_stream<TM, 64, PASS>(p, ep, stream);
}

// The kernels above address both tensors with 32-bit byte offsets in which 0x80000000 means "nowhere": every byte
// of a tensor must lie below that.
static_assert(kMaxBufferBytes <= (size_t(1) << 31), "conv1x1 offsets: 0x80000000 must stay out of range");

bool conv1x1_stream_applies(const ConvDims& d) {
  if (4 * (size_t)d.N * d.P * d.Q * (size_t)(d.C > d.K ? d.C : d.K) > (size_t(1) << 31)) return false;
  return d.R == 1 && d.S == 1 && d.st == 1 && d.pad == 0 && d.C <= kConv1x1MaxChannels && d.K <= kConv1x1MaxChannels &&
         (long long)d.N * d.P * d.Q < (1ll << 31) - 64;
}

// pass: RH_CONV_FWD (src = x, out = y) or RH_CONV_BWD_DATA (src = dy, out = dx).
int launch_conv1x1_stream(const ConvDims& d, int pass, const float* w, const float* src, float* out, float alpha, float beta,
                          const float* bias, int relu, hipStream_t stream, const float* mask) {
  const bool fwd = pass == RH_CONV_FWD;
  Conv1x1Params p;
  p.A = w;
  p.a_row_stride = fwd ? d.C : 1;
  p.a_k_stride = fwd ? 1 : d.C;
  p.src = src;
  p.rows = fwd ? d.K : d.C;
  p.kdim = fwd ? d.C : d.K;
  p.PQ = d.P * d.Q;
  p.cols = (long long)d.N * p.PQ;
  p.src_bytes = (uint32_t)(sizeof(float) * (size_t)p.cols * p.kdim);
  p.tiles = (int)cdiv<long long>(p.cols, 32);
  EpiParams ep;
  ep.out = out; ep.bias = bias; ep.alpha = alpha; ep.beta = beta;
  ep.rows = p.rows; ep.cols = (int)p.cols; ep.inner = p.PQ; ep.ld = 0; ep.relu = relu; ep.split_stride = 0;
  ep.mask = fwd ? nullptr : mask;
  ProfScope prof(fwd ? "conv_fwd_1x1_stream" : "conv_bwd_data_1x1_stream", 2.0 * (double)p.rows * (double)p.cols * (double)p.kdim,
                 stream);
  const int tm = cdiv(p.rows, 32);
  if (fwd) {
    switch (tm) {
      case 1: return pick_kh<1, PassConvFwd>(p, ep, stream);
      case 2: return pick_kh<2, PassConvFwd>(p, ep, stream);
      case 3: return pick_kh<3, PassConvFwd>(p, ep, stream);
      default: return pick_kh<4, PassConvFwd>(p, ep, stream);
    }
  }
  switch (tm) {
    case 1: return pick_kh<1, PassConvBwdData>(p, ep, stream);
    case 2: return pick_kh<2, PassConvBwdData>(p, ep, stream);
    case 3: return pick_kh<3, PassConvBwdData>(p, ep, stream);
    default: return pick_kh<4, PassConvBwdData>(p, ep, stream);
  }
}

}  // namespace rh
