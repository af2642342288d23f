// 3x3 stride-1 convolutions by Winograd's minimal filtering F(2x2, 3x3): forward, backward-data (the forward form of the
// flipped, transposed filter over dy) and the filter gradient (CudnnConvFwdOp / CudnnConvBwdDataOp / CudnnConvBwdFilterOp
// of a 3x3 layer, src/operator/mod.rs:1684-1696, 1765-1793).
//
//   Y = A^T [ (G g G^T) o (B^T d B) ] A      per 2x2 output tile, 4x4 input patch d, 3x3 filter g
//
// 16 multiplications per tile, filter and channel instead of 36: the contraction over the input channels becomes 16
// independent products  M_f (rows x tiles) = U_f (rows x channels) * V_f (channels x tiles),  f = 4i + j the position
// in the 4x4 transformed patch, 2.25 times fewer multiply-adds than the direct form.
//
// Forward / backward-data:
//  * wino_prep_kernel: U = G g G^T for every (row, channel) in the operand order of the product kernel, zero rows and
//    channels up to whole blocks (and V = B^T d B for channel counts that are no multiple of four, see below);
//  * wino_gemm_fused_kernel: a block of four waves owns 128 rows x 32 tiles for all 16 f; wave w holds rows 32w .. 32w+31
//    as 16 accumulator tiles of v_mfma_f32_32x32x2_f32 (256 accumulation registers, one wave per SIMD).  U goes straight
//    from memory to LDS (buffer_load_dwordx4 ... lds) into a ring of three stages of four channels each, two stages
//    ahead of the MFMAs; V is made in the kernel from the image's patches; the one barrier of a stage stands in front
//    of its last quarter of MFMAs.  (wino_gemm_kernel: the same with V read from memory, for other channel counts.)
//  * the epilogue: a lane's element e of the 16 accumulators is the whole 4x4 M of one (row, tile): A^T M A is 24
//    additions in registers, then alpha / beta, bias, ReLU or the mask of a folded ReLU backward, and the 2x2 pixels
//    go to the NCHW result (odd extents: the tile's pixels past the edge are dropped).
//  * blocks past the last whole round of the 256 CUs take slices of the channel loop and wino_tail_reduce_kernel adds
//    their partial results (wino_geom); not where the caller says that other kernels run beside the call.
//  * the forward pass of a 5x5 stride-1 layer is the same kernel over four times the channels: the filter's zero
//    extension to 6x6 is four 3x3 filters, the layer the sum of their four 3x3 layers over the input read 3 rows / 3
//    columns further on, and that sum is taken in the transform domain like the one over the channels
//    (wino_geom_fwd5, WinoImage::blk5): 64 multiply-adds per 2x2 outputs, filter and channel instead of 100.
// Filter gradient: wino_filter_prep_kernel, wino_bwd_filter_kernel, wino_filter_reduce_kernel, described further down.
//
// Operand layout (floats):  U[f][cg][h][rows_p][2],  V[f][cg][h][tiles_p][2]  with channel = 4 cg + 2 h + j.  The MFMA
// takes A[row][k], B[k][col] with k = lane / 32: the half-wave h reads channel 4 cg + 2 h + j for the stage's MFMA j,
// one 8-byte LDS read per operand and stage and f, each half-wave reading 256 consecutive bytes.
//
// A wave's own VALU instructions are not hidden behind its MFMAs (each one between two MFMAs adds its 4-7 cycles;
// LDS, scalar and memory instructions there cost nothing), and these kernels run one wave per SIMD: the loops keep
// vector arithmetic to the transforms themselves.
#include "conv_common.h"

namespace rh {

WinoGeom wino_geom(int N, int Ci, int Hi, int Wi, int Ko, int halo, int blk5) {
  WinoGeom g;
  g.N = N; g.Ci = Ci; g.Hi = Hi; g.Wi = Wi; g.Ko = Ko; g.halo = halo;
  g.P = Hi + 2 * halo - 2; g.Q = Wi + 2 * halo - 2;
  if (blk5) {
    // the 5x5 layer as four 3x3 layers over a zero-bordered copy: the kernel sees an image of Hp x Wp without halo and
    // 4 C channels; patch rows 2 ty + 3 bi .. + 3 of the copy reach row 2 TP + 4
    g.blk5 = 1; g.C5 = Ci; g.H5 = Hi; g.W5 = Wi; g.pad5 = halo;
    g.P = Hi + 2 * halo - 4; g.Q = Wi + 2 * halo - 4;
    g.Hi = 2 * cdiv(g.P > 0 ? g.P : 1, 2) + 5; g.Wi = 2 * cdiv(g.Q > 0 ? g.Q : 1, 2) + 5;
    g.halo = 0; g.Ci = 4 * Ci;
    Ci = g.Ci; Hi = g.Hi; Wi = g.Wi; halo = 0;
    g.img_bytes = align256(sizeof(float) * (size_t)N * g.C5 * g.Hi * g.Wi);
  }
  g.TP = g.P > 0 ? cdiv(g.P, 2) : 0; g.TQ = g.Q > 0 ? cdiv(g.Q, 2) : 0;
  g.tiles = (long long)N * g.TP * g.TQ;
  g.tiles_p = (g.tiles + kWinoBN - 1) / kWinoBN * kWinoBN;
  g.Cg = cdiv(Ci, 4);
  g.rows_p = round_up(Ko, kWinoBM);
  const unsigned long long ub = 16ull * g.Cg * 2 * (unsigned long long)g.rows_p * 8;
  const unsigned long long vb = 16ull * g.Cg * 2 * (unsigned long long)g.tiles_p * 8;
  g.u_bytes = align256((size_t)ub);
  g.v_bytes = Ci % 4 == 0 ? 0 : align256((size_t)vb);   // (channel counts in whole groups of four: V is made in the kernel)
  // 32-bit byte offsets into U and V, 31-bit tile indices
  g.ok = g.P > 0 && g.Q > 0 && halo >= 0 && halo <= 2 && ub < (1ull << 31) && (Ci % 4 == 0 || vb < (1ull << 31)) &&
         g.tiles_p < (1ll << 30) && (long long)N * Ko * g.P * g.Q < (1ll << 30) && (long long)N * Ci * Hi * Wi < (1ll << 30);
  if (blk5) g.ok = g.ok && g.pad5 <= 4 && g.Hi >= g.H5 + g.pad5 && g.Wi >= g.W5 + g.pad5;
  // One block per CU at a time: 784 blocks are four rounds of the 256 CUs with the last one 6 % full.  The blocks past
  // the last whole round are cut into slices of the channel loop (every slice a whole number of stages, four at
  // least), so that the last round is as short as its share of the work; their partial results are added by
  // wino_tail_reduce_kernel.  A block costs about eight stages' time before and after its loop (measured: 1176 blocks
  // of 64 stages gain nothing from five slices of 13), and the slabs and that kernel 3 % of a round.
  g.full_tiles = 0; g.tail_S = 1; g.tail_L = g.Cg; g.part_first = 0; g.slab_elems = 0; g.part_bytes = 0;
  const long long tiles_m = g.rows_p / kWinoBM, T = tiles_m * (g.tiles_p / kWinoBN);
  const long long full = T / 256 * 256, tail = T - full;
  if (g.ok && Ci % 4 == 0 && full > 0 && tail > 0) {
    double best = (double)cdiv<long long>(T, 256) * 0.97;
    for (int S = 2; S <= 16; ++S) {
      const int L = cdiv(g.Cg, S);
      if (L < 4 || cdiv(g.Cg, L) != S) continue;
      const double cost = (double)(full / 256) + (double)cdiv<long long>(tail * S, 256) * (L + 8.0) / (g.Cg + 8.0) + 0.03;
      if (cost < best) { best = cost; g.tail_S = S; g.tail_L = L; }
    }
    if (g.tail_S > 1) {
      g.full_tiles = (int)full;
      const long long first_tile = (full / tiles_m) * kWinoBN;   // first image tile of the first column tile with a tail block
      const long long n0 = first_tile / ((long long)g.TP * g.TQ);
      g.part_first = n0 * g.Ko * g.P * g.Q;
      g.slab_elems = (long long)N * g.Ko * g.P * g.Q - g.part_first;
      g.part_bytes = align256(sizeof(float) * (size_t)g.slab_elems * g.tail_S);
    }
  }
  return g;
}

namespace {

struct WinoPrepArgs {
  const float* w; const float* x; float* U; float* V;
  int Ko, Ci, Cg, rows_p, bwd;
  int blk5, C5;       // the 5x5 form: "channel" v = 4 c + 2 bi + bj is the 3x3 block at (3 bi, 3 bj) of input channel c's filter
  int Hi, Wi, halo;
  unsigned tiles, tiles_p, x_bytes;
  FastDiv dRows, dPairs, dTQ, dTP;
  unsigned filt_items, in_items, in_blocks;
};

// U of rows (row, channels 2 ch, 2 ch + 1): G g G^T with G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]
__device__ __forceinline__ void wino_filter_item(const WinoPrepArgs& a, unsigned idx) {
  uint32_t ch, row;
  a.dRows.divmod(idx, ch, row);
  float u[16][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int c = (int)ch * 2 + j;
    float g[3][3];
    const bool live = (int)row < a.Ko && c < a.Ci;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        // forward: w[row][c][r][s]; backward-data: rows are the input channels of w, the contraction runs over its
        // filters, taps flipped: w[c][row][2-r][2-s]
        if (a.blk5) {
          const int rr = 3 * ((c >> 1) & 1) + r, ss = 3 * (c & 1) + s;   // the 5x5 filter with a sixth row and column of zeros
          g[r][s] = live && rr < 5 && ss < 5 ? a.w[((size_t)row * a.C5 + (c >> 2)) * 25 + (size_t)(rr * 5 + ss)] : 0.0f;
          continue;
        }
        const size_t at = a.bwd ? ((size_t)c * a.Ko + row) * 9 + (size_t)((2 - r) * 3 + (2 - s))
                                : ((size_t)row * a.Ci + c) * 9 + (size_t)(r * 3 + s);
        g[r][s] = live ? a.w[at] : 0.0f;
      }
    float t[4][3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      t[0][s] = g[0][s];
      t[1][s] = 0.5f * (g[0][s] + g[1][s] + g[2][s]);
      t[2][s] = 0.5f * (g[0][s] - g[1][s] + g[2][s]);
      t[3][s] = g[2][s];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u[4 * i + 0][j] = t[i][0];
      u[4 * i + 1][j] = 0.5f * (t[i][0] + t[i][1] + t[i][2]);
      u[4 * i + 2][j] = 0.5f * (t[i][0] - t[i][1] + t[i][2]);
      u[4 * i + 3][j] = t[i][2];
    }
  }
  float2* U2 = reinterpret_cast<float2*>(a.U);
  const size_t plane = (size_t)a.Cg * 2 * a.rows_p;
#pragma unroll
  for (int f = 0; f < 16; ++f) U2[f * plane + (size_t)ch * a.rows_p + row] = make_float2(u[f][0], u[f][1]);
}

// V of (channels 2 ch, 2 ch + 1) x (tiles 2 u, 2 u + 1): B^T d B with B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]
__device__ __forceinline__ void wino_input_item(const WinoPrepArgs& a, unsigned idx) {
  uint32_t ch, up;
  a.dPairs.divmod(idx, ch, up);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, a.x_bytes);
  float v[16][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const unsigned t = 2 * up + tt;
    uint32_t q1, tx, n, ty;
    a.dTQ.divmod(t, q1, tx);
    a.dTP.divmod(q1, n, ty);
    const int h0 = 2 * (int)ty - a.halo, w0 = 2 * (int)tx - a.halo;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = (int)ch * 2 + j;
      const bool live = t < a.tiles && c < a.Ci;
      const unsigned base = (n * (unsigned)a.Ci + (unsigned)c) * (unsigned)(a.Hi * a.Wi);
      float d[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int hh = h0 + i, ww = w0 + k;
          const bool in = live && (unsigned)hh < (unsigned)a.Hi && (unsigned)ww < (unsigned)a.Wi;
          const unsigned off = in ? (base + (unsigned)(hh * a.Wi + ww)) * 4u : kInvalidByteOff;
          d[i][k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (int)off, 0, 0));
        }
      float s[4][4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        s[0][k] = d[0][k] - d[2][k];
        s[1][k] = d[1][k] + d[2][k];
        s[2][k] = d[2][k] - d[1][k];
        s[3][k] = d[1][k] - d[3][k];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[4 * i + 0][2 * tt + j] = s[i][0] - s[i][2];
        v[4 * i + 1][2 * tt + j] = s[i][1] + s[i][2];
        v[4 * i + 2][2 * tt + j] = s[i][2] - s[i][1];
        v[4 * i + 3][2 * tt + j] = s[i][1] - s[i][3];
      }
    }
  }
  float4* V4 = reinterpret_cast<float4*>(a.V);
  const size_t pairs = a.tiles_p / 2, plane = (size_t)a.Cg * 2 * pairs;
#pragma unroll
  for (int f = 0; f < 16; ++f) V4[f * plane + (size_t)ch * pairs + up] = make_float4(v[f][0], v[f][1], v[f][2], v[f][3]);
}

__global__ __launch_bounds__(256) void wino_prep_kernel(WinoPrepArgs a) {
  if (blockIdx.x < a.in_blocks) {
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    if (idx < a.in_items) wino_input_item(a, idx);
  } else {
    const unsigned idx = (blockIdx.x - a.in_blocks) * 256u + threadIdx.x;
    if (idx < a.filt_items) wino_filter_item(a, idx);
  }
}

struct WinoEpi {
  float* out; const float* bias; const float* mask;
  float alpha, beta;
  int relu, Ko, P, Q;
  unsigned tiles, out_bytes;
  FastDiv dTQ, dTP;
};

// A^T M A per (row, tile) with A^T = [1 1 1 0; 0 1 -1 -1], then the blend, bias, ReLU / mask, and the 2x2 pixels out.
// acc[f] holds M_f of rows m0 + 32 wave .. + 31 x tiles n0 .. n0 + 31 in the MFMA's accumulator layout.
// (Accumulators live in the accumulation registers, which ordinary arithmetic cannot read; left alone the compiler
// copies all 256 to ordinary registers behind the loop and the kernel's allocation becomes all 512 registers of a SIMD
// lane: nothing else can run on a CU beside it.  wino_pin_acc says "these are still in accumulation registers here"
// in front of every block of the epilogue, so that a block's 64 values are fetched when its turn comes and the
// allocation stays near 360: a bandwidth-bound kernel of another stream finds room on the same CUs.)
__device__ __forceinline__ void wino_pin_acc(f32x16 (&acc)[16]) {
#pragma unroll
  for (int f = 0; f < 16; ++f) asm volatile("" : "+a"(acc[f]));
}

// One accumulator element, fetched where it is used (written as the instruction itself: as an ordinary element access
// the compiler moves whole 16-register tuples out of the accumulation registers ahead of time).
__device__ __forceinline__ float wino_acc_elem(const f32x16& v, int e) {
  float r;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(v[e]));
  return r;
}

__device__ __forceinline__ void wino_epilogue(f32x16 (&acc)[16], const WinoEpi& ep, int m0, unsigned n0, int wave, int lane) {
  const int h = lane >> 5, r = lane & 31;
  const unsigned t = n0 + (unsigned)r;
  uint32_t q1, tx, n, ty;
  ep.dTQ.divmod(t, q1, tx);
  ep.dTP.divmod(q1, n, ty);
  const int PQ = ep.P * ep.Q;
  const int row_lane = m0 + wave * 32 + 4 * h;     // + 8 (e / 4) + e % 4
  const int rows_left = ep.Ko - row_lane;
  uint32_t voff[2][2];
#pragma unroll
  for (int ai = 0; ai < 2; ++ai)
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
      const bool ok = t < ep.tiles && 2 * (int)ty + ai < ep.P && 2 * (int)tx + bi < ep.Q;
      voff[ai][bi] = ok ? ((n * (unsigned)ep.Ko + 4u * (unsigned)h) * (unsigned)PQ + (2u * ty + ai) * (unsigned)ep.Q + 2u * tx + bi) * 4u
                        : kInvalidByteOff;
    }
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(ep.out, ep.out_bytes);
  const __amdgpu_buffer_rsrc_t rmask = make_rsrc(ep.mask ? ep.mask : ep.out, ep.out_bytes);
  const __amdgpu_buffer_rsrc_t rbias = make_rsrc(ep.bias ? ep.bias : ep.out, ep.bias ? 4u * (unsigned)ep.Ko : 0u);
  float bv[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int re = 8 * (e >> 2) + (e & 3);
    bv[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rbias, (row_lane + re) * 4, 0, 0));
  }
  const int srow = (m0 + wave * 32) * PQ * 4;   // wave-uniform byte offset of the wave's first row
  const bool blend = ep.beta != 0.0f, masked = ep.mask != nullptr;
  constexpr int EB = 4;   // accumulator elements per block (loads of a block stand ahead of its stores)
#pragma unroll
  for (int eb = 0; eb < 16 / EB; ++eb) {
    __builtin_amdgcn_sched_barrier(0);
    wino_pin_acc(acc);
    float y[EB][2][2];
    uint32_t vo[EB][2][2];
    float aux[EB][2][2];   // mask values, or the old result
#pragma unroll
    for (int e4 = 0; e4 < EB; ++e4) {
      const int e = EB * eb + e4, re = 8 * (e >> 2) + (e & 3);
      float s0[4], s1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float m0j = wino_acc_elem(acc[j], e), m1j = wino_acc_elem(acc[4 + j], e), m2j = wino_acc_elem(acc[8 + j], e),
                    m3j = wino_acc_elem(acc[12 + j], e);
        s0[j] = m0j + m1j + m2j;
        s1[j] = m1j - m2j - m3j;
      }
      y[e4][0][0] = s0[0] + s0[1] + s0[2];
      y[e4][0][1] = s0[1] - s0[2] - s0[3];
      y[e4][1][0] = s1[0] + s1[1] + s1[2];
      y[e4][1][1] = s1[1] - s1[2] - s1[3];
      const bool row_ok = re < rows_left;
#pragma unroll
      for (int ai = 0; ai < 2; ++ai)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          vo[e4][ai][bi] = row_ok ? voff[ai][bi] : kInvalidByteOff;
          y[e4][ai][bi] *= ep.alpha;
        }
    }
    if (masked || blend) {
      // (both at once: the mask first, then the old values, block by block; neither occurs in a train step's forward pass)
#pragma unroll
      for (int e4 = 0; e4 < EB; ++e4)
#pragma unroll
        for (int ai = 0; ai < 2; ++ai)
#pragma unroll
          for (int bi = 0; bi < 2; ++bi)
            aux[e4][ai][bi] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(blend ? rout : rmask, (int)vo[e4][ai][bi], srow + (8 * ((EB * eb + e4) >> 2) + ((EB * eb + e4) & 3)) * PQ * 4, 0));
    }
#pragma unroll
    for (int e4 = 0; e4 < EB; ++e4)
#pragma unroll
      for (int ai = 0; ai < 2; ++ai)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          float x = y[e4][ai][bi];
          if (blend) x = fmaf(ep.beta, aux[e4][ai][bi], x);
          x += bv[EB * eb + e4];
          if (ep.relu) x = fmaxf(x, 0.0f);
          if (masked && !blend) x = aux[e4][ai][bi] > 0.0f ? x : 0.0f;
          y[e4][ai][bi] = x;
        }
    if (masked && blend) {
#pragma unroll
      for (int e4 = 0; e4 < EB; ++e4)
#pragma unroll
        for (int ai = 0; ai < 2; ++ai)
#pragma unroll
          for (int bi = 0; bi < 2; ++bi) {
            const float mk = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rmask, (int)vo[e4][ai][bi], srow + (8 * ((EB * eb + e4) >> 2) + ((EB * eb + e4) & 3)) * PQ * 4, 0));
            y[e4][ai][bi] = mk > 0.0f ? y[e4][ai][bi] : 0.0f;
          }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e4 = 0; e4 < EB; ++e4)
#pragma unroll
      for (int ai = 0; ai < 2; ++ai)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, y[e4][ai][bi]), rout, (int)vo[e4][ai][bi],
                                                srow + (8 * ((EB * eb + e4) >> 2) + ((EB * eb + e4) & 3)) * PQ * 4, 0);
  }
}

constexpr int kWinoSA = 16 * 2 * kWinoBM * 8, kWinoSB = 16 * 2 * kWinoBN * 8, kWinoStage = kWinoSA + kWinoSB;
constexpr int kWinoCnt = 10;   // direct loads per thread and stage: 8 of U, 2 of V

__global__ __launch_bounds__(256, 1) void wino_gemm_kernel(const float* __restrict__ U, const float* __restrict__ V, int Cg,
                                                          int rows_p, unsigned tiles_p, int tiles_m, unsigned u_bytes,
                                                          unsigned v_bytes, WinoEpi ep) {
  constexpr int R = kWinoR;
  extern __shared__ float lds_dyn[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_dyn;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r = lane & 31;
  const int logical = __builtin_amdgcn_readfirstlane(xcd_remap(blockIdx.x, gridDim.x));
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m0 = tile_m * kWinoBM;
  const unsigned n0 = (unsigned)tile_n * kWinoBN;

  u32x4 rsU, rsV;
  {
    const uint64_t pu = reinterpret_cast<uint64_t>(U), pv = reinterpret_cast<uint64_t>(V);
    rsU.x = __builtin_amdgcn_readfirstlane((uint32_t)pu);
    rsU.y = __builtin_amdgcn_readfirstlane((uint32_t)(pu >> 32) & 0xffffu);
    rsU.z = u_bytes; rsU.w = 0x00020000u;
    rsV.x = __builtin_amdgcn_readfirstlane((uint32_t)pv);
    rsV.y = __builtin_amdgcn_readfirstlane((uint32_t)(pv >> 32) & 0xffffu);
    rsV.z = v_bytes; rsV.w = 0x00020000u;
  }
  // U: wave-load idx = 8 wave + i covers (f = idx / 2, h = idx % 2): 128 rows x 8 bytes = 64 lanes x 16 bytes
  const uint32_t voffA = (uint32_t)m0 * 8u + (uint32_t)lane * 16u;
  const uint32_t strideA = 2u * (uint32_t)rows_p * 8u;   // bytes per channel group within one f
  // V: wave-load idx = 2 wave + i covers f = 2 idx, 2 idx + 1 and both h: four runs of 32 tiles x 8 bytes
  const int seg = lane >> 4;
  const uint32_t strideB = 2u * tiles_p * 8u;
  const uint32_t voffB = ((uint32_t)(seg >> 1) * (uint32_t)Cg * 2u + (uint32_t)(seg & 1)) * tiles_p * 8u + n0 * 8u +
                         (uint32_t)(lane & 15) * 16u;
  // wave-uniform byte offsets of this wave's loads at channel group 0
  uint32_t soA[8], soB[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int idx = wave * 8 + i;
    soA[i] = ((uint32_t)(idx >> 1) * (uint32_t)Cg * 2u + (uint32_t)(idx & 1)) * (uint32_t)rows_p * 8u;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) soB[i] = (uint32_t)(2 * (wave * 2 + i)) * (uint32_t)Cg * strideB;
  // load i (0..9) of stage cg into ring buffer buf
  auto issue_one = [&](int i, int cg, int buf) {
    const uint32_t la = lds0 + (uint32_t)buf * kWinoStage, lb = la + kWinoSA;
    if (i < 8) dma_load16(rsU, la + (uint32_t)(wave * 8 + i) * 1024u, voffA, soA[i] + (uint32_t)cg * strideA);
    else dma_load16(rsV, lb + (uint32_t)(wave * 2 + (i - 8)) * 1024u, voffB, soB[i - 8] + (uint32_t)cg * strideB);
  };
  auto issue = [&](int cg, int buf) {
#pragma unroll
    for (int i = 0; i < kWinoCnt; ++i) issue_one(i, cg, buf);
  };

  f32x16 acc[16];
#pragma unroll
  for (int f = 0; f < 16; ++f)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[f][v] = 0.0f;

  const int nk = Cg;
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  wait_vmcnt<0>();
  __syncthreads();

  // operand reads: float2 = the two MFMAs of the stage
  const int a_rd = h * (kWinoBM * 2) + (wave * 32 + r) * 2;   // floats within an f's [h][128][2]
  const int b_rd = h * (kWinoBN * 2) + r * 2;
  auto stage_a = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + a_rd); };
  auto stage_b = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + kWinoSA / 4 + b_rd); };
  float2 a[2][4], b[2][4];
  {
    const float2* pa = stage_a(0);
    const float2* pb = stage_b(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      a[0][q] = pa[q * kWinoBM * 2];   // an f is 2 x 128 x 2 floats = kWinoBM * 2 float2
      b[0][q] = pb[q * kWinoBN * 2];
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);

  // One stage = four groups of four f, eight MFMAs each.  The matrix pipe takes an MFMA every 64 cycles and the wave
  // is alone on its SIMD: everything else (the next group's operand reads, the direct loads of the stage two ahead) is
  // written between the MFMAs, in the order it should issue, so that it runs while an MFMA executes.
  auto step = [&](int it, auto more_tag) {
    constexpr bool MORE = decltype(more_tag)::value;   // this stage issues the loads of stage it + 2
    const int rd = it % R, nx = (it + 1) % R, wr = (it + 2) % R;
    const float2* pa = stage_a(rd);
    const float2* pb = stage_b(rd);
    const float2* pna = stage_a(nx);
    const float2* pnb = stage_b(nx);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c = g & 1, n = c ^ 1;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].x, b[c][q].x, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g < 3) {
          a[n][q] = pa[(4 * (g + 1) + q) * kWinoBM * 2];
          b[n][q] = pb[(4 * (g + 1) + q) * kWinoBN * 2];
        } else if (MORE && g == 3 && q < 2) {
          issue_one(8 + q, it + 2, wr);   // (the last two of the ten)
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (g == 3) {
        // Every wave has read all of stage `it` once it is here (its last operands are in registers), so the loads the
        // next stage issues may overwrite it; with only the loads of stage it + 2 allowed in flight, stage it + 1 is
        // complete when all waves are past.
        if (MORE) wait_vmcnt<(R - 2) * kWinoCnt>();
        else wait_vmcnt<0>();
        __syncthreads();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].y, b[c][q].y, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g == 3) {
          a[n][q] = pna[q * kWinoBM * 2];
          b[n][q] = pnb[q * kWinoBN * 2];
        } else if (MORE) {
          // the first eight of the stage's ten direct loads, one behind each MFMA of groups 1 and 2
          if (g == 1) issue_one(q, it + 2, wr);
          if (g == 2) issue_one(4 + q, it + 2, wr);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  int it = 0;
  for (; it + 2 < nk; ++it) step(it, std::true_type());
  for (; it < nk; ++it) step(it, std::false_type());

  wino_epilogue(acc, ep, m0, n0, wave, lane);
}

// ---- the same product with B^T d B made inside the kernel ------------------------------------------------------------
// No V in memory: a stage's image operand (4 channels x 32 tiles x 16 f) is computed by the block from the image's
// patches.  Wave w owns channel 4 cg + w of the stage, lane = (tile, half): a thread brings three rows of its tile's
// 4x4 patch (rows half .. half + 2, what two rows of B^T d need) as twelve 4-byte direct loads into a per-thread LDS
// slot, three stages ahead of their use; one stage ahead it reads them back, forms its two rows of B^T d B (8 values)
// and writes them where the MFMA operand reads expect them.  Out-of-image taps (padding, tiles hanging over the edge)
// are out-of-range buffer offsets: they arrive as zeros.  All vector memory traffic of the loop is direct-to-LDS
// loads counted by hand; everything else is LDS and register work the compiler sees.
struct WinoImage {
  const float* x; unsigned x_bytes; int Ci, Hi, Wi, halo;
  int blk5;   // the 5x5 form: Ci is the planes an image has; the four channels of a stage are one plane read at four offsets
};

constexpr int kWinoRaw = 12 * 256 * 4;             // bytes of one stage's raw patch rows
constexpr int kWinoFusedCnt = 20;                  // direct loads per thread and stage: 12 patch dwords, 8 of U

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_load4(u32x4 rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}
#pragma clang diagnostic pop

struct WinoTail {
  int full, S, L;                     // blocks that take a whole tile; slices of a tail tile; stages per slice
  float* part; long long slab_elems, part_first;
};

__global__ __launch_bounds__(256, 1) void wino_gemm_fused_kernel(const float* __restrict__ U, WinoImage im, int Cg, int rows_p,
                                                                int tiles_m, unsigned u_bytes, WinoEpi ep, WinoTail tl) {
  constexpr int R = kWinoR;
  extern __shared__ float lds_dyn[];   // [R stages: U | V][2 raw patch slots]
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_dyn;
  const uint32_t raw0 = lds0 + (uint32_t)R * kWinoStage;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r = lane & 31;
  // a block past the whole rounds takes one slice of a tail tile's channel loop: stages cg0 .. cg0 + nk - 1, and
  // writes its part of the result unblended into the slice's slab.  The whole-tile blocks and the tail blocks are
  // each dealt evenly to the XCDs (tl.full is a multiple of 256).
  int tile, cg0 = 0, nk = Cg;
  if (tl.S <= 1) {
    tile = __builtin_amdgcn_readfirstlane(xcd_remap(blockIdx.x, gridDim.x));
  } else if ((int)blockIdx.x < tl.full) {
    tile = __builtin_amdgcn_readfirstlane(xcd_remap(blockIdx.x, tl.full));
  } else {
    const int ti = __builtin_amdgcn_readfirstlane(xcd_remap((int)blockIdx.x - tl.full, (int)gridDim.x - tl.full));
    const int slice = ti % tl.S;
    tile = tl.full + ti / tl.S;
    cg0 = slice * tl.L;
    nk = Cg - cg0 < tl.L ? Cg - cg0 : tl.L;
    ep.out = tl.part + (long long)slice * tl.slab_elems - tl.part_first;
    ep.bias = nullptr; ep.mask = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f; ep.relu = 0;
  }
  const int tile_m = tile % tiles_m, tile_n = tile / tiles_m;
  const int m0 = tile_m * kWinoBM;
  const unsigned n0 = (unsigned)tile_n * kWinoBN;

  u32x4 rsU, rsX;
  {
    const uint64_t pu = reinterpret_cast<uint64_t>(U), px = reinterpret_cast<uint64_t>(im.x);
    rsU.x = __builtin_amdgcn_readfirstlane((uint32_t)pu);
    rsU.y = __builtin_amdgcn_readfirstlane((uint32_t)(pu >> 32) & 0xffffu);
    rsU.z = u_bytes; rsU.w = 0x00020000u;
    rsX.x = __builtin_amdgcn_readfirstlane((uint32_t)px);
    rsX.y = __builtin_amdgcn_readfirstlane((uint32_t)(px >> 32) & 0xffffu);
    rsX.z = im.x_bytes; rsX.w = 0x00020000u;
  }
  const uint32_t voffA = (uint32_t)m0 * 8u + (uint32_t)lane * 16u;
  const uint32_t strideA = 2u * (uint32_t)rows_p * 8u;
  uint32_t soA[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int idx = wave * 8 + i;
    soA[i] = ((uint32_t)(idx >> 1) * (uint32_t)Cg * 2u + (uint32_t)(idx & 1)) * (uint32_t)rows_p * 8u;
  }
  // this thread's twelve patch taps: rows h .. h + 2 of the 4x4 patch of tile n0 + r, as byte offsets in channel 0 of its image
  const int HW = im.Hi * im.Wi;
  uint32_t poff[3][4];
  {
    const unsigned t = n0 + (unsigned)r;
    uint32_t q1, tx, n, ty;
    ep.dTQ.divmod(t, q1, tx);
    ep.dTP.divmod(q1, n, ty);
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int hh = 2 * (int)ty - im.halo + h + a, ww = 2 * (int)tx - im.halo + k;
        const bool in = t < ep.tiles && (unsigned)hh < (unsigned)im.Hi && (unsigned)ww < (unsigned)im.Wi;
        poff[a][k] = in ? ((n * (unsigned)im.Ci) * (unsigned)HW + (unsigned)(hh * im.Wi + ww)) * 4u : kInvalidByteOff;
      }
  }
  const uint32_t chan_stride = (uint32_t)HW * 4u;
  // this wave's channel of stage cg lies at cg * tap_mul + tap_add: plane 4 cg + wave, or in the 5x5 form plane cg read
  // 3 (wave / 2) rows and 3 (wave % 2) columns further on
  const uint32_t tap_mul = im.blk5 ? chan_stride : 4u * chan_stride;
  const uint32_t tap_add = im.blk5 ? (uint32_t)(3 * (wave >> 1) * im.Wi + 3 * (wave & 1)) * 4u : (uint32_t)wave * chan_stride;
  // direct load i (0..11: patch taps into raw slot `par`; 12..19: U into ring buffer `buf`) of stage cg
  auto issue_one = [&](int i, int cg, int buf, int par) {
    if (i < 12)
      dma_load4(rsX, raw0 + (uint32_t)par * kWinoRaw + (uint32_t)i * 1024u + (uint32_t)wave * 256u, poff[i >> 2][i & 3],
                (uint32_t)(cg0 + cg) * tap_mul + tap_add);
    else
      dma_load16(rsU, lds0 + (uint32_t)buf * kWinoStage + (uint32_t)(wave * 8 + (i - 12)) * 1024u, voffA,
                 soA[i - 12] + (uint32_t)(cg0 + cg) * strideA);
  };
  // the thread's part of stage s's image operand: raw slot s & 1 -> two rows of B^T d B -> V area of ring buffer buf
  const float* rawp = lds_dyn + R * (kWinoStage / 4) + tid;
  const int fe = h ? 12 : 0, fo = h ? 8 : 4;   // first f of the row made from d(a0) - d(a2), and of the other one
  float* const vdst = lds_dyn + kWinoSA / 4 + (wave >> 1) * (kWinoBN * 2) + r * 2 + (wave & 1);
  float da[3][4];
  auto raw_read = [&](int par, int a) {
#pragma unroll
    for (int k = 0; k < 4; ++k) da[a][k] = rawp[par * (kWinoRaw / 4) + (a * 4 + k) * 256];
  };
  float te[4], to[4];
  auto transform_cols = [&]() {   // the column pass: this thread's two rows of B^T d
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      te[k] = da[0][k] - da[2][k];
      to[k] = h ? da[1][k] - da[0][k] : da[1][k] + da[2][k];
    }
  };
  auto transform_row = [&](int which, int buf) {   // the row pass of one of them, into the V area of ring buffer buf
    float* d = vdst + buf * (kWinoStage / 4) + (which ? fo : fe) * 128;   // an f is 2 x 32 x 2 floats
    const float* t = which ? to : te;
    d[0 * 128] = t[0] - t[2];
    d[1 * 128] = t[1] + t[2];
    d[2 * 128] = t[2] - t[1];
    d[3 * 128] = t[1] - t[3];
  };

  f32x16 acc[16];
#pragma unroll
  for (int f = 0; f < 16; ++f)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[f][v] = 0.0f;

  // Stages 0 and 1 on their way, their image operands made, the taps of stage 2 on their way (into the slot stage
  // 0's were read from): the taps run three stages ahead of the MFMAs, U two.
#pragma unroll
  for (int i = 0; i < kWinoFusedCnt; ++i) issue_one(i, 0, 0, 0);
  if (nk > 1) {
#pragma unroll
    for (int i = 0; i < kWinoFusedCnt; ++i) issue_one(i, 1, 1, 1);
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_sched_barrier(0);
  raw_read(0, 0); raw_read(0, 1); raw_read(0, 2);
  transform_cols();
  transform_row(0, 0);
  transform_row(1, 0);
  if (nk > 1) {
    raw_read(1, 0); raw_read(1, 1); raw_read(1, 2);
    transform_cols();
    transform_row(0, 1);
    transform_row(1, 1);
  }
  __builtin_amdgcn_sched_barrier(0);
  if (nk > 2) {
#pragma unroll
    for (int i = 0; i < 12; ++i) issue_one(i, 2, 2, 0);
  }
  __syncthreads();

  const int a_rd = h * (kWinoBM * 2) + (wave * 32 + r) * 2;
  const int b_rd = h * (kWinoBN * 2) + r * 2;
  auto stage_a = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + a_rd); };
  auto stage_b = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + kWinoSA / 4 + b_rd); };
  float2 a[2][4], b[2][4];
  {
    const float2* pa = stage_a(0);
    const float2* pb = stage_b(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      a[0][q] = pa[q * kWinoBM * 2];
      b[0][q] = pb[q * kWinoBN * 2];
    }
  }

  // Stage `it`: MFMAs on ring buffer rd.  Behind them, one instruction or two per MFMA, in issue order:
  //   groups 0, 1 (first half):  the patch taps of stage it + 3 (12 loads) into raw slot (it + 1) & 1;
  //   groups 1 (second half), 2 (first half):  U of stage it + 2 (8 loads) into ring buffer wr;
  //   group 2:  stage it + 2's taps (issued a stage and a half ago) read back from raw slot it & 1;
  //   group 3, first half:  B^T d B of those, written into ring buffer wr: nobody reads it before the barrier of
  //   stage it + 1, so none of this stands between a stage's last operand reads and the next stage's first;
  //   then the stage's one barrier, which also waits for U of stage it + 1; second half: the first operands of stage it + 1.
  int rd = 0, nx = 1, wr = 2, par = 0;   // ring buffers of stages it, it + 1, it + 2; raw slot of stage it + 2 (= it & 1)
  auto step = [&](int it, auto ip_tag, auto iu_tag) {
    constexpr bool IP = decltype(ip_tag)::value;       // there is a stage it + 3: its taps are issued here
    constexpr bool IU = decltype(iu_tag)::value;       // there is a stage it + 2: its U is issued and its image operand made here
    const float2* pa = stage_a(rd);
    const float2* pb = stage_b(rd);
    const float2* pna = stage_a(nx);
    const float2* pnb = stage_b(nx);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c = g & 1, n = c ^ 1;
      __builtin_amdgcn_sched_barrier(0);
      if (g == 2 && IU) {
        // Stage it + 2's taps are there once all but the loads issued after them are: the taps of stage it + 3 (12)
        // and the first four loads of U of stage it + 2.  (U of stage it + 1 lies between them except in stage 0, and
        // need not be waited for yet; it was issued a stage ago and the barrier below needs it anyway.)
        wait_vmcnt<(IP ? 12 : 0) + 4>();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].x, b[c][q].x, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g < 3) {
          a[n][q] = pa[(4 * (g + 1) + q) * kWinoBM * 2];
          b[n][q] = pb[(4 * (g + 1) + q) * kWinoBN * 2];
        }
        if (IP && g < 2) issue_one(8 * g + q, it + 3, 0, par ^ 1);          // taps 0-3, 8-11
        if (IU && g == 2) issue_one(16 + q, it + 2, wr, 0);                 // U 4-7
        if (IU && g == 2 && q < 3) raw_read(par, q);
        if (IU && g == 3) {
          if (q == 0) transform_cols();
          if (q == 1) transform_row(0, wr);
          if (q == 2) transform_row(1, wr);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (g == 3) {
        // every wave has read all of stage `it` once it is here; U of stage it + 1 is complete when only the loads
        // issued after it are in flight
        wait_vmcnt<(IP ? 12 : 0) + (IU ? 8 : 0)>();
        __syncthreads();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].y, b[c][q].y, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g == 3) {
          a[n][q] = pna[q * kWinoBM * 2];
          b[n][q] = pnb[q * kWinoBN * 2];
        }
        if (IP && g == 0) issue_one(4 + q, it + 3, 0, par ^ 1);             // taps 4-7
        if (IU && g == 1) issue_one(12 + q, it + 2, wr, 0);                 // U 0-3
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const int t = rd; rd = nx; nx = wr; wr = t;
    par ^= 1;
  };
  int it = 0;
  for (; it + 3 < nk; ++it) step(it, std::true_type(), std::true_type());
  if (it + 2 < nk) { step(it, std::false_type(), std::true_type()); ++it; }
  for (; it < nk; ++it) step(it, std::false_type(), std::false_type());

  wino_epilogue(acc, ep, m0, n0, wave, lane);
}

// ---- filter gradient --------------------------------------------------------------------------------------------------
//   dg = G^T [ sum over tiles (A dY A^T) o (B^T d B) ] G      A dY A^T: the 2x2 tile of dy -> 4x4,  A = [1 0; 1 1; 1 -1; 0 -1]
// The same 16 products with the roles turned: rows = filters, columns = input channels, the contraction runs over
// the tiles, four to a stage.  A tile's patch and its dy taps are a few floats in each of hundreds of planes: loaded
// where they lie they are one cache line per lane and 4 bytes used of each (measured: 2 us per stage instead of 1).
// So a prep launch (wino_filter_prep_kernel) writes both operands tile-major:
//   Vt[f][tile / 4][h][channel][2] = B^T d B in the product's operand order (tile = 4 (tile / 4) + 2 h + j), which goes
//      straight to LDS like U in the forward kernel;
//   dyt[tile][filter][4] = the tile's four dy taps, 16 bytes a filter: a lane (= a filter) brings two tiles' taps as two
//      16-byte direct loads into its LDS slot two stages ahead, reads them back a stage ahead, forms A dY A^T of both
//      (12 VALU instructions a tile) and writes the 16 pairs into the next stage's ring buffer.
// Zeros for the tiles the count is rounded up with, for taps past an odd extent, for filters and channels up to
// whole blocks.  The last row of A is taken as (0, 1) instead of (0, -1): no negations in the loop; the reduction flips
// the sign of the f that have exactly one index 3.  Few (filters x channels) tiles exist (36 for 384 x 384), so the
// image's tiles are cut into S slices, one block each; the slices' partial dU go to scratch and
// wino_filter_reduce_kernel adds them in slice order, applies G^T . G and the alpha / beta blend.
struct WinoFilterArgs {
  const float* Vt; const float* dyt; float* part;
  unsigned vt_bytes, dyt_bytes, part_bytes;
  int Kp, Cp, TGs;                // padded filter / channel counts, tile groups (stages) over all slices
  int tiles_m, tiles_c, stages;   // stages (of four tiles) per slice
};

constexpr int kWinoFRaw = 2 * 256 * 16;   // bytes of one stage's dy taps: two tiles x 16 bytes per thread
constexpr int kWinoFCnt = 4;              // direct loads per thread and stage: 2 of dy taps, 2 of Vt

__global__ __launch_bounds__(256, 1) void wino_bwd_filter_kernel(WinoFilterArgs p) {
  constexpr int R = kWinoR;
  extern __shared__ float lds_dyn[];   // [R stages: A | B][2 raw slots]
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_dyn;
  const uint32_t raw0 = lds0 + (uint32_t)R * kWinoStage;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r = lane & 31;
  const int logical = __builtin_amdgcn_readfirstlane(xcd_remap(blockIdx.x, gridDim.x));
  const int tile_m = logical % p.tiles_m, rest = logical / p.tiles_m;
  const int tile_c = rest % p.tiles_c, split = rest / p.tiles_c;
  const int m0 = tile_m * kWinoBM, c0 = tile_c * kWinoBN;
  const uint32_t tg0 = (uint32_t)split * (uint32_t)p.stages;   // this slice's first tile group

  u32x4 rsV, rsY;
  {
    const uint64_t pv = reinterpret_cast<uint64_t>(p.Vt), py = reinterpret_cast<uint64_t>(p.dyt);
    rsV.x = __builtin_amdgcn_readfirstlane((uint32_t)pv);
    rsV.y = __builtin_amdgcn_readfirstlane((uint32_t)(pv >> 32) & 0xffffu);
    rsV.z = p.vt_bytes; rsV.w = 0x00020000u;
    rsY.x = __builtin_amdgcn_readfirstlane((uint32_t)py);
    rsY.y = __builtin_amdgcn_readfirstlane((uint32_t)(py >> 32) & 0xffffu);
    rsY.z = p.dyt_bytes; rsY.w = 0x00020000u;
  }
  // dy taps: filter m0 + 64 (wave & 1) + lane of tiles 4 tg + 2 (wave / 2) + {0, 1}
  const uint32_t voffY = (uint32_t)(m0 + 64 * (wave & 1) + lane) * 16u;
  const uint32_t tileY = (uint32_t)p.Kp * 16u;   // bytes per tile of dyt
  // Vt: wave-load idx = 2 wave + i covers f = 2 idx, 2 idx + 1 and both h: four runs of 32 channels x 8 bytes
  const int seg = lane >> 4;
  const uint32_t strideB = 2u * (uint32_t)p.Cp * 8u;   // bytes per tile group within one f
  const uint32_t voffB = ((uint32_t)(seg >> 1) * (uint32_t)p.TGs * 2u + (uint32_t)(seg & 1)) * (uint32_t)p.Cp * 8u +
                         (uint32_t)c0 * 8u + (uint32_t)(lane & 15) * 16u;
  // direct load i of stage st (tile group tg0 + st): 0, 1 the dy taps of the wave's two tiles into raw slot par;
  // 2, 3 Vt into ring buffer buf
  auto issue_one = [&](int i, int st, int buf, int par) {
    const uint32_t tg = tg0 + (uint32_t)st;
    if (i < 2)
      dma_load16(rsY, raw0 + (uint32_t)par * kWinoFRaw + (uint32_t)i * 4096u + (uint32_t)wave * 1024u, voffY,
                 (4u * tg + 2u * (uint32_t)(wave >> 1) + (uint32_t)i) * tileY);
    else
      dma_load16(rsV, lds0 + (uint32_t)buf * kWinoStage + kWinoSA + (uint32_t)(wave * 2 + (i - 2)) * 1024u, voffB,
                 ((uint32_t)(2 * (wave * 2 + (i - 2))) * (uint32_t)p.TGs + tg) * strideB);
  };
  const float4* rawp = reinterpret_cast<const float4*>(lds_dyn + R * (kWinoStage / 4)) + tid;
  float4 yv[2];
  auto raw_read = [&](int par) {
    yv[0] = rawp[par * (kWinoFRaw / 16)];
    yv[1] = rawp[par * (kWinoFRaw / 16) + 256];
  };
  // A operand: [f][h'][128 filters][2 tiles], this thread's filter 64 (wave & 1) + lane, tile pair h' = wave / 2
  float2* const adst = reinterpret_cast<float2*>(lds_dyn + (wave >> 1) * (kWinoBM * 2) + (64 * (wave & 1) + lane) * 2);
  auto transform_y_rows = [&](int i0, int buf) {   // rows i0, i0 + 1 of A' dY A'^T of both tiles (taps: x y / z w)
    float2* d = adst + buf * (kWinoStage / 8);
#pragma unroll
    for (int i = i0; i < i0 + 2; ++i) {
      float ra[2], rb[2];   // row i of A' dY: (first column, second column), per tile
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        ra[j] = i == 0 ? yv[j].x : i == 1 ? yv[j].x + yv[j].z : i == 2 ? yv[j].x - yv[j].z : yv[j].z;
        rb[j] = i == 0 ? yv[j].y : i == 1 ? yv[j].y + yv[j].w : i == 2 ? yv[j].y - yv[j].w : yv[j].w;
      }
      // an f is 2 x 128 x 2 floats = 256 float2
      d[(4 * i + 0) * 256] = make_float2(ra[0], ra[1]);
      d[(4 * i + 1) * 256] = make_float2(ra[0] + rb[0], ra[1] + rb[1]);
      d[(4 * i + 2) * 256] = make_float2(ra[0] - rb[0], ra[1] - rb[1]);
      d[(4 * i + 3) * 256] = make_float2(rb[0], rb[1]);
    }
  };

  f32x16 acc[16];
#pragma unroll
  for (int f = 0; f < 16; ++f)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[f][v] = 0.0f;

  const int nk = p.stages;
  // stages 0 and 1 on their way (taps ahead of Vt, as in the loop), stage 0's A operand made
#pragma unroll
  for (int i = 0; i < kWinoFCnt; ++i) issue_one(i, 0, 0, 0);
  if (nk > 1) {
#pragma unroll
    for (int i = 0; i < kWinoFCnt; ++i) issue_one(i, 1, 1, 1);
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_sched_barrier(0);
  raw_read(0);
  transform_y_rows(0, 0);
  transform_y_rows(2, 0);
  __syncthreads();

  const int a_rd = h * (kWinoBM * 2) + (wave * 32 + r) * 2;
  const int b_rd = h * (kWinoBN * 2) + r * 2;
  auto stage_a = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + a_rd); };
  auto stage_b = [&](int buf) { return reinterpret_cast<const float2*>(lds_dyn + buf * (kWinoStage / 4) + kWinoSA / 4 + b_rd); };
  float2 a[2][4], b[2][4];
  {
    const float2* pa = stage_a(0);
    const float2* pb = stage_b(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      a[0][q] = pa[q * kWinoBM * 2];
      b[0][q] = pb[q * kWinoBN * 2];
    }
  }

  // Stage `it`: MFMAs on ring buffer rd.  Behind them: group 0, the four loads of stage it + 2 (taps into raw slot
  // it & 1, Vt into ring buffer wr); group 2, stage it + 1's taps read back from the other slot; group 3 (first half), A
  // dY A^T of those written into ring buffer nx; the stage's barrier, which also waits for Vt of stage it + 1; then the
  // first operands of stage it + 1.
  int rd = 0, nx = 1, wr = 2, par = 0;
  auto step = [&](int it, auto i2_tag, auto t1_tag) {
    constexpr bool I2 = decltype(i2_tag)::value;   // there is a stage it + 2: its loads are issued here
    constexpr bool T1 = decltype(t1_tag)::value;   // there is a stage it + 1: its A operand is made here
    const float2* pa = stage_a(rd);
    const float2* pb = stage_b(rd);
    const float2* pna = stage_a(nx);
    const float2* pnb = stage_b(nx);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c = g & 1, n = c ^ 1;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].x, b[c][q].x, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g < 3) {
          a[n][q] = pa[(4 * (g + 1) + q) * kWinoBM * 2];
          b[n][q] = pb[(4 * (g + 1) + q) * kWinoBN * 2];
        }
        if (I2 && g == 0) issue_one(q, it + 2, wr, par);
        if (T1 && g == 3 && q < 2) transform_y_rows(2 * q, nx);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (g == 1 && T1) {
        // stage it + 1's taps (the first two loads issued during stage it - 1) are there once only the two Vt loads
        // behind them and this stage's four are in flight
        if (I2) wait_vmcnt<6>();
        else wait_vmcnt<2>();
      }
      if (g == 3) {
        // every wave has read all of stage `it` and written its part of stage it + 1's A; Vt of stage it + 1 is complete
        // when only this stage's loads are in flight
        if (I2) wait_vmcnt<kWinoFCnt>();
        else wait_vmcnt<0>();
        __syncthreads();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[4 * g + q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][q].y, b[c][q].y, acc[4 * g + q], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (g == 3) {
          a[n][q] = pna[q * kWinoBM * 2];
          b[n][q] = pnb[q * kWinoBN * 2];
        }
        if (T1 && g == 1 && q == 0) raw_read(par ^ 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const int t = rd; rd = nx; nx = wr; wr = t;
    par ^= 1;
  };
  int it = 0;
  for (; it + 2 < nk; ++it) step(it, std::true_type(), std::true_type());
  if (it + 1 < nk) { step(it, std::false_type(), std::true_type()); ++it; }
  if (it < nk) step(it, std::false_type(), std::false_type());

  // this slice's partial dU: part[slice][f][filter][channel]
  const __amdgpu_buffer_rsrc_t rpart = make_rsrc(p.part, p.part_bytes);
  const uint32_t voff = ((uint32_t)(m0 + 32 * wave + 4 * h) * (uint32_t)p.Cp + (uint32_t)(c0 + r)) * 4u;
  const uint32_t plane = (uint32_t)p.Kp * (uint32_t)p.Cp * 4u;
#pragma unroll
  for (int f = 0; f < 16; ++f) {
    __builtin_amdgcn_sched_barrier(0);
    wino_pin_acc(acc);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float v = acc[f][e];   // (a copy: __builtin_bit_cast straight from the vector element takes element 0 every time)
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rpart, (int)voff,
                                            (int)(((uint32_t)split * 16u + (uint32_t)f) * plane +
                                                  (uint32_t)(8 * (e >> 2) + (e & 3)) * (uint32_t)p.Cp * 4u), 0);
    }
  }
}

// dw[k][c][r][s] = alpha * (G^T dU G)[r][s] + beta * dw, dU = the slices' partial sums added in slice order
__global__ __launch_bounds__(256) void wino_filter_reduce_kernel(const float* __restrict__ part, int S, int K, int C, int Kp, int Cp,
                                                               float alpha, float beta, float* __restrict__ dw) {
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= (unsigned)K * (unsigned)C) return;
  const unsigned k = idx / (unsigned)C, c = idx - k * (unsigned)C;
  const size_t plane = (size_t)Kp * Cp;
  float u[16];
#pragma unroll
  for (int f = 0; f < 16; ++f) u[f] = 0.0f;
  for (int sl = 0; sl < S; ++sl) {   // a slice's 16 values in flight together, the slices added in order
    float v[16];
#pragma unroll
    for (int f = 0; f < 16; ++f) v[f] = part[((size_t)sl * 16 + f) * plane + (size_t)k * Cp + c];
#pragma unroll
    for (int f = 0; f < 16; ++f) u[f] += v[f];
  }
#pragma unroll
  for (int f = 0; f < 16; ++f)
    if (((f >> 2) == 3) != ((f & 3) == 3)) u[f] = -u[f];   // the sign the loop's (0, 1) for A's last row left out
  float t[3][4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    t[0][j] = u[j] + 0.5f * (u[4 + j] + u[8 + j]);
    t[1][j] = 0.5f * (u[4 + j] - u[8 + j]);
    t[2][j] = 0.5f * (u[4 + j] + u[8 + j]) + u[12 + j];
  }
  float* o = dw + (size_t)idx * 9;
#pragma unroll
  for (int rr = 0; rr < 3; ++rr) {
    const float g0 = t[rr][0] + 0.5f * (t[rr][1] + t[rr][2]);
    const float g1 = 0.5f * (t[rr][1] - t[rr][2]);
    const float g2 = 0.5f * (t[rr][1] + t[rr][2]) + t[rr][3];
    const float g[3] = {g0, g1, g2};
#pragma unroll
    for (int ss = 0; ss < 3; ++ss) o[rr * 3 + ss] = beta != 0.0f ? fmaf(beta, o[rr * 3 + ss], alpha * g[ss]) : alpha * g[ss];
  }
}

// The filter gradient's operands, both in one launch (two kinds of blocks).
struct WinoFilterPrepArgs {
  const float* x; const float* dy; float* Vt; float* dyt;
  unsigned x_bytes, dy_bytes;
  int N, C, H, W, K, P, Q, halo, Kp, Cp, TGs;
  unsigned tiles;
  FastDiv dTQ, dTP, dPairs, dKp;
  unsigned v_items, y_items, v_blocks;
};

// Vt of channels (2 ch, 2 ch + 1) x tiles (2 up, 2 up + 1): one 16-byte store per f, [channel][tile of the pair]
__device__ __forceinline__ void wino_filter_v_item(const WinoFilterPrepArgs& a, unsigned idx) {
  // eight neighbouring lanes take eight channel pairs of one tile pair (their stores are 128 consecutive bytes), the
  // next eight the next tile pair (their loads are neighbours in eight planes): 0.133 ms for 385 MB; runs of 4 and of 16
  // channel pairs measured 0.174 and 0.149
  uint32_t ch_hi, up;
  a.dPairs.divmod(idx >> 3, ch_hi, up);   // up: tile pair = 2 (tile group) + h
  const uint32_t ch = ch_hi * 8u + (idx & 7u);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, a.x_bytes);
  float v[16][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const unsigned t = 2 * up + tt;
    uint32_t q1, tx, n, ty;
    a.dTQ.divmod(t, q1, tx);
    a.dTP.divmod(q1, n, ty);
    const int h0 = 2 * (int)ty - a.halo, w0 = 2 * (int)tx - a.halo;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = (int)ch * 2 + j;
      const bool live = t < a.tiles && c < a.C;
      const unsigned base = (n * (unsigned)a.C + (unsigned)c) * (unsigned)(a.H * a.W);
      float d[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int hh = h0 + i, ww = w0 + k;
          const bool in = live && (unsigned)hh < (unsigned)a.H && (unsigned)ww < (unsigned)a.W;
          const unsigned off = in ? (base + (unsigned)(hh * a.W + ww)) * 4u : kInvalidByteOff;
          d[i][k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (int)off, 0, 0));
        }
      float s[4][4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        s[0][k] = d[0][k] - d[2][k];
        s[1][k] = d[1][k] + d[2][k];
        s[2][k] = d[2][k] - d[1][k];
        s[3][k] = d[1][k] - d[3][k];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[4 * i + 0][2 * j + tt] = s[i][0] - s[i][2];
        v[4 * i + 1][2 * j + tt] = s[i][1] + s[i][2];
        v[4 * i + 2][2 * j + tt] = s[i][2] - s[i][1];
        v[4 * i + 3][2 * j + tt] = s[i][1] - s[i][3];
      }
    }
  }
  float4* V4 = reinterpret_cast<float4*>(a.Vt);
  const size_t half_cp = (size_t)a.Cp / 2, plane = (size_t)a.TGs * 2 * half_cp;   // float4s per f
#pragma unroll
  for (int f = 0; f < 16; ++f) V4[f * plane + (size_t)up * half_cp + ch] = make_float4(v[f][0], v[f][1], v[f][2], v[f][3]);
}

// dyt[tile][filter] = the tile's four dy taps
__device__ __forceinline__ void wino_filter_y_item(const WinoFilterPrepArgs& a, unsigned idx) {
  uint32_t k_hi, t;   // (eight filters of one tile, then the next tile: as above)
  a.dKp.divmod(idx >> 3, k_hi, t);
  const uint32_t k = k_hi * 8u + (idx & 7u);
  uint32_t q1, tx, n, ty;
  a.dTQ.divmod(t, q1, tx);
  a.dTP.divmod(q1, n, ty);
  const __amdgpu_buffer_rsrc_t ry = make_rsrc(a.dy, a.dy_bytes);
  const bool live = t < a.tiles && (int)k < a.K;
  const unsigned base = (n * (unsigned)a.K + k) * (unsigned)(a.P * a.Q);
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int pp = 2 * (int)ty + (e >> 1), qq = 2 * (int)tx + (e & 1);
    const bool in = live && pp < a.P && qq < a.Q;
    const unsigned off = in ? (base + (unsigned)(pp * a.Q + qq)) * 4u : kInvalidByteOff;
    v[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ry, (int)off, 0, 0));
  }
  reinterpret_cast<float4*>(a.dyt)[(size_t)t * a.Kp + k] = make_float4(v[0], v[1], v[2], v[3]);
}

__global__ __launch_bounds__(256) void wino_filter_prep_kernel(WinoFilterPrepArgs a) {
  if (blockIdx.x < a.v_blocks) {
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    if (idx < a.v_items) wino_filter_v_item(a, idx);
  } else {
    const unsigned idx = (blockIdx.x - a.v_blocks) * 256u + threadIdx.x;
    if (idx < a.y_items) wino_filter_y_item(a, idx);
  }
}

// The tail form's second pass: out = alpha * (sum of the slices' slabs) + beta * out (+ bias, ReLU or mask) on the
// elements that a tail block produced; elements of the same images that a whole-tile block wrote are left alone.
struct WinoTailReduce {
  const float* part; float* out; const float* bias; const float* mask;
  float alpha, beta;
  int relu, S, Ko, P, Q, TP, TQ, tiles_m, full;
  unsigned first, total;       // elements [first, total) of the result
  long long slab_elems;
  FastDiv dPQ, dQ, dKo;
};
__global__ __launch_bounds__(256) void wino_tail_reduce_kernel(WinoTailReduce a) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= a.total - a.first) return;
  const unsigned g = a.first + i;
  uint32_t plane, pix, n, k, pp, qq;
  a.dPQ.divmod(g, plane, pix);
  a.dKo.divmod(plane, n, k);
  a.dQ.divmod(pix, pp, qq);
  const unsigned t = (n * (unsigned)a.TP + (pp >> 1)) * (unsigned)a.TQ + (qq >> 1);
  const unsigned logical = (t / kWinoBN) * (unsigned)a.tiles_m + k / kWinoBM;
  if (logical < (unsigned)a.full) return;
  float v = 0.0f;
  for (int sl = 0; sl < a.S; ++sl) v += a.part[(long long)sl * a.slab_elems + i];
  v *= a.alpha;
  if (a.beta != 0.0f) v = fmaf(a.beta, a.out[g], v);
  if (a.bias) v += a.bias[k];
  if (a.relu) v = fmaxf(v, 0.0f);
  if (a.mask) v = a.mask[g] > 0.0f ? v : 0.0f;
  a.out[g] = v;
}

}  // namespace

// in: (N, Ci, Hi, Wi) with g.halo zeros around; w: the layer's filter (K, C, 3, 3): forward reads it as (Ko, Ci), the
// backward-data form (bwd) as (Ci, Ko) with flipped taps; out: (N, Ko, P, Q).  ws: g.total() bytes, 256-aligned.
int launch_conv_wino(const WinoGeom& g, bool bwd, const float* in, const float* w, float* out, float alpha, float beta,
                     const float* bias, int relu, const float* mask, void* ws, hipStream_t stream, const char* tag) {
  if (!g.ok) return RH_E_UNSUPPORTED;
  float* U = static_cast<float*>(ws);
  float* V = reinterpret_cast<float*>(static_cast<char*>(ws) + g.u_bytes);
  if (g.blk5) {
    // the zero-bordered copy the 5x5 form reads (behind U; V is made in the kernel)
    if (bwd) return RH_E_UNSUPPORTED;
    float* xp = reinterpret_cast<float*>(static_cast<char*>(ws) + g.u_bytes + g.v_bytes);
    launch_pad_image(in, xp, (long long)g.N * g.C5, g.H5, g.W5, g.Hi, g.Wi, g.pad5, stream);
    if (int e = launch_status()) return e;
    in = xp;
  }
  WinoPrepArgs a;
  a.w = w; a.x = in; a.U = U; a.V = V;
  a.blk5 = g.blk5; a.C5 = g.C5;
  a.Ko = g.Ko; a.Ci = g.Ci; a.Cg = g.Cg; a.rows_p = g.rows_p; a.bwd = bwd ? 1 : 0;
  a.Hi = g.Hi; a.Wi = g.Wi; a.halo = g.halo;
  a.tiles = (unsigned)g.tiles; a.tiles_p = (unsigned)g.tiles_p;
  a.x_bytes = (unsigned)(4ull * (unsigned long long)g.N * (g.blk5 ? g.C5 : g.Ci) * g.Hi * g.Wi);
  a.dRows = FastDiv((uint32_t)g.rows_p); a.dPairs = FastDiv((uint32_t)(g.tiles_p / 2));
  a.dTQ = FastDiv((uint32_t)g.TQ); a.dTP = FastDiv((uint32_t)g.TP);
  const unsigned long long fi = (unsigned long long)g.Cg * 2 * g.rows_p, ii = (unsigned long long)g.Cg * 2 * (g.tiles_p / 2);
  if (fi >= (1ull << 31) || ii >= (1ull << 31)) return RH_E_LIMIT;
  // channel counts that fill groups of four take the kernel that makes V itself: only the filter is prepared here
  const bool fused = g.Ci % 4 == 0;
  a.filt_items = (unsigned)fi; a.in_items = fused ? 0u : (unsigned)ii;
  a.in_blocks = (unsigned)cdiv<unsigned long long>(a.in_items, 256);
  const unsigned filt_blocks = (unsigned)cdiv<unsigned long long>(fi, 256);
  {
    ProfScope prof("wino_transform", 4.0 * ((fused ? 0.0 : (double)g.N * g.Ci * g.Hi * g.Wi) + 9.0 * g.Ko * g.Ci) +
                                         128.0 * ((double)g.Cg * g.rows_p + (fused ? 0.0 : (double)g.Cg * g.tiles_p)), stream);
    hipLaunchKernelGGL(wino_prep_kernel, dim3(a.in_blocks + filt_blocks), dim3(256), 0, stream, a);
    if (int e = launch_status()) return e;
  }
  WinoEpi ep;
  ep.out = out; ep.bias = bias; ep.mask = mask; ep.alpha = alpha; ep.beta = beta; ep.relu = relu;
  ep.Ko = g.Ko; ep.P = g.P; ep.Q = g.Q; ep.tiles = (unsigned)g.tiles;
  ep.out_bytes = (unsigned)(4ull * (unsigned long long)g.N * g.Ko * g.P * g.Q);
  ep.dTQ = a.dTQ; ep.dTP = a.dTP;
  const int tiles_m_ = g.rows_p / kWinoBM;
  const long long tiles_n_ = g.tiles_p / kWinoBN;
  if (fused) {
    constexpr size_t lds_f = (size_t)kWinoR * kWinoStage + 2 * (size_t)kWinoRaw;
    static_assert(lds_f <= 160 * 1024, "ring and patch slots do not fit the 160 KB LDS of a CU");
    static const hipError_t attr_f = hipFuncSetAttribute(reinterpret_cast<const void*>(&wino_gemm_fused_kernel),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_f);
    if (attr_f != hipSuccess) return (int)attr_f;
    WinoImage im;
    im.x = in; im.x_bytes = a.x_bytes; im.Ci = g.blk5 ? g.C5 : g.Ci; im.Hi = g.Hi; im.Wi = g.Wi; im.halo = g.halo;
    im.blk5 = g.blk5;
    ProfScope prof(tag, 2.0 * 16.0 * (double)g.Ko * g.Ci * (double)g.tiles, stream);
    WinoTail tl;
    tl.full = g.full_tiles; tl.S = g.tail_S; tl.L = g.tail_L;
    tl.part = reinterpret_cast<float*>(static_cast<char*>(ws) + g.u_bytes + g.v_bytes + g.img_bytes);
    tl.slab_elems = g.slab_elems; tl.part_first = g.part_first;
    const long long T = (long long)tiles_m_ * tiles_n_;
    const long long blocks = g.tail_S > 1 ? g.full_tiles + (T - g.full_tiles) * g.tail_S : T;
    hipLaunchKernelGGL(wino_gemm_fused_kernel, dim3((unsigned)blocks), dim3(256), lds_f, stream, U, im, g.Cg, g.rows_p, tiles_m_,
                       (unsigned)(16ull * g.Cg * 2 * g.rows_p * 8), ep, tl);
    if (g.tail_S > 1) {
      if (int e = launch_status()) return e;
      WinoTailReduce r;
      r.part = tl.part; r.out = out; r.bias = bias; r.mask = mask; r.alpha = alpha; r.beta = beta; r.relu = relu;
      r.S = g.tail_S; r.Ko = g.Ko; r.P = g.P; r.Q = g.Q; r.TP = g.TP; r.TQ = g.TQ; r.tiles_m = tiles_m_; r.full = g.full_tiles;
      r.first = (unsigned)g.part_first; r.total = (unsigned)((long long)g.N * g.Ko * g.P * g.Q);
      r.slab_elems = g.slab_elems;
      r.dPQ = FastDiv((uint32_t)(g.P * g.Q)); r.dQ = FastDiv((uint32_t)g.Q); r.dKo = FastDiv((uint32_t)g.Ko);
      hipLaunchKernelGGL(wino_tail_reduce_kernel, dim3(cdiv((unsigned)g.slab_elems, 256u)), dim3(256), 0, stream, r);
    }
    return launch_status();
  }
  constexpr size_t lds_bytes = (size_t)kWinoR * kWinoStage;
  static_assert(lds_bytes <= 160 * 1024, "the ring does not fit the 160 KB LDS of a CU");
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&wino_gemm_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (attr != hipSuccess) return (int)attr;
  const int tiles_m = g.rows_p / kWinoBM;
  const long long tiles_n = g.tiles_p / kWinoBN;
  // work: the multiply-adds this form executes, 16 per tile, filter and channel (the direct form's 9 per pixel are
  // 2.25 times as many where the tiles cover the image exactly)
  ProfScope prof(tag, 2.0 * 16.0 * (double)g.Ko * g.Ci * (double)g.tiles, stream);
  hipLaunchKernelGGL(wino_gemm_kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), lds_bytes, stream, U, V, g.Cg, g.rows_p,
                     (unsigned)g.tiles_p, tiles_m, (unsigned)(16ull * g.Cg * 2 * g.rows_p * 8),
                     (unsigned)(16ull * g.Cg * 2 * g.tiles_p * 8), ep);
  return launch_status();
}

WinoFilterPlan plan_wino_bwd_filter(const ConvDims& d) {
  WinoFilterPlan p;
  p.ok = false;
  if (!wino_shape(d) || d.P <= 0 || d.Q <= 0) return p;
  p.TP = cdiv(d.P, 2); p.TQ = cdiv(d.Q, 2);
  p.tiles = (long long)d.N * p.TP * p.TQ;
  p.Kp = round_up(d.K, kWinoBM); p.Cp = round_up(d.C, kWinoBN);
  const long long tiles_mc = (long long)(p.Kp / kWinoBM) * (p.Cp / kWinoBN);
  const long long stages_all = (p.tiles + 3) / 4;
  // slices: the count (64 at most, 32 stages a slice at least, 128 MB of partial sums at most) that fills the 256 CUs
  // best in whole rounds, the smaller one on a tie
  int best = 1;
  double best_fill = 0.0;
  const long long slice_bytes = 4ll * 16 * p.Kp * p.Cp;
  for (int S = 1; S <= 64 && (S == 1 || (stages_all / S >= 32 && slice_bytes * S <= (128ll << 20))); ++S) {
    const long long blocks = tiles_mc * S;
    const double fill = (double)blocks / (double)(cdiv<long long>(blocks, 256) * 256);
    if (fill > best_fill + 1e-9) { best_fill = fill; best = S; }
  }
  p.S = best;
  p.stages = (int)cdiv<long long>(stages_all, p.S);
  p.TGs = (long long)p.S * p.stages;
  const unsigned long long vb = 16ull * p.TGs * 2 * p.Cp * 8, yb = 16ull * p.TGs * 4 * p.Kp;
  const unsigned long long pb = 4ull * p.S * 16 * p.Kp * p.Cp;
  p.vt_bytes = align256((size_t)vb); p.dyt_bytes = align256((size_t)yb); p.part_bytes = align256((size_t)pb);
  p.ok = vb < (1ull << 31) && yb < (1ull << 31) && pb < (1ull << 31) && p.TGs * 4 < (1ll << 30);
  return p;
}

int launch_conv_wino_bwd_filter(const ConvDims& d, const WinoFilterPlan& p, const float* x, const float* dy, float* dw, float alpha,
                                float beta, void* ws, hipStream_t stream) {
  if (!p.ok) return RH_E_UNSUPPORTED;
  char* base = static_cast<char*>(ws);
  float* Vt = reinterpret_cast<float*>(base);
  float* dyt = reinterpret_cast<float*>(base + p.vt_bytes);
  float* part = reinterpret_cast<float*>(base + p.vt_bytes + p.dyt_bytes);
  {
    WinoFilterPrepArgs a;
    a.x = x; a.dy = dy; a.Vt = Vt; a.dyt = dyt;
    a.x_bytes = (unsigned)(4ull * d.x_elems); a.dy_bytes = (unsigned)(4ull * d.y_elems);
    a.N = d.N; a.C = d.C; a.H = d.H; a.W = d.W; a.K = d.K; a.P = d.P; a.Q = d.Q; a.halo = d.pad;
    a.Kp = p.Kp; a.Cp = p.Cp; a.TGs = (int)p.TGs; a.tiles = (unsigned)p.tiles;
    a.dTQ = FastDiv((uint32_t)p.TQ); a.dTP = FastDiv((uint32_t)p.TP);
    a.dPairs = FastDiv((uint32_t)(p.TGs * 2)); a.dKp = FastDiv((uint32_t)(p.TGs * 4));   // (dKp: tiles, the divisor of the dy items)
    const unsigned long long vi = (unsigned long long)(p.Cp / 2) * (p.TGs * 2), yi = (unsigned long long)p.TGs * 4 * p.Kp;
    if (vi >= (1ull << 31) || yi >= (1ull << 31)) return RH_E_LIMIT;
    a.v_items = (unsigned)vi; a.y_items = (unsigned)yi;
    a.v_blocks = (unsigned)cdiv<unsigned long long>(vi, 256);
    ProfScope prof("wino_filter_prep", 4.0 * ((double)d.x_elems + (double)d.y_elems) + 128.0 * (double)p.TGs * p.Cp + 16.0 * (double)yi, stream);
    hipLaunchKernelGGL(wino_filter_prep_kernel, dim3(a.v_blocks + (unsigned)cdiv<unsigned long long>(yi, 256)), dim3(256), 0, stream, a);
    if (int e = launch_status()) return e;
  }
  WinoFilterArgs a;
  a.Vt = Vt; a.dyt = dyt; a.part = part;
  a.vt_bytes = (unsigned)(16ull * p.TGs * 2 * p.Cp * 8); a.dyt_bytes = (unsigned)(16ull * p.TGs * 4 * p.Kp);
  a.part_bytes = (unsigned)(4ull * p.S * 16 * p.Kp * p.Cp);
  a.Kp = p.Kp; a.Cp = p.Cp; a.TGs = (int)p.TGs;
  a.tiles_m = p.Kp / kWinoBM; a.tiles_c = p.Cp / kWinoBN; a.stages = p.stages;
  constexpr size_t lds_b = (size_t)kWinoR * kWinoStage + 2 * (size_t)kWinoFRaw;
  static_assert(lds_b <= 160 * 1024, "ring and tap slots do not fit the 160 KB LDS of a CU");
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&wino_bwd_filter_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_b);
  if (attr != hipSuccess) return (int)attr;
  {
    ProfScope prof("conv_bwd_filter_wino", 2.0 * 16.0 * (double)d.K * d.C * (double)p.tiles, stream);
    hipLaunchKernelGGL(wino_bwd_filter_kernel, dim3((unsigned)(a.tiles_m * a.tiles_c * p.S)), dim3(256), lds_b, stream, a);
    if (int e = launch_status()) return e;
  }
  ProfScope prof("wino_filter_reduce", 4.0 * (16.0 * p.S + 9.0) * (double)d.K * d.C, stream);
  hipLaunchKernelGGL(wino_filter_reduce_kernel, dim3(cdiv((unsigned)(d.K * d.C), 256u)), dim3(256), 0, stream, part, p.S, d.K, d.C,
                     p.Kp, p.Cp, alpha, beta, dw);
  return launch_status();
}

}  // namespace rh

using namespace rh;

extern "C" double rh_conv2d_winograd_flops(const rh_conv_geom* g, int pass, int flags) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0.0;
  if (flags & (RH_MATH_BF16_MFMA_FP32ACC | RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT)) return 0.0;
  if (wino_shape5(d) && pass == RH_CONV_FWD) {
    const WinoGeom wg = wino_geom_fwd5(d);
    if (!(flags & RH_ALGO_WINOGRAD ? wg.ok : wino_pays5(wg))) return 0.0;
    return 2.0 * 16.0 * (double)wg.Ko * wg.Ci * (double)wg.tiles;
  }
  if (!wino_shape(d)) return 0.0;
  if (pass == RH_CONV_BWD_FILTER) {
    const WinoFilterPlan wp = plan_wino_bwd_filter(d);
    if (!(flags & RH_ALGO_WINOGRAD ? wp.ok : wino_filter_pays(d, wp))) return 0.0;
    return 2.0 * 16.0 * (double)d.K * d.C * (double)wp.tiles;
  }
  if (pass != RH_CONV_FWD && pass != RH_CONV_BWD_DATA) return 0.0;
  const WinoGeom wg = pass == RH_CONV_FWD ? wino_geom_fwd(d) : wino_geom_bwd_data(d);
  if (!(flags & RH_ALGO_WINOGRAD ? wg.ok : wino_pays(wg))) return 0.0;
  return 2.0 * 16.0 * (double)wg.Ko * wg.Ci * (double)wg.tiles;
}

