// 3x3 stride-1 convolutions by Winograd's minimal filtering F(2x2, 3x3): forward, and backward-data as the forward form
// of the flipped, transposed filter over dy (CudnnConvFwdOp / CudnnConvBwdDataOp of a 3x3 layer, src/operator/mod.rs).
//
//   Y = A^T [ (G g G^T) o (B^T d B) ] A      per 2x2 output tile, 4x4 input patch d, 3x3 filter g
//
// 16 multiplications per tile, filter and channel instead of 36: the contraction over the input channels becomes 16
// independent products  M_f (rows x tiles) = U_f (rows x channels) * V_f (channels x tiles),  f = 4i + j the position
// in the 4x4 transformed patch, 2.25 times fewer multiply-adds than the direct form.
//
// Three kernels:
//  * wino_prep_kernel (one launch, two kinds of blocks): U = G g G^T for every (row, channel) and V = B^T d B for every
//    (channel, tile), both in the operand order of the product kernel, zeros where the patch leaves the image, for
//    rows, channels and tiles that pad the operands to whole blocks;
//  * wino_gemm_kernel: a block of four waves owns 128 rows x 32 tiles for all 16 f; wave w holds rows 32w .. 32w+31 as
//    16 accumulator tiles of v_mfma_f32_32x32x2_f32 (256 accumulator registers, one wave per SIMD).  Both operands go
//    straight from memory to LDS (buffer_load_dwordx4 ... lds) into a ring of three stages of four channels each,
//    two stages ahead of the MFMAs; the one barrier of a stage stands in front of its last quarter of MFMAs;
//  * its epilogue: a lane's element e of the 16 accumulators is the whole 4x4 M of one (row, tile): A^T M A is 24
//    additions in registers, then alpha / beta, bias, ReLU or the mask of a folded ReLU backward, and the 2x2 pixels
//    go to the NCHW result (odd extents: the tile's pixels past the edge are dropped).
//
// Operand layout (floats):  U[f][cg][h][rows_p][2],  V[f][cg][h][tiles_p][2]  with channel = 4 cg + 2 h + j.  The MFMA
// takes A[row][k], B[k][col] with k = lane / 32: the half-wave h reads channel 4 cg + 2 h + j for the stage's MFMA j,
// one 8-byte LDS read per operand and stage and f, each half-wave reading 256 consecutive bytes.
#include "conv_common.h"

namespace rh {

WinoGeom wino_geom(int N, int Ci, int Hi, int Wi, int Ko, int halo) {
  WinoGeom g;
  g.N = N; g.Ci = Ci; g.Hi = Hi; g.Wi = Wi; g.Ko = Ko; g.halo = halo;
  g.P = Hi + 2 * halo - 2; g.Q = Wi + 2 * halo - 2;
  g.TP = g.P > 0 ? cdiv(g.P, 2) : 0; g.TQ = g.Q > 0 ? cdiv(g.Q, 2) : 0;
  g.tiles = (long long)N * g.TP * g.TQ;
  g.tiles_p = (g.tiles + kWinoBN - 1) / kWinoBN * kWinoBN;
  g.Cg = cdiv(Ci, 4);
  g.rows_p = round_up(Ko, kWinoBM);
  const unsigned long long ub = 16ull * g.Cg * 2 * (unsigned long long)g.rows_p * 8;
  const unsigned long long vb = 16ull * g.Cg * 2 * (unsigned long long)g.tiles_p * 8;
  g.u_bytes = align256((size_t)ub);
  g.v_bytes = align256((size_t)vb);
  // 32-bit byte offsets into U and V, 31-bit tile indices
  g.ok = g.P > 0 && g.Q > 0 && halo >= 0 && halo <= 2 && ub < (1ull << 31) && vb < (1ull << 31) && g.tiles_p < (1ll << 30);
  return g;
}

namespace {

struct WinoPrepArgs {
  const float* w; const float* x; float* U; float* V;
  int Ko, Ci, Cg, rows_p, bwd;
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

  // ---- epilogue: A^T M A per (row, tile), A^T = [1 1 1 0; 0 1 -1 -1] -------------------------------------------------
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
#pragma unroll
  for (int eb = 0; eb < 4; ++eb) {
    float y[4][2][2];
    uint32_t vo[4][2][2];
    float aux[4][2][2];   // mask values, or the old result
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int e = 4 * eb + e4, re = 8 * eb + e4;
      float s0[4], s1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s0[j] = acc[j][e] + acc[4 + j][e] + acc[8 + j][e];
        s1[j] = acc[4 + j][e] - acc[8 + j][e] - acc[12 + j][e];
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
      for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
        for (int ai = 0; ai < 2; ++ai)
#pragma unroll
          for (int bi = 0; bi < 2; ++bi)
            aux[e4][ai][bi] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(blend ? rout : rmask, (int)vo[e4][ai][bi], srow + (8 * eb + e4) * PQ * 4, 0));
    }
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
      for (int ai = 0; ai < 2; ++ai)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          float x = y[e4][ai][bi];
          if (blend) x = fmaf(ep.beta, aux[e4][ai][bi], x);
          x += bv[4 * eb + e4];
          if (ep.relu) x = fmaxf(x, 0.0f);
          if (masked && !blend) x = aux[e4][ai][bi] > 0.0f ? x : 0.0f;
          y[e4][ai][bi] = x;
        }
    if (masked && blend) {
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
        for (int ai = 0; ai < 2; ++ai)
#pragma unroll
          for (int bi = 0; bi < 2; ++bi) {
            const float mk = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rmask, (int)vo[e4][ai][bi], srow + (8 * eb + e4) * PQ * 4, 0));
            y[e4][ai][bi] = mk > 0.0f ? y[e4][ai][bi] : 0.0f;
          }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
      for (int ai = 0; ai < 2; ++ai)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, y[e4][ai][bi]), rout, (int)vo[e4][ai][bi],
                                                srow + (8 * eb + e4) * PQ * 4, 0);
  }
}

}  // namespace

// in: (N, Ci, Hi, Wi) with g.halo zeros around; w: the layer's filter (K, C, 3, 3): forward reads it as (Ko, Ci), the
// backward-data form (bwd) as (Ci, Ko) with flipped taps; out: (N, Ko, P, Q).  ws: g.total() bytes, 256-aligned.
int launch_conv_wino(const WinoGeom& g, bool bwd, const float* in, const float* w, float* out, float alpha, float beta,
                     const float* bias, int relu, const float* mask, void* ws, hipStream_t stream, const char* tag) {
  if (!g.ok) return RH_E_UNSUPPORTED;
  float* U = static_cast<float*>(ws);
  float* V = reinterpret_cast<float*>(static_cast<char*>(ws) + g.u_bytes);
  WinoPrepArgs a;
  a.w = w; a.x = in; a.U = U; a.V = V;
  a.Ko = g.Ko; a.Ci = g.Ci; a.Cg = g.Cg; a.rows_p = g.rows_p; a.bwd = bwd ? 1 : 0;
  a.Hi = g.Hi; a.Wi = g.Wi; a.halo = g.halo;
  a.tiles = (unsigned)g.tiles; a.tiles_p = (unsigned)g.tiles_p;
  a.x_bytes = (unsigned)(4ull * (unsigned long long)g.N * g.Ci * g.Hi * g.Wi);
  a.dRows = FastDiv((uint32_t)g.rows_p); a.dPairs = FastDiv((uint32_t)(g.tiles_p / 2));
  a.dTQ = FastDiv((uint32_t)g.TQ); a.dTP = FastDiv((uint32_t)g.TP);
  const unsigned long long fi = (unsigned long long)g.Cg * 2 * g.rows_p, ii = (unsigned long long)g.Cg * 2 * (g.tiles_p / 2);
  if (fi >= (1ull << 31) || ii >= (1ull << 31)) return RH_E_LIMIT;
  a.filt_items = (unsigned)fi; a.in_items = (unsigned)ii;
  a.in_blocks = (unsigned)cdiv<unsigned long long>(ii, 256);
  const unsigned filt_blocks = (unsigned)cdiv<unsigned long long>(fi, 256);
  {
    ProfScope prof("wino_transform", 4.0 * ((double)g.N * g.Ci * g.Hi * g.Wi + 9.0 * g.Ko * g.Ci) +
                                         128.0 * ((double)g.Cg * g.rows_p + (double)g.Cg * g.tiles_p), stream);
    hipLaunchKernelGGL(wino_prep_kernel, dim3(a.in_blocks + filt_blocks), dim3(256), 0, stream, a);
    if (int e = launch_status()) return e;
  }
  WinoEpi ep;
  ep.out = out; ep.bias = bias; ep.mask = mask; ep.alpha = alpha; ep.beta = beta; ep.relu = relu;
  ep.Ko = g.Ko; ep.P = g.P; ep.Q = g.Q; ep.tiles = (unsigned)g.tiles;
  ep.out_bytes = (unsigned)(4ull * (unsigned long long)g.N * g.Ko * g.P * g.Q);
  ep.dTQ = a.dTQ; ep.dTP = a.dTP;
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

}  // namespace rh
