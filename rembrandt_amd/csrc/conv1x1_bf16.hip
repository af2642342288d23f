// 1x1 / stride 1 / unpadded convolution on packed bf16 activations (a forward-only chain's "cccp" layers):
//   yp[n][h + halo][ko/8][w + halo][ko%8] = bf16( act( sum_c w[ko][c] * xp[n][h][c/8][w][c%8] + bias[ko] ) ).
// Such a layer moves 2 bytes per element each way for 2*C FLOPs per output element: at bf16 matrix rates it is a copy
// with a contraction riding along, so the kernel is shaped like one.  In the packed layout the image operand of
// v_mfma_f32_32x32x16_bf16 (lane = pixel, eight consecutive channels of one half of the 16-k step) is one 16-byte load
// per lane from global memory straight into the operand register, consecutive lanes on consecutive 16-byte groups; the
// result's four consecutive channels per lane and the four of the lane 32 away make one 16-byte group, exchanged between
// the two halves of the wave so that every lane stores 16 bytes and every store instruction writes two runs of 512.  The filter (a block's share: at most 128 x 256, 64 KB as bf16) is staged
// once per block in LDS, already in operand order; a wave takes 32-pixel column tiles on its own and the image never
// touches LDS.  Accumulation runs over k in ascending 16-k steps from zero, as in the tiled kernels: the same bits.
#include "conv_common.h"

namespace rh {

struct C1x1bArgs {
  const void* x; uint32_t x_bytes;
  void* y;
  const uint4* wb;     // converted filter [C/8][K] of 16-byte groups
  const float* bias;   // may be null
  int M, K, relu;
  int W, in_img_groups, in_cg_stride;                  // input: halo 0; group (n, h, cg, w) at n*img + (h*Cg + cg)*W + w
  int out_halo, out_Wp, out_img_groups, out_row_groups;  // output: group (n, h, cg, w) at n*img + (h+halo)*row + cg*Wp + w + halo
  FastDiv dHW, dW;
  int tiles, tiles_per_block;
};

template <int TM, int KS>
__global__ __launch_bounds__(256) void conv1x1_bf16_stream_kernel(C1x1bArgs a) {
  extern __shared__ float lds_dyn[];
  uint4* const sA = reinterpret_cast<uint4*>(lds_dyn);                    // [TM][KS][64]
  float* const sBias = reinterpret_cast<float*>(sA + TM * KS * 64);       // [TM * 32]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, col = lane & 31;
  // blockIdx.y: which TM*32 output channels this block computes (layers of more than 128: the image is then read once
  // per chunk, the later reads from the L2 the first one filled)
  const int k0 = blockIdx.y * (TM * 32);
  for (int e = tid; e < TM * KS * 64; e += 256) {
    const int l = e & 63, t = e >> 6, ks = t % KS, i = t / KS;
    sA[e] = a.wb[(size_t)(2 * ks + (l >> 5)) * a.K + k0 + 32 * i + (l & 31)];
  }
  for (int e = tid; e < TM * 32; e += 256) sBias[e] = a.bias ? a.bias[k0 + e] : 0.0f;
  __syncthreads();

  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(a.x, a.x_bytes);
  const int t_begin = blockIdx.x * a.tiles_per_block;
  int t_end = t_begin + a.tiles_per_block;
  if (t_end > a.tiles) t_end = a.tiles;
  char* const ybase = static_cast<char*>(a.y);
  const int cg_step = 2 * a.in_cg_stride * 16;   // bytes between the channel groups of consecutive 16-k steps
  // A wave's tiles, with the image operand of the next tile requested before the current one is multiplied.
  auto tile_base = [&](int t, bool& valid, uint32_t& n, uint32_t& h, uint32_t& w) -> uint32_t {
    const int m = t * 32 + col;
    valid = m < a.M;
    uint32_t r;
    a.dHW.divmod((uint32_t)(valid ? m : 0), n, r);
    a.dW.divmod(r, h, w);
    return valid ? ((uint32_t)((int)n * a.in_img_groups + (int)h * (KS * 2) * a.in_cg_stride + (int)w) +
                    (uint32_t)(half * a.in_cg_stride)) * 16u
                 : 0x80000000u;
  };
  int t = t_begin + wave;
  if (t >= t_end) return;
  bool valid, valid_next = false;
  uint32_t n, h, w, n2 = 0, h2 = 0, w2 = 0;
  constexpr bool AHEAD = KS <= 8;   // (deeper contractions: the second operand set would cost a wave per SIMD)
  uint4 b[KS], bn[AHEAD ? KS : 1];
  {
    const uint32_t vbase = tile_base(t, valid, n, h, w);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      b[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vbase, ks * cg_step, 0));
  }
  for (; t < t_end; t += 4) {
    const bool more = t + 4 < t_end;
    if (AHEAD && more) {
      const uint32_t vbase = tile_base(t + 4, valid_next, n2, h2, w2);
#pragma unroll
      for (int ks = 0; ks < (AHEAD ? KS : 0); ++ks)
        bn[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vbase, ks * cg_step, 0));
    }
    f32x16 acc[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, sA[(i * KS + ks) * 64 + lane]),
                                                         __builtin_bit_cast(bf16x8_t, b[ks]), acc[i], 0, 0, 0);
    // Epilogue.  A lane holds four consecutive channels of its pixel per group of eight, the other four sit in the lane
    // 32 away: the halves of two neighbouring groups are exchanged (v_permlane32_swap), after which lanes 0-31 hold
    // the whole 16-byte group of the even one and lanes 32-63 that of the odd one, and every lane stores 16 bytes.
    {
      char* const yo = ybase + ((size_t)n * a.out_img_groups + (size_t)((int)h + a.out_halo) * a.out_row_groups +
                                (size_t)((int)w + a.out_halo)) * 16;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int vp = 0; vp < 2; ++vp) {
          uint2 o[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int vg = 2 * vp + u;
            const float4 bs = *reinterpret_cast<const float4*>(sBias + 32 * i + 8 * vg + 4 * half);
            float v0 = acc[i][4 * vg] + bs.x, v1 = acc[i][4 * vg + 1] + bs.y, v2 = acc[i][4 * vg + 2] + bs.z,
                  v3 = acc[i][4 * vg + 3] + bs.w;
            if (a.relu) {
              v0 = v0 > 0.0f ? v0 : 0.0f; v1 = v1 > 0.0f ? v1 : 0.0f; v2 = v2 > 0.0f ? v2 : 0.0f; v3 = v3 > 0.0f ? v3 : 0.0f;
            }
            o[u].x = pack_bf16(v0, v1);
            o[u].y = pack_bf16(v2, v3);
          }
          const auto sx = __builtin_amdgcn_permlane32_swap(o[0].x, o[1].x, false, false);
          const auto sy = __builtin_amdgcn_permlane32_swap(o[0].y, o[1].y, false, false);
          uint4 q;
          q.x = sx[0]; q.y = sy[0]; q.z = sx[1]; q.w = sy[1];
          if (valid) *reinterpret_cast<uint4*>(yo + (size_t)(k0 / 8 + 4 * i + 2 * vp + half) * a.out_Wp * 16) = q;
        }
    }
    if (AHEAD && more) {
#pragma unroll
      for (int ks = 0; ks < (AHEAD ? KS : 0); ++ks) b[ks] = bn[ks];
      valid = valid_next; n = n2; h = h2; w = w2;
    } else if (more) {
      const uint32_t vbase = tile_base(t + 4, valid, n, h, w);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        b[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vbase, ks * cg_step, 0));
    }
  }
}

template <int TM, int KS>
static int launch_c1x1b(const C1x1bArgs& a, int blocks, int chunks, hipStream_t stream) {
  const size_t lds = (size_t)TM * KS * 64 * 16 + (size_t)TM * 32 * 4;
  if (lds > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&conv1x1_bf16_stream_kernel<TM, KS>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) return (int)attr;
  }
  hipLaunchKernelGGL((conv1x1_bf16_stream_kernel<TM, KS>), dim3((unsigned)blocks, (unsigned)chunks), dim3(256), lds, stream, a);
  return launch_status();
}

template <int TM>
static int launch_c1x1b_ks(int ks, const C1x1bArgs& a, int blocks, int chunks, hipStream_t stream) {
  switch (ks) {
    case 2: return launch_c1x1b<TM, 2>(a, blocks, chunks, stream);
    case 4: return launch_c1x1b<TM, 4>(a, blocks, chunks, stream);
    case 6: return launch_c1x1b<TM, 6>(a, blocks, chunks, stream);
    case 8: return launch_c1x1b<TM, 8>(a, blocks, chunks, stream);
    case 16: return launch_c1x1b<TM, 16>(a, blocks, chunks, stream);
    default: return RH_E_UNSUPPORTED;
  }
}

// Output channels per block: the largest of 128, 96, 64, 32 that divides K.
static int c1x1b_rows(int K) { return K % 128 == 0 ? 128 : K % 96 == 0 ? 96 : K % 64 == 0 ? 64 : 32; }

// Layers this kernel takes: 1x1, stride 1, no padding, a packed result, C in {32, 64, 96, 128}, 32 | K <= 128.  (The
// kernel also runs 256 input channels and two chunks of output channels, and the tests cover that, but there the tiled
// kernel is the faster one: 256 -> 256 channels on 27 x 27 at batch 128 takes 0.047 ms here, 0.041 ms on the tiles: with
// a 64 KB filter share per block two blocks fit a CU, too few waves for a kernel that lives on loads in flight.)
bool conv1x1_bf16_stream_runs(const ConvDims& d) {
  if (!(d.R == 1 && d.S == 1 && d.st == 1 && d.pad == 0 && d.K % 32 == 0 && (long long)d.N * d.H * d.W < (1ll << 31) - 64))
    return false;
  if (!(d.C == 32 || d.C == 64 || d.C == 96 || d.C == 128 || d.C == 256)) return false;
  return d.K / c1x1b_rows(d.K) <= 2;
}
bool conv1x1_bf16_stream_applies(const ConvDims& d) { return conv1x1_bf16_stream_runs(d) && d.C <= 128 && d.K <= 128; }

// xp: packed input (halo 0); wb: the filter copy of the converted filter (its table is not needed: the contraction is
// the channel index); pk: the packed result.  bias may be null.
int launch_conv1x1_bf16_stream(const ConvDims& d, const void* xp, const void* wb, const float* bias, int relu,
                               const PackedOut& pk, hipStream_t stream) {
  C1x1bArgs a;
  a.x = xp; a.x_bytes = (uint32_t)(2 * (size_t)d.N * d.C * d.H * d.W);
  a.y = pk.ptr; a.wb = static_cast<const uint4*>(wb); a.bias = bias; a.relu = relu;
  a.M = d.N * d.H * d.W; a.K = d.K;
  a.W = d.W; a.in_cg_stride = d.W; a.in_img_groups = d.H * (d.C / 8) * d.W;
  a.out_halo = pk.halo; a.out_Wp = pk.Wp; a.out_row_groups = pk.Cg * pk.Wp; a.out_img_groups = pk.img_groups;
  a.dHW = FastDiv((uint32_t)(d.H * d.W)); a.dW = FastDiv((uint32_t)d.W);
  a.tiles = cdiv(a.M, 32);
  // A block's tiles are one contiguous range that its four waves take in turn: a multiple of four per block, so that
  // the waves of a block carry the same number, and blocks of two tiles per wave while the GPU holds them all at once.
  a.tiles_per_block = 4 * (int)cdiv<long long>(a.tiles, 4ll * 2048) ;
  if (a.tiles_per_block < 8 && a.tiles >= 8 * 256) a.tiles_per_block = 8;
  const int blocks = cdiv(a.tiles, a.tiles_per_block);
  ProfScope prof("conv_fwd_bf16s_1x1", 2.0 * (double)d.K * (double)a.M * (double)d.C, stream);
  const int rows = c1x1b_rows(d.K), chunks = d.K / rows;
  switch (rows / 32) {
    case 1: return launch_c1x1b_ks<1>(d.C / 16, a, blocks, chunks, stream);
    case 2: return launch_c1x1b_ks<2>(d.C / 16, a, blocks, chunks, stream);
    case 3: return launch_c1x1b_ks<3>(d.C / 16, a, blocks, chunks, stream);
    case 4: return launch_c1x1b_ks<4>(d.C / 16, a, blocks, chunks, stream);
    default: return RH_E_UNSUPPORTED;
  }
}

}  // namespace rh
