// Convolution backward-filter (K5) and backward-bias (K6).
//   dw[ko][(c,r,s)] = sum_{n,p,q} dy[n][ko][p][q] * x[n][c][p*st+r-pad][q*st+s-pad]
// The contraction runs over up to N*P*Q = 774 400 pixels while the result is small, so the
// pixel range is cut into `splits` contiguous slices computed by different blocks; each slice
// writes its partial filter gradient to scratch and a second kernel adds the slices in a fixed
// order (results do not depend on scheduling).
#include "conv_common.h"

namespace rh {

struct BwdFilterPlan {
  int bm, bn, tiles, splits;
  size_t tab_bytes, part_bytes;
};

static BwdFilterPlan plan_bwd_filter(const ConvDims& d) {
  BwdFilterPlan p;
  const int CRS = d.C * d.R * d.S;
  p.bm = pick_bm(d.K);
  p.bn = p.bm == 128 ? 128 : 256;
  p.tiles = cdiv(d.K, p.bm) * cdiv(CRS, p.bn);
  const long long M = (long long)d.N * d.P * d.Q;
  const int k_chunks = (int)cdiv<long long>(M, 16);
  // One full co-resident set of blocks (256 CUs x 3 blocks of this kernel per CU) and no partial
  // second round: a block that runs alone on its CU uses the matrix pipe less well than three
  // sharing it, so a ragged tail costs more than its share.  Every slice keeps at least 32 K
  // steps so the prologue and the partial-sum traffic stay small next to the contraction.
  const int slots = 256 * 3;
  int want = slots / p.tiles;
  const int max_by_depth = k_chunks / 32 > 0 ? k_chunks / 32 : 1;
  if (want > max_by_depth) want = max_by_depth;
  if (want > 256) want = 256;
  if (want < 1) want = 1;
  p.splits = want;
  p.tab_bytes = align256(sizeof(int4) * (size_t)round_up(CRS, kTabPad));
  p.part_bytes = align256(sizeof(float) * (size_t)p.splits * d.K * CRS);
  return p;
}

// Second pass of a split contraction: out[i*ld + j] = alpha * sum_s part[s][i*cols + j] + beta*out.
__global__ void split_reduce_kernel(const float* __restrict__ part, int splits, long long split_stride,
                                    float* __restrict__ out, int rows, int cols, int ld, float alpha,
                                    float beta) {
  const long long total = (long long)rows * cols;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    float acc = 0.0f;
    for (int s = 0; s < splits; ++s) acc += part[(long long)s * split_stride + idx];
    const int i = (int)(idx / cols), j = (int)(idx - (long long)i * cols);
    float* dst = out + (size_t)i * ld + j;
    float val = alpha * acc;
    if (beta != 0.0f) val += beta * *dst;
    *dst = val;
  }
}

void launch_split_reduce(const float* part, int splits, long long split_stride, float* out, int rows, int cols,
                         int ld, float alpha, float beta, hipStream_t stream) {
  const size_t total = (size_t)rows * cols;
  ProfScope prof("split_reduce", 4.0 * (double)total * (splits + 1), stream);
  hipLaunchKernelGGL(split_reduce_kernel, dim3(stream_grid(total, 256)), dim3(256), 0, stream, part, splits,
                     split_stride, out, rows, cols, ld, alpha, beta);
}

template <class T>
static int run_bwd_filter(const PixDyParams& ap, const PixXParams& bp, const EpiParams& ep, int M,
                          int splits, int* used, hipStream_t stream, const char* tag) {
  typedef LoadPixDy<T::BM, T::BK, T::NT> AL;
  typedef LoadPixX<T::BN, T::BK, T::NT> BL;
  return launch_mfma_gemm<T, AL, BL, false>(ap, bp, ep, M, splits, used, stream, tag);
}

// db[k] = alpha * sum_{n, i<plane} dy[(n*K + k)*plane + i] + beta * db[k]; one block per k.
__global__ __launch_bounds__(1024) void bwd_bias_kernel(const float* __restrict__ dy, int N, int K,
                                                        int plane, float alpha, float beta,
                                                        float* __restrict__ db) {
  const int k = blockIdx.x;
  float acc = 0.0f;
  const long long total = (long long)N * plane;
  for (long long t = threadIdx.x; t < total; t += blockDim.x) {
    const int n = (int)(t / plane);
    const int i = (int)(t - (long long)n * plane);
    acc += dy[((size_t)n * K + k) * plane + i];
  }
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
  __shared__ float part[16];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) s += part[i];
    float v = alpha * s;
    if (beta != 0.0f) v += beta * db[k];
    db[k] = v;
  }
}

// plane == 1 (affine): dy is [N][K]; one thread per k walks the batch, coalesced across k.
__global__ void bwd_bias_rows_kernel(const float* __restrict__ dy, int N, int K, float alpha,
                                     float beta, float* __restrict__ db) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= K) return;
  float acc = 0.0f;
  for (int n = 0; n < N; ++n) acc += dy[(size_t)n * K + k];
  float v = alpha * acc;
  if (beta != 0.0f) v += beta * db[k];
  db[k] = v;
}

}  // namespace rh

using namespace rh;

extern "C" size_t rh_conv2d_workspace_bytes(const rh_conv_geom* g, int pass) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  const int CRS = d.C * d.R * d.S, KRS = d.K * d.R * d.S;
  switch (pass) {
    case RH_CONV_FWD:
      return align256(sizeof(int4) * (size_t)round_up(CRS, kTabPad));
    case RH_CONV_BWD_DATA:
      return align256(sizeof(int4) * (size_t)round_up(KRS, kTabPad)) +
             align256(sizeof(int) * (size_t)round_up(KRS, kTabPad));
    case RH_CONV_BWD_FILTER: {
      const BwdFilterPlan p = plan_bwd_filter(d);
      return p.tab_bytes + p.part_bytes;
    }
    default:
      return 0;
  }
}

extern "C" int rh_conv2d_bwd_filter(const rh_conv_geom* g, float alpha, const float* x, const float* dy,
                                    float beta, float* dw, void* ws, size_t ws_bytes, int flags,
                                    rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!x || !dy || !dw) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  const BwdFilterPlan plan = plan_bwd_filter(d);
  if (!ws || ws_bytes < plan.tab_bytes + plan.part_bytes || (reinterpret_cast<uintptr_t>(ws) & 255))
    return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  const int CRS = d.C * d.R * d.S;
  const int M = d.N * d.P * d.Q;
  int4* tab = static_cast<int4*>(ws);
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + plan.tab_bytes);
  launch_build_fwd_tab(tab, round_up(CRS, kTabPad), CRS, d.R, d.S, d.H * d.W, d.W, stream);
  if (int e = launch_status()) return e;

  PixDyParams ap;
  ap.ptr = dy; ap.bytes = (uint32_t)(d.y_elems * 4); ap.rows = d.K; ap.M = M; ap.PQ = d.P * d.Q;
  PixXParams bp;
  bp.ptr = x; bp.bytes = (uint32_t)(d.x_elems * 4); bp.rows = CRS; bp.M = M; bp.PQ = d.P * d.Q; bp.Q = d.Q;
  bp.img_stride = d.C * d.H * d.W; bp.H = d.H; bp.W = d.W; bp.st = d.st; bp.pad = d.pad; bp.rtab = tab;
  EpiParams ep;
  ep.out = part; ep.bias = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
  ep.rows = d.K; ep.cols = CRS; ep.inner = 0; ep.ld = CRS; ep.relu = 0;
  ep.split_stride = (long long)d.K * CRS;

  int used = 1, e = 0;
  if (M == 0) {
    used = 0;
  } else {
    switch (plan.bm) {
      case 128: e = run_bwd_filter<T128x128>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_128x128"); break;
      case 96:  e = run_bwd_filter<T96x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x256"); break;
      case 64:  e = run_bwd_filter<T64x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_64x256"); break;
      default:  e = run_bwd_filter<T32x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_32x256"); break;
    }
    if (e) return e;
  }
  launch_split_reduce(part, used, (long long)d.K * CRS, dw, d.K, CRS, CRS, alpha, beta, stream);
  return launch_status();
}

extern "C" int rh_conv2d_bwd_bias(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy,
                                  float beta, float* db, rh_stream_t stream_) {
  if (N <= 0 || K <= 0 || plane <= 0 || !dy || !db) return RH_E_INVALID;
  hipStream_t stream = to_stream(stream_);
  ProfScope prof("bwd_bias", 4.0 * (double)N * K * plane, stream);
  if (plane == 1) {
    hipLaunchKernelGGL(bwd_bias_rows_kernel, dim3(cdiv(K, 256)), dim3(256), 0, stream, dy, N, K, alpha, beta,
                       db);
  } else {
    hipLaunchKernelGGL(bwd_bias_kernel, dim3(K), dim3(1024), 0, stream, dy, N, K, plane, alpha, beta, db);
  }
  return launch_status();
}
