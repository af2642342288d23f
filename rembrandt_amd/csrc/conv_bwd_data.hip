// Convolution backward-data (K7) as an implicit GEMM over the transposed filter:
//   dx[n][c][h][w] = sum_{ko,r,s} w[ko][c][r][s] * dy[n][ko][(h+pad-r)/st][(w+pad-s)/st]
// rows = input channels c (filter read through a k -> offset table), cols = input pixels
// (dy gathered; a term exists only when both divisions are exact and land inside P x Q).
#include "conv_common.h"

namespace rh {

__global__ void build_bwd_data_tab_kernel(int4* tab, int* atab, int n_entries, int KRS, int C, int R,
                                          int S, int PQ, int Q, int st) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n_entries) return;
  if (k < KRS) {
    const int ko = k / (R * S), rs = k - ko * (R * S), r = rs / S, s = rs - r * S;
    const int rq = r / st, rr = r - rq * st, sq = s / st, sr = s - sq * st;
    tab[k] = make_int4(ko * PQ - rq * Q - sq, -rq, -sq, rr * st + sr);
    atab[k] = ko * C * R * S + r * S + s;
  } else {
    tab[k] = make_int4(0, -(1 << 28), 0, -1);
    atab[k] = -1;
  }
}

// Scalar-offset path (stride 1): wT[k][c] = w[ko][c][r][s] for k = (ko,r,s) (zero rows past the end) and
// the k -> byte offset table into the padded dy, soff[k] = 4*(ko*Pp*Qp + (R-1-r)*Qp + (S-1-s)).
__global__ void prep_bwd_data_soff_kernel(const float* __restrict__ w, float* __restrict__ wT, int* __restrict__ soff,
                                          int n_k, int KRS, int C, int R, int S, int PpQp, int Qp) {
  const long long total = (long long)n_k * C;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int k = (int)(i / C), c = (int)(i - (long long)k * C);
    float v = 0.0f;
    int off = 0;
    if (k < KRS) {
      const int ko = k / (R * S), rs = k - ko * (R * S), r = rs / S, s2 = rs - r * S;
      v = w[((size_t)ko * C + c) * (R * S) + rs];
      off = (ko * PpQp + (R - 1 - r) * Qp + (S - 1 - s2)) * 4;
    }
    wT[i] = v;
    if (c == 0) soff[k] = off;
  }
}

template <class T>
static int run_bwd_data_soff(const RowSParams& ap, const RowSParams& bp, EpiParams ep, int n_k, int k_true,
                             hipStream_t stream, const char* tag, int splits, float* part) {
  constexpr int AROWS = T::BM % 64 == 0 ? T::BM : (T::BM + 63) / 64 * 64;
  typedef LoadRowS<AROWS, T::BK, T::NT, true> AL;
  typedef LoadRowS<T::BN, T::BK, T::NT, false> BL;
  if (splits <= 1) return launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, n_k, 1, nullptr, stream, tag, k_true);
  // slices of the contraction write unblended partial results; one reduction applies the alpha / beta blend
  const EpiParams fin = ep;
  const long long total = (long long)ep.rows * ep.cols;
  ep.out = part; ep.split_stride = total;
  int used = 1;
  if (int e = launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, n_k, splits, &used, stream, tag, k_true)) return e;
  launch_split_reduce_nchw(part, used, total, fin.out, total, fin.inner, fin.rows, fin.alpha, fin.beta, nullptr, 0, stream);
  return launch_status();
}

template <class T>
static int run_bwd_data(int KRS, const DenseParams& ap, const GatherParams& bp, const EpiParams& ep,
                        hipStream_t stream, const char* tag) {
  typedef LoadDenseK<T::BM, T::BK, T::NT, true> AL;
  typedef LoadGatherR<T::BN, T::BK, T::NT, true> BL;
  return launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, KRS, 1, nullptr, stream, tag);
}

}  // namespace rh

using namespace rh;

extern "C" int rh_conv2d_bwd_data(const rh_conv_geom* g, float alpha, const float* w, const float* dy,
                                  float beta, float* dx, void* ws, size_t ws_bytes, int flags,
                                  rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!w || !dy || !dx) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  const size_t need = rh_conv2d_workspace_bytes(g, RH_CONV_BWD_DATA);
  if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  const int KRS = d.K * d.R * d.S;
  const SoffPlan sp = plan_soff_bwd_data(d);
  if (sp.ok && !(flags & RH_ALGO_GATHER)) {
    int* soff = static_cast<int*>(ws);
    float* wT = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes);
    const float* img = dy;
    if (sp.img_bytes) {
      float* dyp = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes);
      launch_pad_image(dy, dyp, (long long)d.N * d.K, d.P, d.Q, sp.Hp, sp.Wp, sp.halo, stream, d.st);
      if (int e = launch_status()) return e;
      img = dyp;
    }
    hipLaunchKernelGGL(prep_bwd_data_soff_kernel, dim3(stream_grid((size_t)sp.n_k * d.C, 256)), dim3(256), 0, stream, w,
                       wT, soff, sp.n_k, KRS, d.C, d.R, d.S, sp.Hp * sp.Wp, sp.Wp);
    if (int e = launch_status()) return e;
    RowSParams ap;  // transposed filter [k][c]
    ap.ptr = wT; ap.bytes = (uint32_t)(sizeof(float) * (size_t)sp.n_k * d.C);
    ap.M = d.C; ap.inner = d.C; ap.innerW = d.C; ap.img_stride = 0; ap.a_stride = 0; ap.b_stride = 1;
    ap.soff = nullptr; ap.ldk4 = d.C * 4;
    RowSParams bp;  // padded dy, rows = input pixels
    bp.ptr = img; bp.bytes = (uint32_t)(sizeof(float) * (size_t)d.N * d.K * sp.Hp * sp.Wp);
    bp.M = d.N * d.H * d.W; bp.inner = d.H * d.W; bp.innerW = d.W;
    bp.img_stride = d.K * sp.Hp * sp.Wp; bp.a_stride = sp.Wp; bp.b_stride = 1;
    bp.soff = soff; bp.ldk4 = 0;
    EpiParams ep;
    ep.out = dx; ep.bias = nullptr; ep.alpha = alpha; ep.beta = beta;
    ep.rows = d.C; ep.cols = bp.M; ep.inner = d.H * d.W; ep.ld = 0; ep.relu = 0; ep.split_stride = 0;
    float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes + sp.img_bytes);
    switch (pick_bm(d.C)) {
      case 128: return run_bwd_data_soff<T128x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_128x128", sp.splits, part);
      case 96:  return run_bwd_data_soff<T96x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_96x128", sp.splits, part);
      case 64:
        if (cdiv(d.C, 64) == 1 && prefer_k8_64(ep.cols))
          return run_bwd_data_soff<T64x256k8>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_64x256k8", sp.splits, part);
        return run_bwd_data_soff<T64x256>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_64x256", sp.splits, part);
      default:  return run_bwd_data_soff<T32x256>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_32x256", sp.splits, part);
    }
  }
  const int n_tab = round_up(KRS, kTabPad);
  int4* tab = static_cast<int4*>(ws);
  int* atab = reinterpret_cast<int*>(static_cast<char*>(ws) + align256(sizeof(int4) * (size_t)n_tab));
  hipLaunchKernelGGL(build_bwd_data_tab_kernel, dim3(cdiv(n_tab, 256)), dim3(256), 0, stream, tab, atab,
                     n_tab, KRS, d.C, d.R, d.S, d.P * d.Q, d.Q, d.st);
  if (int e = launch_status()) return e;

  DenseParams ap;
  ap.ptr = w; ap.bytes = (uint32_t)(d.w_elems * 4); ap.rows = d.C; ap.K = KRS; ap.ld = d.R * d.S; ap.ktab = atab;
  GatherParams bp;
  bp.ptr = dy; bp.bytes = (uint32_t)(d.y_elems * 4);
  bp.M = d.N * d.H * d.W; bp.inner = d.H * d.W; bp.innerW = d.W;
  bp.img_stride = d.K * d.P * d.Q; bp.row_stride = d.Q; bp.st = d.st; bp.pad = d.pad;
  bp.Hlim = d.P; bp.Wlim = d.Q; bp.ktab = tab;
  EpiParams ep;
  ep.out = dx; ep.bias = nullptr; ep.alpha = alpha; ep.beta = beta;
  ep.rows = d.C; ep.cols = bp.M; ep.inner = d.H * d.W; ep.ld = 0; ep.relu = 0; ep.split_stride = 0;

  switch (pick_bm(d.C)) {
    case 128: return run_bwd_data<T128x128>(KRS, ap, bp, ep, stream, "conv_bwd_data_128x128");
    case 96:  return run_bwd_data<T96x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_96x256");
    case 64:  return run_bwd_data<T64x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_64x256");
    default:  return run_bwd_data<T32x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_32x256");
  }
}
