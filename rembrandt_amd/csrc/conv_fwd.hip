// Convolution forward (K1) with optional fused bias (K2) and ReLU (K3) as an implicit GEMM:
//   y[n][ko][p][q] = sum_{c,r,s} w[ko][(c,r,s)] * x_gather[(c,r,s)][(n,p,q)]
// rows = output channels (weights, k contiguous), cols = output pixels (gathered, q contiguous).
#include "conv_common.h"

namespace rh {

__global__ void build_fwd_tab_kernel(int4* tab, int n_entries, int CRS, int R, int S, int HW, int W) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n_entries) return;
  if (k < CRS) {
    const int c = k / (R * S), rs = k - c * (R * S), r = rs / S, s = rs - r * S;
    tab[k] = make_int4(c * HW + r * W + s, r, s, 0);
  } else {
    tab[k] = make_int4(0, -(1 << 28), 0, -1);
  }
}

void launch_build_fwd_tab(int4* tab, int n_entries, int CRS, int R, int S, int HW, int W,
                          hipStream_t stream) {
  hipLaunchKernelGGL(build_fwd_tab_kernel, dim3(cdiv(n_entries, 256)), dim3(256), 0, stream, tab,
                     n_entries, CRS, R, S, HW, W);
}

template <class T>
static int run_fwd(const ConvDims& d, const DenseParams& ap, const GatherParams& bp,
                   const EpiParams& ep, hipStream_t stream, const char* tag) {
  typedef LoadDenseK<T::BM, T::BK, T::NT, false> AL;
  typedef LoadGatherR<T::BN, T::BK, T::NT, false> BL;
  return launch_mfma_gemm<T, AL, BL, true>(ap, bp, ep, d.C * d.R * d.S, 1, nullptr, stream, tag);
}

}  // namespace rh

using namespace rh;

extern "C" int32_t rh_conv2d_out_dim(int32_t in, int32_t size, int32_t stride, int32_t pad) {
  if (stride <= 0) return 0;
  return conv_out_dim(in, size, stride, pad);
}

extern "C" int rh_conv2d_fwd(const rh_conv_geom* g, float alpha, const float* x, const float* w,
                             float beta, float* y, const float* bias, void* ws, size_t ws_bytes,
                             int flags, rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!x || !w || !y) return RH_E_INVALID;
  if ((flags & RH_FUSE_BIAS) && !bias) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  if (d.y_elems == 0) return 0;
  const size_t need = rh_conv2d_workspace_bytes(g, RH_CONV_FWD);
  if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  const int CRS = d.C * d.R * d.S;
  const int n_tab = round_up(CRS, kTabPad);
  int4* tab = static_cast<int4*>(ws);
  launch_build_fwd_tab(tab, n_tab, CRS, d.R, d.S, d.H * d.W, d.W, stream);
  if (int e = launch_status()) return e;

  DenseParams ap;
  ap.ptr = w; ap.bytes = (uint32_t)(d.w_elems * 4); ap.rows = d.K; ap.K = CRS; ap.ld = CRS; ap.ktab = nullptr;
  GatherParams bp;
  bp.ptr = x; bp.bytes = (uint32_t)(d.x_elems * 4);
  bp.M = d.N * d.P * d.Q; bp.inner = d.P * d.Q; bp.innerW = d.Q;
  bp.img_stride = d.C * d.H * d.W; bp.row_stride = d.W; bp.st = d.st; bp.pad = d.pad;
  bp.Hlim = d.H; bp.Wlim = d.W; bp.ktab = tab;
  EpiParams ep;
  ep.out = y; ep.bias = (flags & RH_FUSE_BIAS) ? bias : nullptr; ep.alpha = alpha; ep.beta = beta;
  ep.rows = d.K; ep.cols = bp.M; ep.inner = d.P * d.Q; ep.ld = 0; ep.relu = (flags & RH_FUSE_RELU) ? 1 : 0;
  ep.split_stride = 0;

  switch (tile_override()) {
    case 1: return run_fwd<T128x256>(d, ap, bp, ep, stream, "conv_fwd_128x256");
    case 2: return run_fwd<T256x128>(d, ap, bp, ep, stream, "conv_fwd_256x128");
    case 3: return run_fwd<T128x128k32>(d, ap, bp, ep, stream, "conv_fwd_128x128k32");
    case 4: return run_fwd<T128x256k32>(d, ap, bp, ep, stream, "conv_fwd_128x256k32");
    case 5: return run_fwd<T256x256w8>(d, ap, bp, ep, stream, "conv_fwd_256x256w8");
    default: break;
  }
  switch (pick_bm(d.K)) {
    case 128: return run_fwd<T128x128>(d, ap, bp, ep, stream, "conv_fwd_128x128");
    case 96:  return run_fwd<T96x256>(d, ap, bp, ep, stream, "conv_fwd_96x256");
    case 64:  return run_fwd<T64x256>(d, ap, bp, ep, stream, "conv_fwd_64x256");
    default:  return run_fwd<T32x256>(d, ap, bp, ep, stream, "conv_fwd_32x256");
  }
}
