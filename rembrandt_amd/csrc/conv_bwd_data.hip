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

// One residue class of the strided form: wT[k][c] = w[ko][c][a + st*i][b + st*j] for k = (ko, i, j) (zero rows past
// the end) and soff[k] = 4*(ko*Hp*Wp + (Ra-1-i)*Wp + (Sb-1-j)) into the padded dy.
__global__ void prep_bwd_data_phase_kernel(const float* __restrict__ w, float* __restrict__ wT, int* __restrict__ soff,
                                           int n_k, int k_true, int C, int R, int S, int st, int a, int b, int Ra, int Sb,
                                           int HpWp, int Wp) {
  const long long total = (long long)n_k * C;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const int k = (int)(idx / C), c = (int)(idx - (long long)k * C);
    float v = 0.0f;
    int off = 0;
    if (k < k_true) {
      const int ko = k / (Ra * Sb), ij = k - ko * (Ra * Sb), i = ij / Sb, j = ij - i * Sb;
      v = w[(((size_t)ko * C + c) * R + (a + st * i)) * S + (b + st * j)];
      off = (ko * HpWp + (Ra - 1 - i) * Wp + (Sb - 1 - j)) * 4;
    }
    wT[idx] = v;
    if (c == 0) soff[k] = off;
  }
}

// dx[n][c][h][w] = alpha * (result of the class of (h + pad, w + pad) at its (u, v)) + beta * dx; classes without
// filter taps contribute 0.
struct PhaseTable {
  int u0[kMaxPhaseStride * kMaxPhaseStride], U[kMaxPhaseStride * kMaxPhaseStride];
  int v0[kMaxPhaseStride * kMaxPhaseStride], V[kMaxPhaseStride * kMaxPhaseStride];
  long long off[kMaxPhaseStride * kMaxPhaseStride];  // < 0: no taps
};
__global__ __launch_bounds__(256) void phase_interleave_kernel(const float* __restrict__ sub, float* __restrict__ dx,
                                                               unsigned total, FastDiv dW, FastDiv dH, FastDiv dSt, int st,
                                                               int pad, PhaseTable t, float alpha, float beta) {
  // per class: {offset of its result minus the offset of its first pixel, row length V, plane size U*V}; the table is
  // indexed per element, so it lives in LDS rather than in the kernel arguments
  __shared__ long long s_base[kMaxPhaseStride * kMaxPhaseStride];
  __shared__ int s_V[kMaxPhaseStride * kMaxPhaseStride], s_UV[kMaxPhaseStride * kMaxPhaseStride];
  if (threadIdx.x < kMaxPhaseStride * kMaxPhaseStride) {
    const int i = threadIdx.x;
    const bool live = i < st * st && t.off[i] >= 0;
    s_base[i] = live ? t.off[i] - ((long long)t.u0[i] * t.V[i] + t.v0[i]) : -1;
    s_V[i] = live ? t.V[i] : 0;
    s_UV[i] = live ? t.U[i] * t.V[i] : 0;
  }
  __syncthreads();
  // four consecutive elements of dx per thread, one 16-byte store (and load, when blending) if dx is aligned
  const unsigned i0 = (blockIdx.x * blockDim.x + threadIdx.x) * 4u;
  if (i0 >= total) return;
  uint32_t rest, w, plane, h, u, a;
  dW.divmod(i0, rest, w);
  dH.divmod(rest, plane, h);
  dSt.divmod(h + (uint32_t)pad, u, a);
  const bool vec = (reinterpret_cast<uintptr_t>(dx) & 15) == 0 && i0 + 3 < total;
  float old[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (beta != 0.0f) {
    if (vec) {
      const float4 o = *reinterpret_cast<const float4*>(dx + i0);
      old[0] = o.x; old[1] = o.y; old[2] = o.z; old[3] = o.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < total) old[e] = dx[i0 + e];
    }
  }
  float val[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint32_t v, b;
    dSt.divmod(w + (uint32_t)pad, v, b);
    const int ph = (int)(a * st + b);
    const int V = s_V[ph];
    float x = 0.0f;
    if (V > 0 && i0 + e < total) x = sub[s_base[ph] + (long long)plane * s_UV[ph] + (long long)u * V + v];
    x *= alpha;
    if (beta != 0.0f) x = fmaf(beta, old[e], x);
    val[e] = x;
    if (++w == dW.div) {
      w = 0;
      if (++h == dH.div) { h = 0; ++plane; }
      dSt.divmod(h + (uint32_t)pad, u, a);
    }
  }
  if (vec) {
    *reinterpret_cast<float4*>(dx + i0) = make_float4(val[0], val[1], val[2], val[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i0 + e < total) dx[i0 + e] = val[e];
  }
}

template <class T>
static int run_bwd_data_soff(const RowSParams& ap, const RowSParams& bp, EpiParams ep, int n_k, int k_true,
                             hipStream_t stream, const char* tag, int splits, float* part,
                             const TailSplit* tail = nullptr) {
  constexpr int AROWS = T::BM % 64 == 0 ? T::BM : (T::BM + 63) / 64 * 64;
  typedef LoadRowS<AROWS, T::BK, T::NT, true> AL;
  typedef LoadRowS<T::BN, T::BK, T::NT, false> BL;
  if (splits <= 1 && tail && tail->splits > 1) {
    // whole tiles blend into dx as usual; the sliced tail goes through `part` and one reduction over its columns
    const EpiParams fin = ep;
    const long long total = (long long)ep.rows * ep.cols;
    const long long first = tail_first_elem(*tail, ep.inner, ep.rows);
    ep.part = part; ep.part_first = first; ep.split_stride = total - first;
    ep.full_tiles = tail->full_tiles; ep.tail_tiles = tail->tail_tiles; ep.tail_splits = tail->splits;
    if (int e = launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, n_k, 1, nullptr, stream, tag, k_true)) return e;
    launch_split_reduce_nchw(part, tail->splits, total - first, fin.out, total, fin.inner, fin.rows, fin.alpha, fin.beta,
                             nullptr, 0, stream, tail->col0, fin.mask);
    return launch_status();
  }
  // one pass over the whole contraction: K steps that hold nothing but the table's zero padding are left out
  if (splits <= 1)
    return launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, min(n_k, round_up(k_true, T::BK)), 1, nullptr, stream,
                                                             tag, k_true);
  // slices of the contraction write unblended partial results; one reduction applies the alpha / beta blend
  const EpiParams fin = ep;
  const long long total = (long long)ep.rows * ep.cols;
  ep.out = part; ep.split_stride = total;
  int used = 1;
  if (int e = launch_mfma_gemm<T, AL, BL, true, PassConvBwdData>(ap, bp, ep, n_k, splits, &used, stream, tag, k_true)) return e;
  launch_split_reduce_nchw(part, used, total, fin.out, total, fin.inner, fin.rows, fin.alpha, fin.beta, nullptr, 0, stream, 0,
                           fin.mask);
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

// mask: nullptr, or the output of the ReLU whose backward is applied to dx as it is written (never with the
// residue-class form: see rh_conv2d_bwd_data_relu_supported).
static int bwd_data_impl(const rh_conv_geom* g, float alpha, const float* w, const float* dy, float beta, float* dx,
                         void* ws, size_t ws_bytes, int flags, rh_stream_t stream_, const float* mask) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!w || !dy || !dx) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  const size_t need = rh_conv2d_workspace_bytes(g, RH_CONV_BWD_DATA);
  if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  if ((flags & RH_ALGO_WINOGRAD) && (!wino_shape(d) || (flags & (RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT)))) return RH_E_UNSUPPORTED;
  if (!(flags & (RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET)) && conv1x1_stream_applies(d)) {
    if (d.x_elems == 0) return 0;
    return launch_conv1x1_stream(d, RH_CONV_BWD_DATA, w, dy, dx, alpha, beta, nullptr, 0, stream, mask);
  }
  if (wino_shape(d) && !(flags & (RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT))) {
    WinoGeom wg = wino_geom_bwd_data(d);
    if (flags & RH_ALGO_WINOGRAD ? wg.ok : wino_pays(wg)) {
      if (d.x_elems == 0) return 0;
      if (flags & RH_ALGO_SHARED_GPU) wg.tail_S = 1;
      return launch_conv_wino(wg, true, dy, w, dx, alpha, beta, nullptr, 0, mask, ws, stream, "conv_bwd_data_wino");
    }
    if (flags & RH_ALGO_WINOGRAD) return RH_E_UNSUPPORTED;
  }
  const int KRS = d.K * d.R * d.S;
  const PhasePlan pp = plan_phase_bwd_data(d);
  if (pp.ok && !(flags & RH_ALGO_GATHER)) {
    if (mask) return RH_E_UNSUPPORTED;
    if (d.x_elems == 0) return 0;
    char* base = static_cast<char*>(ws);
    int* soff = reinterpret_cast<int*>(base);
    float* wT = reinterpret_cast<float*>(base + pp.tab_bytes);
    float* sub = reinterpret_cast<float*>(base + pp.tab_bytes + pp.wt_bytes + pp.img_bytes);
    float* part = reinterpret_cast<float*>(base + pp.tab_bytes + pp.wt_bytes + pp.img_bytes + pp.sub_bytes);
    const float* img = dy;
    if (pp.img_bytes) {
      float* dyp = reinterpret_cast<float*>(base + pp.tab_bytes + pp.wt_bytes);
      launch_pad_image(dy, dyp, (long long)d.N * d.K, d.P, d.Q, pp.Hp, pp.Wp, pp.L, stream);
      if (int e = launch_status()) return e;
      img = dyp;
    }
    const size_t img_floats = (size_t)d.N * d.K * pp.Hp * pp.Wp;
    PhaseTable tab;
    for (int a = 0; a < d.st; ++a)
      for (int b = 0; b < d.st; ++b) {
        const int i = a * d.st + b;
        const PhaseGeom& g = pp.ph[i];
        const bool live = g.Ra > 0 && g.Sb > 0 && g.U > 0 && g.V > 0;
        tab.u0[i] = g.u0; tab.U[i] = g.U; tab.v0[i] = g.v0; tab.V[i] = g.V; tab.off[i] = live ? g.sub_off : -1;
        if (!live) continue;
        const int k_true = d.K * g.Ra * g.Sb, n_k = round_up(k_true, kTabPad);
        hipLaunchKernelGGL(prep_bwd_data_phase_kernel, dim3(stream_grid((size_t)n_k * d.C, 256)), dim3(256), 0, stream, w, wT,
                           soff, n_k, k_true, d.C, d.R, d.S, d.st, a, b, g.Ra, g.Sb, pp.Hp * pp.Wp, pp.Wp);
        if (int e = launch_status()) return e;
        RowSParams ap;  // transposed sub-filter [k][c]
        ap.ptr = wT; ap.bytes = (uint32_t)(sizeof(float) * (size_t)n_k * d.C);
        ap.M = d.C; ap.inner = d.C; ap.innerW = d.C; ap.img_stride = 0; ap.a_stride = 0; ap.b_stride = 1;
        ap.soff = nullptr; ap.ldk4 = d.C * 4;
        // padded dy seen from the class's first pixel and first tap: rows = (n, u - u0, v - v0)
        const size_t first = (size_t)(g.u0 + pp.L - (g.Ra - 1)) * pp.Wp + (size_t)(g.v0 + pp.L - (g.Sb - 1));
        RowSParams bp;
        bp.ptr = img + first; bp.bytes = (uint32_t)(sizeof(float) * (img_floats - first));
        bp.M = d.N * g.U * g.V; bp.inner = g.U * g.V; bp.innerW = g.V;
        bp.img_stride = d.K * pp.Hp * pp.Wp; bp.a_stride = pp.Wp; bp.b_stride = 1;
        bp.soff = soff; bp.ldk4 = 0;
        EpiParams ep;
        ep.out = sub + g.sub_off; ep.bias = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
        ep.rows = d.C; ep.cols = bp.M; ep.inner = g.U * g.V; ep.ld = 0; ep.relu = 0; ep.split_stride = 0;
        int e;
        switch (pick_bm(d.C)) {
          case 128: e = run_bwd_data_soff<T128x128>(ap, bp, ep, n_k, k_true, stream, "conv_bwd_data_128x128", g.splits, part); break;
          case 96:  e = run_bwd_data_soff<T96x128>(ap, bp, ep, n_k, k_true, stream, "conv_bwd_data_96x128", g.splits, part); break;
          case 64:  e = run_bwd_data_soff<T64x256>(ap, bp, ep, n_k, k_true, stream, "conv_bwd_data_64x256", g.splits, part); break;
          default:  e = run_bwd_data_soff<T32x256>(ap, bp, ep, n_k, k_true, stream, "conv_bwd_data_32x256", g.splits, part); break;
        }
        if (e) return e;
      }
    ProfScope prof("phase_interleave", 8.0 * (double)d.x_elems, stream);
    hipLaunchKernelGGL(phase_interleave_kernel, dim3(stream_grid((size_t)(d.x_elems + 3) / 4, 256)), dim3(256), 0, stream, sub, dx,
                       (unsigned)d.x_elems, FastDiv((uint32_t)d.W), FastDiv((uint32_t)d.H), FastDiv((uint32_t)d.st), d.st, d.pad,
                       tab, alpha, beta);
    return launch_status();
  }
  const SoffPlan sp = plan_soff_bwd_data(d);
  if (sp.ok && !(flags & RH_ALGO_GATHER)) {
    int* soff = static_cast<int*>(ws);
    float* wT = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes);
    const float* img = dy;
    if (sp.img_bytes && d.st == 1) {
      float* dyp = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes);
      launch_pad_image_prep_soff(dy, dyp, (long long)d.N * d.K, d.P, d.Q, sp.Hp, sp.Wp, sp.halo, w, wT, soff, sp.n_k, KRS, d.C,
                                 d.R, d.S, 1, stream);
      img = dyp;
    } else {
      if (sp.img_bytes) {
        float* dyp = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes);
        launch_pad_image(dy, dyp, (long long)d.N * d.K, d.P, d.Q, sp.Hp, sp.Wp, sp.halo, stream, d.st);
        if (int e = launch_status()) return e;
        img = dyp;
      }
      launch_prep_soff(w, wT, soff, sp.n_k, KRS, d.C, d.R, d.S, sp.Hp * sp.Wp, sp.Wp, 1, stream);
    }
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
    ep.mask = mask;
    float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes + sp.img_bytes);
    switch (pick_bm(d.C)) {
      case 128:
        if (sp.narrow128) return run_bwd_data_soff<T128x64>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_128x64", sp.splits, part, &sp.tail);
        return run_bwd_data_soff<T128x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_128x128", sp.splits, part, &sp.tail);
      case 96:  return run_bwd_data_soff<T96x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_96x128", sp.splits, part, &sp.tail);
      case 64:
        if (cdiv(d.C, 64) == 1 && prefer_k8_64(ep.cols))
          return run_bwd_data_soff<T64x256k8>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_64x256k8", sp.splits, part, &sp.tail);
        // (sliced contractions on the half-width tile, as in the forward pass)
        if (sp.splits > 1) return run_bwd_data_soff<T64x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_64x128", sp.splits, part, &sp.tail);
        return run_bwd_data_soff<T64x256>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_64x256", sp.splits, part, &sp.tail);
      default:
        if (sp.splits > 1) return run_bwd_data_soff<T32x128>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_32x128", sp.splits, part, &sp.tail);
        return run_bwd_data_soff<T32x256>(ap, bp, ep, sp.n_k, KRS, stream, "conv_bwd_data_32x256", sp.splits, part, &sp.tail);
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
  ep.mask = mask;

  switch (pick_bm(d.C)) {
    case 128: return run_bwd_data<T128x128>(KRS, ap, bp, ep, stream, "conv_bwd_data_128x128");
    case 96:  return run_bwd_data<T96x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_96x256");
    case 64:  return run_bwd_data<T64x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_64x256");
    default:  return run_bwd_data<T32x256>(KRS, ap, bp, ep, stream, "conv_bwd_data_32x256");
  }
}

extern "C" int rh_conv2d_bwd_data(const rh_conv_geom* g, float alpha, const float* w, const float* dy,
                                  float beta, float* dx, void* ws, size_t ws_bytes, int flags,
                                  rh_stream_t stream_) {
  return bwd_data_impl(g, alpha, w, dy, beta, dx, ws, ws_bytes, flags, stream_, nullptr);
}

extern "C" int rh_conv2d_bwd_data_relu_supported(const rh_conv_geom* g) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  if (conv1x1_stream_applies(d)) return 1;
  return plan_phase_bwd_data(d).ok ? 0 : 1;   // strides above one take the residue-class form, which has no masked epilogue
}

extern "C" int rh_conv2d_bwd_data_relu(const rh_conv_geom* g, float alpha, const float* w, const float* dy,
                                       float beta, float* dx, const float* x_act, void* ws, size_t ws_bytes,
                                       int flags, rh_stream_t stream_) {
  if (!x_act) return RH_E_INVALID;
  if (!rh_conv2d_bwd_data_relu_supported(g)) return RH_E_UNSUPPORTED;
  return bwd_data_impl(g, alpha, w, dy, beta, dx, ws, ws_bytes, flags, stream_, x_act);
}
