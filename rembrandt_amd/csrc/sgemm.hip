// Column-major SGEMM (K8) on the fp32 MFMA tile engine, plus the BLAS-1 calls (K14).
//   C(m,n) = alpha * op(A)(m,k) * op(B)(k,n) + beta * C
// The engine's lanes run along its column index, so C's contiguous index (its row im) is made the
// engine column and C's column jn the engine row:  D[jn][im] = sum_l opB(l,jn) * opA(im,l).
//   engine A operand (row jn): opB.  transB == 0: B[l + jn*ldb] (k contiguous); else B[jn + l*ldb].
//   engine B operand (row im): opA.  transA == 0: A[im + l*lda] (rows contiguous); else A[l + im*lda].
// When the result has too few tiles to fill the GPU (batch-sized GEMMs of the affine layers) and
// scratch is given, the contraction is split across blocks and reduced in a fixed order.
#include <type_traits>

#include "conv_common.h"

namespace rh {

struct SgemmPlan { int bm, bn, splits; };

static SgemmPlan plan_sgemm(int m, int n, int k) {
  SgemmPlan p;
  p.bm = pick_bm(n);
  if (p.bm == 96) p.bm = round_up(n, 128) <= round_up(n, 64) ? 128 : 64;  // no 96-row tile for row-contiguous loads
  p.bn = p.bm == 128 ? 128 : 256;
  const int tiles = cdiv(n, p.bm) * cdiv(m, p.bn);
  const int k_chunks = cdiv(k, 16);
  int want = 1;
  const int slots = 256 * (p.bm == 128 ? RH_OCC_128 : 3);  // blocks of this tile the GPU holds at a time
  if (tiles <= slots / 2) {
    want = slots / tiles;
    const int max_by_depth = (int)slices_by_depth(k_chunks, tiles, slots, 16, 4);
    if (want > max_by_depth) want = max_by_depth;
    if (want > 64) want = 64;
  }
  p.splits = want < 1 ? 1 : want;
  return p;
}

// A rows-contiguous dense operand seen by the scalar-offset loader: lane offset = row, wave-uniform offset = k*ld.
// Used only when k is a multiple of the K step: the scalar offset takes no part in the buffer range check, so a
// K tail must not be read this way.
static RowSParams rows_params(const DenseParams& d) {
  RowSParams r;
  r.ptr = d.ptr; r.bytes = d.bytes;
  r.M = d.rows; r.inner = d.rows > 0 ? d.rows : 1; r.innerW = r.inner;
  r.img_stride = 0; r.a_stride = 0; r.b_stride = 1;
  r.soff = nullptr; r.ldk4 = d.ld * 4;
  return r;
}

// K4: the k-contiguous operands are read 16 bytes at a time (see k4_ok).
template <class T, bool B_TRANS, bool A_TRANS, bool RS, bool K4>
static int run_sgemm(const DenseParams& ap, const DenseParams& bp, const EpiParams& ep, int k, int splits,
                     int* used, hipStream_t stream, const char* tag) {
  // engine A operand = opB: k contiguous unless transB; engine B operand = opA: rows contiguous unless transA
  typedef typename std::conditional<K4, LoadDenseK4<T::BM, T::BK, T::NT>, LoadDenseK<T::BM, T::BK, T::NT, false>>::type AK;
  typedef typename std::conditional<K4, LoadDenseK4<T::BN, T::BK, T::NT>, LoadDenseK<T::BN, T::BK, T::NT, false>>::type BK_;
  if constexpr (RS) {
    typedef LoadRowS<T::BM, T::BK, T::NT, true> AR;
    typedef LoadRowS<T::BN, T::BK, T::NT, true> BR;
    if constexpr (!B_TRANS && !A_TRANS)
      return launch_mfma_gemm<T, AK, BR, false, PassSgemm>(ap, rows_params(bp), ep, k, splits, used, stream, tag);
    else if constexpr (!B_TRANS && A_TRANS)
      return launch_mfma_gemm<T, AK, BK_, false, PassSgemm>(ap, bp, ep, k, splits, used, stream, tag);
    else if constexpr (B_TRANS && !A_TRANS)
      return launch_mfma_gemm<T, AR, BR, false, PassSgemm>(rows_params(ap), rows_params(bp), ep, k, splits, used, stream, tag);
    else
      return launch_mfma_gemm<T, AR, BK_, false, PassSgemm>(rows_params(ap), bp, ep, k, splits, used, stream, tag);
  } else {
    typedef LoadDenseR<T::BM, T::BK, T::NT> AR;
    typedef LoadDenseR<T::BN, T::BK, T::NT> BR;
    if constexpr (!B_TRANS && !A_TRANS)
      return launch_mfma_gemm<T, AK, BR, false, PassSgemm>(ap, bp, ep, k, splits, used, stream, tag);
    else if constexpr (!B_TRANS && A_TRANS)
      return launch_mfma_gemm<T, AK, BK_, false, PassSgemm>(ap, bp, ep, k, splits, used, stream, tag);
    else if constexpr (B_TRANS && !A_TRANS)
      return launch_mfma_gemm<T, AR, BR, false, PassSgemm>(ap, bp, ep, k, splits, used, stream, tag);
    else
      return launch_mfma_gemm<T, AR, BK_, false, PassSgemm>(ap, bp, ep, k, splits, used, stream, tag);
  }
}

// A k-contiguous operand can be read in aligned 16-byte groups that stay inside a row.
static bool k4_ok(const DenseParams& d, int k) {
  return k % 4 == 0 && d.ld % 4 == 0 && (reinterpret_cast<uintptr_t>(d.ptr) & 15) == 0;
}

template <class T, bool B_TRANS, bool A_TRANS, bool RS>
static int run_sgemm_k4(bool k4, const DenseParams& ap, const DenseParams& bp, const EpiParams& ep, int k, int splits,
                        int* used, hipStream_t stream, const char* tag) {
  if constexpr (B_TRANS && !A_TRANS) {   // no k-contiguous operand
    return run_sgemm<T, B_TRANS, A_TRANS, RS, false>(ap, bp, ep, k, splits, used, stream, tag);
  } else {
    return k4 ? run_sgemm<T, B_TRANS, A_TRANS, RS, true>(ap, bp, ep, k, splits, used, stream, tag)
              : run_sgemm<T, B_TRANS, A_TRANS, RS, false>(ap, bp, ep, k, splits, used, stream, tag);
  }
}

template <bool B_TRANS, bool A_TRANS>
static int dispatch_tile(int bm, const DenseParams& ap, const DenseParams& bp, const EpiParams& ep, int k,
                         int splits, int* used, hipStream_t stream) {
  const bool rs = k % 16 == 0 && (B_TRANS || !A_TRANS);
  const bool k4 = (B_TRANS || k4_ok(ap, k)) && (!A_TRANS || k4_ok(bp, k));   // every k-contiguous operand qualifies
  switch (bm) {
    case 128:
      return rs ? run_sgemm_k4<T128x128, B_TRANS, A_TRANS, true>(k4, ap, bp, ep, k, splits, used, stream, "sgemm_128x128")
                : run_sgemm_k4<T128x128, B_TRANS, A_TRANS, false>(k4, ap, bp, ep, k, splits, used, stream, "sgemm_128x128");
    case 64:
      return rs ? run_sgemm_k4<T64x256, B_TRANS, A_TRANS, true>(k4, ap, bp, ep, k, splits, used, stream, "sgemm_64x256")
                : run_sgemm_k4<T64x256, B_TRANS, A_TRANS, false>(k4, ap, bp, ep, k, splits, used, stream, "sgemm_64x256");
    default:  return run_sgemm_k4<T32x256, B_TRANS, A_TRANS, false>(k4, ap, bp, ep, k, splits, used, stream, "sgemm_32x256");
  }
}


// Products with a side of at most a few dozen (the classifier layer of a small network: 500 -> 10 at batch 64) are
// microseconds of arithmetic; on the tile engine they cost a contraction kernel of 10-20 us (one tile, a chain of K
// steps or slices plus their reduction).  Two plain forms with a fixed order of additions:
//   a wave per result element, lanes along the contraction (k >= 64 and at most 4096 elements: both operands of the
//   forward product are k-contiguous), lane sums added by a butterfly;
//   a thread per result element, consecutive threads along C's rows (k < 128 otherwise: data gradient, weight gradient).
// A(im, l) = A[im sa_m + l sa_k], B(l, jn) = B[l sb_k + jn sb_n]; epilogue as the tile engine's.
struct SkinnyArgs {
  const float* A; const float* B; float* C; const float* bias_col;
  int m, n, k, sa_m, sa_k, sb_k, sb_n, ldc, relu;
  float alpha, beta;
};

__device__ __forceinline__ void skinny_store(const SkinnyArgs& a, int im, int jn, float sum) {
  float* c = a.C + (size_t)jn * a.ldc + im;
  float val = a.alpha * sum;
  if (a.beta != 0.0f) val += a.beta * *c;
  if (a.bias_col) val += a.bias_col[im];
  if (a.relu) val = val > 0.0f ? val : 0.0f;
  *c = val;
}

__global__ __launch_bounds__(256) void sgemm_skinny_wave_kernel(SkinnyArgs a) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);   // result element: im fastest
  if (e >= a.m * a.n) return;
  const int jn = e / a.m, im = e - jn * a.m;
  const float* pa = a.A + (size_t)im * a.sa_m;
  const float* pb = a.B + (size_t)jn * a.sb_n;
  float s0 = 0.0f, s1 = 0.0f;
  int l = lane;
  for (; l + 64 < a.k; l += 128) {
    s0 = fmaf(pa[(size_t)l * a.sa_k], pb[(size_t)l * a.sb_k], s0);
    s1 = fmaf(pa[(size_t)(l + 64) * a.sa_k], pb[(size_t)(l + 64) * a.sb_k], s1);
  }
  if (l < a.k) s0 = fmaf(pa[(size_t)l * a.sa_k], pb[(size_t)l * a.sb_k], s0);
  float sum = s0 + s1;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if (lane == 0) skinny_store(a, im, jn, sum);
}

__global__ __launch_bounds__(256) void sgemm_skinny_thread_kernel(SkinnyArgs a) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= a.m * a.n) return;
  const int jn = e / a.m, im = e - jn * a.m;
  const float* pa = a.A + (size_t)im * a.sa_m;
  const float* pb = a.B + (size_t)jn * a.sb_n;
  // four running sums; sixteen steps (thirty-two loads) per trip, so that a thread waits for memory once per trip
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  int l = 0;
  for (; l + 15 < a.k; l += 16) {
    float va[16], vb[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      va[u] = pa[(size_t)(l + u) * a.sa_k];
      vb[u] = pb[(size_t)(l + u) * a.sb_k];
    }
#pragma unroll
    for (int u = 0; u < 16; u += 4) {
      s0 = fmaf(va[u], vb[u], s0);
      s1 = fmaf(va[u + 1], vb[u + 1], s1);
      s2 = fmaf(va[u + 2], vb[u + 2], s2);
      s3 = fmaf(va[u + 3], vb[u + 3], s3);
    }
  }
  for (; l + 3 < a.k; l += 4) {
    s0 = fmaf(pa[(size_t)l * a.sa_k], pb[(size_t)l * a.sb_k], s0);
    s1 = fmaf(pa[(size_t)(l + 1) * a.sa_k], pb[(size_t)(l + 1) * a.sb_k], s1);
    s2 = fmaf(pa[(size_t)(l + 2) * a.sa_k], pb[(size_t)(l + 2) * a.sb_k], s2);
    s3 = fmaf(pa[(size_t)(l + 3) * a.sa_k], pb[(size_t)(l + 3) * a.sb_k], s3);
  }
  for (; l < a.k; ++l) s0 = fmaf(pa[(size_t)l * a.sa_k], pb[(size_t)l * a.sb_k], s0);
  skinny_store(a, im, jn, (s0 + s1) + (s2 + s3));
}

// 0: the tile engine; 1: a wave per element; 2: a thread per element
static int skinny_mode(int m, int n, int k) {
  const long long mn = (long long)m * n;
  if (k >= 64 && mn <= 4096 && (m <= 16 || n <= 16)) return 1;
  if (k >= 128) return 0;
  if (k >= 1 && mn * k <= (1ll << 22) && (m <= 16 || n <= 16 || k <= 16)) return 2;
  return 0;
}

// y[i] += alpha * x[i]
__global__ void saxpy_kernel(long long n, float alpha, const float* __restrict__ x, float* __restrict__ y) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
  if (vec) {
    const long long n4 = n >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    float4* y4 = reinterpret_cast<float4*>(y);
    for (long long i = t; i < n4; i += stride) {
      const float4 a = x4[i];
      float4 b = y4[i];
      b.x = fmaf(alpha, a.x, b.x); b.y = fmaf(alpha, a.y, b.y);
      b.z = fmaf(alpha, a.z, b.z); b.w = fmaf(alpha, a.w, b.w);
      y4[i] = b;
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) y[i] = fmaf(alpha, x[i], y[i]);
  } else {
    for (long long i = t; i < n; i += stride) y[i] = fmaf(alpha, x[i], y[i]);
  }
}

// x[i] *= alpha
__global__ void sscal_kernel(long long n, float alpha, float* __restrict__ x) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const long long n4 = n >> 2;
    float4* x4 = reinterpret_cast<float4*>(x);
    for (long long i = t; i < n4; i += stride) {
      float4 a = x4[i];
      a.x *= alpha; a.y *= alpha; a.z *= alpha; a.w *= alpha;
      x4[i] = a;
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) x[i] *= alpha;
  } else {
    for (long long i = t; i < n; i += stride) x[i] *= alpha;
  }
}

}  // namespace rh

using namespace rh;

extern "C" size_t rh_sgemm_workspace_bytes(int32_t m, int32_t n, int32_t k) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  const SgemmPlan p = plan_sgemm(m, n, k);
  if (p.splits <= 1) return 0;
  return align256(sizeof(float) * (size_t)p.splits * m * n);
}

extern "C" size_t rh_sgemm_workspace_bytes_upto(int32_t m, int32_t n, int32_t k, int which) {
  size_t need = 0;
  const int top = which == 0 ? m : which == 1 ? n : which == 2 ? k : 0;
  for (int v = top; v >= 1; --v) {
    const size_t b = rh_sgemm_workspace_bytes(which == 0 ? v : m, which == 1 ? v : n, which == 2 ? v : k);
    if (b > need) need = b;
  }
  return need;
}

extern "C" int rh_sgemm(int transA, int transB, int32_t m, int32_t n, int32_t k, float alpha, const float* A,
                        int32_t lda, const float* B, int32_t ldb, float beta, float* C, int32_t ldc,
                        void* ws, size_t ws_bytes, int flags, rh_stream_t stream_) {
  return rh_sgemm_bias_act(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, nullptr, ws, ws_bytes, flags,
                           stream_);
}

extern "C" int rh_sgemm_bias_act(int transA, int transB, int32_t m, int32_t n, int32_t k, float alpha, const float* A,
                                 int32_t lda, const float* B, int32_t ldb, float beta, float* C, int32_t ldc,
                                 const float* bias, void* ws, size_t ws_bytes, int flags, rh_stream_t stream_) {
  if ((flags & RH_FUSE_BIAS) && !bias) return RH_E_INVALID;
  const float* bias_col = (flags & RH_FUSE_BIAS) ? bias : nullptr;
  const int relu = (flags & RH_FUSE_RELU) ? 1 : 0;
  if (m < 0 || n < 0 || k < 0 || !C) return RH_E_INVALID;
  if (m == 0 || n == 0) return 0;
  if (k > 0 && (!A || !B)) return RH_E_INVALID;
  if (lda < (transA ? k : m) || ldb < (transB ? n : k) || ldc < m) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  hipStream_t stream = to_stream(stream_);

  const size_t a_elems = k > 0 ? (size_t)lda * ((transA ? m : k) - 1) + (transA ? k : m) : 0;
  const size_t b_elems = k > 0 ? (size_t)ldb * ((transB ? k : n) - 1) + (transB ? n : k) : 0;
  if (a_elems * 4 > kMaxBufferBytes || b_elems * 4 > kMaxBufferBytes ||
      ((size_t)ldc * (n - 1) + m) * 4 > kMaxBufferBytes)
    return RH_E_LIMIT;

  if (!(flags & RH_ALGO_GATHER)) {
    if (const int mode = skinny_mode(m, n, k)) {
      SkinnyArgs a;
      a.A = A; a.B = B; a.C = C; a.bias_col = bias_col;
      a.m = m; a.n = n; a.k = k; a.ldc = ldc; a.relu = relu; a.alpha = alpha; a.beta = beta;
      a.sa_m = transA ? lda : 1; a.sa_k = transA ? 1 : lda;
      a.sb_k = transB ? ldb : 1; a.sb_n = transB ? 1 : ldb;
      ProfScope prof("sgemm_skinny", 2.0 * (double)m * n * k, stream);
      if (mode == 1)
        hipLaunchKernelGGL(sgemm_skinny_wave_kernel, dim3((unsigned)cdiv(m * n, 4)), dim3(256), 0, stream, a);
      else
        hipLaunchKernelGGL(sgemm_skinny_thread_kernel, dim3((unsigned)cdiv(m * n, 256)), dim3(256), 0, stream, a);
      return launch_status();
    }
  }
  DenseParams ap;  // engine A operand = opB, rows = n
  ap.ptr = B; ap.bytes = (uint32_t)(b_elems * 4); ap.rows = n; ap.K = k; ap.ld = ldb; ap.ktab = nullptr;
  DenseParams bp;  // engine B operand = opA, rows = m
  bp.ptr = A; bp.bytes = (uint32_t)(a_elems * 4); bp.rows = m; bp.K = k; bp.ld = lda; bp.ktab = nullptr;

  SgemmPlan plan = plan_sgemm(m, n, k);
  const size_t need = plan.splits > 1 ? align256(sizeof(float) * (size_t)plan.splits * m * n) : 0;
  if (plan.splits > 1 && (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255))) plan.splits = 1;

  EpiParams ep;
  ep.bias = nullptr; ep.alpha = alpha; ep.beta = beta; ep.rows = n; ep.cols = m; ep.inner = 0;
  ep.relu = relu; ep.bias_col = bias_col;   // (ignored by blocks that write partial sums)
  if (plan.splits > 1) {
    ep.out = static_cast<float*>(ws); ep.ld = m; ep.split_stride = (long long)m * n;
  } else {
    ep.out = C; ep.ld = ldc; ep.split_stride = 0;
  }

  int used = 1, e;
  if (!transB && !transA)      e = dispatch_tile<false, false>(plan.bm, ap, bp, ep, k, plan.splits, &used, stream);
  else if (!transB && transA)  e = dispatch_tile<false, true>(plan.bm, ap, bp, ep, k, plan.splits, &used, stream);
  else if (transB && !transA)  e = dispatch_tile<true, false>(plan.bm, ap, bp, ep, k, plan.splits, &used, stream);
  else                         e = dispatch_tile<true, true>(plan.bm, ap, bp, ep, k, plan.splits, &used, stream);
  if (e) return e;
  if (plan.splits > 1) {
    launch_split_reduce(static_cast<const float*>(ws), used, (long long)m * n, C, n, m, ldc, alpha, beta, stream, bias_col,
                        relu);
    return launch_status();
  }
  return 0;
}

extern "C" int rh_saxpy(int64_t n, float alpha, const float* x, float* y, rh_stream_t stream) {
  if (n < 0 || (n > 0 && (!x || !y))) return RH_E_INVALID;
  if (n == 0) return 0;
  ProfScope prof("saxpy", 12.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(saxpy_kernel, dim3(stream_grid((size_t)(n + 3) / 4, 256)), dim3(256), 0, to_stream(stream),
                     (long long)n, alpha, x, y);
  return launch_status();
}

extern "C" int rh_sscal(int64_t n, float alpha, float* x, rh_stream_t stream) {
  if (n < 0 || (n > 0 && !x)) return RH_E_INVALID;
  if (n == 0) return 0;
  ProfScope prof("sscal", 8.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(sscal_kernel, dim3(stream_grid((size_t)(n + 3) / 4, 256)), dim3(256), 0, to_stream(stream),
                     (long long)n, alpha, x);
  return launch_status();
}
