// Fused SGD-momentum parameter update (K14 fused) and the gen-1/gen-2 descend step.
// One pass over {W, g, v}: 24 bytes per parameter instead of the 52 of the BLAS-1 sequence.
// The arithmetic keeps the rounding points of that sequence: g = fma(l2, W, g); v = mu*v;
// v = fma(scale, g, v); W = fma(apply, v, W).
#include "common.h"

namespace rh {

__device__ __forceinline__ void sgd_one(float& w, float& g, float& v, float l2, float scale, float mu, float apply,
                                        bool use_l2, bool zero_grad) {
  float gi = g;
  if (use_l2) gi = fmaf(l2, w, gi);
  float vi = mu * v;
  vi = fmaf(scale, gi, vi);
  w = fmaf(apply, vi, w);
  v = vi;
  g = zero_grad ? 0.0f : gi;
}

__global__ void sgd_momentum_kernel(long long n, float* __restrict__ W, float* __restrict__ G, float* __restrict__ V,
                                    float l2, float scale, float mu, float apply, int zero_grad) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const bool use_l2 = l2 > 0.0f;
  const bool zg = zero_grad != 0;
  const bool vec = ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(G) | reinterpret_cast<uintptr_t>(V)) & 15) == 0;
  if (vec) {
    const long long n4 = n >> 2;
    float4* W4 = reinterpret_cast<float4*>(W);
    float4* G4 = reinterpret_cast<float4*>(G);
    float4* V4 = reinterpret_cast<float4*>(V);
    for (long long i = t; i < n4; i += stride) {
      float4 w = W4[i], g = G4[i], v = V4[i];
      sgd_one(w.x, g.x, v.x, l2, scale, mu, apply, use_l2, zg);
      sgd_one(w.y, g.y, v.y, l2, scale, mu, apply, use_l2, zg);
      sgd_one(w.z, g.z, v.z, l2, scale, mu, apply, use_l2, zg);
      sgd_one(w.w, g.w, v.w, l2, scale, mu, apply, use_l2, zg);
      W4[i] = w; G4[i] = g; V4[i] = v;
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) sgd_one(W[i], G[i], V[i], l2, scale, mu, apply, use_l2, zg);
  } else {
    for (long long i = t; i < n; i += stride) sgd_one(W[i], G[i], V[i], l2, scale, mu, apply, use_l2, zg);
  }
}

// The same update over several tensors in one launch: a network's parameter blocks are mostly small (biases,
// first-layer filters), and a launch per block costs more than its bytes.  Block b serves 1024 consecutive
// elements of the tensor whose block range [first[s], first[s+1]) holds b; the table travels as a kernel argument.
constexpr int kSgdSegs = 48;
struct SgdSegs {
  float* W[kSgdSegs];
  float* G[kSgdSegs];
  float* V[kSgdSegs];
  long long n[kSgdSegs];
  float l2[kSgdSegs];
  int first[kSgdSegs + 1];
  int count;
  unsigned long long keep;   // bit s: segment s keeps its gradient
};

__global__ __launch_bounds__(256) void sgd_momentum_multi_kernel(SgdSegs segs, float scale, float mu, float apply,
                                                                 int zero_grad) {
  const int b = blockIdx.x;
  int lo = 0, hi = segs.count - 1;          // last segment whose first block is <= b (uniform over the block)
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (segs.first[mid] <= b) lo = mid; else hi = mid - 1;
  }
  float* __restrict__ W = segs.W[lo];
  float* __restrict__ G = segs.G[lo];
  float* __restrict__ V = segs.V[lo];
  const long long n = segs.n[lo];
  const float l2 = segs.l2[lo];
  const bool keep = (segs.keep >> lo) & 1ull;   // this tensor's gradient is neither zeroed nor written back
  const bool use_l2 = l2 > 0.0f, zg = zero_grad != 0;
  const long long base = (long long)(b - segs.first[lo]) * 1024;
  const bool vec = ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(G) | reinterpret_cast<uintptr_t>(V)) & 15) == 0;
  const long long i = base + 4 * (long long)threadIdx.x;
  if (vec && i + 3 < n) {
    float4 w = *reinterpret_cast<float4*>(W + i), g = *reinterpret_cast<float4*>(G + i), v = *reinterpret_cast<float4*>(V + i);
    sgd_one(w.x, g.x, v.x, l2, scale, mu, apply, use_l2, zg);
    sgd_one(w.y, g.y, v.y, l2, scale, mu, apply, use_l2, zg);
    sgd_one(w.z, g.z, v.z, l2, scale, mu, apply, use_l2, zg);
    sgd_one(w.w, g.w, v.w, l2, scale, mu, apply, use_l2, zg);
    *reinterpret_cast<float4*>(W + i) = w;
    if (!keep) *reinterpret_cast<float4*>(G + i) = g;
    *reinterpret_cast<float4*>(V + i) = v;
  } else {
    for (int j = 0; j < 4; ++j)
      if (i + j < n) {
        float g = G[i + j];
        sgd_one(W[i + j], g, V[i + j], l2, scale, mu, apply, use_l2, zg);
        if (!keep) G[i + j] = g;
      }
  }
}

// g = fma(l2, W, g) (if l2 > 0); W = fma(-s, g, W)
__global__ void descend_kernel(long long n, float* __restrict__ W, float* __restrict__ G, float s, float l2) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const bool use_l2 = l2 > 0.0f;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float g = G[i];
    const float w = W[i];
    if (use_l2) g = fmaf(l2, w, g);
    G[i] = g;
    W[i] = fmaf(-s, g, w);
  }
}

}  // namespace rh

using namespace rh;

extern "C" int rh_sgd_momentum_step(int64_t n, float* W, float* g, float* v, float l2, float scale, float mu,
                                    float apply, int zero_grad, rh_stream_t stream) {
  if (n < 0 || (n > 0 && (!W || !g || !v)) || l2 < 0.0f) return RH_E_INVALID;
  if (n == 0) return 0;
  ProfScope prof("sgd_fused", 24.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(sgd_momentum_kernel, dim3(stream_grid((size_t)(n + 3) / 4, 256)), dim3(256), 0,
                     to_stream(stream), (long long)n, W, g, v, l2, scale, mu, apply, zero_grad);
  return launch_status();
}

extern "C" int rh_sgd_momentum_step_multi(int32_t count, const rh_sgd_tensor* tensors, float scale, float mu, float apply,
                                          int zero_grad, rh_stream_t stream) {
  if (count < 0 || (count > 0 && !tensors)) return RH_E_INVALID;
  double bytes = 0.0;
  for (int i = 0; i < count; ++i) {
    const rh_sgd_tensor& t = tensors[i];
    if (t.n < 0 || (t.n > 0 && (!t.W || !t.g || !t.v)) || !(t.l2 >= 0.0f)) return RH_E_INVALID;
    if (t.n > (int64_t)1023 * (int64_t)0x7fffffff / 2) return RH_E_LIMIT;
    bytes += (t.keep_grad ? 20.0 : 24.0) * (double)t.n;
  }
  if (bytes == 0.0) return 0;
  ProfScope prof("sgd_fused", bytes, to_stream(stream));
  int i = 0;
  while (i < count) {
    SgdSegs segs;
    segs.count = 0;
    segs.keep = 0;
    long long blocks = 0;
    for (; i < count && segs.count < kSgdSegs; ++i) {
      const rh_sgd_tensor& t = tensors[i];
      if (t.n == 0) continue;
      const long long nb = (t.n + 1023) / 1024;
      if (blocks + nb > 0x7fffffffll) break;       // the rest goes to another launch
      const int s = segs.count++;
      segs.W[s] = t.W; segs.G[s] = t.g; segs.V[s] = t.v; segs.n[s] = t.n; segs.l2[s] = t.l2;
      if (t.keep_grad) segs.keep |= 1ull << s;
      segs.first[s] = (int)blocks;
      blocks += nb;
    }
    if (segs.count == 0) {
      if (i < count && tensors[i].n > 0) return RH_E_LIMIT;   // a single tensor beyond one launch's block range
      continue;
    }
    segs.first[segs.count] = (int)blocks;
    hipLaunchKernelGGL(sgd_momentum_multi_kernel, dim3((unsigned)blocks), dim3(256), 0, to_stream(stream), segs, scale, mu,
                       apply, zero_grad);
    if (int e = launch_status()) return e;
  }
  return 0;
}

extern "C" int rh_descend(int64_t n, float* W, float* g, float s, float l2, rh_stream_t stream) {
  if (n < 0 || (n > 0 && (!W || !g)) || l2 < 0.0f) return RH_E_INVALID;
  if (n == 0) return 0;
  ProfScope prof("descend", 16.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(descend_kernel, dim3(stream_grid((size_t)n, 256)), dim3(256), 0, to_stream(stream),
                     (long long)n, W, g, s, l2);
  return launch_status();
}
