// Spatial batch normalisation over NCHW fp32 tensors: one mean / inverse standard deviation per channel, taken
// over the N*H*W values of that channel.  Stands where the reference calls CudnnBatchNormOp in Spatial mode
// (src/operator/conv.rs:493-535 forward, :594-607 backward).  All three passes are bandwidth bound:
//
//   forward (training)   reduce: read x once            apply: read x (+ y when blending), write y
//   backward             reduce: read x, dy once        apply: read x, dy (+ dx when blending), write dx
//
// A reduce launch covers the tensor with C x G blocks; wave (g, w) of channel c adds work units u = 4g + w,
// 4g + w + 4G, ... where a unit is one 2048-value piece of one image's plane, and leaves one partial per block.
// A finish launch (one thread per channel) adds the G partials in a fixed order in double precision, so results do
// not depend on scheduling.  The variance is accumulated around the channel's first value as a shift, which keeps
// the one-pass E[d^2] - E[d]^2 form free of the cancellation a zero shift would have for a large mean.
#include "common.h"

namespace rh {

constexpr int kBnChunk = 2048;  // values of one plane a wave adds per work unit

struct BnPlan {
  int chunks;        // pieces per plane
  long long units;   // N * chunks, per channel
  int G;             // blocks per channel
};

inline BnPlan bn_plan(int N, int C, int plane) {
  BnPlan p;
  p.chunks = cdiv(plane, kBnChunk);
  p.units = (long long)N * p.chunks;
  long long g = cdiv<long long>(2048, C);
  const long long most = cdiv<long long>(p.units, 4);
  if (g > most) g = most;
  if (g < 1) g = 1;
  p.G = (int)g;
  return p;
}

__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  return v;
}

// MODE 0: (sum d, sum d*d) with d = x - x[first value of the channel].
// MODE 1: (sum dy, sum dy*(x - mean[c])).
// VEC (plane % 4 == 0, 16-byte aligned tensors): a lane reads 16 bytes at a time, two such loads in flight per operand.
// MASK (MODE 1): dy counts only where the forward pass's ReLU let the value through, i.e. where
// bn_affine(x, mean, scale*ivar, bias) > 0, recomputed here exactly as the forward pass computed it.
__device__ __forceinline__ float bn_affine(float x, float mean, float si, float bias) { return fmaf(x - mean, si, bias); }

struct BnMask { const float* scale; const float* ivar; const float* bias; };

template <int MODE, bool VEC, bool MASK = false>
__global__ __launch_bounds__(256) void bn_reduce_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                        const float* __restrict__ mean, int C, int plane, int chunks,
                                                        long long units, float2* __restrict__ part, BnMask mk) {
  const int c = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float shift = MODE == 0 ? x[(size_t)c * plane] : mean[c];
  const float m_si = MASK ? mk.scale[c] * mk.ivar[c] : 0.0f, m_bias = MASK ? mk.bias[c] : 0.0f;
  float s0a = 0.0f, s0b = 0.0f, s1a = 0.0f, s1b = 0.0f;
  for (long long u = (long long)g * 4 + wave; u < units; u += (long long)G * 4) {
    const int n = (int)(u / chunks), ch = (int)(u - (long long)n * chunks);
    const size_t base = ((size_t)n * C + c) * plane;
    const int p0 = ch * kBnChunk, p1 = min(plane, p0 + kBnChunk);
    if (VEC) {
      auto add4 = [&](const float4 xv, const float4 gv, float& t0, float& t1) {
        const float d[4] = {xv.x - shift, xv.y - shift, xv.z - shift, xv.w - shift};
        float gg[4] = {gv.x, gv.y, gv.z, gv.w};
        if (MASK) {
          const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) gg[e] = bn_affine(xs[e], shift, m_si, m_bias) > 0.0f ? gg[e] : 0.0f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (MODE == 0) { t0 += d[e]; t1 = fmaf(d[e], d[e], t1); }
          else { t0 += gg[e]; t1 = fmaf(gg[e], d[e], t1); }
        }
      };
      const float4* x4 = reinterpret_cast<const float4*>(x + base);
      const float4* g4 = reinterpret_cast<const float4*>((MODE == 1 ? dy : x) + base);
      const int q1 = p1 >> 2;
      int q = (p0 >> 2) + lane;
      for (; q + 64 < q1; q += 128) {
        const float4 xa = x4[q], xb = x4[q + 64];
        const float4 ga = MODE == 1 ? g4[q] : xa, gb = MODE == 1 ? g4[q + 64] : xb;
        add4(xa, ga, s0a, s1a);
        add4(xb, gb, s0b, s1b);
      }
      if (q < q1) {
        const float4 xa = x4[q];
        add4(xa, MODE == 1 ? g4[q] : xa, s0a, s1a);
      }
      continue;
    }
    int i = p0 + lane;
    for (; i + 64 < p1; i += 128) {
      const float d0 = x[base + i] - shift, d1 = x[base + i + 64] - shift;
      if (MODE == 0) {
        s0a += d0; s0b += d1;
        s1a = fmaf(d0, d0, s1a); s1b = fmaf(d1, d1, s1b);
      } else {
        float g0 = dy[base + i], g1 = dy[base + i + 64];
        if (MASK) {
          g0 = bn_affine(x[base + i], shift, m_si, m_bias) > 0.0f ? g0 : 0.0f;
          g1 = bn_affine(x[base + i + 64], shift, m_si, m_bias) > 0.0f ? g1 : 0.0f;
        }
        s0a += g0; s0b += g1;
        s1a = fmaf(g0, d0, s1a); s1b = fmaf(g1, d1, s1b);
      }
    }
    if (i < p1) {
      const float d0 = x[base + i] - shift;
      if (MODE == 0) {
        s0a += d0;
        s1a = fmaf(d0, d0, s1a);
      } else {
        float g0 = dy[base + i];
        if (MASK) g0 = bn_affine(x[base + i], shift, m_si, m_bias) > 0.0f ? g0 : 0.0f;
        s0a += g0;
        s1a = fmaf(g0, d0, s1a);
      }
    }
  }
  const float s0 = wave_sum(s0a + s0b), s1 = wave_sum(s1a + s1b);
  __shared__ float2 sm[4];
  if (lane == 0) sm[wave] = make_float2(s0, s1);
  __syncthreads();
  if (threadIdx.x == 0)
    part[(size_t)g * C + c] = make_float2((sm[0].x + sm[1].x) + (sm[2].x + sm[3].x), (sm[0].y + sm[1].y) + (sm[2].y + sm[3].y));
}

// coef[c] = (mean, scale*ivar, bias, unused)
__global__ void bn_fwd_finish_kernel(const float* __restrict__ x, const float2* __restrict__ part, int G, int C, int plane,
                                     double count, double ema, double epsilon, const float* __restrict__ scale,
                                     const float* __restrict__ bias, float* __restrict__ running_mean,
                                     float* __restrict__ running_ivar, float* __restrict__ cached_mean,
                                     float* __restrict__ cached_ivar, float4* __restrict__ coef) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  double s0 = 0.0, s1 = 0.0;
  for (int g = 0; g < G; ++g) {
    const float2 p = part[(size_t)g * C + c];
    s0 += (double)p.x;
    s1 += (double)p.y;
  }
  const double md = s0 / count;
  double var = s1 / count - md * md;
  if (var < 0.0) var = 0.0;
  const float mean = (float)((double)x[(size_t)c * plane] + md);
  const float ivar = (float)(1.0 / sqrt(var + epsilon));
  cached_mean[c] = mean;
  cached_ivar[c] = ivar;
  running_mean[c] = (float)((1.0 - ema) * (double)running_mean[c] + ema * (double)mean);
  running_ivar[c] = (float)((1.0 - ema) * (double)running_ivar[c] + ema * (double)ivar);
  coef[c] = make_float4(mean, scale[c] * ivar, bias[c], 0.0f);
}

__global__ void bn_infer_coef_kernel(int C, const float* __restrict__ scale, const float* __restrict__ bias,
                                     const float* __restrict__ running_mean, const float* __restrict__ running_ivar,
                                     float4* __restrict__ coef) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < C) coef[c] = make_float4(running_mean[c], scale[c] * running_ivar[c], bias[c], 0.0f);
}

// coef[c] = (mean, scale*ivar, sum(dy)/m, ivar^2 * sum(dy*(x-mean))/m)
__global__ void bn_bwd_finish_kernel(const float2* __restrict__ part, int G, int C, double count, float alpha_param,
                                     float beta_param, const float* __restrict__ scale, float* __restrict__ dscale,
                                     float* __restrict__ dbias, const float* __restrict__ cached_mean,
                                     const float* __restrict__ cached_ivar, float4* __restrict__ coef) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  double s0 = 0.0, s1 = 0.0;
  for (int g = 0; g < G; ++g) {
    const float2 p = part[(size_t)g * C + c];
    s0 += (double)p.x;
    s1 += (double)p.y;
  }
  const double ivar = (double)cached_ivar[c];
  const float ds = (float)(s1 * ivar), db = (float)s0;
  dscale[c] = beta_param != 0.0f ? fmaf(beta_param, dscale[c], alpha_param * ds) : alpha_param * ds;
  dbias[c] = beta_param != 0.0f ? fmaf(beta_param, dbias[c], alpha_param * db) : alpha_param * db;
  coef[c] = make_float4(cached_mean[c], scale[c] * (float)ivar, (float)(s0 / count), (float)(s1 * ivar * ivar / count));
}

// Forward:  out = alpha * f((x - mean)*a + b) + beta*out, f = identity or max(., 0) applied after the blend when RELU.
// Backward: out = alpha * a*(dy - c2 - (x - mean)*c3) + beta*out.
// VEC: 4 values per thread (plane % 4 == 0 and 16-byte aligned pointers, so a group never crosses a plane).
// MASK (backward only): dy is taken as 0 where the forward ReLU clamped, see bn_reduce_kernel; mask_bias = the layer's bias.
template <bool BWD, bool RELU, bool VEC, bool MASK = false>
__global__ __launch_bounds__(256) void bn_apply_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                       float* __restrict__ out, const float4* __restrict__ coef,
                                                       long long groups, int C, FastDiv plane_groups, FastDiv chans,
                                                       float alpha, float beta, const float* __restrict__ mask_bias) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += stride) {
    const uint32_t row = plane_groups.quot((uint32_t)i);  // n*C + c
    const uint32_t c = row - chans.quot(row) * (uint32_t)C;
    const float4 k = coef[c];
    const float mb = MASK ? mask_bias[c] : 0.0f;
    auto one = [&](float xv, float gv, float ov) {
      float v;
      if (MASK) gv = bn_affine(xv, k.x, k.y, mb) > 0.0f ? gv : 0.0f;
      if (BWD) v = k.y * (gv - k.z - (xv - k.x) * k.w);
      else v = bn_affine(xv, k.x, k.y, k.z);
      v *= alpha;
      if (beta != 0.0f) v = fmaf(beta, ov, v);
      if (RELU) v = v > 0.0f ? v : 0.0f;
      return v;
    };
    if (VEC) {
      const float4 xv = reinterpret_cast<const float4*>(x)[i];
      float4 gv = make_float4(0.0f, 0.0f, 0.0f, 0.0f), ov = gv;
      if (BWD) gv = reinterpret_cast<const float4*>(dy)[i];
      if (beta != 0.0f) ov = reinterpret_cast<float4*>(out)[i];
      float4 r;
      r.x = one(xv.x, gv.x, ov.x); r.y = one(xv.y, gv.y, ov.y); r.z = one(xv.z, gv.z, ov.z); r.w = one(xv.w, gv.w, ov.w);
      reinterpret_cast<float4*>(out)[i] = r;
    } else {
      out[i] = one(x[i], BWD ? dy[i] : 0.0f, beta != 0.0f ? out[i] : 0.0f);
    }
  }
}

template <bool BWD, bool RELU, bool MASK = false>
void launch_bn_apply(const float* x, const float* dy, float* out, const float4* coef, int N, int C, int plane, float alpha,
                     float beta, hipStream_t st, const float* mask_bias = nullptr) {
  const long long total = (long long)N * C * plane;
  const bool vec = plane % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out) |
                                        reinterpret_cast<uintptr_t>(dy)) & 15) == 0;
  if (vec) {
    const long long groups = total / 4;
    hipLaunchKernelGGL((bn_apply_kernel<BWD, RELU, true, MASK>), dim3(stream_grid((size_t)groups, 256)), dim3(256), 0, st, x, dy,
                       out, coef, groups, C, FastDiv((uint32_t)(plane / 4)), FastDiv((uint32_t)C), alpha, beta, mask_bias);
  } else {
    hipLaunchKernelGGL((bn_apply_kernel<BWD, RELU, false, MASK>), dim3(stream_grid((size_t)total, 256)), dim3(256), 0, st, x, dy,
                       out, coef, total, C, FastDiv((uint32_t)plane), FastDiv((uint32_t)C), alpha, beta, mask_bias);
  }
}

inline size_t bn_part_bytes(const BnPlan& p, int C) { return ((size_t)p.G * C * sizeof(float2) + 255) & ~(size_t)255; }

int bn_check(int N, int C, int plane, long long* total) {
  if (N < 0 || C < 0 || plane < 0) return RH_E_INVALID;
  *total = (long long)N * C * plane;
  if (*total >= (1ll << 31)) return RH_E_LIMIT;
  return 0;
}

}  // namespace rh

using namespace rh;

extern "C" size_t rh_bnorm_workspace_bytes(int N, int C, int plane) {
  if (N <= 0 || C <= 0 || plane <= 0) return 256;
  const BnPlan p = bn_plan(N, C, plane);
  return bn_part_bytes(p, C) + (((size_t)C * sizeof(float4) + 255) & ~(size_t)255);
}

extern "C" size_t rh_bnorm_workspace_bytes_upto(int N, int C, int plane) {
  size_t need = 256;
  for (int n = N; n >= 1; --n) {
    const size_t b = rh_bnorm_workspace_bytes(n, C, plane);
    if (b > need) need = b;
  }
  return need;
}

extern "C" int rh_bnorm_fwd_train(int N, int C, int plane, float alpha, const float* x, float beta, float* y,
                                  double ema_factor, double epsilon, const float* scale, const float* bias,
                                  float* running_mean, float* running_ivar, float* cached_mean, float* cached_ivar,
                                  void* ws, size_t ws_bytes, int flags, rh_stream_t stream) {
  long long total;
  if (int e = bn_check(N, C, plane, &total)) return e;
  if (total == 0) return 0;
  if (!x || !y || !scale || !bias || !running_mean || !running_ivar || !cached_mean || !cached_ivar || !ws) return RH_E_INVALID;
  if (flags & ~RH_FUSE_RELU) return RH_E_UNSUPPORTED;
  if (ws_bytes < rh_bnorm_workspace_bytes(N, C, plane)) return RH_E_WORKSPACE;
  hipStream_t st = to_stream(stream);
  const BnPlan p = bn_plan(N, C, plane);
  float2* part = static_cast<float2*>(ws);
  float4* coef = reinterpret_cast<float4*>(static_cast<char*>(ws) + bn_part_bytes(p, C));
  {
    ProfScope prof("bnorm_fwd_reduce", 4.0 * (double)total, st);
    if (plane % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)
      hipLaunchKernelGGL((bn_reduce_kernel<0, true>), dim3(C, p.G), dim3(256), 0, st, x, (const float*)nullptr,
                         (const float*)nullptr, C, plane, p.chunks, p.units, part, BnMask());
    else
      hipLaunchKernelGGL((bn_reduce_kernel<0, false>), dim3(C, p.G), dim3(256), 0, st, x, (const float*)nullptr,
                         (const float*)nullptr, C, plane, p.chunks, p.units, part, BnMask());
    hipLaunchKernelGGL(bn_fwd_finish_kernel, dim3(cdiv(C, 64)), dim3(64), 0, st, x, part, p.G, C, plane,
                       (double)N * (double)plane, ema_factor, epsilon, scale, bias, running_mean, running_ivar, cached_mean,
                       cached_ivar, coef);
  }
  ProfScope prof("bnorm_fwd_apply", (beta != 0.0f ? 12.0 : 8.0) * (double)total, st);
  if (flags & RH_FUSE_RELU) launch_bn_apply<false, true>(x, nullptr, y, coef, N, C, plane, alpha, beta, st);
  else launch_bn_apply<false, false>(x, nullptr, y, coef, N, C, plane, alpha, beta, st);
  return launch_status();
}

extern "C" int rh_bnorm_fwd_infer(int N, int C, int plane, float alpha, const float* x, float beta, float* y, double epsilon,
                                  const float* scale, const float* bias, const float* running_mean,
                                  const float* running_ivar, void* ws, size_t ws_bytes, int flags, rh_stream_t stream) {
  (void)epsilon;  // already inside the stored inverse standard deviation
  long long total;
  if (int e = bn_check(N, C, plane, &total)) return e;
  if (total == 0) return 0;
  if (!x || !y || !scale || !bias || !running_mean || !running_ivar || !ws) return RH_E_INVALID;
  if (flags & ~RH_FUSE_RELU) return RH_E_UNSUPPORTED;
  if (ws_bytes < rh_bnorm_workspace_bytes(N, C, plane)) return RH_E_WORKSPACE;
  hipStream_t st = to_stream(stream);
  const BnPlan p = bn_plan(N, C, plane);
  float4* coef = reinterpret_cast<float4*>(static_cast<char*>(ws) + bn_part_bytes(p, C));
  ProfScope prof("bnorm_fwd_apply", (beta != 0.0f ? 12.0 : 8.0) * (double)total, st);
  hipLaunchKernelGGL(bn_infer_coef_kernel, dim3(cdiv(C, 64)), dim3(64), 0, st, C, scale, bias, running_mean, running_ivar, coef);
  if (flags & RH_FUSE_RELU) launch_bn_apply<false, true>(x, nullptr, y, coef, N, C, plane, alpha, beta, st);
  else launch_bn_apply<false, false>(x, nullptr, y, coef, N, C, plane, alpha, beta, st);
  return launch_status();
}

static int bnorm_bwd(int N, int C, int plane, float alpha_data, float beta_data, const float* x, const float* dy, float* dx,
                     float alpha_param, float beta_param, const float* scale, float* dscale, float* dbias,
                     const float* cached_mean, const float* cached_ivar, void* ws, size_t ws_bytes, const float* relu_bias,
                     rh_stream_t stream) {
  long long total;
  if (int e = bn_check(N, C, plane, &total)) return e;
  if (total == 0) return 0;
  if (!x || !dy || !dx || !scale || !dscale || !dbias || !cached_mean || !cached_ivar || !ws) return RH_E_INVALID;
  if (ws_bytes < rh_bnorm_workspace_bytes(N, C, plane)) return RH_E_WORKSPACE;
  hipStream_t st = to_stream(stream);
  const BnPlan p = bn_plan(N, C, plane);
  float2* part = static_cast<float2*>(ws);
  float4* coef = reinterpret_cast<float4*>(static_cast<char*>(ws) + bn_part_bytes(p, C));
  const bool vec = plane % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy)) & 15) == 0;
  {
    ProfScope prof("bnorm_bwd_reduce", 8.0 * (double)total, st);
    const dim3 grid(C, p.G);
    if (relu_bias) {
      const BnMask mk = {scale, cached_ivar, relu_bias};
      if (vec)
        hipLaunchKernelGGL((bn_reduce_kernel<1, true, true>), grid, dim3(256), 0, st, x, dy, cached_mean, C, plane, p.chunks,
                           p.units, part, mk);
      else
        hipLaunchKernelGGL((bn_reduce_kernel<1, false, true>), grid, dim3(256), 0, st, x, dy, cached_mean, C, plane, p.chunks,
                           p.units, part, mk);
    } else {
      if (vec)
        hipLaunchKernelGGL((bn_reduce_kernel<1, true>), grid, dim3(256), 0, st, x, dy, cached_mean, C, plane, p.chunks, p.units,
                           part, BnMask());
      else
        hipLaunchKernelGGL((bn_reduce_kernel<1, false>), grid, dim3(256), 0, st, x, dy, cached_mean, C, plane, p.chunks, p.units,
                           part, BnMask());
    }
    hipLaunchKernelGGL(bn_bwd_finish_kernel, dim3(cdiv(C, 64)), dim3(64), 0, st, part, p.G, C, (double)N * (double)plane,
                       alpha_param, beta_param, scale, dscale, dbias, cached_mean, cached_ivar, coef);
  }
  ProfScope prof("bnorm_bwd_apply", (beta_data != 0.0f ? 16.0 : 12.0) * (double)total, st);
  if (relu_bias) launch_bn_apply<true, false, true>(x, dy, dx, coef, N, C, plane, alpha_data, beta_data, st, relu_bias);
  else launch_bn_apply<true, false>(x, dy, dx, coef, N, C, plane, alpha_data, beta_data, st);
  return launch_status();
}

extern "C" int rh_bnorm_bwd(int N, int C, int plane, float alpha_data, float beta_data, const float* x, const float* dy,
                            float* dx, float alpha_param, float beta_param, double epsilon, const float* scale, float* dscale,
                            float* dbias, const float* cached_mean, const float* cached_ivar, void* ws, size_t ws_bytes,
                            rh_stream_t stream) {
  (void)epsilon;  // the cached inverse standard deviation of the forward pass is used
  return bnorm_bwd(N, C, plane, alpha_data, beta_data, x, dy, dx, alpha_param, beta_param, scale, dscale, dbias, cached_mean,
                   cached_ivar, ws, ws_bytes, nullptr, stream);
}

extern "C" int rh_bnorm_bwd_relu(int N, int C, int plane, float alpha_data, float beta_data, const float* x, const float* dy,
                                 float* dx, float alpha_param, float beta_param, double epsilon, const float* scale,
                                 const float* bias, float* dscale, float* dbias, const float* cached_mean,
                                 const float* cached_ivar, void* ws, size_t ws_bytes, rh_stream_t stream) {
  (void)epsilon;
  if (!bias) return RH_E_INVALID;
  return bnorm_bwd(N, C, plane, alpha_data, beta_data, x, dy, dx, alpha_param, beta_param, scale, dscale, dbias, cached_mean,
                   cached_ivar, ws, ws_bytes, bias, stream);
}
