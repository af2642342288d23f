// Bandwidth-bound elementwise kernels: bias add (K2), ReLU forward / backward (K3, K4), fills,
// u8 -> f32 casts.  All are grid-stride loops over 16-byte accesses when the pointers allow.
#include "common.h"

namespace rh {

thread_local int g_last_error = 0;

// y[(n*K + k)*plane + i] = alpha*bias[k] + beta*y[...]; grid = (plane chunks, N*K).
__global__ void add_bias_plane_kernel(const float* __restrict__ bias, float* __restrict__ y, int plane, int K,
                                      float alpha, float beta) {
  const int nk = blockIdx.y;
  const float b = alpha * bias[nk % K];
  float* p = y + (size_t)nk * plane;
  const int stride = gridDim.x * blockDim.x;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    const int n4 = plane >> 2;
    float4* p4 = reinterpret_cast<float4*>(p);
    for (int i = t; i < n4; i += stride) {
      float4 v = p4[i];
      v.x = fmaf(beta, v.x, b); v.y = fmaf(beta, v.y, b); v.z = fmaf(beta, v.z, b); v.w = fmaf(beta, v.w, b);
      p4[i] = v;
    }
    for (int i = (n4 << 2) + t; i < plane; i += stride) p[i] = fmaf(beta, p[i], b);
  } else {
    for (int i = t; i < plane; i += stride) p[i] = fmaf(beta, p[i], b);
  }
}

// Small planes (affine: plane == 1): flat index, channel = (idx / plane) % K.
__global__ void add_bias_flat_kernel(const float* __restrict__ bias, float* __restrict__ y, int plane, int K,
                                     long long total, float alpha, float beta) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int k = (int)((i / plane) % K);
    y[i] = fmaf(beta, y[i], alpha * bias[k]);
  }
}

__global__ void rect_inplace_kernel(float* __restrict__ y, long long n) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(y) & 15) == 0) {
    const long long n4 = n >> 2;
    float4* y4 = reinterpret_cast<float4*>(y);
    for (long long i = t; i < n4; i += stride) {
      float4 v = y4[i];
      v.x = v.x > 0.0f ? v.x : 0.0f; v.y = v.y > 0.0f ? v.y : 0.0f;
      v.z = v.z > 0.0f ? v.z : 0.0f; v.w = v.w > 0.0f ? v.w : 0.0f;
      y4[i] = v;
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) y[i] = y[i] > 0.0f ? y[i] : 0.0f;
  } else {
    for (long long i = t; i < n; i += stride) y[i] = y[i] > 0.0f ? y[i] : 0.0f;
  }
}

__global__ void rect_backprop_inplace_kernel(const float* __restrict__ y, float* __restrict__ dy, long long n) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(dy)) & 15) == 0) {
    const long long n4 = n >> 2;
    const float4* y4 = reinterpret_cast<const float4*>(y);
    float4* d4 = reinterpret_cast<float4*>(dy);
    for (long long i = t; i < n4; i += stride) {
      const float4 a = y4[i];
      float4 d = d4[i];
      d.x = a.x > 0.0f ? d.x : 0.0f; d.y = a.y > 0.0f ? d.y : 0.0f;
      d.z = a.z > 0.0f ? d.z : 0.0f; d.w = a.w > 0.0f ? d.w : 0.0f;
      d4[i] = d;
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) dy[i] = y[i] > 0.0f ? dy[i] : 0.0f;
  } else {
    for (long long i = t; i < n; i += stride) dy[i] = y[i] > 0.0f ? dy[i] : 0.0f;
  }
}

__global__ void fill_kernel(float* __restrict__ d, float v, long long n) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(d) & 15) == 0) {
    const long long n4 = n >> 2;
    float4* d4 = reinterpret_cast<float4*>(d);
    const float4 v4 = make_float4(v, v, v, v);
    for (long long i = t; i < n4; i += stride) d4[i] = v4;
    for (long long i = (n4 << 2) + t; i < n; i += stride) d[i] = v;
  } else {
    for (long long i = t; i < n; i += stride) d[i] = v;
  }
}

__global__ void cast_u8_f32_kernel(const uint8_t* __restrict__ x, float* __restrict__ y, long long n, float scale) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
    const long long n4 = n >> 2;
    const uchar4* x4 = reinterpret_cast<const uchar4*>(x);
    float4* y4 = reinterpret_cast<float4*>(y);
    for (long long i = t; i < n4; i += stride) {
      const uchar4 a = x4[i];
      y4[i] = make_float4(scale * (float)a.x, scale * (float)a.y, scale * (float)a.z, scale * (float)a.w);
    }
    for (long long i = (n4 << 2) + t; i < n; i += stride) y[i] = scale * (float)x[i];
  } else {
    for (long long i = t; i < n; i += stride) y[i] = scale * (float)x[i];
  }
}

}  // namespace rh

using namespace rh;

extern "C" int rh_last_error(void) { return g_last_error; }

extern "C" int rh_add_bias_nchw(const float* bias, float* y, int32_t plane, int32_t K, int32_t N, float alpha,
                                float beta, rh_stream_t stream) {
  if (!bias || !y || plane <= 0 || K <= 0 || N <= 0) return RH_E_INVALID;
  ProfScope prof("add_bias", 8.0 * (double)plane * K * N, to_stream(stream));
  if (plane >= 256 && (long long)N * K <= 65535) {
    dim3 grid((unsigned)cdiv(plane, 256 * 4), (unsigned)(N * K));
    hipLaunchKernelGGL(add_bias_plane_kernel, grid, dim3(256), 0, to_stream(stream), bias, y, plane, K, alpha, beta);
  } else {
    const long long total = (long long)plane * K * N;
    hipLaunchKernelGGL(add_bias_flat_kernel, dim3(stream_grid((size_t)total, 256)), dim3(256), 0,
                       to_stream(stream), bias, y, plane, K, total, alpha, beta);
  }
  return launch_status();
}

extern "C" void rembrandt_kernel_batch_map_rect_inplace(float* y, int32_t frame_len, int32_t batch,
                                                        rh_stream_t stream) {
  const long long n = (long long)frame_len * batch;
  if (n <= 0 || !y) { g_last_error = n == 0 ? 0 : RH_E_INVALID; return; }
  ProfScope prof("rect_fwd", 8.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(rect_inplace_kernel, dim3(stream_grid((size_t)(n + 3) / 4, 256)), dim3(256), 0,
                     to_stream(stream), y, n);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_batch_map_rect_backprop_inplace(const float* y, int32_t frame_len, int32_t batch,
                                                                 float* dy, rh_stream_t stream) {
  const long long n = (long long)frame_len * batch;
  if (n <= 0 || !y || !dy) { g_last_error = n == 0 ? 0 : RH_E_INVALID; return; }
  ProfScope prof("rect_bwd", 12.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(rect_backprop_inplace_kernel, dim3(stream_grid((size_t)(n + 3) / 4, 256)), dim3(256), 0,
                     to_stream(stream), y, dy, n);
  g_last_error = launch_status();
}

extern "C" int rh_memset_f32(float* d, float value, size_t n, rh_stream_t stream) {
  if (n == 0) return 0;
  if (!d) return RH_E_INVALID;
  ProfScope prof("fill", 4.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(fill_kernel, dim3(stream_grid((n + 3) / 4, 256)), dim3(256), 0, to_stream(stream), d, value,
                     (long long)n);
  return launch_status();
}

extern "C" int rh_cast_u8_f32(const uint8_t* x, float* y, size_t n, float scale, rh_stream_t stream) {
  if (n == 0) return 0;
  if (!x || !y) return RH_E_INVALID;
  ProfScope prof("cast_u8_f32", 5.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(cast_u8_f32_kernel, dim3(stream_grid((n + 3) / 4, 256)), dim3(256), 0, to_stream(stream), x,
                     y, (long long)n, scale);
  return launch_status();
}
