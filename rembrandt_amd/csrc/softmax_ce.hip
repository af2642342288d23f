// Softmax, KL/cross-entropy backward, per-sample loss, row sum and row arg-max (K10-K13).
// One 256-thread block per sample row; rows are reduced with wavefront shuffles and one LDS
// stage, so there is no limit on the row length (the reference's kernels assert <= 1024).
#include <math.h>

#include "common.h"

namespace rh {

__device__ __forceinline__ float block_reduce_sum(float v, float* sm) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) sm[wave] = v;
  __syncthreads();
  float r = 0.0f;
  for (int i = 0; i < nw; ++i) r += sm[i];
  __syncthreads();
  return r;
}

__device__ __forceinline__ float block_reduce_max(float v, float* sm) {
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_down(v, o, 64));
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) sm[wave] = v;
  __syncthreads();
  float r = sm[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, sm[i]);
  __syncthreads();
  return r;
}

// p[n,:] = exp(x[n,:] - max) / sum exp(x[n,:] - max)
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const float* __restrict__ x, float* __restrict__ p, int C) {
  __shared__ float sm[4];
  const float* xr = x + (size_t)blockIdx.x * C;
  float* pr = p + (size_t)blockIdx.x * C;
  float mx = -INFINITY;
  for (int c = threadIdx.x; c < C; c += blockDim.x) mx = fmaxf(mx, xr[c]);
  mx = block_reduce_max(mx, sm);
  float z = 0.0f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) z += expf(xr[c] - mx);
  z = block_reduce_sum(z, sm);
  const float inv = 1.0f / z;
  for (int c = threadIdx.x; c < C; c += blockDim.x) pr[c] = expf(xr[c] - mx) * inv;
}

// dx[n,c] = weights[n] * (p[n,c] - [c == labels[n]])
__global__ void softmax_kl_backward_kernel(const float* __restrict__ p, int C, long long total,
                                           const int* __restrict__ labels, const float* __restrict__ weights,
                                           float* __restrict__ dx) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int n = (int)(i / C), c = (int)(i - (long long)n * C);
    dx[i] = weights[n] * (p[i] - (c == labels[n] ? 1.0f : 0.0f));
  }
}

// loss1[n] = beta*loss1[n] - weights[n]*log p[n, labels[n]]   (a label outside [0,C) yields NaN)
__global__ void softmax_kl_loss1_kernel(const float* __restrict__ p, int C, int N, const int* __restrict__ labels,
                                        const float* __restrict__ weights, float beta, float* __restrict__ loss1) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const int l = labels[n];
  float v = (unsigned)l < (unsigned)C ? -weights[n] * logf(p[(size_t)n * C + l]) : NAN;
  if (beta != 0.0f) v += beta * loss1[n];
  loss1[n] = v;
}

// dst[b] = beta*dst[b] + sum_i src[b*len + i]
__global__ __launch_bounds__(256) void blockreduce_sum_kernel(const float* __restrict__ src, int len,
                                                              float* __restrict__ dst, float beta) {
  __shared__ float sm[4];
  const float* r = src + (size_t)blockIdx.x * len;
  float acc = 0.0f;
  for (int i = threadIdx.x; i < len; i += blockDim.x) acc += r[i];
  acc = block_reduce_sum(acc, sm);
  if (threadIdx.x == 0) dst[blockIdx.x] = beta != 0.0f ? beta * dst[blockIdx.x] + acc : acc;
}

// Row maximum and the lowest index attaining it.
__global__ __launch_bounds__(256) void blockreduce_argmax_kernel(const float* __restrict__ src, int len,
                                                                 float* __restrict__ max_out,
                                                                 int* __restrict__ idx_out) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const float* r = src + (size_t)blockIdx.x * len;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < len; i += blockDim.x) {
    const float v = r[i];
    if (v > best || bi == 0x7fffffff) { best = v; bi = i; }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_down(best, o, 64);
    const int oi = __shfl_down(bi, o, 64);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sv[wave] = best; si[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      const float ov = sv[w];
      const int oi = si[w];
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
    }
    max_out[blockIdx.x] = best;
    idx_out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

// Everything a train step takes from the loss operator, in one launch of one block per sample row: softmax_fwd, the
// row arg-max of the probabilities, loss1 (factor 0), the KL backward into dx, and, by the block that finishes last
// (a device-wide counter that this block leaves at zero again), blockreduce_sum of loss1 into loss_sum.  Each value is
// formed by the same operations in the same order as in the separate kernels above: the results are bit-identical.
__global__ __launch_bounds__(256) void softmax_kl_step_kernel(const float* __restrict__ x, int C, int N,
                                                              const int* __restrict__ labels,
                                                              const float* __restrict__ weights, float* __restrict__ p,
                                                              float* __restrict__ max_out, int* __restrict__ idx_out,
                                                              float* __restrict__ loss1, float* __restrict__ loss_sum,
                                                              float* __restrict__ dx, unsigned* __restrict__ counter) {
  __shared__ float sm[4];
  __shared__ float sv[4];
  __shared__ int si[4];
  __shared__ bool last;
  const int n = blockIdx.x;
  const float* xr = x + (size_t)n * C;
  float* pr = p + (size_t)n * C;
  float* dr = dx + (size_t)n * C;
  float mx = -INFINITY;
  for (int c = threadIdx.x; c < C; c += blockDim.x) mx = fmaxf(mx, xr[c]);
  mx = block_reduce_max(mx, sm);
  float z = 0.0f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) z += expf(xr[c] - mx);
  z = block_reduce_sum(z, sm);
  const float inv = 1.0f / z;
  const int label = labels[n];
  const float wgt = weights[n];
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float v = expf(xr[c] - mx) * inv;
    asm volatile("" : "+v"(v));   // the rounded product, as the separate kernels read it back: no fused multiply-subtract below
    pr[c] = v;
    if (v > best || bi == 0x7fffffff) { best = v; bi = c; }
    dr[c] = wgt * (v - (c == label ? 1.0f : 0.0f));
    if (c == label) loss1[n] = -wgt * logf(v);
  }
  if (threadIdx.x == 0 && (unsigned)label >= (unsigned)C) loss1[n] = NAN;
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_down(best, o, 64);
    const int oi = __shfl_down(bi, o, 64);
    if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sv[wave] = best; si[wave] = bi; }
  __threadfence();   // this row's loss1 is visible device-wide before the block is counted
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      const float ov = sv[w];
      const int oi = si[w];
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
    }
    max_out[n] = best;
    idx_out[n] = bi == 0x7fffffff ? 0 : bi;
    last = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)N - 1u;
  }
  __syncthreads();
  if (!last) return;
  __threadfence();
  float acc = 0.0f;
  if (blockDim.x == 64) {
    // one wave adds in the order 256 threads would: lane l stands for threads l, 64 + l, 128 + l, 192 + l, each of the
    // four groups goes through the wave's tree, and the four results are added in wave order
    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      for (int i = 64 * w + (int)threadIdx.x; i < N; i += 256)
        part[w] += __hip_atomic_load(loss1 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (int o = 32; o > 0; o >>= 1) part[w] += __shfl_down(part[w], o, 64);
    }
    acc = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) acc += part[w];
  } else {
    for (int i = threadIdx.x; i < N; i += blockDim.x)
      acc += __hip_atomic_load(loss1 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    acc = block_reduce_sum(acc, sm);
  }
  if (threadIdx.x == 0) {
    loss_sum[0] = acc;
    *counter = 0u;
  }
}

}  // namespace rh

using namespace rh;

extern "C" int rh_softmax_fwd(const float* x, float* p, int32_t C, int32_t N, rh_stream_t stream) {
  if (!x || !p || C <= 0 || N < 0) return RH_E_INVALID;
  if (N == 0) return 0;
  ProfScope prof("softmax_fwd", 8.0 * (double)C * N, to_stream(stream));
  hipLaunchKernelGGL(softmax_fwd_kernel, dim3(N), dim3(256), 0, to_stream(stream), x, p, C);
  return launch_status();
}

extern "C" void rembrandt_kernel_batch_map_softmax_kl_backward(const float* p, int32_t C, int32_t N,
                                                               const int32_t* labels, const float* weights,
                                                               float* dx, rh_stream_t stream) {
  if (!p || !labels || !weights || !dx || C <= 0 || N < 0) { g_last_error = RH_E_INVALID; return; }
  if (N == 0) { g_last_error = 0; return; }
  const long long total = (long long)C * N;
  ProfScope prof("softmax_kl_backward", 8.0 * (double)total, to_stream(stream));
  hipLaunchKernelGGL(softmax_kl_backward_kernel, dim3(stream_grid((size_t)total, 256)), dim3(256), 0,
                     to_stream(stream), p, C, total, labels, weights, dx);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_batch_map_softmax_kl_loss1(const float* p, int32_t C, int32_t N,
                                                            const int32_t* labels, const float* weights,
                                                            float beta, float* loss1, rh_stream_t stream) {
  if (!p || !labels || !weights || !loss1 || C <= 0 || N < 0) { g_last_error = RH_E_INVALID; return; }
  if (N == 0) { g_last_error = 0; return; }
  hipLaunchKernelGGL(softmax_kl_loss1_kernel, dim3(cdiv(N, 256)), dim3(256), 0, to_stream(stream), p, C, N, labels,
                     weights, beta, loss1);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_batch_blockreduce_sum(const float* src, int32_t len, int32_t batch, float* dst,
                                                       float beta, rh_stream_t stream) {
  if (!src || !dst || len < 0 || batch < 0) { g_last_error = RH_E_INVALID; return; }
  if (batch == 0) { g_last_error = 0; return; }
  hipLaunchKernelGGL(blockreduce_sum_kernel, dim3(batch), dim3(256), 0, to_stream(stream), src, len, dst, beta);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_batch_blockreduce_argmax(const float* src, int32_t len, int32_t batch,
                                                          float* max_out, int32_t* idx_out, rh_stream_t stream) {
  if (!src || !max_out || !idx_out || len <= 0 || batch < 0) { g_last_error = RH_E_INVALID; return; }
  if (batch == 0) { g_last_error = 0; return; }
  ProfScope prof("argmax", 4.0 * (double)len * batch, to_stream(stream));
  hipLaunchKernelGGL(blockreduce_argmax_kernel, dim3(batch), dim3(256), 0, to_stream(stream), src, len, max_out,
                     idx_out);
  g_last_error = launch_status();
}

extern "C" int rh_softmax_kl_step(const float* x, int32_t C, int32_t N, const int32_t* labels, const float* weights,
                                  float* p, float* max_out, int32_t* idx_out, float* loss1, float* loss_sum, float* dx,
                                  uint32_t* counter, rh_stream_t stream) {
  if (!x || !labels || !weights || !p || !max_out || !idx_out || !loss1 || !loss_sum || !dx || !counter || C <= 0 || N < 0)
    return RH_E_INVALID;
  if (N == 0) return 0;
  ProfScope prof("softmax_kl_step", 16.0 * (double)C * N, to_stream(stream));
  // Up to 64 categories one wave holds a whole row: the other three would only add identities to the block's reductions
  // (same bits) and take part in its barriers and its fence.
  hipLaunchKernelGGL(softmax_kl_step_kernel, dim3(N), dim3(C <= 64 ? 64 : 256), 0, to_stream(stream), x, C, N, labels, weights,
                     p, max_out, idx_out, loss1, loss_sum, dx, counter);
  return launch_status();
}
