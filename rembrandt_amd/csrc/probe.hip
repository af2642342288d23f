// Calibration kernels for the roofline report: a register-only fp32 MFMA loop (what fraction of the
// datasheet matrix peak the clocks actually sustain) and a plain copy (sustained HBM bandwidth); and the figures the
// bf16 kernels are designed against: a register-only bf16 MFMA loop and the rates of the ways into and out of the LDS.
#include "gemm_core.h"

namespace rh {

// Each wave runs `iters` rounds of NACC independent v_mfma_f32_32x32x2_f32 on register operands.
template <int NACC>
__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, float* sink) {
  f32x16 acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
  float a = (float)threadIdx.x * 1e-3f, b = (float)blockIdx.x * 1e-3f + 1.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  if (s == 123.456f) sink[0] = s;  // keeps the loop alive; never true in practice
}

// Same loop with operands that differ per lane and per instruction (8 A and 8 B registers of pseudo-random
// values in [-2, 2), rotated through): the data toggling of a real contraction, hence its power draw, which the
// constant-operand loop above does not have.
__global__ __launch_bounds__(256) void mfma_loop_varied_kernel(int iters, float* sink) {
  f32x16 acc[8];
  float a[8], b[8];
  uint32_t h = (threadIdx.x + 1u) * 2654435761u ^ (blockIdx.x + 1u) * 40503u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    h = h * 1664525u + 1013904223u;
    a[i] = (float)(int)(h >> 8) * (1.0f / 4194304.0f) - 2.0f;
    h = h * 1664525u + 1013904223u;
    b[i] = (float)(int)(h >> 8) * (1.0f / 4194304.0f) - 2.0f;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = a[i] * (float)v;
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[(i * 3 + 1) & 7], acc[i], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[(i + 5) & 7], b[i], acc[i], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  if (s == 123.456f) sink[0] = s;
}

__global__ void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, long long n4) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

}  // namespace rh

using namespace rh;

// Launches blocks x 256 threads; every wave issues iters * nacc MFMAs (nacc in {4, 8}).  FLOPs of the
// launch = blocks * 4 waves * iters * nacc * 4096.
extern "C" int rh_probe_mfma_loop(int blocks, int nacc, int iters, float* sink, rh_stream_t stream) {
  if (blocks <= 0 || iters <= 0 || !sink) return RH_E_INVALID;
  ProfScope prof("probe_mfma_loop", (double)blocks * 4.0 * iters * nacc * 4096.0, to_stream(stream));
  if (nacc == 4) hipLaunchKernelGGL(mfma_loop_kernel<4>, dim3(blocks), dim3(256), 0, to_stream(stream), iters, sink);
  else if (nacc == 8) hipLaunchKernelGGL(mfma_loop_kernel<8>, dim3(blocks), dim3(256), 0, to_stream(stream), iters, sink);
  else return RH_E_INVALID;
  return launch_status();
}

// Launches blocks x 256 threads; every wave issues iters * 16 MFMAs on varied operands.
extern "C" int rh_probe_mfma_loop_varied(int blocks, int iters, float* sink, rh_stream_t stream) {
  if (blocks <= 0 || iters <= 0 || !sink) return RH_E_INVALID;
  ProfScope prof("probe_mfma_varied", (double)blocks * 4.0 * iters * 16 * 4096.0, to_stream(stream));
  hipLaunchKernelGGL(mfma_loop_varied_kernel, dim3(blocks), dim3(256), 0, to_stream(stream), iters, sink);
  return launch_status();
}

// dst[0..n) = src[0..n); n a multiple of 4, both 16-byte aligned.  Bytes moved = 8 * n.
extern "C" int rh_probe_copy(const float* src, float* dst, size_t n, rh_stream_t stream) {
  if (!src || !dst || n == 0 || (n & 3) || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15))
    return RH_E_INVALID;
  ProfScope prof("probe_copy", 8.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(copy_kernel, dim3(stream_grid(n / 4, 256)), dim3(256), 0, to_stream(stream),
                     reinterpret_cast<const float4*>(src), reinterpret_cast<float4*>(dst), (long long)(n / 4));
  return launch_status();
}
