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

// Register-only loop of v_mfma_f32_32x32x16_bf16: sixteen accumulators per wave, four A and four B operands of
// pseudo-random bf16 values, the A operands rotated every round.
__global__ __launch_bounds__(256, 1) void bf16_mfma_loop_kernel(int iters, float* sink) {
  f32x16 acc[4][4];
  uint4 a[4], b[4];
  uint32_t h = (threadIdx.x + 1u) * 2654435761u ^ (blockIdx.x + 1u) * 40503u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t* pa = reinterpret_cast<uint32_t*>(&a[i]);
    uint32_t* pb = reinterpret_cast<uint32_t*>(&b[i]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {  // two bf16 per dword, magnitudes in [0.5, 2)
      h = h * 1664525u + 1013904223u;
      pa[e] = 0x3f003f00u | ((h >> 8) & 0x00ff00ffu) | ((h & 1u) << 31);
      h = h * 1664525u + 1013904223u;
      pb[e] = 0x3f003f00u | ((h >> 8) & 0x00ff00ffu) | ((h & 2u) << 14);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]), __builtin_bit_cast(bf16x8_t, b[j]),
                                                            acc[i][j], 0, 0, 0);
    const uint4 t = a[0]; a[0] = a[1]; a[1] = a[2]; a[2] = a[3]; a[3] = t;
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  if (s == 123.456f) sink[0] = s;
}

// The ways into and out of the LDS, 64 bytes per thread and round, 16 bytes per access, consecutive lanes on
// consecutive 16-byte pieces (no bank conflicts): MODE 0 ds_read_b128, 1 ds_write_b128, 2 direct global -> LDS loads
// (buffer_load_dwordx4 ... lds) from a 64 KB window of `src` per block (cache hits: the rate of the path, not of HBM).
template <int MODE>
__global__ __launch_bounds__(512, 1) void lds_path_kernel(const uint4* __restrict__ src, int iters, float* sink) {
  extern __shared__ float lds_dyn[];
  uint4* const lds = reinterpret_cast<uint4*>(lds_dyn);   // 64 KB
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int i = tid; i < 4096; i += nt) lds[i] = make_uint4(i, 1u, 2u, 3u);
  __syncthreads();
  uint4 keep = make_uint4(tid, 0u, 0u, 0u);
  if (MODE == 2) {
    u32x4 rsrc;
    const uint64_t a = reinterpret_cast<uint64_t>(src);
    rsrc.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
    rsrc.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    rsrc.z = 0x40000000u;
    rsrc.w = 0x00020000u;
    const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dma_load16(rsrc, base + (uint32_t)(((it & 3) * 4 + i) & 7) * (uint32_t)nt * 16u + wave * 1024u, (uint32_t)tid * 16u,
                   (uint32_t)((blockIdx.x & 255) * 65536 + (((it & 1) * 4 + i) * nt) * 16));
    }
    wait_vmcnt<0>();
  } else {
    if (MODE == 0) {
      for (int it = 0; it < iters; it += 2) {   // two rounds' reads in flight together
        uint4 q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = lds[i * nt + tid];
#pragma unroll
        for (int i = 0; i < 8; ++i) { keep.x ^= q[i].x; keep.y += q[i].y; keep.z ^= q[i].z; keep.w += q[i].w; }
        asm volatile("" ::: "memory");   // every round goes to the LDS again
      }
    } else {
      for (int it = 0; it < iters; ++it) {
        const int base = (it & 1) * 4 * nt;
#pragma unroll
        for (int i = 0; i < 4; ++i) lds[base + i * nt + tid] = keep;
        keep.x += 1u;
        asm volatile("" ::: "memory");
      }
    }
  }
  __syncthreads();
  const uint4 q = lds[tid];
  if (q.x + keep.x + keep.y + keep.z + keep.w == 0x12345678u) sink[0] = 1.0f;
}

}  // namespace rh

using namespace rh;

// blocks x 256 threads; every wave issues iters * 16 bf16 MFMAs (32768 FLOP each).
extern "C" int rh_probe_bf16_mfma_loop(int blocks, int iters, float* sink, rh_stream_t stream) {
  if (blocks <= 0 || iters <= 0 || !sink) return RH_E_INVALID;
  ProfScope prof("probe_bf16_mfma_loop", (double)blocks * 4.0 * iters * 16 * 32768.0, to_stream(stream));
  hipLaunchKernelGGL(bf16_mfma_loop_kernel, dim3(blocks), dim3(256), 0, to_stream(stream), iters, sink);
  return launch_status();
}

// mode 0 / 1 / 2: LDS reads, LDS writes, direct global -> LDS loads; blocks x threads (256 or 512), 64 bytes per thread
// and round.  `src` (mode 2): at least 16 MiB, 16-byte aligned.  The profile tag carries the bytes moved.
extern "C" int rh_probe_lds_path(int mode, int blocks, int threads, int iters, const float* src, float* sink,
                                 rh_stream_t stream) {
  if (blocks <= 0 || iters <= 0 || !sink || (threads != 256 && threads != 512) || mode < 0 || mode > 2) return RH_E_INVALID;
  if (mode == 2 && (!src || (reinterpret_cast<uintptr_t>(src) & 15))) return RH_E_INVALID;
  static const char* tags[3] = {"probe_lds_read", "probe_lds_write", "probe_lds_direct_load"};
  const void* fn = mode == 0 ? (const void*)&lds_path_kernel<0> : mode == 1 ? (const void*)&lds_path_kernel<1>
                                                                           : (const void*)&lds_path_kernel<2>;
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 65536) != hipSuccess) return RH_E_UNSUPPORTED;
  ProfScope prof(tags[mode], (double)blocks * threads * iters * 64.0, to_stream(stream));
  const uint4* s4 = reinterpret_cast<const uint4*>(src);
  if (mode == 0) hipLaunchKernelGGL(lds_path_kernel<0>, dim3(blocks), dim3(threads), 65536, to_stream(stream), s4, iters, sink);
  else if (mode == 1) hipLaunchKernelGGL(lds_path_kernel<1>, dim3(blocks), dim3(threads), 65536, to_stream(stream), s4, iters, sink);
  else hipLaunchKernelGGL(lds_path_kernel<2>, dim3(blocks), dim3(threads), 65536, to_stream(stream), s4, iters, sink);
  return launch_status();
}

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
