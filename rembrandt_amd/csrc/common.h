// Shared helpers of the HIP translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rembrandt_hip.h"

namespace rh {

inline hipStream_t to_stream(rh_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Status of the last launch made through a void rembrandt_kernel_* entry point (per thread).
extern thread_local int g_last_error;

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

template <class T>
constexpr T cdiv(T a, T b) { return (a + b - 1) / b; }

// Largest tensor the buffer-addressed kernels accept: byte offsets are 32-bit and the value
// 0x80000000 is reserved as the "out of range, reads as zero" offset.
constexpr size_t kMaxBufferBytes = size_t(1) << 31;

constexpr int kWave = 64;

// Grid size for a streaming kernel: one work item (normally a 16-byte group) per thread, so the kernels' grid-stride
// loops run once.  Measured on a 1 GiB copy: 4096 blocks striding through the array reach 4.6 TB/s, one float4 per
// thread over 262144 blocks 6.2 TB/s (consecutive blocks sweep the address space in order instead of every wave
// touching pages 16 MB apart).
inline int stream_grid(size_t work_items, int block) {
  size_t want = cdiv<size_t>(work_items, static_cast<size_t>(block));
  const size_t cap = (size_t(1) << 31) - 1;
  if (want > cap) want = cap;
  if (want < 1) want = 1;
  return static_cast<int>(want);
}

// Division of a non-negative 32-bit index (< 2^31) by a runtime constant as multiply-high + add + shift
// (Granlund-Montgomery round-up method); the divisor's constants are computed once on the host.  The
// bandwidth-bound kernels decompose a flat index per element: hardware integer division there costs
// more instructions than everything else in the kernel.
struct FastDiv {
  uint32_t mul, shift, div;
  __host__ __device__ FastDiv() : mul(1), shift(0), div(1) {}
  explicit FastDiv(uint32_t d) : div(d) {
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    mul = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    shift = l;
  }
  __host__ __device__ __forceinline__ uint32_t quot(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    return (__umulhi(mul, n) + n) >> shift;
#else
    return (uint32_t)((((uint64_t)mul * n) >> 32) + n) >> shift;
#endif
  }
  // n = q*div + r
  __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
    q = quot(n);
    r = n - q * div;
  }
};

// Optional per-launch timing with HIP events (off by default; rh_profile_enable).  A scope
// records an event before and after the launches made inside it, on the stream they go to.
// `work` is the algorithmic work of those launches: FLOPs for contractions, bytes otherwise.
struct ProfScope {
  ProfScope(const char* tag, double work, hipStream_t stream);
  ~ProfScope();
  void* slot;
  hipStream_t stream;
};
extern bool g_profile_enabled;

// Per-device address of the library's static scratch array (see rh_conv2d_bwd_bias_noalloc); looks it up on the
// current device the first time.  `out` may be null.
int static_scratch_lookup(void** out);

}  // namespace rh
