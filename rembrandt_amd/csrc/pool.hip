// Max / average pooling, forward and backward (K9 batch form, K9' arg-max mask + ceil extent).
// Forward: one thread per output element scans its window (r outer, s inner; the first maximum
// wins; padding never wins; the average divisor is always size*size).
// Backward: one thread per *input* element gathers from every window that covers it, so
// overlapping windows (3x3 stride 2) need no atomics and the sum order is fixed.
#include "common.h"

namespace rh {

struct PoolDims { int N, C, H, W, k, st, pad, P, Q, mode; FastDiv dP, dQ, dH, dW, dSt, dK; };

// The arg-max mask of a max-pool comes in two encodings.  int32: the index h*W + w of the winning element inside its
// plane, -1 for a window without elements (the form of rh_pool2d_fwd / rh_pool2d_bwd).  uint8: the winner's slot
// r*size + s inside its window, 255 for none (size <= 15): a quarter of the bytes, for an operator's private mask.
template <class MT> struct MaskCode;
template <> struct MaskCode<int> {
  // plane: index inside the plane (or -1); hs, ws: the window's first row / column
  static __device__ __forceinline__ int from_plane(int plane, int, int, int, int) { return plane; }
  static __device__ __forceinline__ int to_plane(int m, int, int, const PoolDims&) { return m; }
};
template <> struct MaskCode<uint8_t> {
  static __device__ __forceinline__ uint8_t from_plane(int plane, int hs, int ws, int W, int k) {
    if (plane < 0) return 255;
    const int h = plane / W, w = plane - h * W;
    return (uint8_t)((h - hs) * k + (w - ws));
  }
  static __device__ __forceinline__ int to_plane(uint8_t m, int hs, int ws, const PoolDims& d) {
    if (m == 255) return -1;
    const uint32_t r = d.dK.quot(m), s2 = m - r * (uint32_t)d.k;
    return (hs + (int)r) * d.W + ws + (int)s2;
  }
};

inline int pool_out_dim(int in, int size, int stride, int pad, int round) {
  if (round == RH_ROUND_CEIL) {
    // max(0, in + 2*pad - size + stride - 1)/stride + 1 (src/layer.rs:1741-1747)
    int t = in + 2 * pad - size + stride - 1;
    if (t < 0) t = 0;
    return t / stride + 1;
  }
  int t = in + 2 * pad - size + stride;
  if (t < 0) t = 0;
  return t / stride;
}

// `xp[i - base]` holds plane element i (base > 0: only the rows from base / W on are staged).
__device__ __forceinline__ int window_argmax(const float* __restrict__ xp, int H, int W, int p, int q, int k, int st,
                                             int pad, float* best_out, int base = 0) {
  float best = 0.0f;
  int bi = -1;
  const int hs = p * st - pad, ws = q * st - pad;
  for (int r = 0; r < k; ++r) {
    const int h = hs + r;
    if ((unsigned)h >= (unsigned)H) continue;
    for (int s = 0; s < k; ++s) {
      const int w = ws + s;
      if ((unsigned)w >= (unsigned)W) continue;
      const float v = xp[h * W + w - base];
      if (bi < 0 || v > best) { best = v; bi = h * W + w; }
    }
  }
  *best_out = best;
  return bi;
}

// I is the flat index type: 32-bit whenever the tensors allow it (64-bit divisions cost ~10x more).
template <class I>
__global__ void pool_fwd_kernel(PoolDims d, const float* __restrict__ x, float* __restrict__ y,
                                int* __restrict__ argmax) {
  const I total = (I)d.N * d.C * d.P * d.Q;
  const I stride = (I)gridDim.x * blockDim.x;
  const float inv = 1.0f / (float)(d.k * d.k);
  for (I idx = (I)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    I t, nc;
    int q, p;
    if (sizeof(I) == 4) {
      uint32_t t32, q32, nc32, p32;
      d.dQ.divmod((uint32_t)idx, t32, q32);
      d.dP.divmod(t32, nc32, p32);
      t = t32; nc = nc32; q = (int)q32; p = (int)p32;
    } else {
      t = idx / (I)d.Q;
      q = (int)(idx - t * (I)d.Q);
      nc = t / (I)d.P;
      p = (int)(t - nc * (I)d.P);
    }
    const float* xp = x + (size_t)nc * d.H * d.W;
    if (d.mode == RH_POOL_MAX) {
      float best;
      const int bi = window_argmax(xp, d.H, d.W, p, q, d.k, d.st, d.pad, &best);
      y[idx] = bi < 0 ? 0.0f : best;
      if (argmax) argmax[idx] = bi;
    } else {
      float acc = 0.0f;
      const int hs = p * d.st - d.pad, ws = q * d.st - d.pad;
      for (int r = 0; r < d.k; ++r) {
        const int h = hs + r;
        if ((unsigned)h >= (unsigned)d.H) continue;
        for (int s = 0; s < d.k; ++s) {
          const int w = ws + s;
          if ((unsigned)w < (unsigned)d.W) acc += xp[h * d.W + w];
        }
      }
      y[idx] = acc * inv;
    }
  }
}

// Max pooling on packed bf16 activations ([n][H][C/8][W][8] in, [n][P + 2*halo][C/8][Q + 2*halo][8] out, the border left
// alone): one thread per output group of eight channels, same scan order and tie rule as above on each channel.
// Rounding to bf16 is monotone, so the maximum of the rounded values is the rounded maximum: a chain that keeps its
// activations packed gets the values a consumer would have rounded from the fp32 result.
__global__ __launch_bounds__(256) void pool_max_fwd_bf16_kernel(PoolDims d, FastDiv dCg, const uint4* __restrict__ x,
                                                               uint4* __restrict__ y, unsigned total, int halo) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  uint32_t t, q, cg, n, p;
  d.dQ.divmod(i, t, q);
  dCg.divmod(t, t, cg);
  d.dP.divmod(t, n, p);
  const int Cg = (int)dCg.div;
  const int hs = (int)p * d.st - d.pad, ws = (int)q * d.st - d.pad;
  float best[8];
  bool any = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) best[e] = 0.0f;
  for (int r = 0; r < d.k; ++r) {
    const int h = hs + r;
    if ((unsigned)h >= (unsigned)d.H) continue;
    const uint4* row = x + ((size_t)((int)n * d.H + h) * Cg + cg) * d.W;
    for (int s = 0; s < d.k; ++s) {
      const int w = ws + s;
      if ((unsigned)w >= (unsigned)d.W) continue;
      const uint4 v = row[w];
      const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __builtin_bit_cast(float, u[e] << 16), hi = __builtin_bit_cast(float, u[e] & 0xffff0000u);
        if (!any || lo > best[2 * e]) best[2 * e] = lo;
        if (!any || hi > best[2 * e + 1]) best[2 * e + 1] = hi;
      }
      any = true;
    }
  }
  uint4 o;
  uint32_t* po = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
  for (int e = 0; e < 4; ++e)   // the values are bf16 already: their upper halves are the encoding
    po[e] = (__builtin_bit_cast(uint32_t, best[2 * e]) >> 16) | (__builtin_bit_cast(uint32_t, best[2 * e + 1]) & 0xffff0000u);
  const int Pp = d.P + 2 * halo, Qp = d.Q + 2 * halo;
  y[((size_t)((int)n * Pp + (int)p + halo) * Cg + cg) * Qp + q + halo] = o;
}

// Forward with the input planes of a block staged in LDS: PB consecutive (n, c) planes are read with coalesced
// loads, windows are scanned in LDS (overlapping windows re-read LDS, not L1), and y / arg-max are written
// coalesced.  Same arithmetic and tie rule as pool_fwd_kernel.
// K, ST > 0 fix the window size and stride at compile time: windows that lie inside the plane (all of them without
// padding and with an exact cover) are scanned by unrolled code from one base address, in the same order.
// Planes above the block's LDS share are cut into bands of `rb` output rows (bands > 1, PB = 1): a block stages the
// input rows its band's windows reach, a contiguous piece of the plane.
template <int K, int ST, class MT>
__global__ __launch_bounds__(256) void pool_fwd_lds_kernel(PoolDims d, FastDiv dPQ, int PB, long long planes, int bands, int rb,
                                                           FastDiv dBands, const float* __restrict__ x,
                                                           float* __restrict__ y, MT* __restrict__ argmax) {
  extern __shared__ float lds_pool[];
  const int HW = d.H * d.W, PQ = d.P * d.Q;
  long long plane0 = (long long)blockIdx.x * PB;
  int np = (int)(planes - plane0 < PB ? planes - plane0 : PB);
  int p0 = 0, h_lo = 0, n_in = np * HW, n_out = np * PQ;
  if (bands > 1) {
    uint32_t pl, bd;
    dBands.divmod(blockIdx.x, pl, bd);
    plane0 = pl;
    np = 1;
    p0 = (int)bd * rb;
    const int p1 = p0 + rb < d.P ? p0 + rb : d.P;
    h_lo = p0 * d.st - d.pad > 0 ? p0 * d.st - d.pad : 0;
    int h_hi = (p1 - 1) * d.st - d.pad + d.k < d.H ? (p1 - 1) * d.st - d.pad + d.k : d.H;
    if (h_hi < h_lo) h_hi = h_lo;
    n_in = (h_hi - h_lo) * d.W;
    n_out = (p1 - p0) * d.Q;
  }
  const int base = h_lo * d.W;
  const float* gx = x + plane0 * HW + base;
  // The staged copy keeps the global address's position inside a 16-byte group, so that the body of the copy
  // is float4 on both sides whatever the plane size (55*55 floats is not a multiple of four).
  const int phase = (int)((reinterpret_cast<uintptr_t>(gx) >> 2) & 3);
  float* const sx = lds_pool + phase;
  const int head = (4 - phase) & 3;
  {
    const int h = head < n_in ? head : n_in;
    if ((int)threadIdx.x < h) sx[threadIdx.x] = gx[threadIdx.x];
    const int n4 = (n_in - h) >> 2;
    const float4* g4 = reinterpret_cast<const float4*>(gx + h);
    float4* s4 = reinterpret_cast<float4*>(sx + h);
    for (int i = threadIdx.x; i < n4; i += 256) s4[i] = g4[i];
    for (int i = h + (n4 << 2) + threadIdx.x; i < n_in; i += 256) sx[i] = gx[i];
  }
  __syncthreads();
  float* gy = y + plane0 * PQ + p0 * d.Q;
  MT* gm = argmax ? argmax + plane0 * PQ + p0 * d.Q : nullptr;
  const float inv = 1.0f / (float)(d.k * d.k);
  for (int o = threadIdx.x; o < n_out; o += 256) {
    uint32_t pl = 0, pq = (uint32_t)(o + p0 * d.Q), p, q;
    if (bands <= 1) dPQ.divmod((uint32_t)o, pl, pq);
    d.dQ.divmod(pq, p, q);
    const float* xp = sx + pl * HW;
    if constexpr (K > 0) {
      const int hs = (int)p * ST - d.pad, ws = (int)q * ST - d.pad;
      if (hs >= 0 && ws >= 0 && hs + K <= d.H && ws + K <= d.W) {
        const int first = hs * d.W + ws;
        const float* b = xp + (first - base);
        if (d.mode == RH_POOL_MAX) {
          float best = b[0];
          int bi = 0;   // the winner's offset from the window's first element, or its slot
#pragma unroll
          for (int r = 0; r < K; ++r)
#pragma unroll
            for (int s2 = 0; s2 < K; ++s2) {
              if (r == 0 && s2 == 0) continue;
              const float v = b[r * d.W + s2];
              if (v > best) { best = v; bi = sizeof(MT) == 1 ? r * K + s2 : r * d.W + s2; }
            }
          gy[o] = best;
          if (gm) gm[o] = sizeof(MT) == 1 ? (MT)bi : (MT)(first + bi);
        } else {
          float acc = 0.0f;
#pragma unroll
          for (int r = 0; r < K; ++r)
#pragma unroll
            for (int s2 = 0; s2 < K; ++s2) acc += b[r * d.W + s2];
          gy[o] = acc * inv;
        }
        continue;
      }
    }
    if (d.mode == RH_POOL_MAX) {
      float best;
      const int bi = window_argmax(xp, d.H, d.W, (int)p, (int)q, d.k, d.st, d.pad, &best, base);
      gy[o] = bi < 0 ? 0.0f : best;
      if (gm) gm[o] = MaskCode<MT>::from_plane(bi, (int)p * d.st - d.pad, (int)q * d.st - d.pad, d.W, d.k);
    } else {
      float acc = 0.0f;
      const int hs = (int)p * d.st - d.pad, ws = (int)q * d.st - d.pad;
      for (int r = 0; r < d.k; ++r) {
        const int h = hs + r;
        if ((unsigned)h >= (unsigned)d.H) continue;
        for (int s2 = 0; s2 < d.k; ++s2) {
          const int w = ws + s2;
          if ((unsigned)w < (unsigned)d.W) acc += xp[h * d.W + w - base];
        }
      }
      gy[o] = acc * inv;
    }
  }
}

// relu_x (average pooling): the pool's input, the output of a ReLU; dx is 0 where it is not > 0 (that ReLU's backward).
template <class I>
__global__ void pool_bwd_kernel(PoolDims d, const float* __restrict__ x, const float* __restrict__ dy,
                                float* __restrict__ dx, const int* __restrict__ argmax,
                                const float* __restrict__ relu_x = nullptr) {
  const I total = (I)d.N * d.C * d.H * d.W;
  const I stride = (I)gridDim.x * blockDim.x;
  const float inv = 1.0f / (float)(d.k * d.k);
  for (I idx = (I)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    I t, nc;
    int w, h;
    if (sizeof(I) == 4) {
      uint32_t t32, w32, nc32, h32;
      d.dW.divmod((uint32_t)idx, t32, w32);
      d.dH.divmod(t32, nc32, h32);
      t = t32; nc = nc32; w = (int)w32; h = (int)h32;
    } else {
      t = idx / (I)d.W;
      w = (int)(idx - t * (I)d.W);
      nc = t / (I)d.H;
      h = (int)(t - nc * (I)d.H);
    }
    // windows p with p*st - pad <= h <= p*st - pad + k - 1
    const int th = h + d.pad - (d.k - 1), tw = w + d.pad - (d.k - 1);
    const int p_lo = th > 0 ? (int)d.dSt.quot((uint32_t)(th + d.st - 1)) : 0;
    const int q_lo = tw > 0 ? (int)d.dSt.quot((uint32_t)(tw + d.st - 1)) : 0;
    int p_hi = (int)d.dSt.quot((uint32_t)(h + d.pad)), q_hi = (int)d.dSt.quot((uint32_t)(w + d.pad));
    if (p_hi > d.P - 1) p_hi = d.P - 1;
    if (q_hi > d.Q - 1) q_hi = d.Q - 1;
    const float* dyp = dy + (size_t)nc * d.P * d.Q;
    float acc = 0.0f;
    if (d.mode == RH_POOL_MAX) {
      const int me = h * d.W + w;
      const float* xp = x ? x + (size_t)nc * d.H * d.W : nullptr;
      const int* ap = argmax ? argmax + (size_t)nc * d.P * d.Q : nullptr;
      for (int p = p_lo; p <= p_hi; ++p)
        for (int q = q_lo; q <= q_hi; ++q) {
          int bi;
          if (ap) {
            bi = ap[p * d.Q + q];
          } else {
            float best;
            bi = window_argmax(xp, d.H, d.W, p, q, d.k, d.st, d.pad, &best);
          }
          if (bi == me) acc += dyp[p * d.Q + q];
        }
    } else {
      for (int p = p_lo; p <= p_hi; ++p)
        for (int q = q_lo; q <= q_hi; ++q) acc += dyp[p * d.Q + q] * inv;
      if (relu_x && !(relu_x[idx] > 0.0f)) acc = 0.0f;
    }
    dx[idx] = acc;
  }
}

// Max-pool backward driven by the arg-max mask, one block per group of PB consecutive planes: the
// group's dy and mask (PB*P*Q values each) are staged in LDS with coalesced reads, then every input
// element looks its covering windows up in LDS and dx is written coalesced.  No dependent global loads.
// With `y` (the pooled outputs) the backward mask of a ReLU that produced x is folded in: an arg-max element
// carries x = y, so "dx = 0 where x <= 0" is "skip windows whose maximum y is <= 0".
__global__ __launch_bounds__(256) void pool_bwd_mask_lds_kernel(PoolDims d, FastDiv dHW, int PB, long long planes,
                                                                const float* __restrict__ dy, const int* __restrict__ argmax,
                                                                const float* __restrict__ y, float* __restrict__ dx) {
  extern __shared__ float lds_pool[];
  const int PQ = d.P * d.Q, HW = d.H * d.W;
  const long long plane0 = (long long)blockIdx.x * PB;
  const int np = (int)(planes - plane0 < PB ? planes - plane0 : PB);
  float* sdy = lds_pool;
  int* smask = reinterpret_cast<int*>(lds_pool + PB * PQ);
  const int n_out = np * PQ, n_in = np * HW;
  const float* gdy = dy + plane0 * PQ;
  const int* gm = argmax + plane0 * PQ;
  if (y) {  // a window whose maximum is not positive routes nothing: give it an index no element has
    const float* gy = y + plane0 * PQ;
    for (int i = threadIdx.x; i < n_out; i += 256) { sdy[i] = gdy[i]; smask[i] = gy[i] > 0.0f ? gm[i] : -1; }
  } else {
    for (int i = threadIdx.x; i < n_out; i += 256) { sdy[i] = gdy[i]; smask[i] = gm[i]; }
  }
  __syncthreads();
  float* gdx = dx + plane0 * HW;
  auto value = [&](int e) -> float {
    uint32_t pl, hw, h, w;
    dHW.divmod((uint32_t)e, pl, hw);
    d.dW.divmod(hw, h, w);
    const int th = (int)h + d.pad - (d.k - 1), tw = (int)w + d.pad - (d.k - 1);
    const int p_lo = th > 0 ? (int)d.dSt.quot((uint32_t)(th + d.st - 1)) : 0;
    const int q_lo = tw > 0 ? (int)d.dSt.quot((uint32_t)(tw + d.st - 1)) : 0;
    int p_hi = (int)d.dSt.quot(h + d.pad), q_hi = (int)d.dSt.quot(w + d.pad);
    if (p_hi > d.P - 1) p_hi = d.P - 1;
    if (q_hi > d.Q - 1) q_hi = d.Q - 1;
    const int base = (int)pl * PQ;
    float acc = 0.0f;
    for (int p = p_lo; p <= p_hi; ++p)
      for (int q = q_lo; q <= q_hi; ++q) {
        const int o = base + p * d.Q + q;
        if (smask[o] == (int)hw) acc += sdy[o];
      }
    return acc;
  };
  // four consecutive elements per thread and one 16-byte store, after a scalar head up to the first aligned address
  const int phase = (int)((reinterpret_cast<uintptr_t>(gdx) >> 2) & 3);
  const int head = ((4 - phase) & 3) < n_in ? ((4 - phase) & 3) : n_in;
  if ((int)threadIdx.x < head) gdx[threadIdx.x] = value((int)threadIdx.x);
  const int n4 = (n_in - head) >> 2;
  float4* g4 = reinterpret_cast<float4*>(gdx + head);
  for (int g = threadIdx.x; g < n4; g += 256) {
    const int e = head + 4 * g;
    float4 v;
    v.x = value(e);
    v.y = value(e + 1);
    v.z = value(e + 2);
    v.w = value(e + 3);
    g4[g] = v;
  }
  for (int e = head + (n4 << 2) + threadIdx.x; e < n_in; e += 256) gdx[e] = value(e);
}

// Max-pool backward from the arg-max mask with the windows dealt out by colour.  Windows p and p' of one axis share
// input rows only if |p - p'| * stride < size, so the windows whose (p mod nA, q mod nA) agree, nA = ceil(size/stride),
// touch disjoint elements: the block zeroes the dx of its PB planes in LDS, adds every window's dy to the element its
// mask names, one colour after the other with a barrier between (plain LDS read-add-write, no atomics, fixed sum order:
// colours in the order (0,0), (0,1), (1,0), (1,1)), and writes the planes out as 16-byte groups.  One pass over dy, the
// mask and dx and some twenty instructions per window, where the gather form spends sixty per input element.
// All of a thread's windows (at most J per colour) are loaded before the first barrier.  nA is 1 or 2.
struct PoolColors {
  int nA;             // colours per axis
  int cnt[4];         // windows of one plane in colour (a, b) = cnt[a * 2 + b]
  int Qb[2];          // windows per row in column colour b
  FastDiv dCnt[4], dQb[2];
};

template <int J, class MT>
__global__ __launch_bounds__(256) void pool_bwd_mask_color_kernel(PoolDims d, PoolColors pc, int PB, long long planes,
                                                                  const float* __restrict__ dy, const MT* __restrict__ argmax,
                                                                  const float* __restrict__ y, float* __restrict__ dx) {
  extern __shared__ float lds_pool[];
  const int PQ = d.P * d.Q, HW = d.H * d.W;
  const long long plane0 = (long long)blockIdx.x * PB;
  const int np = (int)(planes - plane0 < PB ? planes - plane0 : PB);
  const int n_in = np * HW;
  const float* gdy = dy + plane0 * PQ;
  const MT* gm = argmax + plane0 * PQ;
  const float* gy = y ? y + plane0 * PQ : nullptr;
  float* gdx = dx + plane0 * HW;
  // the LDS copy keeps the global address's position inside a 16-byte group
  const int phase = (int)((reinterpret_cast<uintptr_t>(gdx) >> 2) & 3);
  float* const sdx = lds_pool + phase;

  int tgt[4][J];    // LDS index of the element a window routes to, -1: none
  float val[4][J];
  const int ncol = pc.nA * pc.nA;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
#pragma unroll
    for (int j = 0; j < J; ++j) { tgt[c][j] = -1; val[c][j] = 0.0f; }
    if (c < ncol) {
      const int a = pc.nA == 2 ? c >> 1 : 0, b = pc.nA == 2 ? c & 1 : 0;
      const int n_c = np * pc.cnt[c];
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const int t = (int)threadIdx.x + 256 * j;
        if (t < n_c) {
          uint32_t pl, rem, i, jj;
          pc.dCnt[c].divmod((uint32_t)t, pl, rem);
          pc.dQb[b].divmod(rem, i, jj);
          const int wp = (int)i * pc.nA + a, wq = (int)jj * pc.nA + b;
          const int o = (int)pl * PQ + wp * d.Q + wq;
          int m = MaskCode<MT>::to_plane(gm[o], wp * d.st - d.pad, wq * d.st - d.pad, d);
          val[c][j] = gdy[o];
          if (gy && !(gy[o] > 0.0f)) m = -1;  // a window whose maximum is not positive routes nothing
          tgt[c][j] = (unsigned)m < (unsigned)HW ? (int)pl * HW + m : -1;
        }
      }
    }
  }
  {
    float4* z4 = reinterpret_cast<float4*>(lds_pool);
    const int nz = (n_in + 4 + 3) >> 2;
    for (int i = threadIdx.x; i < nz; i += 256) z4[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    if (c < ncol) {
#pragma unroll
      for (int j = 0; j < J; ++j)
        if (tgt[c][j] >= 0) sdx[tgt[c][j]] += val[c][j];
      __syncthreads();
    }
  }
  const int head = ((4 - phase) & 3) < n_in ? ((4 - phase) & 3) : n_in;
  if ((int)threadIdx.x < head) gdx[threadIdx.x] = sdx[threadIdx.x];
  const int n4 = (n_in - head) >> 2;
  float4* g4 = reinterpret_cast<float4*>(gdx + head);
  const float4* s4 = reinterpret_cast<const float4*>(sdx + head);
  for (int g = threadIdx.x; g < n4; g += 256) g4[g] = s4[g];
  for (int e = head + (n4 << 2) + threadIdx.x; e < n_in; e += 256) gdx[e] = sdx[e];
}

// Launches one instantiation of the LDS forward; RH_E_UNSUPPORTED when the block's LDS cannot be had.
template <int K, int ST, class MT>
static int launch_pool_fwd_lds(const PoolDims& d, FastDiv dPQ, int PB, long long planes, long long blocks, size_t lds_bytes,
                               int bands, int rb, const float* x, float* y, MT* argmax, rh_stream_t stream) {
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&pool_fwd_lds_kernel<K, ST, MT>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr != hipSuccess) return RH_E_UNSUPPORTED;
  }
  hipLaunchKernelGGL((pool_fwd_lds_kernel<K, ST, MT>), dim3((unsigned)blocks), dim3(256), lds_bytes, to_stream(stream), d, dPQ, PB,
                     planes, bands, rb, FastDiv((uint32_t)bands), x, y, argmax);
  return launch_status();
}

static int pool_dims(const rh_pool_geom* g, PoolDims* d) {
  if (!g) return RH_E_INVALID;
  if (g->N <= 0 || g->C <= 0 || g->H <= 0 || g->W <= 0 || g->size <= 0 || g->stride <= 0 || g->pad < 0)
    return RH_E_INVALID;
  if (g->mode != RH_POOL_MAX && g->mode != RH_POOL_AVG_INCL_PAD) return RH_E_INVALID;
  if (g->round != RH_ROUND_FLOOR && g->round != RH_ROUND_CEIL) return RH_E_INVALID;
  d->N = g->N; d->C = g->C; d->H = g->H; d->W = g->W; d->k = g->size; d->st = g->stride; d->pad = g->pad;
  d->mode = g->mode;
  d->P = pool_out_dim(g->H, g->size, g->stride, g->pad, g->round);
  d->Q = pool_out_dim(g->W, g->size, g->stride, g->pad, g->round);
  if ((long long)g->H * g->W >= (1ll << 31)) return RH_E_LIMIT;
  d->dP = FastDiv((uint32_t)(d->P > 0 ? d->P : 1));
  d->dQ = FastDiv((uint32_t)(d->Q > 0 ? d->Q : 1));
  d->dH = FastDiv((uint32_t)d->H);
  d->dW = FastDiv((uint32_t)d->W);
  d->dSt = FastDiv((uint32_t)d->st);
  d->dK = FastDiv((uint32_t)d->k);
  return 0;
}

}  // namespace rh

using namespace rh;

extern "C" int32_t rh_pool2d_out_dim(int32_t in, int32_t size, int32_t stride, int32_t pad, int32_t round) {
  if (stride <= 0) return 0;
  return pool_out_dim(in, size, stride, pad, round);
}

// The LDS forward: about 16 KB of input per block (measured best: more LDS per block leaves too few blocks per CU to
// overlap one block's loads with another's window scans): several small planes, one plane, or a band of a larger
// plane's output rows with the input rows its windows reach.  RH_E_UNSUPPORTED: the geometry is outside this form.
template <class MT>
static int pool_fwd_lds(const PoolDims& d, const float* x, float* y, MT* mask, rh_stream_t stream, bool dry_run = false) {
  constexpr int kLdsFloats = 4096;
  if (!(d.P * d.Q > 0 && (long long)d.W * d.k <= 15000)) return RH_E_UNSUPPORTED;
  const int HW = d.H * d.W;
  const long long planes = (long long)d.N * d.C;
  int PB = 1, bands = 1, rb = d.P, rows_in = d.H;
  if (HW <= kLdsFloats) {
    PB = kLdsFloats / HW;
    if (PB > 64) PB = 64;
  } else {
    const int rows_fit = kLdsFloats / d.W;  // input rows in the block's share (at least one window's)
    rb = rows_fit > d.k ? (rows_fit - d.k) / d.st + 1 : 1;
    if (rb > d.P) rb = d.P;
    bands = cdiv(d.P, rb);
    rows_in = (rb - 1) * d.st + d.k < d.H ? (rb - 1) * d.st + d.k : d.H;
  }
  const long long blocks = bands > 1 ? planes * bands : cdiv<long long>(planes, PB);
  const size_t lds_bytes = ((size_t)(bands > 1 ? rows_in * d.W : PB * HW) + 4) * sizeof(float);
  if (!(blocks < (1ll << 31) && (long long)PB * d.P * d.Q < (1ll << 31)) || lds_bytes > 64 * 1024) return RH_E_UNSUPPORTED;
  if (dry_run) return 0;
  const FastDiv dPQ((uint32_t)(d.P * d.Q));
  if (d.k == 3 && d.st == 2) return launch_pool_fwd_lds<3, 2, MT>(d, dPQ, PB, planes, blocks, lds_bytes, bands, rb, x, y, mask, stream);
  if (d.k == 2 && d.st == 2) return launch_pool_fwd_lds<2, 2, MT>(d, dPQ, PB, planes, blocks, lds_bytes, bands, rb, x, y, mask, stream);
  if (d.k == 3 && d.st == 1) return launch_pool_fwd_lds<3, 1, MT>(d, dPQ, PB, planes, blocks, lds_bytes, bands, rb, x, y, mask, stream);
  return launch_pool_fwd_lds<0, 0, MT>(d, dPQ, PB, planes, blocks, lds_bytes, bands, rb, x, y, mask, stream);
}

extern "C" int rh_pool2d_fwd(const rh_pool_geom* g, const float* x, float* y, int32_t* opt_argmax,
                             rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!x || !y) return RH_E_INVALID;
  const long long total = (long long)d.N * d.C * d.P * d.Q;
  if (total == 0) return 0;
  // algorithmic bytes: x read, y written (and the arg-max mask where the caller asks for one)
  ProfScope prof(d.mode == RH_POOL_MAX ? "pool_max_fwd" : "pool_avg_fwd",
                 4.0 * ((double)d.N * d.C * d.H * d.W + (double)total * (opt_argmax ? 2 : 1)), to_stream(stream));
  const long long in_total = (long long)d.N * d.C * d.H * d.W;
  {
    const int e = pool_fwd_lds<int>(d, x, y, opt_argmax, stream);
    if (e != RH_E_UNSUPPORTED) return e;
  }
  const dim3 grid((unsigned)cdiv<long long>(total, 256) > (1u << 20) ? (1u << 20) : (unsigned)cdiv<long long>(total, 256));
  if (total < (1ll << 31) && in_total < (1ll << 31))
    hipLaunchKernelGGL(pool_fwd_kernel<unsigned>, grid, dim3(256), 0, to_stream(stream), d, x, y, opt_argmax);
  else
    hipLaunchKernelGGL(pool_fwd_kernel<long long>, grid, dim3(256), 0, to_stream(stream), d, x, y, opt_argmax);
  return launch_status();
}

extern "C" int rh_pool2d_fwd_bf16_packed(const rh_pool_geom* g, const void* xp, void* yp, int32_t yp_halo,
                                         rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!xp || !yp || yp_halo < 0 || ((reinterpret_cast<uintptr_t>(xp) | reinterpret_cast<uintptr_t>(yp)) & 15)) return RH_E_INVALID;
  if (d.mode != RH_POOL_MAX || d.C % 8 != 0) return RH_E_UNSUPPORTED;
  const long long groups = (long long)d.N * (d.C / 8) * d.P * d.Q;
  const long long in_bytes = 2ll * d.N * d.C * d.H * d.W;
  const long long out_bytes = 2ll * d.N * d.C * (d.P + 2 * yp_halo) * (d.Q + 2 * yp_halo);
  if (groups >= (1ll << 31) || in_bytes > (long long)kMaxBufferBytes || out_bytes > (long long)kMaxBufferBytes) return RH_E_LIMIT;
  if (groups == 0) return 0;
  ProfScope prof("pool_max_fwd_bf16", (double)in_bytes + 16.0 * (double)groups, to_stream(stream));
  hipLaunchKernelGGL(pool_max_fwd_bf16_kernel, dim3(stream_grid((size_t)groups, 256)), dim3(256), 0, to_stream(stream), d,
                     FastDiv((uint32_t)(d.C / 8)), static_cast<const uint4*>(xp), static_cast<uint4*>(yp), (unsigned)groups,
                     yp_halo);
  return launch_status();
}

// The dy and mask of at least one whole plane must fit the block's LDS (8 bytes per pooled element, 32 KB at most).
static bool lds_bwd_ok(const PoolDims& d) { return d.P * d.Q <= 4096 && d.H * d.W <= (1 << 20); }

// The colour form: one or two colours per axis, a plane's dx within 60 KB of LDS, at most 8 windows per thread and
// colour.  Returns RH_E_UNSUPPORTED when the geometry is outside that.
template <int J, class MT>
static int launch_pool_bwd_color_j(const PoolDims& d, const PoolColors& pc, int PB, long long planes, long long blocks,
                                   size_t lds_bytes, const float* dy, const MT* argmax, const float* relu_y, float* dx,
                                   rh_stream_t stream) {
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&pool_bwd_mask_color_kernel<J, MT>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr != hipSuccess) return RH_E_UNSUPPORTED;
  }
  hipLaunchKernelGGL((pool_bwd_mask_color_kernel<J, MT>), dim3((unsigned)blocks), dim3(256), lds_bytes, to_stream(stream), d, pc, PB,
                     planes, dy, argmax, relu_y, dx);
  return launch_status();
}

template <class MT>
static int launch_pool_bwd_color(const PoolDims& d, const float* dy, const MT* argmax, const float* relu_y, float* dx,
                                 rh_stream_t stream, bool dry_run = false) {
  const int nA = cdiv(d.k, d.st);
  const int HW = d.H * d.W;
  if (nA > 2 || HW > 15000 || d.P * d.Q <= 0) return RH_E_UNSUPPORTED;
  PoolColors pc;
  pc.nA = nA;
  int most = 0;
  for (int a = 0; a < 2; ++a)
    for (int b = 0; b < 2; ++b) {
      const int Pa = a < nA && a < d.P ? (d.P - a + nA - 1) / nA : 0;
      const int Qb = b < nA && b < d.Q ? (d.Q - b + nA - 1) / nA : 0;
      const int c = nA == 2 ? a * 2 + b : 0;
      if (nA == 1 && (a || b)) continue;
      pc.cnt[c] = Pa * Qb;
      pc.dCnt[c] = FastDiv((uint32_t)(pc.cnt[c] > 0 ? pc.cnt[c] : 1));
      pc.Qb[b] = Qb;
      pc.dQb[b] = FastDiv((uint32_t)(Qb > 0 ? Qb : 1));
      if (pc.cnt[c] > most) most = pc.cnt[c];
    }
  if (nA == 1) {
    for (int c = 1; c < 4; ++c) { pc.cnt[c] = 0; pc.dCnt[c] = FastDiv(1u); }
    pc.Qb[1] = 0; pc.dQb[1] = FastDiv(1u);
  }
  if (most <= 0 || most > 256 * 8) return RH_E_UNSUPPORTED;
  // planes per block: about 256 windows of the largest colour and 16 KB of dx
  int PB = 256 / most;
  if (PB > 4096 / HW) PB = 4096 / HW;
  if (PB < 1) PB = 1;
  if (PB > 64) PB = 64;
  const int per_thread = cdiv(PB * most, 256);
  const long long planes = (long long)d.N * d.C;
  const long long blocks = cdiv<long long>(planes, PB);
  if (blocks >= (1ll << 31)) return RH_E_LIMIT;
  const size_t lds_bytes = ((size_t)PB * HW + 8) * sizeof(float);
  if (dry_run) return 0;
  if (per_thread <= 1) return launch_pool_bwd_color_j<1, MT>(d, pc, PB, planes, blocks, lds_bytes, dy, argmax, relu_y, dx, stream);
  if (per_thread <= 2) return launch_pool_bwd_color_j<2, MT>(d, pc, PB, planes, blocks, lds_bytes, dy, argmax, relu_y, dx, stream);
  if (per_thread <= 4) return launch_pool_bwd_color_j<4, MT>(d, pc, PB, planes, blocks, lds_bytes, dy, argmax, relu_y, dx, stream);
  return launch_pool_bwd_color_j<8, MT>(d, pc, PB, planes, blocks, lds_bytes, dy, argmax, relu_y, dx, stream);
}

static int launch_pool_bwd_lds(const PoolDims& d, const float* dy, const int32_t* argmax, const float* relu_y, float* dx,
                               rh_stream_t stream) {
  {
    const int e = launch_pool_bwd_color<int>(d, dy, argmax, relu_y, dx, stream);
    if (e != RH_E_UNSUPPORTED) return e;
  }
  const int PQ = d.P * d.Q;
  int PB = 2048 / PQ;
  if (PB > 64) PB = 64;
  if (PB < 1) PB = 1;
  const long long planes = (long long)d.N * d.C;
  const long long blocks = cdiv<long long>(planes, PB);
  if (blocks >= (1ll << 31)) return RH_E_LIMIT;
  hipLaunchKernelGGL(pool_bwd_mask_lds_kernel, dim3((unsigned)blocks), dim3(256), (size_t)PB * PQ * 8, to_stream(stream), d,
                     FastDiv((uint32_t)(d.H * d.W)), PB, planes, dy, argmax, relu_y, dx);
  return launch_status();
}

extern "C" int rh_pool2d_bwd_relu_supported(const rh_pool_geom* g) {
  PoolDims d;
  if (pool_dims(g, &d)) return 0;
  return d.mode == RH_POOL_MAX && lds_bwd_ok(d) && (long long)d.N * d.C < (1ll << 31) ? 1 : 0;
}

extern "C" int rh_pool2d_bwd_relu(const rh_pool_geom* g, const float* y, const float* dy, float* dx, const int32_t* argmax,
                                  rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!y || !dy || !dx || !argmax) return RH_E_INVALID;
  if (!rh_pool2d_bwd_relu_supported(g)) return RH_E_UNSUPPORTED;
  const double in_elems = (double)d.N * d.C * d.H * d.W, out_elems = (double)d.N * d.C * d.P * d.Q;
  if (in_elems == 0) return 0;
  ProfScope prof("pool_max_bwd_relu", 4.0 * (in_elems + 3.0 * out_elems), to_stream(stream));
  return launch_pool_bwd_lds(d, dy, argmax, y, dx, stream);
}

extern "C" int rh_pool2d_bwd_avg_relu(const rh_pool_geom* g, const float* x, const float* dy, float* dx, rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!x || !dy || !dx) return RH_E_INVALID;
  if (d.mode != RH_POOL_AVG_INCL_PAD) return RH_E_UNSUPPORTED;
  const long long total = (long long)d.N * d.C * d.H * d.W;
  if (total == 0) return 0;
  ProfScope prof("pool_avg_bwd_relu", 4.0 * (2.0 * (double)total + (double)d.N * d.C * d.P * d.Q), to_stream(stream));
  const dim3 grid((unsigned)cdiv<long long>(total, 256) > (1u << 20) ? (1u << 20) : (unsigned)cdiv<long long>(total, 256));
  if (total < (1ll << 31))
    hipLaunchKernelGGL(pool_bwd_kernel<unsigned>, grid, dim3(256), 0, to_stream(stream), d, (const float*)nullptr, dy, dx,
                       (const int*)nullptr, x);
  else
    hipLaunchKernelGGL(pool_bwd_kernel<long long>, grid, dim3(256), 0, to_stream(stream), d, (const float*)nullptr, dy, dx,
                       (const int*)nullptr, x);
  return launch_status();
}

// The one-byte mask: max pooling with size <= 15 on the geometries that both the LDS forward and the colour backward take.
extern "C" int rh_pool2d_slot_supported(const rh_pool_geom* g) {
  PoolDims d;
  if (pool_dims(g, &d)) return 0;
  if (d.mode != RH_POOL_MAX || d.k > 15 || !lds_bwd_ok(d) || (long long)d.N * d.C >= (1ll << 31)) return 0;
  return pool_fwd_lds<uint8_t>(d, nullptr, nullptr, nullptr, nullptr, true) == 0 &&
         launch_pool_bwd_color<uint8_t>(d, nullptr, nullptr, nullptr, nullptr, nullptr, true) == 0 ? 1 : 0;
}

extern "C" int rh_pool2d_fwd_slot(const rh_pool_geom* g, const float* x, float* y, uint8_t* slot, rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!x || !y || !slot) return RH_E_INVALID;
  if (!rh_pool2d_slot_supported(g)) return RH_E_UNSUPPORTED;
  const double in_elems = (double)d.N * d.C * d.H * d.W, out_elems = (double)d.N * d.C * d.P * d.Q;
  if (out_elems == 0) return 0;
  // algorithmic bytes: x read, y written; the mask's byte per output is the operator's own bookkeeping and not counted
  ProfScope prof("pool_max_fwd", 4.0 * (in_elems + out_elems), to_stream(stream));
  return pool_fwd_lds<uint8_t>(d, x, y, slot, stream);
}

extern "C" int rh_pool2d_bwd_slot(const rh_pool_geom* g, const float* relu_y, const float* dy, float* dx, const uint8_t* slot,
                                  rh_stream_t stream) {
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!dy || !dx || !slot) return RH_E_INVALID;
  if (!rh_pool2d_slot_supported(g)) return RH_E_UNSUPPORTED;
  const double in_elems = (double)d.N * d.C * d.H * d.W, out_elems = (double)d.N * d.C * d.P * d.Q;
  if (in_elems == 0) return 0;
  // algorithmic bytes: dy read, dx written, and y read where the ReLU mask of the operator below is folded in
  ProfScope prof(relu_y ? "pool_max_bwd_relu" : "pool_max_bwd", 4.0 * (in_elems + (relu_y ? 2.0 : 1.0) * out_elems),
                 to_stream(stream));
  return launch_pool_bwd_color<uint8_t>(d, dy, slot, relu_y, dx, stream);
}

extern "C" int rh_pool2d_bwd(const rh_pool_geom* g, const float* x, const float* y, const float* dy, float* dx,
                             const int32_t* opt_argmax, rh_stream_t stream) {
  (void)y;
  PoolDims d;
  if (int e = pool_dims(g, &d)) return e;
  if (!dy || !dx) return RH_E_INVALID;
  if (d.mode == RH_POOL_MAX && !opt_argmax && !x) return RH_E_INVALID;
  const long long total = (long long)d.N * d.C * d.H * d.W;
  const double out_elems = (double)d.N * d.C * d.P * d.Q;
  // bytes: write dx, read dy, plus the arg-max mask or (max without mask) x itself
  const double bwd_bytes = 4.0 * ((double)total + out_elems + (d.mode == RH_POOL_MAX ? (opt_argmax ? out_elems : (double)total) : 0.0));
  ProfScope prof(d.mode == RH_POOL_MAX ? "pool_max_bwd" : "pool_avg_bwd", bwd_bytes, to_stream(stream));
  if (d.mode == RH_POOL_MAX && opt_argmax && lds_bwd_ok(d) && (long long)d.N * d.C < (1ll << 31))
    return launch_pool_bwd_lds(d, dy, opt_argmax, nullptr, dx, stream);
  const dim3 grid((unsigned)cdiv<long long>(total, 256) > (1u << 20) ? (1u << 20) : (unsigned)cdiv<long long>(total, 256));
  if (total < (1ll << 31))
    hipLaunchKernelGGL(pool_bwd_kernel<unsigned>, grid, dim3(256), 0, to_stream(stream), d, x, dy, dx, opt_argmax);
  else
    hipLaunchKernelGGL(pool_bwd_kernel<long long>, grid, dim3(256), 0, to_stream(stream), d, x, dy, dx, opt_argmax);
  return launch_status();
}
