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


// ---- the classifier tail of a train step: two affine layers and the loss in one launch ---------------------------
// x (B x I) -> h = act(W1 x + b1) (B x H) -> logits = W2 h + b2 (B x C) -> softmax, arg-max, per-sample loss, its sum,
// the KL delta, and the data gradients back through both layers: dlogits, dh = [h > 0] * W2^T dlogits, dx = W1^T dh.
// One block per sample: nothing of a sample's chain depends on another sample, so the whole chain is one kernel
// (the separate operators are eight to ten launches of a few microseconds of work each, on a path that is a chain of
// dependent launches).  Every block reads all of W1 twice, so this form is for first layers of a few hundred KB.
// Plain FMA arithmetic, fixed summation orders.  Each phase asks for its weights in batches of 32-64 loads per lane
// before it uses any (indices past the end are clamped and their products zeroed: no load under a branch), so a phase
// costs a few memory round trips.  Weights are [out][in] (the reference's column-major (in, out)), activations
// [sample][channel].  LDS: x row (I), h (H), dh (H), logits / delta (64).
template <int NT>
__global__ __launch_bounds__(NT) void affine2_softmax_kl_step_kernel(
    int B, int I, int H, int C, int relu1, const float* __restrict__ x, const float* __restrict__ w1,
    const float* __restrict__ b1, const float* __restrict__ w2, const float* __restrict__ b2,
    const int* __restrict__ labels, const float* __restrict__ weights, float* __restrict__ h_out,
    float* __restrict__ logits_out, float* __restrict__ p_out, float* __restrict__ max_out, int* __restrict__ idx_out,
    float* __restrict__ loss1, float* __restrict__ loss_sum, float* __restrict__ dlogits_out, float* __restrict__ dh_out,
    float* __restrict__ dx_out, unsigned* __restrict__ counter) {
  extern __shared__ float lds_tail[];
  float* const xs = lds_tail;          // [I]
  float* const hs = xs + I;            // [H]
  float* const dhs = hs + H;           // [H]
  float* const ls = dhs + H;           // [64] logits, then the delta
  __shared__ float sm[NT / 64];
  __shared__ bool last;
  constexpr int NW = NT / 64;
  const int n = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool have_h = x == nullptr;   // the first layer's forward already ran (a layer too large for this form): I = 0
  if (have_h) {
    for (int j = tid; j < H; j += NT) hs[j] = h_out[(size_t)n * H + j];
  } else {
    for (int i = tid; i < I; i += NT) xs[i] = x[(size_t)n * I + i];
  }
  __syncthreads();
  // h: a wave per group of four outputs, lanes along the input, 16 x 4 weights per lane in flight
  for (int j0 = wave * 4; j0 < H && !have_h; j0 += NW * 4) {
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const float* r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = w1 + (size_t)(j0 + k < H ? j0 + k : H - 1) * I;
    for (int i0 = 0; i0 < I; i0 += 1024) {
      float wv[4][16], xv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int i = i0 + u * 64 + lane, ii = i < I ? i : I - 1;
#pragma unroll
        for (int k = 0; k < 4; ++k) wv[k][u] = r[k][ii];
        xv[u] = i < I ? xs[ii] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u)
#pragma unroll
        for (int k = 0; k < 4; ++k) a[k] = fmaf(wv[k][u], xv[u], a[k]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      for (int o = 32; o > 0; o >>= 1) a[k] += __shfl_xor(a[k], o, 64);
    if (lane < 4 && j0 + lane < H) {
      float v = (lane == 0 ? a[0] : lane == 1 ? a[1] : lane == 2 ? a[2] : a[3]) + b1[j0 + lane];
      if (relu1) v = v > 0.0f ? v : 0.0f;
      hs[j0 + lane] = v;
      h_out[(size_t)n * H + j0 + lane] = v;
    }
  }
  __syncthreads();
  // logits: a wave per class, lanes along h, 16 weights per lane in flight
  for (int c = wave; c < C; c += NW) {
    float a = 0.0f;
    const float* r = w2 + (size_t)c * H;
    for (int j0 = 0; j0 < H; j0 += 1024) {
      float wv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int j = j0 + u * 64 + lane;
        wv[u] = r[j < H ? j : H - 1];
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int j = j0 + u * 64 + lane;
        a = fmaf(wv[u], j < H ? hs[j] : 0.0f, a);
      }
    }
    for (int o = 32; o > 0; o >>= 1) a += __shfl_xor(a, o, 64);
    if (lane == 0) {
      a += b2[c];
      ls[c] = a;
      logits_out[(size_t)n * C + c] = a;
    }
  }
  __syncthreads();
  // softmax, arg-max (first maximum), loss and delta: the first wave, a lane per class (C <= 64)
  if (wave == 0) {
    const float v = lane < C ? ls[lane] : -INFINITY;
    float mx = v;
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float e = lane < C ? expf(v - mx) : 0.0f;
    float z = e;
    for (int o = 32; o > 0; o >>= 1) z += __shfl_xor(z, o, 64);
    float pv = e * (1.0f / z);
    asm volatile("" : "+v"(pv));   // the rounded product is what is stored and what the delta is formed from
    const int label = labels[n];
    const float wgt = weights[n];
    float best = lane < C ? pv : -INFINITY;
    int bi = lane < C ? lane : 0x7fffffff;
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
    }
    const float d = wgt * (pv - (lane == label ? 1.0f : 0.0f));
    if (lane < C) {
      p_out[(size_t)n * C + lane] = pv;
      dlogits_out[(size_t)n * C + lane] = d;
      if (lane == label) loss1[n] = -wgt * logf(pv);
      ls[lane] = d;
    }
    if (lane == 0) {
      if ((unsigned)label >= (unsigned)C) loss1[n] = NAN;
      max_out[n] = best;
      idx_out[n] = bi == 0x7fffffff ? 0 : bi;
    }
  }
  __syncthreads();
  // dh = [h > 0] * W2^T delta: a thread per hidden unit, 16 classes' weights in flight
  for (int j = tid; j < H; j += NT) {
    float a = 0.0f;
    for (int c0 = 0; c0 < C; c0 += 16) {
      float wv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) wv[u] = w2[(size_t)(c0 + u < C ? c0 + u : C - 1) * H + j];
#pragma unroll
      for (int u = 0; u < 16; ++u) a = fmaf(wv[u], c0 + u < C ? ls[c0 + u] : 0.0f, a);
    }
    if (relu1 && !(hs[j] > 0.0f)) a = 0.0f;
    dhs[j] = a;
    dh_out[(size_t)n * H + j] = a;
  }
  __syncthreads();
  // dx = W1^T dh: a thread per input element (rows of W1 read along the lanes), 32 rows' weights in flight
  if (dx_out && !have_h) {
    for (int i = tid; i < I; i += NT) {
      float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
      for (int j0 = 0; j0 < H; j0 += 32) {
        float wv[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) wv[u] = w1[(size_t)(j0 + u < H ? j0 + u : H - 1) * I + i];
#pragma unroll
        for (int u = 0; u < 32; u += 4) {
          a0 = fmaf(wv[u], j0 + u < H ? dhs[j0 + u] : 0.0f, a0);
          a1 = fmaf(wv[u + 1], j0 + u + 1 < H ? dhs[j0 + u + 1] : 0.0f, a1);
          a2 = fmaf(wv[u + 2], j0 + u + 2 < H ? dhs[j0 + u + 2] : 0.0f, a2);
          a3 = fmaf(wv[u + 3], j0 + u + 3 < H ? dhs[j0 + u + 3] : 0.0f, a3);
        }
      }
      dx_out[(size_t)n * I + i] = (a0 + a1) + (a2 + a3);
    }
  }
  // The sum of the per-sample losses, by the block that finishes last (it leaves the counter at zero again).  What
  // that block reads of the others is loss1, written by the thread that counts its block below (its own wave wrote
  // it): the release is part of its atomic, once per block.  (A device-scope fence in every wave of every block
  // writes back and invalidates an XCD's whole L2 sixteen times per block: 40 us of a 50 us kernel.)
  __syncthreads();
  if (tid == 0) last = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)B - 1u;
  __syncthreads();
  if (!last) return;
  if (wave == 0) __threadfence();
  __syncthreads();
  float acc = 0.0f;
  for (int i = tid; i < B; i += NT) acc += __hip_atomic_load(loss1 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  acc = block_reduce_sum(acc, sm);
  if (tid == 0) {
    loss_sum[0] = acc;
    *counter = 0u;
  }
}

// The parameter gradients of the same two layers in one launch: dW1[j][i] = sum_n dh[n][j] x[n][i], db1[j] = sum_n dh[n][j],
// dW2[c][j] = sum_n dlogits[n][c] h[n][j], db2[c] = sum_n dlogits[n][c]; out = sum + beta * old (beta 0: old is not read).
// A block of 256 threads takes 32 result items (four consecutive i of dW1 where I is a multiple of four, else one
// element) and cuts the batch into eight slices, one per group of 32 threads: every thread adds its slice's samples
// (16 of them in flight at a time), the slices' sums meet in LDS and are added in slice order.
__global__ __launch_bounds__(256) void affine2_bwd_params_kernel(int B, int I, int H, int C, int vec, const float* __restrict__ x,
                                                                 const float* __restrict__ h, const float* __restrict__ dh,
                                                                 const float* __restrict__ dl, float beta1, float* __restrict__ dw1,
                                                                 float* __restrict__ db1, float beta2, float* __restrict__ dw2,
                                                                 float* __restrict__ db2, unsigned n1, unsigned n2, unsigned n3) {
  __shared__ float4 part[8][32];
  const int t = threadIdx.x & 31, s = threadIdx.x >> 5;
  const unsigned idx = blockIdx.x * 32u + (unsigned)t, total = n1 + n2 + n3;
  const int per = (B + 7) / 8, nb = s * per, ne = nb + per < B ? nb + per : B;
  // what this item multiplies: a[n * sa + oa] * b[n * sb + ob .. +3] (a scalar of the delta, a run of the activation)
  const float* pa = dh;
  const float* pb = x;
  size_t sa = 0, sb = 0, oa = 0, ob = 0;
  int kind = -1;   // 0: dW1 (four wide), 1: dW1 (one), 2: dW2, 3: db1, 4: db2
  if (idx < n1) {
    if (vec) {
      const unsigned I4 = (unsigned)I >> 2, j = idx / I4, i4 = idx - j * I4;
      kind = 0; sa = H; oa = j; sb = I; ob = 4 * (size_t)i4;
    } else {
      const unsigned j = idx / (unsigned)I, i = idx - j * (unsigned)I;
      kind = 1; sa = H; oa = j; sb = I; ob = i;
    }
  } else if (idx < n1 + n2) {
    const unsigned k = idx - n1, c = k / (unsigned)H, j = k - c * (unsigned)H;
    kind = 2; pa = dl; sa = C; oa = c; pb = h; sb = H; ob = j;
  } else if (idx < total) {
    const unsigned k = idx - n1 - n2, hb = n3 - (unsigned)C;   // hb = H, or 0 when the first layer's gradients are not asked for
    if (k < hb) { kind = 3; sa = H; oa = k; }
    else { kind = 4; pa = dl; sa = C; oa = k - hb; }
  }
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (kind >= 0) {
    for (int n0 = nb; n0 < ne; n0 += 16) {
      float av[16];
      float4 bv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int n = n0 + u < ne ? n0 + u : ne - 1;
        av[u] = pa[(size_t)n * sa + oa];
        if (kind == 0) bv[u] = *reinterpret_cast<const float4*>(pb + (size_t)n * sb + ob);
        else if (kind <= 2) bv[u] = make_float4(pb[(size_t)n * sb + ob], 0.0f, 0.0f, 0.0f);
        else bv[u] = make_float4(1.0f, 0.0f, 0.0f, 0.0f);
        if (n0 + u >= ne) av[u] = 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        acc.x = fmaf(av[u], bv[u].x, acc.x); acc.y = fmaf(av[u], bv[u].y, acc.y);
        acc.z = fmaf(av[u], bv[u].z, acc.z); acc.w = fmaf(av[u], bv[u].w, acc.w);
      }
    }
  }
  part[s][t] = acc;
  __syncthreads();
  if (s != 0 || kind < 0) return;
  float4 r = part[0][t];
#pragma unroll
  for (int k = 1; k < 8; ++k) {
    const float4 v = part[k][t];
    r.x += v.x; r.y += v.y; r.z += v.z; r.w += v.w;
  }
  if (kind == 0) {
    float4* o = reinterpret_cast<float4*>(dw1 + oa * (size_t)I + ob);
    if (beta1 != 0.0f) {
      const float4 old = *o;
      r.x = fmaf(beta1, old.x, r.x); r.y = fmaf(beta1, old.y, r.y); r.z = fmaf(beta1, old.z, r.z); r.w = fmaf(beta1, old.w, r.w);
    }
    *o = r;
    return;
  }
  float* o = kind == 1 ? dw1 + oa * (size_t)I + ob : kind == 2 ? dw2 + oa * (size_t)H + ob : kind == 3 ? db1 + oa : db2 + oa;
  const float beta = kind == 1 || kind == 3 ? beta1 : beta2;
  *o = beta != 0.0f ? fmaf(beta, *o, r.x) : r.x;
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

// The classifier tail is taken as one kernel per direction where a sample's chain fits a block's LDS and every block can
// afford to read the whole first layer (twice): up to 4096 inputs, 2048 hidden units, 64 classes, 2^17 weights (512 KB)
// in the first layer and 2^26 multiply-adds in its products over the batch.  Beyond that the tiled products, which read
// the weights once, are the faster form.
// I = 0 asks for the form that starts from h (the first layer's products stay with the tiled kernels).
extern "C" int rh_affine2_softmax_kl_step_supported(int32_t B, int32_t I, int32_t H, int32_t C) {
  return B > 0 && I >= 0 && H > 0 && C > 0 && I <= 4096 && H <= 2048 && C <= 64 && (long long)I * H <= (1ll << 17) &&
                 (long long)B * I * H <= (1ll << 26) && (long long)B * H < (1ll << 31)
             ? 1 : 0;
}

extern "C" int rh_affine2_softmax_kl_step(int32_t B, int32_t I, int32_t H, int32_t C, int32_t relu1, const float* x,
                                          const float* w1, const float* b1, const float* w2, const float* b2,
                                          const int32_t* labels, const float* weights, float* h, float* logits, float* p,
                                          float* max_out, int32_t* idx_out, float* loss1, float* loss_sum, float* dlogits,
                                          float* dh, float* dx, uint32_t* counter, rh_stream_t stream) {
  if (B < 0 || I < 0 || H <= 0 || C <= 0 || (I == 0) != (x == nullptr)) return RH_E_INVALID;
  if (B == 0) return 0;
  if (!rh_affine2_softmax_kl_step_supported(B, I, H, C)) return RH_E_UNSUPPORTED;
  if ((x && (!w1 || !b1)) || !w2 || !b2 || !labels || !weights || !h || !logits || !p || !max_out || !idx_out || !loss1 ||
      !loss_sum || !dlogits || !dh || !counter)
    return RH_E_INVALID;
  constexpr int NT = 1024;
  const size_t lds = sizeof(float) * ((size_t)I + 2 * (size_t)H + 64);
  ProfScope prof("affine2_softmax_kl_step",
                 4.0 * ((double)B * (2.0 * I + 3.0 * H + 4.0 * C) + 2.0 * ((double)I * H + (double)H * C)), to_stream(stream));
  hipLaunchKernelGGL((affine2_softmax_kl_step_kernel<NT>), dim3(B), dim3(NT), lds, to_stream(stream), B, I, H, C, relu1 ? 1 : 0,
                     x, w1, b1, w2, b2, labels, weights, h, logits, p, max_out, idx_out, loss1, loss_sum, dlogits, dh, dx, counter);
  return launch_status();
}

extern "C" int rh_affine2_bwd_params(int32_t B, int32_t I, int32_t H, int32_t C, const float* x, const float* h, const float* dh,
                                     const float* dlogits, float beta1, float* dw1, float* db1, float beta2, float* dw2,
                                     float* db2, rh_stream_t stream) {
  if (B < 0 || I < 0 || H <= 0 || C <= 0 || (I == 0) != (x == nullptr)) return RH_E_INVALID;
  if (!rh_affine2_softmax_kl_step_supported(B > 0 ? B : 1, I, H, C)) return RH_E_UNSUPPORTED;
  if (!h || !dlogits || !dw2 || !db2 || (x && (!dh || !dw1 || !db1)) || (!x && db1 && !dh)) return RH_E_INVALID;
  const int vec = x && I % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dw1)) & 15) == 0 ? 1 : 0;
  // (without x no dW1 items, and db1 among the bias items only where it is asked for)
  const unsigned n1 = x ? (unsigned)((size_t)H * I / (vec ? 4 : 1)) : 0u, n2 = (unsigned)((size_t)C * H),
                 n3 = (unsigned)((x || db1 ? H : 0) + C);
  const size_t total = (size_t)n1 + n2 + n3;
  ProfScope prof("affine2_bwd_params", 4.0 * ((double)B * (I + 2.0 * H + C) + (double)I * H + (double)H * C), to_stream(stream));
  hipLaunchKernelGGL(affine2_bwd_params_kernel, dim3((unsigned)cdiv<size_t>(total, 32)), dim3(256), 0, to_stream(stream), B, I, H,
                     C, vec, x, h, dh, dlogits, beta1, dw1, db1, beta2, dw2, db2, n1, n2, n3);
  return launch_status();
}

