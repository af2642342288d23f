// Convolution backward-filter (K5) and backward-bias (K6).
//   dw[ko][(c,r,s)] = sum_{n,p,q} dy[n][ko][p][q] * x[n][c][p*st+r-pad][q*st+s-pad]
// The contraction runs over up to N*P*Q = 774 400 pixels while the result is small, so the
// pixel range is cut into `splits` contiguous slices computed by different blocks; each slice
// writes its partial filter gradient to scratch and a second kernel adds the slices in a fixed
// order (results do not depend on scheduling).
#include <mutex>

#include "conv_common.h"

namespace rh {

// Column tile (filter taps) for a row tile: 128-row tiles pair with 128 columns; narrower row tiles take 256
// columns unless 128 pads the tap count less (AlexNet conv1: 363 taps = 3 x 128 - 21 instead of 2 x 256 - 149).
static int pick_bn(int bm, int cols, bool narrow = false) {
  if (bm == 128) return 128;
  if (narrow && bm == 32 && cols <= 128) return cols <= 64 ? 64 : 128;
  if (bm == 96 && round_up(cols, 128) < round_up(cols, 256)) return 128;
  return 256;
}
// Blocks of a tile shape that one CU holds at a time (registers and LDS), times 256 CUs.
static int resident_slots(int bm, int bn) {
  return 256 * (bm == 128 ? RH_OCC_128 : bm == 96 ? (bn == 128 ? 4 : 2) : (bm == 32 && bn <= 128) ? 4 : 3);
}

struct BwdFilterPlan {
  int bm, bn, tiles, splits;
  size_t tab_bytes, part_bytes;
};

static BwdFilterPlan plan_bwd_filter(const ConvDims& d) {
  BwdFilterPlan p;
  const int CRS = d.C * d.R * d.S;
  p.bm = pick_bm(d.K);
  p.bn = pick_bn(p.bm, CRS, !(d.R == 1 && d.S == 1 && d.st == 1 && d.pad == 0));
  p.tiles = cdiv(d.K, p.bm) * cdiv(CRS, p.bn);
  const long long M = (long long)d.N * d.P * d.Q;
  const int k_chunks = (int)cdiv<long long>(M, 16);
  // One full co-resident set of blocks (256 CUs x 3 blocks of this kernel per CU) and no partial
  // second round: a block that runs alone on its CU uses the matrix pipe less well than three
  // sharing it, so a ragged tail costs more than its share.  Every slice keeps at least 32 K
  // steps so the prologue and the partial-sum traffic stay small next to the contraction.
  const int slots = resident_slots(p.bm, p.bn);
  int want = slots / p.tiles;
  const int max_by_depth = (int)slices_by_depth(k_chunks, p.tiles, slots, 32, 8);
  if (want > max_by_depth) want = max_by_depth;
  if (want > 512) want = 512;
  if (want < 1) want = 1;
  // Few blocks in all (up to two per CU): the same number on every CU.  378 blocks are two on 122 CUs and one on the
  // rest, and the launch takes as long as 512 would; 9 tiles x 56 slices instead of x 42 put two on every CU
  // (NIN's 384-channel 1x1 layers: 0.100 -> 0.086 ms).  One block per CU pays about 15 % for having nothing beside it.
  if ((long long)p.tiles * want <= slots / 2) {
    auto cost = [&](int s) {
      const long long rounds = cdiv<long long>((long long)p.tiles * s, 256);
      return (double)rounds * ((double)k_chunks / s + 6.0) * (rounds == 1 ? 1.15 : 1.0);
    };
    int best = want;
    double best_c = cost(want);
    for (int r = 1; r <= 4; ++r) {
      const int s = 256 * r / p.tiles;
      if (s < 1 || s > 512 || s > k_chunks / 8) continue;
      const double c = cost(s);
      if (c < best_c) { best_c = c; best = s; }
    }
    want = best;
  }
  p.splits = want;
  p.tab_bytes = align256(sizeof(int4) * (size_t)round_up(CRS, kTabPad));
  p.part_bytes = align256(sizeof(float) * (size_t)p.splits * d.K * CRS);
  return p;
}

// Sum of part[s*stride + idx] over s < splits in a fixed order: four interleaved partial sums (so that four
// loads are in flight per thread), combined as (a0 + a1) + (a2 + a3).
__device__ __forceinline__ float sum_splits(const float* __restrict__ part, int splits, long long stride, unsigned idx) {
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  const float* p = part + idx;
  int s = 0;
  for (; s + 3 < splits; s += 4) {
    a0 += p[(long long)s * stride];
    a1 += p[(long long)(s + 1) * stride];
    a2 += p[(long long)(s + 2) * stride];
    a3 += p[(long long)(s + 3) * stride];
  }
  for (; s < splits; ++s) a0 += p[(long long)s * stride];
  return (a0 + a1) + (a2 + a3);
}

// Column sums of an [N][K] matrix (dy of an affine layer, or per-image plane sums) for the 64 columns from 64 b on by
// one block of 256 threads: its 4 waves take every fourth row and are combined through LDS in a fixed order.
__device__ __forceinline__ void bwd_bias_rows_block(const float* __restrict__ dy, int N, int K, float alpha, float beta,
                                                    float* __restrict__ db, unsigned b) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int k = (int)b * 64 + lane;
  // eight independent partial sums per thread (rows wave, wave + 4, ... in turn): the loop is a chain of memory round
  // trips, so its length is what the kernel takes
  float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  if (k < K) {
    int n = wave;
    for (; n + 28 < N; n += 32) {
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] += dy[(size_t)(n + 4 * j) * K + k];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (n + 4 * j < N) a[j] += dy[(size_t)(n + 4 * j) * K + k];
  }
  __shared__ float sm[4][64];
  sm[wave][lane] = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
  __syncthreads();
  if (wave == 0 && k < K) {
    float v = alpha * ((sm[0][lane] + sm[1][lane]) + (sm[2][lane] + sm[3][lane]));
    if (beta != 0.0f) v += beta * db[k];
    db[k] = v;
  }
}

// The same sum for one channel by a block of 256 threads, for the small layers whose bias gradient rides in another
// launch: wave w takes the images w, w + 4, ..., eight of them at a time with four strides of the plane each (32 loads
// in flight per lane; a block is alone with its channel, so the chain of memory round trips is what it takes).  A fixed
// order, not the one of bwd_bias_kernel.
__device__ __forceinline__ void bwd_bias_planes_job(const float* __restrict__ dy, int N, int K, int plane, float alpha,
                                                    float beta, float* __restrict__ db, int k) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  for (int n0 = wave; n0 < N; n0 += 32) {
    for (int i0 = lane; i0 < plane; i0 += 256) {
      float v[8][4];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int n = n0 + 4 * u;
        const float* p = dy + ((size_t)(n < N ? n : 0) * K + k) * plane;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[u][j] = n < N && i0 + 64 * j < plane ? p[i0 + 64 * j] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) a[u] += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
    }
  }
  float acc = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
  __shared__ float part[4];
  if (lane == 0) part[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float v = alpha * ((part[0] + part[1]) + (part[2] + part[3]));
    if (beta != 0.0f) v += beta * db[k];
    db[k] = v;
  }
}

// A bias gradient that rides in a reduction launch (BiasJob): block b of the job, 256 threads.
__device__ __forceinline__ void bias_job_block(const BiasJob& j, unsigned b) {
  if (j.plane == 1) bwd_bias_rows_block(j.src, j.N, j.K, j.alpha, j.beta, j.db, b);
  else bwd_bias_planes_job(j.src, j.N, j.K, j.plane, j.alpha, j.beta, j.db, (int)b);
}

// Second pass of a split contraction: out[i*ld + j] = alpha * sum_s part[s][i*cols + j] + beta*out.
// (+ bias_col[j], then ReLU, where given: the epilogue of an affine layer's forward product)
__global__ void split_reduce_kernel(const float* __restrict__ part, int splits, long long split_stride,
                                    float* __restrict__ out, int rows, int cols, int ld, float alpha,
                                    float beta, const float* __restrict__ bias_col, int relu, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  const unsigned nb = bj.db ? bj.first : gridDim.x;
  const unsigned total = (unsigned)rows * (unsigned)cols;  // a filter gradient / GEMM result: far below 2^31
  for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += nb * blockDim.x) {
    const float acc = sum_splits(part, splits, split_stride, idx);
    const int i = (int)(idx / (unsigned)cols), j = (int)(idx - (unsigned)i * (unsigned)cols);
    float* dst = out + (size_t)i * ld + j;
    float val = alpha * acc;
    if (beta != 0.0f) val += beta * *dst;
    if (bias_col) val += bias_col[j];
    if (relu) val = val > 0.0f ? val : 0.0f;
    *dst = val;
  }
}

// The same over a dense result (ld == cols) in 16-byte groups: the sums of each element are formed in the same order.
__device__ __forceinline__ void bias_relu4(float4& v, unsigned idx, const float* __restrict__ bias_col, unsigned cols4, int relu) {
  if (bias_col) {
    const float4 b = reinterpret_cast<const float4*>(bias_col)[idx % cols4];
    v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
  }
  if (relu) {
    v.x = v.x > 0.0f ? v.x : 0.0f; v.y = v.y > 0.0f ? v.y : 0.0f;
    v.z = v.z > 0.0f ? v.z : 0.0f; v.w = v.w > 0.0f ? v.w : 0.0f;
  }
}

__global__ __launch_bounds__(256) void split_reduce_vec_kernel(const float4* __restrict__ part, int splits, long long stride4,
                                                               float4* __restrict__ out, unsigned total4, float alpha,
                                                               float beta, const float* __restrict__ bias_col,
                                                               unsigned cols4, int relu, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  const unsigned idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total4) return;
  const float4 z = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  float4 a0 = z, a1 = z, a2 = z, a3 = z;
  auto add = [](float4& a, const float4 v) { a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; };
  const float4* p = part + idx;
  int s = 0;
  for (; s + 3 < splits; s += 4) {
    add(a0, p[(long long)s * stride4]);
    add(a1, p[(long long)(s + 1) * stride4]);
    add(a2, p[(long long)(s + 2) * stride4]);
    add(a3, p[(long long)(s + 3) * stride4]);
  }
  for (; s < splits; ++s) add(a0, p[(long long)s * stride4]);
  float4 v;
  v.x = alpha * ((a0.x + a1.x) + (a2.x + a3.x));
  v.y = alpha * ((a0.y + a1.y) + (a2.y + a3.y));
  v.z = alpha * ((a0.z + a1.z) + (a2.z + a3.z));
  v.w = alpha * ((a0.w + a1.w) + (a2.w + a3.w));
  if (beta != 0.0f) {
    const float4 o = out[idx];
    v.x += beta * o.x; v.y += beta * o.y; v.z += beta * o.z; v.w += beta * o.w;
  }
  bias_relu4(v, idx, bias_col, cols4, relu);
  out[idx] = v;
}

// The same for a small dense result under many slices (a 1x1 layer's 96 x 96 gradient from a thousand slices): one
// thread per element would be a few dozen waves that each walk every slice.  Here 32 threads share a 16-byte group:
// thread j of them adds slices j, j + 32, ... in increasing order, and the 32 sums meet in LDS in a fixed pairwise tree.
// A block holds eight consecutive groups (128 bytes of every slice it reads).
constexpr int kReduceLanes = 32, kReduceGroups = 8;
__global__ __launch_bounds__(256) void split_reduce_vec_par_kernel(const float4* __restrict__ part, int splits, long long stride4,
                                                                   float4* __restrict__ out, unsigned total4, float alpha,
                                                                   float beta, const float* __restrict__ bias_col,
                                                                   unsigned cols4, int relu, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  __shared__ float4 red[kReduceLanes][kReduceGroups];
  const int g = (int)threadIdx.x % kReduceGroups, j = (int)threadIdx.x / kReduceGroups;
  const unsigned idx = blockIdx.x * kReduceGroups + g;
  float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (idx < total4) {
    const float4* p = part + idx;
    for (int s = j; s < splits; s += kReduceLanes) {
      const float4 v = p[(long long)s * stride4];
      a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
    }
  }
  red[j][g] = a;
  for (int w = kReduceLanes / 2; w >= 1; w >>= 1) {
    __syncthreads();
    if (j < w) {
      const float4 u = red[j][g], v = red[j + w][g];
      red[j][g] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
    }
  }
  if (j == 0 && idx < total4) {
    const float4 t = red[0][g];
    float4 v = make_float4(alpha * t.x, alpha * t.y, alpha * t.z, alpha * t.w);
    if (beta != 0.0f) {
      const float4 o = out[idx];
      v.x += beta * o.x; v.y += beta * o.y; v.z += beta * o.z; v.w += beta * o.w;
    }
    bias_relu4(v, idx, bias_col, cols4, relu);
    out[idx] = v;
  }
}

// The many-slice form for results that are not dense 16-byte groups (odd extents, a padded leading dimension).
__global__ __launch_bounds__(256) void split_reduce_par_kernel(const float* __restrict__ part, int splits, long long split_stride,
                                                               float* __restrict__ out, int rows, int cols, int ld, float alpha,
                                                               float beta, const float* __restrict__ bias_col, int relu, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  __shared__ float red[kReduceLanes][kReduceGroups];
  const int g = (int)threadIdx.x % kReduceGroups, j = (int)threadIdx.x / kReduceGroups;
  const unsigned total = (unsigned)rows * (unsigned)cols;
  const unsigned idx = blockIdx.x * kReduceGroups + g;
  float a = 0.0f;
  if (idx < total)
    for (int s = j; s < splits; s += kReduceLanes) a += part[(long long)s * split_stride + idx];
  red[j][g] = a;
  for (int w = kReduceLanes / 2; w >= 1; w >>= 1) {
    __syncthreads();
    if (j < w) red[j][g] += red[j + w][g];
  }
  if (j == 0 && idx < total) {
    const int i = (int)(idx / (unsigned)cols), c = (int)(idx - (unsigned)i * (unsigned)cols);
    float* dst = out + (size_t)i * ld + c;
    float val = alpha * red[0][g];
    if (beta != 0.0f) val += beta * *dst;
    if (bias_col) val += bias_col[c];
    if (relu) val = val > 0.0f ? val : 0.0f;
    *dst = val;
  }
}

void launch_split_reduce(const float* part, int splits, long long split_stride, float* out, int rows, int cols,
                         int ld, float alpha, float beta, hipStream_t stream, const float* bias_col, int relu,
                         const BiasJob* bias_job) {
  const size_t total = (size_t)rows * cols;
  BiasJob bj;
  if (bias_job) bj = *bias_job;
  const unsigned jb = bj.blocks();
  ProfScope prof("split_reduce", 4.0 * (double)total * (splits + 1) + (jb ? 4.0 * (double)bj.N * bj.K * bj.plane : 0.0), stream);
  if (ld == cols && cols % 4 == 0 && split_stride % 4 == 0 &&
      ((reinterpret_cast<uintptr_t>(part) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(bias_col)) & 15) == 0) {
    if (total / 4 < 64 * 1024 && splits >= 2 * kReduceLanes) {   // under 1024 waves with a thread per group
      bj.first = (unsigned)cdiv<size_t>(total / 4, kReduceGroups);
      hipLaunchKernelGGL(split_reduce_vec_par_kernel, dim3(bj.first + jb), dim3(256), 0,
                         stream, reinterpret_cast<const float4*>(part), splits, split_stride / 4,
                         reinterpret_cast<float4*>(out), (unsigned)(total / 4), alpha, beta, bias_col, (unsigned)(cols / 4), relu, bj);
      return;
    }
    bj.first = stream_grid(total / 4, 256);
    hipLaunchKernelGGL(split_reduce_vec_kernel, dim3(bj.first + jb), dim3(256), 0, stream,
                       reinterpret_cast<const float4*>(part), splits, split_stride / 4, reinterpret_cast<float4*>(out),
                       (unsigned)(total / 4), alpha, beta, bias_col, (unsigned)(cols / 4), relu, bj);
    return;
  }
  if (total < 256 * 1024 && splits >= 2 * kReduceLanes) {
    bj.first = (unsigned)cdiv<size_t>(total, kReduceGroups);
    hipLaunchKernelGGL(split_reduce_par_kernel, dim3(bj.first + jb), dim3(256), 0, stream, part,
                       splits, split_stride, out, rows, cols, ld, alpha, beta, bias_col, relu, bj);
    return;
  }
  bj.first = stream_grid(total, 256);
  hipLaunchKernelGGL(split_reduce_kernel, dim3(bj.first + jb), dim3(256), 0, stream, part, splits,
                     split_stride, out, rows, cols, ld, alpha, beta, bias_col, relu, bj);
}

// ---- scalar-offset path ------------------------------------------------------------------------
// Both operands are read with lanes along rows and a wave-uniform offset per contraction index
// (an output pixel), from channel-last scratch copies:
//   A = dyT[pix][ko]                      (rows ko;      k offset = pix*Kout*4)
//   B = xT[n][hp][wp][c], zero padded     (rows (r,s,c); vbase = 4*((r*Wp+s)*C+c), k offset from a
//                                          per-pixel table 4*C*((n*Hp + p*st)*Wp + q*st))
// The result comes out as dw'[ko][(r,s,c)]; the reduction kernel puts it back in [ko][c][r][s] order.
// The channel-last path pays two transposes; it wins when the contraction is deep relative to them.
static bool use_soff_bwd_filter(const ConvDims& d) {
  // FLOPs of the contraction per byte the two transposes move (measured: 11x11 stride-4 first layers at 59,
  // small 5x5 layers at 75-78 and 1x1 at 12 lose or tie; 3x3 / 5x5 layers at 288-402 win by 25 %)
  const double flops = 2.0 * d.K * d.C * d.R * d.S * (double)d.N * d.P * d.Q;
  const double bytes = 8.0 * ((double)d.y_elems + (double)d.N * d.C * (d.H + 2 * d.pad) * (d.W + 2 * d.pad));
  // The contraction itself runs at about 100 (64-row tiles) / 125 (128-row) TFLOP/s on this path against 65 / 90 with
  // the gather loaders, and the transposes move their bytes at about 3.8 TB/s: break-even near 50 / 85 FLOPs per byte
  // (measured: 64 -> 64 channels 3x3 on 56x56 at 70 wins by 13 %, 128 -> 128 on 28x28 at 134 by 11 %, a stride-2
  // 64 -> 128 layer at 46 loses by 6 %).
  // 32-row tiles (half of the loader rows idle) tie at 75-78.
  const int bm = pick_bm(d.K);
  return flops / bytes >= (bm == 64 ? 60.0 : bm == 32 ? 150.0 : 100.0);
}

struct BwdFilterSoffPlan {
  int n_k, Hp, Wp, bm, bn, tiles, splits;
  size_t tab_bytes, dyt_bytes, xt_bytes, part_bytes;
  bool ok;
  size_t total() const { return tab_bytes + dyt_bytes + xt_bytes + part_bytes; }
};

static BwdFilterSoffPlan plan_bwd_filter_soff(const ConvDims& d) {
  BwdFilterSoffPlan p;
  const int CRS = d.C * d.R * d.S;
  const long long M = (long long)d.N * d.P * d.Q;
  p.Hp = d.H + 2 * d.pad;
  p.Wp = d.W + 2 * d.pad;
  p.n_k = (int)((M + kTabPad - 1) / kTabPad * kTabPad);
  p.bm = pick_bm(d.K);
  p.bn = pick_bn(p.bm, CRS);
  p.tiles = cdiv(d.K, p.bm) * cdiv(CRS, p.bn);
  const int k_chunks = p.n_k / 16;
  const int slots = resident_slots(p.bm, p.bn);
  int want = slots / p.tiles;
  const int max_by_depth = (int)slices_by_depth(k_chunks, p.tiles, slots, 32, 8);
  if (want > max_by_depth) want = max_by_depth;
  if (want > 256) want = 256;
  if (want < 1) want = 1;
  p.splits = want;
  p.tab_bytes = align256(sizeof(int) * (size_t)p.n_k);
  p.dyt_bytes = align256(sizeof(float) * (size_t)p.n_k * d.K);
  p.xt_bytes = align256(sizeof(float) * (size_t)d.N * p.Hp * p.Wp * d.C);
  p.part_bytes = align256(sizeof(float) * (size_t)p.splits * d.K * CRS);
  p.ok = M > 0 && p.dyt_bytes <= kMaxBufferBytes && p.xt_bytes <= kMaxBufferBytes &&
         (long long)d.S * d.C < (1 << 24);
  return p;
}

// dst[n][pix][c] (pix over Hp x Wp, zero halo) = src[n][c][h][w]: 32 x 32 tiles through LDS so that both
// the reads (along w) and the writes (along c) are contiguous.
__device__ __forceinline__ void nchw_to_nhwc_body(float* __restrict__ lds, int bx, int by, int bz,
                                                  const float* __restrict__ src, float* __restrict__ dst,
                                                  int C, int H, int W, int Hp, int Wp, int halo) {
  float (*tile)[33] = reinterpret_cast<float (*)[33]>(lds);
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int pix0 = bx * 32, c0 = by * 32, n = bz;
  const int HpWp = Hp * Wp;
  {
    const int pix = pix0 + tx;
    const int hp = pix / Wp, wp = pix - hp * Wp;
    const int h = hp - halo, w = wp - halo;
    const bool inside = pix < HpWp && (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W;
#pragma unroll
    for (int j = 0; j < 32; j += 8) {
      const int c = c0 + ty + j;
      tile[ty + j][tx] = (inside && c < C) ? src[(((size_t)n * C + c) * H + h) * W + w] : 0.0f;
    }
  }
  __syncthreads();
  const int c = c0 + tx;
#pragma unroll
  for (int j = 0; j < 32; j += 8) {
    const int pix = pix0 + ty + j;
    if (pix < HpWp && c < C) dst[((size_t)n * HpWp + pix) * C + c] = tile[tx][ty + j];
  }
}

__global__ __launch_bounds__(256) void nchw_to_nhwc_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                           int C, int H, int W, int Hp, int Wp, int halo) {
  __shared__ float tile[32 * 33];
  nchw_to_nhwc_body(tile, blockIdx.x, blockIdx.y, blockIdx.z, src, dst, C, H, W, Hp, Wp, halo);
}

// The same for C % 4 == 0 in 16-byte accesses (4-byte accesses top out near 3.8 TB/s on this GPU): a block moves
// 64 pixels x 64 channels; a thread reads four consecutive pixels of one channel (one 16-byte load where they lie in
// one source row, which need not be 16-byte aligned; element by element across row ends and the halo) and writes four
// consecutive channels of one pixel.  LDS tile [pixel][channel], the 16-byte channel groups of a row permuted by the
// pixel's quad index so that the scattered writes of a wave spread over the banks.
// BIAS: the pass over dy that backward-filter makes anyway also yields the bias gradient's first stage.  A block then
// walks all 64-pixel pieces of its (image, 64 channels) itself (grid x = 1), each thread adding its sixteen pixels of
// one channel piece after piece, and leaves bias_part[n][c] = sum over the plane of src[n][c][.]; the sums over n are
// bwd_bias_rows_kernel's.  Fixed order: the same call gives the same bits.
typedef float float4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// (bx, by, bz) of a grid (gx, ., .): the block's place, given by the caller so that the body can also run as one
// range of blocks of a larger launch; `tile` is the block's 16 KB of LDS.
template <bool BIAS>
__device__ __forceinline__ void nchw_to_nhwc_vec_body(float* __restrict__ tile, int bx, int by, int bz, int gx,
                                                      const float* __restrict__ src, float* __restrict__ dst,
                                                      int C, int H, int W, int Hp, int Wp, int halo,
                                                      float* __restrict__ bias_part, long long src_elems) {
  const int c0 = by * 64, n = bz;
  const int HpWp = Hp * Wp;
  float bsum = 0.0f;
  for (int pix0 = bx * 64; pix0 < HpWp; pix0 += gx * 64) {
  {
    const int pq = threadIdx.x & 15, cl0 = threadIdx.x >> 4;
    const int pix = pix0 + 4 * pq;
    // Element offsets within a plane, -1 = zero.  A plane is dense and the map from padded pixels to source elements
    // keeps their order, so the source elements of four consecutive pixels are one run of consecutive addresses
    // however the four lie across row ends and the halo: one 16-byte load from the run's start (4-byte aligned)
    // brings them all, and each pixel picks its element by its distance from that start.
    int off[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int pe = pix + e, hpe = pe / Wp, he = hpe - halo, we = pe - hpe * Wp - halo;
      off[e] = (pe < HpWp && (unsigned)he < (unsigned)H && (unsigned)we < (unsigned)W) ? he * W + we : -1;
    }
    int first = off[3];
    if (off[2] >= 0) first = off[2];
    if (off[1] >= 0) first = off[1];
    if (off[0] >= 0) first = off[0];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int cl = cl0 + 16 * i, c = c0 + cl;
      float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (c < C && first >= 0) {
        const long long base = ((long long)n * C + c) * ((long long)H * W);
        const float* plane = src + base;
        if (base + first + 3 < src_elems) {
          const float4_a4 q = *reinterpret_cast<const float4_a4*>(plane + first);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int d = off[e] - first;
            const float t = d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
            v[e] = off[e] >= 0 ? t : 0.0f;
          }
        } else {   // the tensor's last three elements
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (off[e] >= 0) v[e] = plane[off[e]];
        }
      }
      const int col = 4 * ((cl >> 2) ^ pq) + (cl & 3);
#pragma unroll
      for (int e = 0; e < 4; ++e) tile[(4 * pq + e) * 64 + col] = v[e];
    }
  }
  __syncthreads();
  const int cq = threadIdx.x & 15, c = c0 + 4 * cq;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int pl = (threadIdx.x >> 4) + 16 * j, pix = pix0 + pl;
    if (pix < HpWp && c < C) {
      const float4 q = *reinterpret_cast<const float4*>(&tile[pl * 64 + 4 * (cq ^ ((pl >> 2) & 15))]);
      *reinterpret_cast<float4*>(dst + ((size_t)n * HpWp + pix) * C + c) = q;
    }
  }
  if (BIAS) {
    // channel cl of pixels 16 q .. 16 q + 15 of this piece (pixels past the plane and channels past C were staged as 0)
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int pl = 16 * q + e;
      bsum += tile[pl * 64 + 4 * ((cl >> 2) ^ ((pl >> 2) & 15)) + (cl & 3)];
    }
  }
  __syncthreads();   // the next piece overwrites the tile
  }
  if (BIAS) {
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    tile[q * 64 + cl] = bsum;
    __syncthreads();
    if (q == 0 && c0 + cl < C)
      bias_part[(size_t)n * C + c0 + cl] = (tile[cl] + tile[64 + cl]) + (tile[128 + cl] + tile[192 + cl]);
  }
}

template <bool BIAS>
__global__ __launch_bounds__(256) void nchw_to_nhwc_vec_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                               int C, int H, int W, int Hp, int Wp, int halo,
                                                               float* __restrict__ bias_part) {
  __shared__ __attribute__((aligned(16))) float tile[64 * 64];
  nchw_to_nhwc_vec_body<BIAS>(tile, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x, src, dst, C, H, W, Hp, Wp, halo, bias_part,
                              (long long)gridDim.z * C * H * W);
}

// The 16-byte form can carry the per-image plane sums along (bias_part, N x C floats; no halo).
static bool nhwc_vec_ok(int C, const float* dst) { return C % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0; }

static void launch_nchw_to_nhwc(const float* src, float* dst, int N, int C, int H, int W, int Hp, int Wp, int halo,
                                hipStream_t stream, float* bias_part = nullptr) {
  ProfScope prof("nchw_to_nhwc", 4.0 * ((double)N * C * H * W + (double)N * C * Hp * Wp), stream);
  if (nhwc_vec_ok(C, dst)) {
    if (bias_part) {
      dim3 grid(1, (unsigned)cdiv(C, 64), (unsigned)N);
      hipLaunchKernelGGL(nchw_to_nhwc_vec_kernel<true>, grid, dim3(256), 0, stream, src, dst, C, H, W, Hp, Wp, halo, bias_part);
      return;
    }
    dim3 grid((unsigned)cdiv(Hp * Wp, 64), (unsigned)cdiv(C, 64), (unsigned)N);
    hipLaunchKernelGGL(nchw_to_nhwc_vec_kernel<false>, grid, dim3(256), 0, stream, src, dst, C, H, W, Hp, Wp, halo,
                       (float*)nullptr);
    return;
  }
  dim3 grid((unsigned)cdiv(Hp * Wp, 32), (unsigned)cdiv(C, 32), (unsigned)N);
  hipLaunchKernelGGL(nchw_to_nhwc_kernel, grid, dim3(256), 0, stream, src, dst, C, H, W, Hp, Wp, halo);
}

// soff[pix] = 4*C*((n*Hp + p*st)*Wp + q*st) for pix = (n,p,q) < M, else 0; also zeroes the rows M..n_k of dyT.
__device__ __forceinline__ void prep_bwd_filter_soff_body(int first, int stride, int* __restrict__ soff,
                                                          float* __restrict__ dyT, int n_k, int M, int PQ, int Q, int st,
                                                          int Hp, int Wp, int C, int Kout);
__global__ void prep_bwd_filter_soff_kernel(int* __restrict__ soff, float* __restrict__ dyT, int n_k, int M, int PQ,
                                            int Q, int st, int Hp, int Wp, int C, int Kout) {
  prep_bwd_filter_soff_body(blockIdx.x * blockDim.x + threadIdx.x, gridDim.x * blockDim.x, soff, dyT, n_k, M, PQ, Q, st, Hp, Wp,
                            C, Kout);
}

__device__ __forceinline__ void prep_bwd_filter_soff_body(int first, int stride, int* __restrict__ soff,
                                                          float* __restrict__ dyT, int n_k, int M, int PQ, int Q, int st,
                                                          int Hp, int Wp, int C, int Kout) {
  for (int pix = first; pix < n_k; pix += stride) {
    int off = 0;
    if (pix < M) {
      const int n = pix / PQ, pq = pix - n * PQ, p = pq / Q, q = pq - p * Q;
      off = ((n * Hp + p * st) * Wp + q * st) * C * 4;
    } else {
      for (int k = 0; k < Kout; ++k) dyT[(size_t)pix * Kout + k] = 0.0f;
    }
    soff[pix] = off;
  }
}

// The three operand preparations of the scalar-offset backward-filter in one launch (they are independent of one
// another): blocks [0, nb_dy) copy dy channel-last (BIAS: with the plane sums), the next nb_x blocks copy x channel-last
// with its zero border, the rest write the offset table and zero dyT's tail rows.
struct NhwcCopyArgs {
  const float* src; float* dst;
  int C, H, W, Hp, Wp, halo;
  long long elems;  // elements of src
  int vec;      // 16-byte form (64 x 64 pieces) or the element form (32 x 32 pieces)
  int gx, gy;   // grid of pieces: (gx, gy, images)
};

template <bool BIAS>
__global__ __launch_bounds__(256) void bwd_filter_prep_kernel(NhwcCopyArgs dy, float* __restrict__ bias_part, int nb_dy,
                                                              NhwcCopyArgs x, int nb_x, int* __restrict__ soff, int n_k, int M,
                                                              int PQ, int Q, int st, int Kout) {
  __shared__ __attribute__((aligned(16))) float tile[64 * 64];
  int b = blockIdx.x;
  if (b < nb_dy) {
    const int bx = b % dy.gx, t = b / dy.gx;
    if (BIAS || dy.vec)
      nchw_to_nhwc_vec_body<BIAS>(tile, bx, t % dy.gy, t / dy.gy, dy.gx, dy.src, dy.dst, dy.C, dy.H, dy.W, dy.Hp, dy.Wp, dy.halo,
                                  bias_part, dy.elems);
    else
      nchw_to_nhwc_body(tile, bx, t % dy.gy, t / dy.gy, dy.src, dy.dst, dy.C, dy.H, dy.W, dy.Hp, dy.Wp, dy.halo);
    return;
  }
  b -= nb_dy;
  if (b < nb_x) {
    const int bx = b % x.gx, t = b / x.gx;
    if (x.vec)
      nchw_to_nhwc_vec_body<false>(tile, bx, t % x.gy, t / x.gy, x.gx, x.src, x.dst, x.C, x.H, x.W, x.Hp, x.Wp, x.halo, nullptr,
                                   x.elems);
    else
      nchw_to_nhwc_body(tile, bx, t % x.gy, t / x.gy, x.src, x.dst, x.C, x.H, x.W, x.Hp, x.Wp, x.halo);
    return;
  }
  b -= nb_x;
  const int nb = (int)gridDim.x - nb_dy - nb_x;
  prep_bwd_filter_soff_body(b * (int)blockDim.x + (int)threadIdx.x, nb * (int)blockDim.x, soff, dy.dst, n_k, M, PQ, Q, st, x.Hp,
                            x.Wp, x.C, Kout);
}

// dw[ko][c][r][s] = alpha * sum_s part[s][ko][(r,s,c)] + beta * dw
__global__ void split_reduce_rsc_kernel(const float* __restrict__ part, int splits, long long split_stride,
                                        float* __restrict__ dw, int K, int C, int R, int S, float alpha, float beta, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  const unsigned nb = bj.db ? bj.first : gridDim.x;
  const int CRS = C * R * S;
  const unsigned total = (unsigned)K * (unsigned)CRS;
  for (unsigned idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += nb * blockDim.x) {
    const float acc = sum_splits(part, splits, split_stride, idx);
    const int ko = (int)(idx / (unsigned)CRS), j = (int)(idx - (unsigned)ko * (unsigned)CRS);
    const int r = j / (S * C), rem = j - r * (S * C), s2 = rem / C, c = rem - s2 * C;
    float* dst = dw + (((size_t)ko * C + c) * R + r) * S + s2;
    float val = alpha * acc;
    if (beta != 0.0f) val += beta * *dst;
    *dst = val;
  }
}

// The same for C % 4 == 0: a thread takes four consecutive channels of one (ko, r, s), read as 16-byte groups from
// every slab (4-byte reads top out well below what 16-byte reads reach); sums in the order of sum_splits.
__global__ __launch_bounds__(256) void split_reduce_rsc_vec_kernel(const float4* __restrict__ part, int splits, long long stride4,
                                                                   float* __restrict__ dw, int K, int C, int R, int S,
                                                                   float alpha, float beta, BiasJob bj) {
  if (bj.db && blockIdx.x >= bj.first) { bias_job_block(bj, blockIdx.x - bj.first); return; }
  const int CRS4 = (C * R * S) >> 2;
  const unsigned total4 = (unsigned)K * (unsigned)CRS4;
  const unsigned idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total4) return;
  const float4 z = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  float4 a0 = z, a1 = z, a2 = z, a3 = z;
  auto add = [](float4& a, const float4 v) { a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; };
  const float4* p = part + idx;
  int sp = 0;
  for (; sp + 3 < splits; sp += 4) {
    add(a0, p[(long long)sp * stride4]);
    add(a1, p[(long long)(sp + 1) * stride4]);
    add(a2, p[(long long)(sp + 2) * stride4]);
    add(a3, p[(long long)(sp + 3) * stride4]);
  }
  for (; sp < splits; ++sp) add(a0, p[(long long)sp * stride4]);
  const float v[4] = {(a0.x + a1.x) + (a2.x + a3.x), (a0.y + a1.y) + (a2.y + a3.y), (a0.z + a1.z) + (a2.z + a3.z),
                      (a0.w + a1.w) + (a2.w + a3.w)};
  const int ko = (int)(idx / (unsigned)CRS4), j = 4 * (int)(idx - (unsigned)ko * (unsigned)CRS4);
  const int r = j / (S * C), rem = j - r * (S * C), s2 = rem / C, c = rem - s2 * C;
  float* dst = dw + (((size_t)ko * C + c) * R + r) * S + s2;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float val = alpha * v[e];
    if (beta != 0.0f) val += beta * dst[(size_t)e * R * S];
    dst[(size_t)e * R * S] = val;
  }
}

template <class T>
static int run_bwd_filter_soff(const RowSParams& ap, const RowSParams& bp, const EpiParams& ep, int n_k, int k_true,
                               int splits, int* used, hipStream_t stream, const char* tag) {
  constexpr int AROWS = T::BM % 64 == 0 ? T::BM : (T::BM + 63) / 64 * 64;
  typedef LoadRowS<AROWS, T::BK, T::NT, true> AL;
  typedef LoadRowS<T::BN, T::BK, T::NT, false> BL;
  return launch_mfma_gemm<T, AL, BL, false, PassConvBwdFilter>(ap, bp, ep, n_k, splits, used, stream, tag, k_true);
}

template <class T>
static int run_bwd_filter(const PixDyParams& ap, const PixXParams& bp, const EpiParams& ep, int M,
                          int splits, int* used, hipStream_t stream, const char* tag) {
  typedef LoadPixDy<T::BM, T::BK, T::NT> AL;
  if (bp.pad == 0) {
    typedef LoadPixX<T::BN, T::BK, T::NT, true> BL;
    return launch_mfma_gemm<T, AL, BL, false, PassConvBwdFilter>(ap, bp, ep, M, splits, used, stream, tag);
  }
  typedef LoadPixX<T::BN, T::BK, T::NT, false> BL;
  return launch_mfma_gemm<T, AL, BL, false, PassConvBwdFilter>(ap, bp, ep, M, splits, used, stream, tag);
}

// 1x1 filter, stride 1, no padding: x is read exactly like dy (row c of pixel (n, pq) at (n*C + c)*PQ + pq), so both
// operands take the pixel loader without tap table or bounds checks.
template <class T>
static int run_bwd_filter_1x1(const PixDyParams& ap, const PixDyParams& bp, const EpiParams& ep, int M,
                              int splits, int* used, hipStream_t stream, const char* tag) {
  typedef LoadPixDy<T::BM, T::BK, T::NT> AL;
  typedef LoadPixDy<T::BN, T::BK, T::NT> BL;
  return launch_mfma_gemm<T, AL, BL, false, PassConvBwdFilter>(ap, bp, ep, M, splits, used, stream, tag);
}

// db[k] = alpha * sum_{n, i<plane} dy[(n*K + k)*plane + i] + beta * db[k].  grid = (K, 1): the 16 waves of
// a block each walk whole planes (one image at a time), lanes along the plane, no index divisions.
__global__ __launch_bounds__(1024) void bwd_bias_kernel(const float* __restrict__ dy, int N, int K,
                                                        int plane, float alpha, float beta,
                                                        float* __restrict__ db) {
  const int k = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  // four independent partial sums per lane: the loads of a plane are in flight together instead of one by one
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  for (int n = wave; n < N; n += nwaves) {
    const float* p = dy + ((size_t)n * K + k) * plane;
    // sixteen loads of a plane in flight per lane, added in the order of the plain loop (groups of four strides to
    // a0..a3 while four are left, the rest to a0)
    for (int i0 = lane; i0 < plane; i0 += 1024) {
      float v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = i0 + 64 * j < plane ? p[i0 + 64 * j] : 0.0f;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int i = i0 + 256 * g;
        if (i + 192 < plane) {
          a0 += v[4 * g]; a1 += v[4 * g + 1]; a2 += v[4 * g + 2]; a3 += v[4 * g + 3];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i + 64 * e < plane) a0 += v[4 * g + e];
        }
      }
    }
  }
  float acc = (a0 + a1) + (a2 + a3);
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
  __shared__ float part[16];
  if (lane == 0) part[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (int i = 0; i < nwaves; ++i) s += part[i];
    float v = alpha * s;
    if (beta != 0.0f) v += beta * db[k];
    db[k] = v;
  }
}

// Two-stage form: stage 1 streams dy as an [N*K][plane] matrix, one wave per row, and writes the row sums
// rowsum[n*K + k]; stage 2 (bwd_bias_rows_kernel) adds them over n in a fixed order.
__global__ __launch_bounds__(256) void bwd_bias_rowsum_kernel(const float* __restrict__ dy, long long rows, int plane,
                                                              float* __restrict__ rowsum) {
  const int lane = threadIdx.x & 63;
  const long long wave0 = (long long)blockIdx.x * 4 + (threadIdx.x >> 6), stride = (long long)gridDim.x * 4;
  for (long long r = wave0; r < rows; r += stride) {
    const float* p = dy + r * plane;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    int i = lane;
    for (; i + 192 < plane; i += 256) {
      a0 += p[i];
      a1 += p[i + 64];
      a2 += p[i + 128];
      a3 += p[i + 192];
    }
    for (; i < plane; i += 64) a0 += p[i];
    float acc = (a0 + a1) + (a2 + a3);
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
    if (lane == 0) rowsum[r] = acc;
  }
}

// Small planes (13x13, 27x27): dy viewed as an [N][K*plane] matrix; block column (j, g) adds images n = g, g+G, ...
// for 256 consecutive j, fully coalesced: part[g][j].  bwd_bias_planes_finish_kernel then adds, per channel, the G
// partial planes in a fixed order.
__global__ __launch_bounds__(256) void bwd_bias_colsum_kernel(const float* __restrict__ dy, int N, int KP,
                                                              float* __restrict__ part) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int g = blockIdx.y, G = gridDim.y;
  if (j >= KP) return;
  float a0 = 0.0f, a1 = 0.0f;
  int n = g;
  for (; n + G < N; n += 2 * G) {
    a0 += dy[(size_t)n * KP + j];
    a1 += dy[(size_t)(n + G) * KP + j];
  }
  if (n < N) a0 += dy[(size_t)n * KP + j];
  part[(size_t)g * KP + j] = a0 + a1;
}

// The same with four columns per thread through 16-byte loads (K*plane and the pointers multiples of four floats);
// each column's sum is formed in the same order.
__global__ __launch_bounds__(256) void bwd_bias_colsum_vec_kernel(const float4* __restrict__ dy, int N, int KP4,
                                                                  float4* __restrict__ part) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  const int g = blockIdx.y, G = gridDim.y;
  if (j >= KP4) return;
  float4 a0 = make_float4(0.0f, 0.0f, 0.0f, 0.0f), a1 = a0;
  int n = g;
  for (; n + G < N; n += 2 * G) {
    const float4 u = dy[(size_t)n * KP4 + j], v = dy[(size_t)(n + G) * KP4 + j];
    a0.x += u.x; a0.y += u.y; a0.z += u.z; a0.w += u.w;
    a1.x += v.x; a1.y += v.y; a1.z += v.z; a1.w += v.w;
  }
  if (n < N) {
    const float4 u = dy[(size_t)n * KP4 + j];
    a0.x += u.x; a0.y += u.y; a0.z += u.z; a0.w += u.w;
  }
  part[(size_t)g * KP4 + j] = make_float4(a0.x + a1.x, a0.y + a1.y, a0.z + a1.z, a0.w + a1.w);
}

__global__ __launch_bounds__(256) void bwd_bias_planes_finish_kernel(const float* __restrict__ part, int G, int KP, int plane,
                                                                     float alpha, float beta, float* __restrict__ db) {
  const int k = blockIdx.x;
  float acc = 0.0f;
  for (int g = 0; g < G; ++g) {
    const float* p = part + (size_t)g * KP + (size_t)k * plane;
    for (int i = threadIdx.x; i < plane; i += 256) acc += p[i];
  }
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o, 64);
  __shared__ float sm[4];
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float v = alpha * ((sm[0] + sm[1]) + (sm[2] + sm[3]));
    if (beta != 0.0f) v += beta * db[k];
    db[k] = v;
  }
}

static int bwd_bias_col_groups(int N, long long KP) {
  long long G = cdiv<long long>(1 << 20, KP);
  if (G > 16) G = 16;
  if (G > N) G = N;
  return G < 1 ? 1 : (int)G;
}
constexpr int kBiasSmallPlane = 1024;  // below: column form; from here on: one wave per (n, k) row

// Column sums of an [N][K] matrix (dy of an affine layer, or the row sums above): a block covers 64 columns.
__global__ __launch_bounds__(256) void bwd_bias_rows_kernel(const float* __restrict__ dy, int N, int K, float alpha,
                                                            float beta, float* __restrict__ db) {
  bwd_bias_rows_block(dy, N, K, alpha, beta, db, blockIdx.x);
}

}  // namespace rh

using namespace rh;

// Scratch of the filter gradient proper, and behind it what rh_conv2d_bwd_filter_bias needs for the bias gradient: the
// per-image plane sums that the pass over dy leaves (N x K floats), or the scratch of the two-stage bias gradient.
static size_t bwd_filter_plan_bytes(const ConvDims& d) {
  const BwdFilterPlan p = plan_bwd_filter(d);
  const BwdFilterSoffPlan sp = plan_bwd_filter_soff(d);
  const size_t legacy = p.tab_bytes + p.part_bytes;
  return sp.ok && sp.total() > legacy ? sp.total() : legacy;
}
extern "C" size_t rh_conv2d_bwd_bias_workspace_bytes(int32_t N, int32_t K, int32_t plane);
static size_t bwd_filter_bias_bytes(const ConvDims& d) {
  const size_t part = align256(sizeof(float) * (size_t)d.N * d.K);
  const size_t two = rh_conv2d_bwd_bias_workspace_bytes(d.N, d.K, d.P * d.Q);
  return part > two ? part : two;
}
static int bwd_bias_two_stage(int N, int K, int plane, float alpha, const float* dy, float beta, float* db, float* rowsum,
                              hipStream_t stream);
static int bwd_bias_one_stage(int N, int K, int plane, float alpha, const float* dy, float beta, float* db,
                              hipStream_t stream);

extern "C" size_t rh_conv2d_workspace_bytes(const rh_conv_geom* g, int pass) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  const int CRS = d.C * d.R * d.S, KRS = d.K * d.R * d.S;
  switch (pass) {
    case RH_CONV_FWD: {
      const size_t legacy = align256(sizeof(int4) * (size_t)round_up(CRS, kTabPad));
      const SoffPlan sp = plan_soff_fwd(d);
      size_t need = sp.ok && sp.total() > legacy ? sp.total() : legacy;
      const Bf16FwdPlan bp = plan_bf16_fwd(d);  // the bf16 flag is not known here: room for either form
      if (bp.ok && bp.total() > need) need = bp.total();
      if (wino_shape(d) || wino_shape5(d)) {   // the flags are not known here: room for the Winograd form wherever the geometry has one
        const WinoGeom wg = wino_shape5(d) ? wino_geom_fwd5(d) : wino_geom_fwd(d);
        if (wg.ok && wg.total() > need) need = wg.total();
      }
      return need;
    }
    case RH_CONV_BWD_DATA: {
      const size_t legacy = align256(sizeof(int4) * (size_t)round_up(KRS, kTabPad)) +
                            align256(sizeof(int) * (size_t)round_up(KRS, kTabPad));
      const PhasePlan pp = plan_phase_bwd_data(d);
      if (pp.ok) return pp.total() > legacy ? pp.total() : legacy;
      const SoffPlan sp = plan_soff_bwd_data(d);
      size_t need = sp.ok && sp.total() > legacy ? sp.total() : legacy;
      if (wino_shape(d)) {
        const WinoGeom wg = wino_geom_bwd_data(d);
        if (wg.ok && wg.total() > need) need = wg.total();
      }
      return need;
    }
    case RH_CONV_BWD_FILTER: {
      size_t need = bwd_filter_plan_bytes(d);
      if (wino_shape(d)) {
        const WinoFilterPlan wp = plan_wino_bwd_filter(d);
        if (wp.ok && wp.total() > need) need = wp.total();
      }
      return need + bwd_filter_bias_bytes(d);
    }
    default:
      return 0;
  }
}

extern "C" size_t rh_conv2d_workspace_bytes_upto(const rh_conv_geom* g, int pass) {
  if (!g) return 0;
  rh_conv_geom h = *g;
  size_t need = 0;
  for (int n = g->N; n >= 1; --n) {
    h.N = n;
    const size_t b = rh_conv2d_workspace_bytes(&h, pass);
    if (b > need) need = b;
  }
  return need;
}

// The bias gradient beside the filter gradient (rh_conv2d_bwd_filter_bias).  part: where the pass over dy may leave the
// per-image plane sums (N x K floats) if it makes one in a form that can; folded says whether it did; done: the bias
// gradient was formed in the launch of the filter gradient's reduction, from those sums or, for a small layer, from dy.
struct BiasFold {
  float* db = nullptr;
  float* part = nullptr;
  bool folded = false, done = false;
};
// Up to this many elements of dy one launch (a block per channel) is as fast as the first of the two stages, and the
// small layers it covers are bound by the number of dependent launches.
constexpr long long kBiasOneStageElems = 1ll << 20;

static int bwd_filter_impl(const rh_conv_geom* g, float alpha, const float* x, const float* dy, float beta, float* dw,
                           void* ws, size_t ws_bytes, int flags, rh_stream_t stream_, BiasFold* bf) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  float* const bias_part = bf ? bf->part : nullptr;
  // the job a reduction launch takes along: the sums over the images of what the pass over dy left, or the whole bias
  // gradient of a small layer
  auto bias_job = [&](BiasJob* job) -> const BiasJob* {
    if (!bf || !bf->db || d.y_elems == 0) return nullptr;
    job->db = bf->db; job->N = d.N; job->K = d.K; job->alpha = alpha; job->beta = beta;
    if (bf->folded) { job->src = bf->part; job->plane = 1; }
    else if (d.y_elems <= kBiasOneStageElems) { job->src = dy; job->plane = d.P * d.Q; }
    else return nullptr;
    bf->done = true;
    return job;
  };
  if (!x || !dy || !dw) return RH_E_INVALID;
  if (flags & RH_MATH_BF16_MFMA_FP32ACC) return RH_E_UNSUPPORTED;
  const BwdFilterPlan plan = plan_bwd_filter(d);
  if (!ws || ws_bytes < rh_conv2d_workspace_bytes(g, RH_CONV_BWD_FILTER) || (reinterpret_cast<uintptr_t>(ws) & 255))
    return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  if ((flags & RH_ALGO_WINOGRAD) && (!wino_shape(d) || (flags & (RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT))))
    return RH_E_UNSUPPORTED;
  if (wino_shape(d) && !(flags & (RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT))) {
    const WinoFilterPlan wp = plan_wino_bwd_filter(d);
    if (flags & RH_ALGO_WINOGRAD ? wp.ok : wino_filter_pays(d, wp)) {
      if (d.w_elems == 0) return 0;
      return launch_conv_wino_bwd_filter(d, wp, x, dy, dw, alpha, beta, ws, stream);
    }
    if (flags & RH_ALGO_WINOGRAD) return RH_E_UNSUPPORTED;
  }
  const BwdFilterSoffPlan sp = plan_bwd_filter_soff(d);
  if (sp.ok && !(flags & RH_ALGO_GATHER) && ((flags & RH_ALGO_SCALAR_OFFSET) || use_soff_bwd_filter(d))) {
    const int CRSs = d.C * d.R * d.S, Ms = d.N * d.P * d.Q;
    char* base = static_cast<char*>(ws);
    int* soff = reinterpret_cast<int*>(base);
    float* dyT = reinterpret_cast<float*>(base + sp.tab_bytes);
    float* xT = reinterpret_cast<float*>(base + sp.tab_bytes + sp.dyt_bytes);
    float* parts = reinterpret_cast<float*>(base + sp.tab_bytes + sp.dyt_bytes + sp.xt_bytes);
    float* const bpart = (bias_part && nhwc_vec_ok(d.K, dyT)) ? bias_part : nullptr;
    NhwcCopyArgs a, b;
    a.src = dy; a.dst = dyT; a.C = d.K; a.H = d.P; a.W = d.Q; a.Hp = d.P; a.Wp = d.Q; a.halo = 0;
    a.elems = d.y_elems; b.elems = d.x_elems;
    a.vec = nhwc_vec_ok(d.K, dyT) ? 1 : 0;
    a.gx = bpart ? 1 : cdiv(d.P * d.Q, a.vec ? 64 : 32); a.gy = cdiv(d.K, a.vec ? 64 : 32);
    b.src = x; b.dst = xT; b.C = d.C; b.H = d.H; b.W = d.W; b.Hp = sp.Hp; b.Wp = sp.Wp; b.halo = d.pad;
    b.vec = nhwc_vec_ok(d.C, xT) ? 1 : 0;
    b.gx = cdiv(sp.Hp * sp.Wp, b.vec ? 64 : 32); b.gy = cdiv(d.C, b.vec ? 64 : 32);
    const long long nb_dy = (long long)a.gx * a.gy * d.N, nb_x = (long long)b.gx * b.gy * d.N;
    const long long nb_tab = cdiv(sp.n_k, 256);
    // Small layers: the two channel-last copies and the table share one launch (a launch gap less twice over on a
    // chain of kernels of a few microseconds).  Large layers keep three launches: as one, the copies of a ResNet-18
    // step's filter gradients, which run beside the data gradients of the other stream, made the step 3 % slower.
    if (nb_dy + nb_x <= 4096) {
      ProfScope prof("nchw_to_nhwc", 8.0 * ((double)d.N * d.K * d.P * d.Q) +
                                         4.0 * ((double)d.N * d.C * d.H * d.W + (double)d.N * d.C * sp.Hp * sp.Wp), stream);
      if (bpart)
        hipLaunchKernelGGL(bwd_filter_prep_kernel<true>, dim3((unsigned)(nb_dy + nb_x + nb_tab)), dim3(256), 0, stream, a, bpart,
                           (int)nb_dy, b, (int)nb_x, soff, sp.n_k, Ms, d.P * d.Q, d.Q, d.st, d.K);
      else
        hipLaunchKernelGGL(bwd_filter_prep_kernel<false>, dim3((unsigned)(nb_dy + nb_x + nb_tab)), dim3(256), 0, stream, a,
                           (float*)nullptr, (int)nb_dy, b, (int)nb_x, soff, sp.n_k, Ms, d.P * d.Q, d.Q, d.st, d.K);
      if (int e = launch_status()) return e;
    } else {
      hipLaunchKernelGGL(prep_bwd_filter_soff_kernel, dim3(cdiv(sp.n_k, 256)), dim3(256), 0, stream, soff, dyT, sp.n_k, Ms,
                         d.P * d.Q, d.Q, d.st, sp.Hp, sp.Wp, d.C, d.K);
      if (int e = launch_status()) return e;
      launch_nchw_to_nhwc(dy, dyT, d.N, d.K, d.P, d.Q, d.P, d.Q, 0, stream, bpart);
      if (int e = launch_status()) return e;
      launch_nchw_to_nhwc(x, xT, d.N, d.C, d.H, d.W, sp.Hp, sp.Wp, d.pad, stream);
      if (int e = launch_status()) return e;
    }
    if (bpart) bf->folded = true;
    RowSParams ap;  // dyT [pix][ko]
    ap.ptr = dyT; ap.bytes = (uint32_t)(sizeof(float) * (size_t)sp.n_k * d.K);
    ap.M = d.K; ap.inner = d.K; ap.innerW = d.K; ap.img_stride = 0; ap.a_stride = 0; ap.b_stride = 1;
    ap.soff = nullptr; ap.ldk4 = d.K * 4;
    RowSParams bp;  // xT [n][hp][wp][c]; rows j = (r, s, c)
    bp.ptr = xT; bp.bytes = (uint32_t)(sizeof(float) * (size_t)d.N * sp.Hp * sp.Wp * d.C);
    bp.M = CRSs; bp.inner = d.S * d.C; bp.innerW = d.S * d.C; bp.img_stride = sp.Wp * d.C; bp.a_stride = 0; bp.b_stride = 1;
    bp.soff = soff; bp.ldk4 = 0;
    EpiParams ep;
    ep.out = parts; ep.bias = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
    ep.rows = d.K; ep.cols = CRSs; ep.inner = 0; ep.ld = CRSs; ep.relu = 0;
    ep.split_stride = (long long)d.K * CRSs;
    int used = 1, e = 0;
    switch (sp.bm) {
      case 128: e = run_bwd_filter_soff<T128x128>(ap, bp, ep, sp.n_k, Ms, sp.splits, &used, stream, "conv_bwd_filter_128x128"); break;
      case 96:
        e = sp.bn == 128 ? run_bwd_filter_soff<T96x128>(ap, bp, ep, sp.n_k, Ms, sp.splits, &used, stream, "conv_bwd_filter_96x128")
                         : run_bwd_filter_soff<T96x256>(ap, bp, ep, sp.n_k, Ms, sp.splits, &used, stream, "conv_bwd_filter_96x256");
        break;
      case 64:  e = run_bwd_filter_soff<T64x256>(ap, bp, ep, sp.n_k, Ms, sp.splits, &used, stream, "conv_bwd_filter_64x256"); break;
      default:  e = run_bwd_filter_soff<T32x256>(ap, bp, ep, sp.n_k, Ms, sp.splits, &used, stream, "conv_bwd_filter_32x256"); break;
    }
    if (e) return e;
    const long long total = (long long)d.K * CRSs;
    BiasJob bj;
    bias_job(&bj);
    const unsigned jb = bj.blocks();
    ProfScope prof("split_reduce", 4.0 * (double)total * (used + 1) + (jb ? 4.0 * (double)bj.N * bj.K * bj.plane : 0.0), stream);
    if (d.C % 4 == 0 && (reinterpret_cast<uintptr_t>(parts) & 15) == 0) {
      bj.first = stream_grid((size_t)total / 4, 256);
      hipLaunchKernelGGL(split_reduce_rsc_vec_kernel, dim3(bj.first + jb), dim3(256), 0, stream,
                         reinterpret_cast<const float4*>(parts), used, (long long)d.K * CRSs / 4, dw, d.K, d.C, d.R, d.S, alpha,
                         beta, bj);
    } else {
      bj.first = stream_grid((size_t)total, 256);
      hipLaunchKernelGGL(split_reduce_rsc_kernel, dim3(bj.first + jb), dim3(256), 0, stream, parts, used,
                         (long long)d.K * CRSs, dw, d.K, d.C, d.R, d.S, alpha, beta, bj);
    }
    return launch_status();
  }

  const int CRS = d.C * d.R * d.S;
  const int M = d.N * d.P * d.Q;
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + plan.tab_bytes);
  PixDyParams ap;
  ap.ptr = dy; ap.bytes = (uint32_t)(d.y_elems * 4); ap.rows = d.K; ap.M = M; ap.set_pq(d.P * d.Q);
  if (d.R == 1 && d.S == 1 && d.st == 1 && d.pad == 0 && M > 0) {
    PixDyParams xp;
    xp.ptr = x; xp.bytes = (uint32_t)(d.x_elems * 4); xp.rows = d.C; xp.M = M; xp.set_pq(d.P * d.Q);
    EpiParams ep;
    ep.out = part; ep.bias = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
    ep.rows = d.K; ep.cols = CRS; ep.inner = 0; ep.ld = CRS; ep.relu = 0;
    ep.split_stride = (long long)d.K * CRS;
    int used = 1, e = 0;
    switch (plan.bm) {
      case 128: e = run_bwd_filter_1x1<T128x128>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_128x128"); break;
      case 96:
        e = CRS <= 96 ? run_bwd_filter_1x1<T96x96>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x96")
            : plan.bn == 128 ? run_bwd_filter_1x1<T96x128>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x128")
                             : run_bwd_filter_1x1<T96x256>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x256");
        break;
      case 64:  e = run_bwd_filter_1x1<T64x256>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_64x256"); break;
      default:  e = run_bwd_filter_1x1<T32x256>(ap, xp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_32x256"); break;
    }
    if (e) return e;
    BiasJob bj;
    launch_split_reduce(part, used, (long long)d.K * CRS, dw, d.K, CRS, CRS, alpha, beta, stream, nullptr, 0, bias_job(&bj));
    return launch_status();
  }

  PixXParams bp;
  bp.ptr = x; bp.bytes = (uint32_t)(d.x_elems * 4); bp.rows = CRS; bp.M = M; bp.set_pq(d.P * d.Q, d.Q);
  bp.img_stride = d.C * d.H * d.W; bp.H = d.H; bp.W = d.W; bp.st = d.st; bp.pad = d.pad; bp.set_filter(d.R, d.S);
  EpiParams ep;
  ep.out = part; ep.bias = nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
  ep.rows = d.K; ep.cols = CRS; ep.inner = 0; ep.ld = CRS; ep.relu = 0;
  ep.split_stride = (long long)d.K * CRS;

  int used = 1, e = 0;
  if (M == 0) {
    used = 0;
  } else {
    switch (plan.bm) {
      case 128: e = run_bwd_filter<T128x128>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_128x128"); break;
      case 96:
        e = plan.bn == 128 ? run_bwd_filter<T96x128>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x128")
                           : run_bwd_filter<T96x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_96x256");
        break;
      case 64:  e = run_bwd_filter<T64x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_64x256"); break;
      default:
        e = plan.bn == 64    ? run_bwd_filter<T32x64>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_32x64")
            : plan.bn == 128 ? run_bwd_filter<T32x128>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_32x128")
                             : run_bwd_filter<T32x256>(ap, bp, ep, M, plan.splits, &used, stream, "conv_bwd_filter_32x256");
        break;
    }
    if (e) return e;
  }
  BiasJob bj;
  launch_split_reduce(part, used, (long long)d.K * CRS, dw, d.K, CRS, CRS, alpha, beta, stream, nullptr, 0, bias_job(&bj));
  return launch_status();
}

extern "C" int rh_conv2d_bwd_filter(const rh_conv_geom* g, float alpha, const float* x, const float* dy,
                                    float beta, float* dw, void* ws, size_t ws_bytes, int flags,
                                    rh_stream_t stream_) {
  return bwd_filter_impl(g, alpha, x, dy, beta, dw, ws, ws_bytes, flags, stream_, nullptr);
}

extern "C" int rh_conv2d_bwd_filter_bias(const rh_conv_geom* g, float alpha, const float* x, const float* dy,
                                         float beta, float* dw, float* db, void* ws, size_t ws_bytes, int flags,
                                         rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!db) return RH_E_INVALID;
  if (!ws || ws_bytes < rh_conv2d_workspace_bytes(g, RH_CONV_BWD_FILTER) || (reinterpret_cast<uintptr_t>(ws) & 255))
    return RH_E_WORKSPACE;
  float* const bias_ws = reinterpret_cast<float*>(static_cast<char*>(ws) + bwd_filter_plan_bytes(d));
  BiasFold bf;
  bf.db = db; bf.part = bias_ws;
  if (int e = bwd_filter_impl(g, alpha, x, dy, beta, dw, ws, ws_bytes, flags, stream_, &bf)) return e;
  if (d.y_elems == 0 || bf.done) return 0;
  hipStream_t stream = to_stream(stream_);
  const int plane = d.P * d.Q;
  if (bf.folded) {   // the sums over the images of what the pass over dy left
    ProfScope prof("bwd_bias_finish", 4.0 * (double)d.N * d.K, stream);
    hipLaunchKernelGGL(bwd_bias_rows_kernel, dim3(cdiv(d.K, 64)), dim3(256), 0, stream, bias_ws, d.N, d.K, alpha, beta, db);
    return launch_status();
  }
  ProfScope prof("bwd_bias", 4.0 * (double)d.y_elems, stream);
  if (plane == 1 || rh_conv2d_bwd_bias_workspace_bytes(d.N, d.K, plane) == 0)
    return bwd_bias_one_stage(d.N, d.K, plane, alpha, dy, beta, db, stream);
  return bwd_bias_two_stage(d.N, d.K, plane, alpha, dy, beta, db, bias_ws, stream);
}

extern "C" size_t rh_conv2d_bwd_bias_workspace_bytes(int32_t N, int32_t K, int32_t plane) {
  if (N <= 0 || K <= 0 || plane <= 1) return 0;
  if ((long long)N * K * plane <= kBiasOneStageElems) return 0;
  if (plane < kBiasSmallPlane) return align256(sizeof(float) * (size_t)bwd_bias_col_groups(N, (long long)K * plane) * K * plane);
  return align256(sizeof(float) * (size_t)N * K);
}

extern "C" size_t rh_conv2d_bwd_bias_workspace_bytes_upto(int32_t N, int32_t K, int32_t plane) {
  size_t need = 0;
  for (int n = N; n >= 1; --n) {
    const size_t b = rh_conv2d_bwd_bias_workspace_bytes(n, K, plane);
    if (b > need) need = b;
  }
  return need;
}

// Both stages of the bias gradient with scratch `rowsum` of rh_conv2d_bwd_bias_workspace_bytes(N, K, plane) bytes.
// Every scratch element that the second stage reads is written by the first: nothing has to start at zero.
static int bwd_bias_two_stage(int N, int K, int plane, float alpha, const float* dy, float beta, float* db, float* rowsum,
                              hipStream_t stream) {
  const long long rows = (long long)N * K;
  if (plane < kBiasSmallPlane && (long long)K * plane < (1ll << 31)) {
    const int KP = K * plane, G = bwd_bias_col_groups(N, KP);
    if (KP % 4 == 0 && ((reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(rowsum)) & 15) == 0)
      hipLaunchKernelGGL(bwd_bias_colsum_vec_kernel, dim3(cdiv(KP / 4, 256), G), dim3(256), 0, stream,
                         reinterpret_cast<const float4*>(dy), N, KP / 4, reinterpret_cast<float4*>(rowsum));
    else
      hipLaunchKernelGGL(bwd_bias_colsum_kernel, dim3(cdiv(KP, 256), G), dim3(256), 0, stream, dy, N, KP, rowsum);
    if (int e = launch_status()) return e;
    hipLaunchKernelGGL(bwd_bias_planes_finish_kernel, dim3(K), dim3(256), 0, stream, rowsum, G, KP, plane, alpha, beta, db);
    return launch_status();
  }
  const long long blocks = cdiv<long long>(rows, 4);
  hipLaunchKernelGGL(bwd_bias_rowsum_kernel, dim3((unsigned)(blocks > 65536 ? 65536 : blocks)), dim3(256), 0, stream, dy,
                     rows, plane, rowsum);
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL(bwd_bias_rows_kernel, dim3(cdiv(K, 64)), dim3(256), 0, stream, rowsum, N, K, alpha, beta, db);
  return launch_status();
}

static int bwd_bias_one_stage(int N, int K, int plane, float alpha, const float* dy, float beta, float* db,
                              hipStream_t stream) {
  if (plane == 1) {
    hipLaunchKernelGGL(bwd_bias_rows_kernel, dim3(cdiv(K, 64)), dim3(256), 0, stream, dy, N, K, alpha, beta,
                       db);
  } else {
    hipLaunchKernelGGL(bwd_bias_kernel, dim3(K), dim3(1024), 0, stream, dy, N, K, plane, alpha, beta, db);
  }
  return launch_status();
}

extern "C" int rh_conv2d_bwd_bias_ws(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy, float beta,
                                     float* db, void* ws, size_t ws_bytes, void* stream_) {
  if (N <= 0 || K <= 0 || plane <= 0 || !dy || !db) return RH_E_INVALID;
  const size_t need = rh_conv2d_bwd_bias_workspace_bytes(N, K, plane);
  if (plane == 1 || need == 0 || !ws || ws_bytes < need) return rh_conv2d_bwd_bias(N, K, plane, alpha, dy, beta, db, stream_);
  hipStream_t stream = to_stream(stream_);
  ProfScope prof("bwd_bias", 4.0 * (double)N * K * plane, stream);
  return bwd_bias_two_stage(N, K, plane, alpha, dy, beta, db, static_cast<float*>(ws), stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------------
// The scratch of the two-stage bias gradient in a device array that is part of the library's code object: each GPU
// the library runs on holds its own 8 MiB copy from the first use of the library on it until the process ends.
// `scratch` names the array for the device compiler only; host code uses the per-device address that
// hipGetSymbolAddress returns.
constexpr size_t kStaticScratchBytes = size_t(8) << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];   // per device, set once under g_scratch_mutex
static std::mutex g_scratch_mutex;

namespace rh {
// Address of `scratch` on the current device; looked up once per device (from rh_ctx_create, or on the first call of
// rh_conv2d_bwd_bias_noalloc on a device whose context was made elsewhere).
int static_scratch_lookup(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return RH_E_LIMIT;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p || (reinterpret_cast<uintptr_t>(p) & 255)) return RH_E_INVALID;
    g_scratch_ptr[dev] = p;
  }
  if (out) *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace rh

extern "C" size_t rh_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int rh_conv2d_bwd_bias_noalloc(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy, float beta,
                                          float* db, rh_stream_t stream_) {
  if (N <= 0 || K <= 0 || plane <= 0 || !dy || !db) return RH_E_INVALID;
  hipStream_t stream = to_stream(stream_);
  const size_t need = rh_conv2d_bwd_bias_workspace_bytes(N, K, plane);
  if (plane == 1 || need == 0) return bwd_bias_one_stage(N, K, plane, alpha, dy, beta, db, stream);  // needs no scratch
  if (need > kStaticScratchBytes) return RH_E_LIMIT;
  void* ptr = nullptr;
  if (int e = static_scratch_lookup(&ptr)) return e;
  return bwd_bias_two_stage(N, K, plane, alpha, dy, beta, db, static_cast<float*>(ptr), stream);
}

extern "C" int rh_conv2d_bwd_bias(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy,
                                  float beta, float* db, rh_stream_t stream_) {
  if (N <= 0 || K <= 0 || plane <= 0 || !dy || !db) return RH_E_INVALID;
  hipStream_t stream = to_stream(stream_);
  ProfScope prof("bwd_bias", 4.0 * (double)N * K * plane, stream);
  return bwd_bias_one_stage(N, K, plane, alpha, dy, beta, db, stream);
}
