// Convolution forward (K1) with optional fused bias (K2) and ReLU (K3) as an implicit GEMM:
//   y[n][ko][p][q] = sum_{c,r,s} w[ko][(c,r,s)] * x_gather[(c,r,s)][(n,p,q)]
// rows = output channels (weights, k contiguous), cols = output pixels (gathered, q contiguous).
#include "conv_common.h"

namespace rh {

__global__ void build_fwd_tab_kernel(int4* tab, int n_entries, int CRS, int R, int S, int HW, int W) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= n_entries) return;
  if (k < CRS) {
    const int c = k / (R * S), rs = k - c * (R * S), r = rs / S, s = rs - r * S;
    tab[k] = make_int4(c * HW + r * W + s, r, s, 0);
  } else {
    tab[k] = make_int4(0, -(1 << 28), 0, -1);
  }
}

void launch_build_fwd_tab(int4* tab, int n_entries, int CRS, int R, int S, int HW, int W,
                          hipStream_t stream) {
  hipLaunchKernelGGL(build_fwd_tab_kernel, dim3(cdiv(n_entries, 256)), dim3(256), 0, stream, tab,
                     n_entries, CRS, R, S, HW, W);
}

// dst (planes x Hp x Wp) = src (planes x H x W) surrounded by `halo` zeros.  A thread produces four consecutive
// elements of dst (they may straddle a row or a plane) and writes them as one 16-byte store when dst is aligned:
// stores of 16 bytes per lane over one sweep of consecutive blocks are what this GPU's memory system wants.
__device__ __forceinline__ void pad_image_body(unsigned block, const float* __restrict__ src, float* __restrict__ dst,
                                               unsigned total, int H, int W, FastDiv dHp, FastDiv dWp, int halo, int vec,
                                               unsigned src_total) {
  const unsigned g = block * blockDim.x + threadIdx.x;
  const unsigned i0 = g * 4u;
  if (i0 >= total) return;
  uint32_t t, wp, plane, hp;
  dWp.divmod(i0, t, wp);
  dHp.divmod(t, plane, hp);
  // Source offsets of the four, -1 = zero.  src is dense and the map from dst to src keeps the order of the elements,
  // so the source elements of four consecutive dst elements are one run of consecutive addresses, however the four
  // lie across row ends, plane ends and the halo: one 16-byte load from the run's start (4-byte aligned: it starts
  // anywhere) brings them all, and each element picks its value by its distance from that start.
  int o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int he = (int)hp - halo, we = (int)wp - halo;
    o[e] = ((unsigned)he < (unsigned)H && (unsigned)we < (unsigned)W && i0 + e < total)
               ? (int)((plane * (unsigned)H + (unsigned)he) * (unsigned)W + (unsigned)we) : -1;
    if (++wp == dWp.div) {
      wp = 0;
      if (++hp == dHp.div) { hp = 0; ++plane; }
    }
  }
  int first = o[3];
  if (o[2] >= 0) first = o[2];
  if (o[1] >= 0) first = o[1];
  if (o[0] >= 0) first = o[0];
  float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (first >= 0) {
    if ((unsigned)first + 3u < src_total) {
      typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
      const f4u q = *reinterpret_cast<const f4u*>(src + first);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int d = o[e] - first;
        const float t = d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
        v[e] = o[e] >= 0 ? t : 0.0f;
      }
    } else {   // the tensor's last three elements
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (o[e] >= 0) v[e] = src[o[e]];
    }
  }
  if (vec && i0 + 3 < total) {
    *reinterpret_cast<float4*>(dst + i0) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i0 + e < total) dst[i0 + e] = v[e];
  }
}

__global__ __launch_bounds__(256) void pad_image_kernel(const float* __restrict__ src, float* __restrict__ dst, unsigned total,
                                                        int H, int W, FastDiv dHp, FastDiv dWp, int halo, int vec,
                                                        unsigned src_total) {
  pad_image_body(blockIdx.x, src, dst, total, H, W, dHp, dWp, halo, vec, src_total);
}

// The filter-side scratch of the scalar-offset forward and stride-1 backward-data paths, as a function of a virtual
// grid (first element, stride) so that it can share a launch with the image copy:
//   forward:       wT[k][ko] = w[ko][k] for k = (c,r,s)  (zero rows for k >= CRS), soff[k] = 4*(c*HpWp + r*Wp + s);
//   backward-data: wT[k][c] = w[ko][c][r][s] for k = (ko,r,s), soff[k] = 4*(ko*HpWp + (R-1-r)*Wp + (S-1-s));
// soff is 0 past the end of the contraction.
struct PrepSoffArgs {
  const float* w; float* wT; int* soff;
  int n_k, k_true, rows, R, S, HpWp, Wp, bwd;
};

__device__ __forceinline__ void prep_soff_body(const PrepSoffArgs& a, long long first, long long stride) {
  const long long total = (long long)a.n_k * a.rows;
  const int RS = a.R * a.S;
  for (long long i = first; i < total; i += stride) {
    const int k = (int)(i / a.rows), row = (int)(i - (long long)k * a.rows);
    float v = 0.0f;
    int off = 0;
    if (k < a.k_true) {
      const int c = k / RS, rs = k - c * RS, r = rs / a.S, s2 = rs - r * a.S;
      if (a.bwd) {
        v = a.w[((size_t)c * a.rows + row) * RS + rs];
        off = (c * a.HpWp + (a.R - 1 - r) * a.Wp + (a.S - 1 - s2)) * 4;
      } else {
        v = a.w[(size_t)row * a.k_true + k];
        off = (c * a.HpWp + r * a.Wp + s2) * 4;
      }
    }
    a.wT[i] = v;
    if (row == 0) a.soff[k] = off;
  }
}

__global__ __launch_bounds__(256) void prep_soff_kernel(PrepSoffArgs a) {
  prep_soff_body(a, (long long)blockIdx.x * blockDim.x + threadIdx.x, (long long)gridDim.x * blockDim.x);
}

// Both in one launch: the first pad_blocks blocks copy the image, the others prepare the filter side.  The two are
// independent, and a launch less in front of a contraction is a launch gap less on the chain of a small layer.
__global__ __launch_bounds__(256) void pad_image_prep_soff_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                  unsigned total, int H, int W, FastDiv dHp, FastDiv dWp,
                                                                  int halo, int vec, unsigned pad_blocks, PrepSoffArgs a,
                                                                  unsigned src_total) {
  if (blockIdx.x < pad_blocks) {
    pad_image_body(blockIdx.x, src, dst, total, H, W, dHp, dWp, halo, vec, src_total);
  } else {
    const unsigned b = blockIdx.x - pad_blocks, nb = gridDim.x - pad_blocks;
    prep_soff_body(a, (long long)b * blockDim.x + threadIdx.x, (long long)nb * blockDim.x);
  }
}

// The same with the source dilated: src[h][w] lands on [halo + dil*h][halo + dil*w].
__global__ void pad_dilate_image_kernel(const float* __restrict__ src, float* __restrict__ dst, unsigned total, int H, int W,
                                        FastDiv dHp, FastDiv dWp, int halo, FastDiv dDil) {
  const unsigned stride = gridDim.x * blockDim.x;
  for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    uint32_t t, wp, plane, hp;
    dWp.divmod(i, t, wp);
    dHp.divmod(t, plane, hp);
    const int hd = (int)hp - halo, wd = (int)wp - halo;
    float v = 0.0f;
    if (hd >= 0 && wd >= 0) {
      uint32_t h, hr, w, wr;
      dDil.divmod((uint32_t)hd, h, hr);
      dDil.divmod((uint32_t)wd, w, wr);
      if (hr == 0 && wr == 0 && h < (uint32_t)H && w < (uint32_t)W) v = src[((size_t)plane * H + h) * W + w];
    }
    dst[i] = v;
  }
}

// total elements of dst must be below 2^31 (a tensor is at most 2 GiB here)
void launch_pad_image(const float* src, float* dst, long long planes, int H, int W, int Hp, int Wp, int halo,
                      hipStream_t stream, int dil) {
  const long long total = planes * Hp * Wp;
  ProfScope prof("pad_image", 4.0 * ((double)planes * H * W + (double)total), stream);
  if (dil > 1) {
    hipLaunchKernelGGL(pad_dilate_image_kernel, dim3(stream_grid((size_t)total, 256)), dim3(256), 0, stream, src, dst,
                       (unsigned)total, H, W, FastDiv((uint32_t)Hp), FastDiv((uint32_t)Wp), halo, FastDiv((uint32_t)dil));
    return;
  }
  const int vec = (reinterpret_cast<uintptr_t>(dst) & 15) == 0 ? 1 : 0;
  hipLaunchKernelGGL(pad_image_kernel, dim3(stream_grid((size_t)(total + 3) / 4, 256)), dim3(256), 0, stream, src, dst,
                     (unsigned)total, H, W, FastDiv((uint32_t)Hp), FastDiv((uint32_t)Wp), halo, vec, (unsigned)(planes * H * W));
}

static PrepSoffArgs prep_args(const float* w, float* wT, int* soff, int n_k, int k_true, int rows, int R, int S, int HpWp,
                              int Wp, int bwd) {
  PrepSoffArgs a;
  a.w = w; a.wT = wT; a.soff = soff; a.n_k = n_k; a.k_true = k_true; a.rows = rows; a.R = R; a.S = S; a.HpWp = HpWp; a.Wp = Wp;
  a.bwd = bwd;
  return a;
}

void launch_prep_soff(const float* w, float* wT, int* soff, int n_k, int k_true, int rows, int R, int S, int HpWp, int Wp,
                      int bwd, hipStream_t stream) {
  const PrepSoffArgs a = prep_args(w, wT, soff, n_k, k_true, rows, R, S, HpWp, Wp, bwd);
  hipLaunchKernelGGL(prep_soff_kernel, dim3(stream_grid((size_t)n_k * rows, 256)), dim3(256), 0, stream, a);
}

void launch_pad_image_prep_soff(const float* src, float* dst, long long planes, int H, int W, int Hp, int Wp, int halo,
                                const float* w, float* wT, int* soff, int n_k, int k_true, int rows, int R, int S, int bwd,
                                hipStream_t stream) {
  const long long total = planes * Hp * Wp;
  const PrepSoffArgs a = prep_args(w, wT, soff, n_k, k_true, rows, R, S, Hp * Wp, Wp, bwd);
  ProfScope prof("pad_image", 4.0 * ((double)planes * H * W + (double)total) + 4.0 * 2.0 * (double)n_k * rows, stream);
  const int vec = (reinterpret_cast<uintptr_t>(dst) & 15) == 0 ? 1 : 0;
  const unsigned pad_blocks = (unsigned)stream_grid((size_t)(total + 3) / 4, 256);
  const unsigned prep_blocks = (unsigned)stream_grid((size_t)n_k * rows, 256);
  hipLaunchKernelGGL(pad_image_prep_soff_kernel, dim3(pad_blocks + prep_blocks), dim3(256), 0, stream, src, dst, (unsigned)total,
                     H, W, FastDiv((uint32_t)Hp), FastDiv((uint32_t)Wp), halo, vec, pad_blocks, a, (unsigned)(planes * H * W));
}

// VEC: four consecutive elements per thread through 16-byte loads and stores (slab stride, first element and all
// pointers multiples of four floats); otherwise one element per thread.
template <bool VEC>
__global__ __launch_bounds__(256) void split_reduce_nchw_kernel(const float* __restrict__ part, int splits, long long stride,
                                                                float* __restrict__ out, unsigned first, unsigned total,
                                                                FastDiv inner, FastDiv rows, float alpha, float beta,
                                                                const float* __restrict__ bias, int relu,
                                                                unsigned col0, const float* __restrict__ mask) {
  constexpr int E = VEC ? 4 : 1;
  const unsigned i0 = first + (blockIdx.x * blockDim.x + threadIdx.x) * (unsigned)E;
  if (i0 >= total) return;
  float acc[E], a1[E];
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = a1[e] = 0.0f;
  auto add = [&](float (&dst)[E], int s) {
    const float* p = part + (long long)s * stride + (i0 - first);  // a slab starts at the result's element `first`
    if (VEC) {
      const float4 v = *reinterpret_cast<const float4*>(p);
      dst[0] += v.x; dst[E > 1 ? 1 : 0] += v.y; dst[E > 2 ? 2 : 0] += v.z; dst[E > 3 ? 3 : 0] += v.w;
    } else {
      dst[0] += p[0];
    }
  };
  int s = 0;
  for (; s + 1 < splits; s += 2) {
    add(acc, s);
    add(a1, s + 1);
  }
  if (s < splits) add(acc, s);
  float old[E];
#pragma unroll
  for (int e = 0; e < E; ++e) old[e] = 0.0f;
  if (beta != 0.0f) {
    if (VEC) {
      const float4 o = *reinterpret_cast<const float4*>(out + i0);
      old[0] = o.x; old[E > 1 ? 1 : 0] = o.y; old[E > 2 ? 2 : 0] = o.z; old[E > 3 ? 3 : 0] = o.w;
    } else {
      old[0] = out[i0];
    }
  }
  float res[E];
  bool keep[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const unsigned i = i0 + e;
    const uint32_t plane = inner.quot(i);
    const uint32_t img = rows.quot(plane);
    keep[e] = col0 == 0 || img * inner.div + (i - plane * inner.div) >= col0;  // column = image * inner + pixel
    float v = alpha * (acc[e] + a1[e]);
    if (beta != 0.0f) v = fmaf(beta, old[e], v);
    if (bias) v += bias[plane - img * rows.div];
    if (relu) v = v > 0.0f ? v : 0.0f;
    if (mask && !(mask[i < total ? i : i0] > 0.0f)) v = 0.0f;
    res[e] = v;
  }
  if (VEC) {
    if (keep[0] && keep[E - 1]) {
      *reinterpret_cast<float4*>(out + i0) = make_float4(res[0], res[E > 1 ? 1 : 0], res[E > 2 ? 2 : 0], res[E > 3 ? 3 : 0]);
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e)
    if (keep[e]) out[i0 + e] = res[e];
}

void launch_split_reduce_nchw(const float* part, int splits, long long stride, float* out, long long total, int inner,
                              int rows, float alpha, float beta, const float* bias, int relu, hipStream_t stream,
                              long long col0, const float* mask) {
  // elements before the image that holds column col0 are not part of the reduction
  const long long first = col0 > 0 ? (col0 / inner) * (long long)rows * inner : 0;
  ProfScope prof("split_reduce", 4.0 * (double)(total - first) * (splits + 1), stream);
  const bool vec = stride % 4 == 0 && first % 4 == 0 && total % 4 == 0 &&
                   ((reinterpret_cast<uintptr_t>(part) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  if (vec)
    hipLaunchKernelGGL((split_reduce_nchw_kernel<true>), dim3(stream_grid((size_t)(total - first) / 4, 256)), dim3(256), 0, stream,
                       part, splits, stride, out, (unsigned)first, (unsigned)total, FastDiv((uint32_t)inner),
                       FastDiv((uint32_t)rows), alpha, beta, bias, relu, (unsigned)col0, mask);
  else
    hipLaunchKernelGGL((split_reduce_nchw_kernel<false>), dim3(stream_grid((size_t)(total - first), 256)), dim3(256), 0, stream,
                       part, splits, stride, out, (unsigned)first, (unsigned)total, FastDiv((uint32_t)inner),
                       FastDiv((uint32_t)rows), alpha, beta, bias, relu, (unsigned)col0, mask);
}

// `splits` > 1: slices of the contraction write unblended partial results to `part`, then one reduction applies the
// alpha / beta blend, bias and ReLU.
template <class T>
static int run_fwd_soff(const RowSParams& ap, const RowSParams& bp, EpiParams ep, int n_k, int k_true,
                        hipStream_t stream, const char* tag, int splits = 1, float* part = nullptr,
                        const TailSplit* tail = nullptr) {
  constexpr int AROWS = T::BM % 64 == 0 ? T::BM : (T::BM + 63) / 64 * 64;  // loader rows: a multiple of the wave
  // The transposed filter is read four rows per lane where the tile's shape allows (forward kernel 1-5 % faster alone).
  // The backward passes keep the one-row loader: there the same change made the two-stream step 0.2 ms slower,
  // although each kernel alone was as fast or faster.
  constexpr bool A4 = T::BK % (T::NT / (AROWS / 4)) == 0;
  typedef typename std::conditional<A4, LoadRow4<AROWS, T::BK, T::NT>, LoadRowS<AROWS, T::BK, T::NT, true>>::type AL;
  typedef LoadRowS<T::BN, T::BK, T::NT, false> BL;
  const long long total = (long long)ep.rows * ep.cols;
  if (splits <= 1 && tail && tail->splits > 1) {
    // whole tiles blend into y as usual; the sliced tail goes through `part` and one reduction over its columns
    const EpiParams fin = ep;
    const long long first = tail_first_elem(*tail, ep.inner, ep.rows);
    ep.part = part; ep.part_first = first; ep.split_stride = total - first;
    ep.full_tiles = tail->full_tiles; ep.tail_tiles = tail->tail_tiles; ep.tail_splits = tail->splits;
    if (int e = launch_mfma_gemm<T, AL, BL, true, PassConvFwd>(ap, bp, ep, n_k, 1, nullptr, stream, tag, k_true)) return e;
    launch_split_reduce_nchw(part, tail->splits, total - first, fin.out, total, fin.inner, fin.rows, fin.alpha, fin.beta,
                             fin.bias, fin.relu, stream, tail->col0);
    return launch_status();
  }
  // one pass over the whole contraction: K steps that hold nothing but the table's zero padding are left out
  if (splits <= 1)
    return launch_mfma_gemm<T, AL, BL, true, PassConvFwd>(ap, bp, ep, min(n_k, round_up(k_true, T::BK)), 1, nullptr, stream, tag,
                                                         k_true);
  const EpiParams fin = ep;
  ep.out = part; ep.split_stride = total;
  int used = 1;
  if (int e = launch_mfma_gemm<T, AL, BL, true, PassConvFwd>(ap, bp, ep, n_k, splits, &used, stream, tag, k_true)) return e;
  launch_split_reduce_nchw(part, used, total, fin.out, total, fin.inner, fin.rows, fin.alpha, fin.beta, fin.bias, fin.relu,
                           stream);
  return launch_status();
}

// bf16-operand forward (128x128 tile only: the loader rows must equal the tile rows).
static int run_fwd_soff_bf16(const RowSParams& ap, const RowSParams& bp, const EpiParams& ep, int n_k, int k_true,
                             hipStream_t stream) {
  typedef T128x128bf T;
  typedef LoadRowS<T::BM, T::BK, T::NT, true> AL;
  typedef LoadRowS<T::BN, T::BK, T::NT, false> BL;
  return launch_mfma_gemm_bf16<T, AL, BL, true, PassConvFwd>(ap, bp, ep, n_k, 1, nullptr, stream, "conv_fwd_bf16_128x128",
                                                             k_true);
}

// ------------------------------------------------------------------------------------------
// Packed bf16 operands.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ uint4 pack8_bf16(const float (&v)[8]) {
  uint4 q;
  q.x = pack_bf16(v[0], v[1]);
  q.y = pack_bf16(v[2], v[3]);
  q.z = pack_bf16(v[4], v[5]);
  q.w = pack_bf16(v[6], v[7]);
  return q;
}

// Both operand copies keep the eight k of a group together and put the GEMM row next: consecutive lanes (rows) of a
// 16-byte load then read consecutive 16-byte pieces, i.e. whole cache lines per instruction.  (With the rows strided by
// a pixel's or a filter's full channel vector every lane touches a cache line of its own: the GEMM then ran at 0.55
// instead of 0.86 PFLOP/s on 256 x 96 x 27 x 27 -> 256, 5x5.)
//
// wb[g][ko][8] (bf16) = w[ko][c][r][s] for k' = 8g + e = (r*S + s)*C + c, zero for k' >= C*R*S; one thread per (g, ko).
// The threads of ko == 0 also write the table: soff8[g] = byte offset of (r, s, c/8) in the image copy (0 past the end:
// the filter is zero there).
__global__ __launch_bounds__(256) void prep_bf16_filter_kernel(const float* __restrict__ w, uint4* __restrict__ wb,
                                                               int* __restrict__ soff8, int n_k, int CRS, int K, int C,
                                                               int RS, int S, int Wp) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)(n_k / 8) * K) return;
  const int g = (int)(i / K), ko = (int)(i - (long long)g * K);
  const int k0 = g * 8;
  float v[8];
  const int rs = k0 / C, c0 = k0 - rs * C;  // C % 8 == 0: the eight k' share (r, s)
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = k0 < CRS ? w[(size_t)ko * CRS + (size_t)(c0 + e) * RS + rs] : 0.0f;
  wb[i] = pack8_bf16(v);
  if (ko == 0) {
    const int r = rs / S, s2 = rs - r * S;
    soff8[g] = k0 < CRS ? ((r * (C / 8) + c0 / 8) * Wp + s2) * 16 : 0;
  }
}

// xb[n][hp][c/8][wp][8] (bf16) = x[n][c][hp - halo][wp - halo], zero outside; one thread per 16-byte group: eight
// reads (one per channel, consecutive lanes along w) and one store.
__global__ __launch_bounds__(256) void nchw_to_bf16_groups_kernel(const float* __restrict__ x, uint4* __restrict__ xb,
                                                                 unsigned total, int H, int W, FastDiv dWp, FastDiv dCg,
                                                                 FastDiv dHp, int halo) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  uint32_t t, wp, cg, hp, n;
  dWp.divmod(i, t, wp);
  dCg.divmod(t, t, cg);
  dHp.divmod(t, n, hp);
  const int h = (int)hp - halo, wc = (int)wp - halo;
  float v[8];
  if ((unsigned)h < (unsigned)H && (unsigned)wc < (unsigned)W) {
    const size_t plane = (size_t)H * W;
    const float* src = x + ((size_t)n * dCg.div * 8 + cg * 8) * plane + (size_t)h * W + wc;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = src[e * plane];
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.0f;
  }
  xb[i] = pack8_bf16(v);
}

// The inverse: x[n][c][h][w] (fp32) = xb[n][h + halo][c/8][w + halo][c%8]; one thread per 16-byte group of the interior.
__global__ __launch_bounds__(256) void bf16_groups_to_nchw_kernel(const uint4* __restrict__ xb, float* __restrict__ x,
                                                                 unsigned total, int H, int W, FastDiv dW, FastDiv dCg,
                                                                 FastDiv dH, int halo) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  uint32_t t, wc, cg, h, n;
  dW.divmod(i, t, wc);
  dCg.divmod(t, t, cg);
  dH.divmod(t, n, h);
  const int Hp = H + 2 * halo, Wp = W + 2 * halo;
  const uint4 q = xb[(((size_t)n * Hp + h + halo) * dCg.div + cg) * Wp + wc + halo];
  const uint32_t d[4] = {q.x, q.y, q.z, q.w};
  const size_t plane = (size_t)H * W;
  float* dst = x + ((size_t)n * dCg.div * 8 + cg * 8) * plane + (size_t)h * W + wc;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    dst[(2 * e) * plane] = __builtin_bit_cast(float, d[e] << 16);
    dst[(2 * e + 1) * plane] = __builtin_bit_cast(float, d[e] & 0xffff0000u);
  }
}

// The same two copies for groups of eight filter columns (Bf16FwdPlan::s_groups > 0).
// wb[g][ko][8] = w[ko][c][r][8 sg + e] (zero for columns past S and groups past the end), g = (c*R + r)*Sg + sg;
// soff8[g] = byte offset of (c, r, 8 sg) in one image of the copy.
__global__ __launch_bounds__(256) void prep_bf16_filter_cols_kernel(const float* __restrict__ w, uint4* __restrict__ wb,
                                                                    int* __restrict__ soff8, int n_k, int groups, int K,
                                                                    int CRS, int R, int S, int Sg, int Hp, int Wp) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)(n_k / 8) * K) return;
  const int g = (int)(i / K), ko = (int)(i - (long long)g * K);
  const int cr = g / Sg, sg = g - cr * Sg;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int s2 = 8 * sg + e;
    v[e] = (g < groups && s2 < S) ? w[(size_t)ko * CRS + (size_t)cr * S + s2] : 0.0f;
  }
  wb[i] = pack8_bf16(v);
  if (ko == 0) {
    const int c = cr / R, r = cr - c * R;
    soff8[g] = g < groups ? ((c * Hp + r) * Wp + 8 * sg) * 2 : 0;
  }
}

// xb[n][c][hp][wp] (bf16) = x[n][c][hp - halo][wp - halo], zero outside; one thread per two elements (Wp is even).
__global__ __launch_bounds__(256) void nchw_to_bf16_planes_kernel(const float* __restrict__ x, uint32_t* __restrict__ xb,
                                                                 unsigned total, int H, int W, FastDiv dWp2, FastDiv dHp,
                                                                 int halo) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  uint32_t t, w2, plane, hp;
  dWp2.divmod(i, t, w2);
  dHp.divmod(t, plane, hp);
  const int h = (int)hp - halo, w0 = 2 * (int)w2 - halo;
  float lo = 0.0f, hi = 0.0f;
  if ((unsigned)h < (unsigned)H) {
    const float* row = x + ((size_t)plane * H + h) * W;
    if ((unsigned)w0 < (unsigned)W) lo = row[w0];
    if ((unsigned)(w0 + 1) < (unsigned)W) hi = row[w0 + 1];
  }
  xb[i] = pack_bf16(lo, hi);
}

// The three stages of a packed bf16 forward.  The filter stage's result (table + filter copy, tab_bytes + wt_bytes at
// `wprep`) depends on the weights and the geometry only, so a caller whose weights do not change between calls keeps it.
static int bf16_prep_filter(const ConvDims& d, const Bf16FwdPlan& bpn, const float* w, void* wprep, hipStream_t stream) {
  char* base = static_cast<char*>(wprep);
  int* soff8 = reinterpret_cast<int*>(base);
  uint4* wb = reinterpret_cast<uint4*>(base + bpn.tab_bytes);
  const int CRS = d.C * d.R * d.S;
  ProfScope prof("bf16_filter", 4.0 * (double)d.w_elems + 2.0 * (double)bpn.n_k * d.K, stream);
  const dim3 grid((unsigned)cdiv((long long)(bpn.n_k / 8) * d.K, 256ll));
  if (bpn.s_groups > 0)
    hipLaunchKernelGGL(prep_bf16_filter_cols_kernel, grid, dim3(256), 0, stream, w, wb, soff8, bpn.n_k,
                       d.C * d.R * bpn.s_groups, d.K, CRS, d.R, d.S, bpn.s_groups, bpn.Hp, bpn.Wp);
  else
    hipLaunchKernelGGL(prep_bf16_filter_kernel, grid, dim3(256), 0, stream, w, wb, soff8, bpn.n_k, CRS, d.K, d.C,
                       d.R * d.S, d.S, bpn.Wp);
  return launch_status();
}

// fp32 NCHW image -> the bf16 copy the plan's loaders read (img_bytes at `xb`), zero border included.
static int bf16_pack_input(const ConvDims& d, const Bf16FwdPlan& bpn, const float* x, void* xb, hipStream_t stream) {
  const int HpWp = bpn.Hp * bpn.Wp, Cg = d.C / 8;
  if (bpn.s_groups > 0) {
    const size_t pairs = (size_t)d.N * d.C * HpWp / 2;  // below 2^30: the copy is at most 2 GiB
    ProfScope prof("nchw_to_bf16_planes", 4.0 * (double)d.x_elems + 4.0 * (double)pairs, stream);
    hipLaunchKernelGGL(nchw_to_bf16_planes_kernel, dim3(stream_grid(pairs, 256)), dim3(256), 0, stream, x,
                       reinterpret_cast<uint32_t*>(xb), (unsigned)pairs, d.H, d.W, FastDiv((uint32_t)(bpn.Wp / 2)),
                       FastDiv((uint32_t)bpn.Hp), d.pad);
  } else {
    const size_t groups = (size_t)d.N * Cg * HpWp;  // below 2^28: the copy is at most 2 GiB
    ProfScope prof("nchw_to_bf16_groups", 4.0 * (double)d.x_elems + 16.0 * (double)groups, stream);
    hipLaunchKernelGGL(nchw_to_bf16_groups_kernel, dim3(stream_grid(groups, 256)), dim3(256), 0, stream, x,
                       reinterpret_cast<uint4*>(xb), (unsigned)groups, d.H, d.W, FastDiv((uint32_t)bpn.Wp),
                       FastDiv((uint32_t)Cg), FastDiv((uint32_t)bpn.Hp), d.pad);
  }
  return launch_status();
}

// The contraction on prepared operands: `xb` the image copy, `wprep` the filter stage's result.  The result goes to
// ep.out as fp32 NCHW, or, with pk.ptr set, as packed bf16 for the next convolution (ep.out unused).  Which kernel
// runs depends on the geometry only, so both forms of the result come from the same accumulators.
template <class T, bool DMA, bool PK, int R = 4>
static int bf16_gemm_on(const ConvDims& d, const Bf16FwdPlan& bpn, const void* xb, const void* wprep, const EpiParams& ep,
                        const PackedOut& pk, hipStream_t stream, const char* tag) {
  const char* base = static_cast<const char*>(wprep);
  const int* soff8 = reinterpret_cast<const int*>(base);
  const void* wb = base + bpn.tab_bytes;
  const int CRS = d.C * d.R * d.S, HpWp = bpn.Hp * bpn.Wp, Cg = d.C / 8;
  const bool cols = bpn.s_groups > 0;
  RowV8Params ap;  // filter: row ko of group g at (g*K + ko)*16
  ap.ptr = wb; ap.bytes = (uint32_t)(2 * (size_t)bpn.n_k * d.K);
  ap.M = d.K; ap.inner = 1; ap.innerW = 1; ap.img_stride = 16; ap.a_stride = 0; ap.b_stride = 0; ap.soff = nullptr;
  ap.group_stride = d.K * 16;
  RowV8Params bp;  // image copy, rows = output pixels (n, p, q)
  bp.ptr = xb; bp.bytes = (uint32_t)(2 * (size_t)d.N * d.C * HpWp);
  bp.M = d.N * d.P * d.Q; bp.inner = d.P * d.Q; bp.innerW = d.Q;
  bp.img_stride = HpWp * d.C * 2;
  if (cols) {
    bp.a_stride = d.st * bpn.Wp * 2; bp.b_stride = d.st * 2;
  } else {
    bp.a_stride = d.st * Cg * bpn.Wp * 16; bp.b_stride = d.st * 16;
  }
  bp.soff = soff8;
  bp.group_stride = 0;
  typedef LoadRowV8<T::BM, T::BK, T::NT, true> AL;
  typedef LoadRowV8<T::BN, T::BK, T::NT, false> BL;
  if constexpr (DMA)
    return launch_mfma_gemm_bf16_dma<T, true, false, true, PassConvFwd, PK, R>(ap, bp, ep, bpn.n_k, stream, tag, CRS, pk);
  else
    return launch_mfma_gemm_bf16<T, AL, BL, true, PassConvFwd, PK>(ap, bp, ep, bpn.n_k, 1, nullptr, stream, tag, CRS, pk);
}

static int bf16_gemm(const ConvDims& d, const Bf16FwdPlan& bpn, const void* xb, const void* wprep, const EpiParams& ep,
                     const PackedOut& pk, hipStream_t stream, bool force_stream = false) {
  // 1x1 layers of up to 128 channels between packed activations are copies with a contraction riding along: the
  // streaming kernel (same accumulation order, hence the same bits as the tiles)
  if (pk.ptr && bpn.s_groups == 0 && (conv1x1_bf16_stream_applies(d) || (force_stream && conv1x1_bf16_stream_runs(d))))
    return launch_conv1x1_bf16_stream(d, xb, static_cast<const char*>(wprep) + bpn.tab_bytes, ep.bias, ep.relu, pk, stream);
  // Filter counts that waste no more rows in 256-row tiles than in 128-row ones take a direct-to-LDS kernel:
  //  - 256 x 256 (one block of eight waves per CU, ring of four) for long contractions on grids of two rounds of
  //    the 256 CUs and more: 1.19 PFLOP/s on 256 x 96 x 27 x 27 -> 256, 5x5 (729 tiles);
  //  - 256 x 128 (two blocks of four waves per CU, ring of three) otherwise, from contractions of 256 and grids
  //    of one round on: a block's first loads and its stores hide behind the other block, and a grid of 365
  //    256 x 256 tiles (the same layer at batch 128) is no longer two rounds with the second 43 % full.
  // Short contractions and small grids stay with the 128 x 128 tile (three blocks per CU, through registers).
  const bool rows_ok = cdiv(d.K, 256) * 256 == cdiv(d.K, 128) * 128;
  const long long t256 = (long long)cdiv(d.K, 256) * cdiv(ep.cols, 256);
  const long long t128 = (long long)cdiv(d.K, 256) * cdiv(ep.cols, 128);
  const bool big = rows_ok && bpn.n_k >= 512 && t256 >= 512;
  const bool mid = rows_ok && !big && bpn.n_k >= 256 && t128 >= 96;
  // other filter counts (384: one and a half 256-row tiles) take the same loop on 128 rows x 256 pixels
  const bool mid128 = !rows_ok && bpn.n_k >= 256 && (long long)cdiv(d.K, 128) * cdiv(ep.cols, 256) >= 96;
  if (pk.ptr) {
    if (big) return bf16_gemm_on<T256x256bf, true, true, 4>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_256x256");
    if (mid) return bf16_gemm_on<T256x128bf, true, true, 3>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_256x128");
    if (mid128) return bf16_gemm_on<T128x256bf, true, true, 3>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_128x256");
    return bf16_gemm_on<T128x128bf, false, true>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_128x128");
  }
  if (big) return bf16_gemm_on<T256x256bf, true, false, 4>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_256x256");
  if (mid) return bf16_gemm_on<T256x128bf, true, false, 3>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_256x128");
  if (mid128) return bf16_gemm_on<T128x256bf, true, false, 3>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_128x256");
  return bf16_gemm_on<T128x128bf, false, false>(d, bpn, xb, wprep, ep, pk, stream, "conv_fwd_bf16p_128x128");
}

template <class T>
static int run_fwd(const ConvDims& d, const DenseParams& ap, const GatherParams& bp,
                   const EpiParams& ep, hipStream_t stream, const char* tag) {
  typedef LoadDenseK<T::BM, T::BK, T::NT, false> AL;
  typedef LoadGatherR<T::BN, T::BK, T::NT, false> BL;
  return launch_mfma_gemm<T, AL, BL, true, PassConvFwd>(ap, bp, ep, d.C * d.R * d.S, 1, nullptr, stream, tag);
}

}  // namespace rh

using namespace rh;

extern "C" int32_t rh_conv2d_out_dim(int32_t in, int32_t size, int32_t stride, int32_t pad) {
  if (stride <= 0) return 0;
  return conv_out_dim(in, size, stride, pad);
}

extern "C" int rh_conv2d_fwd(const rh_conv_geom* g, float alpha, const float* x, const float* w,
                             float beta, float* y, const float* bias, void* ws, size_t ws_bytes,
                             int flags, rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!x || !w || !y) return RH_E_INVALID;
  if ((flags & RH_FUSE_BIAS) && !bias) return RH_E_INVALID;
  if (d.y_elems == 0) return 0;
  const size_t need = rh_conv2d_workspace_bytes(g, RH_CONV_FWD);
  if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return RH_E_WORKSPACE;
  hipStream_t stream = to_stream(stream_);

  if ((flags & RH_ALGO_WINOGRAD) && (!(wino_shape(d) || wino_shape5(d)) ||
                                     (flags & (RH_MATH_BF16_MFMA_FP32ACC | RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT))))
    return RH_E_UNSUPPORTED;
  if (!(flags & (RH_MATH_BF16_MFMA_FP32ACC | RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET)) && conv1x1_stream_applies(d))
    return launch_conv1x1_stream(d, RH_CONV_FWD, w, x, y, alpha, beta, (flags & RH_FUSE_BIAS) ? bias : nullptr,
                                 (flags & RH_FUSE_RELU) ? 1 : 0, stream);
  if ((wino_shape(d) || wino_shape5(d)) && !(flags & (RH_MATH_BF16_MFMA_FP32ACC | RH_ALGO_GATHER | RH_ALGO_SCALAR_OFFSET | RH_ALGO_DIRECT))) {
    const bool five = wino_shape5(d);   // a 5x5 layer as four 3x3 layers, added in the transform domain
    WinoGeom wg = five ? wino_geom_fwd5(d) : wino_geom_fwd(d);
    if (flags & RH_ALGO_SHARED_GPU) wg.tail_S = 1;
    if (flags & RH_ALGO_WINOGRAD ? wg.ok : five ? wino_pays5(wg) : wino_pays(wg))
      return launch_conv_wino(wg, false, x, w, y, alpha, beta, (flags & RH_FUSE_BIAS) ? bias : nullptr,
                              (flags & RH_FUSE_RELU) ? 1 : 0, nullptr, ws, stream, "conv_fwd_wino");
    if (flags & RH_ALGO_WINOGRAD) return RH_E_UNSUPPORTED;
  }
  const int CRS = d.C * d.R * d.S;
  if ((flags & RH_MATH_BF16_MFMA_FP32ACC) && !(flags & RH_ALGO_GATHER)) {
    const Bf16FwdPlan bpn = plan_bf16_fwd(d);
    if (bpn.ok) {
      EpiParams ep;
      ep.out = y; ep.bias = (flags & RH_FUSE_BIAS) ? bias : nullptr; ep.alpha = alpha; ep.beta = beta;
      ep.rows = d.K; ep.cols = d.N * d.P * d.Q; ep.inner = d.P * d.Q; ep.ld = 0; ep.relu = (flags & RH_FUSE_RELU) ? 1 : 0;
      ep.split_stride = 0;
      // scratch: [table | filter copy | image copy]
      char* xb = static_cast<char*>(ws) + bpn.tab_bytes + bpn.wt_bytes;
      if (int e = bf16_prep_filter(d, bpn, w, ws, stream)) return e;
      if (int e = bf16_pack_input(d, bpn, x, xb, stream)) return e;
      return bf16_gemm(d, bpn, xb, ws, ep, PackedOut(), stream);
    }
  }
  const SoffPlan sp = plan_soff_fwd(d);
  if ((flags & RH_MATH_BF16_MFMA_FP32ACC) && (!sp.ok || (flags & RH_ALGO_GATHER))) return RH_E_UNSUPPORTED;
  // (fp32, a contraction of up to 32, a 5x5 layer on one channel: the gather form is as fast and needs no launch in front of it)
  const bool tiny_k = CRS <= 32 && !(flags & (RH_MATH_BF16_MFMA_FP32ACC | RH_ALGO_SCALAR_OFFSET));
  if (sp.ok && !(flags & RH_ALGO_GATHER) && !tiny_k) {
    int* soff = static_cast<int*>(ws);
    float* wT = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes);
    const float* img = x;
    if (sp.img_bytes) {
      float* xp = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes);
      launch_pad_image_prep_soff(x, xp, (long long)d.N * d.C, d.H, d.W, sp.Hp, sp.Wp, sp.halo, w, wT, soff, sp.n_k, CRS, d.K,
                                 d.R, d.S, 0, stream);
      img = xp;
    } else {
      launch_prep_soff(w, wT, soff, sp.n_k, CRS, d.K, d.R, d.S, sp.Hp * sp.Wp, sp.Wp, 0, stream);
    }
    if (int e = launch_status()) return e;
    RowSParams ap;  // transposed filter [k][ko]
    ap.ptr = wT; ap.bytes = (uint32_t)(sizeof(float) * (size_t)sp.n_k * d.K + kRow4Slack);
    ap.M = d.K; ap.inner = d.K; ap.innerW = d.K; ap.img_stride = 0; ap.a_stride = 0; ap.b_stride = 1;
    ap.soff = nullptr; ap.ldk4 = d.K * 4;
    RowSParams bp;  // padded image, rows = output pixels
    bp.ptr = img; bp.bytes = (uint32_t)(sizeof(float) * (size_t)d.N * d.C * sp.Hp * sp.Wp);
    bp.M = d.N * d.P * d.Q; bp.inner = d.P * d.Q; bp.innerW = d.Q;
    bp.img_stride = d.C * sp.Hp * sp.Wp; bp.a_stride = d.st * sp.Wp; bp.b_stride = d.st;
    bp.soff = soff; bp.ldk4 = 0;
    EpiParams ep;
    ep.out = y; ep.bias = (flags & RH_FUSE_BIAS) ? bias : nullptr; ep.alpha = alpha; ep.beta = beta;
    ep.rows = d.K; ep.cols = bp.M; ep.inner = d.P * d.Q; ep.ld = 0; ep.relu = (flags & RH_FUSE_RELU) ? 1 : 0;
    ep.split_stride = 0;
    if (flags & RH_MATH_BF16_MFMA_FP32ACC) return run_fwd_soff_bf16(ap, bp, ep, sp.n_k, CRS, stream);
    float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + sp.tab_bytes + sp.wt_bytes + sp.img_bytes);
    switch (pick_bm(d.K)) {
      case 128:
        // (sliced contractions on the half-width tile, as below: NIN's 6 x 6 layers 4-7 % faster)
        if (sp.narrow128) return run_fwd_soff<T128x64>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_128x64", sp.splits, part, &sp.tail);
        return run_fwd_soff<T128x128>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_128x128", sp.splits, part, &sp.tail);
      case 96:  return run_fwd_soff<T96x128>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_96x128", sp.splits, part, &sp.tail);
      case 64:
        if (cdiv(d.K, 64) == 1 && prefer_k8_64(ep.cols))
          return run_fwd_soff<T64x256k8>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_64x256k8", sp.splits, part, &sp.tail);
        // a sliced contraction (a small layer) on the half-width tile: twice the blocks over the same slices, so that a
        // CU has others to run while one waits for its next K step's loads
        if (sp.splits > 1) return run_fwd_soff<T64x128>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_64x128", sp.splits, part, &sp.tail);
        return run_fwd_soff<T64x256>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_64x256", sp.splits, part, &sp.tail);
      default:
        if (sp.splits > 1) return run_fwd_soff<T32x128>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_32x128", sp.splits, part, &sp.tail);
        return run_fwd_soff<T32x256>(ap, bp, ep, sp.n_k, CRS, stream, "conv_fwd_32x256", sp.splits, part, &sp.tail);
    }
  }
  const int n_tab = round_up(CRS, kTabPad);
  int4* tab = static_cast<int4*>(ws);
  launch_build_fwd_tab(tab, n_tab, CRS, d.R, d.S, d.H * d.W, d.W, stream);
  if (int e = launch_status()) return e;

  DenseParams ap;
  ap.ptr = w; ap.bytes = (uint32_t)(d.w_elems * 4); ap.rows = d.K; ap.K = CRS; ap.ld = CRS; ap.ktab = nullptr;
  GatherParams bp;
  bp.ptr = x; bp.bytes = (uint32_t)(d.x_elems * 4);
  bp.M = d.N * d.P * d.Q; bp.inner = d.P * d.Q; bp.innerW = d.Q;
  bp.img_stride = d.C * d.H * d.W; bp.row_stride = d.W; bp.st = d.st; bp.pad = d.pad;
  bp.Hlim = d.H; bp.Wlim = d.W; bp.ktab = tab;
  EpiParams ep;
  ep.out = y; ep.bias = (flags & RH_FUSE_BIAS) ? bias : nullptr; ep.alpha = alpha; ep.beta = beta;
  ep.rows = d.K; ep.cols = bp.M; ep.inner = d.P * d.Q; ep.ld = 0; ep.relu = (flags & RH_FUSE_RELU) ? 1 : 0;
  ep.split_stride = 0;

  switch (pick_bm(d.K)) {
    case 128: return run_fwd<T128x128>(d, ap, bp, ep, stream, "conv_fwd_128x128");
    case 96:  return run_fwd<T96x256>(d, ap, bp, ep, stream, "conv_fwd_96x256");
    case 64:  return run_fwd<T64x256>(d, ap, bp, ep, stream, "conv_fwd_64x256");
    default:  return run_fwd<T32x256>(d, ap, bp, ep, stream, "conv_fwd_32x256");
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Packed bf16 activations between layers: a forward-only chain keeps its activations as bf16 in the layout the next
// convolution's loaders read, written by the producing kernel's epilogue, and its converted filters for as long as
// the weights stay the same.
// ---------------------------------------------------------------------------------------------------------------
static bool packed_act_dims_ok(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo) {
  return N > 0 && C > 0 && C % 8 == 0 && H > 0 && W > 0 && halo >= 0 &&
         2 * (size_t)N * C * (size_t)(H + 2 * halo) * (size_t)(W + 2 * halo) <= kMaxBufferBytes;
}

extern "C" size_t rh_bf16_act_bytes(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo) {
  if (!packed_act_dims_ok(N, C, H, W, halo)) return 0;
  return align256(2 * (size_t)N * C * (size_t)(H + 2 * halo) * (size_t)(W + 2 * halo));
}

extern "C" int rh_bf16_pack_nchw(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo, const float* x, void* xp,
                                 rh_stream_t stream_) {
  if (!packed_act_dims_ok(N, C, H, W, halo) || !x || !xp || (reinterpret_cast<uintptr_t>(xp) & 15)) return RH_E_INVALID;
  const int Hp = H + 2 * halo, Wp = W + 2 * halo, Cg = C / 8;
  const size_t groups = (size_t)N * Cg * Hp * Wp;
  hipStream_t stream = to_stream(stream_);
  ProfScope prof("nchw_to_bf16_groups", 4.0 * (double)N * C * H * W + 16.0 * (double)groups, stream);
  hipLaunchKernelGGL(nchw_to_bf16_groups_kernel, dim3(stream_grid(groups, 256)), dim3(256), 0, stream, x,
                     static_cast<uint4*>(xp), (unsigned)groups, H, W, FastDiv((uint32_t)Wp), FastDiv((uint32_t)Cg),
                     FastDiv((uint32_t)Hp), halo);
  return launch_status();
}

extern "C" int rh_bf16_unpack_nchw(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo, const void* xp, float* x,
                                   rh_stream_t stream_) {
  if (!packed_act_dims_ok(N, C, H, W, halo) || !x || !xp || (reinterpret_cast<uintptr_t>(xp) & 15)) return RH_E_INVALID;
  const int Cg = C / 8;
  const size_t groups = (size_t)N * Cg * H * W;
  hipStream_t stream = to_stream(stream_);
  ProfScope prof("bf16_groups_to_nchw", 4.0 * (double)N * C * H * W + 16.0 * (double)groups, stream);
  hipLaunchKernelGGL(bf16_groups_to_nchw_kernel, dim3(stream_grid(groups, 256)), dim3(256), 0, stream,
                     static_cast<const uint4*>(xp), x, (unsigned)groups, H, W, FastDiv((uint32_t)W), FastDiv((uint32_t)Cg),
                     FastDiv((uint32_t)H), halo);
  return launch_status();
}

extern "C" size_t rh_conv2d_fwd_bf16_filter_bytes(const rh_conv_geom* g) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  const Bf16FwdPlan bpn = plan_bf16_fwd(d);
  return bpn.ok ? bpn.tab_bytes + bpn.wt_bytes : 0;
}

extern "C" int rh_conv2d_fwd_bf16_takes_packed(const rh_conv_geom* g) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  const Bf16FwdPlan bpn = plan_bf16_fwd(d);
  return bpn.ok && bpn.s_groups == 0 ? 1 : 0;
}

extern "C" size_t rh_conv2d_fwd_bf16_workspace_bytes(const rh_conv_geom* g) {
  ConvDims d;
  if (conv_dims(g, &d)) return 0;
  const Bf16FwdPlan bpn = plan_bf16_fwd(d);
  return bpn.ok ? bpn.img_bytes : 0;
}

extern "C" int rh_conv2d_fwd_bf16_prep_filter(const rh_conv_geom* g, const float* w, void* wprep, size_t wprep_bytes,
                                              rh_stream_t stream) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if (!w || !wprep || (reinterpret_cast<uintptr_t>(wprep) & 255)) return RH_E_INVALID;
  const Bf16FwdPlan bpn = plan_bf16_fwd(d);
  if (!bpn.ok) return RH_E_UNSUPPORTED;
  if (wprep_bytes < bpn.tab_bytes + bpn.wt_bytes) return RH_E_WORKSPACE;
  return bf16_prep_filter(d, bpn, w, wprep, to_stream(stream));
}

extern "C" int rh_conv2d_fwd_bf16_packed(const rh_conv_geom* g, const void* xp, const float* x, const void* wprep,
                                         const float* bias, float* y, void* yp, int32_t yp_halo, void* ws, size_t ws_bytes,
                                         int flags, rh_stream_t stream_) {
  ConvDims d;
  if (int e = conv_dims(g, &d)) return e;
  if ((!xp) == (!x) || !wprep || (!y) == (!yp)) return RH_E_INVALID;  // one input form, one output form
  if ((flags & RH_FUSE_BIAS) && !bias) return RH_E_INVALID;
  if (flags & ~(RH_FUSE_BIAS | RH_FUSE_RELU | RH_ALGO_SCALAR_OFFSET)) return RH_E_INVALID;
  const Bf16FwdPlan bpn = plan_bf16_fwd(d);
  if (!bpn.ok) return RH_E_UNSUPPORTED;
  if (xp && bpn.s_groups > 0) return RH_E_UNSUPPORTED;  // grouped by filter columns: the copy is made from the fp32 image
  if (d.y_elems == 0) return 0;
  hipStream_t stream = to_stream(stream_);
  const void* xb = xp;
  if (x) {
    if (!ws || ws_bytes < bpn.img_bytes || (reinterpret_cast<uintptr_t>(ws) & 255)) return RH_E_WORKSPACE;
    if (int e = bf16_pack_input(d, bpn, x, ws, stream)) return e;
    xb = ws;
  } else if (reinterpret_cast<uintptr_t>(xp) & 15) {
    return RH_E_INVALID;
  }
  EpiParams ep;
  ep.out = y; ep.bias = (flags & RH_FUSE_BIAS) ? bias : nullptr; ep.alpha = 1.0f; ep.beta = 0.0f;
  ep.rows = d.K; ep.cols = d.N * d.P * d.Q; ep.inner = d.P * d.Q; ep.ld = 0; ep.relu = (flags & RH_FUSE_RELU) ? 1 : 0;
  ep.split_stride = 0;
  PackedOut pk;
  if (yp) {
    if (d.K % 8 != 0 || yp_halo < 0 || !packed_act_dims_ok(d.N, d.K, d.P, d.Q, yp_halo) ||
        (reinterpret_cast<uintptr_t>(yp) & 15))
      return RH_E_INVALID;
    pk.ptr = yp; pk.halo = yp_halo; pk.Cg = d.K / 8; pk.Wp = d.Q + 2 * yp_halo;
    pk.img_groups = (d.P + 2 * yp_halo) * pk.Cg * pk.Wp;
    pk.dQ = FastDiv((uint32_t)d.Q);
  }
  // (RH_ALGO_SCALAR_OFFSET: the streaming 1x1 kernel wherever it can run, not only where it is the faster one)
  return bf16_gemm(d, bpn, xb, wprep, ep, pk, stream, (flags & RH_ALGO_SCALAR_OFFSET) != 0);
}
