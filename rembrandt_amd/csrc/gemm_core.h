// fp32 MFMA tile engine shared by the convolution passes and the SGEMM entry point.
//
// One kernel template computes  D[i][j] = sum_k A(i,k) * B(k,j)  for a BM x BN block tile with
// v_mfma_f32_32x32x2_f32.  What differs between conv forward, backward-data, backward-filter and
// the four SGEMM transposition cases is only *where element (row, k) of an operand lives in
// global memory*; that is the job of the loader types below.  A loader brings a ROWS x BK slab
// of its operand into registers (buffer loads: out-of-range offsets read as zero, which is how
// zero padding, ragged tile edges and the K tail are handled without branches) and then writes
// it to LDS in [k][row] order.  The MFMA loop reads LDS with one ds_read_b32 per operand
// register; LDS is double buffered so one barrier per K step suffices.
//
// Lane mapping of v_mfma_f32_32x32x2_f32 (A is 32x2, B is 2x32, D is 32x32, one block):
//   a = A[lane % 32][lane / 32],  b = B[lane / 32][lane % 32],
//   d[v] = D[8*(v/4) + 4*(lane/32) + v%4][lane % 32],  v = 0..15.
// Lanes run along j, so j is always mapped to the memory-contiguous index of the output.
#pragma once
#include "common.h"

namespace rh {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Element offset whose byte offset (x4) is 0x80000000: beyond every accepted tensor, so a
// buffer load from it returns 0.  Sums of offsets are clamped to it before the shift.
constexpr uint32_t kInvalidOff = 0x20000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float buf_load_f32(__amdgpu_buffer_rsrc_t r, uint32_t elem_off) {
  const uint32_t o = elem_off < kInvalidOff ? elem_off : kInvalidOff;
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)(o << 2), 0, 0));
}

template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int NT = WM * WN * kWave;
  static constexpr int TM = BM / (WM * 32), TN = BN / (WN * 32);
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile / wave mismatch");
  static_assert(BK % 2 == 0, "BK must be even");
};

// Row padding of an LDS slab [BK][ROWS + pad].  Lanes-along-k loaders write a column of the
// slab per 16- or 32-lane group; the pad spreads those writes over the banks.
template <int BK> constexpr int lds_pad_kfast() { return BK == 16 ? 2 : 1; }

// ------------------------------------------------------------------------------------------
// Dense operand, k contiguous in memory: element (row, k) at ptr[row*ld + koff(k)], where
// koff(k) = k, or ktab[k] (negative = absent) when HAS_TAB.  Lanes run along k.
// ------------------------------------------------------------------------------------------
struct DenseParams {
  const float* ptr; uint32_t bytes;
  int rows, K, ld;
  const int* ktab;
};

template <int ROWS, int BK, int NT, bool HAS_TAB>
struct LoadDenseK {
  static constexpr int CNT = ROWS * BK / NT, RSTEP = NT / BK;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % BK == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef DenseParams Params;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t rowoff[CNT];
  const int* ktab;
  int kk, K, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kk = tid % BK;
    const int r = tid / BK;
    K = p.K;
    ktab = p.ktab;
    sbase = kk * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int row = row0 + r + i * RSTEP;
      rowoff[i] = row < p.rows ? (uint32_t)row * (uint32_t)p.ld : kInvalidOff;
    }
  }
  __device__ __forceinline__ void load(int k0, float (&v)[CNT]) {
    const int k = k0 + kk;
    uint32_t koff = kInvalidOff;
    if (k < K) {
      if (HAS_TAB) { const int t = ktab[k]; koff = t >= 0 ? (uint32_t)t : kInvalidOff; }
      else koff = (uint32_t)k;
    }
#pragma unroll
    for (int i = 0; i < CNT; ++i) v[i] = buf_load_f32(rsrc, rowoff[i] + koff);
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * RSTEP] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Dense operand, rows contiguous in memory: element (row, k) at ptr[k*ld + row].
// Lanes run along rows.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BK, int NT>
struct LoadDenseR {
  static constexpr int CNT = ROWS * BK / NT, KSTEP = NT / ROWS;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % ROWS == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef DenseParams Params;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t rowoff;
  int kk0, K, ld, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    const int row = tid % ROWS;
    kk0 = tid / ROWS;
    K = p.K;
    ld = p.ld;
    sbase = kk0 * LD + row;
    rowoff = (row0 + row) < p.rows ? (uint32_t)(row0 + row) : kInvalidOff;
  }
  __device__ __forceinline__ void load(int k0, float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int k = k0 + kk0 + i * KSTEP;
      const uint32_t koff = k < K ? (uint32_t)k * (uint32_t)ld : kInvalidOff;
      v[i] = buf_load_f32(rsrc, rowoff + koff);
    }
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * KSTEP * LD] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Gathered image operand with pixels as rows (conv forward: x; backward-data: dy).
// Row m is a pixel of the *result* tensor; k runs over the contraction (c,r,s) or (ko,r,s) and
// is described by a table entry {off, dr, ds, phase} (one int4 per k, wave-uniform):
//     element (m, k) = ptr[base(m) + off(k)]   if 0 <= h0(m)+dr(k) < Hlim, 0 <= w0(m)+ds(k) < Wlim
//                                                 and phase(m) == phase(k),   else 0.
// Forward:  m=(n,p,q): h0 = p*st-pad, w0 = q*st-pad, base = n*C*H*W + h0*W + w0, phase 0;
//           k=(c,r,s): off = c*H*W + r*W + s, dr = r, ds = s, phase 0; limits (H, W).
// Backward-data: m=(n,h,w): h+pad = st*hq + hr, w+pad = st*wq + wr; h0 = hq, w0 = wq,
//           base = n*K*P*Q + hq*Q + wq, phase = hr*st + wr;
//           k=(ko,r,s): r = st*rq + rr, s = st*sq + sr: off = ko*P*Q - rq*Q - sq, dr = -rq,
//           ds = -sq, phase = rr*st + sr; limits (P, Q).   (dy[n,ko,p,q] feeds dx[n,c,h,w] through
//           w[ko,c,r,s] exactly when h+pad-r = st*p and w+pad-s = st*q.)
// Table entries past the contraction length hold phase = -1, which never matches.
// ------------------------------------------------------------------------------------------
struct GatherParams {
  const float* ptr; uint32_t bytes;
  int M;           // number of pixel rows
  int inner;       // pixels per image   (P*Q forward, H*W backward-data)
  int innerW;      // pixels per row     (Q forward, W backward-data)
  int img_stride;  // elements per image of the gathered tensor
  int row_stride;  // elements per row of the gathered tensor (W forward, Q backward-data)
  int st, pad;
  int Hlim, Wlim;
  const int4* ktab;
};

template <int ROWS, int BK, int NT, bool BWD>
struct LoadGatherR {
  static constexpr int CNT = ROWS * BK / NT, KSTEP = NT / ROWS;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % ROWS == 0 && (ROWS * BK) % NT == 0 && ROWS % kWave == 0, "loader shape");
  typedef GatherParams Params;
  __amdgpu_buffer_rsrc_t rsrc;
  const int4* ktab;
  int base, h0, w0, phase, Hlim, Wlim, kk0, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    ktab = p.ktab;
    Hlim = p.Hlim;
    Wlim = p.Wlim;
    const int row = tid % ROWS;
    kk0 = __builtin_amdgcn_readfirstlane(tid / ROWS);  // ROWS % 64 == 0: uniform per wave
    sbase = kk0 * LD + row;
    const int m = row0 + row;
    const bool valid = m < p.M;
    const int mm = valid ? m : 0;
    const int n = mm / p.inner;
    const int rem = mm - n * p.inner;
    const int a = rem / p.innerW;
    const int b = rem - a * p.innerW;
    if (!BWD) {
      h0 = a * p.st - p.pad;
      w0 = b * p.st - p.pad;
      phase = 0;
    } else {
      const int hp = a + p.pad, wp = b + p.pad;
      h0 = hp / p.st;
      w0 = wp / p.st;
      phase = (hp - h0 * p.st) * p.st + (wp - w0 * p.st);
    }
    base = n * p.img_stride + h0 * p.row_stride + w0;
    if (!valid) phase = -2;
  }
  __device__ __forceinline__ void load(int k0, float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int4 e = ktab[k0 + kk0 + i * KSTEP];
      const bool ok = (unsigned)(h0 + e.y) < (unsigned)Hlim && (unsigned)(w0 + e.z) < (unsigned)Wlim &&
                      e.w == phase;
      v[i] = buf_load_f32(rsrc, ok ? (uint32_t)(base + e.x) : kInvalidOff);
    }
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * KSTEP * LD] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Backward-filter operands: the contraction index k is an output pixel (n,p,q); lanes run
// along k because both dy and x are contiguous along q.
//   A = dy:  element (ko, pix) = dy[(n*Kout + ko)*PQ + pq]
//   B = x :  element ((c,r,s), pix) = x[n*C*H*W + c*H*W + (p*st-pad+r)*W + q*st-pad+s] or 0
// The (c,r,s) rows of a thread are fixed for the whole K loop; their {off, r, s} come from the
// same table the forward pass uses and are kept in registers.
// ------------------------------------------------------------------------------------------
struct PixDyParams {
  const float* ptr; uint32_t bytes;
  int rows;  // Kout
  int M;     // N*P*Q
  int PQ;
};

template <int ROWS, int BK, int NT>
struct LoadPixDy {
  static constexpr int CNT = ROWS * BK / NT, RSTEP = NT / BK;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % BK == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef PixDyParams Params;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t rowoff[CNT];
  int kk, M, PQ, img, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kk = tid % BK;
    const int r = tid / BK;
    M = p.M;
    PQ = p.PQ;
    img = p.rows * p.PQ;
    sbase = kk * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int row = row0 + r + i * RSTEP;
      rowoff[i] = row < p.rows ? (uint32_t)row * (uint32_t)p.PQ : kInvalidOff;
    }
  }
  __device__ __forceinline__ void load(int k0, float (&v)[CNT]) {
    const int pix = k0 + kk;
    uint32_t kbase = kInvalidOff;
    if (pix < M) {
      const int n = pix / PQ;
      kbase = (uint32_t)(n * img + (pix - n * PQ));
    }
#pragma unroll
    for (int i = 0; i < CNT; ++i) v[i] = buf_load_f32(rsrc, rowoff[i] + kbase);
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * RSTEP] = v[i];
  }
};

struct PixXParams {
  const float* ptr; uint32_t bytes;
  int rows;  // C*R*S
  int M, PQ, Q;
  int img_stride;  // C*H*W
  int H, W, st, pad;
  const int4* rtab;  // per (c,r,s): {c*H*W + r*W + s, r, s, 0}
};

template <int ROWS, int BK, int NT>
struct LoadPixX {
  static constexpr int CNT = ROWS * BK / NT, RSTEP = NT / BK;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % BK == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef PixXParams Params;
  __amdgpu_buffer_rsrc_t rsrc;
  int roff[CNT], rr[CNT], rs[CNT];
  int kk, M, PQ, Q, img, H, W, st, pad, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kk = tid % BK;
    const int r = tid / BK;
    M = p.M; PQ = p.PQ; Q = p.Q; img = p.img_stride; H = p.H; W = p.W; st = p.st; pad = p.pad;
    sbase = kk * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int row = row0 + r + i * RSTEP;
      if (row < p.rows) {
        const int4 e = p.rtab[row];
        roff[i] = e.x; rr[i] = e.y; rs[i] = e.z;
      } else {
        roff[i] = 0; rr[i] = -(1 << 28); rs[i] = 0;
      }
    }
  }
  __device__ __forceinline__ void load(int k0, float (&v)[CNT]) {
    const int pix = k0 + kk;
    int h0 = -(1 << 28), w0 = 0, base = 0;
    if (pix < M) {
      const int n = pix / PQ;
      const int pq = pix - n * PQ;
      const int p = pq / Q;
      const int q = pq - p * Q;
      h0 = p * st - pad;
      w0 = q * st - pad;
      base = n * img + h0 * W + w0;
    }
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const bool ok = (unsigned)(h0 + rr[i]) < (unsigned)H && (unsigned)(w0 + rs[i]) < (unsigned)W;
      v[i] = buf_load_f32(rsrc, ok ? (uint32_t)(base + roff[i]) : kInvalidOff);
    }
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * RSTEP] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Epilogue.  Element (row i, col j) of the tile result goes to
//   NCHW : out[((j / inner) * rows + i) * inner + j % inner]    (j = pixel, i = channel)
//   dense: out[i * ld + j]
// value = alpha*acc + beta*old (+ bias[i]) (clamped at 0 if relu).  With split_stride != 0 the
// block writes its partial sum, unblended, to out + blockIdx.y * split_stride (dense).
// ------------------------------------------------------------------------------------------
struct EpiParams {
  float* out;
  const float* bias;
  float alpha, beta;
  int rows, cols, inner, ld;
  int relu;
  long long split_stride;
};

// Blocks are handed to the 8 XCDs round-robin by the hardware.  Renumber them so that every
// XCD works on one contiguous range of tiles (row tiles fastest): neighbouring tiles share
// their B slab, so it is fetched into that XCD's L2 once.
__device__ __forceinline__ int xcd_remap(int b, int nb) {
  const int per = nb >> 3, rem = nb & 7;
  const int xcd = b & 7, idx = b >> 3;
  const int start = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
  return start + idx;
}

template <class T, class AL, class BL, bool NCHW>
__global__ __launch_bounds__(T::NT) void mfma_gemm_kernel(typename AL::Params ap,
                                                          typename BL::Params bp, EpiParams ep,
                                                          int tiles_m, int k_chunks,
                                                          int chunks_per_split) {
  constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN;
  constexpr int LDA = AL::LD, LDB = BL::LD;
  __shared__ float sA[2][BK * LDA];
  __shared__ float sB[2][BK * LDB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;

  const int logical = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int c_begin = blockIdx.y * chunks_per_split;
  int c_end = c_begin + chunks_per_split;
  if (c_end > k_chunks) c_end = k_chunks;
  const int nk = c_end - c_begin;

  AL la;
  BL lb;
  la.init(ap, m0, tid);
  lb.init(bp, n0, tid);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  float ra[AL::CNT], rb[BL::CNT];
  if (nk > 0) {
    la.load(c_begin * BK, ra);
    lb.load(c_begin * BK, rb);
    la.store(sA[0], ra);
    lb.store(sB[0], rb);
  }
  __syncthreads();

  const int a_rd = (lane >> 5) * LDA + wm * (TM * 32) + (lane & 31);
  const int b_rd = (lane >> 5) * LDB + wn * (TN * 32) + (lane & 31);

  for (int it = 0; it < nk; ++it) {
    const int cur = it & 1;
    const bool more = it + 1 < nk;
    if (more) {
      la.load((c_begin + it + 1) * BK, ra);
      lb.load((c_begin + it + 1) * BK, rb);
    }
    const float* pa = sA[cur] + a_rd;
    const float* pb = sB[cur] + b_rd;
#pragma unroll
    for (int k2 = 0; k2 < BK; k2 += 2) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = pa[k2 * LDA + i * 32];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = pb[k2 * LDB + j * 32];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      la.store(sA[cur ^ 1], ra);
      lb.store(sB[cur ^ 1], rb);
    }
    __syncthreads();
  }

  // ---- epilogue
  const bool split = ep.split_stride != 0;
  float* out = ep.out + (split ? (long long)blockIdx.y * ep.split_stride : 0ll);
  const float alpha = split ? 1.0f : ep.alpha;
  const float beta = split ? 0.0f : ep.beta;
  const int row_stride = NCHW ? ep.inner : ep.ld;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * (TN * 32) + j * 32 + (lane & 31);
    if (col >= ep.cols) continue;
    int coloff;
    if (NCHW) {
      const int img = col / ep.inner;
      coloff = img * ep.rows * ep.inner + (col - img * ep.inner);
    } else {
      coloff = col;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int rbase = m0 + wm * (TM * 32) + i * 32 + (lane >> 5) * 4;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = rbase + (v >> 2) * 8 + (v & 3);
        if (row < ep.rows) {
          float* dst = out + (size_t)coloff + (size_t)row * row_stride;
          float val = alpha * acc[i][j][v];
          if (beta != 0.0f) val += beta * *dst;
          if (!split && ep.bias) val += ep.bias[row];
          if (!split && ep.relu) val = val > 0.0f ? val : 0.0f;
          *dst = val;
        }
      }
    }
  }
}

}  // namespace rh
