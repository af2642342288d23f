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
#include <type_traits>

#include "common.h"

namespace rh {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Element offset whose byte offset (x4) is 0x80000000: beyond every accepted tensor, so a
// buffer load from it returns 0.  Sums of offsets are clamped to it before the shift.
constexpr uint32_t kInvalidOff = 0x20000000u;
constexpr uint32_t kInvalidByteOff = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float buf_load_f32(__amdgpu_buffer_rsrc_t r, uint32_t elem_off) {
  const uint32_t o = elem_off < kInvalidOff ? elem_off : kInvalidOff;
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)(o << 2), 0, 0));
}

// OCC = waves per SIMD the register allocation must leave room for (blocks per CU for 4-wave blocks).
template <int BM_, int BN_, int BK_, int WM_, int WN_, int OCC_ = 1>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, OCC = OCC_;
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
  typedef float Reg;
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
  uint32_t koff;
  __device__ __forceinline__ void prep(int k0) {
    const int k = k0 + kk;
    koff = kInvalidOff;
    if (k < K) {
      if (HAS_TAB) { const int t = ktab[k]; koff = t >= 0 ? (uint32_t)t : kInvalidOff; }
      else koff = (uint32_t)k;
    }
  }
  __device__ __forceinline__ float load_one(int i) const { return buf_load_f32(rsrc, rowoff[i] + koff); }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * RSTEP] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// The same operand read four k at a time: a lane loads 16 bytes (k = 4q .. 4q+3 of one row) with one
// buffer_load_dwordx4, a quarter of the load instructions and address additions of LoadDenseK, and writes the four
// values to four k rows of the same [k][row] slab.  A wave's instruction covers 16 rows of 64 contiguous bytes.
// Needs ld % 4 == 0 and a 16-byte aligned base (aligned loads) and K % 4 == 0 (a group never straddles the end of
// its row: it is read whole or not at all).
// ------------------------------------------------------------------------------------------
template <int ROWS, int BK, int NT>
struct LoadDenseK4 {
  static constexpr int QPR = BK / 4;                      // lanes per row
  static constexpr int RPI = NT / QPR;                    // rows one instruction of the block covers
  static constexpr int CNT = (ROWS + RPI - 1) / RPI;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(BK % 4 == 0 && NT % QPR == 0, "loader shape");
  typedef DenseParams Params;
  typedef float4 Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t rowoff[CNT];
  int kq, r, K, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kq = (tid % QPR) * 4;
    r = tid / QPR;
    K = p.K;
    sbase = kq * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int slot = r + i * RPI, row = row0 + slot;
      rowoff[i] = (slot < ROWS && row < p.rows) ? (uint32_t)row * (uint32_t)p.ld : kInvalidOff;
    }
  }
  uint32_t koff;
  __device__ __forceinline__ void prep(int k0) {
    const int k = k0 + kq;
    koff = k < K ? (uint32_t)k : kInvalidOff;
  }
  __device__ __forceinline__ float4 load_one(int i) const {
    const uint32_t e = rowoff[i] + koff;
    const uint32_t o = e < kInvalidOff ? e : kInvalidOff;
    return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(o << 2), 0, 0));
  }
  __device__ __forceinline__ void store(float* s, const float4 (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      if (ROWS % RPI != 0 && r + i * RPI >= ROWS) continue;   // a thread past the slab's rows (tiles narrower than RPI)
      float* d = s + sbase + i * RPI;
      d[0] = v[i].x; d[LD] = v[i].y; d[2 * LD] = v[i].z; d[3 * LD] = v[i].w;
    }
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
  typedef float Reg;
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
  int kcur;
  __device__ __forceinline__ void prep(int k0) { kcur = k0 + kk0; }
  __device__ __forceinline__ float load_one(int i) const {
    const int k = kcur + i * KSTEP;
    const uint32_t koff = k < K ? (uint32_t)k * (uint32_t)ld : kInvalidOff;
    return buf_load_f32(rsrc, rowoff + koff);
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
  // Thread (row, kk0) loads the CNT consecutive k values kk0*CNT .. kk0*CNT + CNT-1 of its row, so the
  // table entries a wave needs in one K step are contiguous and wave-uniform: the compiler fetches
  // them with a few wide scalar loads issued together, instead of one dependent load per element.
  static constexpr int CNT = ROWS * BK / NT;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % ROWS == 0 && (ROWS * BK) % NT == 0 && ROWS % kWave == 0, "loader shape");
  typedef GatherParams Params;
  typedef float Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  const int4* ktab;
  int base, h0, w0, phase, Hlim, Wlim, sbase;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    Hlim = p.Hlim;
    Wlim = p.Wlim;
    const int row = tid % ROWS;
    const int kk0 = __builtin_amdgcn_readfirstlane(tid / ROWS);  // ROWS % 64 == 0: uniform per wave
    ktab = p.ktab + kk0 * CNT;
    sbase = kk0 * CNT * LD + row;
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
  int4 e[CNT];
  __device__ __forceinline__ void prep(int k0) {
    const int4* t = ktab + k0;
#pragma unroll
    for (int i = 0; i < CNT; ++i) e[i] = t[i];
  }
  __device__ __forceinline__ float load_one(int i) const {
    // bitwise, not short-circuit: no branches in the load path
    const int ok = (int)((unsigned)(h0 + e[i].y) < (unsigned)Hlim) & (int)((unsigned)(w0 + e[i].z) < (unsigned)Wlim) &
                   (int)(e[i].w == phase);
    return buf_load_f32(rsrc, ok ? (uint32_t)(base + e[i].x) : kInvalidOff);
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * LD] = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Scalar-offset operand: element (row, k) at  ptr + vbase(row) + soff(k)  (byte offsets), rows
// along lanes.  vbase is fixed per lane for the whole K loop (VGPR), soff is wave-uniform (SGPR,
// the soffset field of the buffer load), so loading an element costs no vector ALU work at all.
// Used on operands prepared so that every (row, k) pair of a valid row is in range:
//   * the filter transposed to [k][row] and zero padded to a multiple of the K step (LINEAR);
//   * the gathered image, zero padded by the conv padding, with a k -> byte offset table
//     (entries past the contraction length are 0: the filter rows there are zero).
// A row past the end gets vbase = 0x80000000, which reads as 0.
// Row decomposition: m -> (n, a, b) = (m / inner, (m % inner) / innerW, m % innerW);
// vbase = 4 * (n*img_stride + a*a_stride + b*b_stride).
// ------------------------------------------------------------------------------------------
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// {lo, hi} -> one dword of two bf16 (lo in bits 0-15), each rounded to nearest even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2_t p;
  p[0] = (__bf16)lo;
  p[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, p);
}

struct RowSParams {
  const float* ptr; uint32_t bytes;
  int M, inner, innerW;
  int img_stride, a_stride, b_stride;
  const int* soff;  // table of byte offsets (not LINEAR)
  int ldk4;         // bytes between consecutive k (LINEAR)
};

template <int ROWS, int BK, int NT, bool LINEAR>
struct LoadRowS {
  static constexpr int CNT = ROWS * BK / NT;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % ROWS == 0 && (ROWS * BK) % NT == 0 && ROWS % kWave == 0, "loader shape");
  typedef RowSParams Params;
  typedef float Reg;  // what load_one returns and store_bf16 takes
  __amdgpu_buffer_rsrc_t rsrc;
  const int* tab;
  uint32_t vbase;
  int ldk4, kk0c, sbase;
  int so[CNT];

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    const int row = tid % ROWS;
    const int kk0 = __builtin_amdgcn_readfirstlane(tid / ROWS);
    kk0c = kk0 * CNT;
    tab = p.soff;
    ldk4 = p.ldk4;
    sbase = kk0c * LD + row;
    const int m = row0 + row;
    const bool valid = m < p.M;
    const int mm = valid ? m : 0;
    const int n = mm / p.inner;
    const int rem = mm - n * p.inner;
    const int a = rem / p.innerW;
    const int b = rem - a * p.innerW;
    vbase = valid ? (uint32_t)(n * p.img_stride + a * p.a_stride + b * p.b_stride) << 2 : 0x80000000u;
  }
  __device__ __forceinline__ void prep(int k0) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so[i] = LINEAR ? (k0 + kk0c + i) * ldk4 : tab[k0 + kk0c + i];
  }
  __device__ __forceinline__ float load_one(int i) const {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)vbase, so[i], 0));
  }
  __device__ __forceinline__ void store(float* s, const float (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[sbase + i * LD] = v[i];
  }
  // bf16 form of store(): a thread's CNT values are consecutive k of one row.  They are rounded to bf16
  // (round to nearest even) and written as 16-byte groups of 8 consecutive k: slab[kgroup][row] (uint4),
  // which is exactly one lane's operand of v_mfma_f32_32x32x16_bf16.
  __device__ __forceinline__ void store_bf16(uint4* s, const float (&v)[CNT]) {
    static_assert(CNT % 8 == 0, "bf16 packing needs 8 consecutive k per thread");
    const int row = sbase - kk0c * LD;
#pragma unroll
    for (int g = 0; g < CNT / 8; ++g) {
      uint4 q;
      q.x = pack_bf16(v[8 * g + 0], v[8 * g + 1]);
      q.y = pack_bf16(v[8 * g + 2], v[8 * g + 3]);
      q.z = pack_bf16(v[8 * g + 4], v[8 * g + 5]);
      q.w = pack_bf16(v[8 * g + 6], v[8 * g + 7]);
      s[(kk0c / 8 + g) * ROWS + row] = q;
    }
  }
};

// ------------------------------------------------------------------------------------------
// LINEAR scalar-offset operand whose rows are contiguous in memory (row m+1 sits 4 bytes after row m: the
// transposed filter [k][row]): a lane loads four rows of one k with one buffer_load_dwordx4 and writes them with one
// ds_write_b128, a quarter of the loader instructions of LoadRowS.  A wave's load covers 64/(ROWS/4) values of k,
// so the lane's share of the k offset is part of its vector offset.  Same Params as LoadRowS (b_stride == 1, no
// n / a decomposition).  The 12 bytes after the last valid row of the buffer must be readable: rows past M
// inside a group read whatever follows, and only feed result rows that are never stored.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BK, int NT>
struct LoadRow4 {
  static constexpr int LPK = ROWS / 4;           // lanes per k
  static constexpr int KPI = NT / LPK;           // k values one instruction of the block covers
  static constexpr int CNT = BK / KPI;           // loads per thread and K step
  static constexpr int LD = ROWS + 4;            // rows of 16-byte aligned groups
  static_assert(ROWS % 4 == 0 && NT % LPK == 0 && BK % KPI == 0 && CNT >= 1, "loader shape");
  typedef RowSParams Params;
  typedef float4 Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t vbase;
  int ldk4, sbase;
  int so[CNT];

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    const int row = (tid % LPK) * 4;
    const int kl = tid / LPK;  // this thread's k within an instruction
    ldk4 = p.ldk4;
    sbase = kl * LD + row;
    const int m = row0 + row;
    vbase = m < p.M ? ((uint32_t)m << 2) + (uint32_t)(kl * ldk4) : 0x80000000u;
  }
  __device__ __forceinline__ void prep(int k0) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so[i] = (k0 + i * KPI) * ldk4;
  }
  __device__ __forceinline__ float4 load_one(int i) const {
    return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vbase, so[i], 0));
  }
  __device__ __forceinline__ void store(float* s, const float4 (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) *reinterpret_cast<float4*>(s + sbase + i * KPI * LD) = v[i];
  }
};

// ------------------------------------------------------------------------------------------
// Packed bf16 operand for the bf16 kernel: the operand already sits in memory as bf16 in groups of eight consecutive
// k of one row (16 bytes), so a lane's load is one buffer_load_dwordx4 of exactly what one v_mfma_f32_32x32x16_bf16
// operand register holds, and the LDS slab [k/8][row] receives it unchanged: no conversion, an eighth of the load
// instructions and half of the bytes of the fp32 loaders.
//   lane = row m -> (n, a, b) as in LoadRowS, byte offset vbase = n*img_stride + a*a_stride + b*b_stride;
//   group g of the contraction (k = 8g .. 8g+7): wave-uniform byte offset g*group_stride (LINEAR) or soff[g].
// ------------------------------------------------------------------------------------------
struct RowV8Params {
  const void* ptr; uint32_t bytes;
  int M, inner, innerW;
  int img_stride, a_stride, b_stride;  // bytes
  const int* soff;                     // per group of 8 k, bytes (not LINEAR)
  int group_stride;                    // bytes between consecutive groups (LINEAR)
};

template <int ROWS, int BK, int NT, bool LINEAR>
struct LoadRowV8 {
  static constexpr int KG = BK / 8;
  static constexpr int CNT = ROWS * KG / NT;  // 16-byte groups per thread and K step
  static_assert(BK % 8 == 0 && NT % ROWS == 0 && (ROWS * KG) % NT == 0 && ROWS % kWave == 0, "loader shape");
  typedef RowV8Params Params;
  typedef uint4 Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  const int* tab;
  uint32_t vbase;
  int g0, row, gstride;
  int so[CNT];

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    row = tid % ROWS;
    g0 = __builtin_amdgcn_readfirstlane(tid / ROWS) * CNT;
    tab = p.soff;
    gstride = p.group_stride;
    const int m = row0 + row;
    const bool valid = m < p.M;
    const int mm = valid ? m : 0;
    const int n = mm / p.inner;
    const int rem = mm - n * p.inner;
    const int a = rem / p.innerW;
    const int b = rem - a * p.innerW;
    vbase = valid ? (uint32_t)(n * p.img_stride + a * p.a_stride + b * p.b_stride) : 0x80000000u;
  }
  __device__ __forceinline__ void prep(int k0) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so[i] = LINEAR ? ((k0 >> 3) + g0 + i) * gstride : tab[(k0 >> 3) + g0 + i];
  }
  __device__ __forceinline__ uint4 load_one(int i) const {
    return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vbase, so[i], 0));
  }
  __device__ __forceinline__ void store_bf16(uint4* s, const uint4 (&v)[CNT]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) s[(g0 + i) * ROWS + row] = v[i];
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
  FastDiv dPQ;  // division by PQ (set_pq): the loaders split a pixel index every K step
  void set_pq(int pq) { PQ = pq; dPQ = FastDiv((uint32_t)(pq > 0 ? pq : 1)); }
};

template <int ROWS, int BK, int NT>
struct LoadPixDy {
  static constexpr int CNT = ROWS * BK / NT, RSTEP = NT / BK;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % BK == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef PixDyParams Params;
  typedef float Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t rowoff[CNT];
  int kk, M, img, sbase;
  FastDiv dPQ;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kk = tid % BK;
    const int r = tid / BK;
    M = p.M;
    dPQ = p.dPQ;
    img = p.rows * p.PQ;
    sbase = kk * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int row = row0 + r + i * RSTEP;
      rowoff[i] = row < p.rows ? ((uint32_t)row * (uint32_t)p.PQ) << 2 : kInvalidByteOff;
    }
  }
  // Byte offsets; an absent row or pixel carries 0x80000000, so the sum of a present and an absent part lies past
  // every accepted tensor (the load returns 0) without a clamp.  (Both absent: the sum wraps to a small offset and
  // the load returns some element, into a product of an absent row and an absent pixel, which is never stored.)
  uint32_t kbase;
  __device__ __forceinline__ void prep(int k0) {
    const int pix = k0 + kk;
    kbase = kInvalidByteOff;
    if (pix < M) {
      uint32_t n, pq;
      dPQ.divmod((uint32_t)pix, n, pq);
      kbase = (n * (uint32_t)img + pq) << 2;
    }
  }
  __device__ __forceinline__ float load_one(int i) const {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(rowoff[i] + kbase), 0, 0));
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
  FastDiv dPQ, dQ;   // divisions by PQ and Q (set_pq)
  FastDiv dRS, dS;   // a row (c,r,s) is decoded where the loader starts: tap (r, s) at c*H*W + r*W + s (set_filter)
  void set_pq(int pq, int q) {
    PQ = pq; Q = q;
    dPQ = FastDiv((uint32_t)(pq > 0 ? pq : 1));
    dQ = FastDiv((uint32_t)(q > 0 ? q : 1));
  }
  void set_filter(int R, int S) {
    dRS = FastDiv((uint32_t)(R * S > 0 ? R * S : 1));
    dS = FastDiv((uint32_t)(S > 0 ? S : 1));
  }
};

// NOPAD: no padding, so every tap of every output pixel lies inside the image and the bounds checks fall away
// (three vector instructions per element instead of nine; the loader's arithmetic shares the issue port with the
// MFMAs: AlexNet conv1's filter gradient ran nine vector instructions per MFMA with the checks and runtime divisions).
template <int ROWS, int BK, int NT, bool NOPAD = false>
struct LoadPixX {
  static constexpr int CNT = ROWS * BK / NT, RSTEP = NT / BK;
  static constexpr int LD = ROWS + lds_pad_kfast<BK>();
  static_assert(NT % BK == 0 && (ROWS * BK) % NT == 0, "loader shape");
  typedef PixXParams Params;
  typedef float Reg;
  __amdgpu_buffer_rsrc_t rsrc;
  int roff[CNT], rr[CNT], rs[CNT];
  int kk, M, img, H, W, st, pad, sbase;
  FastDiv dPQ, dQ;

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    rsrc = make_rsrc(p.ptr, p.bytes);
    kk = tid % BK;
    const int r = tid / BK;
    M = p.M; dPQ = p.dPQ; dQ = p.dQ; img = p.img_stride; H = p.H; W = p.W; st = p.st; pad = p.pad;
    sbase = kk * LD + r;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const int row = row0 + r + i * RSTEP;
      if (row < p.rows) {
        uint32_t c, t, r2, s2;
        p.dRS.divmod((uint32_t)row, c, t);
        p.dS.divmod(t, r2, s2);
        roff[i] = (int)c * p.H * p.W + (int)r2 * p.W + (int)s2; rr[i] = (int)r2; rs[i] = (int)s2;
      } else {
        roff[i] = NOPAD ? (int)kInvalidByteOff : 0; rr[i] = -(1 << 28); rs[i] = 0;
      }
      if (NOPAD && row < p.rows) roff[i] <<= 2;  // byte offsets, as in LoadPixDy
    }
  }
  int h0, w0, base;
  __device__ __forceinline__ void prep(int k0) {
    const int pix = k0 + kk;
    h0 = -(1 << 28); w0 = 0; base = NOPAD ? (int)kInvalidByteOff : 0;
    if (pix < M) {
      uint32_t n, pq, p, q;
      dPQ.divmod((uint32_t)pix, n, pq);
      dQ.divmod(pq, p, q);
      h0 = (int)p * st - pad;
      w0 = (int)q * st - pad;
      base = (int)n * img + h0 * W + w0;
      if (NOPAD) base <<= 2;
    }
  }
  __device__ __forceinline__ float load_one(int i) const {
    if (NOPAD)
      return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)((uint32_t)base + (uint32_t)roff[i]), 0, 0));
    const int ok = (int)((unsigned)(h0 + rr[i]) < (unsigned)H) & (int)((unsigned)(w0 + rs[i]) < (unsigned)W);
    return buf_load_f32(rsrc, ok ? (uint32_t)(base + roff[i]) : kInvalidOff);
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
// block writes its partial sum, unblended, to out + split * split_stride (dense).
//
// Tail form (tail_tiles > 0, 1-D grid): the first full_tiles tiles of the logical order are computed whole and
// blended into `out`; each of the last tail_tiles tiles is computed by tail_splits blocks over slices of the
// contraction, which write unblended partial sums to part + slice * split_stride - part_first: a slab holds the
// result's elements from index part_first on (the first image any tail column belongs to), not the whole result.
// It evens out a grid whose tile count is a little over a multiple of the CU count (676 tiles on 256 CUs: a quarter
// of the CUs would carry three tiles, the rest two) without paying partial-sum traffic for the whole result.
// ------------------------------------------------------------------------------------------
struct EpiParams {
  float* out;
  const float* bias;
  float alpha, beta;
  int rows, cols, inner, ld;
  int relu;
  long long split_stride;
  const float* bias_col = nullptr;   // one value per result column (the dense, non-NCHW form: an affine layer's bias)
  // NCHW form: a tensor of the result's shape; result elements whose mask value is not > 0 are stored as 0 (backward-data
  // that also applies the backward of the ReLU that produced its input: the mask is that ReLU's output).
  const float* mask = nullptr;
  float* part = nullptr;
  long long part_first = 0;
  int full_tiles = 0, tail_tiles = 0, tail_splits = 0;
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

// Epilogue shared by the fp32 and bf16 kernels: D (in the 32x32 MFMA accumulator layout: lane%32 = column,
// rows 8*(v/4) + 4*(lane/32) + v%4) -> out, with the alpha/beta blend, optional bias and ReLU, or unblended
// into this split's slab of the partial-sum buffer.
//
// Loads and stores of a wave complete in order and share one counter, and the compiler cannot know that bias and
// mask do not alias the result: written element by element (load bias, load mask, store) every load waits for
// the store before it, a round trip to memory per element.  So the loads stand ahead of the stores here: the
// result goes out one 32 x 32 block at a time, and the bias of the next row of blocks (or the mask values of the
// next block) is fetched before the current block's stores are issued, never between two stores.
// Addresses: buffer instructions over the result (and the mask, which has its shape), a per-lane byte offset for
// each column block plus a wave-uniform offset for the row, so that a store costs no vector arithmetic and no
// address registers.  (Results, like operands, are at most kMaxBufferBytes long: the callers check.)
template <class T, bool NCHW>
__device__ __forceinline__ void store_tile(const f32x16 (&acc)[T::TM][T::TN], const EpiParams& ep, int m0, int n0,
                                           int wm, int wn, int lane, int split_idx) {
  constexpr int TM = T::TM, TN = T::TN;
  const bool split = split_idx >= 0;  // < 0: blend into the result
  float* out = !split ? ep.out
               : ep.tail_tiles > 0 ? ep.part + ((long long)split_idx * ep.split_stride - ep.part_first)
                                   : ep.out + (long long)split_idx * ep.split_stride;
  const float alpha = split ? 1.0f : ep.alpha;
  const float beta = split ? 0.0f : ep.beta;
  const uint32_t rs4 = 4u * (uint32_t)(NCHW ? ep.inner : ep.ld);  // bytes from a row to the next
  const int rlane = m0 + wm * (TM * 32) + (lane >> 5) * 4;
  const int clane = n0 + wn * (TN * 32) + (lane & 31);
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(out, 0x80000000u);
  // byte offset of (row rlane, this lane's column of block j)
  uint32_t voff[TN];
  bool col_ok[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = clane + j * 32;
    col_ok[j] = col < ep.cols;
    uint32_t e = (uint32_t)col;
    if (NCHW) {
      const int img = col / ep.inner;
      e = (uint32_t)img * (uint32_t)ep.rows * (uint32_t)ep.inner + (uint32_t)(col - img * ep.inner);
    }
    voff[j] = e * 4u + (uint32_t)rlane * rs4;
  }
  auto krow = [](int i, int v) { return i * 32 + (v >> 2) * 8 + (v & 3); };  // row of element v of block row i, from rlane
  const bool has_bias = !split && ep.bias != nullptr;
  const bool has_cbias = !NCHW && !split && ep.bias_col != nullptr;
  const bool relu = !split && ep.relu;
  const float* mask = NCHW && !split ? ep.mask : nullptr;
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(has_bias ? ep.bias : out, has_bias ? 4u * (uint32_t)ep.rows : 0u);
  const __amdgpu_buffer_rsrc_t rm = make_rsrc(mask ? mask : out, mask ? 0x80000000u : 0u);

  // One 32 x 32 block at a time, so that only its 16 values are live next to the accumulators (which die block
  // by block) and whatever has been fetched ahead.
  auto run = [&](auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;  // no element of this block's tile lies outside the result
    auto ok = [&](int i, int j, int v) { return FULL || (col_ok[j] && rlane + krow(i, v) < ep.rows); };
    // the block's elements of a tensor shaped like the result; elements outside it read 0.  Without branches where
    // the wave-uniform part of the offset cannot reach 2^31 (an offset with the top bit set is out of the buffer's
    // range): a load under a branch is waited for before the next one is issued.
    const bool select_form = rs4 <= 0x7fffffffu / (32u * TM);
    auto load16 = [&](__amdgpu_buffer_rsrc_t rs, int i, int j, float (&x)[16]) {
      if (FULL || select_form) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const uint32_t vo = ok(i, j, v) ? voff[j] : 0x80000000u;
          x[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, (int)vo, (int)((uint32_t)krow(i, v) * rs4), 0));
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          x[v] = 0.0f;
          if (ok(i, j, v))
            x[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, (int)voff[j], (int)((uint32_t)krow(i, v) * rs4), 0));
        }
      }
    };
    auto load_bias = [&](int i, float (&x)[16]) {  // rows past the last read as 0
#pragma unroll
      for (int v = 0; v < 16; ++v)
        x[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rb, rlane * 4, krow(i, v) * 4, 0));
    };
    auto store16 = [&](int i, int j, const float (&x)[16]) {
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (ok(i, j, v))
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(x[v]), rout, (int)voff[j], (int)((uint32_t)krow(i, v) * rs4), 0);
    };
    float cb[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) cb[j] = 0.0f;
    if (has_cbias) {
      const __amdgpu_buffer_rsrc_t rc = make_rsrc(ep.bias_col, 4u * (uint32_t)ep.cols);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        cb[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rc, (clane + j * 32) * 4, 0, 0));
    }
    // value = alpha * acc (+ beta * old) (+ bias[row]) (+ bias_col[col]) (clamped at 0) (0 where the mask is not > 0)
    if (beta != 0.0f || (mask && (has_bias || has_cbias))) {
      // accumulating calls (and combinations nothing in the library asks for): what a block needs is read
      // ahead of its own stores, behind those of the block before, one kind of operand at a time (registers)
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float x[16], t[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) x[v] = alpha * acc[i][j][v];
          if (beta != 0.0f) {
            load16(rout, i, j, t);
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] += beta * t[v];
          }
          __builtin_amdgcn_sched_barrier(0);
          if (has_bias) {
            load_bias(i, t);
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] += t[v];
          }
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            if (has_cbias) x[v] += cb[j];
            if (relu) x[v] = x[v] > 0.0f ? x[v] : 0.0f;
          }
          __builtin_amdgcn_sched_barrier(0);
          if (mask) {
            load16(rm, i, j, t);
#pragma unroll
            for (int v = 0; v < 16; ++v)
              if (!(t[v] > 0.0f)) x[v] = 0.0f;
          }
          store16(i, j, x);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    } else if (mask) {
      // backward-data with the ReLU backward folded in: a block's mask values are fetched after the block before
      // it has taken its own (one set of registers) and before that block's stores are issued
      float mk[16];
      load16(rm, 0, 0, mk);
#pragma unroll
      for (int b = 0; b < TM * TN; ++b) {
        const int i = b % TM, j = b / TM;
        float x[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float val = alpha * acc[i][j][v];
          if (relu) val = val > 0.0f ? val : 0.0f;
          if (!(mk[v] > 0.0f)) val = 0.0f;
          x[v] = val;
        }
        __builtin_amdgcn_sched_barrier(0);
        if (b + 1 < TM * TN) load16(rm, (b + 1) % TM, (b + 1) / TM, mk);
        store16(i, j, x);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      // forward passes and partial sums: the bias of the next row of blocks is fetched once the last block of
      // this row has taken its own, before that block's stores are issued
      float bv[16];
      if (has_bias) load_bias(0, bv);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float x[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float val = alpha * acc[i][j][v];
            if (has_bias) val += bv[v];
            if (has_cbias) val += cb[j];
            if (relu) val = val > 0.0f ? val : 0.0f;
            x[v] = val;
          }
          __builtin_amdgcn_sched_barrier(0);
          if (has_bias && j == TN - 1 && i + 1 < TM) load_bias(i + 1, bv);
          store16(i, j, x);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  if (m0 + T::BM <= ep.rows && n0 + T::BN <= ep.cols) run(std::true_type());
  else run(std::false_type());
}

// Packed bf16 result: the NCHW result (img, row, p, q) written as bf16 in the operand layout the packed loaders read,
//   [img][Hp][Cg][Wp][8]:  16-byte group ((img*Hp + p + halo)*Cg + row/8)*Wp + q + halo, element row % 8,
// Hp = P + 2*halo, Wp = Q + 2*halo, Cg = rows / 8 (rows a multiple of 8); the border is left alone (the owner of the
// buffer zeroed it once).  A consumer convolution with padding `halo` then reads it as it is: no conversion pass and
// half the bytes of an fp32 store.  value = acc (+ bias[row]) (clamped at 0 if relu), rounded to nearest even.
struct PackedOut {
  void* ptr = nullptr;
  int halo = 0, Cg = 0, Wp = 0;
  int img_groups = 0;  // 16-byte groups per image: Hp * Cg * Wp
  FastDiv dQ;          // division of a pixel index by Q
};

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <class T>
__device__ __forceinline__ void store_tile_packed(const f32x16 (&acc)[T::TM][T::TN], const EpiParams& ep, const PackedOut& pk,
                                                  int m0, int n0, int wm, int wn, int lane) {
  constexpr int TM = T::TM, TN = T::TN;
  const int sub = (lane >> 5) * 4;  // this lane's four rows inside a group of eight
  const int rwave = m0 + wm * (TM * 32);  // first row of the wave's part: a multiple of 32
  float r[TM][TN][16];  // separate scalars (see store_tile)
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) r[i][j][v] = acc[i][j][v];
  // bias first, for all of the lane's rows, so that no load stands between the stores (see store_tile);
  // rows past the last read as 0
  if (ep.bias) {
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(ep.bias, 4u * (uint32_t)ep.rows);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float bv[16];
#pragma unroll
      for (int v = 0; v < 16; ++v)
        bv[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rb, (rwave + sub) * 4,
                                                                               (i * 32 + (v >> 2) * 8 + (v & 3)) * 4, 0));
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) r[i][j][v] += bv[v];
    }
  }
  if (ep.relu) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) r[i][j][v] = r[i][j][v] > 0.0f ? r[i][j][v] : 0.0f;
  }
  // Buffer stores: a per-lane byte offset for each column block (the pixel's group of row group 0, plus this
  // lane's half of the group) and a wave-uniform one for the row group.  (The packed tensor is at most
  // kMaxBufferBytes long: the callers check.)
  const __amdgpu_buffer_rsrc_t rout = make_rsrc(pk.ptr, 0x80000000u);
  const uint32_t wp16 = 16u * (uint32_t)pk.Wp;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * (TN * 32) + j * 32 + (lane & 31);
    if (col >= ep.cols) continue;
    const int img = col / ep.inner;
    uint32_t p, q;
    pk.dQ.divmod((uint32_t)(col - img * ep.inner), p, q);
    const uint32_t voff = 16u * ((uint32_t)img * (uint32_t)pk.img_groups + (uint32_t)((int)p + pk.halo) * (uint32_t)(pk.Cg * pk.Wp) +
                                 (uint32_t)((int)q + pk.halo)) + (uint32_t)sub * 2u;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int vg = 0; vg < 4; ++vg) {
        const int rg = (rwave >> 3) + i * 4 + vg;  // row group of eight (wave-uniform)
        if (rg * 8 < ep.rows) {
          u32x2 w;
          w.x = pack_bf16(r[i][j][vg * 4 + 0], r[i][j][vg * 4 + 1]);
          w.y = pack_bf16(r[i][j][vg * 4 + 2], r[i][j][vg * 4 + 3]);
          __builtin_amdgcn_raw_buffer_store_b64(w, rout, (int)voff, (int)((uint32_t)rg * wp16), 0);
        }
      }
    }
  }
}

// Pass tags: they only make the instantiations of one pass distinct kernels (and kernel names) from
// those of another pass that uses the same tile and loaders.
struct PassConvFwd {};
struct PassConvBwdData {};
struct PassConvBwdFilter {};
struct PassSgemm {};

template <class T, class AL, class BL, bool NCHW, class PASS>
__global__ __launch_bounds__(T::NT, T::OCC) void mfma_gemm_kernel(typename AL::Params ap,
                                                          typename BL::Params bp, EpiParams ep,
                                                          int tiles_m, int k_chunks,
                                                          int chunks_per_split) {
  constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN;
  constexpr int LDA = AL::LD, LDB = BL::LD;
  // dynamic LDS: [2][BK*LDA] for A, then [2][BK*LDB] for B
  extern __shared__ float lds_dyn[];
  float* const sA_base = lds_dyn;
  float* const sB_base = lds_dyn + 2 * BK * LDA;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;

  // Blocks of the whole grid (tiles x splits, x fastest) are dealt to the 8 XCDs round-robin; remap so that
  // each XCD's L2 sees a contiguous range of (split, tile): all tiles of a split read the same K range.
  int slice, logical, dst_split;  // slice of the contraction, tile, and where the result goes (< 0: blended into out)
  if (ep.tail_tiles > 0) {
    const int b = blockIdx.x;
    if (b < ep.full_tiles) {
      logical = xcd_remap(b, ep.full_tiles);
      slice = 0;
      dst_split = -1;
    } else {
      const int r = xcd_remap(b - ep.full_tiles, ep.tail_tiles * ep.tail_splits);
      slice = r / ep.tail_tiles;
      logical = ep.full_tiles + (r - slice * ep.tail_tiles);
      dst_split = slice;
    }
  } else {
    const int tiles = gridDim.x;
    const int linear = xcd_remap(blockIdx.y * tiles + blockIdx.x, tiles * gridDim.y);
    slice = linear / tiles;
    logical = linear - slice * tiles;
    dst_split = ep.split_stride != 0 ? slice : -1;
  }
  slice = __builtin_amdgcn_readfirstlane(slice);
  logical = __builtin_amdgcn_readfirstlane(logical);
  dst_split = __builtin_amdgcn_readfirstlane(dst_split);
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // whole tiles of the tail form cover the full contraction; every other block covers its slice
  const bool whole = ep.tail_tiles > 0 && dst_split < 0;
  const int c_begin = whole ? 0 : slice * chunks_per_split;
  int c_end = whole ? k_chunks : c_begin + chunks_per_split;
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

  typename AL::Reg ra[AL::CNT];
  typename BL::Reg rb[BL::CNT];
  if (nk > 0) {
    la.prep(c_begin * BK);
    lb.prep(c_begin * BK);
#pragma unroll
    for (int i = 0; i < AL::CNT; ++i) ra[i] = la.load_one(i);
#pragma unroll
    for (int i = 0; i < BL::CNT; ++i) rb[i] = lb.load_one(i);
    la.store(sA_base, ra);
    lb.store(sB_base, rb);
  }
  __syncthreads();

  const int a_rd = (lane >> 5) * LDA + wm * (TM * 32) + (lane & 31);
  const int b_rd = (lane >> 5) * LDB + wn * (TN * 32) + (lane & 31);

  // One K step.  The instruction order is pinned with scheduling barriers into BK/2 groups of
  //   [LDS operand reads of the next group] [address math + global loads of a slice of the next
  //   K step's slabs] [TM*TN MFMAs of this group]
  // so that a wave keeps the matrix pipe fed by itself: LDS latency hides behind the MFMAs of
  // the group before, and the loader's VALU work issues in the shadow of running MFMAs.  The
  // global loads sit in the first half of the step, giving them the second half (and the other
  // waves' turns) to land before they are written to the other LDS buffer.
  constexpr int STEPS = BK / 2;
  constexpr int LSTEPS = STEPS / 2 > 0 ? STEPS / 2 : 1;  // groups that carry global loads
  constexpr int A_PER = (AL::CNT + LSTEPS - 1) / LSTEPS, B_PER = (BL::CNT + LSTEPS - 1) / LSTEPS;
  if (nk > 1) {
    la.prep((c_begin + 1) * BK);
    lb.prep((c_begin + 1) * BK);
  }
  auto k_step = [&](int it, auto more_tag) {
    constexpr bool MORE = decltype(more_tag)::value;
    const int cur = it & 1;
    const float* pa = sA_base + cur * (BK * LDA) + a_rd;
    const float* pb = sB_base + cur * (BK * LDB) + b_rd;
    float a[2][TM], b[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a[0][i] = pa[i * 32];
#pragma unroll
    for (int j = 0; j < TN; ++j) b[0][j] = pb[j * 32];
#pragma unroll
    for (int g = 0; g < STEPS; ++g) {
      const int c = g & 1, n = c ^ 1;
      __builtin_amdgcn_sched_barrier(0);  // nothing moves between groups
      if (g + 1 < STEPS) {
#pragma unroll
        for (int i = 0; i < TM; ++i) a[n][i] = pa[(2 * g + 2) * LDA + i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[n][j] = pb[(2 * g + 2) * LDB + j * 32];
      }
      if (MORE && g < LSTEPS) {
#pragma unroll
        for (int e = g * A_PER; e < (g + 1) * A_PER; ++e)
          if (e < AL::CNT) ra[e] = la.load_one(e);
#pragma unroll
        for (int e = g * B_PER; e < (g + 1) * B_PER; ++e)
          if (e < BL::CNT) rb[e] = lb.load_one(e);
      }
      __builtin_amdgcn_sched_barrier(0);  // loads and reads issue before this group's MFMAs
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c][i], b[c][j], acc[i][j], 0, 0, 0);
      if (MORE && g == (LSTEPS < STEPS ? LSTEPS : STEPS - 1)) {
        // the table entries / pixel decomposition of the step after next: all loads of the next
        // step have been issued by now, and this leaves a whole half step for the scalar loads
        if (it + 2 < nk) {
          la.prep((c_begin + it + 2) * BK);
          lb.prep((c_begin + it + 2) * BK);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (MORE) {
      la.store(sA_base + (cur ^ 1) * (BK * LDA), ra);
      lb.store(sB_base + (cur ^ 1) * (BK * LDB), rb);
    }
    __syncthreads();
  };
  for (int it = 0; it + 1 < nk; ++it) k_step(it, std::true_type());
  if (nk > 0) k_step(nk - 1, std::false_type());

  store_tile<T, NCHW>(acc, ep, m0, n0, wm, wn, lane, dst_split);
}

// ------------------------------------------------------------------------------------------
// bf16-operand form of the same tile engine (RH_MATH_BF16_MFMA_FP32ACC): operands reach LDS as bf16 (rounded by the
// fp32 loaders as they write, or already packed in memory: LoadRowV8), are multiplied with
// v_mfma_f32_32x32x16_bf16 (8 k per lane per operand) and accumulated in fp32.  LDS slabs are [k/8][row] of
// 16-byte groups, double buffered: a loader writes one ds_write_b128 per 8 values and an MFMA operand is one
// ds_read_b128.
// ------------------------------------------------------------------------------------------
template <class T, class AL, class BL, bool NCHW, class PASS, bool PK = false>
__global__ __launch_bounds__(T::NT, T::OCC) void mfma_gemm_bf16_kernel(typename AL::Params ap,
                                                                       typename BL::Params bp, EpiParams ep,
                                                                       int tiles_m, int k_chunks,
                                                                       int chunks_per_split, PackedOut pk) {
  constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN;
  static_assert(BK % 16 == 0, "one bf16 MFMA contracts 16 k");
  constexpr int KG = BK / 8;  // 16-byte groups per row and K step
  extern __shared__ float lds_dyn[];
  uint4* const sA_base = reinterpret_cast<uint4*>(lds_dyn);  // [2][KG][BM]
  uint4* const sB_base = sA_base + 2 * KG * BM;              // [2][KG][BN]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;

  const int tiles = gridDim.x;
  const int linear = xcd_remap(blockIdx.y * tiles + blockIdx.x, tiles * gridDim.y);
  const int split_idx = __builtin_amdgcn_readfirstlane(linear / tiles);
  const int logical = __builtin_amdgcn_readfirstlane(linear - split_idx * tiles);
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int c_begin = split_idx * chunks_per_split;
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

  typename AL::Reg ra[AL::CNT];
  typename BL::Reg rb[BL::CNT];
  if (nk > 0) {
    la.prep(c_begin * BK);
    lb.prep(c_begin * BK);
#pragma unroll
    for (int i = 0; i < AL::CNT; ++i) ra[i] = la.load_one(i);
#pragma unroll
    for (int i = 0; i < BL::CNT; ++i) rb[i] = lb.load_one(i);
    la.store_bf16(sA_base, ra);
    lb.store_bf16(sB_base, rb);
  }
  if (nk > 1) {
    la.prep((c_begin + 1) * BK);
    lb.prep((c_begin + 1) * BK);
  }
  __syncthreads();

  const int a_rd = (lane >> 5) * BM + wm * (TM * 32) + (lane & 31);
  const int b_rd = (lane >> 5) * BN + wn * (TN * 32) + (lane & 31);

  auto k_step = [&](int it, auto more_tag) {
    constexpr bool MORE = decltype(more_tag)::value;
    const int cur = it & 1;
    if (MORE) {
#pragma unroll
      for (int i = 0; i < AL::CNT; ++i) ra[i] = la.load_one(i);
#pragma unroll
      for (int i = 0; i < BL::CNT; ++i) rb[i] = lb.load_one(i);
    }
    const uint4* pa = sA_base + cur * (KG * BM) + a_rd;
    const uint4* pb = sB_base + cur * (KG * BN) + b_rd;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8_t a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = __builtin_bit_cast(bf16x8_t, pa[(2 * ks) * BM + i * 32]);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = __builtin_bit_cast(bf16x8_t, pb[(2 * ks) * BN + j * 32]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (MORE) {
      if (it + 2 < nk) {  // all loads of the next step are issued: the offsets of the one after can be fetched
        la.prep((c_begin + it + 2) * BK);
        lb.prep((c_begin + it + 2) * BK);
      }
      la.store_bf16(sA_base + (cur ^ 1) * (KG * BM), ra);
      lb.store_bf16(sB_base + (cur ^ 1) * (KG * BN), rb);
    }
    __syncthreads();
  };
  for (int it = 0; it + 1 < nk; ++it) k_step(it, std::true_type());
  if (nk > 0) k_step(nk - 1, std::false_type());

  if constexpr (PK) store_tile_packed<T>(acc, ep, pk, m0, n0, wm, wn, lane);
  else store_tile<T, NCHW>(acc, ep, m0, n0, wm, wn, lane, ep.split_stride != 0 ? split_idx : -1);
}

// ------------------------------------------------------------------------------------------
// The bf16 kernel for operands that are already packed in memory (RowV8Params on both sides), with the operand slabs
// brought into a ring of four LDS buffers by direct global -> LDS loads (buffer_load_dwordx4 ... lds: lane l's 16
// bytes land at M0 + 16 l, which is exactly 64 neighbouring rows of one 8-k group of a [k/8][row] slab).
//
// Why: through registers (global load, then ds_write_b128) the LDS accepts about 70 bytes per clock and CU, and a
// wave that issues its writes stalls while the queue is full, so the writes of a step stand in front of its MFMAs
// instead of under them; and a 128x128 tile needs 64 bytes per clock of such fill at full MFMA rate, which is all
// the path has.  A 256x256 tile halves the fill per MFMA, the direct loads need no registers, no ds_write and no
// issue slots beyond the load itself, and they complete in the background.
//
// Ring of R buffers, loads issued D = R - 1 steps ahead.  Step `it` of a wave: multiplies out of buffer it; issues
// the loads of step it+D into buffer it+D (= it-1 mod R, read for the last time before the barrier of step it-1);
// in front of its last group of MFMAs waits until only the loads of steps it+2 .. it+D are still in flight,
// meets the other waves at the step's one barrier, and reads the first operands of step it+1 (whose buffer is now
// complete for every wave) under that last group.  A load therefore has D - 1/2 steps to land (2.5 with a ring of
// four), and nothing the matrix pipe has to wait for follows a barrier: with the barrier at the end of the step and
// two steps to land the same loop was 14 % slower on 256 x 2400 x 186624.
// The compiler does not see these loads (inline asm): their completion is counted by hand (vmcnt is in order),
// and no other vector memory instruction is issued between the prologue and the epilogue.
// Shapes: 256 x 256 with eight waves and a ring of four (128 KB: one block per CU, so the first loads and the
// stores of a tile are not hidden behind another block: long contractions on large grids), or 256 x 128 with four
// waves and a ring of three (72 KB: two blocks per CU).
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// (M0 is a reserved register to the compiler, which warns about it in a clobber list; on this target it does not
// keep values of its own there across statements, LDS instructions need no M0.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_load16(u32x4 rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory", "m0");
}
#pragma clang diagnostic pop
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// RowV8Params operand loaded straight into an LDS slab.  Thread -> (row, groups) as in LoadRowV8; a wave covers 64
// neighbouring rows of each of its groups.  Two sets of group offsets: the loads of a step use `so` while `so_next`
// is being fetched for the step after.
template <int ROWS, int BK, int NT, bool LINEAR>
struct DmaRowV8 {
  static constexpr int KG = BK / 8;
  static constexpr int CNT = ROWS * KG / NT;
  static_assert(BK % 8 == 0 && NT % ROWS == 0 && (ROWS * KG) % NT == 0 && ROWS % kWave == 0, "loader shape");
  typedef RowV8Params Params;
  typedef const __attribute__((address_space(4))) int* ctab_t;
  u32x4 rsrc;
  const int* tab;
  uint32_t vbase;
  int g0, wrow, gstride;
  int so[CNT], so_next[CNT];

  __device__ __forceinline__ void init(const Params& p, int row0, int tid) {
    const uint64_t a = reinterpret_cast<uint64_t>(p.ptr);
    rsrc.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
    rsrc.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    rsrc.z = __builtin_amdgcn_readfirstlane(p.bytes);
    rsrc.w = 0x00020000u;
    const int row = tid % ROWS;
    wrow = __builtin_amdgcn_readfirstlane((tid & ~(kWave - 1)) % ROWS);
    g0 = __builtin_amdgcn_readfirstlane(tid / ROWS) * CNT;
    tab = p.soff;
    gstride = p.group_stride;
    const int m = row0 + row;
    const bool valid = m < p.M;
    const int mm = valid ? m : 0;
    const int n = mm / p.inner;
    const int rem = mm - n * p.inner;
    const int a2 = rem / p.innerW;
    const int b2 = rem - a2 * p.innerW;
    vbase = valid ? (uint32_t)(n * p.img_stride + a2 * p.a_stride + b2 * p.b_stride) : 0x80000000u;
  }
  // The table is read through the constant address space: scalar loads, which the hand-counted vmcnt of the
  // direct loads does not see.  (As a global load it becomes a vector load, since the asm statements may write
  // memory for all the compiler knows, and the wait for it would also wait for every direct load in flight.)
  __device__ __forceinline__ int group_off(int k0, int i) const {
    return LINEAR ? ((k0 >> 3) + g0 + i) * gstride : ((ctab_t)(uintptr_t)tab)[(k0 >> 3) + g0 + i];
  }
  __device__ __forceinline__ void prep(int k0) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so[i] = group_off(k0, i);
  }
  __device__ __forceinline__ void prep_next(int k0) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so_next[i] = group_off(k0, i);
  }
  __device__ __forceinline__ void rotate() {
#pragma unroll
    for (int i = 0; i < CNT; ++i) so[i] = so_next[i];
  }
  // slab_addr: LDS byte address of the [KG][ROWS] slab of 16-byte groups
  __device__ __forceinline__ void issue(uint32_t slab_addr) const {
#pragma unroll
    for (int i = 0; i < CNT; ++i)
      dma_load16(rsrc, slab_addr + (uint32_t)((g0 + i) * ROWS + wrow) * 16u, vbase, (uint32_t)so[i]);
  }
};

template <class T, bool A_LINEAR, bool B_LINEAR, bool NCHW, class PASS, bool PK = false, int R = 4>
__global__ __launch_bounds__(T::NT, T::OCC) void mfma_gemm_bf16_dma_kernel(RowV8Params ap, RowV8Params bp, EpiParams ep,
                                                                           int tiles_m, int k_chunks, PackedOut pk) {
  constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN;
  static_assert(BK % 32 == 0, "an even number of 16-k groups per step keeps the operand register sets in phase");
  typedef DmaRowV8<BM, BK, T::NT, A_LINEAR> AL;
  typedef DmaRowV8<BN, BK, T::NT, B_LINEAR> BL;
  constexpr int KG = BK / 8, STEPS = BK / 16, D = R - 1;  // D: how many steps ahead the loads are issued
  static_assert(R >= 3, "the ring holds the step being read, one landed or landing, and one in flight at least");
  constexpr int SA = KG * BM, SB = KG * BN;  // 16-byte groups per buffer
  extern __shared__ float lds_dyn[];
  uint4* const sA_base = reinterpret_cast<uint4*>(lds_dyn);  // [R][KG][BM]
  uint4* const sB_base = sA_base + R * SA;                   // [R][KG][BN]
  const uint32_t ldsA = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)sA_base;
  const uint32_t ldsB = ldsA + R * SA * 16;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;

  const int logical = __builtin_amdgcn_readfirstlane(xcd_remap(blockIdx.x, gridDim.x));
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int nk = k_chunks;

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

  auto prep_step = [&](int s) {
    la.prep(s * BK);
    lb.prep(s * BK);
  };
  auto issue_step = [&](int buf) {
    la.issue(ldsA + (uint32_t)(buf * SA) * 16u);
    lb.issue(ldsB + (uint32_t)(buf * SB) * 16u);
  };
  // steps 0..D-1 on their way, the offsets of step D fetched
#pragma unroll
  for (int s = 0; s < D; ++s)
    if (s < nk) { prep_step(s); issue_step(s); }
  if (nk > D) prep_step(D);
  wait_vmcnt<0>();
  __syncthreads();

  const int a_rd = (lane >> 5) * BM + wm * (TM * 32) + (lane & 31);
  const int b_rd = (lane >> 5) * BN + wn * (TN * 32) + (lane & 31);
  uint4 a[2][TM], b[2][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a[0][i] = sA_base[a_rd + i * 32];
#pragma unroll
  for (int j = 0; j < TN; ++j) b[0][j] = sB_base[b_rd + j * 32];
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the loop is entered with nothing in flight, so its waits can be exact

  auto step = [&](int it, auto more_tag) {
    constexpr bool MORE = decltype(more_tag)::value;  // this step issues the loads of step it+D
    const int rd = it % R, nx = (it + 1) % R;
    const uint4* pa = sA_base + rd * SA + a_rd;
    const uint4* pb = sB_base + rd * SB + b_rd;
    const uint4* pna = sA_base + nx * SA + a_rd;
    const uint4* pnb = sB_base + nx * SB + b_rd;
#pragma unroll
    for (int g = 0; g < STEPS; ++g) {
      const int c = g & 1, n = c ^ 1;
      __builtin_amdgcn_sched_barrier(0);
      // Everything this wave has asked of the LDS and of the scalar cache was issued at least a group of MFMAs
      // ago: an explicit wait here costs nothing, and it lets the wait in front of this group's MFMAs disappear
      // (otherwise that one, being a wait for "everything" because scalar loads return out of order, would also
      // cover the operand reads issued just before it).
      __builtin_amdgcn_s_waitcnt(0xc07f);
      if (MORE && g == 0) {
        // the offsets of step it+D+1 (used by the loads the next step issues), fetched first for the same reason
        const int s4 = it + D + 1 < nk ? it + D + 1 : nk - 1;
        la.prep_next(s4 * BK);
        lb.prep_next(s4 * BK);
      }
      if (g + 1 < STEPS) {
#pragma unroll
        for (int i = 0; i < TM; ++i) a[n][i] = pa[(2 * g + 2) * BM + i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[n][j] = pb[(2 * g + 2) * BN + j * 32];
      } else {
        // The step's one barrier stands here, in front of its last group of MFMAs.  Every wave has read all it
        // needs of buffer `it` (the wait above), so the loads the next step issues may overwrite it; and with
        // only the loads of steps it+2 .. it+D allowed in flight, buffer it+1 is complete once all waves are
        // past: its first operands are read under this group's MFMAs.  A load has D - 1/STEPS steps to land.
        // (After the last step this reads a buffer nobody uses: harmless.)
        if (MORE) wait_vmcnt<(R - 2) * (AL::CNT + BL::CNT)>();
        else wait_vmcnt<0>();
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TM; ++i) a[n][i] = pna[i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[n][j] = pnb[j * 32];
      }
      if (MORE && g == 0) issue_step((it + D) % R);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[c][i]),
                                                              __builtin_bit_cast(bf16x8_t, b[c][j]), acc[i][j], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (MORE) {
      la.rotate();
      lb.rotate();
    }
  };
  int it = 0;
  for (; it + D < nk; ++it) step(it, std::true_type());
  for (; it < nk; ++it) step(it, std::false_type());

  if constexpr (PK) store_tile_packed<T>(acc, ep, pk, m0, n0, wm, wn, lane);
  else store_tile<T, NCHW>(acc, ep, m0, n0, wm, wn, lane, -1);
}

}  // namespace rh
