// Kernels either side of the operator chain: input preprocessing of the Data3d operator (crop, x-flip,
// PCA lighting noise), dropout, the device form of the seeded uniform generator, and cross-channel
// local response normalisation.  All are bandwidth-bound maps; index arithmetic uses FastDiv.
#include "common.h"

namespace rh {

// dst[p][h][w] = src[p][offH + h][offW + w] for p < planes (planes = batch * channels).
__global__ void crop_kernel(const float* __restrict__ src, float* __restrict__ dst, long long total, int inW, int inH,
                            int cropW, int offW, int offH, FastDiv dCropW, FastDiv dCropHW) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    uint32_t p, rem, h, w;
    dCropHW.divmod((uint32_t)i, p, rem);
    dCropW.divmod(rem, h, w);
    dst[i] = src[((size_t)p * inH + (offH + h)) * inW + (offW + w)];
  }
}

// dst[r][w] = src[r][width - 1 - w] for r < rows.
__global__ void flip_rows_kernel(const float* __restrict__ src, float* __restrict__ dst, long long total, int width,
                                 FastDiv dW) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    uint32_t r, w;
    dW.divmod((uint32_t)i, r, w);
    dst[i] = src[(size_t)r * width + (width - 1 - w)];
  }
}

// dst[n][c][i] = src[n][c][i] + sum_j svecs[j*3 + c] * (alphas[n*3 + j] * svals[j]),  c < 3.
__global__ void pca3_noise_kernel(const float* __restrict__ src, int spatial, int batch,
                                  const float* __restrict__ alphas, const float* __restrict__ svals,
                                  const float* __restrict__ svecs, float* __restrict__ dst) {
  const int nc = blockIdx.y;  // n*3 + c
  const int n = nc / 3, c = nc - n * 3;
  float shift = 0.0f;
  for (int j = 0; j < 3; ++j) shift += svecs[j * 3 + c] * (alphas[n * 3 + j] * svals[j]);
  const float* s = src + (size_t)nc * spatial;
  float* d = dst + (size_t)nc * spatial;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < spatial; i += gridDim.x * blockDim.x) d[i] = s[i] + shift;
}

// mask = rand > ratio; out = scale * in where kept, 0 where dropped.
__global__ void dropout_kernel(const float* __restrict__ in, long long n, float ratio, float scale,
                               const float* __restrict__ rnd, float* __restrict__ out, int* __restrict__ mask) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int keep = rnd[i] > ratio ? 1 : 0;
    mask[i] = keep;
    out[i] = keep ? scale * in[i] : 0.0f;
  }
}

__global__ void dropout_backprop_kernel(const float* __restrict__ out_delta, long long n, float scale,
                                        const int* __restrict__ mask, float* __restrict__ in_delta) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    in_delta[i] = mask[i] ? scale * out_delta[i] : 0.0f;
}

__device__ __forceinline__ uint64_t dev_mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// dst[i] = 24-bit uniform in [0,1) number (first + i) of the stream with this key: the same value the
// host generator gives for that index.
__global__ void uniform01_kernel(uint64_t key, uint64_t first, float* __restrict__ dst, long long n) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t z = dev_mix64(key + (first + (uint64_t)i + 1) * 0x9E3779B97F4A7C15ull);
    dst[i] = (float)(z >> 40) * (1.0f / 16777216.0f);
  }
}

// Cross-channel local response normalisation, one thread per (n, pixel) walking the channels:
// d[c] = min_div + scale * sum_{c' in win(c)} x[c']^2,  y[c] = x[c] * d[c]^-power,
// win(c) = [c - size/2, c + (size-1)/2] clipped to the channel range.  d is kept for the backward pass.
__global__ void lrn_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, float* __restrict__ denom,
                               long long pixels, int C, int plane, int size, float scale, float power, float min_div,
                               FastDiv dPlane) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const int lo = size / 2, hi = (size - 1) / 2;
  for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t < pixels; t += stride) {
    uint32_t n, i;
    dPlane.divmod((uint32_t)t, n, i);
    const float* px = x + ((size_t)n * C) * plane + i;
    float* py = y + ((size_t)n * C) * plane + i;
    float* pd = denom + ((size_t)n * C) * plane + i;
    for (int c = 0; c < C; ++c) {
      // the window sum is recomputed per channel (no running subtraction: the result does not depend on history;
      // the re-reads hit in cache)
      float s = 0.0f;
      const int c0 = c - lo < 0 ? 0 : c - lo, c1 = c + hi >= C ? C - 1 : c + hi;
      for (int cc = c0; cc <= c1; ++cc) { const float v = px[(size_t)cc * plane]; s += v * v; }
      const float d = min_div + scale * s;
      pd[(size_t)c * plane] = d;
      py[(size_t)c * plane] = px[(size_t)c * plane] * powf(d, -power);
    }
  }
}

// dx[c] = dy[c] * d[c]^-power - 2 * scale * power * x[c] * sum_{c' : c in win(c')} dy[c'] * y[c'] / d[c'].
__global__ void lrn_bwd_kernel(const float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ denom,
                               const float* __restrict__ dy, float* __restrict__ dx, long long pixels, int C, int plane,
                               int size, float scale, float power, FastDiv dPlane) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  const int lo = size / 2, hi = (size - 1) / 2;
  for (long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x; t < pixels; t += stride) {
    uint32_t n, i;
    dPlane.divmod((uint32_t)t, n, i);
    const size_t base = ((size_t)n * C) * plane + i;
    for (int c = 0; c < C; ++c) {
      // c is in win(c') iff c' - lo <= c <= c' + hi  iff  c - hi <= c' <= c + lo
      const int c0 = c - hi < 0 ? 0 : c - hi, c1 = c + lo >= C ? C - 1 : c + lo;
      float s = 0.0f;
      for (int cc = c0; cc <= c1; ++cc) {
        const size_t o = base + (size_t)cc * plane;
        s += dy[o] * y[o] / denom[o];
      }
      const size_t o = base + (size_t)c * plane;
      dx[o] = dy[o] * powf(denom[o], -power) - 2.0f * scale * power * x[o] * s;
    }
  }
}

}  // namespace rh

using namespace rh;

namespace {
inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
}  // namespace

extern "C" int rh_crop_nchw(const float* src, float* dst, int64_t planes, int32_t in_w, int32_t in_h, int32_t crop_w,
                            int32_t crop_h, int32_t off_w, int32_t off_h, rh_stream_t stream) {
  if (planes < 0 || in_w <= 0 || in_h <= 0 || crop_w <= 0 || crop_h <= 0 || off_w < 0 || off_h < 0 ||
      off_w + crop_w > in_w || off_h + crop_h > in_h)
    return RH_E_INVALID;
  const long long total = (long long)planes * crop_w * crop_h;
  if (total == 0) return 0;
  if (!src || !dst) return RH_E_INVALID;
  if (total >= (1ll << 31) || (long long)planes * in_w * in_h >= (1ll << 31)) return RH_E_LIMIT;
  ProfScope prof("crop", 8.0 * (double)total, to_stream(stream));
  hipLaunchKernelGGL(crop_kernel, dim3(stream_grid((size_t)total, 256)), dim3(256), 0, to_stream(stream), src, dst, total,
                     in_w, in_h, crop_w, off_w, off_h, FastDiv((uint32_t)crop_w), FastDiv((uint32_t)(crop_w * crop_h)));
  return launch_status();
}

extern "C" void rembrandt_kernel_batch_blockmap256_flip(const float* src, int32_t width, int32_t rows, float* dst,
                                                        rh_stream_t stream) {
  const long long total = (long long)width * rows;
  if (width < 0 || rows < 0 || (total > 0 && (!src || !dst)) || total >= (1ll << 31)) {
    g_last_error = total >= (1ll << 31) ? RH_E_LIMIT : RH_E_INVALID;
    return;
  }
  if (total == 0) { g_last_error = 0; return; }
  ProfScope prof("flip", 8.0 * (double)total, to_stream(stream));
  hipLaunchKernelGGL(flip_rows_kernel, dim3(stream_grid((size_t)total, 256)), dim3(256), 0, to_stream(stream), src, dst,
                     total, width, FastDiv((uint32_t)width));
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_batch_map_preproc_pca3_noise(const float* src, int32_t spatial, int32_t batch,
                                                              const float* alphas, const float* svals,
                                                              const float* svecs, float* dst, rh_stream_t stream) {
  if (spatial < 0 || batch < 0 || batch > 21845) { g_last_error = RH_E_INVALID; return; }
  if (spatial == 0 || batch == 0) { g_last_error = 0; return; }
  if (!src || !alphas || !svals || !svecs || !dst) { g_last_error = RH_E_INVALID; return; }
  ProfScope prof("pca3_noise", 24.0 * (double)spatial * batch, to_stream(stream));
  const unsigned gx = (unsigned)std::min(cdiv(spatial, 256), 64);
  hipLaunchKernelGGL(pca3_noise_kernel, dim3(gx, (unsigned)batch * 3), dim3(256), 0, to_stream(stream), src, spatial,
                     batch, alphas, svals, svecs, dst);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_map_dropout(const float* in, int32_t n, float drop_ratio, float scale, const float* rnd,
                                             float* out, int32_t* mask, rh_stream_t stream) {
  if (n < 0 || (n > 0 && (!in || !rnd || !out || !mask))) { g_last_error = RH_E_INVALID; return; }
  if (n == 0) { g_last_error = 0; return; }
  ProfScope prof("dropout_fwd", 16.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(dropout_kernel, dim3(stream_grid((size_t)n, 256)), dim3(256), 0, to_stream(stream), in, (long long)n,
                     drop_ratio, scale, rnd, out, mask);
  g_last_error = launch_status();
}

extern "C" void rembrandt_kernel_map_dropout_backprop(const float* out_delta, int32_t n, float /*drop_ratio*/, float scale,
                                                      const int32_t* mask, float* in_delta, rh_stream_t stream) {
  if (n < 0 || (n > 0 && (!out_delta || !mask || !in_delta))) { g_last_error = RH_E_INVALID; return; }
  if (n == 0) { g_last_error = 0; return; }
  ProfScope prof("dropout_bwd", 12.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(dropout_backprop_kernel, dim3(stream_grid((size_t)n, 256)), dim3(256), 0, to_stream(stream),
                     out_delta, (long long)n, scale, mask, in_delta);
  g_last_error = launch_status();
}

extern "C" int rh_rng_fill_uniform01_device(uint64_t seed, uint64_t stream_id, uint64_t first, float* dst, size_t n,
                                            rh_stream_t stream) {
  if (n == 0) return 0;
  if (!dst) return RH_E_INVALID;
  const uint64_t key = mix64(seed ^ mix64(stream_id + 0x9E3779B97F4A7C15ull));
  ProfScope prof("rng_uniform01", 4.0 * (double)n, to_stream(stream));
  hipLaunchKernelGGL(uniform01_kernel, dim3(stream_grid(n, 256)), dim3(256), 0, to_stream(stream), key, first, dst,
                     (long long)n);
  return launch_status();
}

static int lrn_check(const rh_lrn_geom* g, long long* pixels) {
  if (!g || g->N < 0 || g->C <= 0 || g->H <= 0 || g->W <= 0 || g->size <= 0 || g->min_div <= 0.0f) return RH_E_INVALID;
  *pixels = (long long)g->N * g->H * g->W;
  if ((long long)g->N * g->C * g->H * g->W >= (1ll << 31)) return RH_E_LIMIT;
  return 0;
}

extern "C" int rh_lrn_fwd(const rh_lrn_geom* g, const float* x, float* y, float* denom, rh_stream_t stream) {
  long long pixels;
  if (int e = lrn_check(g, &pixels)) return e;
  if (pixels == 0) return 0;
  if (!x || !y || !denom) return RH_E_INVALID;
  const int plane = g->H * g->W;
  ProfScope prof("lrn_fwd", 12.0 * (double)pixels * g->C, to_stream(stream));
  hipLaunchKernelGGL(lrn_fwd_kernel, dim3(stream_grid((size_t)pixels, 256)), dim3(256), 0, to_stream(stream), x, y, denom,
                     pixels, g->C, plane, g->size, g->scale, g->power, g->min_div, FastDiv((uint32_t)plane));
  return launch_status();
}

extern "C" int rh_lrn_bwd(const rh_lrn_geom* g, const float* x, const float* y, const float* denom, const float* dy,
                          float* dx, rh_stream_t stream) {
  long long pixels;
  if (int e = lrn_check(g, &pixels)) return e;
  if (pixels == 0) return 0;
  if (!x || !y || !denom || !dy || !dx) return RH_E_INVALID;
  const int plane = g->H * g->W;
  ProfScope prof("lrn_bwd", 20.0 * (double)pixels * g->C, to_stream(stream));
  hipLaunchKernelGGL(lrn_bwd_kernel, dim3(stream_grid((size_t)pixels, 256)), dim3(256), 0, to_stream(stream), x, y, denom,
                     dy, dx, pixels, g->C, plane, g->size, g->scale, g->power, FastDiv((uint32_t)plane));
  return launch_status();
}
