// Context, device memory, error strings and the host-side seeded generator.
#include <math.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <thread>
#include <string>
#include <cstring>
#include <vector>

#include "common.h"

struct rh_ctx {
  int device;
  hipStream_t stream;
  // second stream for work that may overlap the main stream's (created on first use), and the two events
  // that order the streams against each other
  hipStream_t aux = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  bool aux_dirty = false;   // the second stream was given work (fork) that the main stream has not waited for yet
  bool capturing = false;   // between rh_ctx_begin_capture and rh_ctx_end_capture
  // copy stream for host -> device loads that run beside the main stream's kernels (created on first use)
  hipStream_t copy = nullptr;
  hipEvent_t ev_copied = nullptr, ev_consumed = nullptr;
  bool consumed_valid = false;  // ev_consumed was recorded after the last reader of the buffer loaded that way
  // device -> host stores on the copy stream (rh_store_begin / rh_store_wait)
  hipEvent_t ev_store_ready = nullptr, ev_stored = nullptr;
  bool store_pending = false;
};

// The copy stream and its events, created on first use.
static hipError_t ensure_copy_stream(rh_ctx* ctx) {
  if (ctx->copy) return hipSuccess;
  hipError_t e;
  if ((e = hipSetDevice(ctx->device)) != hipSuccess) return e;
  hipStream_t s = nullptr;
  hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
  if ((e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking)) != hipSuccess) return e;  // default priority
  for (int i = 0; i < 4; ++i)
    if ((e = hipEventCreateWithFlags(&ev[i], hipEventDisableTiming)) != hipSuccess) {
      for (int j = 0; j < i; ++j) (void)hipEventDestroy(ev[j]);
      (void)hipStreamDestroy(s);
      return e;
    }
  ctx->copy = s; ctx->ev_copied = ev[0]; ctx->ev_consumed = ev[1]; ctx->ev_store_ready = ev[2]; ctx->ev_stored = ev[3];
  return hipSuccess;
}

// A captured and instantiated sequence of launches of one context (both streams).
struct rh_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

using namespace rh;

// RH_SOURCE_HASH: a hash over the library's sources, set by the build (rembrandt_amd/build.py); summaries of measured
// runs quote it, so that a reader can tell whether they describe the library at hand.
#ifndef RH_SOURCE_HASH
#define RH_SOURCE_HASH "unknown"
#endif
extern "C" const char* rh_version(void) { return "rembrandt-hip 0.1 (gfx950, fp32 MFMA) src " RH_SOURCE_HASH; }

extern "C" const char* rh_error_string(int code) {
  switch (code) {
    case 0: return "ok";
    case RH_E_INVALID: return "invalid argument";
    case RH_E_WORKSPACE: return "workspace missing, misaligned or too small";
    case RH_E_UNSUPPORTED: return "unsupported option";
    case RH_E_LIMIT: return "size beyond a documented limit";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown error";
  }
}

extern "C" int rh_ctx_create(int device, rh_ctx** out) {
  if (!out) return RH_E_INVALID;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess) return (int)e;
  if (device < 0 || device >= count) return RH_E_INVALID;
  if ((e = hipSetDevice(device)) != hipSuccess) return (int)e;
  // set-up of the entry point that must not allocate: the address of the static scratch array on this device
  if (int se = rh::static_scratch_lookup(nullptr)) return se;
  rh_ctx* c = new rh_ctx;
  c->device = device;
  // default priority, non-blocking with respect to the legacy default stream
  if ((e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking)) != hipSuccess) { delete c; return (int)e; }
  *out = c;
  return 0;
}

extern "C" int rh_ctx_destroy(rh_ctx* ctx) {
  if (!ctx) return RH_E_INVALID;
  if (ctx->aux) {
    (void)hipStreamSynchronize(ctx->aux);
    (void)hipStreamDestroy(ctx->aux);
    (void)hipEventDestroy(ctx->ev_fork);
    (void)hipEventDestroy(ctx->ev_join);
  }
  if (ctx->copy) {
    (void)hipStreamSynchronize(ctx->copy);
    (void)hipStreamDestroy(ctx->copy);
    (void)hipEventDestroy(ctx->ev_copied);
    (void)hipEventDestroy(ctx->ev_consumed);
    (void)hipEventDestroy(ctx->ev_store_ready);
    (void)hipEventDestroy(ctx->ev_stored);
  }
  hipError_t e = hipStreamSynchronize(ctx->stream);
  hipError_t e2 = hipStreamDestroy(ctx->stream);
  delete ctx;
  return (int)(e != hipSuccess ? e : e2);
}

extern "C" rh_stream_t rh_ctx_stream(rh_ctx* ctx) { return ctx ? (rh_stream_t)ctx->stream : nullptr; }

extern "C" int rh_ctx_sync(rh_ctx* ctx) {
  if (!ctx) return RH_E_INVALID;
  if (ctx->aux) {
    hipError_t e = hipStreamSynchronize(ctx->aux);
    if (e != hipSuccess) return (int)e;
  }
  hipError_t e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) return (int)e;
  if (ctx->copy) {  // after the main stream: a store begun with rh_store_begin waits for a point of it
    if ((e = hipStreamSynchronize(ctx->copy)) != hipSuccess) return (int)e;
    ctx->store_pending = false;
  }
  return 0;
}

extern "C" rh_stream_t rh_ctx_aux_stream(rh_ctx* ctx) {
  if (!ctx) return nullptr;
  if (!ctx->aux) {
    if (hipSetDevice(ctx->device) != hipSuccess) return nullptr;
    hipStream_t s = nullptr;
    hipEvent_t a = nullptr, b = nullptr;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) return nullptr;  // default priority
    if (hipEventCreateWithFlags(&a, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&b, hipEventDisableTiming) != hipSuccess) {
      (void)hipStreamDestroy(s);
      if (a) (void)hipEventDestroy(a);
      return nullptr;
    }
    ctx->aux = s; ctx->ev_fork = a; ctx->ev_join = b;
  }
  ctx->aux_dirty = true;  // whoever asked for the stream may put work on it
  return (rh_stream_t)ctx->aux;
}

// Work enqueued on the second stream after this call runs after everything the main stream holds now.
extern "C" int rh_ctx_fork(rh_ctx* ctx) {
  if (!ctx || !rh_ctx_aux_stream(ctx)) return RH_E_INVALID;
  hipError_t e = hipEventRecord(ctx->ev_fork, ctx->stream);
  if (e != hipSuccess) return (int)e;
  ctx->aux_dirty = true;
  return (int)hipStreamWaitEvent(ctx->aux, ctx->ev_fork, 0);
}

// Work enqueued on the main stream after this call runs after everything the second stream holds now.
extern "C" int rh_ctx_join(rh_ctx* ctx) {
  if (!ctx) return RH_E_INVALID;
  if (!ctx->aux || !ctx->aux_dirty) return 0;  // nothing was forked since the last join
  hipError_t e = hipEventRecord(ctx->ev_join, ctx->aux);
  if (e != hipSuccess) return (int)e;
  ctx->aux_dirty = false;
  return (int)hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0);
}

// ---- stream capture: a launch-bound sequence (a whole train step of a small network) recorded once and replayed ----
// Between begin and end every launch on the context's streams is recorded instead of executed; the second stream
// joins the recording through rh_ctx_fork and must have been joined again (rh_ctx_join) before the end.  Only kernel
// launches and device-to-device copies may be recorded: no host copies, synchronisation, allocation or memset calls.
extern "C" int rh_ctx_begin_capture(rh_ctx* ctx) {
  if (!ctx || ctx->capturing) return RH_E_INVALID;
  if (ctx->aux_dirty) {  // work forked before the recording must not leak into it
    if (int e = rh_ctx_join(ctx)) return e;
  }
  hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) return (int)e;
  ctx->capturing = true;
  return 0;
}

// Ends the recording; with `out` the graph is instantiated and returned, without it the recording is discarded
// (the way out of a sequence that failed half-way).
extern "C" int rh_ctx_end_capture(rh_ctx* ctx, rh_graph** out) {
  if (!ctx || !ctx->capturing) return RH_E_INVALID;
  ctx->capturing = false;
  if (out) *out = nullptr;
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g);
  ctx->aux_dirty = false;
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return (int)e;
  }
  if (!out) {
    if (g) (void)hipGraphDestroy(g);
    return 0;
  }
  hipGraphExec_t x = nullptr;
  e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    return (int)e;
  }
  rh_graph* r = new rh_graph;
  r->graph = g;
  r->exec = x;
  *out = r;
  return 0;
}

extern "C" int rh_graph_launch(rh_graph* g, rh_ctx* ctx) {
  if (!g || !ctx || ctx->capturing) return RH_E_INVALID;
  ctx->consumed_valid = false;  // the recorded launches may read a buffer that rh_load_overlapped fills
  return (int)hipGraphLaunch(g->exec, ctx->stream);
}

extern "C" int rh_graph_destroy(rh_graph* g) {
  if (!g) return RH_E_INVALID;
  hipError_t e = hipGraphExecDestroy(g->exec);
  hipError_t e2 = hipGraphDestroy(g->graph);
  delete g;
  return (int)(e != hipSuccess ? e : e2);
}

extern "C" int rh_malloc(rh_ctx* ctx, size_t bytes, void** dptr) {
  if (!ctx || !dptr) return RH_E_INVALID;
  *dptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipMalloc(dptr, bytes);
  if (e != hipSuccess) return (int)e;
  // zero with a fill kernel on the context's stream (buffers start as DeviceBuffer::zeros does)
  const size_t words = bytes / 4;
  if (words) {
    if (int r = rh_memset_f32(static_cast<float*>(*dptr), 0.0f, words, (rh_stream_t)ctx->stream)) return r;
  }
  if (bytes % 4) {
    e = hipMemsetAsync(static_cast<char*>(*dptr) + words * 4, 0, bytes % 4, ctx->stream);
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}

extern "C" int rh_free(rh_ctx* ctx, void* dptr) {
  if (!ctx) return RH_E_INVALID;
  if (!dptr) return 0;
  hipError_t e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) return (int)e;
  return (int)hipFree(dptr);
}

// Page-locked host memory for buffers that are copied to the device every batch (the input frames): copies from it
// run at the link's rate and need no staging copy inside the driver.  Zero-filled.
extern "C" int rh_host_malloc(rh_ctx* ctx, size_t bytes, void** hptr) {
  if (!ctx || !hptr) return RH_E_INVALID;
  *hptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipHostMalloc(hptr, bytes, hipHostMallocDefault);
  if (e != hipSuccess) return (int)e;
  memset(*hptr, 0, bytes);
  return 0;
}

extern "C" int rh_host_free(rh_ctx* ctx, void* hptr) {
  if (!ctx) return RH_E_INVALID;
  if (!hptr) return 0;
  hipError_t e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) return (int)e;
  return (int)hipHostFree(hptr);
}

extern "C" int rh_copy_d2d(void* dst, const void* src, size_t bytes, rh_stream_t stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return RH_E_INVALID;
  return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, to_stream(stream));
}

extern "C" int rh_load_sync(rh_ctx* ctx, void* dst_d, const void* src_h, size_t bytes) {
  if (!ctx) return RH_E_INVALID;
  if (bytes == 0) return 0;
  if (!dst_d || !src_h) return RH_E_INVALID;
  hipError_t e = hipMemcpyAsync(dst_d, src_h, bytes, hipMemcpyHostToDevice, ctx->stream);
  if (e != hipSuccess) return (int)e;
  return (int)hipStreamSynchronize(ctx->stream);
}

// Host -> device load that does not wait for the main stream's queued kernels: the copy runs on a stream of its own,
// after the last reader of dst_d that rh_mark_consumed recorded, and the main stream's later work waits for it.
// Returns when the copy is complete (src_h may be reused), like rh_load_sync.  Without a valid consumed mark (none
// recorded yet, or the readers were launched inside a recording or a graph replay) it first waits for the main stream.
extern "C" int rh_load_overlapped(rh_ctx* ctx, void* dst_d, const void* src_h, size_t bytes) {
  if (!ctx) return RH_E_INVALID;
  if (bytes == 0) return 0;
  if (!dst_d || !src_h) return RH_E_INVALID;
  if (ctx->capturing) return RH_E_UNSUPPORTED;
  hipError_t e;
  if ((e = ensure_copy_stream(ctx)) != hipSuccess) return (int)e;
  if (ctx->consumed_valid) {
    if ((e = hipStreamWaitEvent(ctx->copy, ctx->ev_consumed, 0)) != hipSuccess) return (int)e;
  } else if ((e = hipStreamSynchronize(ctx->stream)) != hipSuccess) {
    return (int)e;
  }
  ctx->consumed_valid = false;  // the next readers have to be marked again
  if ((e = hipMemcpyAsync(dst_d, src_h, bytes, hipMemcpyHostToDevice, ctx->copy)) != hipSuccess) return (int)e;
  if ((e = hipEventRecord(ctx->ev_copied, ctx->copy)) != hipSuccess) return (int)e;
  if ((e = hipStreamWaitEvent(ctx->stream, ctx->ev_copied, 0)) != hipSuccess) return (int)e;
  return (int)hipStreamSynchronize(ctx->copy);
}

// Marks the point of the main stream after which the buffer last filled by rh_load_overlapped is no longer read.
// Inside a recording nothing is marked (the recorded readers run at replay time, unknown to the host).
extern "C" int rh_mark_consumed(rh_ctx* ctx) {
  if (!ctx) return RH_E_INVALID;
  if (ctx->capturing || !ctx->copy) { ctx->consumed_valid = false; return 0; }
  hipError_t e = hipEventRecord(ctx->ev_consumed, ctx->stream);
  if (e != hipSuccess) return (int)e;
  ctx->consumed_valid = true;
  return 0;
}

extern "C" int rh_store_sync(rh_ctx* ctx, void* dst_h, const void* src_d, size_t bytes) {
  if (!ctx) return RH_E_INVALID;
  if (bytes == 0) return 0;
  if (!dst_h || !src_d) return RH_E_INVALID;
  hipError_t e = hipMemcpyAsync(dst_h, src_d, bytes, hipMemcpyDeviceToHost, ctx->stream);
  if (e != hipSuccess) return (int)e;
  return (int)hipStreamSynchronize(ctx->stream);
}

// sync_store in two halves.  rh_store_begin: the copy runs on the copy stream once everything the main stream holds
// now is complete; the main stream itself does not wait for it, so launches made after this call run on while the
// copy is under way.  rh_store_wait: blocks the host until every copy begun so far has landed.  The caller keeps
// src_d unchanged between the two (launches enqueued in between must not write it) and passes page-locked host
// memory (rh_host_malloc): with pageable memory the runtime may block inside rh_store_begin.
extern "C" int rh_store_begin(rh_ctx* ctx, void* dst_h, const void* src_d, size_t bytes) {
  if (!ctx) return RH_E_INVALID;
  if (bytes == 0) return 0;
  if (!dst_h || !src_d) return RH_E_INVALID;
  if (ctx->capturing) return RH_E_UNSUPPORTED;
  hipError_t e;
  if ((e = ensure_copy_stream(ctx)) != hipSuccess) return (int)e;
  if ((e = hipEventRecord(ctx->ev_store_ready, ctx->stream)) != hipSuccess) return (int)e;
  if ((e = hipStreamWaitEvent(ctx->copy, ctx->ev_store_ready, 0)) != hipSuccess) return (int)e;
  if ((e = hipMemcpyAsync(dst_h, src_d, bytes, hipMemcpyDeviceToHost, ctx->copy)) != hipSuccess) return (int)e;
  if ((e = hipEventRecord(ctx->ev_stored, ctx->copy)) != hipSuccess) return (int)e;
  ctx->store_pending = true;
  return 0;
}

extern "C" int rh_store_wait(rh_ctx* ctx) {
  if (!ctx) return RH_E_INVALID;
  if (!ctx->store_pending) return 0;
  ctx->store_pending = false;
  return (int)hipEventSynchronize(ctx->ev_stored);
}

// ---- per-launch timing -------------------------------------------------------------------
namespace rh {

bool g_profile_enabled = false;

namespace {
struct ProfRecord { const char* tag; double work; hipEvent_t e0, e1; };
std::vector<ProfRecord*> g_records;
std::mutex g_prof_mutex;
std::string g_prof_prefix;   // when non-empty only tags that start with it are recorded
}  // namespace

ProfScope::ProfScope(const char* tag, double work, hipStream_t s) : slot(nullptr), stream(s) {
  if (!g_profile_enabled) return;
  if (!g_prof_prefix.empty() && std::strncmp(tag, g_prof_prefix.c_str(), g_prof_prefix.size()) != 0) return;
  ProfRecord* r = new ProfRecord{tag, work, nullptr, nullptr};
  if (hipEventCreate(&r->e0) != hipSuccess || hipEventCreate(&r->e1) != hipSuccess) { delete r; return; }
  (void)hipEventRecord(r->e0, s);
  slot = r;
}

ProfScope::~ProfScope() {
  if (!slot) return;
  ProfRecord* r = static_cast<ProfRecord*>(slot);
  (void)hipEventRecord(r->e1, stream);
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_records.push_back(r);
}

}  // namespace rh

extern "C" int rh_profile_enabled(void) { return rh::g_profile_enabled ? 1 : 0; }

extern "C" int rh_profile_enable(int on) {
  rh::g_profile_enabled = on != 0;
  return 0;
}

extern "C" int rh_profile_filter(const char* prefix) {
  std::lock_guard<std::mutex> lock(rh::g_prof_mutex);
  rh::g_prof_prefix = prefix ? prefix : "";
  return 0;
}

extern "C" int rh_profile_count(void) {
  std::lock_guard<std::mutex> lock(rh::g_prof_mutex);
  return (int)rh::g_records.size();
}

// Record i: tag, algorithmic work, elapsed milliseconds (waits for the record's end event).
extern "C" int rh_profile_get(int i, const char** tag, double* work, float* ms) {
  std::lock_guard<std::mutex> lock(rh::g_prof_mutex);
  if (i < 0 || i >= (int)rh::g_records.size() || !tag || !work || !ms) return RH_E_INVALID;
  rh::ProfRecord* r = rh::g_records[(size_t)i];
  hipError_t e = hipEventSynchronize(r->e1);
  if (e != hipSuccess) return (int)e;
  if ((e = hipEventElapsedTime(ms, r->e0, r->e1)) != hipSuccess) return (int)e;
  *tag = r->tag;
  *work = r->work;
  return 0;
}

extern "C" int rh_profile_reset(void) {
  std::lock_guard<std::mutex> lock(rh::g_prof_mutex);
  for (rh::ProfRecord* r : rh::g_records) {
    (void)hipEventDestroy(r->e0);
    (void)hipEventDestroy(r->e1);
    delete r;
  }
  rh::g_records.clear();
  return 0;
}

// ---- seeded generator --------------------------------------------------------------------
namespace {

inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
inline uint64_t stream_key(uint64_t seed, uint64_t stream_id) {
  return mix64(seed ^ mix64(stream_id + 0x9E3779B97F4A7C15ull));
}
inline uint64_t draw(uint64_t key, uint64_t i) { return mix64(key + (i + 1) * 0x9E3779B97F4A7C15ull); }

template <class F>
void parallel_for(size_t n, F f) {
  unsigned hw = std::thread::hardware_concurrency();
  size_t nt = std::min<size_t>(hw ? hw : 1, 16);
  if (n < (size_t)1 << 16) nt = 1;
  if (nt <= 1) { f(0, n); return; }
  std::vector<std::thread> th;
  const size_t chunk = (n + nt - 1) / nt;
  for (size_t t = 0; t < nt; ++t) {
    const size_t b = t * chunk, e = std::min(n, b + chunk);
    if (b < e) th.emplace_back(f, b, e);
  }
  for (auto& t : th) t.join();
}

}  // namespace

extern "C" int rh_rng_fill_uniform(uint64_t seed, uint64_t stream_id, float* host, size_t n, float lo, float hi) {
  if (n && !host) return RH_E_INVALID;
  const uint64_t key = stream_key(seed, stream_id);
  parallel_for(n, [=](size_t b, size_t e) {
    for (size_t i = b; i < e; ++i) {
      const float u = (float)(draw(key, i) >> 40) * (1.0f / 16777216.0f);  // 24 bits: exact, in [0,1)
      host[i] = lo + (hi - lo) * u;
    }
  });
  return 0;
}

extern "C" int rh_rng_fill_normal(uint64_t seed, uint64_t stream_id, float* host, size_t n, float mean, float std) {
  if (n && !host) return RH_E_INVALID;
  const uint64_t key = stream_key(seed, stream_id);
  parallel_for(n, [=](size_t b, size_t e) {
    for (size_t i = b; i < e; ++i) {
      // Box-Muller in double from two 53-bit uniforms; u1 in (0,1], u2 in [0,1)
      const double u1 = (double)((draw(key, 2 * i) >> 11) + 1) * (1.0 / 9007199254740992.0);
      const double u2 = (double)(draw(key, 2 * i + 1) >> 11) * (1.0 / 9007199254740992.0);
      const double r = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
      host[i] = (float)((double)mean + (double)std * r);
    }
  });
  return 0;
}

extern "C" int rh_rng_fill_int(uint64_t seed, uint64_t stream_id, int32_t* host, size_t n, int32_t modulus) {
  if ((n && !host) || modulus <= 0) return RH_E_INVALID;
  const uint64_t key = stream_key(seed, stream_id);
  for (size_t i = 0; i < n; ++i) host[i] = (int32_t)(draw(key, i) % (uint64_t)modulus);
  return 0;
}
