// Host-side services behind the C ABI (see zmi_host.h).
#include "zmi_host.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <list>
#include <map>
#include <mutex>
#include <tuple>
#include <set>
#include <string>
#include <vector>

// ---- environment switches (see zmi_launch.h) ----
namespace {
const char *const kEnvNames[ZE_COUNT] = {
    "ZMI_DECODE_ROWGROUP_KERNEL",
    "ZMI_DECODE_SELFQ_MIN_WGS",
    "ZMI_DECODE_SELFQ_MAX_M",
    "ZMI_NO_DECODE_SELFQ",
    "ZMI_DECODE_NO_ROW_PAIRS",
    "ZMI_DECODE_RPW",
    "ZMI_NO_GROUP_DECODE",
    "ZMI_PERGROUP_GENERIC",
    "ZMI_NO_S4_STREAM",
    "ZMI_PRING_GRID",
    "ZMI_NO_GROUP_STREAM",
    "ZMI_WOQ_BLOCKS",
    "ZMI_DECODE_MAX_M",
    "ZMI_NO_DECODE_KERNEL",
    "ZMI_NO_DECODE_SLICED",
    "ZMI_GEMM_TOP",
    "ZMI_RING_SPLITK",
    "ZMI_PRING",
    "ZMI_RING_MIN_M",
    "ZMI_PGRING_MIN_M",
    "ZMI_NO_FUSED_QUANT",
    "ZMI_GROUP_TOP",
    "ZMI_GROUP_STREAM_TOP",
    "ZMI_GROUP_STREAM_SLICES",
    "ZMI_GROUP_DECODE",
    "ZENDNNL_LRU_CACHE_CAPACITY",
    "ZMI_NO_SLICE_ARRIVALS",
    "ZMI_NO_SIDE_STREAM",
    "ZMI_FUSED_WAIT_US",
    "ZENDNNL_DIAGNOSTICS_ENABLE",
    "ZENDNNL_MATMUL_WEIGHT_CACHE",
    "ZMI_NO_UNCACHED_FLAGS",
    "ZMI_NO_GROUP_RING_SLICES"};
struct EnvTable {
  std::string val[ZE_COUNT];
  bool set[ZE_COUNT] = {};
  bool live = false;
  void load() {
    for (int i = 0; i < ZE_COUNT; ++i) {
      const char *e = std::getenv(kEnvNames[i]);
      set[i] = e != nullptr;
      val[i] = e ? e : "";
    }
    const char *l = std::getenv("ZMI_ENV_LIVE");
    live = l && l[0] && l[0] != '0';
  }
};
EnvTable &env_table() {
  static EnvTable t = [] { EnvTable x; x.load(); return x; }();
  return t;
}
}  // namespace

const char *zmi_env(ZmiEnvVar v) {
  EnvTable &t = env_table();
  if (t.live) return std::getenv(kEnvNames[v]);
  return t.set[v] ? t.val[v].c_str() : nullptr;
}

// Reads the switches again (not while calls of other threads are in flight).
extern "C" __attribute__((visibility("default"))) void zmi_reload_env(void) { env_table().load(); }

namespace zmi {

namespace {
struct ThreadCtx {
  std::string error;
  const char *kernel = "";
  hipStream_t stream = nullptr;
  Arena arena;
  // upload ring
  static constexpr int kSlots = 8;
  static constexpr size_t kSlotBytes = 512 * 1024;
  char *pinned = nullptr;
  char *dev = nullptr;
  hipEvent_t ev[kSlots] = {};
  bool ev_live[kSlots] = {};   // an event is recorded and the slot is busy until it fires
  bool used[kSlots] = {};      // written during the current call, not fenced yet
  int next = 0;
  // hand-off words of the launches that quantize their own rows (ZmiFusedQuant::sync / error)
  unsigned int *fq_flags = nullptr;      // device: one flag per row, holding the epoch of the launch that published it
  unsigned int *fq_flags_plain = nullptr;   // the same in ordinary device memory (uncached memory refused or switched off)
  bool fq_uncached_refused = false;
  unsigned int fq_epoch = 0;             // name of this thread's latest launch of that kind
  unsigned int *fq_err_host = nullptr;   // pinned host word the kernels set when a wait ran out
  unsigned int *fq_err_dev = nullptr;    // the same word as the device addresses it
  // stream hand-over (zmi_set_stream): work of this thread may still be queued on `stream`
  bool enqueued = false;
  bool low_operand = false;   // (see note_operand())
  hipEvent_t handover = nullptr;
  // arrival words of K-sliced launches (see slice_arrivals())
  unsigned int *arrivals = nullptr;
  int64_t n_arrivals = 0;
  // side stream (see side_stream())
  hipStream_t side = nullptr;
  hipEvent_t side_fork = nullptr, side_join = nullptr;
  bool side_tried = false;
};
thread_local ThreadCtx tctx;

std::mutex g_mu;
bool g_device_ready = false;

struct CacheKey {
  const void *ptr;
  int64_t K, N, ldb;
  bool transB;
  bool operator<(const CacheKey &o) const {
    return std::tie(ptr, K, N, ldb, transB) < std::tie(o.ptr, o.K, o.N, o.ldb, o.transB);
  }
};
struct CacheVal {
  uint8_t *blob;
  std::list<CacheKey>::iterator lru;
};
std::map<CacheKey, CacheVal> g_cache;
std::list<CacheKey> g_lru;
std::set<std::tuple<const void *, int64_t, int64_t>> g_checked_blobs;   // (blob, K, N) whose header was read

size_t cache_capacity() {
  // same variable the reference reads for its weight caches
  static const size_t cap = [] {
    const char *e = zmi_env(ZE_ZENDNNL_LRU_CACHE_CAPACITY);
    long v = e ? std::atol(e) : 0;
    return v > 0 ? (size_t)v : (size_t)1 << 30;
  }();
  return cap;
}
}  // namespace

void set_error(const std::string &msg) { tctx.error = msg; }
void clear_error() { tctx.error.clear(); tctx.low_operand = false; }
// An operand address in the first 64 KiB is no memory (a placeholder, an offset taken for a pointer): the entry points
// note their operands here and ensure_device() refuses the call before anything is queued, instead of a kernel
// faulting on it.  No more than that: whether an address above is device memory is the caller's business.
void note_operand(const void *p) {
  if (p && (uintptr_t)p < 65536) tctx.low_operand = true;
}
void set_kernel_name(const char *name) { tctx.kernel = name; }
hipStream_t stream() { return tctx.stream; }

bool hip_ok(hipError_t e, const char *what) {
  if (e == hipSuccess) return true;
  set_error(std::string(what) + ": " + hipGetErrorString(e));
  (void)hipGetLastError();
  return false;
}

unsigned int *slice_arrivals(int64_t n) {
  auto &c = tctx;
  if (zmi_env(ZE_NO_SLICE_ARRIVALS)) return nullptr;
  if (n > c.n_arrivals) {
    // (launches still in flight count in the old words)
    if (c.arrivals) {
      if (hipStreamSynchronize(c.stream) != hipSuccess || hipFree(c.arrivals) != hipSuccess) (void)hipGetLastError();
      c.arrivals = nullptr;
      c.n_arrivals = 0;
    }
    const int64_t want = n < 4096 ? 4096 : n * 2;
    void *d = nullptr;
    if (hipMalloc(&d, (size_t)want * sizeof(unsigned int)) != hipSuccess ||
        hipMemset(d, 0, (size_t)want * sizeof(unsigned int)) != hipSuccess) {
      (void)hipGetLastError();
      if (d) (void)hipFree(d);
      return nullptr;
    }
    c.arrivals = (unsigned int *)d;
    c.n_arrivals = want;
  }
  return c.arrivals;
}

// Words of the persistent large-M kernel's in-launch quantization (two counters that are zero between launches, then
// one flag per chunk of eight rows that keeps the number of the launch that wrote it): zeroed once, grown on demand.
ZmiRingSide side_stream() {
  auto &c = tctx;
  if (!c.side_tried) {
    c.side_tried = true;
    if (!zmi_env(ZE_NO_SIDE_STREAM)) {
      bool ok = hipStreamCreateWithFlags(&c.side, hipStreamNonBlocking) == hipSuccess &&
                hipEventCreateWithFlags(&c.side_fork, hipEventDisableTiming) == hipSuccess &&
                hipEventCreateWithFlags(&c.side_join, hipEventDisableTiming) == hipSuccess;
      if (!ok) {
        (void)hipGetLastError();
        c.side = nullptr;
      }
    }
  }
  ZmiRingSide s = {c.side, c.side_fork, c.side_join};
  return s;
}

static bool device_present() {
  static std::atomic<bool> ready{false};
  if (ready.load(std::memory_order_acquire)) return true;
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_device_ready) { ready.store(true, std::memory_order_release); return true; }
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    set_error("no HIP device available (the library has no CPU fallback)");
    (void)hipGetLastError();
    return false;
  }
  g_device_ready = true;
  ready.store(true, std::memory_order_release);
  return true;
}

bool ensure_device() {
  tctx.enqueued = true;   // every entry point passes here before it queues work
  if (tctx.low_operand) {
    set_error("an operand address lies in the first 64 KiB: that is no memory a kernel can be launched on");
    return false;
  }
  return device_present();
}

void note_enqueue() { tctx.enqueued = true; }

// ---- arena ---------------------------------------------------------------------
bool Arena::begin(size_t total) {
  used_ = 0;
  if (total <= cap_) return true;
  // kernels of earlier calls may still read the old buffer
  if (base_) {
    if (!hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize")) return false;
    if (!hip_ok(hipFree(base_), "hipFree(scratch)")) return false;
    base_ = nullptr;
    cap_ = 0;
  }
  size_t want = total + total / 4 + (1 << 20);
  void *p = nullptr;
  if (!hip_ok(hipMalloc(&p, want), "hipMalloc(scratch)")) return false;
  base_ = (char *)p;
  cap_ = want;
  return true;
}

void *Arena::alloc(size_t bytes) {
  size_t n = padded(bytes);
  if (used_ + n > cap_) return nullptr;
  void *p = base_ + used_;
  used_ += n;
  return p;
}

void Arena::release() {
  if (base_) {
    (void)hipStreamSynchronize(stream());
    (void)hipFree(base_);
  }
  base_ = nullptr;
  cap_ = used_ = 0;
}

Arena &arena() { return tctx.arena; }

// ---- upload ring ------------------------------------------------------------------
void *upload(const void *host, size_t bytes) {
  ThreadCtx &c = tctx;
  if (bytes == 0) return nullptr;
  if (bytes > ThreadCtx::kSlotBytes) {
    // too large for a ring slot: plain (synchronous for pageable memory) copy into the arena
    void *d = c.arena.alloc(bytes);
    if (!d) { set_error("upload: scratch arena too small"); return nullptr; }
    if (!hip_ok(hipMemcpyAsync(d, host, bytes, hipMemcpyHostToDevice, c.stream), "hipMemcpyAsync(upload)"))
      return nullptr;
    return d;
  }
  if (!c.pinned) {
    void *p = nullptr, *d = nullptr;
    if (!hip_ok(hipHostMalloc(&p, ThreadCtx::kSlots * ThreadCtx::kSlotBytes, hipHostMallocDefault),
                "hipHostMalloc(upload ring)"))
      return nullptr;
    if (!hip_ok(hipMalloc(&d, ThreadCtx::kSlots * ThreadCtx::kSlotBytes), "hipMalloc(upload ring)")) return nullptr;
    c.pinned = (char *)p;
    c.dev = (char *)d;
    for (int i = 0; i < ThreadCtx::kSlots; ++i)
      if (!hip_ok(hipEventCreateWithFlags(&c.ev[i], hipEventDisableTiming), "hipEventCreate")) return nullptr;
  }
  const int s = c.next;
  c.next = (c.next + 1) % ThreadCtx::kSlots;
  if (c.used[s]) {
    // the ring wrapped inside one call: fence the slot before it is rewritten
    if (!hip_ok(hipEventRecord(c.ev[s], c.stream), "hipEventRecord(upload slot)")) return nullptr;
    c.ev_live[s] = true;
    c.used[s] = false;
  }
  if (c.ev_live[s]) {
    if (!hip_ok(hipEventSynchronize(c.ev[s]), "hipEventSynchronize(upload slot)")) return nullptr;
    c.ev_live[s] = false;
  }
  char *hp = c.pinned + (size_t)s * ThreadCtx::kSlotBytes;
  char *dp = c.dev + (size_t)s * ThreadCtx::kSlotBytes;
  std::memcpy(hp, host, bytes);
  if (!hip_ok(hipMemcpyAsync(dp, hp, bytes, hipMemcpyHostToDevice, c.stream), "hipMemcpyAsync(upload)"))
    return nullptr;
  // the slot is free again once every kernel of this call that reads it has run;
  // upload_fence() records that point
  c.used[s] = true;
  return dp;
}

// Marks every slot used since the last fence as busy until the stream reaches
// this point.  Called at the end of each API entry point that uploaded tables.
void upload_fence() {
  ThreadCtx &c = tctx;
  if (!c.pinned) return;
  for (int i = 0; i < ThreadCtx::kSlots; ++i) {
    if (c.used[i]) {
      (void)hipEventRecord(c.ev[i], c.stream);
      c.ev_live[i] = true;
      c.used[i] = false;
    }
  }
}

// copies of the hand-off flags, a page apart (the waiters of a launch spread over them)
constexpr int kFqCopies = 16;

bool fused_handoff(ZmiFusedQuant *fq) {
  ThreadCtx &c = tctx;
  if (!c.fq_err_host) {
    void *h = nullptr, *hd = nullptr;
    if (!hip_ok(hipHostMalloc(&h, 64, hipHostMallocMapped), "hipHostMalloc(error word)")) return false;
    std::memset(h, 0, 64);
    if (!hip_ok(hipHostGetDevicePointer(&hd, h, 0), "hipHostGetDevicePointer(error word)")) return false;
    c.fq_err_host = (unsigned int *)h;
    c.fq_err_dev = (unsigned int *)hd;
  }
  // Uncached device memory: the waiting side may read the flags through the scalar unit, which cannot ask for device
  // scope.  Never freed -- memory of this kind that a kernel has read stays allocated until the process ends.  A
  // device that refuses the uncached kind (or ZMI_NO_UNCACHED_FLAGS, which the tests use to reach that path) gets
  // ordinary memory, and the kernels then wait with device-scope vector loads.
  const bool want_plain = zmi_env(ZE_NO_UNCACHED_FLAGS) != nullptr;
  if (!want_plain && !c.fq_flags && !c.fq_uncached_refused) {
    void *d = nullptr;
    if (hipExtMallocWithFlags(&d, kFqCopies * 4096, hipDeviceMallocUncached) != hipSuccess) {
      (void)hipGetLastError();
      c.fq_uncached_refused = true;
    } else {
      if (!hip_ok(hipMemset(d, 0, kFqCopies * 4096), "hipMemset(hand-off words)")) return false;
      c.fq_flags = (unsigned int *)d;
    }
  }
  const bool plain = want_plain || !c.fq_flags;
  if (plain && !c.fq_flags_plain) {
    void *d = nullptr;
    if (!hip_ok(hipMalloc(&d, 512), "hipMalloc(hand-off words)")) return false;
    if (!hip_ok(hipMemset(d, 0, 512), "hipMemset(hand-off words)")) return false;
    c.fq_flags_plain = (unsigned int *)d;
  }
  // (the two sets of words share the epoch counter: a set that sat out some launches holds older epochs, never newer)
  fq->flags = plain ? c.fq_flags_plain : c.fq_flags;
  fq->flags_uncached = plain ? 0 : 1;
  fq->n_copies = plain ? 1 : kFqCopies;
  if (++c.fq_epoch == 0) c.fq_epoch = 1;   // (0 is what the flags hold before the first launch)
  fq->epoch = c.fq_epoch;
  fq->error = c.fq_err_dev;
  // 100 ms unless ZMI_FUSED_WAIT_US says otherwise (0: every wait gives up at once; the tests of the
  // failure path use it)
  uint64_t us = 100000;
  if (const char *e = zmi_env(ZE_FUSED_WAIT_US)) us = (uint64_t)std::strtoull(e, nullptr, 10);
  const uint64_t ticks = us * 100;
  fq->wait_ticks = ticks > 0xffffffffull ? 0xffffffffu : (uint32_t)ticks;
  return true;
}

bool async_failure_pending() {
  ThreadCtx &c = tctx;
  if (!c.fq_err_host || *(volatile unsigned int *)c.fq_err_host == 0) return false;
  // a launch of this thread gave up waiting for its quantized rows and stored nothing
  (void)hipStreamSynchronize(c.stream);
  *(volatile unsigned int *)c.fq_err_host = 0;
  (void)hipGetLastError();
  set_error("an earlier call on this thread did not get its quantized rows in time and wrote no output "
            "(fused per-token quantization hand-off timed out)");
  return true;
}

// ---- one-element parameters ------------------------------------------------------
bool is_device_pointer(const void *p) {
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return false;   // ordinary host memory
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

bool scalar_param_f32(const void *buff, int32_t dt, float *value, const void **dev_ptr) {
  *dev_ptr = nullptr;
  *value = 1.0f;
  if (!buff) return true;
  if (is_device_pointer(buff)) {
    *dev_ptr = buff;
    return true;
  }
  switch (dt) {
  case ZMI_DT_F32: *value = *(const float *)buff; return true;
  case ZMI_DT_BF16: {
    uint32_t u = ((uint32_t) * (const uint16_t *)buff) << 16;
    std::memcpy(value, &u, 4);
    return true;
  }
  case ZMI_DT_S32: *value = (float)*(const int32_t *)buff; return true;
  case ZMI_DT_S8: *value = (float)*(const int8_t *)buff; return true;
  case ZMI_DT_U8: *value = (float)*(const uint8_t *)buff; return true;
  default: set_error("unsupported dtype for a one-element scale / zero-point"); return false;
  }
}

bool scalar_param_s32(const void *buff, int32_t dt, int32_t *value, const int32_t **dev_ptr) {
  *dev_ptr = nullptr;
  *value = 0;
  if (!buff) return true;
  if (dt != ZMI_DT_S32) {
    set_error("source zero-point must be s32");
    return false;
  }
  if (is_device_pointer(buff)) {
    *dev_ptr = (const int32_t *)buff;
    return true;
  }
  *value = *(const int32_t *)buff;
  return true;
}

// ---- packed weights ------------------------------------------------------------------
const uint8_t *packed_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB,
                              int32_t src_dtype, bool use_cache, void *arena_slot) {
  if (!use_cache) {
    if (!hip_ok(zmi_launch_prepack((const int8_t *)weight, K, N, ldb, transB, src_dtype, 0,
                                   (uint8_t *)arena_slot, stream()), "prepack launch"))
      return nullptr;
    return (const uint8_t *)arena_slot;
  }
  std::lock_guard<std::mutex> lk(g_mu);
  CacheKey key{weight, K, N, ldb, transB};
  auto it = g_cache.find(key);
  if (it != g_cache.end()) {
    g_lru.splice(g_lru.begin(), g_lru, it->second.lru);
    return it->second.blob;
  }
  void *blob = nullptr;
  if (!hip_ok(hipMalloc(&blob, (size_t)zmi_blob_bytes(K, N)), "hipMalloc(packed weights)")) return nullptr;
  // the entry becomes visible to every thread (each on its own stream) as soon as it is inserted: the blob
  // must be complete by then
  if (!hip_ok(zmi_launch_prepack((const int8_t *)weight, K, N, ldb, transB, src_dtype, 0, (uint8_t *)blob,
                                 stream()), "prepack launch") ||
      !hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize(prepack)")) {
    (void)hipFree(blob);
    return nullptr;
  }
  g_lru.push_front(key);
  g_cache[key] = CacheVal{(uint8_t *)blob, g_lru.begin()};
  while (g_cache.size() > cache_capacity()) {
    // an evicted blob may still be read by enqueued kernels
    (void)hipDeviceSynchronize();
    CacheKey old = g_lru.back();
    g_lru.pop_back();
    (void)hipFree(g_cache[old].blob);
    g_cache.erase(old);
  }
  return (const uint8_t *)blob;
}

// GGML Q8_0 weights: unpacked and prepacked once per weight pointer (reference: unpack_ggml_weights_and_cache,
// matmul/ggml_weight_unpack.cpp:367-480: cache keyed by pointer, K, N, ldb, trans; the cached buffer holds the
// reordered weights followed by the bf16 scales).  One device allocation: blob, then the {K/32, N} scales.
const uint8_t *packed_ggml_q8_0(const void *weight, int64_t K, int64_t N, const void **scales) {
  std::lock_guard<std::mutex> lk(g_mu);
  CacheKey key{weight, K, N, /*ldb (marks the packed format)*/ -34, true};
  const size_t blob_bytes = (size_t)zmi_round_up(zmi_blob_bytes(K, N), 256);
  auto it = g_cache.find(key);
  if (it != g_cache.end()) {
    g_lru.splice(g_lru.begin(), g_lru, it->second.lru);
    *scales = it->second.blob + blob_bytes;
    return it->second.blob;
  }
  void *buf = nullptr, *rows = nullptr;
  if (!hip_ok(hipMalloc(&buf, blob_bytes + (size_t)(K / 32) * N * 2), "hipMalloc(GGML weights)")) return nullptr;
  if (!hip_ok(hipMalloc(&rows, (size_t)N * K), "hipMalloc(GGML unpack)")) { (void)hipFree(buf); return nullptr; }
  bool ok = hip_ok(zmi_launch_ggml_q8_0_unpack(weight, N, K, (int8_t *)rows, (uint16_t *)((uint8_t *)buf + blob_bytes),
                                               stream()), "GGML unpack launch") &&
            hip_ok(zmi_launch_prepack((const int8_t *)rows, K, N, K, /*transposed*/ 1, ZMI_DT_S8, 0, (uint8_t *)buf,
                                      stream()), "prepack launch") &&
            hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize");   // the unpacked rows are freed next
  (void)hipFree(rows);
  if (!ok) { (void)hipFree(buf); return nullptr; }
  g_lru.push_front(key);
  g_cache[key] = CacheVal{(uint8_t *)buf, g_lru.begin()};
  while (g_cache.size() > cache_capacity()) {
    (void)hipDeviceSynchronize();
    CacheKey old = g_lru.back();
    g_lru.pop_back();
    (void)hipFree(g_cache[old].blob);
    g_cache.erase(old);
  }
  *scales = (uint8_t *)buf + blob_bytes;
  return (const uint8_t *)buf;
}

// W4A8 weights: widened s4 -> s8 and reordered (reference: w4a8ReorderAndCacheWeightsAocl,
// matmul/backends/aocl/aocl_kernel.cpp:704-793: a cache of its own keyed like the int8 one; here the key's
// leading dimension is stored negated, which no s8 entry has).
const uint8_t *packed_s4_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB, bool use_cache,
                                 void *widen_slot, void *arena_slot, const uint8_t **tiles_s4) {
  const int64_t rows = transB ? N : K, cols = transB ? K : N;
  // one allocation per cached weight: the blob of widened codes (every kernel reads it), then the 4-bit tiles
  // the decode-shaped kernel streams instead (half the bytes per call)
  const size_t blob_bytes = (size_t)zmi_round_up(zmi_blob_bytes(K, N), 256);
  *tiles_s4 = nullptr;
  if (!use_cache) {
    if (!hip_ok(zmi_launch_s4_widen(weight, rows, cols, ldb, (int8_t *)widen_slot, stream()), "s4 widen launch") ||
        !hip_ok(zmi_launch_prepack((const int8_t *)widen_slot, K, N, cols, transB, ZMI_DT_S8, 0, (uint8_t *)arena_slot,
                                   stream()), "prepack launch"))
      return nullptr;
    return (const uint8_t *)arena_slot;
  }
  std::lock_guard<std::mutex> lk(g_mu);
  CacheKey key{weight, K, N, -ldb - 1000, transB};
  auto it = g_cache.find(key);
  if (it != g_cache.end()) {
    g_lru.splice(g_lru.begin(), g_lru, it->second.lru);
    *tiles_s4 = it->second.blob + blob_bytes;
    return it->second.blob;
  }
  void *blob = nullptr, *wide = nullptr;
  if (!hip_ok(hipMalloc(&blob, blob_bytes + (size_t)zmi_s4_tiles_bytes(K, N)), "hipMalloc(W4A8 weights)")) return nullptr;
  if (!hip_ok(hipMalloc(&wide, (size_t)K * N), "hipMalloc(s4 widen)")) { (void)hipFree(blob); return nullptr; }
  bool ok = hip_ok(zmi_launch_s4_widen(weight, rows, cols, ldb, (int8_t *)wide, stream()), "s4 widen launch") &&
            hip_ok(zmi_launch_prepack((const int8_t *)wide, K, N, cols, transB, ZMI_DT_S8, 0, (uint8_t *)blob, stream()),
                   "prepack launch") &&
            hip_ok(zmi_launch_s4_tiles((const uint8_t *)blob, K, N, (uint8_t *)blob + blob_bytes, stream()), "s4 tiles launch") &&
            hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize");   // the widened copy is freed next
  (void)hipFree(wide);
  if (!ok) { (void)hipFree(blob); return nullptr; }
  g_lru.push_front(key);
  g_cache[key] = CacheVal{(uint8_t *)blob, g_lru.begin()};
  while (g_cache.size() > cache_capacity()) {
    (void)hipDeviceSynchronize();
    CacheKey old = g_lru.back();
    g_lru.pop_back();
    (void)hipFree(g_cache[old].blob);
    g_cache.erase(old);
  }
  *tiles_s4 = (const uint8_t *)blob + blob_bytes;
  return (const uint8_t *)blob;
}

// Weight-only quantization: the 4-bit codes in the order the kernel's wavefronts read them, followed by the scales and
// the zero-points as f32 [G][N] each (reference: woqReorderAndCacheWeightsAocl, matmul/backends/aocl/aocl_kernel.cpp:
// 640-702, which caches the dequantized bf16 matrix per weight pointer -- scales and zero-points included, as here;
// the codes stay 4-bit).  The key's leading dimension is stored negated and far below W4A8's.
const uint8_t *packed_woq_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB, int64_t G,
                                  const ZmiWoqParamSrc &sc, const ZmiWoqParamSrc &zp, bool use_cache, void *arena_slot) {
  const size_t tiles = (size_t)zmi_woq_tiles_bytes(K, N), total = tiles + 2 * sizeof(float) * (size_t)(G * N);
  auto fill = [&](uint8_t *blob) {
    return hip_ok(zmi_launch_woq_tiles(weight, K, N, ldb, transB, (uint32_t *)blob, stream()), "4-bit tiles launch") &&
           hip_ok(zmi_launch_woq_params(sc, zp, G, N, (float *)(blob + tiles), (float *)(blob + tiles) + G * N, stream()),
                  "4-bit scales launch");
  };
  if (!use_cache) return fill((uint8_t *)arena_slot) ? (const uint8_t *)arena_slot : nullptr;
  std::lock_guard<std::mutex> lk(g_mu);
  CacheKey key{weight, K, N, -ldb - ((int64_t)1 << 40) - (G << 41), transB};
  auto it = g_cache.find(key);
  if (it != g_cache.end()) {
    g_lru.splice(g_lru.begin(), g_lru, it->second.lru);
    return it->second.blob;
  }
  void *blob = nullptr;
  if (!hip_ok(hipMalloc(&blob, total), "hipMalloc(4-bit weights)")) return nullptr;
  // (the entry becomes visible to threads on other streams: its contents must be there first)
  if (!fill((uint8_t *)blob) || !hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize(4-bit weights)")) {
    (void)hipFree(blob);
    return nullptr;
  }
  g_lru.push_front(key);
  g_cache[key] = CacheVal{(uint8_t *)blob, g_lru.begin()};
  while (g_cache.size() > cache_capacity()) {
    (void)hipDeviceSynchronize();
    CacheKey old = g_lru.back();
    g_lru.pop_back();
    (void)hipFree(g_cache[old].blob);
    g_cache.erase(old);
  }
  return (const uint8_t *)blob;
}

void clear_weight_cache() {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_cache.empty()) (void)hipDeviceSynchronize();
  for (auto &kv : g_cache) (void)hipFree(kv.second.blob);
  g_cache.clear();
  g_lru.clear();
  g_checked_blobs.clear();
}

bool blob_matches(const void *blob, int64_t K, int64_t N) {
  {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_checked_blobs.count(std::make_tuple(blob, K, N))) return true;
  }
  ZmiBlobHeader h;
  if (!hip_ok(hipMemcpyAsync(&h, blob, sizeof(h), hipMemcpyDeviceToHost, stream()), "hipMemcpy(blob header)"))
    return false;
  if (!hip_ok(hipStreamSynchronize(stream()), "hipStreamSynchronize")) return false;
  if (h.magic != ZMI_BLOB_MAGIC || h.K != K || h.N != N) {
    set_error("mem_format_b == 'r': the weight buffer is not a blob packed by reorder_direct for this K and N");
    return false;
  }
  std::lock_guard<std::mutex> lk(g_mu);
  g_checked_blobs.insert(std::make_tuple(blob, K, N));
  return true;
}

int64_t nelems(const zmi_quant_t &q) {
  int64_t n = 1;
  for (int i = 0; i < q.ndims && i < ZMI_MAX_DIMS; ++i) n *= q.dims[i];
  return n;
}

bool diagnostics_enabled() {
  // validation gate of the reference (ZENDNNL_DIAGNOSTICS_ENABLE, on unless "0")
  const char *e = zmi_env(ZE_ZENDNNL_DIAGNOSTICS_ENABLE);
  return !(e && e[0] == '0' && e[1] == 0);
}

int weight_cache_env() {
  const char *e = zmi_env(ZE_ZENDNNL_MATMUL_WEIGHT_CACHE);
  if (!e) return 2;
  int v = std::atoi(e);
  return v < 0 ? 0 : (v > 2 ? 2 : v);
}

}  // namespace zmi

// ---- C ABI: library services ---------------------------------------------------------
extern "C" {

int32_t zmi_init(int32_t device) {
  zmi::clear_error();
  if (!zmi::ensure_device()) return ZMI_FAILURE;
  if (!zmi::hip_ok(hipSetDevice(device), "hipSetDevice")) return ZMI_FAILURE;
  if (!zmi::noalloc_setup()) return ZMI_FAILURE;   // the device's address of zmi_matmul_direct_noalloc's scratch array
  return ZMI_SUCCESS;
}

void zmi_set_stream(void *hip_stream) {
  // The thread's scratch arena, upload ring and hand-off words are ordered by the stream its calls
  // run on: work queued on the old stream has to finish before calls on the new one reuse them.
  auto &c = zmi::tctx;
  hipStream_t next = (hipStream_t)hip_stream;
  if (next != c.stream && c.enqueued) {
    bool chained = false;
    if (!c.handover && hipEventCreateWithFlags(&c.handover, hipEventDisableTiming) != hipSuccess) c.handover = nullptr;
    if (c.handover && hipEventRecord(c.handover, c.stream) == hipSuccess &&
        hipStreamWaitEvent(next, c.handover, 0) == hipSuccess)
      chained = true;
    if (!chained) {
      // (e.g. the old stream no longer exists: whatever ran on it has then finished or is lost)
      (void)hipGetLastError();
      (void)hipDeviceSynchronize();
      (void)hipGetLastError();
    }
    c.enqueued = false;
  }
  c.stream = next;
}
void *zmi_get_stream(void) { return (void *)zmi::tctx.stream; }
const char *zmi_last_error(void) { return zmi::tctx.error.c_str(); }
const char *zmi_last_kernel(void) { return zmi::tctx.kernel; }
void zmi_clear_weight_cache(void) { zmi::clear_weight_cache(); }
void zmi_clear_scratch(void) { zmi::tctx.arena.release(); }
const char *zmi_version(void) { return "zmi-lowoha 0.1.0 (gfx950)"; }

}  // extern "C"
