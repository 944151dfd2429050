// Host-side state shared by the C ABI entry points: error text, stream,
// scratch arena, upload ring, packed-weight cache.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "zmi_device.h"
#include "zmi_launch.h"

namespace zmi {

// ---- per-thread call context ------------------------------------------------
void set_error(const std::string &msg);
void clear_error();
void set_kernel_name(const char *name);
hipStream_t stream();

// Returns false (and records the error) when a HIP call failed.
bool hip_ok(hipError_t e, const char *what);

// Makes sure a GPU is usable and the per-device state exists; refuses the call when one of the operands noted since
// clear_error() lies in the first 64 KiB of the address space (no memory: a placeholder or an offset).
bool ensure_device();
void note_operand(const void *p);

// Zeroed device words (one per 32-column block, at least n of them) that K-sliced launches count their arrivals in and
// leave zeroed; null when they cannot be had or ZMI_NO_SLICE_ARRIVALS is set (the launch then ends in a reduction kernel).
unsigned int *slice_arrivals(int64_t n);

// The calling thread's side stream (default priority, created on first use) with a fork and a join event, for work
// that may run beside the stream's own; null fields when it cannot be had or ZMI_NO_SIDE_STREAM is set.
ZmiRingSide side_stream();

// ---- scratch arena ------------------------------------------------------------
// Grow-only device buffer owned by the calling thread.  begin() sizes it for
// one API call (synchronising the stream only when it has to grow); alloc()
// bump-allocates 256-byte aligned pieces until the next begin().
class Arena {
 public:
  bool begin(size_t total_bytes);
  void *alloc(size_t bytes);
  void release();
  static size_t padded(size_t bytes) { return (bytes + 255) / 256 * 256; }

 private:
  char *base_ = nullptr;
  size_t cap_ = 0, used_ = 0;
};
Arena &arena();

// ---- host -> device table upload ---------------------------------------------
// Copies a small host table to device memory, ordered on the stream, without
// synchronising: pinned staging slots recycled behind events.  Returns the
// device address (valid until the slot is recycled, i.e. for this call).
void *upload(const void *host, size_t bytes);
// Ends a call's uploads: the slots it used stay reserved until the stream gets here.
void upload_fence();

// ---- fused-quantization hand-off ------------------------------------------------------
// Fills the hand-off fields of a launch that quantizes its own rows (ZmiFusedQuant::sync, error,
// wait_ticks) with the calling thread's words, allocating them on first use.
bool fused_handoff(ZmiFusedQuant *fq);
// True (with the error text set) when a launch of this thread gave up waiting for its quantized rows
// since the last check; entry points call it first and return failure.
bool async_failure_pending();
// Marks that the calling thread has queued work on its current stream (see zmi_set_stream).
void note_enqueue();

// ---- one-element parameters ------------------------------------------------------
// A scale / zero-point of one element may live in host or device memory.
// Host: *value receives it and *dev_ptr is null.  Device: *dev_ptr receives
// the pointer and the kernel reads it.
// True for device (or managed) memory, false for ordinary host memory.
bool is_device_pointer(const void *p);
bool scalar_param_f32(const void *buff, int32_t dt, float *value, const void **dev_ptr);
bool scalar_param_s32(const void *buff, int32_t dt, int32_t *value, const int32_t **dev_ptr);

// ---- packed weights ------------------------------------------------------------------
// Returns the blob for plain [K,N] weights, packing on a miss.  With use_cache
// the blob is kept for the life of the process keyed by (pointer, shape,
// layout); otherwise it is packed into the arena (arena_slot must then have
// been reserved by the caller with blob_bytes).
const uint8_t *packed_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB,
                              int32_t src_dtype, bool use_cache, void *arena_slot);
// GGML Q8_0 packed weights [N][K/32] blocks: cached blob + bf16 scales {K/32, N} (null on failure)
const uint8_t *packed_ggml_q8_0(const void *weight, int64_t K, int64_t N, const void **scales);
// packed s4 weights ([K, ldb] nibbles, or [N, ldb] when transB): widened to s8 and reordered.  With use_cache the
// blob is kept per (pointer, shape, layout); otherwise widen_slot (K * N bytes) and arena_slot (blob_bytes) must
// have been reserved in the arena by the caller.
// *tiles_s4 receives the 4-bit tiles kept behind a cached blob (null when not cached: a one-off pack streams s8).
const uint8_t *packed_s4_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB, bool use_cache,
                                 void *widen_slot, void *arena_slot, const uint8_t **tiles_s4);
// packed s4 / u4 weights of the weight-only path: the codes in the kernel's tile order (zmi_woq_tiles_bytes(K, N)
// bytes), then the scales and the zero-points as f32 [G][N] each; cached per weight pointer like the others (the
// scales are part of the cached weights, as in the reference), or written into arena_slot.
const uint8_t *packed_woq_weights(const void *weight, int64_t K, int64_t N, int64_t ldb, bool transB, int64_t G,
                                  const ZmiWoqParamSrc &sc, const ZmiWoqParamSrc &zp, bool use_cache, void *arena_slot);
void clear_weight_cache();

// Checks (once per pointer) that a caller-supplied blob carries the header of a
// blob packed for this K and N.
bool blob_matches(const void *blob, int64_t K, int64_t N);

// Looks up the current device's copy of zmi_matmul_direct_noalloc's scratch array (zmi_api_noalloc.hip).
bool noalloc_setup();

int64_t nelems(const zmi_quant_t &q);
bool diagnostics_enabled();
int weight_cache_env();

}  // namespace zmi
