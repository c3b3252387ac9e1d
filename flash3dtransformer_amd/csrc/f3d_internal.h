// Shared host-side plumbing of the gfx950 library: error reporting, per-device workspace,
// stream synchronisation flag.  Device helpers live in f3d_device.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/f3d_hip.h"

namespace f3d {

// Message of the last failing call on this thread (returned by f3d_last_error()).
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Grow-only scratch buffer owned by the library, one per device.  Work that uses it is ordered on
// the caller's stream; calls that overlap on different streams of one device must not share it, so
// every entry point that needs scratch documents that it is not re-entrant per device.
// `stream`: the caller's stream; when the buffer has to grow while that stream is being captured the call fails with a
// message (warm the shapes up outside capture) and does not touch the device.
// Returns nullptr (and sets the error) on failure.
void* workspace(int device, size_t bytes, hipStream_t stream);

// Device memory for the weights a dense op prepares per call (LayerNorm folded into the weight, fragment-major
// copies): the buffer the caller staged with f3d_stage_weights for this call, else the per-device workspace.
// *ready: the staged buffer already holds this call's prepared weights, the preparation launch is skipped.
// nullptr + error message when the staged buffer is too small or the workspace cannot grow.
void* weight_area(int device, size_t bytes, bool* ready, hipStream_t stream);
// Declared at the top of every dense entry point: whatever the call does, the staging ends with it.
struct StagedWeightsScope {
  ~StagedWeightsScope();
};

// This device's copy of the fixed scratch array behind f3d_batch_psh_scatter_pad_hash_noalloc (resolved on the first
// call per device; f3d_init_dev_info does it ahead of time).  nullptr + error message on failure.
uint32_t* psh_noalloc_scratch(int device);

// Streaming attention backward (buck_swin_bwd_stream.hip): any scope size, head_dim 16 / 32 / 64 / 128, optional
// valid lengths per bucket; dq / dk / dv rows are `ldg` elements apart.  Launches on `s`; F3D_ERR_UNSUPPORTED (+ message)
// for other head sizes.
int launch_attn_bwd_stream(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, const uint16_t* o,
                           const uint16_t* d_o, const float* lse, float* delta, uint16_t* dq, uint16_t* dk, uint16_t* dv,
                           const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                           uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t head_dim, const int32_t* kv_len,
                           uint32_t ldg, int device, hipStream_t s);

bool sync_stream_enabled();
uint32_t global_seed();
int rebalance_mode();
// 0x80000000 when the voxel quantiser divides (f3d_set_quantiser(1)), else 0: OR-ed into a kernel's num_vox argument
uint32_t quantiser_bit();

#define F3D_CHECK_ARG(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      ::f3d::set_error(__VA_ARGS__);        \
      return F3D_ERR_INVALID;               \
    }                                       \
  } while (0)

#define F3D_CHECK_HIP(expr)                                                              \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    if (_e != hipSuccess) {                                                              \
      ::f3d::set_error("HIP error %d (%s) at %s:%d", (int)_e, hipGetErrorString(_e),    \
                       __FILE__, __LINE__);                                              \
      return F3D_ERR_RUNTIME;                                                            \
    }                                                                                    \
  } while (0)

// RAII bracket reproducing the reference's optional stream synchronisation around an op
// (src/psh/batch_psh_bucket_dispatcher.cu:278-280, 323-325).
// A stream that is being captured is left alone (synchronising it would invalidate the capture).
struct SyncBracket {
  hipStream_t s;
  bool on;
  explicit SyncBracket(hipStream_t stream) : s(stream), on(false) {
    if (!sync_stream_enabled()) return;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    on = hipStreamIsCapturing(s, &st) == hipSuccess && st == hipStreamCaptureStatusNone;
    if (on) (void)hipStreamSynchronize(s);
  }
  ~SyncBracket() {
    if (on) (void)hipStreamSynchronize(s);
  }
};

// Makes `device` current for the lifetime of the object and restores the previous one.
struct DeviceGuard {
  int prev = -1;
  bool ok = true;
  explicit DeviceGuard(int device) {
    if (hipGetDevice(&prev) != hipSuccess) prev = -1;
    if (prev != device) ok = hipSetDevice(device) == hipSuccess;
  }
  ~DeviceGuard() {
    int cur = -1;
    if (prev >= 0 && hipGetDevice(&cur) == hipSuccess && cur != prev) (void)hipSetDevice(prev);
  }
};

static inline uint32_t cdiv_u32(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

}  // namespace f3d
