// Module-level state of libf3d_hip.so: last-error string, per-device workspace, the global
// sync-stream flag and RNG seed (the counterpart of the reference's DeviceManagerSingleton,
// src/common/device_manager.cu:58-119).
#include <stdarg.h>

#include <mutex>
#include <unordered_map>

#include "f3d_internal.h"

namespace f3d {

static thread_local char g_err[512] = "";
static std::mutex g_mu;
struct Ws {
  void* ptr = nullptr;
  size_t bytes = 0;
};
static std::unordered_map<int, Ws> g_ws;
static bool g_sync = false;
static uint32_t g_seed = 3407u;
static int g_rebalance = 1;
static int g_quantiser = 0;

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

void* workspace(int device, size_t bytes, hipStream_t stream) {
  std::lock_guard<std::mutex> lk(g_mu);
  Ws& w = g_ws[device];
  if (w.bytes >= bytes && w.ptr) return w.ptr;
  DeviceGuard guard(device);
  // Work queued on the old buffer must finish before it is released.
  if (w.ptr) {
    // Refused while the caller's stream is being captured: the device cannot be synchronised then (the attempt itself
    // would invalidate the capture), so the capture state is asked first and the device is left alone.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    hipError_t es = hipSuccess;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      es = hipErrorStreamCaptureUnsupported;
    else
      es = hipDeviceSynchronize();
    if (es != hipSuccess) {
      set_error("the workspace of device %d must grow from %zu to %zu bytes, but the device cannot be synchronised (%s): "
                "warm the shapes up outside stream capture", device, w.bytes, bytes, hipGetErrorString(es));
      return nullptr;
    }
    (void)hipFree(w.ptr);
    w.ptr = nullptr;
    w.bytes = 0;
  }
  size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes + bytes / 4;
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, want);
  if (e != hipSuccess) {
    set_error("workspace allocation of %zu bytes failed: %s", want, hipGetErrorString(e));
    return nullptr;
  }
  w.ptr = p;
  w.bytes = want;
  return p;
}

// weights staged by the caller for the next dense call on this thread (f3d_stage_weights)
static thread_local struct {
  void* buf = nullptr;
  size_t bytes = 0;
  bool ready = false, armed = false;
} g_staged;

void* weight_area(int device, size_t bytes, bool* ready, hipStream_t stream) {
  *ready = false;
  if (g_staged.armed) {
    if (g_staged.bytes < bytes) {
      set_error("the buffer given to f3d_stage_weights holds %zu bytes, this call prepares %zu", g_staged.bytes, bytes);
      return nullptr;
    }
    *ready = g_staged.ready;
    return g_staged.buf;
  }
  return workspace(device, bytes, stream);
}

StagedWeightsScope::~StagedWeightsScope() { g_staged.armed = false; }

bool sync_stream_enabled() { return g_sync; }
uint32_t global_seed() { return g_seed; }
int rebalance_mode() { return g_rebalance; }
uint32_t quantiser_bit() { return g_quantiser ? 0x80000000u : 0u; }

}  // namespace f3d

extern "C" {

const char* f3d_last_error(void) { return f3d::g_err; }

int f3d_init_dev_info(int device) {
  int n = 0;
  F3D_CHECK_HIP(hipGetDeviceCount(&n));
  // The reference silently ignores a device that does not exist (device_manager.cu:59-60).
  if (device < 0 || device >= n) return F3D_OK;
  if (!f3d::psh_noalloc_scratch(device)) return F3D_ERR_RUNTIME;
  return f3d::workspace(device, 1, nullptr) ? F3D_OK : F3D_ERR_RUNTIME;
}

int f3d_set_sync_stream(int enable) {
  f3d::g_sync = enable != 0;
  return f3d::g_sync ? 1 : 0;
}

int f3d_get_sync_stream(void) { return f3d::g_sync ? 1 : 0; }

int f3d_set_seed(uint32_t seed) {
  f3d::g_seed = seed;
  return F3D_OK;
}

uint32_t f3d_get_seed(void) { return f3d::g_seed; }

int f3d_set_psh_rebalance(int mode) {
  if (mode != 0 && mode != 1) {
    f3d::set_error("rebalance mode must be 0 or 1, got %d", mode);
    return F3D_ERR_INVALID;
  }
  f3d::g_rebalance = mode;
  return F3D_OK;
}

int f3d_get_psh_rebalance(void) { return f3d::g_rebalance; }

int f3d_set_quantiser(int mode) {
  if (mode != 0 && mode != 1) {
    f3d::set_error("quantiser mode must be 0 (multiply by the reciprocal) or 1 (IEEE division), got %d", mode);
    return F3D_ERR_INVALID;
  }
  f3d::g_quantiser = mode;
  return F3D_OK;
}

int f3d_get_quantiser(void) { return f3d::g_quantiser; }

int f3d_stage_weights(void* buf, size_t bytes, int ready) {
  if (!buf || ((uintptr_t)buf & 255u) != 0) {
    f3d::set_error("f3d_stage_weights needs a 256-byte aligned device buffer");
    return F3D_ERR_INVALID;
  }
  f3d::g_staged.buf = buf;
  f3d::g_staged.bytes = bytes;
  f3d::g_staged.ready = ready != 0;
  f3d::g_staged.armed = true;
  return F3D_OK;
}

}  // extern "C"
