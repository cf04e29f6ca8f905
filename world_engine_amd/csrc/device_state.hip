// One-time, per-device set-up of the ring-buffer attention library (gfx950) and the only mutable
// state it keeps: a table of per-device facts, filled once per device under a mutex and read-only
// afterwards.
#include "device_state.h"

#include "../../include/we_attn.h"

#include <atomic>
#include <mutex>

// Split-context partial results of we_attn_ring_fwd_static: part of the library's device image, so
// that the entry point needs no allocation and no caller-owned workspace.  Every GPU the library
// runs on holds its own copy at its own address; host code must never use the array's name as an
// address (on the host it is a stand-in for the symbol), only what hipGetSymbolAddress returns
// with the device in question current.
static __device__ __align__(256) unsigned char scratch[WE_STATIC_SCRATCH_BYTES];

namespace we {

namespace {

constexpr int kMaxDevices = 64;
struct Entry {
  std::atomic<bool> ready{false};
  host::DeviceState st{};
};
Entry g_dev[kMaxDevices];
std::mutex g_mu;
std::atomic<int> g_cus[kMaxDevices];

}  // namespace

namespace host {

int compute_units() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = g_cus[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
  g_cus[dev].store(n, std::memory_order_relaxed);
  return n;
}

int init_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return WE_ERR_LAUNCH;
  if (dev < 0 || dev >= kMaxDevices) return WE_ERR_UNSUPPORTED;
  Entry& e = g_dev[dev];
  if (e.ready.load(std::memory_order_acquire)) return WE_OK;
  std::lock_guard<std::mutex> lock(g_mu);
  if (e.ready.load(std::memory_order_acquire)) return WE_OK;
  if (configure_attn_ring_bf16_128() != hipSuccess || configure_attn_ring_bf16_64() != hipSuccess ||
      configure_attn_ring_f16_128() != hipSuccess || configure_attn_ring_f16_64() != hipSuccess ||
      configure_qkv_rope_store() != hipSuccess)
    return WE_ERR_LAUNCH;
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return WE_ERR_LAUNCH;
  e.st.scratch = p;
  e.st.cus = compute_units();
  e.ready.store(true, std::memory_order_release);
  return WE_OK;
}

int device_state(hipStream_t stream, const DeviceState** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return WE_ERR_LAUNCH;
  if (dev < 0 || dev >= kMaxDevices) return WE_ERR_UNSUPPORTED;
  Entry& e = g_dev[dev];
  if (!e.ready.load(std::memory_order_acquire)) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return WE_ERR_NOT_READY;
    }
    const int rc = init_current_device();
    if (rc != WE_OK) return rc;
  }
  *out = &e.st;
  return WE_OK;
}

}  // namespace host
}  // namespace we
