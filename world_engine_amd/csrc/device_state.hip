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
// with the device in question current.  Zero when the image is loaded, which is what the arrival
// counters at its start need.
static __device__ __align__(256) unsigned char scratch[WE_STATIC_SCRATCH_BYTES];

// XCC id of every workgroup of the probe launch.
static __device__ uint32_t xcc_seen[1024];

namespace we {

namespace {

constexpr int kMaxDevices = 64;
constexpr unsigned kProbeX = 32, kProbeY = 2, kProbeZ = 3;

// Every workgroup records the id of the XCD (accelerator complex) it runs on.
__global__ void xcc_probe_kernel(uint32_t* out) {
  const uint32_t xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 0xfu;  // HW_REG_XCC_ID, bits 3:0
  if (threadIdx.x == 0) out[blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)] = xcc;
}

// The in-kernel merge of split-context partials relies on all workgroups with the same
// blockIdx.x % 8 (grid x a multiple of 8) running on one XCD, i.e. sharing one L2.  The hardware
// deals workgroups to the XCDs of a partition round-robin in linear order; this launch checks that
// on the device at hand instead of assuming it.
bool probe_xcd_mapping() {
  void* out = nullptr;
  if (hipGetSymbolAddress(&out, HIP_SYMBOL(xcc_seen)) != hipSuccess || out == nullptr) return false;
  hipLaunchKernelGGL(xcc_probe_kernel, dim3(kProbeX, kProbeY, kProbeZ), dim3(64), 0, nullptr, static_cast<uint32_t*>(out));
  if (hipGetLastError() != hipSuccess) return false;
  uint32_t seen[kProbeX * kProbeY * kProbeZ];
  if (hipMemcpy(seen, out, sizeof(seen), hipMemcpyDeviceToHost) != hipSuccess) return false;
  uint32_t of_slot[8];
  for (unsigned i = 0; i < kProbeX * kProbeY * kProbeZ; ++i) {
    const unsigned slot = (i % kProbeX) & 7u;
    if (i < 8) of_slot[slot] = seen[i];
    else if (seen[i] != of_slot[slot]) return false;
  }
  return true;
}

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
  e.st.xcd_merge = probe_xcd_mapping();
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
