// Per-device facts and one-time set-up of the library (device_state.hip).
#pragma once
#include <hip/hip_runtime.h>

namespace we {
namespace host {

struct DeviceState {
  int cus;        // compute units
  void* scratch;  // device address of the library's static split-context buffer on this device
};

// Compute units of the current device (256 when no device can be asked, e.g. on a build host).
// Cheap, never synchronises, safe under stream capture.
int compute_units();

// One-time set-up of the current device: kernel LDS limits, the static buffer's address, the
// compute-unit count.  Launches nothing and does not synchronise; later calls return at once.
int init_current_device();

// State of the current device for a call that will enqueue on `stream`.  Sets the device up on
// first use - unless `stream` is being captured (the set-up's runtime calls do not belong into a
// capture): WE_ERR_NOT_READY then.
int device_state(hipStream_t stream, const DeviceState** out);

}  // namespace host

// per translation unit: raise the dynamic-LDS limit of its kernels on the current device
hipError_t configure_attn_ring_bf16_128();
hipError_t configure_attn_ring_bf16_64();
hipError_t configure_attn_ring_f16_128();
hipError_t configure_attn_ring_f16_64();
hipError_t configure_qkv_rope_store();

}  // namespace we
