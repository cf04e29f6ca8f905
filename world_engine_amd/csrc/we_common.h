// Shared device helpers for the gfx950 ring-buffer attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace we {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

// Floor division / modulo on int64, the semantics of `//` and `%` on torch int64 tensors
// (src/model/kv_cache.py:129-130,140).
__device__ __forceinline__ int64_t floor_div(int64_t a, int64_t b) {
  int64_t q = a / b, r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}
__device__ __forceinline__ int64_t floor_mod(int64_t a, int64_t b) {
  int64_t r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r;
}

// Ring slot of a frame and whether the frame persists (src/model/kv_cache.py:126-131,140).
struct SlotInfo {
  int slot;
  bool write_step;
};
__device__ __forceinline__ SlotInfo ring_slot(int64_t frame_t, int dilation, int num_buckets) {
  SlotInfo s;
  // Frame indices are small and non-negative in practice: 32-bit unsigned arithmetic, a fraction
  // of the instructions of the emulated 64-bit signed divisions (kernels are launched once per
  // layer and frame, so their straight-line start-up code is paid for by instruction fetch).
  if (__builtin_expect((uint64_t)frame_t < 0x7fff0000ull && dilation > 0 && dilation < 0x10000, 1)) {
    const uint32_t t = (uint32_t)frame_t;
    if (dilation == 1) {
      s.slot = (int)(t % (uint32_t)num_buckets);
      s.write_step = true;
    } else {
      const uint32_t bucket = (t + (uint32_t)dilation - 1u) / (uint32_t)dilation;
      s.slot = (int)(bucket % (uint32_t)num_buckets);
      s.write_step = t % (uint32_t)dilation == 0u;
    }
    return s;
  }
  int64_t bucket = floor_div(frame_t + (dilation - 1), (int64_t)dilation);
  s.slot = (int)floor_mod(bucket, (int64_t)num_buckets);
  s.write_step = floor_mod(frame_t, (int64_t)dilation) == 0;
  return s;
}

// fp32 -> bf16 bits, round-to-nearest-even, NaN -> 0x7FC0 (c10::BFloat16's rule).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

}  // namespace we
