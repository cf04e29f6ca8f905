// MFMA wrappers and small wave-level helpers shared by the attention kernels (gfx950).
#pragma once
#include "we_common.h"

namespace we {

constexpr int BN = 64;  // keys per tile

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

struct Bf16Mma {
  typedef bf16x8_t frag_t;
  typedef __bf16 elem_t;
  __device__ static __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ frag_t pack8(float v0, float v1, float v2, float v3, float v4,
                                                 float v5, float v6, float v7) {
    frag_t r;
    r[0] = (__bf16)v0; r[1] = (__bf16)v1; r[2] = (__bf16)v2; r[3] = (__bf16)v3;
    r[4] = (__bf16)v4; r[5] = (__bf16)v5; r[6] = (__bf16)v6; r[7] = (__bf16)v7;
    return r;
  }
  // acc + the two elements of one packed register (v_dot2c_f32_bf16 with a (1, 1) operand)
  __device__ static __forceinline__ float add_pair(float acc, frag_t f, int pair) {
    const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
    const bf16x2_t v = {f[2 * pair], f[2 * pair + 1]};
    return __builtin_amdgcn_fdot2_f32_bf16(v, ones, acc, false);
  }
};
struct F16Mma {
  typedef f16x8_t frag_t;
  typedef _Float16 elem_t;
  __device__ static __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ frag_t pack8(float v0, float v1, float v2, float v3, float v4,
                                                 float v5, float v6, float v7) {
    frag_t r;
    r[0] = (_Float16)v0; r[1] = (_Float16)v1; r[2] = (_Float16)v2; r[3] = (_Float16)v3;
    r[4] = (_Float16)v4; r[5] = (_Float16)v5; r[6] = (_Float16)v6; r[7] = (_Float16)v7;
    return r;
  }
  __device__ static __forceinline__ float add_pair(float acc, frag_t f, int pair) {
    const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
    const f16x2_t v = {f[2 * pair], f[2 * pair + 1]};
    return __builtin_amdgcn_fdot2(v, ones, acc, false);
  }
};

// Both half-waves get (lower half's x, upper half's x).
__device__ __forceinline__ void half_wave_pair(float x, float& lower, float& upper) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  lower = __uint_as_float(r[0]);
  upper = __uint_as_float(r[1]);
}

typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;

// One 1-KB LDS-DMA: lane i copies 16 bytes from gbase + voff to LDS byte lds_addr + 16*i.
// Hidden from the compiler's counter bookkeeping on purpose; completion is awaited with
// dma_wait<N>() (vmcnt) followed by a workgroup barrier.
__device__ __forceinline__ void dma16(uint64_t gbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(gbase), "s"(lds_addr)
               : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ uint64_t uniform64(uint64_t x) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// Head gate of output row (b, h, t): the given value, or sigmoid(gate_proj(x[b, t, :H]))[h] with
// the module's rounding steps (src/model/attn.py:117-118: the projection's output and the sigmoid's
// are both element-type tensors).  The dot product runs in fp32 in channel order.
template <typename E, typename P>
__device__ __forceinline__ float head_gate(const P& p, int b, int h, int64_t t) {
  if (p.gate_w != nullptr) {
    const E* x = reinterpret_cast<const E*>(p.gate_x) + b * p.gx_b + t * p.gx_t;
    const E* w = reinterpret_cast<const E*>(p.gate_w) + (int64_t)h * p.H;
    float acc = 0.f;
    for (int j = 0; j < p.H; ++j) acc = __builtin_fmaf((float)x[j], (float)w[j], acc);
    const float pre = (float)(E)acc;
    return (float)(E)(1.f / (1.f + __expf(-pre)));
  }
  return (float)reinterpret_cast<const E*>(p.gate)[b * p.gs_b + h * p.gs_h + t * p.gs_t];
}

}  // namespace we
