// Per-item work of the fused RoPE + ring-slot K/V store kernel (rope_kv_store.hip, gfx950): one
// item = 16 consecutive input elements of one (tensor, batch, head, token) row.
#pragma once
#include "we_common.h"
#include "we_kernels.h"

namespace we {

struct Bf16Tag {
  typedef uint16_t store_t;
  static constexpr int kBytes = 2;
  __device__ static float to_f32(uint16_t b) { return bf16_bits_to_f32(b); }
  // v_cvt_pk_bf16_f32 (round-to-nearest-even) with c10::BFloat16's NaN (0x7FC0) patched in
  __device__ static uint16_t from_f32(float f) {
    const uint16_t r = __builtin_bit_cast(uint16_t, (__bf16)f);
    return f != f ? (uint16_t)0x7fc0 : r;
  }
};
struct F16Tag {
  typedef uint16_t store_t;
  static constexpr int kBytes = 2;
  __device__ static float to_f32(uint16_t b) { return f16_bits_to_f32(b); }
  __device__ static uint16_t from_f32(float f) { return f32_to_f16_bits(f); }
};
struct F32Tag {
  typedef float store_t;
  static constexpr int kBytes = 4;
  __device__ static float to_f32(float b) { return b; }
  __device__ static float from_f32(float f) { return f; }
};

// 16 elements of a row as raw storage.
template <typename Tag>
struct Chunk16 {
  typename Tag::store_t e[16];
};
template <typename Tag>
struct Chunk8 {
  typename Tag::store_t e[8];
};

template <typename Tag>
__device__ __forceinline__ void load16(Chunk16<Tag>& c, const void* p) {
  constexpr int nvec = 16 * Tag::kBytes / 16;
  const uint4* src = reinterpret_cast<const uint4*>(p);
  uint4* dst = reinterpret_cast<uint4*>(c.e);
#pragma unroll
  for (int i = 0; i < nvec; ++i) dst[i] = src[i];
}
template <typename Tag>
__device__ __forceinline__ void store16(void* p, const Chunk16<Tag>& c) {
  constexpr int nvec = 16 * Tag::kBytes / 16;
  uint4* dst = reinterpret_cast<uint4*>(p);
  const uint4* src = reinterpret_cast<const uint4*>(c.e);
#pragma unroll
  for (int i = 0; i < nvec; ++i) dst[i] = src[i];
}
template <typename Tag>
__device__ __forceinline__ void store8(void* p, const Chunk8<Tag>& c) {
  constexpr int nvec = 8 * Tag::kBytes / 16;
  uint4* dst = reinterpret_cast<uint4*>(p);
  const uint4* src = reinterpret_cast<const uint4*>(c.e);
#pragma unroll
  for (int i = 0; i < nvec; ++i) dst[i] = src[i];
}

// Weightless RMS norm of a row held 16 elements per lane by `cpr` consecutive lanes (a power of
// two, at most 64): x * rsqrt(mean(x^2) + eps) in fp32, rounded to the element type, as
// F.rms_norm on a low-precision tensor does (src/model/nn.py:55-56).
template <typename Tag>
__device__ __forceinline__ void rms_norm_chunk(Chunk16<Tag>& c, int cpr, int Dh, float eps) {
  float x[16];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    x[i] = Tag::to_f32(c.e[i]);
    ss += x[i] * x[i];
  }
  for (int m = 1; m < cpr; m <<= 1) ss += __shfl_xor(ss, m);
  const float r = rsqrtf(ss / (float)Dh + eps);
#pragma unroll
  for (int i = 0; i < 16; ++i) c.e[i] = Tag::from_f32(x[i] * r);
}

// torch.lerp(v, v1, w) on 16 elements: fp32 arithmetic, the formula switches at |w| = 0.5
// (ATen/native/Lerp.h), result rounded to the element type.
template <typename Tag>
__device__ __forceinline__ void lerp_chunk(Chunk16<Tag>& v, const Chunk16<Tag>& v1, float w) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float a = Tag::to_f32(v.e[i]), b = Tag::to_f32(v1.e[i]);
    const float d = b - a;
    v.e[i] = Tag::from_f32(fabsf(w) < 0.5f ? a + w * d : b - d * (1.f - w));
  }
}

// Row of the cos / sin tables for token t of batch element b (src/model/attn.py:33-36): the
// three position ids select one row of the flattened [frames, height, width] table.
__device__ __forceinline__ int64_t rope_table_row(const StoreParams& p, int b, int t) {
  int64_t pos = p.t_pos[b * p.pos_stride_b + t] * p.grid_hw + p.y_pos[b * p.pos_stride_b + t] * p.grid_w +
                p.x_pos[b * p.pos_stride_b + t];
  return pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
}

// cos / sin of the 8 pairs of chunk `chunk` of a table row.
__device__ __forceinline__ void load_cos_sin(const float* cos_row, const float* sin_row, int chunk, float (&c)[8],
                                             float (&s)[8]) {
  const float4* cp = reinterpret_cast<const float4*>(cos_row + chunk * 8);
  const float4* sp = reinterpret_cast<const float4*>(sin_row + chunk * 8);
  *reinterpret_cast<float4*>(c) = cp[0];
  *reinterpret_cast<float4*>(c + 4) = cp[1];
  *reinterpret_cast<float4*>(s) = sp[0];
  *reinterpret_cast<float4*>(s + 4) = sp[1];
}

// Rotation of the 8 (even, odd) pairs of one 16-element chunk: lo gets x0*cos - x1*sin (elements
// [8*chunk, 8*chunk+8) of the output row), hi gets x1*cos + x0*sin (the same range of the second
// half; the reference concatenates the rotated halves, attn.py:38-40).  Every product and sum is
// rounded separately, as eager fp32 tensor ops do: contraction into fused multiply-adds is
// switched off for this function (plain operators; the pragma does not govern inlined intrinsics).
template <typename Tag>
__device__ __forceinline__ void rotate_values(const Chunk16<Tag>& in, const float (&c)[8], const float (&s)[8],
                                              Chunk8<Tag>& lo, Chunk8<Tag>& hi) {
#pragma clang fp contract(off)
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float x0 = Tag::to_f32(in.e[2 * i]);
    const float x1 = Tag::to_f32(in.e[2 * i + 1]);
    const float p0 = x0 * c[i], p1 = x1 * s[i], p2 = x1 * c[i], p3 = x0 * s[i];
    const float y0 = p0 - p1;
    const float y1 = p2 + p3;
    lo.e[i] = Tag::from_f32(y0);
    hi.e[i] = Tag::from_f32(y1);
  }
}
// Destination rows of a K/V item: tail always, ring slot on an unfrozen persisting frame.
template <typename Tag>
__device__ __forceinline__ void store_kv_rows(const StoreParams& p, int which, int b, int h, int t, int chunk,
                                              const SlotInfo& si, bool rotated, const Chunk16<Tag>& in,
                                              const Chunk8<Tag>& lo, const Chunk8<Tag>& hi) {
  typedef typename Tag::store_t st_t;
  const int64_t cap = p.L + p.T;
  const int plane = which - 1;
  st_t* plane_base = (st_t*)p.kv + (((int64_t)plane * p.B + b) * p.Hkv + h) * cap * p.Dh;
  const bool to_ring = (!p.frozen) && si.write_step;
  const int64_t tail_row = p.L + t;
  const int64_t ring_row = (int64_t)si.slot * p.T + t;
  st_t* d0 = plane_base + tail_row * p.Dh;
  st_t* d1 = plane_base + ring_row * p.Dh;
  if (rotated) {
    store8<Tag>(d0 + chunk * 8, lo);
    store8<Tag>(d0 + (p.Dh >> 1) + chunk * 8, hi);
    if (to_ring) {
      store8<Tag>(d1 + chunk * 8, lo);
      store8<Tag>(d1 + (p.Dh >> 1) + chunk * 8, hi);
    }
  } else {
    store16<Tag>(d0 + chunk * 16, in);
    if (to_ring) store16<Tag>(d1 + chunk * 16, in);
  }
  // written[dst] = True for the rows the unfrozen write went to (kv_cache.py:149-151).
  if (!p.frozen && which == 1 && b == 0 && h == 0 && chunk == 0) p.written[to_ring ? ring_row : tail_row] = 1;
}

// Everything after the load of a K (which = 1) or V (which = 2) item: K is normalised (optional)
// and rotated, V is blended with the value residual (optional); the tail row is written always
// and the ring-slot row when this is an unfrozen persisting frame; `written` is marked
// (src/model/attn.py:105-110, src/model/kv_cache.py:138,147-151).  cos / sin are the item's 8
// table values (used when `rotate`), `res` the matching 16 elements of the value residual (used
// when p.v1 is set).
template <typename Tag>
__device__ __forceinline__ void finish_kv_chunk(const StoreParams& p, int which, int b, int h, int t, int chunk,
                                                const SlotInfo& si, Chunk16<Tag>& in, bool rotate,
                                                const float (&c)[8], const float (&s)[8], const Chunk16<Tag>& res,
                                                float lamb) {
  if (which == 1 && p.norm_eps > 0.f) rms_norm_chunk<Tag>(in, p.Dh >> 4, p.Dh, p.norm_eps);
  if (which == 2 && p.v1 != nullptr) lerp_chunk<Tag>(in, res, lamb);
  Chunk8<Tag> lo, hi;
  if (rotate) rotate_values<Tag>(in, c, s, lo, hi);
  store_kv_rows<Tag>(p, which, b, h, t, chunk, si, rotate, in, lo, hi);
}

// Everything after the load of a Q item: optional norm, rotation (or plain copy when there is no
// table), store into the contiguous [B, H, T, Dh] output.
template <typename Tag>
__device__ __forceinline__ void finish_q_chunk(const StoreParams& p, int b, int h, int t, int chunk,
                                               Chunk16<Tag>& in, bool rotate, const float (&c)[8],
                                               const float (&s)[8]) {
  typedef typename Tag::store_t st_t;
  if (p.norm_eps > 0.f) rms_norm_chunk<Tag>(in, p.Dh >> 4, p.Dh, p.norm_eps);
  st_t* dst = (st_t*)p.q_out + (((int64_t)b * p.H + h) * p.T + t) * p.Dh;
  if (rotate) {
    Chunk8<Tag> lo, hi;
    rotate_values<Tag>(in, c, s, lo, hi);
    store8<Tag>(dst + chunk * 8, lo);
    store8<Tag>(dst + (p.Dh >> 1) + chunk * 8, hi);
  } else {
    store16<Tag>(dst + chunk * 16, in);
  }
}

// What an item needs besides its own 16 elements: the 8 cos / sin values of its pairs (rotated
// items) and the value residual's 16 elements with the blend weight (V items of a layer that has
// one).  Separate from the arithmetic so that a caller can request them long before it has the
// item's own values.
template <typename Tag>
struct ItemSide {
  float c[8], s[8];
  Chunk16<Tag> res;
  float lamb;
  bool rotate;
};
template <typename Tag>
__device__ __forceinline__ void load_item_side(const StoreParams& p, int which, int b, int h, int t, int chunk,
                                               ItemSide<Tag>& sd) {
  typedef typename Tag::store_t st_t;
  sd.rotate = which != 2 && p.cos_t != nullptr;
  sd.lamb = 0.f;
  if (sd.rotate) {
    const int64_t pos = rope_table_row(p, b, t);
    const int half = p.Dh >> 1;
    load_cos_sin(p.cos_t + pos * half, p.sin_t + pos * half, chunk, sd.c, sd.s);
  }
  if (which == 2 && p.v1 != nullptr) {
    load16<Tag>(sd.res, (const st_t*)p.v1 + b * p.v1s_b + h * p.v1s_h + t * p.v1s_t + chunk * 16);
    sd.lamb = Tag::to_f32(*reinterpret_cast<const st_t*>(p.v_lamb));
  }
}

// One K or V item of the stand-alone store kernel: load, then the above.
template <typename Tag>
__device__ __forceinline__ void store_kv_item(const StoreParams& p, int which, int b, int h, int t, int chunk,
                                              const SlotInfo& si) {
  typedef typename Tag::store_t st_t;
  const st_t* src = which == 1 ? (const st_t*)p.k + b * p.ks_b + h * p.ks_h + t * p.ks_t
                               : (const st_t*)p.v + b * p.vs_b + h * p.vs_h + t * p.vs_t;
  Chunk16<Tag> in;
  load16<Tag>(in, src + chunk * 16);
  ItemSide<Tag> sd;
  load_item_side<Tag>(p, which, b, h, t, chunk, sd);
  finish_kv_chunk<Tag>(p, which, b, h, t, chunk, si, in, sd.rotate, sd.c, sd.s, sd.res, sd.lamb);
}

}  // namespace we
