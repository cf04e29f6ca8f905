// Fused RoPE + ring-slot K/V store for one frame (gfx950).
//
// One launch replaces, for a single attention layer, the reference's RoPE on q and k
// (src/model/attn.py:33-40), torch.stack([k, v]) (src/model/kv_cache.py:192), the tail
// index_copy_ (:138), the unfrozen ring index_copy_ and the `written` update (:147-151).
// The ring slot is derived on the device from t_pos[0] (:126-131,:140).
//
// Work item: one thread per 16 consecutive input elements of one (tensor, b, head, token)
// row; a workgroup covers 256 consecutive (token, chunk) pairs of one head.  For a rotated row those are 8 (even, odd) pairs; the thread writes 8 contiguous
// elements into the first half of the output row and 8 into the second half (the reference
// concatenates the rotated halves, attn.py:40).  Threads are ordered chunk-fastest, then
// token, so a wavefront reads whole 256-byte input rows and writes contiguous cache rows.
// HBM-bound: bytes = elements read once + written once (twice for K/V on a persisting call).
#include "we_common.h"
#include "we_kernels.h"

// The rotation must round each product and the sum separately, like eager fp32 tensor ops;
// hipcc's default would contract them into fused multiply-adds.
#pragma clang fp contract(off)

namespace we {

struct Bf16Tag {
  typedef uint16_t store_t;
  static constexpr int kBytes = 2;
  __device__ static float to_f32(uint16_t b) { return bf16_bits_to_f32(b); }
  __device__ static uint16_t from_f32(float f) { return f32_to_bf16_bits(f); }
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

template <typename Tag>
__global__ void __launch_bounds__(256) rope_kv_store_kernel(StoreParams p) {
  typedef typename Tag::store_t st_t;
  // grid: x = 256-thread slices of the (token, chunk) pairs of one row block, y = head among
  // [q heads | k heads | v heads], z = batch; everything below the block level is 32-bit math
  const int cpr = p.Dh >> 4;  // 16-element chunks per row
  const int hq = p.q ? p.H : 0;
  const int hkv = p.k ? p.Hkv : 0;  // rotation-only launches carry no k/v
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.T * cpr) return;
  const int t = p.cpr_shift >= 0 ? idx >> p.cpr_shift : idx / cpr;  // head dims are powers of two in practice
  const int chunk = idx - t * cpr;
  const int head_all = blockIdx.y;
  const int b = blockIdx.z;

  // which tensor this row belongs to: 0 = q, 1 = k, 2 = v
  int which, h;
  if (head_all < hq) {
    which = 0;
    h = head_all;
  } else if (head_all < hq + hkv) {
    which = 1;
    h = head_all - hq;
  } else {
    which = 2;
    h = head_all - hq - hkv;
  }

  const st_t* src;
  if (which == 0)
    src = (const st_t*)p.q + b * p.qs_b + h * p.qs_h + t * p.qs_t;
  else if (which == 1)
    src = (const st_t*)p.k + b * p.ks_b + h * p.ks_h + t * p.ks_t;
  else
    src = (const st_t*)p.v + b * p.vs_b + h * p.vs_h + t * p.vs_t;

  Chunk16<Tag> in;
  load16<Tag>(in, src + chunk * 16);
  const int64_t frame_t = p.t_pos[0];  // requested together with the row, used only for k/v rows

  const bool rotate = (which != 2) && (p.cos_t != nullptr);
  Chunk8<Tag> lo, hi;  // outputs for [8*chunk, 8*chunk+8) and [Dh/2 + 8*chunk, ...)
  if (rotate) {
    int64_t pos = p.t_pos[b * p.pos_stride_b + t] * p.grid_hw +
                  p.y_pos[b * p.pos_stride_b + t] * p.grid_w + p.x_pos[b * p.pos_stride_b + t];
    pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
    const int half = p.Dh >> 1;
    const float4* cp = reinterpret_cast<const float4*>(p.cos_t + pos * half + chunk * 8);
    const float4* sp = reinterpret_cast<const float4*>(p.sin_t + pos * half + chunk * 8);
    float c[8], s[8];
    *reinterpret_cast<float4*>(c) = cp[0];
    *reinterpret_cast<float4*>(c + 4) = cp[1];
    *reinterpret_cast<float4*>(s) = sp[0];
    *reinterpret_cast<float4*>(s + 4) = sp[1];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float x0 = Tag::to_f32(in.e[2 * i]);
      const float x1 = Tag::to_f32(in.e[2 * i + 1]);
      // y0 = x0*cos - x1*sin ; y1 = x1*cos + x0*sin with every product and the sum rounded
      // separately (no fused multiply-add), as eager fp32 tensor ops do (attn.py:38-39).
      // (plain operators: the contract(off) pragma above governs them, not inlined intrinsics)
      const float p0 = x0 * c[i], p1 = x1 * s[i], p2 = x1 * c[i], p3 = x0 * s[i];
      const float y0 = p0 - p1;
      const float y1 = p2 + p3;
      lo.e[i] = Tag::from_f32(y0);
      hi.e[i] = Tag::from_f32(y1);
    }
  }

  if (which == 0) {
    st_t* dst = (st_t*)p.q_out + (((int64_t)b * p.H + h) * p.T + t) * p.Dh;
    if (rotate) {
      store8<Tag>(dst + chunk * 8, lo);
      store8<Tag>(dst + (p.Dh >> 1) + chunk * 8, hi);
    } else {
      store16<Tag>(dst + chunk * 16, in);
    }
    return;
  }

  // K or V row: tail always, ring slot when this is an unfrozen persisting frame.
  const int64_t cap = p.L + p.T;
  const SlotInfo si = ring_slot(frame_t, p.dilation, p.num_buckets);
  const int plane = which - 1;
  st_t* plane_base = (st_t*)p.kv + (((int64_t)plane * p.B + b) * p.Hkv + h) * cap * p.Dh;
  const bool to_ring = (!p.frozen) && si.write_step;
  const int64_t tail_row = p.L + t;
  const int64_t ring_row = (int64_t)si.slot * p.T + t;

  st_t* d0 = plane_base + tail_row * p.Dh;
  st_t* d1 = plane_base + ring_row * p.Dh;
  if (rotate) {
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
  if (!p.frozen && which == 1 && b == 0 && h == 0 && chunk == 0)
    p.written[to_ring ? ring_row : tail_row] = 1;
}

hipError_t launch_rope_kv_store(const StoreParams& p, int dtype, hipStream_t stream) {
  const int hq = p.q ? p.H : 0;
  const int hkv = p.k ? p.Hkv : 0;
  const dim3 grid((unsigned)((p.T * (p.Dh >> 4) + 255) / 256), (unsigned)(hq + 2 * hkv), (unsigned)p.B);
  if (dtype == 0)
    hipLaunchKernelGGL(rope_kv_store_kernel<Bf16Tag>, grid, dim3(256), 0, stream, p);
  else if (dtype == 1)
    hipLaunchKernelGGL(rope_kv_store_kernel<F16Tag>, grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(rope_kv_store_kernel<F32Tag>, grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace we
