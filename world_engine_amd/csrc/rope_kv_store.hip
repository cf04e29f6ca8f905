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
#include "rope_kv_store.h"

namespace we {

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

  if (head_all >= hq) {  // K or V row
    const int64_t frame_t = p.t_pos[0];
    const int which = head_all < hq + hkv ? 1 : 2;
    const SlotInfo si = ring_slot(frame_t, p.dilation, p.num_buckets);
    store_kv_item<Tag>(p, which, b, head_all - hq - (which == 2 ? hkv : 0), t, chunk, si);
    return;
  }

  // Q row: rotate (or copy when there is no table) into the contiguous output
  const int h = head_all;
  Chunk16<Tag> in;
  load16<Tag>(in, (const st_t*)p.q + b * p.qs_b + h * p.qs_h + t * p.qs_t + chunk * 16);
  ItemSide<Tag> sd;
  load_item_side<Tag>(p, 0, b, h, t, chunk, sd);
  finish_q_chunk<Tag>(p, b, h, t, chunk, in, sd.rotate, sd.c, sd.s);
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
