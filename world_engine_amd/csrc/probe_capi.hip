// Entry points of the measurement library (include/we_attn_probe.h): the attention call with
// per-workgroup clocks, and the tile-stream probe.  Built into libwe_probe.so together with a copy
// of the product's sources compiled with WE_WITH_PROBES; the product library holds none of this.
#include "../../include/we_attn_probe.h"
#include "attn_plan.h"
#include "device_state.h"
#include "we_kernels.h"

static_assert(WE_CLOCK_SLOTS == we::kClockSlots, "header and kernels disagree on the clock record");

extern "C" {

int we_attn_ring_fwd_clocked(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                             const int64_t* t_pos, void* out, const int64_t out_strides[3], void* workspace,
                             size_t workspace_bytes, int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh,
                             int64_t L, int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                             int32_t dtype, uint64_t* clocks, size_t clocks_len, void* stream) {
  if (!clocks) return WE_ERR_NULL_POINTER;
  if (dtype == WE_DTYPE_F32) return WE_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const we::host::DeviceState* ds = nullptr;
  const int rc_dev = we::host::device_state(st, &ds);
  if (rc_dev != WE_OK) return rc_dev;
  we::AttnParams p;
  we::host::AttnPlan pl;
  const int rc = we::host::prepare_attn(q, q_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes,
                                        B, H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, ds->cus, p, pl);
  if (rc != WE_OK) return rc;
  const size_t wgs = (size_t)(8 * p.q_tiles) * (size_t)p.group * (size_t)((p.unit_splits + 7) / 8);
  if (clocks_len < WE_CLOCK_SLOTS * wgs) return WE_ERR_WORKSPACE;
  p.clock_out = clocks;
  return we::host::launch_attn(p, pl, Dh, dtype, st);
}

int we_stream_probe(const void* buf, size_t buf_bytes, int32_t workgroups, int32_t tiles, int32_t share, void* stream) {
  if (!buf) return WE_ERR_NULL_POINTER;
  if (workgroups <= 0 || workgroups % 8 != 0 || workgroups > 65536 || tiles <= 0 || tiles > 65536 || share <= 0 ||
      (workgroups / 8) % share != 0)
    return WE_ERR_BAD_SHAPE;
  if (!we::host::aligned16(buf)) return WE_ERR_ALIGNMENT;
  const uint64_t region = (uint64_t)tiles * 16384u;
  if (region >= (1ull << 32)) return WE_ERR_UNSUPPORTED;  // 32-bit DMA offsets within a region
  if ((uint64_t)(workgroups / share) * region > buf_bytes) return WE_ERR_WORKSPACE;
  return we::launch_stream_probe(buf, workgroups, tiles, share, static_cast<hipStream_t>(stream)) == hipSuccess
             ? WE_OK : WE_ERR_LAUNCH;
}

}  // extern "C"
