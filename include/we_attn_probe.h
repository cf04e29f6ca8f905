/*
 * we_attn_probe.h - C ABI of the measurement library (libwe_probe.so) that goes with we_attn.h.
 *
 * Nothing here has a counterpart in world_engine and nothing here is part of the drop-in surface:
 * these entry points exist for the benchmark and its tests.  libwe_probe.so is a separate build of
 * the same kernels that also contains the clocked instantiations of the attention kernel and the
 * tile-stream probe; libwe_attn.so contains neither.  It exports every symbol of we_attn.h as
 * well (the same code), so a process that measures loads it instead of, or next to, the product
 * library; the two keep separate per-device state.
 */
#ifndef WE_ATTN_PROBE_H
#define WE_ATTN_PROBE_H

#include "we_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * we_attn_ring_fwd that also records how long every workgroup of the main kernel ran, on two
 * clocks, and when it passed the kernel's stages.  Workgroup w (the linear workgroup id of the
 * launch) owns clocks[WE_CLOCK_SLOTS * w ...]: [0] its duration in shader-clock cycles, [1] the
 * same interval in ticks of the device's constant 100 MHz counter (their ratio is the shader
 * clock the kernel actually ran at; boards lower it under their power limit), [2 + s] the ticks
 * from its start to stage s as seen by its first thread: 0 slot list built, 1 first K tile in
 * LDS, 2 tile loop left, 3 wavefront pair merged, 4 (partial) results stored.
 * clocks_len = number of uint64 elements available; at least WE_CLOCK_SLOTS * (workgroups of the
 * launch) or WE_ERR_WORKSPACE is returned; entries of workgroups that own no work, and of stages
 * a workgroup does not pass, stay untouched (zero them beforehand).  bf16 / f16 only.  Everything
 * else as we_attn_ring_fwd; the output has the same bits.
 */
#define WE_CLOCK_SLOTS 16
int we_attn_ring_fwd_clocked(const void* q, const int64_t q_strides[3],
                             const void* kv, const uint8_t* written, const int64_t* t_pos,
                             void* out, const int64_t out_strides[3],
                             void* workspace, size_t workspace_bytes,
                             int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                             int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                             int32_t dtype, uint64_t* clocks, size_t clocks_len, void* stream);

/*
 * The attention kernel's way of fetching K and V tiles at 256-token frames with the arithmetic
 * taken away.  `workgroups` workgroups (one per CU, a multiple of 8: workgroup id % 8 is the XCD)
 * each stream `tiles` 16-KB tiles of one contiguous region of `buf` into LDS by DMA, three tiles in
 * flight, one barrier per tile; `share` consecutive workgroups of an XCD walk the same region (the
 * query tiles and grouped heads of one K/V stream).  Region r starts at byte r * tiles * 16384;
 * buf_bytes must cover the workgroups / share regions (WE_ERR_WORKSPACE otherwise).  Nothing is
 * written.  The duration of a launch is the floor for a kernel of this shape, whatever it computes.
 */
int we_stream_probe(const void* buf, size_t buf_bytes, int32_t workgroups, int32_t tiles, int32_t share,
                    void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WE_ATTN_PROBE_H */
