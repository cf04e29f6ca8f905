// Kernel parameter blocks and host-side launchers shared by the C ABI translation unit.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace we {

struct StoreParams {
  const void* q;
  const void* k;
  const void* v;
  void* q_out;
  void* kv;
  uint8_t* written;
  const float* cos_t;
  const float* sin_t;
  const int64_t* t_pos;
  const int64_t* y_pos;
  const int64_t* x_pos;
  int64_t qs_b, qs_h, qs_t;  // element strides
  int64_t ks_b, ks_h, ks_t;
  int64_t vs_b, vs_h, vs_t;
  int64_t pos_stride_b;
  int64_t table_rows;
  int64_t grid_hw, grid_w;
  int64_t L;
  int B, H, Hkv, T, Dh;
  int dilation, num_buckets, frozen;
  int cpr_shift;  // log2(Dh / 16) when Dh / 16 is a power of two, else -1
  // optional work of the attention module in front of RoPE (src/model/attn.py:105-109)
  float norm_eps;             // > 0: q and k rows are RMS-normalised (no weight) first
  const void* v1;             // value residual [B, Hkv, T, Dh] or null: v = lerp(v, v1, *v_lamb)
  const void* v_lamb;         // device pointer to the lerp weight, element type
  int64_t v1s_b, v1s_h, v1s_t;
};

// uint64 slots per workgroup of AttnParams::clock_out (measurement library only)
constexpr int kClockSlots = 16;

struct AttnParams {
  const void* q;
  const void* kv;
  const uint8_t* written;
  const int64_t* t_pos;
  void* out;
  uint16_t* ws_o;  // [n_splits][rows >= ws_row0][Dh] normalised partial outputs / row scale, fp16 in [-1, 1]
  float* ws_ml;    // [n_splits][rows >= ws_row0][4]  softmax reference (log2 domain), sum, row scale, unused
  int64_t qs_b, qs_h, qs_t;
  int64_t os_b, os_h, os_t;
  int64_t L;
  int B, H, Hkv, T;
  int n_slots, dilation, num_buckets;
  int n_splits;     // context splits of the units that are split (1 = nothing is split)
  int units_whole;  // leading (batch, kv head) units processed unsplit, writing the output directly
  int64_t ws_row0;  // first query row covered by the split-context workspace
  int q_tiles;      // ceil(T / queries per workgroup)
  int group;        // query heads per kv head, H / Hkv
  int members;      // workgroups that share one K/V stream: group * q_tiles
  int unit_splits;  // units_whole + (B * Hkv - units_whole) * n_splits
  float scale_log2;  // softmax scale * log2(e), applied to the raw logits in fp32
  // optional per (batch, head, token) output gate, element type (src/model/attn.py:117-119): either
  // given (sigmoid applied), or computed here from the module's input and gate_proj.weight
  const void* gate;
  int64_t gs_b, gs_h, gs_t;
  const void* gate_x;   // x[b, t, 0:H], channel stride 1, element strides gx_b / gx_t (null: no projection here)
  const void* gate_w;   // gate_proj.weight [H, H] row-major (out, in), element type
  int64_t gx_b, gx_t;
  // measurement library only (the product's kernels hold no code that reads it): every workgroup
  // of the main kernel leaves its duration as (shader-clock cycles, ticks of the constant 100 MHz
  // counter) at [2 * linear workgroup id]
  uint64_t* clock_out;
  int q_dma;            // 128-query workgroups fetch their Q tile by DMA (row offsets fit 32 bits)
};

// The merged q/k/v projection with the store's work as its epilogue (qkv_proj_store.hip).
struct ProjParams {
  StoreParams s;        // q / k / v inputs unused; everything else as for the store kernel
  const void* x;        // [B, T, K] module input, channel stride 1
  int64_t xs_b, xs_t;   // element strides
  const void* w;        // [(H + 2 Hkv) Dh, K] merged projection weight, row-major (out, in)
  int64_t ws_n;         // element stride between weight rows
  int K;                // d_model
  void* v_out;          // optional: the projected v rows before the blend (the layer's v1 output)
  int64_t vo_b, vo_h, vo_t;
  int m_tiles;          // ceil(T / 64)
  int n_tiles;          // (H + 2 Hkv) Dh / 128
};

hipError_t launch_rope_kv_store(const StoreParams& p, int dtype, hipStream_t stream);
hipError_t launch_qkv_rope_store(const ProjParams& p, int dtype, hipStream_t stream);

// main kernel, one launcher per (element type, head dim) family: ksplit = 2 -> 128 queries per
// workgroup, 1 -> 256
hipError_t launch_attn_ring_bf16_128(const AttnParams& p, int ksplit, hipStream_t stream);
hipError_t launch_attn_ring_bf16_64(const AttnParams& p, int ksplit, hipStream_t stream);
hipError_t launch_attn_ring_f16_128(const AttnParams& p, int ksplit, hipStream_t stream);
hipError_t launch_attn_ring_f16_64(const AttnParams& p, int ksplit, hipStream_t stream);
// fp32 caches: plain vector-ALU kernel, one pass, no context splitting
hipError_t launch_attn_ring_f32(const AttnParams& p, int Dh, hipStream_t stream);
hipError_t launch_attn_combine(const AttnParams& p, int Dh, int dtype, hipStream_t stream);
// Measurement library only (stream_probe.hip): the 256-token-frame tile stream without the arithmetic.
hipError_t launch_stream_probe(const void* src, int workgroups, int tiles, int share, hipStream_t stream);

}  // namespace we
