// Host side of an attention call: argument validation, the choice of kernel shape and context
// splitting, and the kernel parameter block.  Shared by the C ABI (capi.hip) and by the
// measurement library's entry points (probe_capi.hip), so that both plan a call identically.
#pragma once
#include "../../include/we_attn.h"
#include "we_kernels.h"

namespace we {
namespace host {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int elem_bytes(int dtype) { return dtype == WE_DTYPE_F32 ? 4 : 2; }

// element strides whose byte value keeps every row start 16-byte aligned
inline bool strides_ok(const int64_t s[3], int dtype) {
  const int per16 = 16 / elem_bytes(dtype);
  return s[0] % per16 == 0 && s[1] % per16 == 0 && s[2] % per16 == 0;
}

inline int ring_shape_ok(int B, int H, int Hkv, int T, int Dh, int64_t L, int dilation) {
  if (B <= 0 || H <= 0 || Hkv <= 0 || T <= 0 || Dh <= 0 || L <= 0 || dilation <= 0) return WE_ERR_BAD_SHAPE;
  if (H % Hkv != 0 || L % T != 0 || (L / T) % dilation != 0) return WE_ERR_BAD_SHAPE;
  return WE_OK;
}

struct AttnPlan {
  int variant;      // 1: 128 queries per workgroup, 2: 256
  int block_m;      // queries per workgroup
  int n_splits;     // context splits of the units that are split (1: none)
  int units_whole;  // leading (batch, kv head) units that are not split
  int64_t ws_rows;  // query rows that go through the split-context workspace
};

inline int variant_of(int q_tile) {
  switch (q_tile) {
    case 0: return 0;
    case 128: return 1;
    case 256: return 2;
    default: return -1;
  }
}

// Pick the kernel shape and the context splitting for a part with `cus` compute units (256 on an
// MI355X; every count below was measured there and is carried to other sizes as a fraction).
//  * Shape: 256 queries per workgroup when that alone gives at least one workgroup per CU, else
//    128 queries (two wavefronts share each query block and split every tile's keys).
//  * Few workgroups (256-token frames): every unit is split into the same number of context
//    parts - as many as fit the CUs in one round up to four parts, then as many as give 5/8 to
//    15/16 of the CUs a workgroup (more for long contexts, fewer for many parts) - but never fewer
//    than two 64-key tiles per part.
//  * Many workgroups that do not divide into whole rounds of CUs (e.g. 384 on 256): only the units
//    of the last, partial round are split, so that round finishes in a fraction of the time.
inline AttnPlan plan_attn(int B, int H, int Hkv, int T, int64_t L, int n_splits, int variant, int cus) {
  AttnPlan pl;
  if (cus < 8) cus = 8;
  const int64_t wg256 = (int64_t)B * H * ((T + 255) / 256);
  const int64_t wg128 = (int64_t)B * H * ((T + 127) / 128);
  // 256 queries per workgroup when that alone fills the CUs - or when 128 would spill into a
  // second round that 256 avoids (136 to 256 heads of a 256-token frame: one round of fat
  // workgroups beats one and a bit rounds of thin ones by 5 to 17 %)
  pl.variant = variant ? variant : ((T >= 256 && (wg256 >= cus || wg128 > cus)) ? 2 : 1);
  pl.block_m = pl.variant == 2 ? 256 : 128;
  const int units = B * Hkv;
  const int group = H / Hkv;
  const int q_tiles = (T + pl.block_m - 1) / pl.block_m;
  const int members = group * q_tiles;
  const int64_t wgs = (int64_t)units * members;
  const int64_t tiles = L / 64;  // visible 64-key tiles at steady state
  const int64_t max_s = tiles / 2 > 0 ? tiles / 2 : 1;
  pl.units_whole = 0;
  pl.n_splits = 1;
  if (n_splits > 0) {
    pl.n_splits = n_splits;
  } else if (wgs < cus) {
    // Never more workgroups than CUs (a second, nearly empty round costs a whole kernel's
    // time); and when the context is cut four ways or more, fewer workgroups than CUs: a part's
    // fixed costs do not shrink with its length, the partial results grow with the number of
    // parts, and the board clocks the kernel lower the more CUs are busy (16 heads of a 256-token
    // frame over 16 slots: 6 parts 25.1 us per frame-step, 8 parts 27.2; 24 such rings: 653
    // against 717).  Measured over 8 to 160 workgroups per call: the best count is about 15/16 of
    // the CUs for up to six parts and about 3/4 for more.
    // Long contexts (32 slots of a 256-token frame and more) amortise the extra parts and the lower
    // clock over longer loops: about 15/16 there too (32 slots: 7 parts 32.0 us per frame-step,
    // 6 parts 32.8), and all CUs when that is exactly four parts (a quarter of the CUs unsplit:
    // 4 parts beat 3 by 2 to 7 %).
    // Beyond sixteen parts every part's own cost weighs more: about 5/8 of the CUs (4 heads: 20
    // parts 21.2 to 27.2 us per frame-step over 16 to 64 slots, 24 parts 21.7 to 27.4).
    const int64_t c15 = (int64_t)cus * 15 / 16, c34 = (int64_t)cus * 3 / 4, c58 = (int64_t)cus * 5 / 8;
    int64_t s = cus / wgs;
    if (s > 4) s = ((wgs * 32 >= (int64_t)cus * 5 || (tiles >= 96 && c15 / wgs <= 16)) ? c15 : (c34 / wgs > 16 ? c58 : c34)) / wgs;
    if (s > max_s) s = max_s;
    if (s > 64) s = 64;
    if (s < 1) s = 1;
    pl.n_splits = (int)s;
  } else if (wgs < 4 * (int64_t)cus && members <= cus) {
    const int whole_units = (int)((wgs / cus) * cus / members);
    const int64_t rem_wgs = (int64_t)(units - whole_units) * members;
    if (rem_wgs > 0 && rem_wgs <= cus / 2) {
      int64_t s = cus / rem_wgs;
      if (s > 8) s = 8;
      if (s > max_s / 2) s = max_s / 2;
      if (s > 1) {
        pl.n_splits = (int)s;
        pl.units_whole = whole_units;
      }
    }
  }
  const int split_units = units - pl.units_whole;
  pl.ws_rows = pl.n_splits > 1 ? (int64_t)split_units * group * T : 0;
  return pl;
}

inline size_t workspace_bytes_of(const AttnPlan& pl, int Dh) {
  if (pl.n_splits <= 1 || pl.ws_rows <= 0) return 0;
  return (size_t)pl.n_splits * (size_t)pl.ws_rows * ((size_t)Dh * 2 + 4 * sizeof(float));
}

// Validation of a we_attn_ring_fwd call, its plan and its kernel parameters.  `cus`: compute units
// of the device the call will run on.
inline int prepare_attn(const void* q, const int64_t* q_strides, const void* kv, const uint8_t* written,
                        const int64_t* t_pos, void* out, const int64_t* out_strides, void* workspace,
                        size_t workspace_bytes, int B, int H, int Hkv, int T, int Dh, int64_t L, int dilation,
                        float scale, int n_splits, int q_tile, int dtype, int cus, AttnParams& p, AttnPlan& pl) {
  if (!q || !q_strides || !kv || !written || !t_pos || !out || !out_strides) return WE_ERR_NULL_POINTER;
  int rc = ring_shape_ok(B, H, Hkv, T, Dh, L, dilation);
  if (rc != WE_OK) return rc;
  if (dtype != WE_DTYPE_BF16 && dtype != WE_DTYPE_F16 && dtype != WE_DTYPE_F32) return WE_ERR_UNSUPPORTED;
  if (Dh != 64 && Dh != 128) return WE_ERR_UNSUPPORTED;
  if (L / T > WE_MAX_SLOTS) return WE_ERR_UNSUPPORTED;
  if ((uint64_t)(L + T) * (uint64_t)Dh * 2u >= (1ull << 32)) return WE_ERR_UNSUPPORTED;  // 32-bit tile offsets
  if (!(scale > 0.f) || n_splits < 0 || n_splits > 64) return WE_ERR_BAD_SHAPE;
  if (variant_of(q_tile) < 0) return WE_ERR_UNSUPPORTED;
  if (dtype == WE_DTYPE_F32) {
    // fp32 caches take the plain one-pass kernel: no context splitting, no tile choice
    if (n_splits > 1 || H > 65535 || B > 65535) return WE_ERR_UNSUPPORTED;
    n_splits = 1;
  }
  if (!aligned16(q) || !aligned16(kv) || !aligned16(out) || !strides_ok(q_strides, dtype) ||
      !strides_ok(out_strides, dtype))
    return WE_ERR_ALIGNMENT;

  pl = plan_attn(B, H, Hkv, T, L, n_splits, variant_of(q_tile), cus);
  const size_t ws_need = workspace_bytes_of(pl, Dh);
  if (ws_need > 0) {
    if (!workspace || !aligned16(workspace)) return WE_ERR_WORKSPACE;
    if (workspace_bytes < ws_need) return WE_ERR_WORKSPACE;
  }

  p.q = q; p.kv = kv; p.written = written; p.t_pos = t_pos; p.out = out;
  p.ws_o = ws_need ? static_cast<uint16_t*>(workspace) : nullptr;
  p.ws_ml = ws_need ? reinterpret_cast<float*>(p.ws_o + (size_t)pl.n_splits * (size_t)pl.ws_rows * Dh) : nullptr;
  p.qs_b = q_strides[0]; p.qs_h = q_strides[1]; p.qs_t = q_strides[2];
  p.os_b = out_strides[0]; p.os_h = out_strides[1]; p.os_t = out_strides[2];
  p.L = L;
  p.B = B; p.H = H; p.Hkv = Hkv; p.T = T;
  p.n_slots = (int)(L / T); p.dilation = dilation; p.num_buckets = p.n_slots / dilation;
  p.n_splits = pl.n_splits;
  p.units_whole = pl.units_whole;
  p.ws_row0 = (int64_t)B * H * T - pl.ws_rows;
  p.q_tiles = (T + pl.block_m - 1) / pl.block_m;
  p.group = H / Hkv;
  p.members = p.group * p.q_tiles;
  p.unit_splits = pl.units_whole + (B * Hkv - pl.units_whole) * pl.n_splits;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.gate = nullptr; p.gs_b = p.gs_h = p.gs_t = 0;
  p.gate_x = nullptr; p.gate_w = nullptr; p.gx_b = p.gx_t = 0;
  p.clock_out = nullptr;
  p.q_dma = (q_strides[2] > 0 && (uint64_t)T * (uint64_t)q_strides[2] * 2u < (1ull << 31)) ? 1 : 0;

  if ((p.unit_splits + 7) / 8 > 65535 || p.group > 65535 || (int64_t)B * H - (int64_t)pl.units_whole * p.group > 65535)
    return WE_ERR_UNSUPPORTED;  // grid y / z limits of the two launches
  return WE_OK;
}

// The launches of one planned attention call.
inline int launch_attn(const AttnParams& p, const AttnPlan& pl, int Dh, int dtype, hipStream_t st) {
  if (dtype == WE_DTYPE_F32) return launch_attn_ring_f32(p, Dh, st) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
  const int ksplit = pl.variant == 1 ? 2 : 1;
  hipError_t e;
  if (dtype == WE_DTYPE_BF16) e = Dh == 128 ? launch_attn_ring_bf16_128(p, ksplit, st) : launch_attn_ring_bf16_64(p, ksplit, st);
  else e = Dh == 128 ? launch_attn_ring_f16_128(p, ksplit, st) : launch_attn_ring_f16_64(p, ksplit, st);
  if (e != hipSuccess) return WE_ERR_LAUNCH;
  if (pl.n_splits > 1 && launch_attn_combine(p, Dh, dtype, st) != hipSuccess) return WE_ERR_LAUNCH;
  return WE_OK;
}

}  // namespace host
}  // namespace we
