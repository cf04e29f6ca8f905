// C ABI of the ring-buffer attention library: argument validation and kernel dispatch.
// Declarations and the reference call sites each entry point replaces: include/we_attn.h.
#include "../../include/we_attn.h"
#include "we_kernels.h"

#include <mutex>

// Split-context partial results of we_attn_ring_fwd_static: part of the library's device image, so
// that the entry point needs no allocation and no caller-owned workspace.  Every GPU the library
// runs on holds its own copy at its own address; host code must never use the array's name as an
// address (on the host it is a stand-in for the symbol), only what hipGetSymbolAddress returns
// with the device in question current.
static __device__ __align__(256) unsigned char scratch[WE_STATIC_SCRATCH_BYTES];

namespace {

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* ptr[kMaxDevices] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return WE_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return WE_ERR_LAUNCH;
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return WE_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int elem_bytes(int dtype) { return dtype == WE_DTYPE_F32 ? 4 : 2; }

// element strides whose byte value keeps every row start 16-byte aligned
bool strides_ok(const int64_t s[3], int dtype) {
  const int per16 = 16 / elem_bytes(dtype);
  return s[0] % per16 == 0 && s[1] % per16 == 0 && s[2] % per16 == 0;
}

int ring_shape_ok(int B, int H, int Hkv, int T, int Dh, int64_t L, int dilation) {
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

// Pick the kernel shape and the context splitting.
//  * Shape: 256 queries per workgroup when that alone gives at least one workgroup per CU, else
//    128 queries (two wavefronts share each query block and split every tile's keys).
//  * Few workgroups (256-token frames): every unit is split into the same number of context
//    parts - as many as fit the CUs in one round up to four parts, then as many as give 160 to
//    240 workgroups (more for long contexts, fewer for many parts) - but never fewer than two
//    64-key tiles per part.
//  * Many workgroups that do not divide into whole rounds of 256 CUs (e.g. 384): only the units
//    of the last, partial round are split, so that round finishes in a fraction of the time.
AttnPlan plan_attn(int B, int H, int Hkv, int T, int64_t L, int n_splits, int variant) {
  AttnPlan pl;
  const int64_t wg256 = (int64_t)B * H * ((T + 255) / 256);
  const int64_t wg128 = (int64_t)B * H * ((T + 127) / 128);
  // 256 queries per workgroup when that alone fills the CUs - or when 128 would spill into a
  // second round that 256 avoids (136 to 256 heads of a 256-token frame: one round of fat
  // workgroups beats one and a bit rounds of thin ones by 5 to 17 %)
  pl.variant = variant ? variant : ((T >= 256 && (wg256 >= 256 || wg128 > 256)) ? 2 : 1);
  pl.block_m = pl.variant == 2 ? 256 : 128;
  const int units = B * Hkv;
  const int members = (H / Hkv) * ((T + pl.block_m - 1) / pl.block_m);
  const int64_t wgs = (int64_t)units * members;
  const int64_t tiles = L / 64;  // visible 64-key tiles at steady state
  const int64_t max_s = tiles / 2 > 0 ? tiles / 2 : 1;
  pl.units_whole = 0;
  pl.n_splits = 1;
  if (n_splits > 0) {
    pl.n_splits = n_splits;
  } else if (wgs < 256) {
    // Never more workgroups than CUs (a second, nearly empty round costs a whole kernel's
    // time); and when the context is cut four ways or more, fewer workgroups than CUs: a part's
    // fixed costs do not shrink with its length, the partial results grow with the number of
    // parts, and the board clocks the kernel lower the more CUs are busy (cfg1: 6 parts 25.1 us
    // per frame-step, 8 parts 27.2; 24 rings: 653 against 717).  Measured over 8 to 160
    // workgroups per call: the best count is about 240 workgroups for up to six parts and about
    // 192 for more.
    // Long contexts (32 slots of a 256-token frame and more) amortise the extra parts and the lower
    // clock over longer loops: about 240 workgroups there too (cfg4: 7 parts 32.0 us per frame-step,
    // 6 parts 32.8), and all 256 when that is exactly four parts (64 workgroups: 4 parts beat 3 by
    // 2 to 7 %).
    // Beyond sixteen parts every part's own cost weighs more: about 160 workgroups (4 heads: 20
    // parts 21.2 to 27.2 us per frame-step over 16 to 64 slots, 24 parts 21.7 to 27.4).
    int64_t s = 256 / wgs;
    if (s > 4) s = ((wgs >= 40 || (tiles >= 96 && 240 / wgs <= 16)) ? 240 : (192 / wgs > 16 ? 160 : 192)) / wgs;
    if (s > max_s) s = max_s;
    if (s > 64) s = 64;
    if (s < 1) s = 1;
    pl.n_splits = (int)s;
  } else if (wgs < 4 * 256 && members <= 256) {
    const int whole_units = (int)((wgs / 256) * 256 / members);
    const int64_t rem_wgs = (int64_t)(units - whole_units) * members;
    if (rem_wgs > 0 && rem_wgs <= 128) {
      int64_t s = 256 / rem_wgs;
      if (s > 8) s = 8;
      if (s > max_s / 2) s = max_s / 2;
      if (s > 1) {
        pl.n_splits = (int)s;
        pl.units_whole = whole_units;
      }
    }
  }
  pl.ws_rows = pl.n_splits > 1 ? (int64_t)(units - pl.units_whole) * (H / Hkv) * T : 0;
  return pl;
}

int variant_of(int q_tile) {
  switch (q_tile) {
    case 0: return 0;
    case 128: return 1;
    case 256: return 2;
    default: return -1;
  }
}

// Validation of a we_rope_kv_store call and its kernel parameters.
int prepare_store(const void* q, const void* k, const void* v, const int64_t* q_strides, const int64_t* k_strides,
                  const int64_t* v_strides, void* q_out, const float* cos_table, const float* sin_table,
                  int64_t table_rows, const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                  int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written, int B, int H,
                  int Hkv, int T, int Dh, int64_t L, int dilation, int is_frozen, int dtype, we::StoreParams& p) {
  if (!k || !v || !k_strides || !v_strides || !t_pos || !kv || !written) return WE_ERR_NULL_POINTER;
  if ((q == nullptr) != (q_out == nullptr)) return WE_ERR_NULL_POINTER;
  if (q && !q_strides) return WE_ERR_NULL_POINTER;
  if ((cos_table == nullptr) != (sin_table == nullptr)) return WE_ERR_NULL_POINTER;
  if (cos_table && (!y_pos || !x_pos)) return WE_ERR_NULL_POINTER;
  if (dtype != WE_DTYPE_BF16 && dtype != WE_DTYPE_F16 && dtype != WE_DTYPE_F32) return WE_ERR_UNSUPPORTED;
  int rc = ring_shape_ok(B, H, Hkv, T, Dh, L, dilation);
  if (rc != WE_OK) return rc;
  if (Dh % 16 != 0) return WE_ERR_UNSUPPORTED;
  if (cos_table && (table_rows <= 0 || grid_h <= 0 || grid_w <= 0)) return WE_ERR_BAD_SHAPE;
  if (!aligned16(k) || !aligned16(v) || !aligned16(kv) || (q && (!aligned16(q) || !aligned16(q_out))) ||
      (cos_table && (!aligned16(cos_table) || !aligned16(sin_table))))
    return WE_ERR_ALIGNMENT;
  if (!strides_ok(k_strides, dtype) || !strides_ok(v_strides, dtype) || (q && !strides_ok(q_strides, dtype)))
    return WE_ERR_ALIGNMENT;

  p.q = q; p.k = k; p.v = v; p.q_out = q_out; p.kv = kv; p.written = written;
  p.cos_t = cos_table; p.sin_t = sin_table;
  p.t_pos = t_pos; p.y_pos = y_pos; p.x_pos = x_pos;
  p.qs_b = q ? q_strides[0] : 0; p.qs_h = q ? q_strides[1] : 0; p.qs_t = q ? q_strides[2] : 0;
  p.ks_b = k_strides[0]; p.ks_h = k_strides[1]; p.ks_t = k_strides[2];
  p.vs_b = v_strides[0]; p.vs_h = v_strides[1]; p.vs_t = v_strides[2];
  p.pos_stride_b = pos_stride_b;
  p.table_rows = table_rows;
  p.grid_hw = grid_h * grid_w; p.grid_w = grid_w;
  p.cpr_shift = -1;
  for (int sh = 0; sh < 16; ++sh)
    if ((Dh >> 4) == (1 << sh)) p.cpr_shift = sh;
  p.L = L;
  p.B = B; p.H = H; p.Hkv = Hkv; p.T = T; p.Dh = Dh;
  p.dilation = dilation; p.num_buckets = (int)((L / T) / dilation); p.frozen = is_frozen ? 1 : 0;
  p.norm_eps = 0.f; p.v1 = nullptr; p.v_lamb = nullptr; p.v1s_b = p.v1s_h = p.v1s_t = 0;
  return WE_OK;
}

// Validation of a we_attn_ring_fwd call, its plan and its kernel parameters.
int prepare_attn(const void* q, const int64_t* q_strides, const void* kv, const uint8_t* written,
                 const int64_t* t_pos, void* out, const int64_t* out_strides, void* workspace, size_t workspace_bytes,
                 int B, int H, int Hkv, int T, int Dh, int64_t L, int dilation, float scale, int n_splits, int q_tile,
                 int dtype, we::AttnParams& p, AttnPlan& pl) {
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

  pl = plan_attn(B, H, Hkv, T, L, n_splits, variant_of(q_tile));
  const size_t ws_need = (size_t)pl.n_splits * (size_t)pl.ws_rows * ((size_t)Dh * 2 + 4 * sizeof(float));
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

// Validation of the projection operands and the parameters of the fused projection + store kernel.
int prepare_proj(const we_qkv_proj* proj, void* q_out, const float* cos_table, const float* sin_table,
                 int64_t table_rows, const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                 int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written, int B, int H,
                 int Hkv, int T, int Dh, int64_t L, int dilation, int is_frozen, int dtype,
                 const we_attn_extras* extras, we::ProjParams& pp) {
  if (!proj || !proj->x || !proj->w || !q_out || !cos_table || !sin_table || !y_pos || !x_pos || !t_pos || !kv ||
      !written)
    return WE_ERR_NULL_POINTER;
  if (dtype != WE_DTYPE_BF16 && dtype != WE_DTYPE_F16) return WE_ERR_UNSUPPORTED;
  int rc = ring_shape_ok(B, H, Hkv, T, Dh, L, dilation);
  if (rc != WE_OK) return rc;
  if (proj->d_model <= 0 || table_rows <= 0 || grid_h <= 0 || grid_w <= 0) return WE_ERR_BAD_SHAPE;
  const int64_t feats = (int64_t)(H + 2 * Hkv) * Dh;
  if ((Dh != 64 && Dh != 128) || proj->d_model % 128 != 0 || feats % 128 != 0 || feats / 128 > (1 << 20))
    return WE_ERR_UNSUPPORTED;
  if (proj->w_row_stride < proj->d_model || proj->x_strides[1] < proj->d_model) return WE_ERR_BAD_SHAPE;
  // per-lane offsets are 32-bit: a frame of x and a 128-row slab of w stay below 2 GiB
  if ((uint64_t)T * (uint64_t)proj->x_strides[1] * 2u >= (1ull << 31) ||
      128ull * (uint64_t)proj->w_row_stride * 2u >= (1ull << 31))
    return WE_ERR_UNSUPPORTED;
  const int64_t m_tiles = (T + 63) / 64;
  if (m_tiles * B * 8 * ((feats / 128 + 7) / 8) >= (1ll << 31)) return WE_ERR_UNSUPPORTED;
  if (!aligned16(proj->x) || !aligned16(proj->w) || !aligned16(q_out) || !aligned16(kv) || !aligned16(cos_table) ||
      !aligned16(sin_table) || proj->x_strides[0] % 8 != 0 || proj->x_strides[1] % 8 != 0 || proj->w_row_stride % 8 != 0)
    return WE_ERR_ALIGNMENT;
  if (proj->v_out && (!aligned16(proj->v_out) || !strides_ok(proj->v_out_strides, dtype))) return WE_ERR_ALIGNMENT;

  we::StoreParams& p = pp.s;
  p = we::StoreParams{};
  p.q_out = q_out; p.kv = kv; p.written = written;
  p.cos_t = cos_table; p.sin_t = sin_table;
  p.t_pos = t_pos; p.y_pos = y_pos; p.x_pos = x_pos;
  p.pos_stride_b = pos_stride_b;
  p.table_rows = table_rows;
  p.grid_hw = grid_h * grid_w; p.grid_w = grid_w;
  p.cpr_shift = Dh == 128 ? 3 : 2;
  p.L = L;
  p.B = B; p.H = H; p.Hkv = Hkv; p.T = T; p.Dh = Dh;
  p.dilation = dilation; p.num_buckets = (int)((L / T) / dilation); p.frozen = is_frozen ? 1 : 0;
  if (extras) {
    const we_attn_extras& x = *extras;
    if (x.qk_norm_eps < 0.f || x.qk_norm_eps != x.qk_norm_eps) return WE_ERR_BAD_SHAPE;
    if ((x.v1 == nullptr) != (x.v_lamb == nullptr)) return WE_ERR_NULL_POINTER;
    if (x.v1 && (!aligned16(x.v1) || !strides_ok(x.v1_strides, dtype))) return WE_ERR_ALIGNMENT;
    p.norm_eps = x.qk_norm_eps;
    p.v1 = x.v1; p.v_lamb = x.v_lamb;
    p.v1s_b = x.v1_strides[0]; p.v1s_h = x.v1_strides[1]; p.v1s_t = x.v1_strides[2];
  }
  pp.x = proj->x; pp.xs_b = proj->x_strides[0]; pp.xs_t = proj->x_strides[1];
  pp.w = proj->w; pp.ws_n = proj->w_row_stride;
  pp.K = proj->d_model;
  pp.v_out = proj->v_out;
  pp.vo_b = proj->v_out ? proj->v_out_strides[0] : 0;
  pp.vo_h = proj->v_out ? proj->v_out_strides[1] : 0;
  pp.vo_t = proj->v_out ? proj->v_out_strides[2] : 0;
  pp.m_tiles = (int)m_tiles;
  pp.n_tiles = (int)(feats / 128);
  return WE_OK;
}

// the attention module's gate arguments of `extras`
int apply_gate_extras(const we_attn_extras* extras, int dtype, we::AttnParams& p) {
  if (!extras) return WE_OK;
  const we_attn_extras& x = *extras;
  if ((x.gate_x == nullptr) != (x.gate_w == nullptr)) return WE_ERR_NULL_POINTER;
  if (x.gate_w != nullptr && (x.gate != nullptr || dtype == WE_DTYPE_F32)) return WE_ERR_UNSUPPORTED;
  p.gate = x.gate;
  p.gs_b = x.gate_strides[0]; p.gs_h = x.gate_strides[1]; p.gs_t = x.gate_strides[2];
  p.gate_x = x.gate_x; p.gate_w = x.gate_w;
  p.gx_b = x.gate_x_strides[0]; p.gx_t = x.gate_x_strides[1];
  return WE_OK;
}

int launch_attn(const we::AttnParams& p, const AttnPlan& pl, int Dh, int dtype, hipStream_t st) {
  if (dtype == WE_DTYPE_F32) return we::launch_attn_ring_f32(p, Dh, st) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
  const int ksplit = pl.variant == 1 ? 2 : 1;
  hipError_t e;
  if (dtype == WE_DTYPE_BF16) e = Dh == 128 ? we::launch_attn_ring_bf16_128(p, ksplit, st) : we::launch_attn_ring_bf16_64(p, ksplit, st);
  else e = Dh == 128 ? we::launch_attn_ring_f16_128(p, ksplit, st) : we::launch_attn_ring_f16_64(p, ksplit, st);
  if (e != hipSuccess) return WE_ERR_LAUNCH;
  if (pl.n_splits > 1 && we::launch_attn_combine(p, Dh, dtype, st) != hipSuccess) return WE_ERR_LAUNCH;
  return WE_OK;
}

}  // namespace

extern "C" {

int we_version(void) { return 100; }

const char* we_error_string(int code) {
  switch (code) {
    case WE_OK: return "ok";
    case WE_ERR_NULL_POINTER: return "required pointer is NULL";
    case WE_ERR_BAD_SHAPE: return "inconsistent sizes (need sizes > 0, H % Hkv == 0, L % T == 0, (L/T) % dilation == 0)";
    case WE_ERR_UNSUPPORTED: return "head dim, frame length, slot count or dtype not covered by the kernels";
    case WE_ERR_ALIGNMENT: return "pointer or stride breaks 16-byte alignment";
    case WE_ERR_WORKSPACE: return "split-context workspace missing or too small";
    case WE_ERR_LAUNCH: return "HIP runtime refused the kernel launch";
    case WE_ERR_SCRATCH_LIMIT: return "sizes need more split-context scratch than the library's static buffer (WE_STATIC_SCRATCH_BYTES) holds";
    default: return "unknown error code";
  }
}

int we_rope_kv_store(const void* q, const void* k, const void* v, const int64_t q_strides[3],
                     const int64_t k_strides[3], const int64_t v_strides[3], void* q_out,
                     const float* cos_table, const float* sin_table, int64_t table_rows,
                     const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                     int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written,
                     int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                     int32_t dilation, int32_t is_frozen, int32_t dtype, void* stream) {
  we::StoreParams p;
  const int rc = prepare_store(q, k, v, q_strides, k_strides, v_strides, q_out, cos_table, sin_table, table_rows,
                               t_pos, y_pos, x_pos, pos_stride_b, grid_h, grid_w, kv, written, B, H, Hkv, T, Dh,
                               L, dilation, is_frozen, dtype, p);
  if (rc != WE_OK) return rc;
  return we::launch_rope_kv_store(p, dtype, static_cast<hipStream_t>(stream)) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
}

int we_rope_apply(const void* x, const int64_t x_strides[3], void* x_out, const float* cos_table,
                  const float* sin_table, int64_t table_rows, const int64_t* t_pos, const int64_t* y_pos,
                  const int64_t* x_pos, int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, int32_t B,
                  int32_t H, int32_t T, int32_t Dh, int32_t dtype, void* stream) {
  if (!x || !x_strides || !x_out || !cos_table || !sin_table || !t_pos || !y_pos || !x_pos)
    return WE_ERR_NULL_POINTER;
  if (dtype != WE_DTYPE_BF16 && dtype != WE_DTYPE_F16 && dtype != WE_DTYPE_F32) return WE_ERR_UNSUPPORTED;
  if (B <= 0 || H <= 0 || T <= 0 || Dh <= 0 || table_rows <= 0 || grid_h <= 0 || grid_w <= 0)
    return WE_ERR_BAD_SHAPE;
  if (Dh % 16 != 0) return WE_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(x_out) || !aligned16(cos_table) || !aligned16(sin_table) ||
      !strides_ok(x_strides, dtype))
    return WE_ERR_ALIGNMENT;
  we::StoreParams p = {};
  p.q = x; p.q_out = x_out;
  p.cos_t = cos_table; p.sin_t = sin_table;
  p.t_pos = t_pos; p.y_pos = y_pos; p.x_pos = x_pos;
  p.qs_b = x_strides[0]; p.qs_h = x_strides[1]; p.qs_t = x_strides[2];
  p.pos_stride_b = pos_stride_b;
  p.table_rows = table_rows;
  p.grid_hw = grid_h * grid_w; p.grid_w = grid_w;
  p.cpr_shift = -1;
  for (int sh = 0; sh < 16; ++sh)
    if ((Dh >> 4) == (1 << sh)) p.cpr_shift = sh;
  p.L = T;
  p.B = B; p.H = H; p.Hkv = 0; p.T = T; p.Dh = Dh;
  p.dilation = 1; p.num_buckets = 1; p.frozen = 1;
  return we::launch_rope_kv_store(p, dtype, static_cast<hipStream_t>(stream)) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
}

int32_t we_attn_auto_splits(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L) {
  (void)Dh;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv != 0 || T <= 0 || L <= 0) return 1;
  return plan_attn(B, H, Hkv, T, L, 0, 0).n_splits;
}

size_t we_attn_workspace_bytes(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                               int32_t n_splits, int32_t q_tile) {
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv != 0 || T <= 0 || Dh <= 0 || L <= 0 || n_splits < 0) return 0;
  const int variant = variant_of(q_tile);
  if (variant < 0) return 0;
  const AttnPlan pl = plan_attn(B, H, Hkv, T, L, n_splits, variant);
  return (size_t)pl.n_splits * (size_t)pl.ws_rows * ((size_t)Dh * 2 + 4 * sizeof(float));
}

int we_attn_ring_fwd(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                     const int64_t* t_pos, void* out, const int64_t out_strides[3], void* workspace,
                     size_t workspace_bytes, int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh,
                     int64_t L, int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                     int32_t dtype, void* stream) {
  we::AttnParams p;
  AttnPlan pl;
  const int rc = prepare_attn(q, q_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B, H,
                              Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return launch_attn(p, pl, Dh, dtype, st);
}

int we_attn_ring_fwd_clocked(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                             const int64_t* t_pos, void* out, const int64_t out_strides[3], void* workspace,
                             size_t workspace_bytes, int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh,
                             int64_t L, int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                             int32_t dtype, uint64_t* clocks, size_t clocks_len, void* stream) {
  if (!clocks) return WE_ERR_NULL_POINTER;
  if (dtype == WE_DTYPE_F32) return WE_ERR_UNSUPPORTED;
  we::AttnParams p;
  AttnPlan pl;
  const int rc = prepare_attn(q, q_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B, H,
                              Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  const size_t wgs = (size_t)(8 * p.q_tiles) * (size_t)p.group * (size_t)((p.unit_splits + 7) / 8);
  if (clocks_len < 2 * wgs) return WE_ERR_WORKSPACE;
  p.clock_out = clocks;
  return launch_attn(p, pl, Dh, dtype, static_cast<hipStream_t>(stream));
}

int we_stream_probe(const void* buf, size_t buf_bytes, int32_t workgroups, int32_t tiles, int32_t share, void* stream) {
  if (!buf) return WE_ERR_NULL_POINTER;
  if (workgroups <= 0 || workgroups % 8 != 0 || workgroups > 65536 || tiles <= 0 || tiles > 65536 || share <= 0 ||
      (workgroups / 8) % share != 0)
    return WE_ERR_BAD_SHAPE;
  if (!aligned16(buf)) return WE_ERR_ALIGNMENT;
  const uint64_t region = (uint64_t)tiles * 16384u;
  if (region >= (1ull << 32)) return WE_ERR_UNSUPPORTED;  // 32-bit DMA offsets within a region
  if ((uint64_t)(workgroups / share) * region > buf_bytes) return WE_ERR_WORKSPACE;
  return we::launch_stream_probe(buf, workgroups, tiles, share, static_cast<hipStream_t>(stream)) == hipSuccess
             ? WE_OK : WE_ERR_LAUNCH;
}

int we_attn_ring_fwd_static(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                            const int64_t* t_pos, void* out, const int64_t out_strides[3], int32_t B, int32_t H,
                            int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t dilation, float scale,
                            int32_t n_splits, int32_t q_tile, int32_t dtype, void* stream) {
  // sizes first, so that a call that cannot fit is refused before anything else happens
  if (B > 0 && H > 0 && Hkv > 0 && H % Hkv == 0 && T > 0 && Dh > 0 && L > 0 && n_splits >= 0 && variant_of(q_tile) >= 0 &&
      dtype != WE_DTYPE_F32) {
    const AttnPlan sz = plan_attn(B, H, Hkv, T, L, n_splits, variant_of(q_tile));
    const unsigned long long need =
        (unsigned long long)sz.n_splits * (unsigned long long)sz.ws_rows * ((unsigned long long)Dh * 2 + 4 * sizeof(float));
    if (need > WE_STATIC_SCRATCH_BYTES) return WE_ERR_SCRATCH_LIMIT;
  }
  void* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc != WE_OK) return rc;
  we::AttnParams p;
  AttnPlan pl;
  rc = prepare_attn(q, q_strides, kv, written, t_pos, out, out_strides, ws, WE_STATIC_SCRATCH_BYTES, B, H, Hkv, T, Dh,
                    L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  return launch_attn(p, pl, Dh, dtype, static_cast<hipStream_t>(stream));
}

int we_rope_kv_attn_fwd(const void* q, const void* k, const void* v, const int64_t q_strides[3],
                        const int64_t k_strides[3], const int64_t v_strides[3], void* q_out,
                        const float* cos_table, const float* sin_table, int64_t table_rows,
                        const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos, int64_t pos_stride_b,
                        int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written, void* out,
                        const int64_t out_strides[3], void* workspace, size_t workspace_bytes, int32_t B,
                        int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t dilation,
                        int32_t is_frozen, float scale, int32_t n_splits, int32_t q_tile, int32_t dtype,
                        const we_attn_extras* extras, void* stream) {
  if (!q || !q_out || !cos_table) return WE_ERR_NULL_POINTER;
  we::StoreParams sp;
  int rc = prepare_store(q, k, v, q_strides, k_strides, v_strides, q_out, cos_table, sin_table, table_rows, t_pos,
                         y_pos, x_pos, pos_stride_b, grid_h, grid_w, kv, written, B, H, Hkv, T, Dh, L, dilation,
                         is_frozen, dtype, sp);
  if (rc != WE_OK) return rc;
  // the attention reads the rotated q the store leaves in q_out, contiguous [B, H, T, Dh]
  const int64_t qo_strides[3] = {(int64_t)H * T * Dh, (int64_t)T * Dh, (int64_t)Dh};
  we::AttnParams p;
  AttnPlan pl;
  rc = prepare_attn(q_out, qo_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B, H, Hkv,
                    T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  if (extras) {
    const we_attn_extras& x = *extras;
    if (x.qk_norm_eps < 0.f || x.qk_norm_eps != x.qk_norm_eps) return WE_ERR_BAD_SHAPE;
    if (x.qk_norm_eps > 0.f && (sp.cpr_shift < 0 || (Dh >> 4) > 64)) return WE_ERR_UNSUPPORTED;
    if ((x.v1 == nullptr) != (x.v_lamb == nullptr)) return WE_ERR_NULL_POINTER;
    if (x.v1 && (!aligned16(x.v1) || !strides_ok(x.v1_strides, dtype))) return WE_ERR_ALIGNMENT;
    sp.norm_eps = x.qk_norm_eps;
    sp.v1 = x.v1; sp.v_lamb = x.v_lamb;
    sp.v1s_b = x.v1_strides[0]; sp.v1s_h = x.v1_strides[1]; sp.v1s_t = x.v1_strides[2];
    rc = apply_gate_extras(extras, dtype, p);
    if (rc != WE_OK) return rc;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Everything is validated before the first launch; the kernels follow each other on the stream.
  if (we::launch_rope_kv_store(sp, dtype, st) != hipSuccess) return WE_ERR_LAUNCH;
  return launch_attn(p, pl, Dh, dtype, st);
}

int we_qkv_rope_kv_store(const we_qkv_proj* proj, void* q_out, const float* cos_table, const float* sin_table,
                         int64_t table_rows, const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                         int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written, int32_t B,
                         int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t dilation,
                         int32_t is_frozen, int32_t dtype, const we_attn_extras* extras, void* stream) {
  we::ProjParams pp;
  const int rc = prepare_proj(proj, q_out, cos_table, sin_table, table_rows, t_pos, y_pos, x_pos, pos_stride_b, grid_h,
                              grid_w, kv, written, B, H, Hkv, T, Dh, L, dilation, is_frozen, dtype, extras, pp);
  if (rc != WE_OK) return rc;
  return we::launch_qkv_rope_store(pp, dtype, static_cast<hipStream_t>(stream)) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
}

int we_qkv_rope_kv_attn_fwd(const we_qkv_proj* proj, void* q_out, const float* cos_table, const float* sin_table,
                            int64_t table_rows, const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                            int64_t pos_stride_b, int64_t grid_h, int64_t grid_w, void* kv, uint8_t* written,
                            void* out, const int64_t out_strides[3], void* workspace, size_t workspace_bytes,
                            int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t dilation,
                            int32_t is_frozen, float scale, int32_t n_splits, int32_t q_tile, int32_t dtype,
                            const we_attn_extras* extras, void* stream) {
  we::ProjParams pp;
  int rc = prepare_proj(proj, q_out, cos_table, sin_table, table_rows, t_pos, y_pos, x_pos, pos_stride_b, grid_h,
                        grid_w, kv, written, B, H, Hkv, T, Dh, L, dilation, is_frozen, dtype, extras, pp);
  if (rc != WE_OK) return rc;
  const int64_t qo_strides[3] = {(int64_t)H * T * Dh, (int64_t)T * Dh, (int64_t)Dh};
  we::AttnParams p;
  AttnPlan pl;
  rc = prepare_attn(q_out, qo_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B, H, Hkv,
                    T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  rc = apply_gate_extras(extras, dtype, p);
  if (rc != WE_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (we::launch_qkv_rope_store(pp, dtype, st) != hipSuccess) return WE_ERR_LAUNCH;
  return launch_attn(p, pl, Dh, dtype, st);
}

}  // extern "C"
