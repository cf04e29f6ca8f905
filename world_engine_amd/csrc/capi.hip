// C ABI of the ring-buffer attention library: argument validation and kernel dispatch.
// Declarations and the reference call sites each entry point replaces: include/we_attn.h.
#include "../../include/we_attn.h"
#include "attn_plan.h"
#include "device_state.h"
#include "we_kernels.h"

namespace {

using we::host::aligned16;
using we::host::AttnPlan;
using we::host::DeviceState;
using we::host::launch_attn;
using we::host::plan_attn;
using we::host::ring_shape_ok;
using we::host::strides_ok;
using we::host::variant_of;
using we::host::workspace_bytes_of;

// The device a call will run on.  Without one (or while its set-up is impossible: first use under
// stream capture) `rc` says why, and `state` is a stand-in so that argument errors are still
// reported first.
struct Dev {
  int rc;
  DeviceState state;
};
Dev dev_for(hipStream_t st) {
  const DeviceState* ds = nullptr;
  Dev d;
  d.rc = we::host::device_state(st, &ds);
  d.state = ds ? *ds : DeviceState{256, nullptr};
  return d;
}

// prepare_attn for the device the call will run on
int prepare_attn(const DeviceState& ds, const void* q, const int64_t* q_strides, const void* kv, const uint8_t* written,
                 const int64_t* t_pos, void* out, const int64_t* out_strides, void* workspace, size_t workspace_bytes,
                 int B, int H, int Hkv, int T, int Dh, int64_t L, int dilation, float scale, int n_splits, int q_tile,
                 int dtype, we::AttnParams& p, AttnPlan& pl) {
  return we::host::prepare_attn(q, q_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B, H,
                                Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, ds.cus, p, pl);
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
    case WE_ERR_NOT_READY: return "first call on this device made under stream capture: call we_init() on the device beforehand";
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

int we_init(void) { return we::host::init_current_device(); }

int32_t we_attn_auto_splits(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L) {
  (void)Dh;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv != 0 || T <= 0 || L <= 0) return 1;
  return plan_attn(B, H, Hkv, T, L, 0, 0, we::host::compute_units()).n_splits;
}

size_t we_attn_workspace_bytes(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                               int32_t n_splits, int32_t q_tile) {
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv != 0 || T <= 0 || Dh <= 0 || L <= 0 || n_splits < 0) return 0;
  const int variant = variant_of(q_tile);
  if (variant < 0) return 0;
  return workspace_bytes_of(plan_attn(B, H, Hkv, T, L, n_splits, variant, we::host::compute_units()), Dh);
}

int we_attn_plan(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t n_splits,
                 int32_t q_tile, int32_t compute_units, int32_t plan[WE_PLAN_FIELDS]) {
  if (!plan) return WE_ERR_NULL_POINTER;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv != 0 || T <= 0 || Dh <= 0 || L <= 0 || L % T != 0 || n_splits < 0 ||
      n_splits > 64 || compute_units < 0)
    return WE_ERR_BAD_SHAPE;
  const int variant = variant_of(q_tile);
  if (variant < 0) return WE_ERR_UNSUPPORTED;
  const int cus = compute_units > 0 ? compute_units : we::host::compute_units();
  const AttnPlan pl = plan_attn(B, H, Hkv, T, L, n_splits, variant, cus);
  const int q_tiles = (T + pl.block_m - 1) / pl.block_m;
  const int64_t wgs = (int64_t)q_tiles * (H / Hkv) * (pl.units_whole + (int64_t)(B * Hkv - pl.units_whole) * pl.n_splits);
  plan[0] = pl.block_m;
  plan[1] = pl.n_splits;
  plan[2] = pl.units_whole;
  plan[3] = (int32_t)(wgs > 0x7fffffff ? 0x7fffffff : wgs);
  plan[4] = cus;
  return WE_OK;
}

int we_attn_ring_fwd(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                     const int64_t* t_pos, void* out, const int64_t out_strides[3], void* workspace,
                     size_t workspace_bytes, int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh,
                     int64_t L, int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                     int32_t dtype, void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Dev dev = dev_for(st);
  we::AttnParams p;
  AttnPlan pl;
  const int rc = prepare_attn(dev.state, q, q_strides, kv, written, t_pos, out, out_strides, workspace,
                              workspace_bytes, B, H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  if (dev.rc != WE_OK) return dev.rc;
  return launch_attn(p, pl, Dh, dtype, st);
}

int we_attn_ring_fwd_static(const void* q, const int64_t q_strides[3], const void* kv, const uint8_t* written,
                            const int64_t* t_pos, void* out, const int64_t out_strides[3], int32_t B, int32_t H,
                            int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t dilation, float scale,
                            int32_t n_splits, int32_t q_tile, int32_t dtype, void* stream) {
  // sizes first, so that a call that cannot fit is refused before anything else happens
  if (we_attn_workspace_bytes(B, H, Hkv, T, Dh, L, n_splits, q_tile) > WE_STATIC_SCRATCH_BYTES && dtype != WE_DTYPE_F32)
    return WE_ERR_SCRATCH_LIMIT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Dev dev = dev_for(st);
  // (a stand-in address keeps the argument checks of a call without a device those of we_attn_ring_fwd)
  void* ws = dev.state.scratch ? dev.state.scratch : reinterpret_cast<void*>(uintptr_t{4096});
  we::AttnParams p;
  AttnPlan pl;
  const int rc = prepare_attn(dev.state, q, q_strides, kv, written, t_pos, out, out_strides, ws,
                              WE_STATIC_SCRATCH_BYTES, B, H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  if (dev.rc != WE_OK) return dev.rc;
  return launch_attn(p, pl, Dh, dtype, st);
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Dev dev = dev_for(st);
  we::AttnParams p;
  AttnPlan pl;
  rc = prepare_attn(dev.state, q_out, qo_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B,
                    H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
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
  if (dev.rc != WE_OK) return dev.rc;
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Dev dev = dev_for(st);  // (the kernel's LDS limit is raised by the device's set-up)
  if (dev.rc != WE_OK) return dev.rc;
  return we::launch_qkv_rope_store(pp, dtype, st) == hipSuccess ? WE_OK : WE_ERR_LAUNCH;
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  const Dev dev = dev_for(st);
  we::AttnParams p;
  AttnPlan pl;
  rc = prepare_attn(dev.state, q_out, qo_strides, kv, written, t_pos, out, out_strides, workspace, workspace_bytes, B,
                    H, Hkv, T, Dh, L, dilation, scale, n_splits, q_tile, dtype, p, pl);
  if (rc != WE_OK) return rc;
  rc = apply_gate_extras(extras, dtype, p);
  if (rc != WE_OK) return rc;
  if (dev.rc != WE_OK) return dev.rc;
  if (we::launch_qkv_rope_store(pp, dtype, st) != hipSuccess) return WE_ERR_LAUNCH;
  return launch_attn(p, pl, Dh, dtype, st);
}

}  // extern "C"
