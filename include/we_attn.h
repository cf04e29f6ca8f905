/*
 * we_attn.h - C ABI of the MI355X (gfx950) frame-causal ring-buffer attention library.
 *
 * The library replaces, for one DiT attention layer and one frame, the work world_engine
 * does between its q/k/v projection and its output projection:
 *
 *   RoPE(q), RoPE(k)                      src/model/attn.py:22-40, :110
 *   kv_cache.upsert(k, v, pos_ids, layer) src/model/kv_cache.py:104-154, :191-193
 *   flex_attention(q, k, v, block_mask)   src/model/attn.py:116, src/patch_model.py:133
 *
 * world_engine has no native code: these are the calls a binding would replace with the
 * entry points below.  All pointers are DEVICE pointers owned by the caller.  Every call only
 * enqueues work on `stream`; it never allocates and never synchronises, so it is re-entrant and
 * capturable into a HIP graph once the device it runs on has had its one-time set-up (we_init).
 * The only state the library keeps is what that set-up noted about each device (read-only
 * afterwards).  The frame index that
 * selects the ring slot is read by the kernels from device memory (`t_pos[0]`), exactly as the
 * reference derives it from a device tensor (src/model/kv_cache.py:126), so no host value of
 * it is ever needed.
 *
 * Return value: 0 on success, a negative WE_ERR_* code otherwise (nothing is launched then).
 */
#ifndef WE_ATTN_H
#define WE_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of q/k/v, the cache buffer and the attention output */
#define WE_DTYPE_BF16 0
#define WE_DTYPE_F16 1
#define WE_DTYPE_F32 2 /* fp32 caches: the store rotates in fp32, the attention takes a plain one-pass kernel */

#define WE_OK 0
#define WE_ERR_NULL_POINTER (-1)
#define WE_ERR_BAD_SHAPE (-2)     /* zero/negative sizes, L % T != 0, (L/T) % dilation != 0, H % Hkv != 0 */
#define WE_ERR_UNSUPPORTED (-3)   /* head dim, frame length, slot count or dtype outside what the kernels cover */
#define WE_ERR_ALIGNMENT (-4)     /* pointer or stride not 16-byte aligned */
#define WE_ERR_WORKSPACE (-5)     /* split-context workspace missing or too small */
#define WE_ERR_LAUNCH (-6)        /* the HIP runtime refused the launch */
#define WE_ERR_SCRATCH_LIMIT (-7) /* we_attn_ring_fwd_static: sizes need more scratch than WE_STATIC_SCRATCH_BYTES */
#define WE_ERR_NOT_READY (-8)     /* first call on a device made under stream capture: call we_init() beforehand */

#define WE_MAX_SLOTS 256 /* maximum number of ring slots L / T */

/* size of the library's own split-context scratch buffer (see we_attn_ring_fwd_static) */
#define WE_STATIC_SCRATCH_BYTES (32u << 20)

/* Library version: major*10000 + minor*100 + patch. */
int we_version(void);

/* Static description of a WE_ERR_* code. */
const char* we_error_string(int code);

/*
 * One-time set-up of the CURRENT device (hipSetDevice), without a counterpart in the reference:
 * raises the kernels' dynamic-LDS limits, looks up the static scratch buffer's address and notes
 * the device's compute-unit count.  Launches nothing, does not synchronise; idempotent and
 * thread-safe.  Every entry point that launches does the same implicitly on its first call on a
 * device - except when its stream is being captured (these runtime calls do not belong into a
 * capture), where it returns WE_ERR_NOT_READY instead: callers that capture graphs call we_init()
 * (or make one ordinary call) on the device first.
 */
int we_init(void);

/*
 * Fused RoPE + ring-slot K/V store for one frame.
 *
 * Replaces RoPE.forward on q and k (src/model/attn.py:33-40), torch.stack([k, v])
 * (src/model/kv_cache.py:192), the tail index_copy_ (:138), the unfrozen ring index_copy_ and
 * the `written` update (:147-151), with the slot arithmetic of :126-131,:140 done on the device.
 *
 *   q        [B, H,   T, Dh]  element strides q_strides  = {batch, head, token}; Dh contiguous.
 *                             May be NULL (then q_out must be NULL): K/V store only.
 *   k, v     [B, Hkv, T, Dh]  element strides k_strides / v_strides, same convention.
 *   q_out    [B, H, T, Dh] contiguous: RoPE(q).
 *   cos_table, sin_table  [table_rows, Dh/2] fp32.  Both NULL: no rotation (k is stored as
 *            given, q is copied), which is the behaviour of StaticKVCache.upsert on an already
 *            rotated k.
 *   t_pos, y_pos, x_pos   int64 [B, T], row stride pos_stride_b.  Table row of token (b, i) is
 *            t_pos*grid_h*grid_w + y_pos*grid_w + x_pos (src/model/attn.py:27).  The kernel clamps
 *            it into [0, table_rows) for memory safety only: a row outside the table is a caller
 *            error (the reference's index_select raises there, src/model/attn.py:25-30), which the
 *            Python wrapper checks in eager mode; the C entry point cannot without reading device
 *            memory.  y_pos/x_pos may be NULL when the tables are NULL.
 *            t_pos[0] is the frame index that selects the ring slot.
 *   kv       [2, B, Hkv, L + T, Dh] contiguous cache buffer (plane 0 = K, 1 = V).
 *   written  [L + T] bytes (torch.bool).
 *   L        ring length in tokens (multiple of T); dilation = pinned_dilation, divides L/T.
 *   is_frozen  non-zero: only the tail rows [L, L+T) are written.  Zero: additionally, when
 *            t_pos[0] % dilation == 0, rows [slot*T, (slot+1)*T) with
 *            slot = ceil(t_pos[0]/dilation) % ((L/T)/dilation) are written and marked in
 *            `written`; otherwise the tail is marked.
 *
 * Rotation is computed in fp32 with separately rounded products and rounded once to the
 * element type (round-to-nearest-even), so ring contents are bit-identical to eager PyTorch.
 * Requirements: Dh % 16 == 0; all pointers and row starts 16-byte aligned.
 */
int we_rope_kv_store(const void* q, const void* k, const void* v,
                     const int64_t q_strides[3], const int64_t k_strides[3],
                     const int64_t v_strides[3], void* q_out,
                     const float* cos_table, const float* sin_table, int64_t table_rows,
                     const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                     int64_t pos_stride_b, int64_t grid_h, int64_t grid_w,
                     void* kv, uint8_t* written,
                     int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                     int32_t dilation, int32_t is_frozen, int32_t dtype, void* stream);

/*
 * RoPE alone on one [B, H, T, Dh] tensor: x_out = RoPE(x), x_out contiguous.  Replaces a
 * stand-alone RoPE.forward call (src/model/attn.py:33-40); same arithmetic, arguments and
 * requirements as the rotation inside we_rope_kv_store.
 */
int we_rope_apply(const void* x, const int64_t x_strides[3], void* x_out,
                  const float* cos_table, const float* sin_table, int64_t table_rows,
                  const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                  int64_t pos_stride_b, int64_t grid_h, int64_t grid_w,
                  int32_t B, int32_t H, int32_t T, int32_t Dh, int32_t dtype, void* stream);

/*
 * Number of context parts we_attn_ring_fwd cuts split units into when called with n_splits = 0
 * (1 = nothing is split).  Sizing helper without a counterpart in the reference.
 */
int32_t we_attn_auto_splits(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L);

/*
 * Bytes of split-context workspace we_attn_ring_fwd needs for these sizes and the given n_splits /
 * q_tile arguments (0 when nothing is split).  Depends on the compute-unit count of the current
 * device (256 when there is none to ask).  Sizing helper without a counterpart in the reference.
 */
size_t we_attn_workspace_bytes(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                               int32_t n_splits, int32_t q_tile);

/*
 * What the library would do with an attention call of these sizes (inspection helper without a
 * counterpart in the reference; launches nothing): plan[0] = queries per workgroup, [1] = context
 * parts of the units that are split, [2] = leading (batch, kv head) units left whole, [3] =
 * workgroups of the main launch, [4] = compute units planned for.  compute_units = 0 asks the
 * current device (256 without one).
 */
#define WE_PLAN_FIELDS 5
int we_attn_plan(int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L, int32_t n_splits,
                 int32_t q_tile, int32_t compute_units, int32_t plan[WE_PLAN_FIELDS]);

/*
 * Frame-block-causal attention of one frame's queries over the ring buffer.
 *
 * Replaces make_block_mask (src/model/kv_cache.py:12-61, :141-144) and the flex_attention call
 * (src/model/attn.py:116).  Key row j of the cache is visible iff it lies in the tail
 * [L, L+T), or in a ring slot s with written[s*T] != 0 that is not the slot the current frame
 * maps to on a persisting frame (t_pos[0] % dilation == 0).  Visibility does not depend on
 * batch, head or query, so no mask tensor is materialised: the kernel walks the visible slots
 * of `kv` in place.  out = softmax(scale * q k^T) v over the visible keys, fp32 accumulation,
 * probabilities rounded to the element type before the second product.
 *
 *   q    [B, H, T, Dh]   element strides q_strides = {batch, head, token}; Dh contiguous.
 *   kv, written, t_pos   as in we_rope_kv_store, after that call for the same frame.
 *   out  [B, H, T, Dh]   element strides out_strides = {batch, head, token}; Dh contiguous.
 *   workspace            device scratch of at least we_attn_workspace_bytes(...) bytes for the
 *                        same sizes, n_splits and q_tile; may be NULL when that is 0.  Nothing in
 *                        it has to start at any value; calls that overlap in time need a
 *                        workspace each.
 *   n_splits             0 = choose automatically (small grids: every (batch, kv head) unit is
 *                        split so that most CUs have work; grids that leave a partial last round
 *                        of workgroups: only that round's units are split); 1 = single pass;
 *                        2..64 = split the visible context of every unit into that many parts.
 *                        Split parts are combined by a second kernel.
 *   q_tile               queries per workgroup: 0 = choose automatically, or 128 / 256.
 *   scale                softmax scale (> 0); the reference uses 1/sqrt(Dh).
 *
 * Requirements: dtype bf16 or f16 (MFMA kernel) or f32 (plain one-pass kernel on the vector
 * ALUs, fp32 arithmetic throughout, n_splits 0 or 1, q_tile ignored); Dh in {64, 128};
 * any T (frames that are not a multiple of the 64-key tile cost one masked tile per slot);
 * L/T <= WE_MAX_SLOTS; H % Hkv == 0; pointers and row starts 16-byte aligned.
 */
int we_attn_ring_fwd(const void* q, const int64_t q_strides[3],
                     const void* kv, const uint8_t* written, const int64_t* t_pos,
                     void* out, const int64_t out_strides[3],
                     void* workspace, size_t workspace_bytes,
                     int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                     int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                     int32_t dtype, void* stream);

/*
 * we_attn_ring_fwd for callers that cannot allocate device memory, not even a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose attention call allocates through torch as it pleases).
 * Arguments, requirements and results are those of we_attn_ring_fwd, bit for bit, without the
 * workspace pair: the split-context partial results go to a buffer of WE_STATIC_SCRATCH_BYTES that
 * is part of the library's device image (every GPU the library runs on holds one copy until the
 * process ends; its address is looked up once per device by that device's set-up, see we_init:
 * under stream capture the device must have been set up beforehand).  Sizes whose
 * we_attn_workspace_bytes(...) exceeds WE_STATIC_SCRATCH_BYTES are
 * rejected with WE_ERR_SCRATCH_LIMIT and nothing is launched.  The call itself performs no
 * hipMalloc / hipFree and calls no allocating library routine.
 * All calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (different
 * streams, or parallel branches of one graph) race on it; calls that follow each other on a
 * stream do not.  Nothing in the buffer has to start at any value (every partial row a call reads
 * was written by that call's first kernel).
 */
int we_attn_ring_fwd_static(const void* q, const int64_t q_strides[3],
                            const void* kv, const uint8_t* written, const int64_t* t_pos,
                            void* out, const int64_t out_strides[3],
                            int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                            int32_t dilation, float scale, int32_t n_splits, int32_t q_tile,
                            int32_t dtype, void* stream);

/*
 * Optional work of the reference's attention module that sits right in front of and right behind
 * the path and touches the same tiles (src/model/attn.py:105-109,117-119): done inside the two
 * kernels instead of as five to seven element-wise launches per layer.  A zeroed struct (or a
 * NULL pointer to one) switches everything off.
 *   qk_norm_eps  > 0: q and k rows are RMS-normalised without weight before RoPE,
 *                x * rsqrt(mean(x^2) + eps) in fp32, rounded to the element type (F.rms_norm;
 *                torch uses the fp32 machine epsilon for low-precision inputs).  Needs Dh / 16 to
 *                be a power of two <= 64.
 *   v1, v_lamb   v = lerp(v, v1, *v_lamb) before the store (value residual); v1 [B, Hkv, T, Dh]
 *                with element strides v1_strides = {batch, head, token}, v_lamb a device pointer
 *                to one element.  Both NULL = off.
 *   gate         out[b, h, t, :] *= gate[b, h, t] (sigmoid already applied), element strides
 *                gate_strides = {batch, head, token}; the attention output is rounded to the
 *                element type first, as the module's own multiply sees it.  NULL = off.
 *   gate_x, gate_w   instead of `gate`: the gate is computed in the kernels' epilogues as
 *                sigmoid(gate_proj(x[..., :H])) (src/model/attn.py:117-118), which saves the module
 *                a GEMM launch and a sigmoid launch per layer.  gate_x points at x[b, t, 0] of the
 *                module's input [B, T, >= H] (channel stride 1, element strides gate_x_strides =
 *                {batch, token}), gate_w at gate_proj.weight [H, H] row-major (out, in).  The
 *                projection's output and the sigmoid's are rounded to the element type like the
 *                module's tensors.  Both NULL = off; not together with `gate`; bf16 / f16 only.
 * Results equal the separate torch operations up to the last bit of the row reduction, of the
 * lerp's fused multiply-add and of the gate's dot product (1 ulp of the element type); the gate
 * multiply itself is exact.
 */
typedef struct we_attn_extras {
  float qk_norm_eps;
  const void* v1;
  int64_t v1_strides[3];
  const void* v_lamb;
  const void* gate;
  int64_t gate_strides[3];
  const void* gate_x;
  int64_t gate_x_strides[2];
  const void* gate_w;
} we_attn_extras;

/*
 * RoPE + K/V store + attention of one frame in a single call: we_rope_kv_store followed by
 * we_attn_ring_fwd on the rotated q, i.e. the whole per-layer sequence of the reference from
 * `q, k = rope(q), rope(k)` to the flex_attention call (src/model/attn.py:110-116 with
 * src/model/kv_cache.py:126-151).  Arguments, requirements and results (cache rows, `written`,
 * q_out, out) are those of the two calls, bit for bit; q, q_out and the tables are mandatory.
 * Both calls are validated before anything is launched, and a host language pays for one
 * foreign call per layer and frame instead of two.  `extras` (may be NULL) adds the module's
 * element-wise neighbours of the path, see we_attn_extras; q_out then holds RoPE(rms_norm(q)).
 */
int we_rope_kv_attn_fwd(const void* q, const void* k, const void* v,
                        const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                        void* q_out,
                        const float* cos_table, const float* sin_table, int64_t table_rows,
                        const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                        int64_t pos_stride_b, int64_t grid_h, int64_t grid_w,
                        void* kv, uint8_t* written,
                        void* out, const int64_t out_strides[3],
                        void* workspace, size_t workspace_bytes,
                        int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                        int32_t dilation, int32_t is_frozen, float scale, int32_t n_splits, int32_t q_tile,
                        int32_t dtype, const we_attn_extras* extras, void* stream);

/*
 * The module's merged q/k/v projection as the producer of the path (next-row 3 of the scope:
 * `q, k, v = self.qkv_proj(x).split(...)`, src/patch_model.py:116-122, weights merged as in
 * :102-114).  Describes the GEMM operands for we_qkv_rope_kv_store / we_qkv_rope_kv_attn_fwd:
 *   x            module input [B, T, d_model], channel stride 1, element strides x_strides =
 *                {batch, token} (multiples of 8), 16-byte aligned.
 *   w            qkv_proj.weight [(H + 2 Hkv) * Dh, d_model] row-major (out, in): q rows, then k
 *                rows, then v rows; element stride w_row_stride between rows (multiple of 8).
 *   d_model      contraction length, a multiple of 128.
 *   v_out        optional: the projected v rows as the GEMM leaves them (before the value blend),
 *                [B, Hkv, T, Dh] with element strides v_out_strides = {batch, head, token} - what
 *                the first layer hands on as `v1` (src/model/attn.py:107).  NULL = not wanted.
 * The projection accumulates in fp32 and rounds once to the element type, like the GEMM's output
 * tensor; sums are taken in an order fixed by the shapes and the token's 64-token tile (results
 * are reproducible, and exact whenever the fp32 sums are exact) that differs from a BLAS
 * library's, i.e. rows may differ from torch.nn.functional.linear's in the last bit of the
 * element type.  bf16 / f16 only;
 * (H + 2 Hkv) * Dh must be a multiple of 128 and Dh 64 or 128.
 */
typedef struct we_qkv_proj {
  const void* x;
  int64_t x_strides[2];
  const void* w;
  int64_t w_row_stride;
  int32_t d_model;
  void* v_out;
  int64_t v_out_strides[3];
} we_qkv_proj;

/*
 * we_rope_kv_store with the projection in front, in one kernel: computes q, k, v = x W^T tile by
 * tile on the matrix cores and applies the store's work (optional RMS norm and value blend from
 * `extras`, RoPE, q_out, tail / ring-slot rows, `written`) to each tile while it is still on the
 * CU; the [B, T, (H + 2 Hkv) Dh] projection output never exists in memory.  Arguments other than
 * `proj` are those of we_rope_kv_store (q_out and the tables may not be NULL); of `extras` only
 * qk_norm_eps, v1 and v_lamb are used.  Replaces src/patch_model.py:116-122 +
 * src/model/attn.py:105-110 + src/model/kv_cache.py:126-151,192.
 */
int we_qkv_rope_kv_store(const we_qkv_proj* proj, void* q_out,
                         const float* cos_table, const float* sin_table, int64_t table_rows,
                         const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                         int64_t pos_stride_b, int64_t grid_h, int64_t grid_w,
                         void* kv, uint8_t* written,
                         int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                         int32_t dilation, int32_t is_frozen, int32_t dtype,
                         const we_attn_extras* extras, void* stream);

/*
 * we_rope_kv_attn_fwd with the projection in front: we_qkv_rope_kv_store, then we_attn_ring_fwd on
 * the rotated q (two or three launches for everything between the module's input and out_proj).
 * Both are validated before anything is launched.
 */
int we_qkv_rope_kv_attn_fwd(const we_qkv_proj* proj, void* q_out,
                            const float* cos_table, const float* sin_table, int64_t table_rows,
                            const int64_t* t_pos, const int64_t* y_pos, const int64_t* x_pos,
                            int64_t pos_stride_b, int64_t grid_h, int64_t grid_w,
                            void* kv, uint8_t* written,
                            void* out, const int64_t out_strides[3],
                            void* workspace, size_t workspace_bytes,
                            int32_t B, int32_t H, int32_t Hkv, int32_t T, int32_t Dh, int64_t L,
                            int32_t dilation, int32_t is_frozen, float scale, int32_t n_splits, int32_t q_tile,
                            int32_t dtype, const we_attn_extras* extras, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WE_ATTN_H */
