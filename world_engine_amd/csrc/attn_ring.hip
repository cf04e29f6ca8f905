// Frame-block-causal flash attention over the KV ring buffer: 8-wavefront workgroups fed by
// LDS-DMA (gfx950, wave64, MFMA).
//
// Replaces the reference's make_block_mask + flex_attention pair (src/model/kv_cache.py:12-61,
// :141-144; src/model/attn.py:116).  A key row is visible iff it is in the tail [L, L+T) or in
// a ring slot s with written[s*T] set that is not the slot the current frame replaces on a
// persisting frame.  Visibility is per slot and identical for every batch element, head and
// query, so the kernel builds a short list of visible slots and walks those slots of the
// cache buffer in place, 64 keys at a time; no mask tensor and no gathered context exist.
//
// One workgroup = 8 wavefronts = one CU (2 wavefronts per SIMD, so one wavefront's vector work
// overlaps the other's matrix work).  Two shapes:
//   KSPLIT = 1: 256 queries; each wavefront owns 32 queries and handles both 32-key blocks of
//               every tile (large frames).
//   KSPLIT = 2: 128 queries; two wavefronts share a block of 32 queries, each taking one of the
//               two 32-key blocks of every tile, and merge their (reference, sum, O) through LDS
//               at the end.  Twice the parallelism per query without more split-context
//               partials (256-token frames, where the grid alone cannot fill the chip).
// K/V tiles travel HBM -> LDS directly (global_load_lds_dwordx4, no VGPR staging) into rings
// of 4 slots per operand, issued two to three tiles ahead.  LDS tiles are unpadded; bank
// conflicts are avoided by XOR-swizzling 16-byte chunks, applied on the global side of the DMA
// (lane i always lands at LDS offset 16*i) and undone in the fragment addresses.
// Per 32-key block and wavefront:
//   S^T = K Q^T        v_mfma_f32_32x32x16, A = K rows (ds_read_b128), B = Q in registers as
//                      loaded (no scaling, so nothing is rounded in front of the matrix core).
//   P = 2^((S-m) c)    one fused multiply-add per logit applies the softmax scale (c = scale *
//                      log2 e) and the running reference m, then v_exp_f32 + v_cvt_pk +
//                      v_dot2c row sum; each lane owns one query column.
//   O^T += V^T P^T     A = V^T via ds_read_b64_tr_b16, B = P straight from registers.
// The three are software-pipelined across blocks (logits of block i+1 and product of block i-1
// run on the matrix cores while the VALU handles block i); LDS fragment reads are stated up to 15
// reads ahead of their MFMAs, also across steps and barriers, and the order is pinned with
// sched_barrier.  When the workgroup count leaves a partial last round of CUs, only that round's
// (batch, kv head) units are context-split (see the planner in attn_plan.h); split workgroups leave
// normalised partial outputs that a second kernel merges (attn_combine.hip).
//
// The grid is 3-D (8 * query tiles, query heads per kv head, rounds of 8 units): no division by
// run-time values is needed to find a workgroup's unit, and blockIdx.x % 8 is the XCD it runs on,
// so the workgroups that share one K/V stream share an L2.  Start-up code is kept short on purpose:
// a 256-token frame runs 8 tiles per workgroup and start-up is a third of the kernel.
//
// Frame lengths that are not a multiple of 64 use the RAGGED instantiation: the short last tile
// of a slot is loaded with its missing rows clamped and its missing keys masked to -inf.
//
// Roofline: 4*T*N_vis*Dh flops and 4*N_vis*Dh bytes of K/V per (batch, kv head).
#include "attn_mma.h"
#include "device_state.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

#include <type_traits>

namespace we {

template <int DH>
struct RingLds {
  static constexpr int CPR = DH / 8;          // 16-byte chunks per row
  static constexpr int ROW_B = DH * 2;        // bytes per K/V row
  static constexpr int TILE_B = BN * ROW_B;   // bytes per K or V tile
  static constexpr int SLOTS = 4;             // ring slots per operand over all wave groups
  static constexpr int V_OFF = SLOTS * TILE_B;
  static constexpr int MISC_OFF = 2 * SLOTS * TILE_B;
  static constexpr int kBytes = MISC_OFF + 8 * (WE_MAX_SLOTS + 64) * 4;  // + a slot-list strip per wavefront
};

// chunk swizzles: physical 16-byte chunk = logical chunk ^ swz(row)
template <int DH>
__device__ __forceinline__ int k_swz(int row) {
  return DH == 128 ? (row & 15) : ((row >> 1) & 7);
}
template <int DH>
__device__ __forceinline__ int v_swz(int row) {
  return DH == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

template <int V>
struct IntC {
  static constexpr int value = V;
};

// ---- LDS fragment reads ---------------------------------------------------------------------
// Left alone, the compiler keeps a single fragment read in flight ahead of the MFMA that needs
// it, which exposes the full LDS latency on every MFMA.  The hot loop therefore states its reads
// early in program order, several fragments ahead of their MFMAs, and pins that order with
// sched_barrier; the reads stay ordinary loads, so the compiler still places the (counted)
// lgkmcnt waits itself and knows the registers are in flight.
template <int OFF>
__device__ __forceinline__ u32x4_t lds_read128(const unsigned char* smem, uint32_t off) {
  return *reinterpret_cast<const u32x4_t*>(smem + off + OFF);
}
template <int OFF>
__device__ __forceinline__ u32x2_t lds_read_tr(const unsigned char* smem, uint32_t off) {
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(smem + off + OFF));
  return __builtin_bit_cast(u32x2_t, v);
}

// RAGGED: the frame length is not a multiple of the 64-key tile (separate instantiation: the
// masking of the short tiles costs registers the common case cannot spare).
// CLOCKED: measurement library only - every workgroup reports its duration (p.clock_out).
template <typename M, int DH, int KSPLIT, bool RAGGED, bool CLOCKED>
__global__ void __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2)))
attn_ring_kernel(AttnParams p) {
  typedef typename M::frag_t frag_t;
  typedef RingLds<DH> L;
  constexpr int KS = DH / 16;               // contraction steps of K Q^T
  constexpr int DB = DH / 32;               // 32-row blocks of O^T
  constexpr int NV = 2 * DB;                // V^T fragments of one 32-key block
  constexpr int QW = 8 / KSPLIT;            // wavefronts with distinct query blocks
  constexpr int BM = 32 * QW;               // queries per workgroup
  constexpr int NST = 4;                    // ring slots per operand
  constexpr int CPR = L::CPR, ROW_B = L::ROW_B, TILE_B = L::TILE_B;
  constexpr int KB_B = 32 * ROW_B;          // bytes of one 32-key block of a tile
  constexpr int RPI = 1024 / ROW_B;         // rows moved by one DMA instruction
  constexpr int NDMA = TILE_B / 1024 / 8;   // DMA instructions per wavefront and tile operand

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t lds0 =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  // shader-clock and constant-rate (100 MHz) counters at the workgroup's start
  const uint64_t clk0 = CLOCKED ? (uint64_t)__builtin_readcyclecounter() : 0;
  const uint64_t wall0 = CLOCKED ? (uint64_t)__builtin_amdgcn_s_memrealtime() : 0;
  // CLOCKED: thread 0 also leaves the time (100 MHz ticks since the start) at which it passed each
  // stage, at [kClockSlots * workgroup + 2 + stage]
  const uint64_t wg_id = blockIdx.x + (uint64_t)gridDim.x * (blockIdx.y + (uint64_t)gridDim.y * blockIdx.z);
  auto stamp = [&](int stage) __attribute__((always_inline)) {
    if (CLOCKED && tid == 0)
      p.clock_out[kClockSlots * wg_id + 2 + stage] = (uint64_t)__builtin_amdgcn_s_memrealtime() - wall0;
  };
  const int qb = wave % QW;   // query block of this wavefront
  const int hb = wave / QW;   // key block of every tile it handles when KSPLIT == 2 (else 0)

  // ---- frame index and slot flags: they need nothing but the kernel arguments ----
  const int64_t frame_t = p.t_pos[0];
  uint8_t flag = lane < p.n_slots ? p.written[(int64_t)lane * p.T] : (uint8_t)0;

  // ---- which (batch, head, query tile, split) this workgroup owns ----
  // The grid is (8 * query tiles, query heads per kv head, rounds): workgroups are dispatched
  // to XCDs round-robin in linear order, so XCD = blockIdx.x % 8, and the workgroups that share
  // one K/V stream (the x * y of one round) all land on the same XCD and its L2.
  const int xcd = blockIdx.x & 7, qtile = blockIdx.x >> 3, hq_in = blockIdx.y;
  const int us_raw = blockIdx.z * 8 + xcd;
  // a workgroup past the end computes the addresses of the last one and leaves further down, so
  // that the requests above and below do not wait behind a branch
  const int us = us_raw < p.unit_splits ? us_raw : p.unit_splits - 1;
  // leading units run unsplit; the rest are cut into n_splits context parts each
  int unit, split, nsp;
  if (us < p.units_whole) {
    unit = us; split = 0; nsp = 1;
  } else {
    const int r = us - p.units_whole;
    unit = p.units_whole + r / p.n_splits; split = r % p.n_splits; nsp = p.n_splits;
  }
  const int b = unit / p.Hkv, hkv = unit - b * p.Hkv;
  const int h = hkv * p.group + hq_in;

  // ---- raw Q fragments ----
  // A lane's fragment loads touch 32 rows x 32 bytes each: 512 small requests per wavefront, which
  // the 256-query shape (long loops) does not notice and the 128-query shape does: the tile DMAs
  // below cannot go out before Q is back.  There the workgroup's 128 x Dh tile comes by DMA - 16
  // lanes per row, whole cache lines - into the V ring's slots 2 and 3, laid out and swizzled like
  // two K tiles, while the slot flags are on their way; the fragments are read from there once the
  // first K tile is in (the V stream's first request for those slots goes out after the next barrier).
  constexpr int Q_OFF = L::V_OFF + 2 * TILE_B;
  const bool q_dma = KSPLIT == 2 && p.q_dma != 0;
  frag_t qf[KS];
  const int qrow = qtile * BM + qb * 32 + l32;
  if (!q_dma) {
    const uint16_t* qbase = reinterpret_cast<const uint16_t*>(p.q) + b * p.qs_b + h * p.qs_h;
    const int qr = qrow < p.T ? qrow : p.T - 1;
    const uint16_t* src = qbase + (int64_t)qr * p.qs_t + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const frag_t*>(src + ks * 16);
  }
  if (us_raw >= p.unit_splits) return;
  if (KSPLIT == 2 && q_dma) {
    const uint64_t qplane = uniform64((uint64_t)(uintptr_t)p.q + (uint64_t)(((int64_t)b * p.qs_b + (int64_t)h * p.qs_h) * 2));
    const uint32_t q_lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + Q_OFF + wave * 1024));
#pragma unroll
    for (int i = 0; i < 2 * NDMA; ++i) {
      const int row = (wave + i * 8) * RPI + lane / CPR;   // row of the 128-query tile
      int qr = qtile * BM + row;
      qr = qr < p.T ? qr : p.T - 1;
      dma16(qplane, (uint32_t)qr * (uint32_t)(p.qs_t * 2) + (uint32_t)(((lane % CPR) ^ k_swz<DH>(row)) << 4), q_lds + i * 8 * 1024);
    }
  }

  // ---- list of visible slots (the tail is pseudo-slot n_slots) ----
  // Every wavefront builds it for itself (no barrier, no serial section) in a private strip of
  // LDS: lane i of round k looks at slot 64*k + i.
  int* vis = reinterpret_cast<int*>(smem + L::MISC_OFF) + wave * (WE_MAX_SLOTS + 64);
  int nvis = 0;
  {
    const SlotInfo si = ring_slot(frame_t, p.dilation, p.num_buckets);
    for (int base = 0; base < p.n_slots; base += 64) {
      const int sl = base + lane;
      const bool f = flag != 0 && !(si.write_step && sl == si.slot);
      if (base + 64 < p.n_slots) flag = sl + 64 < p.n_slots ? p.written[(int64_t)(sl + 64) * p.T] : (uint8_t)0;
      const unsigned long long m = __ballot(f);
      if (f) vis[nvis + __popcll(m & ((1ull << lane) - 1ull))] = sl;
      nvis += __popcll(m);
    }
    if (lane == 0) vis[nvis] = p.n_slots;
    ++nvis;
  }
  stamp(0);  // slot list built
  // tiles per slot; the last one of a slot holds t_last of its 64 keys when T % 64 != 0
  const int tps = (p.T + BN - 1) / BN;
  const int t_last = p.T - (tps - 1) * BN;
  constexpr bool ragged = RAGGED;
  const int nt = nvis * tps;
  int t_begin = 0, t_end = nt;
  if (nsp > 1) {  // nt <= 257 * T / 64 and nsp <= 64: the products fit 32 bits
    t_begin = (int)((unsigned)split * (unsigned)nt / (unsigned)nsp);
    t_end = (int)((unsigned)(split + 1) * (unsigned)nt / (unsigned)nsp);
  }
  const int ntile = t_end - t_begin;

  const int64_t cap = p.L + p.T;
  const uint64_t kbase = (uint64_t)(uintptr_t)p.kv + (uint64_t)(((int64_t)b * p.Hkv + hkv) * cap) * ROW_B;
  const uint64_t vbase = kbase + (uint64_t)((int64_t)p.B * p.Hkv * cap) * ROW_B;

  // ---- DMA plumbing ----
  // Instruction i of this wavefront moves rows [q*RPI, (q+1)*RPI) of a tile, q = wave + 8*i.
  uint32_t kvoff[NDMA], vvoff[NDMA];
#pragma unroll
  for (int i = 0; i < NDMA; ++i) {
    const int row = (wave + i * 8) * RPI + lane / CPR;
    const int phys = lane % CPR;
    kvoff[i] = row * ROW_B + ((phys ^ k_swz<DH>(row)) << 4);
    vvoff[i] = row * ROW_B + ((phys ^ v_swz<DH>(row)) << 4);
  }
  // The split's visible tiles, 64 at a time: lane i of toff holds the byte offset, inside the
  // (batch, kv head) plane, of tile 64*k + i of the split (fits 32 bits, checked on the host).
  // Bit 0 (row starts are multiples of 128 bytes) marks the short last tile of a slot.  The tile
  // loop then needs one v_readlane per tile instead of walking slots and tiles with scalar code.
  // The workgroups that share this K/V stream (query tiles x grouped query heads) take the tiles
  // in groups of rot_g = 2 or 4, member m starting at tile m of every group: they then ask for
  // different lines at any one time, each line comes from HBM at one member's request and is an
  // L2 hit for the others a tile later.  (Asking together, every member waits the whole way to
  // HBM for every tile; a model's layers each bring their own ring, so K/V is never cache-warm:
  // 24 rings of 4096 tokens, 256-token frames: 757 -> 719 us per frame-step.)  The order of the
  // keys does not matter to a softmax.
  int rot_g = 1;
  while (rot_g * 2 <= p.members && rot_g < 4) rot_g *= 2;
  const unsigned rot_m = (unsigned)(qtile * p.group + hq_in) & (unsigned)(rot_g - 1);
  const unsigned rot_end = (unsigned)ntile & ~(unsigned)(rot_g - 1);
  uint32_t toff = 0;
  auto load_offsets = [&](int first) __attribute__((always_inline)) {
    unsigned kk = (unsigned)(first + lane);
    if (!RAGGED && kk < rot_end) kk = (kk & ~(unsigned)(rot_g - 1)) | ((kk + rot_m) & (unsigned)(rot_g - 1));
    unsigned ti = (unsigned)t_begin + kk;
    if (ti > (unsigned)(t_end - 1)) ti = (unsigned)(t_end - 1);
    const unsigned sidx = ti / (unsigned)tps;
    const unsigned sub = ti - sidx * (unsigned)tps;
    const uint32_t o = ((uint32_t)vis[sidx] * (uint32_t)p.T + sub * BN) * (uint32_t)ROW_B;
    toff = (ragged && sub == (unsigned)(tps - 1)) ? (o | 1u) : o;
  };
  int kc = 0;  // tile the K stream requests next; it stays on the last one
  auto next_off = [&]() __attribute__((always_inline)) {
    if ((kc & 63) == 0) load_offsets(kc);
    const uint32_t o = (uint32_t)__builtin_amdgcn_readlane((int)toff, kc & 63);
    if (kc < ntile - 1) ++kc;
    return o;
  };
  const uint64_t kplane = uniform64(kbase), vplane = uniform64(vbase);
  const uint32_t wave_lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + wave * 1024));
  // A short tile must not read rows of the next slot (or past the end of the buffer): its rows
  // beyond t_last repeat row t_last - 1; their keys are masked out of the softmax further down.
  auto clamp_rows = [&](uint32_t voff, int i) __attribute__((always_inline)) {
    const int row = (wave + i * 8) * RPI + lane / CPR;
    return row < t_last ? voff : voff - (uint32_t)(row - (t_last - 1)) * ROW_B;
  };
  // the tile offset is uniform: it goes into the scalar base address, not into every lane's offset
  auto dma_k = [&](uint32_t off, int slot) __attribute__((always_inline)) {
    const bool cut = RAGGED && (off & 1u) != 0u;
    const uint64_t base = kplane + (off & ~1u);
#pragma unroll
    for (int i = 0; i < NDMA; ++i)
      dma16(base, cut ? clamp_rows(kvoff[i], i) : kvoff[i], wave_lds + slot * TILE_B + i * 8 * 1024);
  };
  auto dma_v = [&](uint32_t off, int slot) __attribute__((always_inline)) {
    const bool cut = RAGGED && (off & 1u) != 0u;
    const uint64_t base = vplane + (off & ~1u);
#pragma unroll
    for (int i = 0; i < NDMA; ++i)
      dma16(base, cut ? clamp_rows(vvoff[i], i) : vvoff[i], wave_lds + L::V_OFF + slot * TILE_B + i * 8 * 1024);
  };
  // keys of 32-key block blk of the tile at position sub of its slot that exist (0 .. 32)
  auto block_keys = [&](int sub, int blk) __attribute__((always_inline)) {
    if (!RAGGED) return 32;
    const int n = ((ragged && sub == tps - 1) ? t_last : BN) - 32 * blk;
    return n < 0 ? 0 : (n > 32 ? 32 : n);
  };
  // logits of keys that do not exist become -inf (register i of a lane is key row
  // (i / 4) * 8 + 4 * hh + i % 4 of the block)
  auto mask_keys = [&](f32x16_t& sv, int nkeys) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if ((i / 4) * 8 + 4 * hh + (i % 4) >= nkeys) sv[i] = -INFINITY;
  };

  // ---- fragment read addresses (byte offsets into smem) ----
  // K row l32 of a key block, logical chunk 2*ks + hh: physical chunk bits [3:1] are
  // ks ^ (swz >> 1), so the address for step ks is the step-0 address with bits 5.. flipped.
  uint32_t k_rd;
  {
    const int x = k_swz<DH>(l32);
    k_rd = hb * KB_B + l32 * ROW_B + ((((x >> 1) << 1) | (hh ^ (x & 1))) << 4);
  }
  // V rows 4*hh + r (r = lane bits 3:2) of each 8-row group, logical chunk 4*db + c.
  uint32_t v_rd;
  {
    const int r = 4 * hh + ((lane & 15) >> 2);
    const int y = v_swz<DH>(r) >> 2;
    const int c = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    v_rd = L::V_OFF + hb * KB_B + r * ROW_B + ((y * 4 + c) << 4) + (lane & 1) * 8;
  }

  f32x16_t o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m_ref = -INFINITY, l_run = 0.f;

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // Softmax scale and reference: the logits are the exact products' sums of the element-type q
  // and k (nothing is rounded before the matrix core); the scale c = softmax scale * log2(e) and
  // the running reference m_ref of this lane's query (every lane owns one query column of the
  // transposed scores) are applied by one fused multiply-add per logit in front of its
  // exponential: p = 2^(s * c + msc), msc = -m_ref * c.
  const float lmul = p.scale_log2;
  float msc = 0.f;
  auto set_shift = [&]() __attribute__((always_inline)) { msc = -m_ref * lmul; };

  // probabilities of one 32-key block from its logits: p = 2^((s - sub) * lmul), packed to the
  // element type; returns this half-wave's share of the row sum (of the rounded values)
  auto probabilities = [&](frag_t(&pf)[2], const f32x16_t& s, float sub) __attribute__((always_inline)) {
    float rs = 0.f;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f((s[8 * m + j] - sub) * lmul);
      pf[m] = M::pack8(e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]);
#pragma unroll
      for (int j = 0; j < 4; ++j) rs = M::add_pair(rs, pf[m], j);
    }
    return rs;
  };
  auto block_max = [&](const f32x16_t& s) __attribute__((always_inline)) {
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    float lo, up;
    half_wave_pair(mx, lo, up);
    return fmaxf(lo, up);
  };

  // The pipeline runs on 32-key blocks.  One step computes, for this wavefront,
  //   matrix cores: the logits of the block read at K offset KOFF (-> s_next) and the
  //                 product of the previous block's probabilities with the V block at VOFF;
  //   VALU:         the probabilities of the current block (s_cur -> p_cur).
  // LDS reads are issued in consumption order - K fragments 0..KS-1, then the NV V^T fragments
  // (two transposing reads each) - running up to 15 reads ahead of the MFMAs.
  frag_t p_prev[2];
  f32x16_t s_cur;
  // RAGGED only: this wavefront has not seen a key yet (its first block was an empty block of a
  // short tile), so its reference exponent is a placeholder; cur_keys = keys of the block whose
  // probabilities the next step computes.
  bool ref_unset = false;
  int cur_keys = 32;
  // Fragment registers live across steps: every step starts with its first PRE reads (all K
  // fragments and the first V^T fragment) already in flight, issued during the previous step.
  constexpr int PRE = KS + 2;
  u32x4_t kf[KS];
  u32x2_t v0[NV], v1[NV];
  auto read_k = [&](auto koff_c, int ks) __attribute__((always_inline)) {
    kf[ks] = lds_read128<decltype(koff_c)::value>(smem, k_rd ^ (ks << 5));
  };
  auto read_v = [&](auto voff_c, int i) __attribute__((always_inline)) {  // fragment i = (m, db) = (i / DB, i % DB)
    constexpr int VOFF = decltype(voff_c)::value;
    const uint32_t a = v_rd ^ ((i % DB) << 6);
    if (i / DB == 0) {
      v0[i] = lds_read_tr<VOFF>(smem, a);
      v1[i] = lds_read_tr<VOFF + 8 * ROW_B>(smem, a);
    } else {
      v0[i] = lds_read_tr<VOFF + 16 * ROW_B>(smem, a);
      v1[i] = lds_read_tr<VOFF + 24 * ROW_B>(smem, a);
    }
  };
  auto prefetch = [&](auto koff_c, auto voff_c) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) read_k(koff_c, ks);
    read_v(voff_c, 0);
  };
  // nkeys: keys that exist in the block whose logits this step computes (32 = all, 0 = the block
  // lies past the end of the split)
  // (the K fragments at koff_c were requested by the previous step; the offset documents the call)
  // first_c (128-query shape only): the workgroup's very first step has no previous block, so it
  // skips the product and its V reads instead of multiplying a zeroed tile by zeros.
  auto step = [&](auto /*koff_c*/, auto voff_c, auto nkoff_c, auto nvoff_c, int nkeys, auto&& mid, auto first_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_c)::value;
    // (logits of a block past the end of the split are never consumed; a short tile's empty block
    // is masked after its products)
    // next own V fragment to request / next-step read pairs requested so far
    int vnext = 1, npair = 0;
    constexpr int NPAIR = PRE / 2;            // the next step's first reads go out two at a time
    constexpr int I0 = NV - 1 - NPAIR;        // ... after the product MFMAs I0, I0+1, ...
    auto next_pair = [&]() __attribute__((always_inline)) {
      if (2 * npair < KS) {
        read_k(nkoff_c, 2 * npair);
        read_k(nkoff_c, 2 * npair + 1);
      } else {
        read_v(nvoff_c, 0);
      }
      ++npair;
    };

    // From here to the end of the product the issue order is pinned statement by statement
    // (sched_barrier): MFMA, the reads that refill the queue, a slice of the VALU work.
    __builtin_amdgcn_sched_barrier(0);
    frag_t p_cur[2];
    float e[16];
    float rs = 0.f;
    // VALU slices: the 16 exponentials of the current block are spread evenly over the MFMAs of
    // the step.  The two wavefronts of a SIMD run in phase, so bunching them under the logits
    // would saturate the quarter-rate unit there and leave it idle under the product.
    constexpr int EPS = 16 / (KS + NV);
    static_assert(EPS * (KS + NV) == 16, "exponentials per slot");
    auto exp_slot = [&](int g) __attribute__((always_inline)) {
#pragma unroll
      for (int t = 0; t < EPS; ++t)
        if (g * EPS + t < 16) {
          e[g * EPS + t] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[g * EPS + t], lmul, msc));
          // an exponential has no side effect, so nothing else keeps it in its slot: left alone the
          // compiler sinks the first nine of a step below the tile DMAs
          asm volatile("" : "+v"(e[g * EPS + t]));
        }
    };
    f32x16_t s_next;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      s_next = M::mma(__builtin_bit_cast(frag_t, kf[ks]), qf[ks], ks == 0 ? zero16 : s_next);
      // keep the read queue full without exceeding the 15 reads the counter can track
      if (!FIRST && vnext < NV && ks <= 12 - KS) {
        read_v(voff_c, vnext);
        ++vnext;
        }
      exp_slot(ks);
      __builtin_amdgcn_sched_barrier(0);
    }
    mid();  // the tile DMAs of this iteration go out here, under the MFMAs already queued
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (!FIRST) {
        if (vnext < NV) {  // reads 0..KS+2i-1 have completed: room for one more fragment
          read_v(voff_c, vnext);
          ++vnext;
        }
        typedef unsigned int u32x4v __attribute__((ext_vector_type(4)));
        const u32x4v a4 = __builtin_shufflevector(v0[i], v1[i], 0, 1, 2, 3);
        o[i % DB] = M::mma(__builtin_bit_cast(frag_t, a4), p_prev[i / DB], o[i % DB]);
      }
      if (i >= I0 && npair < NPAIR) next_pair();
      // VALU slices: the last exponentials; packing of the two 16-key halves and their row sums
      exp_slot(KS + i);
      if (i == 1) p_cur[0] = M::pack8(e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]);
      if (i == 2) {
#pragma unroll
        for (int t = 0; t < 4; ++t) rs = M::add_pair(rs, p_cur[0], t);
      }
      if (i == NV - 1) p_cur[1] = M::pack8(e[8], e[9], e[10], e[11], e[12], e[13], e[14], e[15]);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) rs = M::add_pair(rs, p_cur[1], t);

    // first block with keys of a wavefront that started on an empty block: nothing is accumulated
    // yet, so the placeholder reference is replaced by this block's own maximum, up or down
    // (a placeholder far above every real logit would make all of them underflow to zero)
    const bool seed = RAGGED && ref_unset && cur_keys > 0;
    if (seed || __ballot(!(rs <= 256.f)) != 0ull) {
      // Rare: some probability of this block may exceed 2^8.  Raise the reference of the rows
      // that need it, redo the block's probabilities exactly and rescale the accumulators: they
      // hold the blocks before this one (the last of those products was issued above).
      const float mx = block_max(s_cur);
      const float m_new = (seed ? mx > -INFINITY : mx > m_ref) ? mx : m_ref;
      const float alpha = seed ? 1.f : __builtin_amdgcn_exp2f((m_ref - m_new) * lmul);  // seed: sums and accumulators are still zero
      if (RAGGED) ref_unset = false;
      rs = probabilities(p_cur, s_cur, m_new);
      l_run *= alpha;
      m_ref = m_new;
      set_shift();
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    }
    l_run += rs;
    p_prev[0] = p_cur[0];
    p_prev[1] = p_cur[1];
    if (RAGGED && nkeys < 32) mask_keys(s_next, nkeys);  // short last tile of a slot (or an empty block of it)
    if (RAGGED) cur_keys = nkeys;
    s_cur = s_next;
  };

  if (ntile > 0) {
    // 256-query shape: zero V slot 3, which stands in for "tile -1", and P, so that the first
    // product adds zeros (the 128-query shape skips the product of its first step instead)
    if (KSPLIT == 1) {
      const u32x4_t z = {0u, 0u, 0u, 0u};
      unsigned char* vz = smem + L::V_OFF + 3 * TILE_B;
      for (int i = tid; i < TILE_B / 16; i += 512) *reinterpret_cast<u32x4_t*>(vz + i * 16) = z;
    }
    {
      const u32x4_t z = {0u, 0u, 0u, 0u};
      p_prev[0] = __builtin_bit_cast(frag_t, z);
      p_prev[1] = __builtin_bit_cast(frag_t, z);
    }
    // Iteration j issues K(j+KA) and V(j+2) (KA = 3, or 4 when every wavefront handles one key
    // block per tile and prefetches its next fragments across the barrier); the prologue issues
    // what the iterations before 0 would have.
    constexpr int KA = KSPLIT == 1 ? 3 : 4;
    // The V stream trails the K stream by KA - 2 tiles, so it reuses the K stream's offsets.
    int csub = t_begin - (t_begin / tps) * tps;  // position in its slot of the tile whose logits are computed next
    uint32_t off1, off2;  // offsets of the last and the last-but-one tile the K stream visited
    // Q was requested before the slot flags and loads return in order, so it is here; stating a
    // use now keeps the wait for it from landing behind the tile DMAs issued next.
    if (!q_dma) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(qf[ks]));
    }
    {
      const uint32_t o0 = next_off();
      const uint32_t o1 = next_off();
      const uint32_t o2 = next_off();
      dma_k(o0, 0);
      dma_k(o1, 1);
      if (KSPLIT == 2) dma_k(o2, 2);
      dma_v(o0, 0);
      if (KSPLIT == 1) {
        dma_k(o2, 2);
        off1 = o2; off2 = o1;
      } else {
        const uint32_t o3 = next_off();
        dma_k(o3, 3);
        off1 = o3; off2 = o2;
      }
      dma_v(o1, 1);
    }
    dma_wait<(KA + 1) * NDMA>();
    __syncthreads();  // K(0) and the zeroed V slot (128-query shape: the Q tile, requested long before K(0)) are in LDS
    stamp(1);  // first K tile landed
    if (KSPLIT == 2 && q_dma) {
      // row qb*32 + l32 of the tile, logical chunk 2*ks + hh: the K fragment's address arithmetic
      const int x = k_swz<DH>(l32);
      const uint32_t q_rd = (uint32_t)(Q_OFF + qb * KB_B + l32 * ROW_B + ((((x >> 1) << 1) | (hh ^ (x & 1))) << 4));
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const frag_t*>(smem + (q_rd ^ (ks << 5)));
    }
    // (Q stays in registers for the rest of the kernel)
    // first block: reference = its row max
    {
      s_cur = zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const frag_t a = *reinterpret_cast<const frag_t*>(smem + (k_rd ^ (ks << 5)));
        s_cur = M::mma(a, qf[ks], s_cur);
      }
      const int nk0 = block_keys(csub, hb);
      if (RAGGED && nk0 < 32) mask_keys(s_cur, nk0);
      const float mx0 = block_max(s_cur);
      m_ref = mx0 > -INFINITY ? mx0 : 0.f;  // (a block of the first tile may be empty)
      if (RAGGED) {
        ref_unset = nk0 == 0;
        cur_keys = nk0;
      }
      set_shift();
    }
    // (every wavefront has read its Q fragments before it passes the barrier below: the staging area
    // becomes V slots again)
    dma_wait<2 * NDMA>();
    __syncthreads();  // everything but the last K and V tile issued so far has landed
    // first reads of the first step
    if (KSPLIT == 1) {
      prefetch(IntC<KB_B>(), IntC<3 * TILE_B + KB_B>());
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) read_k(IntC<TILE_B>(), ks);
    }

    // one tile iteration with compile-time ring positions (JM = j mod 4)
    auto iteration = [&](int j, auto jm_c, auto first_c) __attribute__((always_inline)) {
      constexpr int JM = decltype(jm_c)::value;
      auto issue_dma = [&]() __attribute__((always_inline)) {
        const uint32_t o = next_off();
        dma_k(o, (JM + KA) % NST);                       // K(j+KA)
        dma_v(KA == 3 ? off1 : off2, (JM + 2) % NST);    // V(j+2)
        off2 = off1;
        off1 = o;
      };
      auto nothing = [&]() __attribute__((always_inline)) {};
      // csub is tile j's position in its slot; nsub tile j+1's
      const int nsub = csub + 1 == tps ? 0 : csub + 1;
      if (KSPLIT == 1) {
        // block (j, 0) -> probabilities; logits of (j, 1); product of (j-1, 1)
        step(IntC<JM * TILE_B + KB_B>(), IntC<((JM + 3) % NST) * TILE_B + KB_B>(),
             IntC<((JM + 1) % NST) * TILE_B>(), IntC<JM * TILE_B>(), block_keys(csub, 1), issue_dma, std::false_type());
        // block (j, 1) -> probabilities; logits of (j+1, 0); product of (j, 0)
        step(IntC<((JM + 1) % NST) * TILE_B>(), IntC<JM * TILE_B>(),
             IntC<((JM + 1) % NST) * TILE_B + KB_B>(), IntC<JM * TILE_B + KB_B>(),
             j + 1 < ntile ? block_keys(nsub, 0) : 0, nothing, std::false_type());
      } else {
        // block (j, hb) -> probabilities; logits of (j+1, hb); product of (j-1, hb)
        step(IntC<((JM + 1) % NST) * TILE_B>(), IntC<((JM + 3) % NST) * TILE_B>(),
             IntC<((JM + 2) % NST) * TILE_B>(), IntC<JM * TILE_B>(),
             j + 1 < ntile ? block_keys(nsub, __builtin_amdgcn_readfirstlane(hb)) : 0, issue_dma, first_c);
      }
      csub = nsub;
      dma_wait<2 * NDMA>();  // all but this iteration's two tiles have landed (this wavefront's part)
      // A bare barrier: __syncthreads() would also wait for every LDS read in flight, i.e. for the
      // next step's fragments requested a moment ago.  Nothing needs that: the tiles arrive by DMA,
      // whose completion the counter wait above tracks, fragment reads are awaited where they are
      // used, and the reads still in flight here target ring slots that no DMA overwrites before
      // the barrier after next.  The empty asm keeps the compiler from moving memory accesses across.
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    };

    int j = 0;
    const std::false_type not_first;
    if (KSPLIT == 2) {
      // the first tile's step has no product to do: peeled, with the three iterations that bring
      // the ring position back to zero
      iteration(0, IntC<0>(), std::true_type());
      j = 1;
      if (j < ntile) { iteration(j, IntC<1>(), not_first); ++j; }
      if (j < ntile) { iteration(j, IntC<2>(), not_first); ++j; }
      if (j < ntile) { iteration(j, IntC<3>(), not_first); ++j; }
    }
    for (; j + 4 <= ntile; j += 4) {
      iteration(j, IntC<0>(), not_first);
      iteration(j + 1, IntC<1>(), not_first);
      iteration(j + 2, IntC<2>(), not_first);
      iteration(j + 3, IntC<3>(), not_first);
    }
    if (j < ntile) { iteration(j, IntC<0>(), not_first); ++j; }
    if (j < ntile) { iteration(j, IntC<1>(), not_first); ++j; }
    if (j < ntile) { iteration(j, IntC<2>(), not_first); ++j; }

    stamp(2);  // tile loop left
    // product of the last block: (ntile-1, 1) for full-tile wavefronts, (ntile-1, hb) otherwise
    {
      const int last = (ntile - 1) % NST;
      const unsigned char* vt = smem + v_rd + last * TILE_B + (KSPLIT == 1 ? KB_B : 0);
#pragma unroll
      for (int m = 0; m < 2; ++m) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const unsigned char* va = smem + ((uint32_t)(vt - smem) ^ (db << 6)) + 16 * m * ROW_B;
          const s16x4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va));
          const s16x4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va + 8 * ROW_B));
          typedef short s16x8_t __attribute__((ext_vector_type(8)));
          const s16x8_t a8 = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
          o[db] = M::mma(__builtin_bit_cast(frag_t, a8), p_prev[m], o[db]);
        }
      }
    }
    dma_wait<0>();  // no DMA may still be writing LDS when the rings are reused or the CU is freed
  } else if (q_dma) {
    dma_wait<0>();  // (a split without visible keys: the Q tile it asked for must not land after the merge below)
  }

  float lo, up;
  half_wave_pair(l_run, lo, up);
  float l_tot = lo + up;
  m_ref *= lmul;  // from raw logits to the log2 domain the merges work in

  if (KSPLIT == 2) {
    // ---- the two wavefronts of a query block merge their (m, l, O) through LDS ----
    // 16-byte accesses: vector k of lane l sits at ((qb * (DB * 4 + 1) + k) * 64 + l) * 16.
    __syncthreads();  // every wavefront is done with the rings
    f32x4_t* mb = reinterpret_cast<f32x4_t*>(smem) + (qb * (DB * 4 + 1)) * 64 + lane;
    if (hb == 1) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          mb[(db * 4 + c) * 64] = f32x4_t{o[db][4 * c], o[db][4 * c + 1], o[db][4 * c + 2], o[db][4 * c + 3]};
      mb[(DB * 4) * 64] = f32x4_t{m_ref, l_tot, 0.f, 0.f};
    }
    __syncthreads();
    if (hb == 1) return;
    const f32x4_t ml1 = mb[(DB * 4) * 64];
    // a wavefront whose sum is zero saw no key (or only keys that vanish against its reference):
    // its reference must not take part in the maximum
    const float m1 = ml1[1] > 0.f ? ml1[0] : -INFINITY, l1 = ml1[1];
    if (!(l_tot > 0.f)) m_ref = -INFINITY;
    const float mm = fmaxf(m_ref, m1);
    if (mm > -INFINITY) {
      const float a0 = __builtin_amdgcn_exp2f(m_ref - mm), a1 = __builtin_amdgcn_exp2f(m1 - mm);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const f32x4_t other = mb[(db * 4 + c) * 64];
#pragma unroll
          for (int e = 0; e < 4; ++e) o[db][4 * c + e] = a0 * o[db][4 * c + e] + a1 * other[e];
        }
      l_tot = a0 * l_tot + a1 * l1;
      m_ref = mm;
    }
  }

  stamp(3);  // pair merged
  // ---- epilogue ----
  const int64_t rows = (int64_t)p.B * p.H * p.T - p.ws_row0;  // rows in the workspace
  const bool valid = qrow < p.T;
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const int64_t row = ((int64_t)b * p.H + h) * p.T + qrow;
  float gate_v = 1.f;
  const bool gated = p.gate != nullptr || p.gate_w != nullptr;
  if (gated && nsp == 1 && qrow < p.T) gate_v = head_gate<typename M::elem_t>(p, b, h, qrow);
  // A split leaves its partial output as fp16 values in [-1, 1] plus one fp32 scale per row (the
  // row's largest normalised magnitude): 11 significant bits whatever the element type, for the
  // bytes of a bf16 row, and no overflow for any finite V.  A row that holds an infinity keeps the
  // plain normalised values (scale 1), so that only the columns concerned turn non-finite, as in a
  // single pass; a row whose largest magnitude is too small for its reciprocal is scaled by 2^100.
  float mul = inv;
  if (nsp > 1) {
    float amax = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(o[db][i]));
    float alo, aup;
    half_wave_pair(amax, alo, aup);
    amax = fmaxf(alo, aup);
    float row_scale;
    if (amax < INFINITY) {
      const float a = fmaxf(amax, 0x1p-100f);
      mul = 1.f / a;
      row_scale = a * inv;
    } else {
      mul = inv;
      row_scale = 1.f;
    }
    if (valid && hh == 0)
      *reinterpret_cast<f32x4_t*>(p.ws_ml + ((int64_t)split * rows + (row - p.ws_row0)) * 4) =
          f32x4_t{l_tot > 0.f ? m_ref : -INFINITY, l_tot, row_scale, 0.f};
  }
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int c = 0; c < 4; c += 2) {
      // register quad c holds head-dim rows 8c + 4*half + 0..3; after the swap a lane of the
      // lower half owns rows 8c..8c+7 and a lane of the upper half rows 8(c+1)..8(c+1)+7.
      float f[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(o[db][4 * c + e] * mul),
                                                  __float_as_uint(o[db][4 * c + 4 + e] * mul), false, false);
        f[e] = __uint_as_float(r[0]);
        f[4 + e] = __uint_as_float(r[1]);
      }
      const int d0 = 32 * db + 8 * (c + hh);
      if (valid) {
        if (nsp == 1) {
          uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h +
                          (int64_t)qrow * p.os_t + d0;
          frag_t y = M::pack8(f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]);
          if (gated) {  // y * gate on element-type values, as the module's own multiply
            y = M::pack8((float)y[0] * gate_v, (float)y[1] * gate_v, (float)y[2] * gate_v, (float)y[3] * gate_v,
                         (float)y[4] * gate_v, (float)y[5] * gate_v, (float)y[6] * gate_v, (float)y[7] * gate_v);
          }
          *reinterpret_cast<frag_t*>(dst) = y;
        } else {
          uint16_t* dst = p.ws_o + ((int64_t)split * rows + (row - p.ws_row0)) * DH + d0;
          *reinterpret_cast<f16x8_t*>(dst) = F16Mma::pack8(f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]);
        }
      }
    }
  }
  stamp(4);  // results / partial results stored (requests issued)
  if (CLOCKED && tid == 0) {
    p.clock_out[kClockSlots * wg_id] = (uint64_t)__builtin_readcyclecounter() - clk0;
    p.clock_out[kClockSlots * wg_id + 1] = (uint64_t)__builtin_amdgcn_s_memrealtime() - wall0;
  }
}

// WE_WITH_PROBES (the measurement library's build) adds the CLOCKED instantiations; the product's
// objects hold none of their code.
#ifdef WE_WITH_PROBES
constexpr bool kWithProbes = true;
#else
constexpr bool kWithProbes = false;
#endif

template <typename M, int DH, int KSPLIT, bool RAGGED, bool CLOCKED>
static hipError_t launch_ring_c(const AttnParams& p, hipStream_t stream) {
  const int rounds = (p.unit_splits + 7) / 8;
  const dim3 grid((unsigned)(8 * p.q_tiles), (unsigned)p.group, (unsigned)rounds);
  hipLaunchKernelGGL((attn_ring_kernel<M, DH, KSPLIT, RAGGED, CLOCKED>), grid, dim3(512), RingLds<DH>::kBytes, stream, p);
  return hipGetLastError();
}
template <typename M, int DH, int KSPLIT, bool RAGGED>
static hipError_t launch_ring_r(const AttnParams& p, hipStream_t stream) {
  if constexpr (kWithProbes) {
    if (p.clock_out != nullptr) return launch_ring_c<M, DH, KSPLIT, RAGGED, true>(p, stream);
  }
  return launch_ring_c<M, DH, KSPLIT, RAGGED, false>(p, stream);
}
template <typename M, int DH, int KSPLIT>
static hipError_t launch_ring_t(const AttnParams& p, hipStream_t stream) {
  return p.T % BN == 0 ? launch_ring_r<M, DH, KSPLIT, false>(p, stream) : launch_ring_r<M, DH, KSPLIT, true>(p, stream);
}

// The kernels use more LDS than a launch may ask for by default; the limit is a per-device
// setting of each kernel, raised once per device by the library's set-up (device_state.hip).
template <typename M, int DH, int KSPLIT, bool RAGGED, bool CLOCKED>
static hipError_t configure_one() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_ring_kernel<M, DH, KSPLIT, RAGGED, CLOCKED>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, RingLds<DH>::kBytes);
}
template <typename M, int DH>
static hipError_t configure_family() {
  hipError_t e = configure_one<M, DH, 1, false, false>();
  if (e == hipSuccess) e = configure_one<M, DH, 1, true, false>();
  if (e == hipSuccess) e = configure_one<M, DH, 2, false, false>();
  if (e == hipSuccess) e = configure_one<M, DH, 2, true, false>();
  if constexpr (kWithProbes) {
    if (e == hipSuccess) e = configure_one<M, DH, 1, false, true>();
    if (e == hipSuccess) e = configure_one<M, DH, 1, true, true>();
    if (e == hipSuccess) e = configure_one<M, DH, 2, false, true>();
    if (e == hipSuccess) e = configure_one<M, DH, 2, true, true>();
  }
  return e;
}

// The four (element type, head dim) families are compiled as separate objects (WE_RING_PART selects
// one; undefined = all of them in this translation unit) so that they build in parallel.
#if !defined(WE_RING_PART) || WE_RING_PART == 0
hipError_t launch_attn_ring_bf16_128(const AttnParams& p, int ksplit, hipStream_t stream) {
  return ksplit == 2 ? launch_ring_t<Bf16Mma, 128, 2>(p, stream) : launch_ring_t<Bf16Mma, 128, 1>(p, stream);
}
hipError_t configure_attn_ring_bf16_128() { return configure_family<Bf16Mma, 128>(); }
#endif
#if !defined(WE_RING_PART) || WE_RING_PART == 1
hipError_t launch_attn_ring_bf16_64(const AttnParams& p, int ksplit, hipStream_t stream) {
  return ksplit == 2 ? launch_ring_t<Bf16Mma, 64, 2>(p, stream) : launch_ring_t<Bf16Mma, 64, 1>(p, stream);
}
hipError_t configure_attn_ring_bf16_64() { return configure_family<Bf16Mma, 64>(); }
#endif
#if !defined(WE_RING_PART) || WE_RING_PART == 2
hipError_t launch_attn_ring_f16_128(const AttnParams& p, int ksplit, hipStream_t stream) {
  return ksplit == 2 ? launch_ring_t<F16Mma, 128, 2>(p, stream) : launch_ring_t<F16Mma, 128, 1>(p, stream);
}
hipError_t configure_attn_ring_f16_128() { return configure_family<F16Mma, 128>(); }
#endif
#if !defined(WE_RING_PART) || WE_RING_PART == 3
hipError_t launch_attn_ring_f16_64(const AttnParams& p, int ksplit, hipStream_t stream) {
  return ksplit == 2 ? launch_ring_t<F16Mma, 64, 2>(p, stream) : launch_ring_t<F16Mma, 64, 1>(p, stream);
}
hipError_t configure_attn_ring_f16_64() { return configure_family<F16Mma, 64>(); }
#endif

}  // namespace we
