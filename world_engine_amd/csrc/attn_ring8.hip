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
// overlaps the other's matrix work), each wavefront owning 32 queries.  Two shapes:
//   GROUPS = 1: 256 queries; all 8 wavefronts share every K/V tile (large frames).
//   GROUPS = 2: 128 queries; the wavefronts form two groups that take alternate tiles of the
//               context and merge their (max, sum, O) through LDS at the end.  This doubles
//               the parallelism inside a CU without doubling split-context partials
//               (256-token frames, where the grid alone cannot fill the chip).
// K/V tiles travel HBM -> LDS directly (global_load_lds_dwordx4, no VGPR staging) into rings
// of 4/GROUPS slots per operand, issued up to three tiles ahead.  LDS tiles are unpadded; bank
// conflicts are avoided by XOR-swizzling 16-byte chunks, applied on the global side of the DMA
// (lane i always lands at LDS offset 16*i) and undone in the fragment addresses.
// Per 64-key tile and wavefront:
//   S^T = K Q^T        v_mfma_f32_32x32x16, A = K rows (ds_read_b128), B = Q in registers,
//                      pre-multiplied by scale*log2(e); one extra MFMA (ones x -m_ref) makes the
//                      logits leave the matrix core already shifted by the running reference.
//   P = 2^S            v_exp_f32 + v_cvt_pk + v_dot2c row sum; each lane owns one query column.
//   O^T += V^T P^T     A = V^T via ds_read_b64_tr_b16, B = P straight from registers.
// The three are software-pipelined across tiles (logits of tile i+1 and product of tile i-1 run
// on the matrix cores while the VALU handles tile i).
//
// Roofline: 4*T*N_vis*Dh flops and 4*N_vis*Dh bytes of K/V per (batch, kv head).
#include "attn_mma.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

namespace we {

template <int DH>
struct Ring8Lds {
  static constexpr int CPR = DH / 8;          // 16-byte chunks per row
  static constexpr int ROW_B = DH * 2;        // bytes per K/V row
  static constexpr int TILE_B = BN * ROW_B;   // bytes per K or V tile
  static constexpr int SLOTS = 4;             // ring slots per operand over all wave groups
  static constexpr int V_OFF = SLOTS * TILE_B;
  static constexpr int MISC_OFF = 2 * SLOTS * TILE_B;
  static constexpr int kBytes = MISC_OFF + (WE_MAX_SLOTS + 2) * 4;
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

// One 1-KB LDS-DMA: lane i copies 16 bytes from gbase + voff to LDS byte lds_addr + 16*i.
// Hidden from the compiler's counter bookkeeping on purpose; completion is awaited with
// dma_wait<N>() (vmcnt) followed by a workgroup barrier.
__device__ __forceinline__ void dma16(uint64_t gbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(gbase), "s"(lds_addr)
               : "memory");
}
template <int N>
__device__ __forceinline__ void dma_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ uint64_t uniform64(uint64_t x) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
  return ((uint64_t)hi << 32) | lo;
}

template <int V>
struct IntC {
  static constexpr int value = V;
};

template <typename M, int DH, int GROUPS>
__global__ void __launch_bounds__(512, 2) attn_ring8_kernel(AttnParams p) {
  typedef typename M::frag_t frag_t;
  typedef Ring8Lds<DH> L;
  constexpr int KS = DH / 16;               // contraction steps of K Q^T
  constexpr int DB = DH / 32;               // 32-row blocks of O^T
  constexpr int WPG = 8 / GROUPS;           // wavefronts per group
  constexpr int NST = 4 / GROUPS;           // ring slots per operand and group
  constexpr int BM = 32 * WPG;              // queries per workgroup
  constexpr int CPR = L::CPR, ROW_B = L::ROW_B, TILE_B = L::TILE_B;
  constexpr int RPI = 1024 / ROW_B;         // rows moved by one DMA instruction
  constexpr int NDMA = TILE_B / 1024 / WPG; // DMA instructions per wavefront and tile operand

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  int* vis = reinterpret_cast<int*>(smem + L::MISC_OFF);  // visible slots, then their count
  const uint32_t lds0 =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int grp = wave / WPG, wig = wave % WPG;

  // ---- which (batch, head, query tile, split) this workgroup owns; XCD = blockIdx % 8 ----
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int round = jj / p.members, member = jj - round * p.members;
  const int us = round * 8 + xcd;
  if (us >= p.unit_splits) return;
  const int unit = us / p.n_splits, split = us - unit * p.n_splits;
  const int b = unit / p.Hkv, hkv = unit - b * p.Hkv;
  const int hq_in = member / p.q_tiles, qtile = member - hq_in * p.q_tiles;
  const int h = hkv * (p.H / p.Hkv) + hq_in;

  // ---- list of visible slots (the tail is pseudo-slot n_slots) ----
  if (wave == 0) {
    const SlotInfo si = ring_slot(p.t_pos[0], p.dilation, p.num_buckets);
    int count = 0;
    for (int base = 0; base < p.n_slots; base += 64) {
      const int s = base + lane;
      bool f = false;
      if (s < p.n_slots) f = (p.written[(int64_t)s * p.T] != 0) && !(si.write_step && s == si.slot);
      const unsigned long long m = __ballot(f);
      if (f) vis[count + __popcll(m & ((1ull << lane) - 1ull))] = s;
      count += __popcll(m);
    }
    if (lane == 0) {
      vis[count] = p.n_slots;
      vis[WE_MAX_SLOTS + 1] = count + 1;
    }
  }
  __syncthreads();
  const int nvis = __builtin_amdgcn_readfirstlane(vis[WE_MAX_SLOTS + 1]);
  const int tps = p.T / BN;  // tiles per slot
  const int nt = nvis * tps;
  const int t_begin = (int)((int64_t)split * nt / p.n_splits);
  const int t_end = (int)((int64_t)(split + 1) * nt / p.n_splits);
  const int ntile = t_end - t_begin;
  // this group's tiles: t_begin + grp + j*GROUPS, j < n_g; every group runs n_iter iterations
  const int n_g = ntile > grp ? (ntile - grp + GROUPS - 1) / GROUPS : 0;
  const int n_iter = (ntile + GROUPS - 1) / GROUPS;

  // ---- Q fragments stay in registers, pre-multiplied by scale*log2(e) ----
  const float c2 = p.scale_log2;
  frag_t qf[KS];
  const int qrow = qtile * BM + wig * 32 + l32;
  {
    const uint16_t* qbase = reinterpret_cast<const uint16_t*>(p.q) + b * p.qs_b + h * p.qs_h;
    const int qr = qrow < p.T ? qrow : p.T - 1;
    const uint16_t* src = qbase + (int64_t)qr * p.qs_t + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const frag_t raw = *reinterpret_cast<const frag_t*>(src + ks * 16);
      qf[ks] = M::pack8((float)raw[0] * c2, (float)raw[1] * c2, (float)raw[2] * c2, (float)raw[3] * c2,
                        (float)raw[4] * c2, (float)raw[5] * c2, (float)raw[6] * c2, (float)raw[7] * c2);
    }
  }

  const int64_t cap = p.L + p.T;
  const uint64_t kbase = (uint64_t)(uintptr_t)p.kv + (uint64_t)(((int64_t)b * p.Hkv + hkv) * cap) * ROW_B;
  const uint64_t vbase = kbase + (uint64_t)((int64_t)p.B * p.Hkv * cap) * ROW_B;

  // ---- DMA plumbing ----
  // Instruction i of this wavefront moves rows [q*RPI, (q+1)*RPI) of a tile, q = wig + i*WPG.
  uint32_t kvoff[NDMA], vvoff[NDMA];
#pragma unroll
  for (int i = 0; i < NDMA; ++i) {
    const int row = (wig + i * WPG) * RPI + lane / CPR;
    const int phys = lane % CPR;
    kvoff[i] = row * ROW_B + ((phys ^ k_swz<DH>(row)) << 4);
    vvoff[i] = row * ROW_B + ((phys ^ v_swz<DH>(row)) << 4);
  }
  const uint32_t k_ring = lds0 + grp * NST * TILE_B;              // this group's K slots
  const uint32_t v_ring = lds0 + L::V_OFF + grp * NST * TILE_B;   // this group's V slots
  struct TileWalk {  // position of a load stream in the split's list of visible tiles
    int sidx, sub, left;
  };
  auto walk_init = [&](int j) __attribute__((always_inline)) {  // group-local tile j (clamped)
    TileWalk w;
    const int last = n_g > 0 ? n_g - 1 : 0;
    const int jc = j < last ? j : last;
    int g = t_begin + grp + jc * GROUPS;
    if (g >= t_end) g = t_end - 1;  // group without tiles: any valid tile, its result is discarded
    w.sidx = g / tps;
    w.sub = g - w.sidx * tps;
    w.left = last - jc;
    return w;
  };
  auto walk_next = [&](TileWalk& w) __attribute__((always_inline)) {
    if (w.left > 0) {
      --w.left;
      w.sub += GROUPS;
      while (w.sub >= tps) {
        w.sub -= tps;
        ++w.sidx;
      }
    }
  };
  auto tile_base = [&](uint64_t base, const TileWalk& w) __attribute__((always_inline)) {
    const int slot = __builtin_amdgcn_readfirstlane(vis[w.sidx]);
    const int64_t row0 = (int64_t)slot * p.T + (int64_t)w.sub * BN;
    return uniform64(base + (uint64_t)row0 * ROW_B);
  };
  auto dma_k = [&](const TileWalk& w, int slot) __attribute__((always_inline)) {
    const uint64_t g = tile_base(kbase, w);
#pragma unroll
    for (int i = 0; i < NDMA; ++i)
      dma16(g, kvoff[i], __builtin_amdgcn_readfirstlane(k_ring + slot * TILE_B + (wig + i * WPG) * 1024));
  };
  auto dma_v = [&](const TileWalk& w, int slot) __attribute__((always_inline)) {
    const uint64_t g = tile_base(vbase, w);
#pragma unroll
    for (int i = 0; i < NDMA; ++i)
      dma16(g, vvoff[i], __builtin_amdgcn_readfirstlane(v_ring + slot * TILE_B + (wig + i * WPG) * 1024));
  };

  // ---- fragment read addresses (bytes from smem) ----
  // K row l32 (+32 per key block), logical chunk 2*ks + hh: physical chunk bits [3:1] are
  // ks ^ (swz >> 1), so the address for step ks is the step-0 address with bits 5.. flipped.
  uint32_t k_rd[KS];
  {
    const int x = k_swz<DH>(l32);
    const uint32_t a0 = grp * NST * TILE_B + l32 * ROW_B + ((((x >> 1) << 1) | (hh ^ (x & 1))) << 4);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_rd[ks] = a0 ^ (ks << 5);
  }
  // V rows 4*hh + r (r = lane bits 3:2) of each 8-row group, logical chunk 4*db + c.
  uint32_t v_rd[DB];
  {
    const int r = 4 * hh + ((lane & 15) >> 2);
    const int y = v_swz<DH>(r) >> 2;
    const int c = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_rd[db] = L::V_OFF + grp * NST * TILE_B + r * ROW_B + (((db ^ y) * 4 + c) << 4) + (lane & 1) * 8;
  }

  f32x16_t o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m_ref = -INFINITY, l_run = 0.f;

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float kDead = 3.0e4f;  // shift of logits that must not count (tiles past the group's end)
  // K-side fragment of the shift product: contraction index 0 is one for every key
  frag_t ones_frag = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
  if (hh == 0) ones_frag[0] = (typename M::elem_t)1.0f;
  // Q-side fragments: contraction index 0 carries -m_ref of this lane's query, or -kDead
  frag_t shift = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
  frag_t dead = shift;
  if (hh == 0) dead[0] = (typename M::elem_t)(-kDead);
  auto set_shift = [&]() __attribute__((always_inline)) {
    shift = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
    if (hh == 0) shift[0] = (typename M::elem_t)(-m_ref);
  };

  // logits of the 64-key tile in K slot `slot`, starting from `init` (a shift product or zero)
  auto logits = [&](f32x16_t(&s)[2], int slot, bool shifted, const frag_t& sh) __attribute__((always_inline)) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      s[kb] = shifted ? M::mma(ones_frag, sh, zero16) : zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const frag_t a = *reinterpret_cast<const frag_t*>(smem + k_rd[ks] + slot * TILE_B + kb * 32 * ROW_B);
        s[kb] = M::mma(a, qf[ks], s[kb]);
      }
    }
  };
  // O^T += V^T P^T for the tile in V slot `slot`
  auto accumulate = [&](const frag_t(&pf)[4], int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const unsigned char* va = smem + v_rd[db] + slot * TILE_B + 16 * m * ROW_B;
        const s16x4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va));
        const s16x4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va + 8 * ROW_B));
        typedef short s16x8_t __attribute__((ext_vector_type(8)));
        const s16x8_t a8 = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        o[db] = M::mma(__builtin_bit_cast(frag_t, a8), pf[m], o[db]);
      }
    }
  };
  // probabilities of one tile from its shifted logits: p = 2^(s - sub), packed to the element
  // type; returns this half-wave's share of the row sum (of the rounded values)
  auto probabilities = [&](frag_t(&pf)[4], const f32x16_t(&s)[2], float sub) __attribute__((always_inline)) {
    float rs = 0.f;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const f32x16_t& sv = s[m >> 1];
      const int r0 = 8 * (m & 1);
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(sv[r0 + j] - sub);
      pf[m] = M::pack8(e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]);
#pragma unroll
      for (int j = 0; j < 4; ++j) rs = M::add_pair(rs, pf[m], j);
    }
    return rs;
  };
  auto tile_max = [&](const f32x16_t(&s)[2]) __attribute__((always_inline)) {
    float mx = s[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
    float lo, up;
    half_wave_pair(mx, lo, up);
    return fmaxf(lo, up);
  };

  if (ntile > 0) {
    frag_t p_prev[4];
    f32x16_t s_cur[2];
    {
      // zero the V slot that stands in for "tile -1" and P, so the first product adds zeros
      const u32x4_t z = {0u, 0u, 0u, 0u};
      unsigned char* vz = smem + L::V_OFF + (grp * NST + NST - 1) * TILE_B;
      for (int i = wig * 64 + lane; i < TILE_B / 16; i += WPG * 64) *reinterpret_cast<u32x4_t*>(vz + i * 16) = z;
#pragma unroll
      for (int m = 0; m < 4; ++m) p_prev[m] = __builtin_bit_cast(frag_t, z);
    }
    // Prologue issue order mirrors the loop's (K(j+NST), V(j+NST-2) in iteration j).
    TileWalk kw = walk_init(0), vw = walk_init(0);
    if (NST == 4) {
      dma_k(kw, 0); walk_next(kw);
      dma_k(kw, 1); walk_next(kw);
      dma_k(kw, 2); walk_next(kw);
      dma_v(vw, 0); walk_next(vw);
      dma_k(kw, 3); walk_next(kw);
      dma_v(vw, 1); walk_next(vw);
      dma_wait<5 * NDMA>();
    } else {
      dma_k(kw, 0); walk_next(kw);
      dma_k(kw, 1); walk_next(kw);
      dma_wait<NDMA>();
    }
    __syncthreads();  // K(0) and the zeroed V slot are in LDS
    // first tile: plain logits, reference = its row max, shifted by hand
    logits(s_cur, 0, false, shift);
    if (n_g > 0) {
      m_ref = M::round_up(tile_max(s_cur));
      set_shift();
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_cur[kb][i] -= m_ref;
    } else {  // this group has no tile of its own: everything it computes is weighted 2^-kDead
      m_ref = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_cur[kb][i] = -kDead;
    }
    if (NST == 4) dma_wait<4 * NDMA>(); else dma_wait<0>();
    __syncthreads();  // K(1) landed; K slot 0 may be overwritten

    // A raise decided in iteration j rescales the accumulators after the product of tile j-1
    // and before that of tile j, i.e. at the top of iteration j+1; with the branch there the
    // rest of the body stays one basic block for the scheduler to interleave.
    bool pending = false;
    float alpha = 1.f;
    auto rescale = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    };

    // one iteration with compile-time ring positions (JM = j mod NST)
    auto iteration = [&](int j, auto jm_c) __attribute__((always_inline)) {
      constexpr int JM = decltype(jm_c)::value;
      if (pending) rescale();
      pending = false;
      dma_k(kw, JM);                          // K(j+NST)
      walk_next(kw);
      dma_v(vw, (JM + NST - 2) % NST);        // V(j+NST-2)
      walk_next(vw);

      // matrix cores: shifted logits of tile j+1 (weighted out if past this group's end)
      f32x16_t s_next[2];
      logits(s_next, (JM + 1) % NST, true, (j + 1 < n_g) ? shift : dead);

      // VALU: probabilities of tile j
      frag_t p_cur[4];
      float rs = probabilities(p_cur, s_cur, 0.f);

      // matrix cores: O += P(j-1) V(j-1)
      accumulate(p_prev, (JM + NST - 1) % NST);

      // Issue order for the block above: keep several LDS fragment reads in flight ahead of the
      // MFMA that consumes them and spread the vector work between the MFMAs.
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int i = 0; i < 6; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
      }
#pragma unroll
      for (int i = 6; i < 2 * KS + 2 + 4 * DB; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
      }

      if (__ballot(!(rs <= 256.f)) != 0ull) {
        // Rare: some probability of this tile may exceed 2^8.  Raise the reference of the rows
        // that need it, redo the tile's probabilities exactly, and re-base the logits of the
        // next tile, which were produced with the old reference.
        const float mx = tile_max(s_cur);
        const float m_new = mx > 0.f ? M::round_up(m_ref + mx) : m_ref;
        const float delta = m_new - m_ref;
        alpha = __builtin_amdgcn_exp2f(-delta);
        rs = probabilities(p_cur, s_cur, delta);
        l_run *= alpha;
        m_ref = m_new;
        set_shift();
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) s_next[kb][i] -= delta;
        pending = true;
      }
      l_run += rs;
#pragma unroll
      for (int m = 0; m < 4; ++m) p_prev[m] = p_cur[m];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) s_cur[kb] = s_next[kb];
      dma_wait<(NST - 2) * 2 * NDMA>();  // K(j+2) and V(j) have landed (this wavefront's part)
      __syncthreads();
    };

    int j = 0;
    if (NST == 4) {
      for (; j + 4 <= n_iter; j += 4) {
        iteration(j, IntC<0>());
        iteration(j + 1, IntC<1>());
        iteration(j + 2, IntC<2>());
        iteration(j + 3, IntC<3>());
      }
      if (j < n_iter) { iteration(j, IntC<0>()); ++j; }
      if (j < n_iter) { iteration(j, IntC<1>()); ++j; }
      if (j < n_iter) { iteration(j, IntC<2>()); ++j; }
    } else {
      for (; j + 2 <= n_iter; j += 2) {
        iteration(j, IntC<0>());
        iteration(j + 1, IntC<1>());
      }
      if (j < n_iter) { iteration(j, IntC<0>()); ++j; }
    }
    if (pending) rescale();
    // product of the last tile: V(n_iter-1) sits in slot (n_iter-1) mod NST
    {
      const int last = (n_iter - 1) % NST;
      if (last == 0) accumulate(p_prev, 0);
      else if (last == 1) accumulate(p_prev, 1);
      else if (NST == 4 && last == 2) accumulate(p_prev, 2);
      else accumulate(p_prev, NST - 1);
    }
    dma_wait<0>();  // no DMA may still be writing LDS when the rings are reused or the CU is freed
  }
  if (n_g == 0) {
    m_ref = -INFINITY;
    l_run = 0.f;
  }

  float lo, up;
  half_wave_pair(l_run, lo, up);
  float l_tot = lo + up;

  if (GROUPS == 2) {
    // ---- merge the two groups' (m, l, O) through LDS; group 0 keeps the result ----
    __syncthreads();  // every wavefront is done with the rings
    float* mb = reinterpret_cast<float*>(smem) + (wig * (DB * 16 + 2)) * 64 + lane;
    if (grp == 1) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) mb[(db * 16 + i) * 64] = o[db][i];
      mb[(DB * 16) * 64] = m_ref;
      mb[(DB * 16 + 1) * 64] = l_tot;
    }
    __syncthreads();
    if (grp == 1) return;
    const float m1 = mb[(DB * 16) * 64], l1 = mb[(DB * 16 + 1) * 64];
    const float mm = fmaxf(m_ref, m1);
    if (mm > -INFINITY) {
      const float a0 = __builtin_amdgcn_exp2f(m_ref - mm), a1 = __builtin_amdgcn_exp2f(m1 - mm);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = a0 * o[db][i] + a1 * mb[(db * 16 + i) * 64];
      l_tot = a0 * l_tot + a1 * l1;
      m_ref = mm;
    }
  }

  // ---- epilogue ----
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const bool valid = qrow < p.T;
  const float inv = (p.n_splits == 1) ? 1.f / l_tot : 1.f;
  const int64_t row = ((int64_t)b * p.H + h) * p.T + qrow;
  if (p.n_splits > 1 && valid && hh == 0) {
    float2 ml = make_float2(m_ref, l_tot);
    *reinterpret_cast<float2*>(p.ws_ml + ((int64_t)split * rows + row) * 2) = ml;
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
        auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(o[db][4 * c + e] * inv),
                                                  __float_as_uint(o[db][4 * c + 4 + e] * inv), false, false);
        f[e] = __uint_as_float(r[0]);
        f[4 + e] = __uint_as_float(r[1]);
      }
      const int d0 = 32 * db + 8 * (c + hh);
      if (valid) {
        if (p.n_splits == 1) {
          uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h +
                          (int64_t)qrow * p.os_t + d0;
          *reinterpret_cast<frag_t*>(dst) = M::pack8(f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]);
        } else {
          float* dst = p.ws_o + ((int64_t)split * rows + row) * DH + d0;
          *reinterpret_cast<float4*>(dst) = make_float4(f[0], f[1], f[2], f[3]);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(f[4], f[5], f[6], f[7]);
        }
      }
    }
  }
}

template <typename M, int DH, int GROUPS>
static hipError_t launch_ring8_t(const AttnParams& p, hipStream_t stream) {
  static bool configured = false;
  const int lds = Ring8Lds<DH>::kBytes;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_ring8_kernel<M, DH, GROUPS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int rounds = (p.unit_splits + 7) / 8;
  const unsigned grid = (unsigned)(rounds * 8 * p.members);
  hipLaunchKernelGGL((attn_ring8_kernel<M, DH, GROUPS>), dim3(grid), dim3(512), lds, stream, p);
  return hipGetLastError();
}

hipError_t launch_attn_ring8(const AttnParams& p, int Dh, int dtype, int groups, hipStream_t stream) {
  if (dtype == WE_DTYPE_BF16) {
    if (Dh == 128) return groups == 2 ? launch_ring8_t<Bf16Mma, 128, 2>(p, stream) : launch_ring8_t<Bf16Mma, 128, 1>(p, stream);
    if (Dh == 64) return groups == 2 ? launch_ring8_t<Bf16Mma, 64, 2>(p, stream) : launch_ring8_t<Bf16Mma, 64, 1>(p, stream);
  } else if (dtype == WE_DTYPE_F16) {
    if (Dh == 128) return groups == 2 ? launch_ring8_t<F16Mma, 128, 2>(p, stream) : launch_ring8_t<F16Mma, 128, 1>(p, stream);
    if (Dh == 64) return groups == 2 ? launch_ring8_t<F16Mma, 64, 2>(p, stream) : launch_ring8_t<F16Mma, 64, 1>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace we
