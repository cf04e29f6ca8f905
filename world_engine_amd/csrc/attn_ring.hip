// Frame-block-causal flash attention over the KV ring buffer (gfx950, wave64, MFMA).
//
// Replaces the reference's make_block_mask + flex_attention pair (src/model/kv_cache.py:12-61,
// :141-144; src/model/attn.py:116).  A key row is visible iff it is in the tail [L, L+T) or in
// a ring slot s with written[s*T] set that is not the slot the current frame replaces on a
// persisting frame.  Visibility is per slot and identical for every batch element, head and
// query, so the kernel builds a short list of visible slots and walks those slots of the
// cache buffer in place, 64 keys at a time; no mask tensor and no gathered context exist.
//
// Work decomposition: one workgroup of 4 wavefronts per (batch, head, query tile, context
// split).  Each wavefront owns NQB blocks of 32 queries.  Per 64-key tile:
//   S^T[key][query] = K Q^T       v_mfma_f32_32x32x16 with A = K rows from LDS (one 16-byte
//                                 ds_read per fragment), B = Q rows held in registers.
//   online softmax                every lane owns ONE query column of S^T, so the row max
//                                 and row sum are register reductions plus one
//                                 v_permlane32_swap between the two half-waves.
//   O^T[d][query] += V^T P^T      A = V^T fragments fetched with ds_read_b64_tr_b16 from the
//                                 row-major V tile (the LDS transposing read of gfx950),
//                                 B = P^T: the S^T accumulators already have the B-operand
//                                 layout, so P never leaves registers.
// K/V tiles go HBM -> registers -> LDS (double buffered, one barrier per tile); the global
// loads of tile i+1 are in flight while tile i is being computed.
// Workgroup ids are laid out so that the workgroups sharing one K/V stream (query tiles and
// grouped query heads) run on the same XCD and hit in its L2.
//
// Roofline: 4*T*N_vis*Dh flops and 4*N_vis*Dh bytes of K/V per (batch, kv head); HBM-bound for
// 256-query frames (with context splits to fill 256 CUs), MFMA-bound for 1024-query frames.
#include "attn_mma.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

namespace we {

template <int DH>
struct AttnLds {
  static constexpr int KSTR = DH + 8;   // K row stride: 16-byte reads of 16 consecutive rows hit all banks
  static constexpr int VSTR = DH + 32;  // V row stride: transposing 8-byte reads of 4 rows x 64 bytes hit all banks
  static constexpr int kBytes = 2 * BN * KSTR * 2 + 2 * BN * VSTR * 2 + (WE_MAX_SLOTS + 2) * 4;
};

template <typename M, int DH, int NQB>
__global__ void __launch_bounds__(256, NQB == 1 ? 2 : 1) attn_ring_kernel(AttnParams p) {
  typedef typename M::frag_t frag_t;
  constexpr int KSTR = AttnLds<DH>::KSTR, VSTR = AttnLds<DH>::VSTR;
  constexpr int KS = DH / 16;            // contraction steps of K Q^T
  constexpr int DB = DH / 32;            // 32-row blocks of O^T
  constexpr int BM = 128 * NQB;          // queries per workgroup
  constexpr int CPR = DH / 8;            // 16-byte chunks per K/V row
  constexpr int CPT = BN * CPR / 256;    // chunks per thread per tile

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* lds_k = reinterpret_cast<uint16_t*>(smem);  // [2][BN][KSTR]
  uint16_t* lds_v = lds_k + 2 * BN * KSTR;              // [2][BN][VSTR]
  int* vis = reinterpret_cast<int*>(lds_v + 2 * BN * VSTR);  // visible slots, then their count

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;

  // ---- which (batch, head, query tile, split) this workgroup owns; XCD = blockIdx % 8 ----
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int round = jj / p.members, member = jj - round * p.members;
  const int us = round * 8 + xcd;
  if (us >= p.unit_splits) return;
  // leading units run unsplit; the rest are cut into n_splits context parts each
  int unit, split, nsp;
  if (us < p.units_whole) {
    unit = us; split = 0; nsp = 1;
  } else {
    const int r = us - p.units_whole;
    unit = p.units_whole + r / p.n_splits; split = r % p.n_splits; nsp = p.n_splits;
  }
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
  const int nvis = vis[WE_MAX_SLOTS + 1];
  const int tps = p.T / BN;  // tiles per slot
  const int nt = nvis * tps;
  const int t_begin = (int)((int64_t)split * nt / nsp);
  const int t_end = (int)((int64_t)(split + 1) * nt / nsp);
  const int ntile = t_end - t_begin;

  // ---- Q fragments stay in registers for the whole kernel, pre-multiplied by scale*log2(e) so
  // the matrix product yields base-2 logits directly ----
  const float c2 = p.scale_log2;
  frag_t qf[NQB][KS];
  int qrow[NQB];
  {
    const uint16_t* qbase = reinterpret_cast<const uint16_t*>(p.q) + b * p.qs_b + h * p.qs_h;
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
      qrow[qb] = qtile * BM + wave * (32 * NQB) + qb * 32 + l32;
      const int qr = qrow[qb] < p.T ? qrow[qb] : p.T - 1;
      const uint16_t* src = qbase + (int64_t)qr * p.qs_t + hh * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const frag_t raw = *reinterpret_cast<const frag_t*>(src + ks * 16);
        qf[qb][ks] = M::pack8((float)raw[0] * c2, (float)raw[1] * c2, (float)raw[2] * c2, (float)raw[3] * c2,
                              (float)raw[4] * c2, (float)raw[5] * c2, (float)raw[6] * c2, (float)raw[7] * c2);
      }
    }
  }

  const int64_t cap = p.L + p.T;
  const uint16_t* kbase =
      reinterpret_cast<const uint16_t*>(p.kv) + ((int64_t)b * p.Hkv + hkv) * cap * DH;
  const uint16_t* vbase = kbase + (int64_t)p.B * p.Hkv * cap * DH;

  // ---- software pipeline -------------------------------------------------------------------
  // Iteration `it` holds the logits of tile `it` (s_cur), computes the logits of tile it+1 and
  // the P*V product of tile it-1 on the matrix cores while the VALU turns s_cur into
  // probabilities.  LDS: K(it+1) in kb[(it+1)&1], V(it-1) in vb[(it-1)&1]; the stores of K(it+2)
  // and V(it) go into the two buffers nobody reads during this iteration, so one barrier per
  // tile is enough.  Global loads run one iteration ahead of their LDS store (K(it+3), V(it+1)).
  // Tile indices past the end are clamped (the last tile is re-loaded and its logits recomputed
  // once), which keeps the loop body free of branches.
  //
  // The logits leave the matrix cores already shifted by the running reference m_ref: one extra
  // MFMA per 32-key block multiplies a column of ones (K side) with a fragment holding -m_ref
  // (Q side; m_ref is kept representable in the element type so the shift is exact).  The VALU
  // work per element is then exp2, a pack, and half a dot2 for the row sum.  m_ref is raised
  // only when a row sum shows a probability above 2^8 (then that tile is redone exactly); being
  // larger than the true running max is never needed for fp32 accumulators.
  u32x4_t kreg[CPT], vreg[CPT];
  const int ld_r = tid / CPR, ld_c8 = tid % CPR;  // chunk c = tid + 256*i -> row ld_r + i*(256/CPR)
  struct TileWalk {  // position of a load stream in this split's list of visible tiles
    int sidx, sub, left;
  };
  auto walk_init = [&](int ti) __attribute__((always_inline)) {
    TileWalk w;
    const int g = t_begin + (ti < ntile ? ti : ntile - 1);
    w.sidx = g / tps;
    w.sub = g - w.sidx * tps;
    w.left = ntile - 1 - (ti < ntile ? ti : ntile - 1);
    return w;
  };
  auto walk_next = [&](TileWalk& w) __attribute__((always_inline)) {
    if (w.left > 0) {
      --w.left;
      if (++w.sub == tps) {
        w.sub = 0;
        ++w.sidx;
      }
    }
  };
  auto tile_ptr = [&](const uint16_t* base, const TileWalk& w) __attribute__((always_inline)) {
    const int slot = __builtin_amdgcn_readfirstlane(vis[w.sidx]);
    const int64_t row0 = (int64_t)slot * p.T + (int64_t)w.sub * BN;
    return base + (row0 + ld_r) * DH + ld_c8 * 8;
  };
  auto gload = [&](u32x4_t(&r)[CPT], const uint16_t* src) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      r[i] = *reinterpret_cast<const u32x4_t*>(src + (int64_t)i * (256 / CPR) * DH);
  };
  auto lstore = [&](uint16_t* dst, int stride, const u32x4_t(&r)[CPT]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) *reinterpret_cast<u32x4_t*>(dst + i * (256 / CPR) * stride) = r[i];
  };
  uint16_t* const k_st = lds_k + ld_r * KSTR + ld_c8 * 8;  // this thread's staging slots
  uint16_t* const v_st = lds_v + ld_r * VSTR + ld_c8 * 8;
  // per-lane offsets of the fragment reads
  const uint16_t* const k_rd = lds_k + l32 * KSTR + hh * 8;
  const uint16_t* const v_rd =
      lds_v + (4 * hh + ((lane & 15) >> 2)) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  f32x16_t o[NQB][DB];
  float m_ref[NQB], l_run[NQB];
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    m_ref[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
  }

  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // K-side fragment of the shift product: contraction index 0 is one for every key
  frag_t ones_frag = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
  if (hh == 0) ones_frag[0] = (typename M::elem_t)1.0f;
  // Q-side fragment: contraction index 0 carries -m_ref of this lane's query
  frag_t shift[NQB];
  auto set_shift = [&](int qb) __attribute__((always_inline)) {
    shift[qb] = __builtin_bit_cast(frag_t, u32x4_t{0u, 0u, 0u, 0u});
    if (hh == 0) shift[qb][0] = (typename M::elem_t)(-m_ref[qb]);
  };

  // logits of one 64-key tile in LDS buffer `kt`, already minus m_ref when `shifted`
  auto logits = [&](f32x16_t(&s)[NQB][2], const uint16_t* kt, bool shifted) __attribute__((always_inline)) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
        s[qb][kb] = shifted ? M::mma(ones_frag, shift[qb], zero16) : zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const frag_t a = *reinterpret_cast<const frag_t*>(kt + kb * 32 * KSTR + ks * 16);
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) s[qb][kb] = M::mma(a, qf[qb][ks], s[qb][kb]);
      }
    }
  };
  // O^T += V^T P^T for one 64-key tile in LDS buffer `vt`
  auto accumulate = [&](const frag_t(&pf)[NQB][4], const uint16_t* vt) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const uint16_t* va = vt + 16 * m * VSTR + 32 * db;
        const s16x4_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va));
        const s16x4_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(va + 8 * VSTR));
        typedef short s16x8_t __attribute__((ext_vector_type(8)));
        const s16x8_t a8 = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        const frag_t a = __builtin_bit_cast(frag_t, a8);
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) o[qb][db] = M::mma(a, pf[qb][m], o[qb][db]);
      }
    }
  };
  // probabilities of one tile from its shifted logits: p = 2^s, packed to the element type;
  // returns this half-wave's share of the row sum (of the rounded values)
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
    frag_t p_prev[NQB][4];
    f32x16_t s_cur[NQB][2];
    {
      // zero V buffer 1 and P so that the first iteration's product adds exact zeros
      const u32x4_t z = {0u, 0u, 0u, 0u};
      for (int i = tid; i < BN * VSTR / 8; i += 256)
        *reinterpret_cast<u32x4_t*>(lds_v + BN * VSTR + i * 8) = z;
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int m = 0; m < 4; ++m) p_prev[qb][m] = __builtin_bit_cast(frag_t, z);
    }
    TileWalk kw = walk_init(0), vw = walk_init(0);
    gload(kreg, tile_ptr(kbase, kw));  // K(0)
    walk_next(kw);
    gload(vreg, tile_ptr(kbase, kw));  // K(1)
    walk_next(kw);
    lstore(k_st, KSTR, kreg);
    lstore(k_st + BN * KSTR, KSTR, vreg);
    gload(kreg, tile_ptr(kbase, kw));  // K(2)
    walk_next(kw);
    gload(vreg, tile_ptr(vbase, vw));  // V(0)
    walk_next(vw);
    __syncthreads();
    // first tile: plain logits, reference = its row max, then shift by hand
    logits(s_cur, k_rd, false);
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
      m_ref[qb] = M::round_up(tile_max(s_cur[qb]));
      set_shift(qb);
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_cur[qb][kb][i] -= m_ref[qb];
    }
    __syncthreads();  // K buffer 0 is overwritten by the first iteration

    // A raise decided in iteration it rescales the accumulators after the product of tile it-1
    // and before that of tile it, i.e. at the top of iteration it+1; with the branch there the
    // rest of the body stays one basic block for the scheduler to interleave.
    bool pending = false;
    float alpha[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) alpha[qb] = 1.f;
    auto rescale = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha[qb];
    };

    for (int it = 0; it < ntile; ++it) {
      if (pending) rescale();
      pending = false;
      const int cur = it & 1, nxt = cur ^ 1;
      lstore(k_st + cur * BN * KSTR, KSTR, kreg);  // K(it+2)
      lstore(v_st + cur * BN * VSTR, VSTR, vreg);  // V(it)
      gload(kreg, tile_ptr(kbase, kw));            // K(it+3)
      walk_next(kw);
      gload(vreg, tile_ptr(vbase, vw));            // V(it+1)
      walk_next(vw);

      // matrix cores: shifted logits of tile it+1
      f32x16_t s_next[NQB][2];
      logits(s_next, k_rd + nxt * BN * KSTR, true);

      // VALU: probabilities of tile it
      frag_t p_cur[NQB][4];
      float rs[NQB];
      bool bad = false;
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) {
        rs[qb] = probabilities(p_cur[qb], s_cur[qb], 0.f);
        bad = bad || !(rs[qb] <= 256.f);
      }

      // matrix cores: O += P(it-1) V(it-1)
      accumulate(p_prev, v_rd + nxt * BN * VSTR);

      if (__ballot(bad) != 0ull) {
        // Rare: some probability of this tile may exceed 2^8.  Raise the reference of the rows
        // that need it, redo the tile's probabilities exactly, and re-base the logits of the
        // next tile, which were produced with the old reference.
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
          const float mx = tile_max(s_cur[qb]);
          const float m_new = mx > 0.f ? M::round_up(m_ref[qb] + mx) : m_ref[qb];
          const float delta = m_new - m_ref[qb];
          alpha[qb] = __builtin_amdgcn_exp2f(-delta);
          rs[qb] = probabilities(p_cur[qb], s_cur[qb], delta);
          l_run[qb] *= alpha[qb];
          m_ref[qb] = m_new;
          set_shift(qb);
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s_next[qb][kb][i] -= delta;
        }
        pending = true;
      }
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb) {
        l_run[qb] += rs[qb];
#pragma unroll
        for (int m = 0; m < 4; ++m) p_prev[qb][m] = p_cur[qb][m];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) s_cur[qb][kb] = s_next[qb][kb];
      }
      __syncthreads();
    }
    if (pending) rescale();
    accumulate(p_prev, v_rd + ((ntile - 1) & 1) * BN * VSTR);
  }
  float m_run[NQB];
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) m_run[qb] = m_ref[qb];

  // ---- epilogue ----
  const int64_t rows = (int64_t)p.B * p.H * p.T - p.ws_row0;  // rows in the workspace
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    float lo, up;
    half_wave_pair(l_run[qb], lo, up);
    const float l_tot = lo + up;
    const bool valid = qrow[qb] < p.T;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int64_t row = ((int64_t)b * p.H + h) * p.T + qrow[qb];
    if (nsp > 1 && valid && hh == 0) {
      float2 ml = make_float2(m_run[qb], l_tot);
      *reinterpret_cast<float2*>(p.ws_ml + ((int64_t)split * rows + (row - p.ws_row0)) * 2) = ml;
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
          auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(o[qb][db][4 * c + e] * inv),
                                                    __float_as_uint(o[qb][db][4 * c + 4 + e] * inv),
                                                    false, false);
          f[e] = __uint_as_float(r[0]);
          f[4 + e] = __uint_as_float(r[1]);
        }
        const int d0 = 32 * db + 8 * (c + hh);
        if (valid) {
          if (nsp == 1) {
            uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h +
                            (int64_t)qrow[qb] * p.os_t + d0;
            *reinterpret_cast<frag_t*>(dst) = M::pack8(f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]);
          } else {
            uint16_t* dst = p.ws_o + ((int64_t)split * rows + (row - p.ws_row0)) * DH + d0;
            *reinterpret_cast<frag_t*>(dst) = M::pack8(f[0], f[1], f[2], f[3], f[4], f[5], f[6], f[7]);
          }
        }
      }
    }
  }
}

// Second pass of the split-context path.  Every split left, per query row, its normalised
// output O_s (element type), its reference m_s (log2 domain) and its sum l_s; the result is
// sum_s w_s O_s / sum_s w_s with w_s = 2^(m_s - max m) * l_s.  One thread per (row, 8 columns).
template <typename M, int DH>
__global__ void __launch_bounds__(256) attn_combine_kernel(AttnParams p) {
  typedef typename M::frag_t frag_t;
  const int64_t rows = (int64_t)p.B * p.H * p.T - p.ws_row0;  // rows that were split
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * (DH / 8)) return;
  const int64_t row = idx / (DH / 8);  // workspace row; query row = row + ws_row0
  const int dg = (int)(idx % (DH / 8));
  // Splits are merged eight at a time with all sixteen loads of a batch issued before the first
  // use (a plain loop over a run-time split count would serialise one memory round trip per split).
  float mmax = -INFINITY, den = 0.f;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int s0 = 0; s0 < p.n_splits; s0 += 8) {
    float2 ml[8];
    frag_t ov[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < p.n_splits ? s0 + j : p.n_splits - 1;  // clamp: duplicates get weight 0 below
      ml[j] = *reinterpret_cast<const float2*>(p.ws_ml + ((int64_t)s * rows + row) * 2);
      ov[j] = *reinterpret_cast<const frag_t*>(p.ws_o + ((int64_t)s * rows + row) * DH + dg * 8);
    }
    float bmax = mmax;
#pragma unroll
    for (int j = 0; j < 8; ++j) bmax = fmaxf(bmax, ml[j].x);
    const float carry = bmax > -INFINITY ? __builtin_amdgcn_exp2f(mmax - bmax) : 0.f;  // 0 on the first batch
    den *= carry;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= carry;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float w = (s0 + j < p.n_splits && ml[j].y > 0.f) ? __builtin_amdgcn_exp2f(ml[j].x - bmax) * ml[j].y : 0.f;
      den += w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w * (float)ov[j][e];
    }
    mmax = bmax;
  }
  const float inv = 1.f / den;
  const int64_t qrow = row + p.ws_row0;
  const int t = (int)(qrow % p.T);
  const int64_t bh = qrow / p.T;
  const int h = (int)(bh % p.H);
  const int b = (int)(bh / p.H);
  uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)t * p.os_t + dg * 8;
  *reinterpret_cast<frag_t*>(dst) = M::pack8(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv, acc[4] * inv,
                                             acc[5] * inv, acc[6] * inv, acc[7] * inv);
}

template <typename M, int DH, int NQB>
static hipError_t launch_attn_t(const AttnParams& p, hipStream_t stream) {
  static bool configured = false;
  const int lds = AttnLds<DH>::kBytes;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_ring_kernel<M, DH, NQB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int rounds = (p.unit_splits + 7) / 8;
  const unsigned grid = (unsigned)(rounds * 8 * p.members);
  hipLaunchKernelGGL((attn_ring_kernel<M, DH, NQB>), dim3(grid), dim3(256), lds, stream, p);
  return hipGetLastError();
}

hipError_t launch_attn_ring(const AttnParams& p, int Dh, int dtype, int variant, hipStream_t stream) {
  const bool big = variant == 2;
  if (dtype == WE_DTYPE_BF16) {
    if (Dh == 128) return big ? launch_attn_t<Bf16Mma, 128, 2>(p, stream) : launch_attn_t<Bf16Mma, 128, 1>(p, stream);
    if (Dh == 64) return big ? launch_attn_t<Bf16Mma, 64, 2>(p, stream) : launch_attn_t<Bf16Mma, 64, 1>(p, stream);
  } else if (dtype == WE_DTYPE_F16) {
    if (Dh == 128) return big ? launch_attn_t<F16Mma, 128, 2>(p, stream) : launch_attn_t<F16Mma, 128, 1>(p, stream);
    if (Dh == 64) return big ? launch_attn_t<F16Mma, 64, 2>(p, stream) : launch_attn_t<F16Mma, 64, 1>(p, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_attn_combine(const AttnParams& p, int Dh, int dtype, hipStream_t stream) {
  const int64_t total = ((int64_t)p.B * p.H * p.T - p.ws_row0) * (Dh / 8);
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (dtype == WE_DTYPE_BF16) {
    if (Dh == 128) hipLaunchKernelGGL((attn_combine_kernel<Bf16Mma, 128>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((attn_combine_kernel<Bf16Mma, 64>), dim3(grid), dim3(256), 0, stream, p);
  } else {
    if (Dh == 128) hipLaunchKernelGGL((attn_combine_kernel<F16Mma, 128>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((attn_combine_kernel<F16Mma, 64>), dim3(grid), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace we
