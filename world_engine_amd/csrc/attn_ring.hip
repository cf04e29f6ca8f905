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
#include "we_common.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

namespace we {

constexpr int BN = 64;  // keys per tile

struct Bf16Mma {
  typedef bf16x8_t frag_t;
  __device__ static __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ frag_t pack8(float v0, float v1, float v2, float v3, float v4,
                                                 float v5, float v6, float v7) {
    frag_t r;
    r[0] = (__bf16)v0; r[1] = (__bf16)v1; r[2] = (__bf16)v2; r[3] = (__bf16)v3;
    r[4] = (__bf16)v4; r[5] = (__bf16)v5; r[6] = (__bf16)v6; r[7] = (__bf16)v7;
    return r;
  }
};
struct F16Mma {
  typedef f16x8_t frag_t;
  __device__ static __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ frag_t pack8(float v0, float v1, float v2, float v3, float v4,
                                                 float v5, float v6, float v7) {
    frag_t r;
    r[0] = (_Float16)v0; r[1] = (_Float16)v1; r[2] = (_Float16)v2; r[3] = (_Float16)v3;
    r[4] = (_Float16)v4; r[5] = (_Float16)v5; r[6] = (_Float16)v6; r[7] = (_Float16)v7;
    return r;
  }
};

// Both half-waves get (lower half's x, upper half's x).
__device__ __forceinline__ void half_wave_pair(float x, float& lower, float& upper) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  lower = __uint_as_float(r[0]);
  upper = __uint_as_float(r[1]);
}

typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;

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
  const int nvis = vis[WE_MAX_SLOTS + 1];
  const int tps = p.T / BN;  // tiles per slot
  const int nt = nvis * tps;
  const int t_begin = (int)((int64_t)split * nt / p.n_splits);
  const int t_end = (int)((int64_t)(split + 1) * nt / p.n_splits);
  const int ntile = t_end - t_begin;

  // ---- Q fragments stay in registers for the whole kernel ----
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
      for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = *reinterpret_cast<const frag_t*>(src + ks * 16);
    }
  }

  const int64_t cap = p.L + p.T;
  const uint16_t* kbase =
      reinterpret_cast<const uint16_t*>(p.kv) + ((int64_t)b * p.Hkv + hkv) * cap * DH;
  const uint16_t* vbase = kbase + (int64_t)p.B * p.Hkv * cap * DH;

  // One tile in flight: global -> registers (issued a whole compute phase before use) -> LDS.
  u32x4_t kreg[CPT], vreg[CPT];
  const int ld_r = tid / CPR, ld_c8 = tid % CPR;  // chunk c = tid + 256*i -> row ld_r + i*(256/CPR)
  auto load_tile = [&](int ti) __attribute__((always_inline)) {
    const int sidx = ti / tps;
    const int64_t row0 = (int64_t)vis[sidx] * p.T + (int64_t)(ti - sidx * tps) * BN;
    const uint16_t* kp = kbase + (row0 + ld_r) * DH + ld_c8 * 8;
    const uint16_t* vp = vbase + (row0 + ld_r) * DH + ld_c8 * 8;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      kreg[i] = *reinterpret_cast<const u32x4_t*>(kp + (int64_t)i * (256 / CPR) * DH);
      vreg[i] = *reinterpret_cast<const u32x4_t*>(vp + (int64_t)i * (256 / CPR) * DH);
    }
  };
  auto store_tile = [&](int buf) __attribute__((always_inline)) {
    uint16_t* kd = lds_k + buf * BN * KSTR + ld_r * KSTR + ld_c8 * 8;
    uint16_t* vd = lds_v + buf * BN * VSTR + ld_r * VSTR + ld_c8 * 8;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      *reinterpret_cast<u32x4_t*>(kd + i * (256 / CPR) * KSTR) = kreg[i];
      *reinterpret_cast<u32x4_t*>(vd + i * (256 / CPR) * VSTR) = vreg[i];
    }
  };

  f32x16_t o[NQB][DB];
  float m_run[NQB], l_run[NQB];
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
  }

  if (ntile > 0) load_tile(t_begin);

  const float c2 = p.scale_log2;
  // per-lane offsets of the fragment reads
  const int k_off = l32 * KSTR + hh * 8;
  const int v_off = (4 * hh + ((lane & 15) >> 2)) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  for (int it = 0; it < ntile; ++it) {
    // Stage tile `it` into buffer it&1.  Every wave finished reading that buffer (tile it-2)
    // before it passed the previous iteration's barrier, so one barrier per tile suffices.
    const int buf = it & 1;
    store_tile(buf);
    __syncthreads();
    if (it + 1 < ntile) load_tile(t_begin + it + 1);
    const uint16_t* kt = lds_k + buf * BN * KSTR + k_off;
    const uint16_t* vt = lds_v + buf * BN * VSTR + v_off;

    // ---- S^T = K Q^T : two 32-key blocks ----
    f32x16_t s[NQB][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[qb][kb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const frag_t a = *reinterpret_cast<const frag_t*>(kt + kb * 32 * KSTR + ks * 16);
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) s[qb][kb] = M::mma(a, qf[qb][ks], s[qb][kb]);
      }
    }

    // ---- online softmax; each lane owns one query column ----
    frag_t pf[NQB][4];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
      float mx = s[qb][0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[qb][kb][i]);
      float lo, up;
      half_wave_pair(mx, lo, up);
      mx = fmaxf(lo, up);
      const float m_new = fmaxf(m_run[qb], mx * c2);
      const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_new);
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][kb][i], c2, -m_new));
          s[qb][kb][i] = e;
          rs += e;
        }
      l_run[qb] = l_run[qb] * alpha + rs;
      m_run[qb] = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const f32x16_t& sv = s[qb][m >> 1];
        const int r0 = 8 * (m & 1);
        pf[qb][m] = M::pack8(sv[r0], sv[r0 + 1], sv[r0 + 2], sv[r0 + 3], sv[r0 + 4], sv[r0 + 5],
                             sv[r0 + 6], sv[r0 + 7]);
      }
    }

    // ---- O^T += V^T P^T : 4 chunks of 16 keys x DB blocks of 32 head-dim rows ----
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

  }

  // ---- epilogue ----
  const int64_t rows = (int64_t)p.B * p.H * p.T;
#pragma unroll
  for (int qb = 0; qb < NQB; ++qb) {
    float lo, up;
    half_wave_pair(l_run[qb], lo, up);
    const float l_tot = lo + up;
    const bool valid = qrow[qb] < p.T;
    const float inv = (p.n_splits == 1) ? 1.f / l_tot : 1.f;
    const int64_t row = ((int64_t)b * p.H + h) * p.T + qrow[qb];
    if (p.n_splits > 1 && valid && hh == 0) {
      float2 ml = make_float2(m_run[qb], l_tot);
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
          auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(o[qb][db][4 * c + e] * inv),
                                                    __float_as_uint(o[qb][db][4 * c + 4 + e] * inv),
                                                    false, false);
          f[e] = __uint_as_float(r[0]);
          f[4 + e] = __uint_as_float(r[1]);
        }
        const int d0 = 32 * db + 8 * (c + hh);
        if (valid) {
          if (p.n_splits == 1) {
            uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h +
                            (int64_t)qrow[qb] * p.os_t + d0;
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
}

// Second pass of the split-context path: out = sum_s w_s O_s / sum_s w_s l_s with
// w_s = 2^(m_s - max_s m_s).  One thread per (query row, 4 head-dim columns).
template <typename M, int DH>
__global__ void __launch_bounds__(256) attn_combine_kernel(AttnParams p) {
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * (DH / 4)) return;
  const int64_t row = idx / (DH / 4);
  const int dg = (int)(idx % (DH / 4));
  float mmax = -INFINITY;
  for (int s = 0; s < p.n_splits; ++s) mmax = fmaxf(mmax, p.ws_ml[((int64_t)s * rows + row) * 2]);
  float den = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s = 0; s < p.n_splits; ++s) {
    const float2 ml = *reinterpret_cast<const float2*>(p.ws_ml + ((int64_t)s * rows + row) * 2);
    const float w = __builtin_amdgcn_exp2f(ml.x - mmax);
    const float4 ov = *reinterpret_cast<const float4*>(p.ws_o + ((int64_t)s * rows + row) * DH + dg * 4);
    den += w * ml.y;
    acc.x += w * ov.x;
    acc.y += w * ov.y;
    acc.z += w * ov.z;
    acc.w += w * ov.w;
  }
  const float inv = 1.f / den;
  const int t = (int)(row % p.T);
  const int64_t bh = row / p.T;
  const int h = (int)(bh % p.H);
  const int b = (int)(bh / p.H);
  uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)t * p.os_t + dg * 4;
  typename M::frag_t pk = M::pack8(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv, 0.f, 0.f, 0.f, 0.f);
  const uint4 bits = __builtin_bit_cast(uint4, pk);
  *reinterpret_cast<uint2*>(dst) = make_uint2(bits.x, bits.y);
}

int attn_block_m(int Dh, int variant) {
  (void)Dh;
  return variant == 2 ? 256 : 128;
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
  const int64_t total = (int64_t)p.B * p.H * p.T * (Dh / 4);
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
