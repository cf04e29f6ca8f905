// Merge of split-context partial results (gfx950): one output item = 8 consecutive head-dim
// columns of one query row.  Used by the second-pass kernel (attn_combine.hip).
#pragma once
#include "attn_mma.h"
#include "we_kernels.h"


namespace we {

// Every split left, per query row, its normalised output as fp16 values times a row scale r_s, its
// reference m_s (log2 domain) and its sum l_s; the result is sum_s w_s r_s O_s / sum_s w_s with
// w_s = 2^(m_s - max m) * l_s.  Splits are merged eight at a time with all sixteen loads of a batch
// issued before the first use (a plain loop over a run-time split count would serialise one memory
// round trip per split).
struct PartialBatch {
  f32x4_t ml[8];   // (m, l, row scale, -)
  f16x8_t ov[8];
};

// Requests splits [s0, s0 + 8) of one item: ml_off / o_off are the byte offsets of split 0's record
// and of its 8 columns in the two workspace areas, ml_step / o_step the distance between splits.
__device__ __forceinline__ void load_batch(PartialBatch& pb, const AttnParams& p, int64_t ml_off, int64_t o_off,
                                           int64_t ml_step, int64_t o_step, int s0) {
  const unsigned char* ml = reinterpret_cast<const unsigned char*>(p.ws_ml) + ml_off + (int64_t)s0 * ml_step;
  const unsigned char* ov = reinterpret_cast<const unsigned char*>(p.ws_o) + o_off + (int64_t)s0 * o_step;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if (s0 + j < p.n_splits) {  // (uniform: a request is 16 cycles of the CU's address path whether wanted or not)
      pb.ml[j] = *reinterpret_cast<const f32x4_t*>(ml);
      pb.ov[j] = *reinterpret_cast<const f16x8_t*>(ov);
    } else {
      pb.ml[j] = f32x4_t{-INFINITY, 0.f, 0.f, 0.f};
      pb.ov[j] = f16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
    ml += ml_step;
    ov += o_step;
  }
}

// Adds the batch's first `n_valid` splits to the running (reference, denominator, numerators).
__device__ __forceinline__ void accumulate_batch(const PartialBatch& pb, int n_valid, float& mmax, float& den, float (&acc)[8]) {
  float bmax = mmax;
#pragma unroll
  for (int j = 0; j < 8; ++j) bmax = fmaxf(bmax, pb.ml[j][0]);
  const float carry = bmax > -INFINITY ? __builtin_amdgcn_exp2f(mmax - bmax) : 0.f;  // 0 on the first batch
  den *= carry;
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] *= carry;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    // a part past the end, or one without keys, contributes nothing - not even 0 * inf
    if (j < n_valid && pb.ml[j][1] > 0.f) {
      const float w = __builtin_amdgcn_exp2f(pb.ml[j][0] - bmax) * pb.ml[j][1];
      den += w;
      const float wr = w * pb.ml[j][2];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wr * (float)pb.ov[j][e];
    }
  }
  mmax = bmax;
}

// Normalises, applies the head gate and stores columns [8 dg, 8 dg + 8) of query row (b, h, t).
template <typename M>
__device__ __forceinline__ void finish_item(const AttnParams& p, const float (&acc)[8], float den, int b, int h, int t, int dg) {
  typedef typename M::frag_t frag_t;
  const float inv = 1.f / den;
  uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)t * p.os_t + dg * 8;
  frag_t y = M::pack8(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv, acc[4] * inv, acc[5] * inv,
                      acc[6] * inv, acc[7] * inv);
  if (p.gate != nullptr || p.gate_w != nullptr) {  // y * gate on element-type values, as the module's own multiply
    const float g = head_gate<typename M::elem_t>(p, b, h, t);
    y = M::pack8((float)y[0] * g, (float)y[1] * g, (float)y[2] * g, (float)y[3] * g, (float)y[4] * g,
                 (float)y[5] * g, (float)y[6] * g, (float)y[7] * g);
  }
  *reinterpret_cast<frag_t*>(dst) = y;
}

// One output item, any number of splits: ml_off / o_off / ml_step / o_step as for load_batch, query
// row (b, h, t), columns [8 dg, 8 dg + 8).
template <typename M>
__device__ __forceinline__ void merge_item(const AttnParams& p, int64_t ml_off, int64_t o_off, int64_t ml_step,
                                           int64_t o_step, int b, int h, int t, int dg) {
  float mmax = -INFINITY, den = 0.f;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma nounroll
  for (int s0 = 0; s0 < p.n_splits; s0 += 8) {
    PartialBatch pb;
    load_batch(pb, p, ml_off, o_off, ml_step, o_step, s0);
    accumulate_batch(pb, p.n_splits - s0, mmax, den, acc);
  }
  finish_item<M>(p, acc, den, b, h, t, dg);
}

}  // namespace we
