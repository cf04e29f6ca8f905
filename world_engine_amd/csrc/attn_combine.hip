// Second pass of split-context attention over the KV ring buffer (gfx950): merges the per-split
// partial results the main kernel (attn_ring.hip) leaves in the workspace.
// HBM-bound: reads n_splits * (Dh * 2 + 16) bytes and writes Dh * 2 bytes per query row that was
// split.
#include "attn_mma.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

namespace we {

// Second pass of the split-context path.  Every split left, per query row, its normalised
// output as fp16 values in [-1, 1] times a row scale r_s, its reference m_s (log2 domain) and its
// sum l_s; the result is sum_s w_s r_s O_s / sum_s w_s with w_s = 2^(m_s - max m) * l_s.  One
// thread per (row, 8 columns);
// grid = (256-thread slices of one head's T * DH/8 items, split (batch, head) pairs), so that the
// start-up code has one 32-bit division in it (the kernel is short enough for that to show).
template <typename M, int DH>
__global__ void __launch_bounds__(256) attn_combine_kernel(AttnParams p) {
  typedef typename M::frag_t frag_t;
  const int64_t rows = (int64_t)p.B * p.H * p.T - p.ws_row0;  // rows that were split
  const int item = blockIdx.x * 256 + threadIdx.x;
  if (item >= p.T * (DH / 8)) return;
  const int t = item / (DH / 8), dg = item % (DH / 8);
  const int64_t row = (int64_t)blockIdx.y * p.T + t;  // workspace row; query row = row + ws_row0
  // Splits are merged eight at a time with all sixteen loads of a batch issued before the first
  // use (a plain loop over a run-time split count would serialise one memory round trip per split).
  float mmax = -INFINITY, den = 0.f;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  for (int s0 = 0; s0 < p.n_splits; s0 += 8) {
    f32x4_t ml[8];   // (m, l, row scale, -)
    f16x8_t ov[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < p.n_splits ? s0 + j : p.n_splits - 1;  // clamp: duplicates get weight 0 below
      ml[j] = *reinterpret_cast<const f32x4_t*>(p.ws_ml + ((int64_t)s * rows + row) * 4);
      ov[j] = *reinterpret_cast<const f16x8_t*>(p.ws_o + ((int64_t)s * rows + row) * DH + dg * 8);
    }
    float bmax = mmax;
#pragma unroll
    for (int j = 0; j < 8; ++j) bmax = fmaxf(bmax, ml[j][0]);
    const float carry = bmax > -INFINITY ? __builtin_amdgcn_exp2f(mmax - bmax) : 0.f;  // 0 on the first batch
    den *= carry;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= carry;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float w = (s0 + j < p.n_splits && ml[j][1] > 0.f) ? __builtin_amdgcn_exp2f(ml[j][0] - bmax) * ml[j][1] : 0.f;
      den += w;
      const float wr = w * ml[j][2];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wr * (float)ov[j][e];
    }
    mmax = bmax;
  }
  const float inv = 1.f / den;
  const unsigned bh = (unsigned)(p.units_whole * p.group) + blockIdx.y;  // first split pair + y
  const int b = (int)(bh / (unsigned)p.H), h = (int)(bh % (unsigned)p.H);
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

hipError_t launch_attn_combine(const AttnParams& p, int Dh, int dtype, hipStream_t stream) {
  const dim3 grid((unsigned)((p.T * (Dh / 8) + 255) / 256), (unsigned)(p.B * p.H - p.units_whole * p.group));
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
