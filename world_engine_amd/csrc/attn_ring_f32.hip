// fp32 attention over the KV ring buffer (gfx950): the same visibility rule and ring walk as the
// MFMA kernel (attn_ring.hip), computed entirely in fp32 on the vector ALUs.
//
// fp32 is the reference's CPU plumbing configuration (one layer, 64-token frames), not a serving
// path; this kernel exists so that the whole interface also works on fp32 caches, with results
// that follow the reference's fp32 arithmetic (fp32 scores, fp32 softmax, fp32 P V,
// src/model/attn.py:116 in eager mode).  It is a plain tiled kernel, not tuned.
//
// One workgroup = 64 queries of one (batch, head); a query is shared by 4 lanes that own DH/4
// head-dim values each.  K/V go through LDS 32 keys at a time; the softmax runs online per tile.
#include "we_common.h"
#include "we_kernels.h"
#include "../../include/we_attn.h"

namespace we {

template <int DH>
__global__ void __launch_bounds__(256) attn_ring_f32_kernel(AttnParams p) {
  constexpr int PART = DH / 4;   // head-dim values per lane
  constexpr int TK = 32;         // keys per tile
  __shared__ float ks[TK][DH];
  __shared__ float vs[TK][DH];
  __shared__ int vis[WE_MAX_SLOTS + 2];

  const int tid = threadIdx.x, lane = tid & 63;
  const int qi = tid >> 2, part = tid & 3;
  const int b = blockIdx.z, h = blockIdx.y, hkv = h / p.group;
  const int qrow = blockIdx.x * 64 + qi;

  // ---- list of visible slots; the tail is pseudo-slot n_slots ----
  if (tid < 64) {
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

  // ---- this lane's part of its query, pre-multiplied by scale * log2(e) ----
  float q[PART];
  {
    const int qr = qrow < p.T ? qrow : p.T - 1;
    const float* src = reinterpret_cast<const float*>(p.q) + b * p.qs_b + h * p.qs_h + (int64_t)qr * p.qs_t + part * PART;
#pragma unroll
    for (int d = 0; d < PART; d += 4) {
      const f32x4_t x = *reinterpret_cast<const f32x4_t*>(src + d);
      q[d] = x[0] * p.scale_log2; q[d + 1] = x[1] * p.scale_log2;
      q[d + 2] = x[2] * p.scale_log2; q[d + 3] = x[3] * p.scale_log2;
    }
  }
  float o[PART];
#pragma unroll
  for (int d = 0; d < PART; ++d) o[d] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const int64_t cap = p.L + p.T;
  const float* kplane = reinterpret_cast<const float*>(p.kv) + (((int64_t)b * p.Hkv + hkv) * cap) * DH;
  const float* vplane = kplane + (int64_t)p.B * p.Hkv * cap * DH;

  for (int vi = 0; vi < nvis; ++vi) {
    const int64_t row0 = (int64_t)vis[vi] * p.T;
    for (int t0 = 0; t0 < p.T; t0 += TK) {
      __syncthreads();  // the previous tile is no longer read
      for (int i = tid; i < TK * DH / 4; i += 256) {
        const int r = i / (DH / 4), c = i % (DH / 4);
        const int tr = t0 + r < p.T ? t0 + r : p.T - 1;  // a short last tile repeats its last row; masked below
        *reinterpret_cast<f32x4_t*>(&ks[r][4 * c]) = *reinterpret_cast<const f32x4_t*>(kplane + (row0 + tr) * DH + 4 * c);
        *reinterpret_cast<f32x4_t*>(&vs[r][4 * c]) = *reinterpret_cast<const f32x4_t*>(vplane + (row0 + tr) * DH + 4 * c);
      }
      __syncthreads();
      float s[TK];
      float mx = m_run;
#pragma unroll
      for (int kk = 0; kk < TK; ++kk) {
        float acc = 0.f;
#pragma unroll
        for (int d = 0; d < PART; ++d) acc += q[d] * ks[kk][part * PART + d];
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
        if (t0 + kk >= p.T) acc = -INFINITY;
        s[kk] = acc;
        mx = fmaxf(mx, acc);
      }
      const float alpha = __builtin_amdgcn_exp2f(m_run - mx);  // 0 on the first tile
      l_run *= alpha;
#pragma unroll
      for (int d = 0; d < PART; ++d) o[d] *= alpha;
#pragma unroll
      for (int kk = 0; kk < TK; ++kk) {
        const float pr = __builtin_amdgcn_exp2f(s[kk] - mx);
        l_run += pr;
#pragma unroll
        for (int d = 0; d < PART; ++d) o[d] += pr * vs[kk][part * PART + d];
      }
      m_run = mx;
    }
  }

  if (qrow < p.T) {
    float inv = 1.f / l_run;
    // fp32: o * inv is the attention output; the gate multiplies that rounded value
    const float g = p.gate != nullptr ? reinterpret_cast<const float*>(p.gate)[b * p.gs_b + h * p.gs_h + (int64_t)qrow * p.gs_t] : 1.f;
    float* dst = reinterpret_cast<float*>(p.out) + b * p.os_b + h * p.os_h + (int64_t)qrow * p.os_t + part * PART;
#pragma unroll
    for (int d = 0; d < PART; d += 4)
      *reinterpret_cast<f32x4_t*>(dst + d) = f32x4_t{(o[d] * inv) * g, (o[d + 1] * inv) * g, (o[d + 2] * inv) * g, (o[d + 3] * inv) * g};
  }
}

hipError_t launch_attn_ring_f32(const AttnParams& p, int Dh, hipStream_t stream) {
  const dim3 grid((unsigned)((p.T + 63) / 64), (unsigned)p.H, (unsigned)p.B);
  if (Dh == 128) hipLaunchKernelGGL(attn_ring_f32_kernel<128>, grid, dim3(256), 0, stream, p);
  else if (Dh == 64) hipLaunchKernelGGL(attn_ring_f32_kernel<64>, grid, dim3(256), 0, stream, p);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace we
