// Merged q/k/v projection of one frame with RoPE + ring-slot K/V store as its epilogue (gfx950).
//
// One launch replaces the module's qkv_proj GEMM (src/patch_model.py:116-122) and everything the
// store kernel does after it (src/model/attn.py:105-110, src/model/kv_cache.py:138,147-151,192):
// the projected rows never travel through HBM as a [B, T, (H + 2 Hkv) Dh] tensor.  Meant for
// frames of a few hundred tokens, where the projection is a skinny GEMM (tokens x features x
// d_model = 256 x 6144 x 2048) whose cost is streaming the weight matrix once.
//
// One workgroup = 8 wavefronts = one CU computes a 64-token x 128-feature tile of x W^T, i.e. one
// head of 64 tokens (two heads when Dh = 64).  x and W tiles of 128 contraction elements travel
// HBM/L2 -> LDS by DMA (global_load_lds_dwordx4) into a ring of 3 slots, two ahead; rows are 256
// bytes, 16-byte chunks XOR-swizzled with (row & 15) on the global side of the DMA.  Wavefront w
// takes feature half (w & 1) and the contraction steps (w >> 1) and (w >> 1) + 4 of every slot:
// per slot 8 fragment reads (ds_read_b128) feed 8 v_mfma_f32_32x32x16 (A = W rows, B = x rows, so
// a lane owns one token and registers run along features).  The four partial sums of a tile are
// added through LDS in a fixed order, rounded to the element type as the GEMM's output tensor
// would be, and laid out as a [64][128] tile in LDS; then every thread takes one 16-element item
// exactly like a thread of the store kernel (same functions, same bits): RMS norm, rotation,
// value blend, tail / ring-slot rows, `written`.  cos / sin values, position ids and the value
// residual of a thread's item are requested before the main loop.
//
// The grid is 1-D: workgroup id % 8 is the XCD, and the token tiles of one feature tile follow
// each other on one XCD, so a weight slab is fetched from HBM once and re-read from that L2.
// Roofline: the weight matrix once (2 K N bytes) + x once; 2 T N K flops.
#include "attn_mma.h"
#include "rope_kv_store.h"
#include "device_state.h"
#include "we_kernels.h"

namespace we {

namespace {
constexpr int PM = 64;                       // tokens per tile
constexpr int PN = 128;                      // features per tile
constexpr int PK = 128;                      // contraction elements per ring slot
constexpr int P_ROW_B = PK * 2;              // bytes per tile row
constexpr int X_TILE_B = PM * P_ROW_B;       // 16 KB
constexpr int W_TILE_B = PN * P_ROW_B;       // 32 KB
constexpr int SLOT_B = X_TILE_B + W_TILE_B;  // 48 KB
constexpr int NSLOT = 3;
constexpr int BLK_B = 32 * 32 * 4;           // one 32 x 32 fp32 block of partial sums
constexpr int OUT_OFF = 2 * 4 * 4 * BLK_B;   // the element-type output tile sits behind the exchange area
constexpr int PROJ_LDS_B = NSLOT * SLOT_B;
static_assert(OUT_OFF + PM * PN * 2 <= PROJ_LDS_B, "exchange area and output tile reuse the ring");
}  // namespace

template <typename M, typename Tag>
__global__ void __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2)))
qkv_rope_store_kernel(ProjParams p) {
  typedef typename M::frag_t frag_t;
  typedef typename Tag::store_t st_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  const StoreParams& s = p.s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  const int nh = wave & 1;     // feature half of the tile
  const int kg = wave >> 1;    // contraction group

  // ---- which tile ----
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int mt_all = p.m_tiles * s.B;
  const int ng = j / mt_all;
  const int mi = j - ng * mt_all;
  const int nt = ng * 8 + xcd;
  if (nt >= p.n_tiles) return;
  const int b = mi / p.m_tiles;
  const int m0 = (mi - b * p.m_tiles) * PM;
  const int n0 = nt * PN;

  // ---- this thread's item of the epilogue: 16 features of one token ----
  const int e_row = tid >> 3;
  const int e_t = m0 + e_row;
  const bool e_live = e_t < s.T;
  const int e_tc = e_live ? e_t : s.T - 1;
  const int f0 = n0 + (tid & 7) * 16;
  const int q_feats = s.H * s.Dh, k_end = q_feats + s.Hkv * s.Dh;
  const int which = f0 < q_feats ? 0 : (f0 < k_end ? 1 : 2);
  const int f_in = f0 - (which == 0 ? 0 : (which == 1 ? q_feats : k_end));
  const int dh_shift = s.Dh == 128 ? 7 : 6;
  const int e_h = f_in >> dh_shift;
  const int e_chunk = (f_in & (s.Dh - 1)) >> 4;
  const int64_t frame_t = s.t_pos[0];

  // ---- DMA plumbing: instruction q of a tile moves its rows 4q .. 4q+3 ----
  uint32_t xvo[2], wvo[4];
  {
    const int phys = lane & 15;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 4 * (wave + 8 * i) + (lane >> 4);
      int tok = m0 + row;
      tok = tok < s.T ? tok : s.T - 1;  // rows past the frame repeat its last token; never stored
      xvo[i] = (uint32_t)tok * (uint32_t)(p.xs_t * 2) + (uint32_t)((phys ^ (row & 15)) << 4);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * (wave + 8 * i) + (lane >> 4);
      wvo[i] = (uint32_t)row * (uint32_t)(p.ws_n * 2) + (uint32_t)((phys ^ (row & 15)) << 4);
    }
  }
  const uint64_t xbase = uniform64((uint64_t)(uintptr_t)p.x + (uint64_t)((int64_t)b * p.xs_b * 2));
  const uint64_t wbase = uniform64((uint64_t)(uintptr_t)p.w + (uint64_t)((int64_t)n0 * p.ws_n * 2));
  const uint32_t wave_lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + wave * 1024));
  auto dma_slot = [&](int c, int slot) __attribute__((always_inline)) {
    const uint64_t kb = (uint64_t)c * P_ROW_B;
#pragma unroll
    for (int i = 0; i < 2; ++i) dma16(xbase + kb, xvo[i], wave_lds + slot * SLOT_B + i * 8 * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(wbase + kb, wvo[i], wave_lds + slot * SLOT_B + X_TILE_B + i * 8 * 1024);
  };
  constexpr int NDMA = 6;  // DMA instructions per wavefront and slot

  const int nc = p.K / PK;
  // Contraction chunks are taken in groups of G, and within a group token tile i starts at chunk
  // i mod G: the tiles that share a weight slab then ask for different lines at any one time, each
  // line comes from HBM at one tile's request and is an L2 hit for the others a slot or two later.
  // (A CU streams from HBM at less than half the rate it reads L2 at, so tiles asking for the same
  // lines together move the slab at a fraction of what they could.  Groups longer than 8 slots
  // keep more of the slab alive in L2 than pays.)
  const int G = mt_all >= 8 ? 8 : (mt_all >= 4 ? 4 : (mt_all >= 2 ? 2 : 1));
  const int rot = mi & (G - 1), ncg = nc & ~(G - 1);
  auto chunk = [&](int c) __attribute__((always_inline)) { return c < ncg ? (c & ~(G - 1)) | ((c + rot) & (G - 1)) : c; };
  dma_slot(chunk(0), 0);
  if (nc > 1) dma_slot(chunk(1), 1);

  // ---- what the item needs besides the projection: requested now, used after the loop ----
  ItemSide<Tag> side;
  load_item_side<Tag>(s, which, b, e_h, e_tc, e_chunk, side);

  // ---- fragment read addresses: row l32 of a 32-row block, logical chunk 2 * step + hh ----
  uint32_t a_rd[2], b_rd[2];
#pragma unroll
  for (int h2 = 0; h2 < 2; ++h2) {
    const int phys = (2 * (kg + 4 * h2) + hh) ^ (l32 & 15);
    b_rd[h2] = (uint32_t)(l32 * P_ROW_B + phys * 16);
    a_rd[h2] = (uint32_t)(X_TILE_B + (nh * 64 + l32) * P_ROW_B + phys * 16);
  }

  f32x16_t acc[2][2];  // [feature block][token block]
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][mb][i] = 0.f;

  // ---- main loop: one barrier per slot ----
  uint32_t slot_off = 0;   // byte offset of the slot being consumed
  int fill = 2 % NSLOT;    // slot the next DMA goes to
  for (int c = 0; c < nc; ++c) {
    if (c + 1 < nc) dma_wait<NDMA>(); else dma_wait<0>();  // this wavefront's part of slot c has landed
    // every wavefront's part has landed, and everybody is done with the slot refilled next
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (c + 2 < nc) dma_slot(chunk(c + 2), fill);
    fill = fill + 1 == NSLOT ? 0 : fill + 1;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const unsigned char* ab = smem + slot_off + a_rd[h2];
      const unsigned char* bb = smem + slot_off + b_rd[h2];
      const frag_t a0 = *reinterpret_cast<const frag_t*>(ab);
      const frag_t a1 = *reinterpret_cast<const frag_t*>(ab + 32 * P_ROW_B);
      const frag_t b0 = *reinterpret_cast<const frag_t*>(bb);
      const frag_t b1 = *reinterpret_cast<const frag_t*>(bb + 32 * P_ROW_B);
      acc[0][0] = M::mma(a0, b0, acc[0][0]);
      acc[0][1] = M::mma(a0, b1, acc[0][1]);
      acc[1][0] = M::mma(a1, b0, acc[1][0]);
      acc[1][1] = M::mma(a1, b1, acc[1][1]);
    }
    slot_off = slot_off + SLOT_B == (uint32_t)PROJ_LDS_B ? 0u : slot_off + SLOT_B;
  }

  // ---- the four contraction groups add their partial sums through LDS ----
  // Block (nb, mb) of feature half nh belongs to the wavefront with kg == 2 * nb + mb.  Vector g
  // of lane l of the block that group k hands to that owner sits at
  // ((((nh * 4 + k) * 4 + block) * 4 + g) * 64 + l) * 16.
  __syncthreads();  // everybody is done with the ring
  f32x4_t* xch = reinterpret_cast<f32x4_t*>(smem);
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int blk = 2 * nb + mb;
      if (blk != kg) {
        f32x4_t* dst = xch + (((nh * 4 + kg) * 4 + blk) * 4) * 64 + lane;
#pragma unroll
        for (int g = 0; g < 4; ++g)
          dst[g * 64] = f32x4_t{acc[nb][mb][4 * g], acc[nb][mb][4 * g + 1], acc[nb][mb][4 * g + 2], acc[nb][mb][4 * g + 3]};
      }
    }
  __syncthreads();
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int blk = 2 * nb + mb;
      if (blk == kg) {
        // sum in the order of the contraction groups, whoever the owner is
        f32x16_t r;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          f32x16_t part;
          if (k == kg) {
            part = acc[nb][mb];
          } else {
            const f32x4_t* src = xch + (((nh * 4 + k) * 4 + blk) * 4) * 64 + lane;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              const f32x4_t v = src[g * 64];
              part[4 * g] = v[0]; part[4 * g + 1] = v[1]; part[4 * g + 2] = v[2]; part[4 * g + 3] = v[3];
            }
          }
          if (k == 0) r = part;
          else
#pragma unroll
            for (int i = 0; i < 16; ++i) r[i] += part[i];
        }
        // register 4 g + e of a lane is feature 8 g + 4 hh + e of the block, for token l32
        unsigned char* orow = smem + OUT_OFF + (mb * 32 + l32) * (PN * 2) + (nh * 64 + nb * 32 + 4 * hh) * 2;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint16_t e4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) e4[e] = Tag::from_f32(r[4 * g + e]);
          u32x2_t pk;
          pk[0] = (uint32_t)e4[0] | ((uint32_t)e4[1] << 16);
          pk[1] = (uint32_t)e4[2] | ((uint32_t)e4[3] << 16);
          *reinterpret_cast<u32x2_t*>(orow + g * 16) = pk;
        }
      }
    }
  __syncthreads();

  // ---- epilogue: the store kernel's work on this thread's item ----
  if (!e_live) return;
  Chunk16<Tag> in;
  {
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(smem + OUT_OFF + e_row * (PN * 2) + (tid & 7) * 32);
    u32x4_t* dst = reinterpret_cast<u32x4_t*>(in.e);
    dst[0] = src[0];
    dst[1] = src[1];
  }
  if (which == 0) {
    finish_q_chunk<Tag>(s, b, e_h, e_t, e_chunk, in, side.rotate, side.c, side.s);
  } else {
    if (which == 2 && p.v_out != nullptr)
      store16<Tag>((st_t*)p.v_out + b * p.vo_b + e_h * p.vo_h + e_t * p.vo_t + e_chunk * 16, in);
    const SlotInfo si = ring_slot(frame_t, s.dilation, s.num_buckets);
    finish_kv_chunk<Tag>(s, which, b, e_h, e_t, e_chunk, si, in, side.rotate, side.c, side.s, side.res, side.lamb);
  }
}

template <typename M, typename Tag>
static hipError_t launch_proj(const ProjParams& p, hipStream_t stream) {
  const unsigned groups = (unsigned)((p.n_tiles + 7) / 8);
  const dim3 grid(8u * groups * (unsigned)(p.m_tiles * p.s.B));
  hipLaunchKernelGGL((qkv_rope_store_kernel<M, Tag>), grid, dim3(512), PROJ_LDS_B, stream, p);
  return hipGetLastError();
}

hipError_t launch_qkv_rope_store(const ProjParams& p, int dtype, hipStream_t stream) {
  if (dtype == 0) return launch_proj<Bf16Mma, Bf16Tag>(p, stream);
  return launch_proj<F16Mma, F16Tag>(p, stream);
}

// The kernel's LDS ring exceeds the default per-launch limit: raised once per device by the
// library's set-up (device_state.hip).
hipError_t configure_qkv_rope_store() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&qkv_rope_store_kernel<Bf16Mma, Bf16Tag>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, PROJ_LDS_B);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&qkv_rope_store_kernel<F16Mma, F16Tag>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, PROJ_LDS_B);
  return e;
}

}  // namespace we
