// Measurement aid: what the memory system delivers for the access pattern of the ring attention
// kernel at 256-token frames, with the arithmetic taken away (gfx950).
//
// Every workgroup (8 wavefronts, one CU) streams `tiles` 16-KB tiles of one contiguous region into a
// ring of four LDS slots by DMA, exactly as the attention kernel fetches K and V tiles - three tiles
// in flight, one barrier per tile - and does nothing with them.  `share` consecutive workgroups of
// an XCD walk the same region, as the query tiles / grouped heads of one K/V stream do.  The time
// of a launch is what a kernel of this shape cannot go below however little it computes.
#include "attn_mma.h"
#include "we_kernels.h"

namespace we {

namespace {
constexpr int PROBE_TILE_B = 16384;
constexpr int PROBE_SLOTS = 4;
}  // namespace

__global__ void __launch_bounds__(512) stream_probe_kernel(const unsigned char* src, int tiles, int share) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroup id % 8 is the XCD; the sharers of a region follow each other on one XCD
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const uint64_t base = uniform64((uint64_t)(uintptr_t)src +
                                  (uint64_t)((j / share) * 8 + xcd) * (uint64_t)tiles * (uint64_t)PROBE_TILE_B);
  const uint32_t wave_lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + wave * 1024));
  const uint32_t vo = (uint32_t)(wave * 1024 + lane * 16);
  auto issue = [&](int t) __attribute__((always_inline)) {
    const uint32_t slot = (uint32_t)(t % PROBE_SLOTS) * PROBE_TILE_B;
    dma16(base, (uint32_t)t * PROBE_TILE_B + vo, wave_lds + slot);
    dma16(base, (uint32_t)t * PROBE_TILE_B + vo + 8192u, wave_lds + slot + 8192u);
  };
  for (int t = 0; t < PROBE_SLOTS - 1 && t < tiles; ++t) issue(t);
  for (int t = 0; t < tiles; ++t) {
    if (t + PROBE_SLOTS - 1 < tiles) {
      issue(t + PROBE_SLOTS - 1);
      dma_wait<2 * (PROBE_SLOTS - 1)>();
    } else {
      dma_wait<0>();
    }
    __builtin_amdgcn_s_barrier();
  }
}

hipError_t launch_stream_probe(const void* src, int workgroups, int tiles, int share, hipStream_t stream) {
  hipLaunchKernelGGL(stream_probe_kernel, dim3((unsigned)workgroups), dim3(512), PROBE_SLOTS * PROBE_TILE_B, stream,
                     static_cast<const unsigned char*>(src), tiles, share);
  return hipGetLastError();
}

}  // namespace we
