// Second pass of split-context attention over the KV ring buffer (gfx950): merges the per-split
// partial results the main kernel (attn_ring.hip) leaves in the workspace.
// HBM-bound: reads n_splits * (Dh * 2 + 16) bytes and writes Dh * 2 bytes per query row that was
// split.
#include "attn_merge.h"
#include "../../include/we_attn.h"

namespace we {

// Second pass of the split-context path.  One thread per (row, 8 columns);
// grid = (256-thread slices of one head's T * DH/8 items, split (batch, head) pairs), so that the
// start-up code has one 32-bit division in it (the kernel is short enough for that to show).
template <typename M, int DH>
__global__ void __launch_bounds__(256) attn_combine_kernel(AttnParams p) {
  const int64_t rows = (int64_t)p.B * p.H * p.T - p.ws_row0;  // rows that were split
  const int item = blockIdx.x * 256 + threadIdx.x;
  if (item >= p.T * (DH / 8)) return;
  const int t = item / (DH / 8), dg = item % (DH / 8);
  const int64_t row = (int64_t)blockIdx.y * p.T + t;  // workspace row; query row = row + ws_row0
  const unsigned bh = (unsigned)(p.units_whole * p.group) + blockIdx.y;  // first split pair + y
  const int b = (int)(bh / (unsigned)p.H), h = (int)(bh % (unsigned)p.H);
  merge_item<M>(p, row * 16, (row * DH + dg * 8) * 2, rows * 16, rows * DH * 2, b, h, t, dg);
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
