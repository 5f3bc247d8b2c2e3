// Sparse-layer decode-attention kernel instantiations for BF16 K/V (see sparse_attn.cuh).
#include "sparse_attn.cuh"

namespace tidal {
int launch_sparse_bf16(const DecodeParams& p, int nw, int rows, bool probe, bool wide, bool merge_kernel,
                      dim3 grid, hipStream_t st) {
  const int rc = launch_sparse<BF16>(p, nw, rows, probe, wide, grid, st);
  if (rc == TD_OK && merge_kernel && !probe)
    hipLaunchKernelGGL((merge_partials_kernel<BF16, 128, 1, 512>), dim3(grid.x, grid.y), dim3(512), 0, st, p);
  return rc;
}
}  // namespace tidal
