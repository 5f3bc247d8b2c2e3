// Sparse-layer decode-attention kernel instantiations for F16 K/V (see sparse_attn.cuh).
#include "sparse_attn.cuh"

namespace tidal {
int launch_sparse_f16(const DecodeParams& p, int nw, int rows, bool probe, bool wide, bool merge_kernel,
                      dim3 grid, hipStream_t st) {
  const int rc = launch_sparse<F16>(p, nw, rows, probe, wide, grid, st);
  if (rc == TD_OK && merge_kernel && !probe)
    hipLaunchKernelGGL((merge_partials_kernel<F16, 128, 1, 512>), dim3(grid.x, grid.y), dim3(512), 0, st, p);
  return rc;
}
}  // namespace tidal
