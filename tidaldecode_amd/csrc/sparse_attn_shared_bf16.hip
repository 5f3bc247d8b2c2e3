// Sparse-layer decode-attention kernel with shared KV rows (2, 4 or 8 query heads per list walk),
// instantiations for BF16 K/V (see sparse_attn.cuh).
#include "sparse_attn.cuh"

namespace tidal {
int launch_sparse_shared_bf16(const DecodeParams& p, int nw, int qpg, bool wide, bool merge_kernel, dim3 grid,
                             hipStream_t st) {
  const int rc = launch_sparse_shared<BF16>(p, nw, qpg, wide, grid, st);
  if (rc == TD_OK && merge_kernel) {
    const dim3 mg(grid.x, grid.y);
    if (qpg == 2) hipLaunchKernelGGL((merge_partials_kernel<BF16, 128, 2, 512>), mg, dim3(512), 0, st, p);
    if (qpg == 4) hipLaunchKernelGGL((merge_partials_kernel<BF16, 128, 4, 512>), mg, dim3(512), 0, st, p);
    if (qpg == 8) hipLaunchKernelGGL((merge_partials_kernel<BF16, 128, 8, 512>), mg, dim3(512), 0, st, p);
  }
  return rc;
}
}  // namespace tidal
