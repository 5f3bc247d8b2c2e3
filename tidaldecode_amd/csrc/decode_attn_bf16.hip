// Decode-attention kernel instantiations for BF16 K/V (see decode_attn.cuh).
#include "decode_attn.cuh"

namespace tidal {
int launch_decode_bf16(const DecodeParams& p, int head_dim, int qpg, int nw, int rows, bool page_mode,
                      bool emit, bool merge_kernel, dim3 grid, hipStream_t st) {
  return launch_shape<BF16>(p, head_dim, qpg, nw, rows, page_mode, emit, merge_kernel, grid, st);
}
}  // namespace tidal
