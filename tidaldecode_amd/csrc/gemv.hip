// Matrix-vector products of a batch-1 decode step for gfx950 (MI355X): y = W x with a row-major
// 16-bit W, fp32 accumulation, and the element-wise work around it folded in:
//   x_mode 0  x as given
//   x_mode 1  x = RMSNorm(x) * norm_weight            (the norm before the q/k/v and MLP products)
//   x_mode 2  x = silu(x[:cols]) * x[cols:]           (the gated MLP, before the down projection)
//   residual  y = residual + W x                      (the two residual additions of a layer)
//   pair      y[i] = silu(W[i] x) * (W[i + rows/2] x) (gate and up projection in one launch: a
//             wavefront owns row i and row i + rows/2, so the down projection gets a plain vector)
// HBM-bound: every weight is read once (non-temporal 16-byte loads, 16 of them in flight per
// lane), x is staged in LDS once per workgroup, a wavefront owns two rows at a time and reduces
// with DPP.  Used by the decoder harness around the attention path (the reference runs torch
// nn.Linear there: tidal/models/SparseAttention.py:122,216, tidal/models/llama.py:108-122).

#include "common.cuh"

namespace tidal {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;
constexpr int kGemvMaxCols = 30720; // x in LDS: 60 KiB (covers the 28672-wide MLP of 70B-class models)

struct GemvParams {
  const uint16_t* w;
  int64_t w_row_stride;  // elements
  int32_t rows, cols;
  const uint16_t* x;
  const uint16_t* norm_weight;
  float eps;
  const uint16_t* residual;
  uint16_t* y;
};

__device__ __forceinline__ float wave_sum64(float x) {
  x = group_sum<16>(x);
  x += __shfl_xor(x, 16, 64);
  x += __shfl_xor(x, 32, 64);
  return x;
}

// R rows per wavefront, UN 16-byte chunks per lane and row in flight (R * UN loads per lane),
// XR 16-byte chunks of x per thread (XR * 256 * 8 >= cols)
template <typename T, int MODE, bool PAIR, int R, int UN, int XR>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(
    const uint16_t* a_w, int64_t a_stride, int32_t a_rows, int32_t a_cols, const uint16_t* a_x,
    const uint16_t* a_norm, float a_eps, const uint16_t* a_res, uint16_t* a_y) {
  // Scalar arguments instead of one struct: the compiler flag of this file preloads the first 16
  // argument dwords into SGPRs, so the first weight loads do not wait for a kernel-argument load.
  const GemvParams p{a_w, a_stride, a_rows, a_cols, a_x, a_norm, a_eps, a_res, a_y};
  constexpr int kGemvRows = R, kGemvUnroll = UN;
  // x in LDS, sized by the instantiation (XR * 4 KiB), so that short vectors leave room for more
  // resident workgroups; the gated mode stages through a loop and keeps the full size
  constexpr int kXsWords = MODE == 2 ? kGemvMaxCols / 2 : XR * kGemvThreads * 4;
  __shared__ uint32_t xs[kXsWords];
  __shared__ float red[kGemvWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cols = p.cols;
  const int chunks = cols / 8;

  // ---- rows of this wavefront; the first batch of weight loads is issued before x is staged: the
  // weights do not depend on x, so the staging (and the norm's reduction) hides behind them ------
  const int half = p.rows / 2;
  const int unit = blockIdx.x * kGemvWaves + wave;  // two consecutive rows, or a gate/up row pair
  const int n_units = PAIR ? (half + kGemvRows / 2 - 1) / (kGemvRows / 2) : (p.rows + kGemvRows - 1) / kGemvRows;
  const bool unit_live = unit < n_units;  // a wave without rows still helps staging x
  // PAIR: rows [unit * R/2, +R/2) of the gate block and the same rows of the up block
  constexpr int HR = kGemvRows > 1 ? kGemvRows / 2 : 1;
  int row_of[kGemvRows];
#pragma unroll
  for (int r = 0; r < kGemvRows; ++r)
    row_of[r] = PAIR ? unit * HR + (r % HR) + (r / HR) * half : unit * kGemvRows + r;
  float acc[kGemvRows];
#pragma unroll
  for (int r = 0; r < kGemvRows; ++r) acc[r] = 0.f;
  const u32x4* wrow[kGemvRows];
#pragma unroll
  for (int r = 0; r < kGemvRows; ++r) {
    const int row = row_of[r] < p.rows ? row_of[r] : p.rows - 1;  // a clamped row is computed, not stored
    wrow[r] = reinterpret_cast<const u32x4*>(p.w + (int64_t)row * p.w_row_stride);
  }
  // Program order of the loads matters (the wait counter retires in order): x first, then the
  // weights, so that waiting for x does not wait for the weights.
  u32x4 xr[XR], nr[XR];
  if constexpr (MODE != 2) {
#pragma unroll
    for (int k = 0; k < XR; ++k) {
      const int c = tid + k * kGemvThreads;
      const int cc = c < chunks ? c : chunks - 1;
      xr[k] = reinterpret_cast<const u32x4*>(p.x)[cc];
      if constexpr (MODE == 1) nr[k] = reinterpret_cast<const u32x4*>(p.norm_weight)[cc];
    }
  }
  u32x4 wv[kGemvRows][kGemvUnroll];
  auto load_trip = [&](int c0) {
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const int c = c0 + u * 64 + lane;
      const int cc = c < chunks ? c : chunks - 1;  // unconditional loads; masked in the product
#pragma unroll
      for (int r = 0; r < kGemvRows; ++r) wv[r][u] = __builtin_nontemporal_load(wrow[r] + cc);
    }
  };
  load_trip(0);

  // ---- stage x (and what is folded into it) in LDS, as packed 16-bit pairs ----------------------
  if constexpr (MODE == 0) {
#pragma unroll
    for (int k = 0; k < XR; ++k) {
      const int c = tid + k * kGemvThreads;
      if (c < chunks) reinterpret_cast<u32x4*>(xs)[c] = xr[k];
    }
  } else if constexpr (MODE == 1) {
    // RMSNorm as the model computes it: fp32 statistics, the normalised value rounded to the
    // storage type, then the weight applied in the storage type
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < XR; ++k) {
      if (tid + k * kGemvThreads < chunks) {
        const uint32_t w4[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float a, b;
          unpack2<T>(w4[q], a, b);
          ss = fmaf(a, a, fmaf(b, b, ss));
        }
      }
    }
    ss = wave_sum64(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kGemvWaves; ++w) tot += red[w];
    const float inv = rsqrtf(tot / (float)cols + p.eps);
#pragma unroll
    for (int k = 0; k < XR; ++k) {
      const int c = tid + k * kGemvThreads;
      if (c < chunks) {
        const uint32_t x4[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
        const uint32_t n4[4] = {nr[k].x, nr[k].y, nr[k].z, nr[k].w};
        uint32_t o4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float a, b, wa, wb, na, nb;
          unpack2<T>(x4[q], a, b);
          unpack2<T>(n4[q], wa, wb);
          unpack2<T>(pack2<T>(a * inv, b * inv), na, nb);
          o4[q] = pack2<T>(na * wa, nb * wb);
        }
        reinterpret_cast<u32x4*>(xs)[c] = u32x4{o4[0], o4[1], o4[2], o4[3]};
      }
    }
  } else {
    // gated MLP input: silu(gate) rounded to the storage type, times up, rounded again
    for (int c = tid; c < cols / 2; c += kGemvThreads) {
      float ga, gb, ua, ub;
      unpack2<T>(reinterpret_cast<const uint32_t*>(p.x)[c], ga, gb);
      unpack2<T>(reinterpret_cast<const uint32_t*>(p.x + cols)[c], ua, ub);
      float sa, sb;
      unpack2<T>(pack2<T>(ga / (1.f + __expf(-ga)), gb / (1.f + __expf(-gb))), sa, sb);
      xs[c] = pack2<T>(sa * ua, sb * ub);
    }
  }
  __syncthreads();

  if (!unit_live) return;
  for (int c0 = 0;;) {
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      const int c = c0 + u * 64 + lane;
      const int cc = c < chunks ? c : chunks - 1;
      u32x4 xv = reinterpret_cast<const u32x4*>(xs)[cc];
      if (c >= chunks) xv = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int r = 0; r < kGemvRows; ++r) {
        acc[r] = dot2<T>(wv[r][u].x, xv.x, acc[r]);
        acc[r] = dot2<T>(wv[r][u].y, xv.y, acc[r]);
        acc[r] = dot2<T>(wv[r][u].z, xv.z, acc[r]);
        acc[r] = dot2<T>(wv[r][u].w, xv.w, acc[r]);
      }
    }
    c0 += 64 * kGemvUnroll;
    if (c0 >= chunks) break;
    load_trip(c0);
  }
  float sum[kGemvRows];
#pragma unroll
  for (int r = 0; r < kGemvRows; ++r) sum[r] = wave_sum64(acc[r]);
  if (lane != 0) return;
  if constexpr (PAIR) {
    // as the model does it: both products, silu(gate) and the product each rounded to the storage type
#pragma unroll
    for (int r = 0; r < HR; ++r) {
      if (row_of[r] < half) {
        const float gte = to_float<T>(from_float<T>(sum[r]));
        const float up = to_float<T>(from_float<T>(sum[r + HR]));
        const float act = to_float<T>(from_float<T>(gte / (1.f + __expf(-gte))));
        p.y[row_of[r]] = from_float<T>(act * up);
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r) {
      if (row_of[r] < p.rows) {
        float out = sum[r];
        if (p.residual) out += to_float<T>(p.residual[row_of[r]]);
        p.y[row_of[r]] = from_float<T>(out);
      }
    }
  }
}

template <typename T, int R, int UN, int XR>
static void launch_gemv_x(const GemvParams& p, int mode, bool pair, hipStream_t st) {
  const int units = pair ? (p.rows / 2 + R / 2 - 1) / (R / 2) : (p.rows + R - 1) / R;
  const dim3 grid((units + kGemvWaves - 1) / kGemvWaves), block(kGemvThreads);
  if (pair) {
    if (mode == 0)
      hipLaunchKernelGGL((gemv_kernel<T, 0, true, R, UN, XR>), grid, block, 0, st, p.w, p.w_row_stride, p.rows, p.cols, p.x,
                       p.norm_weight, p.eps, p.residual, p.y);
    else
      hipLaunchKernelGGL((gemv_kernel<T, 1, true, R, UN, XR>), grid, block, 0, st, p.w, p.w_row_stride, p.rows, p.cols, p.x,
                       p.norm_weight, p.eps, p.residual, p.y);
  } else if (mode == 0) {
    hipLaunchKernelGGL((gemv_kernel<T, 0, false, R, UN, XR>), grid, block, 0, st, p.w, p.w_row_stride, p.rows, p.cols, p.x,
                       p.norm_weight, p.eps, p.residual, p.y);
  } else if (mode == 1) {
    hipLaunchKernelGGL((gemv_kernel<T, 1, false, R, UN, XR>), grid, block, 0, st, p.w, p.w_row_stride, p.rows, p.cols, p.x,
                       p.norm_weight, p.eps, p.residual, p.y);
  } else {
    hipLaunchKernelGGL((gemv_kernel<T, 2, false, R, UN, 1>), grid, block, 0, st, p.w, p.w_row_stride, p.rows, p.cols, p.x,
                       p.norm_weight, p.eps, p.residual, p.y);
  }
}

template <typename T, int R, int UN>
static void launch_gemv_shape(const GemvParams& p, int mode, bool pair, hipStream_t st) {
  const int per_thread = (p.cols / 8 + kGemvThreads - 1) / kGemvThreads;  // x chunks per thread
  if (per_thread <= 2)
    launch_gemv_x<T, R, UN, 2>(p, mode, pair, st);
  else if (per_thread <= 6)
    launch_gemv_x<T, R, UN, 6>(p, mode, pair, st);
  else if (per_thread <= 8)
    launch_gemv_x<T, R, UN, 8>(p, mode, pair, st);
  else
    launch_gemv_x<T, R, UN, 15>(p, mode, pair, st);
}

// Tall matrices: four rows per wavefront (fewer, longer-lived waves stream better); short ones:
// two rows, so that the launch still has a few workgroups per compute unit (measured on
// 4096..32000 x 4096 and 4096 x 11008: 4.4-6.0 TB/s).
template <typename T>
static void launch_gemv(const GemvParams& p, int mode, bool pair, hipStream_t st) {
  if (p.rows >= 8192)
    launch_gemv_shape<T, 4, 4>(p, mode, pair, st);
  else if (p.cols > 8192)  // few, long rows (the down projection): deeper batches, 19.0 -> 18.0 us
    launch_gemv_shape<T, 2, 8>(p, mode, pair, st);
  else
    launch_gemv_shape<T, 2, 4>(p, mode, pair, st);
}

}  // namespace tidal

using namespace tidal;

extern "C" int td_gemv(const void* w, int64_t w_row_stride, int32_t rows, int32_t cols,
                       const void* x, int32_t x_mode, const void* norm_weight, float eps,
                       const void* residual, int32_t pair_gated, void* y, int32_t dtype,
                       void* stream) {
  TD_REQUIRE(w && x && y, "td_gemv: NULL argument");
  TD_REQUIRE(rows >= 1 && cols >= 8 && cols % 8 == 0 && cols <= kGemvMaxCols,
             "td_gemv: rows %d, cols %d (cols: multiple of 8, at most %d)", rows, cols, kGemvMaxCols);
  TD_REQUIRE(w_row_stride >= cols && w_row_stride % 8 == 0,
             "td_gemv: row stride %lld (multiple of 8, at least cols)", (long long)w_row_stride);
  TD_REQUIRE(x_mode >= 0 && x_mode <= 2, "td_gemv: x_mode %d", x_mode);
  TD_REQUIRE(x_mode != 1 || norm_weight, "td_gemv: x_mode 1 needs norm_weight");
  TD_REQUIRE(!pair_gated || (rows % 2 == 0 && x_mode != 2 && !residual),
             "td_gemv: pair_gated needs an even row count, x_mode 0 or 1 and no residual");
  TD_REQUIRE((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) % 16 == 0,
             "td_gemv: w and x must be 16-byte aligned");
  GemvParams p;
  p.w = reinterpret_cast<const uint16_t*>(w);
  p.w_row_stride = w_row_stride;
  p.rows = rows;
  p.cols = cols;
  p.x = reinterpret_cast<const uint16_t*>(x);
  p.norm_weight = reinterpret_cast<const uint16_t*>(norm_weight);
  p.eps = eps;
  p.residual = reinterpret_cast<const uint16_t*>(residual);
  p.y = reinterpret_cast<uint16_t*>(y);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == TD_F16)
    launch_gemv<F16>(p, x_mode, pair_gated != 0, st);
  else if (dtype == TD_BF16)
    launch_gemv<BF16>(p, x_mode, pair_gated != 0, st);
  else
    return fail(TD_ERR_UNSUPPORTED, "td_gemv failed to dispatch with dtype %d", dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
