// Shared device/host helpers for the gfx950 kernels of libtidal_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/tidal_hip.h"

namespace tidal {

// ---------------------------------------------------------------------------------------------
// Error reporting (host)
// ---------------------------------------------------------------------------------------------
char* error_buffer();  // thread-local, 512 bytes, defined in capi.hip

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define TD_REQUIRE(cond, ...)                                         \
  do {                                                                \
    if (!(cond)) return ::tidal::fail(TD_ERR_INVALID_ARG, __VA_ARGS__); \
  } while (0)

#define TD_HIP_CHECK(expr)                                                                   \
  do {                                                                                       \
    hipError_t e_ = (expr);                                                                  \
    if (e_ != hipSuccess)                                                                    \
      return ::tidal::fail(TD_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));       \
  } while (0)

// ---------------------------------------------------------------------------------------------
// Vector types: one lane moves 16 bytes (8 two-byte elements) per global access.
// ---------------------------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct F16 {};   // tag types for the two KV element formats
struct BF16 {};

// dot of two packed pairs, fp32 accumulate (v_dot2_f32_f16 / v_dot2_f32_bf16)
template <typename T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c,
                                false);
}
template <>
__device__ __forceinline__ float dot2<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a),
                                         __builtin_bit_cast(bf16x2, b), c, false);
}

// unpack a packed pair to two floats
template <typename T>
__device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi);
template <>
__device__ __forceinline__ void unpack2<F16>(uint32_t w, float& lo, float& hi) {
  f16x2 h = __builtin_bit_cast(f16x2, w);
  lo = (float)h.x;
  hi = (float)h.y;
}
template <>
__device__ __forceinline__ void unpack2<BF16>(uint32_t w, float& lo, float& hi) {
  lo = __builtin_bit_cast(float, w << 16);
  hi = __builtin_bit_cast(float, w & 0xffff0000u);
}

// round-to-nearest-even pack of two floats
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<F16>(float lo, float hi) {
  f16x2 h;
  h.x = (_Float16)lo;
  h.y = (_Float16)hi;
  return __builtin_bit_cast(uint32_t, h);
}
// gfx950 converts in hardware (v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN)
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <>
__device__ __forceinline__ uint32_t pack2<BF16>(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

// scalar conversions (used by the small kernels)
template <typename T>
__device__ __forceinline__ float to_float(uint16_t b);
template <>
__device__ __forceinline__ float to_float<F16>(uint16_t b) {
  return (float)__builtin_bit_cast(_Float16, b);
}
template <>
__device__ __forceinline__ float to_float<BF16>(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
template <typename T>
__device__ __forceinline__ uint16_t from_float(float f);
template <>
__device__ __forceinline__ uint16_t from_float<F16>(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
template <>
__device__ __forceinline__ uint16_t from_float<BF16>(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

// Maximum / sum over the four 16-lane rows of a wavefront (lanes l, l ^ 16, l ^ 32, l ^ 48), result
// in every lane.  gfx950's v_permlane16_swap / v_permlane32_swap exchange rows between two
// registers in the vector pipeline: given the same value twice, the first result holds the even
// row (lower half) of each pair in both of its rows (halves), the second result the odd row
// (upper half).
// The instruction swaps in place between two different registers; the copy below is made opaque
// so that the two operands are never allocated to one register (a swap of a register with itself
// exchanges nothing).
typedef unsigned int u32pair __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t opaque_copy(uint32_t u) {
  uint32_t c = u;
  asm volatile("" : "+v"(c));
  return c;
}
__device__ __forceinline__ void swap_rows16(float v, float& even, float& odd) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const u32pair a = __builtin_amdgcn_permlane16_swap(u, opaque_copy(u), false, false);
  const uint32_t lo = a.x, hi = a.y;  // elements are copied out before the bit cast
  even = __builtin_bit_cast(float, lo);
  odd = __builtin_bit_cast(float, hi);
}
__device__ __forceinline__ void swap_halves32(float v, float& lower, float& upper) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const u32pair a = __builtin_amdgcn_permlane32_swap(u, opaque_copy(u), false, false);
  const uint32_t lo = a.x, hi = a.y;
  lower = __builtin_bit_cast(float, lo);
  upper = __builtin_bit_cast(float, hi);
}
__device__ __forceinline__ float rows_max(float v) {
  float a, b;
  swap_rows16(v, a, b);
  swap_halves32(fmaxf(a, b), a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float rows_sum(float v) {
  float a, b;
  swap_rows16(v, a, b);
  swap_halves32(a + b, a, b);
  return a + b;
}

// ---------------------------------------------------------------------------------------------
// Cross-lane sums inside a group of W adjacent lanes (W = 8, 16 or 32) of a 64-wide wavefront,
// result in every lane of the group.  DPP modifiers fold into the v_add_f32.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

template <int W>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(W == 8 || W == 16 || W == 32, "lane group width");
  x += dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]
  x += dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]
  x += dpp_move<0x141>(x);  // row_half_mirror: other quad of the 8-lane half row
  if constexpr (W >= 16) x += dpp_move<0x140>(x);  // row_mirror: other half of the 16-lane row
  if constexpr (W >= 32) {
    // xor 16 inside each 32-lane half: ds_swizzle bit-mask mode, and=0x1f or=0 xor=0x10
    x += __builtin_bit_cast(
        float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), (0x10 << 10) | 0x1f));
  }
  return x;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// ---- pieces of the shared-KV-row (grouped-query) path ------------------------------------------
// exchange with the lane whose index differs in one bit (inside a 16-lane DPP row)
template <int MASK>
__device__ __forceinline__ float lane_xor16(float x) {
  static_assert(MASK == 1 || MASK == 2 || MASK == 4, "one of the low three bits");
  if constexpr (MASK == 1) return dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]
  if constexpr (MASK == 2) return dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]
  // row_half_mirror gives lane i ^ 7, quad_perm [3,2,1,0] then gives (i ^ 7) ^ 3 = i ^ 4
  return dpp_move<0x1B>(dpp_move<0x141>(x));
}

// a[j] holds this lane's partial sum for query head j (Q heads, Q = 2, 4 or 8).  Returns the
// sum over the 16 lanes of the row for head (lane % Q): the first log2(Q) butterfly steps halve
// the set of heads a lane keeps while exchanging the other half (reduce-scatter), the remaining
// steps are plain sums among lanes that hold the same head.
template <int Q>
__device__ __forceinline__ float reduce_scatter16(float (&a)[Q], int li) {
  static_assert(Q == 2 || Q == 4 || Q == 8, "query heads per shared row");
  float cur[Q];
#pragma unroll
  for (int j = 0; j < Q; ++j) cur[j] = a[j];
  if constexpr (Q >= 2) {
    const bool hi = li & 1;
#pragma unroll
    for (int i = 0; i < Q / 2; ++i) {
      const float keep = hi ? cur[2 * i + 1] : cur[2 * i];
      const float send = hi ? cur[2 * i] : cur[2 * i + 1];
      cur[i] = keep + lane_xor16<1>(send);
    }
  }
  if constexpr (Q >= 4) {
    const bool hi = li & 2;
#pragma unroll
    for (int i = 0; i < Q / 4; ++i) {
      const float keep = hi ? cur[2 * i + 1] : cur[2 * i];
      const float send = hi ? cur[2 * i] : cur[2 * i + 1];
      cur[i] = keep + lane_xor16<2>(send);
    }
  } else {
    cur[0] += lane_xor16<2>(cur[0]);
  }
  if constexpr (Q >= 8) {
    const bool hi = li & 4;
    const float keep = hi ? cur[1] : cur[0];
    const float send = hi ? cur[0] : cur[1];
    cur[0] = keep + lane_xor16<4>(send);
  } else {
    cur[0] += dpp_move<0x124>(cur[0]);  // row_ror:4 (sums need no exact partner, only the class)
  }
  cur[0] += dpp_move<0x128>(cur[0]);    // row_ror:8
  return cur[0];
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));

// D(16x16, fp32) += A(16x16) * B(16x16) with 16-bit operands: a lane holds A[lane % 16][4g .. 4g+3]
// and B[4g .. 4g+3][lane % 16] (g = lane / 16) as two packed dwords, and D[4g + i][lane % 16].
template <typename T>
__device__ __forceinline__ f32x4 mfma_16x16x16(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1,
                                               f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma_16x16x16<BF16>(uint32_t a0, uint32_t a1, uint32_t b0,
                                                     uint32_t b1, f32x4 c) {
  const u32x2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                   __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma_16x16x16<F16>(uint32_t a0, uint32_t a1, uint32_t b0,
                                                    uint32_t b1, f32x4 c) {
  const u32x2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h16x4, a),
                                               __builtin_bit_cast(h16x4, b), c, 0, 0, 0);
}

// gfx950: D(16x16, fp32) += A(16x32) * B(32x16); a lane holds A[lane % 16][8g .. 8g+7] and
// B[8g .. 8g+7][lane % 16] (g = lane / 16) as four packed dwords.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
template <typename T>
__device__ __forceinline__ f32x4 mfma_16x16x32(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma_16x16x32<BF16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma_16x16x32<F16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

constexpr float kNegBig = -1.0e30f;  // finite stand-in for -inf in running maxima

__host__ __device__ __forceinline__ int64_t ceil_div64(int64_t a, int64_t b) {
  return (a + b - 1) / b;
}

}  // namespace tidal
