// Row-wise top-k selection and the cross-head score reduction for gfx950 (MI355X).
//
// One 1024-thread workgroup (16 wavefronts) per row (rows of up to 65536 elements are held in
// registers, longer ones are re-read from L2 per pass) runs an MSB-first radix select over
// order-preserving integer keys with LDS histograms (11/11/10-bit digits for fp32 keys, 8/8 for
// fp16/bf16 keys), which yields the exact k-th largest key T and the number r of elements equal
// to T that still fit.  A final ordered pass emits every element above T plus the first r
// elements equal to T, so ties go to the lower position and the output is sorted by position:
// the result is a pure function of the input row.
//
// Replaces decode_select_k (kernels/include/topk/decode_select_k.cuh:25-62 of the reference),
// which launches RAFT's radix_topk_one_block_kernel, one 512-thread block per head.

#include "common.cuh"

namespace tidal {

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / 64;
constexpr int kMaxBins = 2048;

struct TopkParams {
  const void* values;
  int64_t values_stride;
  int32_t len;
  int32_t k;
  const int32_t* in_idx;
  int64_t in_idx_stride;
  const int32_t* page_table;
  int32_t page_size;
  void* out_values;
  int32_t* out_idx;
  int64_t out_stride;
};

struct F32 {};

// Order-preserving keys: larger value <=> larger unsigned key.  -0 is folded onto +0 and every
// NaN onto the maximum key so that equal values have equal keys.
template <typename T>
struct KeyTraits;
template <>
struct KeyTraits<F32> {
  typedef uint32_t key_t;
  typedef float elem_t;
  static constexpr int kBits = 32;
  static constexpr int kPasses = 3;
  __device__ static constexpr int digit_bits(int pass) { return pass < 2 ? 11 : 10; }
  __device__ static key_t key(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) == 0u) u = 0u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  }
};
template <>
struct KeyTraits<F16> {
  typedef uint32_t key_t;
  typedef uint16_t elem_t;
  static constexpr int kBits = 16;
  static constexpr int kPasses = 2;
  __device__ static constexpr int digit_bits(int) { return 8; }
  __device__ static key_t key(uint16_t h) {
    uint32_t u = h;
    if ((u & 0x7fffu) == 0u) u = 0u;
    if ((u & 0x7fffu) > 0x7c00u) return 0xffffu;
    return (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
  }
};
template <>
struct KeyTraits<BF16> {
  typedef uint32_t key_t;
  typedef uint16_t elem_t;
  static constexpr int kBits = 16;
  static constexpr int kPasses = 2;
  __device__ static constexpr int digit_bits(int) { return 8; }
  __device__ static key_t key(uint16_t h) {
    uint32_t u = h;
    if ((u & 0x7fffu) == 0u) u = 0u;
    if ((u & 0x7fffu) > 0x7f80u) return 0xffffu;
    return (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
  }
};

// inclusive suffix sum inside a wavefront: lane i gets the sum over lanes >= i
__device__ __forceinline__ uint32_t wave_suffix_sum(uint32_t x, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    uint32_t y = __shfl_down(x, off, 64);
    if (lane + off < 64) x += y;
  }
  return x;
}

template <typename T>
__global__ __launch_bounds__(kTopkThreads) void topk_kernel(const TopkParams p) {
  typedef KeyTraits<T> KT;
  typedef typename KT::elem_t elem_t;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int len = p.len;
  const int k = p.k;  // 1 <= k <= len (host-checked)
  const elem_t* vals = reinterpret_cast<const elem_t*>(p.values) + (int64_t)row * p.values_stride;

  __shared__ uint32_t hist[kMaxBins];
  __shared__ uint32_t wave_tot[kTopkWaves];
  __shared__ uint32_t sh_bin, sh_krem;
  __shared__ uint32_t seg_gt[kTopkWaves], seg_eq[kTopkWaves];

  uint32_t prefix = 0, mask = 0, krem = (uint32_t)k;
  int shift = KT::kBits;
#pragma unroll
  for (int pass = 0; pass < KT::kPasses; ++pass) {
    const int bits = KT::digit_bits(pass);
    const int nb = 1 << bits;
    shift -= bits;
    for (int i = tid; i < nb; i += kTopkThreads) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < len; i += kTopkThreads) {
      const uint32_t key = KT::key(vals[i]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & (nb - 1)], 1u);
    }
    __syncthreads();
    // locate the digit whose bin holds the krem-th largest remaining key
    const int bpt = nb >= kTopkThreads ? nb / kTopkThreads : 1;  // bins per thread
    const int my_bin = tid * bpt;
    uint32_t local = 0;
    if (my_bin < nb)
      for (int j = 0; j < bpt; ++j) local += hist[my_bin + j];
    const uint32_t suf = wave_suffix_sum(local, lane);
    if (lane == 0) wave_tot[wave] = suf;
    __syncthreads();
    uint32_t above = suf - local;  // keys in bins above this thread's bins
    for (int w = wave + 1; w < kTopkWaves; ++w) above += wave_tot[w];
    if (my_bin < nb) {
      for (int j = bpt - 1; j >= 0; --j) {
        const uint32_t c = hist[my_bin + j];
        if (above < krem && krem <= above + c) {
          sh_bin = (uint32_t)(my_bin + j);
          sh_krem = krem - above;
        }
        above += c;
      }
    }
    __syncthreads();
    prefix |= sh_bin << shift;
    mask |= (uint32_t)(nb - 1) << shift;
    krem = sh_krem;
    __syncthreads();
  }
  const uint32_t thr = prefix;  // the k-th largest key
  const uint32_t r = krem;      // elements equal to thr that are selected (lowest positions)

  // ordered emission: each wave owns a contiguous segment of the row
  int seg = (len + kTopkWaves - 1) / kTopkWaves;
  seg = (seg + 63) & ~63;
  const int s0 = wave * seg;
  int s1 = s0 + seg;
  s1 = s1 > len ? len : s1;
  uint32_t n_gt = 0, n_eq = 0;
  for (int base = s0; base < s1; base += 64) {
    const int i = base + lane;
    uint32_t key = 0;
    const bool in = i < s1;
    if (in) key = KT::key(vals[i]);
    n_gt += __popcll(__ballot(in && key > thr));
    n_eq += __popcll(__ballot(in && key == thr));
  }
  if (lane == 0) {
    seg_gt[wave] = n_gt;
    seg_eq[wave] = n_eq;
  }
  __syncthreads();
  uint32_t eq_run = 0, out_run = 0;
  for (int w = 0; w < wave; ++w) {
    const uint32_t e = seg_eq[w];
    const uint32_t room = r > eq_run ? r - eq_run : 0u;
    out_run += seg_gt[w] + (e < room ? e : room);
    eq_run += e;
  }
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int32_t* out_idx = p.out_idx + (int64_t)row * p.out_stride;
  elem_t* out_val =
      p.out_values ? reinterpret_cast<elem_t*>(p.out_values) + (int64_t)row * p.out_stride : nullptr;
  for (int base = s0; base < s1; base += 64) {
    const int i = base + lane;
    const bool in = i < s1;
    elem_t v = 0;
    uint32_t key = 0;
    if (in) {
      v = vals[i];
      key = KT::key(v);
    }
    const bool gt = in && key > thr;
    const bool eq = in && key == thr;
    const uint64_t eq_mask = __ballot(eq);
    const uint32_t eq_rank = eq_run + (uint32_t)__popcll(eq_mask & lt_mask);
    const bool sel = gt || (eq && eq_rank < r);
    const uint64_t sel_mask = __ballot(sel);
    const uint32_t pos = out_run + (uint32_t)__popcll(sel_mask & lt_mask);
    if (sel && pos < (uint32_t)k) {
      int32_t payload;
      if (p.in_idx)
        payload = p.in_idx[(int64_t)row * p.in_idx_stride + i];
      else if (p.page_table)
        payload = p.page_table[i / p.page_size] * p.page_size + i % p.page_size;
      else
        payload = i;
      out_idx[pos] = payload;
      if (out_val) out_val[pos] = v;
    }
    eq_run += (uint32_t)__popcll(eq_mask);
    out_run += (uint32_t)__popcll(sel_mask);
  }
}

// inclusive prefix sum inside a wavefront
__device__ __forceinline__ uint32_t wave_prefix_sum(uint32_t x, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    uint32_t y = __shfl_up(x, off, 64);
    if (lane >= off) x += y;
  }
  return x;
}

// exclusive prefix sum over the 1024 threads of the workgroup; `total` gets the grand total.
// scratch: 16 words of LDS.  Contains two barriers.
__device__ __forceinline__ uint32_t block_exclusive_sum(uint32_t x, int lane, int wave,
                                                        uint32_t* scratch, uint32_t& total) {
  const uint32_t incl = wave_prefix_sum(x, lane);
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kTopkWaves; ++w) {
    const uint32_t t = scratch[w];
    before += w < wave ? t : 0u;
    all += t;
  }
  __syncthreads();
  total = all;
  return before + incl - x;
}

// Register-resident variant for rows of up to 1024 * IPT elements: thread t owns elements
// j * 1024 + t (j < IPT), so the row is read from memory exactly once (coalesced, IPT loads in
// flight per thread) and every radix pass and the ordered emission work on registers.  In index
// order the row is a sequence of 64-element runs (j, wave); per-run counts are prefix-summed in
// LDS and the lanes of a run rank themselves with ballots.
template <typename T, int IPT>
__global__ __launch_bounds__(kTopkThreads) void topk_reg_kernel(const TopkParams p) {
  typedef KeyTraits<T> KT;
  typedef typename KT::elem_t elem_t;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int len = p.len;
  const int k = p.k;  // 1 <= k <= len <= 1024 * IPT (host-checked)
  const elem_t* vals = reinterpret_cast<const elem_t*>(p.values) + (int64_t)row * p.values_stride;

  __shared__ uint32_t hist[kMaxBins];
  __shared__ uint32_t wave_tot[kTopkWaves];
  __shared__ uint32_t sh_bin, sh_krem;
  __shared__ uint32_t run_eq[IPT * kTopkWaves], run_out[IPT * kTopkWaves];

  // key 0 is below every real key (it would be the image of a negative NaN, which maps to the
  // maximum instead), so it marks the slots past the end of the row
  uint32_t key[IPT];
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const int i = j * kTopkThreads + tid;
    key[j] = i < len ? KT::key(vals[i]) : 0u;
  }

  uint32_t prefix = 0, mask = 0, krem = (uint32_t)k;
  int shift = KT::kBits;
#pragma unroll
  for (int pass = 0; pass < KT::kPasses; ++pass) {
    const int bits = KT::digit_bits(pass);
    const int nb = 1 << bits;
    shift -= bits;
    for (int i = tid; i < nb; i += kTopkThreads) hist[i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < IPT; ++j)
      if ((key[j] & mask) == prefix && key[j] != 0u)
        atomicAdd(&hist[(key[j] >> shift) & (nb - 1)], 1u);
    __syncthreads();
    const int bpt = nb >= kTopkThreads ? nb / kTopkThreads : 1;
    const int my_bin = tid * bpt;
    uint32_t local = 0;
    if (my_bin < nb)
      for (int j = 0; j < bpt; ++j) local += hist[my_bin + j];
    const uint32_t suf = wave_suffix_sum(local, lane);
    if (lane == 0) wave_tot[wave] = suf;
    __syncthreads();
    uint32_t above = suf - local;
    for (int w = wave + 1; w < kTopkWaves; ++w) above += wave_tot[w];
    if (my_bin < nb) {
      for (int j = bpt - 1; j >= 0; --j) {
        const uint32_t c = hist[my_bin + j];
        if (above < krem && krem <= above + c) {
          sh_bin = (uint32_t)(my_bin + j);
          sh_krem = krem - above;
        }
        above += c;
      }
    }
    __syncthreads();
    prefix |= sh_bin << shift;
    mask |= (uint32_t)(nb - 1) << shift;
    krem = sh_krem;
    __syncthreads();
  }
  const uint32_t thr = prefix;
  const uint32_t r = krem;

  // per-run counts: run (j, wave) covers elements j*1024 + wave*64 .. +64
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const uint32_t n_gt = (uint32_t)__popcll(__ballot(key[j] > thr));
    const uint32_t n_eq = (uint32_t)__popcll(__ballot(key[j] == thr));
    if (lane == 0) {
      run_eq[j * kTopkWaves + wave] = n_eq;
      run_out[j * kTopkWaves + wave] = n_gt;
    }
  }
  __syncthreads();
  // thread x handles run x (IPT * 16 <= 1024 runs): ties taken from each run, then output offsets
  {
    const bool has = tid < IPT * kTopkWaves;
    const uint32_t e = has ? run_eq[tid] : 0u;
    const uint32_t g = has ? run_out[tid] : 0u;
    uint32_t total;
    const uint32_t eq_before = block_exclusive_sum(e, lane, wave, wave_tot, total);
    const uint32_t room = r > eq_before ? r - eq_before : 0u;
    const uint32_t take = e < room ? e : room;
    const uint32_t out_before = block_exclusive_sum(g + take, lane, wave, wave_tot, total);
    if (has) {
      run_eq[tid] = eq_before;
      run_out[tid] = out_before;
    }
  }
  __syncthreads();

  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int32_t* out_idx = p.out_idx + (int64_t)row * p.out_stride;
  elem_t* out_val =
      p.out_values ? reinterpret_cast<elem_t*>(p.out_values) + (int64_t)row * p.out_stride : nullptr;
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const bool gt = key[j] > thr;
    const bool eq = key[j] == thr;
    const uint64_t eq_mask = __ballot(eq);
    const uint32_t eq_rank = run_eq[j * kTopkWaves + wave] + (uint32_t)__popcll(eq_mask & lt_mask);
    const bool sel = gt || (eq && eq_rank < r);
    const uint64_t sel_mask = __ballot(sel);
    const uint32_t pos = run_out[j * kTopkWaves + wave] + (uint32_t)__popcll(sel_mask & lt_mask);
    if (sel && pos < (uint32_t)k) {
      const int i = j * kTopkThreads + tid;
      int32_t payload;
      if (p.in_idx)
        payload = p.in_idx[(int64_t)row * p.in_idx_stride + i];
      else if (p.page_table)
        payload = p.page_table[i / p.page_size] * p.page_size + i % p.page_size;
      else
        payload = i;
      out_idx[pos] = payload;
      if (out_val) out_val[pos] = vals[i];
    }
  }
}

template <typename T>
static void launch_topk(const TopkParams& p, int rows, hipStream_t st) {
  const dim3 grid(rows), block(kTopkThreads);
  if (p.len <= 8 * kTopkThreads)
    hipLaunchKernelGGL((topk_reg_kernel<T, 8>), grid, block, 0, st, p);
  else if (p.len <= 16 * kTopkThreads)
    hipLaunchKernelGGL((topk_reg_kernel<T, 16>), grid, block, 0, st, p);
  else if (p.len <= 32 * kTopkThreads)
    hipLaunchKernelGGL((topk_reg_kernel<T, 32>), grid, block, 0, st, p);
  else if (p.len <= 48 * kTopkThreads)
    hipLaunchKernelGGL((topk_reg_kernel<T, 48>), grid, block, 0, st, p);
  else if (p.len <= 64 * kTopkThreads)
    hipLaunchKernelGGL((topk_reg_kernel<T, 64>), grid, block, 0, st, p);
  else
    hipLaunchKernelGGL(topk_kernel<T>, grid, block, 0, st, p);
}

// out[r, i] = sum_{h in row r} exp(logits[h, i] - lse[h])
__global__ __launch_bounds__(256) void score_reduce_kernel(const float* __restrict__ logits,
                                                           int64_t logits_stride,
                                                           const float* __restrict__ lse,
                                                           int heads_per_row, int n,
                                                           float* __restrict__ out,
                                                           int64_t out_stride) {
  const int r = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float acc = 0.f;
  for (int j = 0; j < heads_per_row; ++j) {
    const int h = r * heads_per_row + j;
    acc += fast_exp2((logits[(int64_t)h * logits_stride + i] - lse[h]) * kLog2e);
  }
  out[(int64_t)r * out_stride + i] = acc;
}

}  // namespace tidal

using namespace tidal;

extern "C" int td_topk(const void* values, int32_t values_dtype, int64_t values_stride,
                       int32_t rows, int32_t len, int32_t k, const int32_t* in_idx,
                       int64_t in_idx_stride, const int32_t* page_table, int32_t page_size,
                       void* out_values, int32_t* out_idx, int64_t out_stride, void* stream) {
  TD_REQUIRE(values && out_idx, "td_topk: NULL values or out_idx");
  TD_REQUIRE(rows >= 1, "td_topk: rows %d < 1", rows);
  TD_REQUIRE(len >= 0 && k >= 0, "td_topk: len %d / k %d", len, k);
  TD_REQUIRE(values_stride >= len, "td_topk: values_stride %lld < len %d", (long long)values_stride,
             len);
  if (k > len) k = len;
  TD_REQUIRE(out_stride >= k, "td_topk: out_stride %lld < k %d", (long long)out_stride, k);
  TD_REQUIRE(!in_idx || in_idx_stride >= 0, "td_topk: in_idx_stride %lld", (long long)in_idx_stride);
  TD_REQUIRE(!page_table || page_size >= 1, "td_topk: page_size %d", page_size);
  if (k == 0) return TD_OK;
  TopkParams p;
  p.values = values;
  p.values_stride = values_stride;
  p.len = len;
  p.k = k;
  p.in_idx = in_idx;
  p.in_idx_stride = in_idx_stride;
  p.page_table = in_idx ? nullptr : page_table;
  p.page_size = page_size;
  p.out_values = out_values;
  p.out_idx = out_idx;
  p.out_stride = out_stride;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  switch (values_dtype) {
    case TD_F32: launch_topk<F32>(p, rows, st); break;
    case TD_F16: launch_topk<F16>(p, rows, st); break;
    case TD_BF16: launch_topk<BF16>(p, rows, st); break;
    default:
      return fail(TD_ERR_UNSUPPORTED, "Top-k filtering failed to dispatch with dtype %d",
                  values_dtype);
  }
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_score_reduce(const float* logits, int64_t logits_stride, const float* lse,
                               int32_t num_qo_heads, int32_t num_kv_heads, int32_t n, int32_t mode,
                               float* out, int64_t out_stride, void* stream) {
  TD_REQUIRE(logits && lse && out, "td_score_reduce: NULL argument");
  TD_REQUIRE(num_kv_heads >= 1 && num_qo_heads >= num_kv_heads && num_qo_heads % num_kv_heads == 0,
             "td_score_reduce: heads %d / %d", num_qo_heads, num_kv_heads);
  TD_REQUIRE(n >= 0 && logits_stride >= n, "td_score_reduce: n %d, logits_stride %lld", n,
             (long long)logits_stride);
  TD_REQUIRE(mode == TD_REDUCE_HEAD_SUM || mode == TD_REDUCE_GROUP_SUM, "td_score_reduce: mode %d",
             mode);
  const int rows = mode == TD_REDUCE_HEAD_SUM ? 1 : num_kv_heads;
  TD_REQUIRE(rows == 1 || out_stride >= n, "td_score_reduce: out_stride %lld < n %d",
             (long long)out_stride, n);
  if (n == 0) return TD_OK;
  hipLaunchKernelGGL(score_reduce_kernel, dim3((n + 255) / 256, rows), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), logits, logits_stride, lse,
                     num_qo_heads / rows, n, out, out_stride);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
