// Row-wise top-k selection and the cross-head score reduction for gfx950 (MI355X).
//
// One 1024-thread workgroup (16 wavefronts) per row (rows of up to 65536 elements are held in
// registers, longer ones are re-read from L2 per pass; given scratch memory, rows of more than
// 8192 elements are split over several workgroups, see topk_coop_select_kernel) runs an MSB-first radix select over
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
  int64_t page_table_stride;  // elements between the tables of consecutive row groups
  int32_t rows_per_table;     // rows that share one table / one length (all rows when there is one)
  const int32_t* len_arr;     // per row group: elements that take part (clamped to 1..len), or null
  int32_t page_size;
  int32_t page_shift;  // log2(page_size) when it is a power of two, else -1
  void* out_values;
  int32_t* out_idx;
  int64_t out_stride;
};

// physical slot of position i through the page table
__device__ __forceinline__ const int32_t* table_of(const TopkParams& p, int row) {
  if (p.page_table == nullptr || p.page_table_stride == 0) return p.page_table;
  return p.page_table + (int64_t)(row / p.rows_per_table) * p.page_table_stride;
}
// elements of this row that take part, and how many of them are selected
__device__ __forceinline__ int row_len(const TopkParams& p, int row) {
  if (p.len_arr == nullptr) return p.len;
  const int n = p.len_arr[row / p.rows_per_table];
  return n < 1 ? 1 : (n > p.len ? p.len : n);
}
__device__ __forceinline__ int row_k(const TopkParams& p, int len) { return p.k < len ? p.k : len; }

__device__ __forceinline__ int32_t slot_of(const TopkParams& p, const int32_t* table, int i) {
  if (p.page_shift >= 0)
    return (table[i >> p.page_shift] << p.page_shift) | (i & (p.page_size - 1));
  return table[i / p.page_size] * p.page_size + i % p.page_size;
}

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
  const int32_t* table = table_of(p, row);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int len = row_len(p, row);
  const int k = row_k(p, len);  // 1 <= k <= len
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
        payload = slot_of(p, table, i);
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
  const int32_t* table = table_of(p, row);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int len = row_len(p, row);
  const int k = row_k(p, len);  // 1 <= k <= len <= 1024 * IPT (host-checked for p.len)
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
    const uint32_t kv = KT::key(vals[i < len ? i : len - 1]);  // unconditional load: all IPT in flight
    key[j] = i < len ? kv : 0u;
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
        payload = slot_of(p, table, i);
      else
        payload = i;
      out_idx[pos] = payload;
      if (out_val) out_val[pos] = vals[i];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Cooperative variant: G workgroups per row, two launches.  One compute unit needs ~40 us to
// push a 32K-element row through the single-workgroup kernels above (the row costs ~40K wave
// instructions); with a handful of rows that leaves the other 200+ compute units idle.
//
//   launch 1 (topk_coop_hist_kernel, grid G x rows): every workgroup histograms the top 11 key
//     bits of its slice in LDS and adds the non-empty bins to a per-row global histogram.
//   launch 2 (topk_coop_select_kernel, grid G x rows): every workgroup locates the threshold bin
//     in the row histogram (the same scan, redundantly: it is cheap), counts what its slice holds
//     above the bin and appends the slice's members of the bin (key, index) to the row's
//     candidate list; the last workgroup of a row to arrive (ticket) loads the list (a few
//     thousand entries instead of the row), finishes the radix select on it, and publishes the
//     threshold key T, the number r of ties to take and per-slice output / tie offsets.
//     A bin with more members than the list holds (most keys share 11 leading bits) is left to
//     the last workgroup, which narrows it with streaming passes over the row.
//   launch 3 (topk_coop_emit_kernel, grid G x rows): every workgroup emits its slice in index
//     order at its published offset.
//
// Scratch per row (uint32): [0,2048) histogram, 2048 ticket, 2049 T, 2050 r, then per slice
// (out_before, eq_before), the candidate count, per slice the count above the bin, and the
// candidate keys and indices.  Histogram, ticket and candidate count must be zero before the
// first call; launch 2 leaves them zero again.  Values are keyed as fp32 whatever the input type.
// ---------------------------------------------------------------------------------------------
constexpr int kCoopIPT = 8;                       // keys per thread and slice
constexpr int kCoopSlice = kCoopIPT * kTopkThreads;  // 8192 elements per workgroup
constexpr int kCoopMaxSlices = 32;
constexpr int kCoopBatch = 4;                     // slices per trip of the row pass
constexpr int kCoopCand = 6144;                   // candidates kept in LDS
constexpr int kCoopOffsets = 2051;                            // (out_before, eq_before) per slice
constexpr int kCoopCandCount = kCoopOffsets + 2 * kCoopMaxSlices;
constexpr int kCoopSliceGt = kCoopCandCount + 1;              // per slice: keys above the bin
constexpr int kCoopCandKey = kCoopSliceGt + kCoopMaxSlices;
constexpr int kCoopCandIdx = kCoopCandKey + kCoopCand;
constexpr int kCoopRowWords = kCoopCandIdx + kCoopCand;

__device__ __forceinline__ uint32_t load_agent(const uint32_t* at) {
  return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(uint32_t* at, uint32_t v) {
  __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T>
__device__ __forceinline__ uint32_t coop_key(const void* base, int64_t i);
template <>
__device__ __forceinline__ uint32_t coop_key<F32>(const void* base, int64_t i) {
  return KeyTraits<F32>::key(reinterpret_cast<const float*>(base)[i]);
}
template <>
__device__ __forceinline__ uint32_t coop_key<F16>(const void* base, int64_t i) {
  return KeyTraits<F32>::key(to_float<F16>(reinterpret_cast<const uint16_t*>(base)[i]));
}
template <>
__device__ __forceinline__ uint32_t coop_key<BF16>(const void* base, int64_t i) {
  return KeyTraits<F32>::key(to_float<BF16>(reinterpret_cast<const uint16_t*>(base)[i]));
}

// Workgroups are handed to the 8 XCDs round-robin by linear id.  All slices of a row go to one
// XCD, so that what the row's workgroups read in the first phase is in the L2 that the row's
// last workgroup (and the emit launch) reads again: linear id = (row / 8 * slices + slice) * 8 +
// row % 8, grid = ceil(rows / 8) * slices * 8 workgroups; ids of rows past the end do nothing.
constexpr int kXcds = 8;
__device__ __forceinline__ bool coop_decode(int n_slices, int rows, int& slice, int& row) {
  const int id = blockIdx.x;
  const int t = id / kXcds;
  row = t / n_slices * kXcds + id % kXcds;
  slice = t % n_slices;
  return row < rows;
}

template <typename T> struct ElemOf { typedef uint16_t type; };
template <> struct ElemOf<F32> { typedef float type; };

// lanes below this one whose bit is set in a wave-wide mask
__device__ __forceinline__ uint32_t lanes_below(uint64_t m) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}

// One radix level over the candidates in LDS: histogram the `bits`-wide digit at `shift` of the
// candidates whose key matches (mask, prefix); updates prefix / mask / krem.
__device__ __forceinline__ void coop_level(const uint32_t* ckey, int n_cand, uint32_t* hist,
                                           uint32_t* wave_tot, uint32_t* sh, int bits, int shift,
                                           uint32_t& prefix, uint32_t& mask, uint32_t& krem, int tid,
                                           int lane, int wave) {
  const int nb = 1 << bits;
  for (int i = tid; i < nb; i += kTopkThreads) hist[i] = 0;
  __syncthreads();
  for (int i = tid; i < n_cand; i += kTopkThreads) {
    const uint32_t key = ckey[i];
    if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & (nb - 1)], 1u);
  }
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
        sh[0] = (uint32_t)(my_bin + j);
        sh[1] = krem - above;
      }
      above += c;
    }
  }
  __syncthreads();
  prefix |= sh[0] << shift;
  mask |= (uint32_t)(nb - 1) << shift;
  krem = sh[1];
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(kTopkThreads) void topk_coop_hist_kernel(const TopkParams p,
                                                                      uint32_t* scratch,
                                                                      int n_slices, int rows) {
  int slice, row;
  if (!coop_decode(n_slices, rows, slice, row)) return;
  const int tid = threadIdx.x;
  const int len = row_len(p, row);
  const void* vals = reinterpret_cast<const char*>(p.values) +
                     (int64_t)row * p.values_stride * sizeof(typename ElemOf<T>::type);
  uint32_t* rs = scratch + (int64_t)row * kCoopRowWords;
  __shared__ uint32_t hist[2048];
  for (int i = tid; i < 2048; i += kTopkThreads) hist[i] = 0;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    const int i = slice * kCoopSlice + j * kTopkThreads + tid;
    const uint32_t kv = coop_key<T>(vals, i < len ? i : len - 1);  // loads stay unconditional
    if (i < len) atomicAdd(&hist[kv >> 21], 1u);
  }
  __syncthreads();
  for (int i = tid; i < 2048; i += kTopkThreads) {
    const uint32_t c = hist[i];
    if (c) __hip_atomic_fetch_add(rs + i, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <typename T>
__global__ __launch_bounds__(kTopkThreads) void topk_coop_select_kernel(const TopkParams p,
                                                                        uint32_t* scratch,
                                                                        int n_slices, int rows) {
  int slice, row;
  if (!coop_decode(n_slices, rows, slice, row)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int len = row_len(p, row);
  const void* vals = reinterpret_cast<const char*>(p.values) +
                     (int64_t)row * p.values_stride * sizeof(typename ElemOf<T>::type);
  uint32_t* rs = scratch + (int64_t)row * kCoopRowWords;

  __shared__ uint32_t hist[2048];
  __shared__ uint32_t wave_tot[kTopkWaves];
  __shared__ uint32_t sh[4];
  __shared__ uint32_t ckey[kCoopCand];
  __shared__ int32_t cidx[kCoopCand];
  __shared__ uint32_t slice_gt[kCoopMaxSlices], slice_eq[kCoopMaxSlices];
  __shared__ uint32_t n_cand_sh, n_above_sh, cand_base_sh;

  // ---- every workgroup: its slice's keys (in flight while the histogram is scanned) ------------
  uint32_t own[kCoopIPT];
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    const int i = slice * kCoopSlice + j * kTopkThreads + tid;
    const uint32_t kv = coop_key<T>(vals, i < len ? i : len - 1);
    own[j] = i < len ? kv : 0u;  // 0 lies below every real key
  }
  // ---- threshold bin of level 1 from the row histogram of the launch before -------------------
  for (int i = tid; i < 2048; i += kTopkThreads) hist[i] = load_agent(rs + i);
  if (tid < kCoopMaxSlices) slice_gt[tid] = slice_eq[tid] = 0;
  if (tid == 0) n_cand_sh = n_above_sh = 0;
  __syncthreads();
  uint32_t prefix = 0, mask = 0, krem = (uint32_t)row_k(p, len);
  {
    const int my_bin = tid * 2;
    const uint32_t local = hist[my_bin] + hist[my_bin + 1];
    const uint32_t suf = wave_suffix_sum(local, lane);
    if (lane == 0) wave_tot[wave] = suf;
    __syncthreads();
    uint32_t above = suf - local;
    for (int w = wave + 1; w < kTopkWaves; ++w) above += wave_tot[w];
    for (int j = 1; j >= 0; --j) {
      const uint32_t c = hist[my_bin + j];
      if (above < krem && krem <= above + c) {
        sh[0] = (uint32_t)(my_bin + j);
        sh[1] = krem - above;
        sh[3] = c;  // candidates in the threshold bin
      }
      above += c;
    }
    __syncthreads();
    prefix = sh[0] << 21;
    mask = 0x7ffu << 21;
    krem = sh[1];
  }
  int n_in_bin = (int)sh[3];
  const bool crowded = n_in_bin > kCoopCand;  // the same in every workgroup of the row
  __syncthreads();

  // ---- every workgroup: count above the bin, append the slice's members of the bin -------------
  if (!crowded) {
    uint32_t n_above = 0, n_in = 0;
    uint64_t cm[kCoopIPT];
#pragma unroll
    for (int j = 0; j < kCoopIPT; ++j) {
      n_above += (uint32_t)__popcll(__ballot((own[j] & mask) > prefix));
      cm[j] = __ballot(own[j] != 0u && (own[j] & mask) == prefix);
      n_in += (uint32_t)__popcll(cm[j]);
    }
    uint32_t at = 0;
    if (lane == 0) {
      if (n_in) at = atomicAdd(&n_cand_sh, n_in);
      if (n_above) atomicAdd(&n_above_sh, n_above);
    }
    at = __shfl(at, 0, 64);
#pragma unroll
    for (int j = 0; j < kCoopIPT; ++j) {
      const uint32_t mine = at + lanes_below(cm[j]);
      if ((cm[j] >> lane) & 1ull) {  // at most n_in_bin <= kCoopCand candidates in the whole row
        ckey[mine] = own[j];
        cidx[mine] = slice * kCoopSlice + j * kTopkThreads + tid;
      }
      at += (uint32_t)__popcll(cm[j]);
    }
    __syncthreads();
    const uint32_t n_mine = n_cand_sh;
    if (tid == 0) {
      cand_base_sh = n_mine ? __hip_atomic_fetch_add(rs + kCoopCandCount, n_mine, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT)
                            : 0u;
      store_agent(rs + kCoopSliceGt + slice, n_above_sh);
    }
    __syncthreads();
    const uint32_t cbase = cand_base_sh;
    for (uint32_t i = tid; i < n_mine; i += kTopkThreads) {
      store_agent(rs + kCoopCandKey + cbase + i, ckey[i]);
      store_agent(rs + kCoopCandIdx + cbase + i, (uint32_t)cidx[i]);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this workgroup's stores are performed
  __syncthreads();
  if (tid == 0)
    sh[2] = __hip_atomic_fetch_add(rs + 2048, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (sh[2] != (uint32_t)(n_slices - 1)) return;

  // ---- last workgroup of the row: finish (the scratch is cleaned at the very end: a store issued
  // here would sit in front of the candidate loads in the in-order memory queue) -----------------
  if (tid == 0) n_cand_sh = 0;
  int shift = 21;
  if (!crowded) {
    // the row's candidates, from every slice
    for (int i = tid; i < n_in_bin; i += kTopkThreads) {
      ckey[i] = load_agent(rs + kCoopCandKey + i);
      cidx[i] = (int32_t)load_agent(rs + kCoopCandIdx + i);
    }
    if (tid < n_slices) slice_gt[tid] = load_agent(rs + kCoopSliceGt + tid);
    if (tid == 0) n_cand_sh = (uint32_t)n_in_bin;
  }
  __syncthreads();

  // A bin too crowded for the list is narrowed with streaming passes over the row (11 more bits,
  // then 10): only pathological rows (most keys share 11 leading bits) get here.
  while (n_in_bin > kCoopCand && shift > 0) {
    const int bits = shift > 10 ? 11 : 10;
    const int nb = 1 << bits;
    shift -= bits;
    for (int i = tid; i < nb; i += kTopkThreads) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < len; i += kTopkThreads) {
      const uint32_t key = coop_key<T>(vals, i);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & (nb - 1)], 1u);
    }
    __syncthreads();
    const int bpt = nb / kTopkThreads;  // 2 or 1
    const int my_bin = tid * bpt;
    uint32_t local = 0;
    for (int j = 0; j < bpt; ++j) local += hist[my_bin + j];
    const uint32_t suf = wave_suffix_sum(local, lane);
    if (lane == 0) wave_tot[wave] = suf;
    __syncthreads();
    uint32_t above = suf - local;
    for (int w = wave + 1; w < kTopkWaves; ++w) above += wave_tot[w];
    for (int j = bpt - 1; j >= 0; --j) {
      const uint32_t c = hist[my_bin + j];
      if (above < krem && krem <= above + c) {
        sh[0] = (uint32_t)(my_bin + j);
        sh[1] = krem - above;
        sh[3] = c;
      }
      above += c;
    }
    __syncthreads();
    prefix |= sh[0] << shift;
    mask |= (uint32_t)(nb - 1) << shift;
    krem = sh[1];
    n_in_bin = (int)sh[3];
    __syncthreads();
  }

  // ---- phase 3: one pass over the row: count per slice what lies above the candidate range,
  //      gather the candidates (keys matching the prefix) unless the range is a single key -------
  const bool gather = shift > 0;  // shift == 0: all bits fixed, every candidate equals the threshold
  // (crowded rows only; otherwise the slices have done this.)  kCoopBatch slices per trip: a
  // thread keeps 32 loads in flight, which is what it takes to cover the memory latency from one
  // compute unit
  for (int base0 = 0; crowded && base0 < len; base0 += kCoopBatch * kCoopSlice) {
    uint32_t key[kCoopBatch][kCoopIPT];
#pragma unroll
    for (int s = 0; s < kCoopBatch; ++s)
#pragma unroll
      for (int j = 0; j < kCoopIPT; ++j) {
        const int i = base0 + s * kCoopSlice + j * kTopkThreads + tid;
        const uint32_t kv = coop_key<T>(vals, i < len ? i : len - 1);
        key[s][j] = i < len ? kv : 0u;  // 0 lies below every real key
      }
#pragma unroll
    for (int s = 0; s < kCoopBatch; ++s) {
      const int base = base0 + s * kCoopSlice;
      if (base >= len) break;
      const int sl = base / kCoopSlice;
      uint32_t n_above = 0, n_in = 0;
      uint64_t cm[kCoopIPT];
#pragma unroll
      for (int j = 0; j < kCoopIPT; ++j) {
        n_above += (uint32_t)__popcll(__ballot((key[s][j] & mask) > prefix));
        cm[j] = __ballot(key[s][j] != 0u && (key[s][j] & mask) == prefix);
        n_in += (uint32_t)__popcll(cm[j]);
      }
      if (gather && n_in) {  // wave-uniform: one LDS reservation per wave and slice
        uint32_t at = 0;
        if (lane == 0) at = atomicAdd(&n_cand_sh, n_in);
        at = __shfl(at, 0, 64);
#pragma unroll
        for (int j = 0; j < kCoopIPT; ++j) {
          const uint32_t mine = at + lanes_below(cm[j]);
          if (((cm[j] >> lane) & 1ull) && mine < (uint32_t)kCoopCand) {
            ckey[mine] = key[s][j];
            cidx[mine] = base + j * kTopkThreads + tid;
          }
          at += (uint32_t)__popcll(cm[j]);
        }
      }
      if (lane == 0) {
        if (n_above) atomicAdd(&slice_gt[sl], n_above);
        if (!gather && n_in) atomicAdd(&slice_eq[sl], n_in);
      }
    }
  }
  __syncthreads();
  uint32_t thr = prefix, r = krem;
  if (gather) {
    const int n_cand = (int)n_cand_sh;  // == n_in_bin <= kCoopCand
    // ---- phase 4: finish the radix select on the candidates ----------------------------------
    while (shift > 0) {
      const int bits = shift > 10 ? 11 : 10;
      shift -= bits;
      coop_level(ckey, n_cand, hist, wave_tot, sh, bits, shift, prefix, mask, krem, tid, lane, wave);
    }
    thr = prefix;
    r = krem;
    // ---- phase 5: candidates above / equal to T, per slice -----------------------------------
    for (int base = 0; base < n_cand; base += kTopkThreads) {
      const int i = base + tid;
      const bool have = i < n_cand;
      const uint32_t ck = have ? ckey[i] : 0u;
      const int csl = have ? cidx[i] / kCoopSlice : -1;
      for (int sl = 0; sl < n_slices; ++sl) {
        const uint64_t gm = __ballot(csl == sl && ck > thr);
        const uint64_t em = __ballot(csl == sl && ck == thr);
        if (lane == 0) {
          if (gm) atomicAdd(&slice_gt[sl], (uint32_t)__popcll(gm));
          if (em) atomicAdd(&slice_eq[sl], (uint32_t)__popcll(em));
        }
      }
    }
    __syncthreads();
  }
  // ---- phase 6: publish T, r and the per-slice offsets ------------------------------------------
  if (tid == 0) {
    rs[2049] = thr;
    rs[2050] = r;
    uint32_t out_run = 0, eq_run = 0;
    for (int sl = 0; sl < n_slices; ++sl) {
      rs[kCoopOffsets + 2 * sl] = out_run;
      rs[kCoopOffsets + 1 + 2 * sl] = eq_run;
      const uint32_t e = slice_eq[sl];
      const uint32_t room = r > eq_run ? r - eq_run : 0u;
      out_run += slice_gt[sl] + (e < room ? e : room);
      eq_run += e;
    }
    store_agent(rs + 2048, 0u);
    store_agent(rs + kCoopCandCount, 0u);
  }
  // leave the histogram zero for the next call
  for (int i = tid; i < 2048; i += kTopkThreads) store_agent(rs + i, 0u);
}

template <typename T>
__global__ __launch_bounds__(kTopkThreads) void topk_coop_emit_kernel(const TopkParams p,
                                                                      const uint32_t* scratch,
                                                                      int n_slices, int rows) {
  typedef typename ElemOf<T>::type elem_t;
  int slice, row;
  if (!coop_decode(n_slices, rows, slice, row)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int len = row_len(p, row);
  const elem_t* vals = reinterpret_cast<const elem_t*>(p.values) + (int64_t)row * p.values_stride;
  const uint32_t* rs = scratch + (int64_t)row * kCoopRowWords;
  const uint32_t thr = rs[2049], r = rs[2050];
  const uint32_t slice_out = rs[kCoopOffsets + 2 * slice], slice_eq = rs[kCoopOffsets + 1 + 2 * slice];

  __shared__ uint32_t wave_tot[kTopkWaves];
  __shared__ uint32_t run_eq[kCoopIPT * kTopkWaves], run_out[kCoopIPT * kTopkWaves];

  uint32_t key[kCoopIPT];
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    const int i = slice * kCoopSlice + j * kTopkThreads + tid;
    const uint32_t kv = coop_key<T>(vals, i < len ? i : len - 1);
    key[j] = i < len ? kv : 0u;  // 0 lies below every real key
  }
  int32_t* out_idx = p.out_idx + (int64_t)row * p.out_stride;
  elem_t* out_val =
      p.out_values ? reinterpret_cast<elem_t*>(p.out_values) + (int64_t)row * p.out_stride : nullptr;
  // Payloads and values of every element are fetched right away, unconditionally (they sit in
  // L2): together with the keys they are one round trip, and no load follows a store (vector
  // loads and stores complete in order on one counter).
  const int32_t* table = table_of(p, row);
  int32_t payload[kCoopIPT];
  elem_t val[kCoopIPT];
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    int i = slice * kCoopSlice + j * kTopkThreads + tid;
    i = i < len ? i : len - 1;
    if (p.in_idx)
      payload[j] = p.in_idx[(int64_t)row * p.in_idx_stride + i];
    else if (p.page_table)
      payload[j] = slot_of(p, table, i);
    else
      payload[j] = i;
    if (out_val) val[j] = vals[i];
  }
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    const uint32_t n_gt = (uint32_t)__popcll(__ballot(key[j] > thr));
    const uint32_t n_eq = (uint32_t)__popcll(__ballot(key[j] == thr));
    if (lane == 0) {
      run_eq[j * kTopkWaves + wave] = n_eq;
      run_out[j * kTopkWaves + wave] = n_gt;
    }
  }
  __syncthreads();
  {
    const bool has = tid < kCoopIPT * kTopkWaves;
    const uint32_t e = has ? run_eq[tid] : 0u;
    const uint32_t g = has ? run_out[tid] : 0u;
    uint32_t total;
    const uint32_t eq_before = slice_eq + block_exclusive_sum(e, lane, wave, wave_tot, total);
    const uint32_t room = r > eq_before ? r - eq_before : 0u;
    const uint32_t take = e < room ? e : room;
    const uint32_t out_before = slice_out + block_exclusive_sum(g + take, lane, wave, wave_tot, total);
    if (has) {
      run_eq[tid] = eq_before;
      run_out[tid] = out_before;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kCoopIPT; ++j) {
    const bool gt = key[j] > thr;
    const bool eq = key[j] == thr;
    const uint64_t eq_mask = __ballot(eq);
    const uint32_t eq_rank = run_eq[j * kTopkWaves + wave] + lanes_below(eq_mask);
    const bool sel = gt || (eq && eq_rank < r);
    const uint64_t sel_mask = __ballot(sel);
    const uint32_t pos = run_out[j * kTopkWaves + wave] + lanes_below(sel_mask);
    if (sel && pos < (uint32_t)row_k(p, len)) {
      out_idx[pos] = payload[j];
      if (out_val) out_val[pos] = val[j];
    }
  }
}

// workgroups per row for the cooperative path, 0 if it does not apply
static int coop_slices(int len, int rows) {
  const int g = (len + kCoopSlice - 1) / kCoopSlice;
  if (g < 2 || g > kCoopMaxSlices) return 0;  // short rows: one workgroup is as fast
  return g;
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
// A 256-thread workgroup covers 64 tokens: wave w sums heads w, w + 4, ... of the row (four
// independent 256-byte row reads in flight per wave and trip), the four partial sums meet in LDS.
__global__ __launch_bounds__(256) void score_reduce_kernel(const float* __restrict__ logits,
                                                           int64_t logits_stride,
                                                           const float* __restrict__ lse,
                                                           int heads_per_row, int n,
                                                           float* __restrict__ out,
                                                           int64_t out_stride) {
  const int r = blockIdx.y;
  const int t = threadIdx.x & 63, hg = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + t;
  const int ic = i < n ? i : n - 1;  // loads stay unconditional
  const float* base = logits + (int64_t)r * heads_per_row * logits_stride + ic;
  const float* lrow = lse + r * heads_per_row;
  float acc = 0.f;
  int j = hg;
  for (; j + 12 < heads_per_row; j += 16) {
    const float x0 = base[(int64_t)j * logits_stride], x1 = base[(int64_t)(j + 4) * logits_stride],
                x2 = base[(int64_t)(j + 8) * logits_stride], x3 = base[(int64_t)(j + 12) * logits_stride];
    acc += fast_exp2((x0 - lrow[j]) * kLog2e);
    acc += fast_exp2((x1 - lrow[j + 4]) * kLog2e);
    acc += fast_exp2((x2 - lrow[j + 8]) * kLog2e);
    acc += fast_exp2((x3 - lrow[j + 12]) * kLog2e);
  }
  for (; j < heads_per_row; j += 4)
    acc += fast_exp2((base[(int64_t)j * logits_stride] - lrow[j]) * kLog2e);
  __shared__ float part[4][64];
  part[hg][t] = acc;
  __syncthreads();
  if (hg == 0 && i < n)
    out[(int64_t)r * out_stride + i] = (part[0][t] + part[1][t]) + (part[2][t] + part[3][t]);
}

}  // namespace tidal

using namespace tidal;

extern "C" int td_topk(const void* values, int32_t values_dtype, int64_t values_stride,
                       int32_t rows, int32_t len, int32_t k, const int32_t* in_idx,
                       int64_t in_idx_stride, const int32_t* page_table,
                       int64_t page_table_stride, int32_t rows_per_table,
                       const int32_t* len_arr, int32_t page_size, void* out_values, int32_t* out_idx, int64_t out_stride, void* workspace,
                       int64_t workspace_bytes, void* stream) {
  TD_REQUIRE(values && out_idx, "td_topk: NULL values or out_idx");
  TD_REQUIRE(rows >= 1, "td_topk: rows %d < 1", rows);
  TD_REQUIRE(len >= 0 && k >= 0, "td_topk: len %d / k %d", len, k);
  TD_REQUIRE(values_stride >= len, "td_topk: values_stride %lld < len %d", (long long)values_stride,
             len);
  if (k > len) k = len;
  TD_REQUIRE(out_stride >= k, "td_topk: out_stride %lld < k %d", (long long)out_stride, k);
  TD_REQUIRE(!in_idx || in_idx_stride >= 0, "td_topk: in_idx_stride %lld", (long long)in_idx_stride);
  TD_REQUIRE(!page_table || page_size >= 1, "td_topk: page_size %d", page_size);
  TD_REQUIRE((!page_table && !len_arr) || (rows_per_table >= 0 && page_table_stride >= 0),
             "td_topk: rows_per_table %d / page_table_stride %lld", rows_per_table,
             (long long)page_table_stride);
  if (k == 0) return TD_OK;
  TopkParams p;
  p.values = values;
  p.values_stride = values_stride;
  p.len = len;
  p.k = k;
  p.in_idx = in_idx;
  p.in_idx_stride = in_idx_stride;
  p.page_table = in_idx ? nullptr : page_table;
  p.page_table_stride = page_table_stride;
  p.rows_per_table = rows_per_table >= 1 ? rows_per_table : rows;
  p.len_arr = len_arr;
  p.page_size = page_size;
  p.page_shift = -1;
  if (page_size >= 1 && (page_size & (page_size - 1)) == 0) p.page_shift = __builtin_ctz(page_size);
  p.out_values = out_values;
  p.out_idx = out_idx;
  p.out_stride = out_stride;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int slices = coop_slices(len, rows);
  if (slices && workspace && workspace_bytes >= (int64_t)rows * kCoopRowWords * 4 &&
      (values_dtype == TD_F32 || values_dtype == TD_F16 || values_dtype == TD_BF16)) {
    uint32_t* ws = reinterpret_cast<uint32_t*>(workspace);
    const dim3 grid((rows + kXcds - 1) / kXcds * slices * kXcds), block(kTopkThreads);
    if (values_dtype == TD_F32) {
      hipLaunchKernelGGL(topk_coop_hist_kernel<F32>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_select_kernel<F32>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_emit_kernel<F32>, grid, block, 0, st, p, ws, slices, rows);
    } else if (values_dtype == TD_F16) {
      hipLaunchKernelGGL(topk_coop_hist_kernel<F16>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_select_kernel<F16>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_emit_kernel<F16>, grid, block, 0, st, p, ws, slices, rows);
    } else {
      hipLaunchKernelGGL(topk_coop_hist_kernel<BF16>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_select_kernel<BF16>, grid, block, 0, st, p, ws, slices, rows);
      hipLaunchKernelGGL(topk_coop_emit_kernel<BF16>, grid, block, 0, st, p, ws, slices, rows);
    }
    TD_HIP_CHECK(hipGetLastError());
    return TD_OK;
  }
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

extern "C" int64_t td_topk_workspace_bytes(int32_t rows) {
  return (int64_t)(rows < 1 ? 1 : rows) * kCoopRowWords * 4;
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
  hipLaunchKernelGGL(score_reduce_kernel, dim3((n + 63) / 64, rows), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), logits, logits_stride, lse,
                     num_qo_heads / rows, n, out, out_stride);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
