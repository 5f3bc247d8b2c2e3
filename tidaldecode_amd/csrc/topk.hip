// Row-wise top-k selection and the cross-head score reduction for gfx950 (MI355X).
//
// Exact selection by radix select over order-preserving integer images of the fp32 scores (fp16 /
// bf16 scores are widened first): the k-th largest key T and the number r of elements equal to T
// that still fit, then an ordered pass that emits every element above T plus the first r elements
// equal to T.  Ties go to the lower position and each output row is sorted by position: the
// result is a pure function of the input row.  -0 equals +0, every NaN ranks above +inf.
//
// Two routes:
//   * topk_slice_kernel, one launch: every workgroup (1024 threads) of a row runs the selection on
//     the whole row -- up to 64K elements from registers -- and emits its own slice of it.  All
//     rows of up to 65536 elements, and longer ones when there are many rows or no scratch.
//   * topk_coop_{hist,select,emit}_kernel, three launches over a zeroed scratch: the workgroups of
//     a row share the row.  A few rows of more than 65536 elements.
//
// Replaces decode_select_k (kernels/include/topk/decode_select_k.cuh:25-62 of the reference),
// which launches RAFT's radix_topk_one_block_kernel, one 512-thread block per head.

#include <type_traits>

#include "common.cuh"

namespace tidal {

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / 64;

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
  const float* row_bound;  // per row: a value no score of the row exceeds (NaN: none known), or null
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
  __device__ static key_t key(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) == 0u) u = 0u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
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

// ---------------------------------------------------------------------------------------------
// Cooperative variant: G workgroups per row, three launches, for rows too long to keep in the
// registers of one workgroup (more than 65536 elements) when there are few of them: the
// workgroups of a row split the row instead of each going through all of it.
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

// ---------------------------------------------------------------------------------------------
// Sliced variant: one launch, no scratch, no exchange between workgroups.  A row is served by
// n_slices workgroups that ALL run the selection on the whole row (the row is small: 128 KiB at
// 32K fp32 scores, read once from HBM and again from the XCD's L2 by the other workgroups of the
// row) and then each emit their own slice of it in position order.  Every workgroup of a row
// computes the same threshold from the same data, so the slices agree.
//
// The selection is a radix select on d = kmax - key (kmax: the row's largest key; the k-th largest
// key is the k-th smallest d) that starts at the first bit the row actually uses:
//   1. the row as fp32-order keys in registers (IPT per thread; IPT == 0: rows that do not fit are
//      re-read from L2 in every pass), kmax and kmin by reduction;
//   2. an 8192-bin LDS histogram of (d - lo) >> s over the window [lo, lo + limit): first the
//      8191 << 16 smallest d (values within 2^-64 of the maximum: 128 bins per binade, so the
//      scores around the threshold spread over hundreds of bins and same-address LDS atomics are
//      rare), or all of [0, kmax - kmin] with the smallest s that fits when that is narrower;
//      what lies beyond the window is not counted at all;
//   3. a scan finds the bin of the k-th smallest d; if it lies beyond the window, or the bin holds
//      more keys than the LDS list, step 2 runs again on that narrower range;
//   4. the bin's members (a few dozen) are gathered in LDS and ranked against each other by all
//      threads (larger lists: further radix levels on the list): exact threshold T and the number
//      r of keys equal to T that are taken, those at the lowest positions;
//   5. one pass counts the selected elements in front of the slice and per 64-element run of the
//      slice, a scan turns that into output offsets, and the slice is emitted.
// ---------------------------------------------------------------------------------------------
constexpr int kSliceBins = 8192;
constexpr int kSliceCand = 1024;    // list entries in LDS; a fuller bin gets another level instead
constexpr int kSliceRank = 128;     // lists up to this size are ranked directly
constexpr int kSliceMaxRuns = 64;   // 1024-element runs a slice may hold

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t x) {  // 0 where the source lane does not exist
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
}
// inclusive prefix sum inside every row of 16 lanes (row_shr:1,2,4,8)
__device__ __forceinline__ uint32_t row_prefix_sum(uint32_t x) {
  x += dpp_u32<0x111>(x);
  x += dpp_u32<0x112>(x);
  x += dpp_u32<0x114>(x);
  x += dpp_u32<0x118>(x);
  return x;
}
// inclusive prefix sum over the wavefront
__device__ __forceinline__ uint32_t wave_prefix_sum_dpp(uint32_t x, int lane) {
  x = row_prefix_sum(x);
  const uint32_t t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31),
                 t2 = __builtin_amdgcn_readlane(x, 47);
  return x + (lane >= 16 ? t0 : 0u) + (lane >= 32 ? t1 : 0u) + (lane >= 48 ? t2 : 0u);
}
// arr[0] + ... + arr[n - 1], n <= 16 and the same in the whole wavefront; result in a scalar
__device__ __forceinline__ uint32_t sum_first(const uint32_t* arr, int n, int lane) {
  const uint32_t v = row_prefix_sum(lane < n ? arr[lane & 15] : 0u);
  return __builtin_amdgcn_readlane(v, 15);
}
// maximum over the wavefront (rows of 16 lanes by DPP, then the four rows); result in a scalar
__device__ __forceinline__ int32_t wave_max_i32(int32_t x) {
  int32_t y;
  y = (int32_t)dpp_u32<0xB1>((uint32_t)x), x = x > y ? x : y;   // quad_perm [1,0,3,2]
  y = (int32_t)dpp_u32<0x4E>((uint32_t)x), x = x > y ? x : y;   // quad_perm [2,3,0,1]
  y = (int32_t)dpp_u32<0x141>((uint32_t)x), x = x > y ? x : y;  // row_half_mirror
  y = (int32_t)dpp_u32<0x140>((uint32_t)x), x = x > y ? x : y;  // row_mirror
  const int32_t a = __builtin_amdgcn_readlane(x, 0), b = __builtin_amdgcn_readlane(x, 16),
                c = __builtin_amdgcn_readlane(x, 32), d = __builtin_amdgcn_readlane(x, 48);
  const int32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

struct SliceLds {
  uint32_t hist[kSliceBins];
  uint32_t cd[kSliceCand];   // list: d of the members of the threshold bin
  int32_t ci[kSliceCand];    //       and their positions
  uint32_t run_eq[kSliceMaxRuns * kTopkWaves], run_gt[kSliceMaxRuns * kTopkWaves];
  uint32_t wa[kTopkWaves], wb[kTopkWaves], wc[kTopkWaves];
  uint32_t sh[4];
  uint32_t n_cand;
};

// One radix level: histogram of (d - lo) >> s over the elements with d - lo < limit (for_each
// hands every d of the row or of the list to its argument), then the bin of the krem-th smallest
// of them.  True: bin in tb, its count in n_in, krem becomes the rank inside the bin.  False: fewer
// than krem elements in the window; krem loses their number.  Four barriers; the caller has none
// to add before the next level.
template <class ForEach>
__device__ __forceinline__ bool slice_level(SliceLds& L, ForEach for_each, uint32_t lo, int s,
                                            uint32_t limit, uint32_t& krem, uint32_t& tb,
                                            uint32_t& n_in, int tid, int lane, int wave) {
  uint4* h4 = reinterpret_cast<uint4*>(L.hist);
  h4[tid] = make_uint4(0, 0, 0, 0);
  h4[tid + kTopkThreads] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  for_each([&](uint32_t d) {
    const uint32_t x = d - lo;
    if (x < limit) atomicAdd(&L.hist[x >> s], 1u);
  });
  __syncthreads();
  const uint4 a = h4[2 * tid], b = h4[2 * tid + 1];  // bins 8 tid .. 8 tid + 7
  const uint32_t c[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  const uint32_t local = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
  const uint32_t incl = wave_prefix_sum_dpp(local, lane);
  if (lane == 63) L.wa[wave] = incl;
  __syncthreads();
  const uint32_t total = sum_first(L.wa, kTopkWaves, lane);
  uint32_t before = sum_first(L.wa, wave, lane) + incl - local;
  if (before < krem && krem <= before + local) {  // one thread of the workgroup, if any
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (before < krem && krem <= before + c[i]) {
        L.sh[0] = (uint32_t)(8 * tid + i);
        L.sh[1] = krem - before;
        L.sh[2] = c[i];
      }
      before += c[i];
    }
  }
  __syncthreads();
  if (krem > total) {
    krem -= total;
    return false;
  }
  tb = __builtin_amdgcn_readfirstlane(L.sh[0]);
  krem = __builtin_amdgcn_readfirstlane(L.sh[1]);
  n_in = __builtin_amdgcn_readfirstlane(L.sh[2]);
  return true;
}

// A row of scores behind a buffer descriptor: loads take the descriptor (scalar registers), one
// 32-bit lane offset that is the same for every run, and the run's offset as a scalar, so dozens
// of loads are in flight without an address register pair each; reads past the end of the row
// return 0.  score_bits: bits of the fp32 value of element run * 1024 + tid.
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_descriptor(const void* row, int len) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(row), 0,
                                           len * (int)sizeof(typename ElemOf<T>::type), 0x00020000);
}
// stored_bits: element run * 1024 + tid as it is stored (16-bit types zero-extended); widen: the
// bits of its fp32 value; score_bits: both at once.  A row kept in registers is kept as stored
// and widened where it is used, so that it occupies one register per element on every path.
template <typename T>
__device__ __forceinline__ uint32_t stored_bits(__amdgpu_buffer_rsrc_t row, int tid, int run) {
  if constexpr (std::is_same<T, F32>::value)
    return __builtin_amdgcn_raw_buffer_load_b32(row, tid * 4, run * (kTopkThreads * 4), 0);
  else
    return (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(row, tid * 2, run * (kTopkThreads * 2), 0);
}
template <typename T>
__device__ __forceinline__ uint32_t widen(uint32_t stored) {
  if constexpr (std::is_same<T, F32>::value)
    return stored;
  else
    return __builtin_bit_cast(uint32_t, to_float<T>((uint16_t)stored));
}
template <typename T>
__device__ __forceinline__ uint32_t score_bits(__amdgpu_buffer_rsrc_t row, int tid, int run) {
  return widen<T>(stored_bits<T>(row, tid, run));
}

constexpr int kRunGroup = 8;              // runs of a register-held row that share one "is there such a run" test
constexpr int kStream = 16;               // loads in flight per thread where a row is re-read per pass
constexpr int kOwn = 8;                   // runs of a slice that stay in registers for the emission
constexpr uint32_t kNoElement = ~0u;      // d of the slots past the end of the row: beyond every window

template <typename T, int IPT>
__global__ __launch_bounds__(kTopkThreads) void topk_slice_kernel(const TopkParams p, int n_slices,
                                                                  int rps, int rows) {
  typedef typename ElemOf<T>::type elem_t;
  int slice, row;
  if (!coop_decode(n_slices, rows, slice, row)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int len = row_len(p, row);
  const int k = row_k(p, len);
  const elem_t* vals = reinterpret_cast<const elem_t*>(p.values) + (int64_t)row * p.values_stride;
  const int nruns = (len + kTopkThreads - 1) / kTopkThreads;
  const int j_lo = slice * rps;
  if (j_lo >= nruns) return;  // a slice past the end of a short row (lengths on the device)
  const int j_hi = j_lo + rps < nruns ? j_lo + rps : nruns;
  const int n_own = j_hi - j_lo;
  const int32_t* table = table_of(p, row);
  auto payload_of = [&](int i) -> int32_t {
    if (p.in_idx) return p.in_idx[(int64_t)row * p.in_idx_stride + i];
    if (p.page_table) return slot_of(p, table, i);
    return i;
  };

  __shared__ SliceLds L;

  // ---- 1. the row's scores as raw fp32 bits; the reference point that fixes the mapping to d -------
  // d: 0 for the reference point, growing as the scores fall, equal for equal scores (-0 == +0).
  //   kMixed  the reference is >= +0: d = top - u for the non-negative scores (integer order is
  //           value order there), top + |u| for the negative ones, top = bits of the reference
  //   kNeg    the reference is negative (so is every score): d = u - top
  //   kCanon  a NaN in the row: d = kmax - key with the canonical keys (every NaN the maximum)
  // The reference is the caller's bound of the row when there is one (the row is then mapped and
  // counted as its loads arrive), else the row's largest score, found by a pass of its own.
  enum { kMixed, kNeg, kCanon };
  const __amdgpu_buffer_rsrc_t scores = row_descriptor<T>(vals, len);
  float bound = __builtin_nanf("");
  if (p.row_bound) bound = p.row_bound[row];
  const bool bounded = __builtin_fabsf(bound) < __builtin_inff();  // not for NaN or an infinity
  uint32_t reg[IPT > 0 ? IPT : 1];
  if constexpr (IPT > 0) {
#pragma unroll
    for (int j = 0; j < IPT; ++j) reg[j] = stored_bits<T>(scores, tid, j);  // all in flight
  }
  int mode;
  uint32_t top, dmax;
  if (bounded) {
    top = __builtin_bit_cast(uint32_t, bound + 0.f);  // -0 becomes +0
    if constexpr (!std::is_same<T, F32>::value) {
      // 16-bit scores may have been rounded up past a bound formed in fp32: one bf16 step of room
      if ((int32_t)top >= 0) top += 0x10000u;
      else top = top - 0x10000u >= 0x80000000u ? top - 0x10000u : 0u;
    }
    mode = (int32_t)top >= 0 ? kMixed : kNeg;
    // the largest d a score can have: -inf under a non-negative bound, -inf under a negative one
    dmax = mode == kMixed ? top + 0x7f800000u : 0xff800000u - top;
  } else {
    const uint32_t reg0 = score_bits<T>(scores, 0, 0);  // element 0, which every row has
    int32_t imax = INT32_MIN;       // largest as signed integers: the largest non-negative score, if any
    uint32_t umax = 0u, umin = ~0u;  // as unsigned integers: most negative score / smallest non-negative
    // (only the row's last run has slots past the end; the empty asm keeps the compiler from turning
    // the scalar branch around that case into selects on every run)
    auto extremes = [&](int j, uint32_t u) {
      if ((j + 1) * kTopkThreads > len) {
        asm volatile("");
        if (j * kTopkThreads + tid >= len) u = reg0;
      }
      imax = (int32_t)u > imax ? (int32_t)u : imax;
      umax = u > umax ? u : umax;
      umin = u < umin ? u : umin;
    };
    if constexpr (IPT > 0) {
#pragma unroll
      for (int j8 = 0; j8 < IPT; j8 += kRunGroup) {
        if (j8 < nruns) {
#pragma unroll
          for (int j = j8; j < j8 + kRunGroup; ++j) extremes(j, widen<T>(reg[j]));
        }
      }
    } else {
      for (int jb = 0; jb < nruns; jb += kStream) {
        uint32_t uu[kStream];
#pragma unroll
        for (int u = 0; u < kStream; ++u) uu[u] = score_bits<T>(scores, tid, jb + u);
#pragma unroll
        for (int u = 0; u < kStream; ++u) extremes(jb + u, uu[u]);
      }
    }
    imax = wave_max_i32(imax);
    umax = (uint32_t)wave_max_i32((int32_t)(umax ^ 0x80000000u)) ^ 0x80000000u;
    umin = ~((uint32_t)wave_max_i32((int32_t)(~umin ^ 0x80000000u)) ^ 0x80000000u);
    if (lane == 0) {
      L.wa[wave] = (uint32_t)imax;
      L.wb[wave] = umax ^ 0x80000000u;
      L.wc[wave] = ~umin ^ 0x80000000u;
    }
    __syncthreads();
    imax = wave_max_i32((int32_t)L.wa[lane & 15]);
    umax = (uint32_t)wave_max_i32((int32_t)L.wb[lane & 15]) ^ 0x80000000u;
    umin = ~((uint32_t)wave_max_i32((int32_t)L.wc[lane & 15]) ^ 0x80000000u);
    if (imax > 0x7f800000 || umax > 0xff800000u) {
      mode = kCanon;
      uint32_t kx = 0u, kn = ~0u;
      auto key_extremes = [&](int j, uint32_t u) {
        const uint32_t kv = KeyTraits<F32>::key(__builtin_bit_cast(float, u));
        if (j * kTopkThreads + tid < len) {
          kx = kv > kx ? kv : kx;
          kn = kv < kn ? kv : kn;
        }
      };
      if constexpr (IPT > 0) {
#pragma unroll
        for (int j = 0; j < IPT; ++j) key_extremes(j, widen<T>(reg[j]));
      } else {
        for (int j = 0; j < nruns; ++j) key_extremes(j, score_bits<T>(scores, tid, j));
      }
      kx = (uint32_t)wave_max_i32((int32_t)(kx ^ 0x80000000u));
      kn = (uint32_t)wave_max_i32((int32_t)(~kn ^ 0x80000000u));
      __syncthreads();  // wa, wb have been read
      if (lane == 0) {
        L.wa[wave] = kx;
        L.wb[wave] = kn;
      }
      __syncthreads();
      top = (uint32_t)wave_max_i32((int32_t)L.wa[lane & 15]) ^ 0x80000000u;
      dmax = top - ~((uint32_t)wave_max_i32((int32_t)L.wb[lane & 15]) ^ 0x80000000u);
    } else if (imax >= 0) {
      mode = kMixed;
      top = (uint32_t)imax;
      dmax = umax >= 0x80000000u ? top + (umax - 0x80000000u) : top - umin;
    } else {
      mode = kNeg;
      top = umin;
      dmax = umax - umin;
    }
  }
  // (uniform values: keep them in scalar registers, the rows held in registers need the others)
  mode = __builtin_amdgcn_readfirstlane(mode);
  top = __builtin_amdgcn_readfirstlane(top);
  dmax = __builtin_amdgcn_readfirstlane(dmax);
  // kMixed: d = u + neg_add for u with the sign bit; kNeg: the same form gives u - top
  const uint32_t neg_add = mode == kMixed ? top - 0x80000000u : 0u - top;
  auto to_d = [&](uint32_t u) -> uint32_t {
    if (mode != kCanon) return (int32_t)u >= 0 ? top - u : u + neg_add;
    return top - KeyTraits<F32>::key(__builtin_bit_cast(float, u));
  };
  // The registers go from scores to d inside the first radix level, run by run as the loads arrive
  // (slots past the end of the row: beyond every window).  canon: the canonical keys of a NaN row.
  auto map_run = [&](int j, auto canon) {
    const uint32_t u = widen<T>(reg[j]);
    if constexpr (decltype(canon)::value)
      reg[j] = top - KeyTraits<F32>::key(__builtin_bit_cast(float, u));
    else
      reg[j] = (int32_t)u >= 0 ? top - u : u + neg_add;
    if ((j + 1) * kTopkThreads > len) {  // uniform: only the row's last run has slots past the end
      asm volatile("");
      reg[j] = j * kTopkThreads + tid < len ? reg[j] : kNoElement;
    }
  };
  // f(j, d of element j * 1024 + tid) for the runs j0 <= j < j1 (j uniform); all = true: every
  // run of the row, without the checks (the runs past the end hold nothing)
  auto for_runs = [&](int j0, int j1, auto all, auto f) {
    if constexpr (IPT > 0) {
#pragma unroll
      for (int j8 = 0; j8 < IPT; j8 += kRunGroup) {
        if (j8 < nruns) {  // (rows of a batch can be much shorter than the longest one)
#pragma unroll
          for (int j = j8; j < j8 + kRunGroup; ++j)
            if (decltype(all)::value || (j >= j0 && j < j1)) f(j, reg[j]);
        }
      }
    } else {
      for (int jb = j0; jb < j1; jb += kStream) {
        uint32_t uu[kStream];
#pragma unroll
        for (int u = 0; u < kStream; ++u) uu[u] = score_bits<T>(scores, tid, jb + u);
#pragma unroll
        for (int u = 0; u < kStream; ++u)
          if (jb + u < j1)
            f(jb + u, (jb + u) * kTopkThreads + tid < len ? to_d(uu[u]) : kNoElement);
      }
    }
  };
  const std::true_type every_run;
  const std::false_type some_runs;

  // ---- 2./3. radix levels over the whole row until the threshold bin fits the list --------------
  auto nbits = [](uint32_t x) { return x ? 32 - __builtin_clz(x) : 0; };
  uint32_t lo = 0, krem = (uint32_t)k, tb = 0, n_in = 0;
  int s = nbits(dmax) - 13;
  uint32_t limit = dmax + 1u;  // dmax <= 0xff800000
  if (s < 0) s = 0;
  if (s > 16) {  // the 8191 << 16 smallest d first: 128 bins per binade
    s = 16;
    limit = (uint32_t)(kSliceBins - 1) << 16;
  }
  // The first level always runs (a row of one value, dmax == 0, ends it at once: one bin, s == 0)
  // and is the one place where the registers are written: every later pass only reads them.
  // (Rows of 56 and 64 runs have no registers to spare for the interleaving: they are mapped in a
  // pass of their own before the first level, which then only reads, like the others.)
  constexpr bool kMapInLevel = IPT > 0 && IPT <= 48;
  if constexpr (IPT > 0 && !kMapInLevel) {
    if (mode == kCanon) {
#pragma unroll
      for (int j = 0; j < IPT; ++j) map_run(j, std::true_type());
    } else {
#pragma unroll
      for (int j = 0; j < IPT; ++j) map_run(j, std::false_type());
    }
  }
  auto first_level = [&](auto canon) {
    return slice_level(
        L,
        [&](auto f) {
          if constexpr (kMapInLevel) {
#pragma unroll
            for (int j8 = 0; j8 < IPT; j8 += kRunGroup) {
              if (j8 < nruns) {
#pragma unroll
                for (int j = j8; j < j8 + kRunGroup; ++j) {
                  map_run(j, canon);
                  f(reg[j]);
                }
              }
            }
          } else {
            for_runs(0, nruns, every_run, [&](int, uint32_t d) { f(d); });
          }
        },
        lo, s, limit, krem, tb, n_in, tid, lane, wave);
  };
  bool found = mode == kCanon ? first_level(std::true_type()) : first_level(std::false_type());
  for (;;) {
    if (!found) {  // the threshold lies beyond the window: the rest of the range, as finely as fits
      if (limit > dmax - lo) {
        // The window reached the end of the range and the row still holds fewer than k elements:
        // the caller's bound lies below some score (such scores wrap to d > dmax and are never
        // counted).  The selection is unspecified then; take every element, the writes stop at k.
        lo = kNoElement;
        krem = 0u;
        s = 0;
        break;
      }
      lo += limit;
      const uint32_t rem = dmax - lo;
      s = nbits(rem) - 13;
      if (s < 0) s = 0;
      limit = rem + 1u;
    } else {
      lo += tb << s;
      if (s == 0 || n_in <= (uint32_t)kSliceCand) break;
      limit = 1u << s;  // a crowded bin: its own range, 13 bits further down
      s = s > 13 ? s - 13 : 0;
    }
    found = slice_level(
        L, [&](auto f) { for_runs(0, nruns, every_run, [&](int, uint32_t d) { f(d); }); }, lo, s, limit,
        krem, tb, n_in, tid, lane, wave);
  }
  // the first runs of the own slice once more, as raw bits (they come from L2 while the members are
  // ranked): the emission works on them with constant register numbers
  uint32_t own[kOwn];
#pragma unroll
  for (int jj = 0; jj < kOwn; ++jj) own[jj] = score_bits<T>(scores, tid, j_lo + jj);
  // the threshold is among the n_in elements with d - lo < 2^s, as the krem-th smallest of them
  uint32_t thr = lo, r = krem;  // s == 0: they are all equal
  if (s > 0) {
    // ---- 4. the members into LDS, then rank them ---------------------------------------------------
    if (tid == 0) L.n_cand = 0;
    if (tid < kSliceRank) L.cd[tid] = kNoElement;  // padding: ranks behind every member
    __syncthreads();
    const uint32_t width = 1u << s;
    for_runs(0, nruns, every_run, [&](int j, uint32_t d) {
      const uint64_t m = __ballot(d - lo < width);
      if (m) {  // rare: one LDS reservation per run and wave that holds a member
        uint32_t at = 0;
        if (lane == 0) at = atomicAdd(&L.n_cand, (uint32_t)__popcll(m));
        at = __builtin_amdgcn_readfirstlane(at) + lanes_below(m);
        if ((m >> lane) & 1ull) {
          L.cd[at] = d;
          L.ci[at] = j * kTopkThreads + tid;
        }
      }
    });
    __syncthreads();
    if (n_in <= (uint32_t)kSliceRank) {
      // Every member against every other, without another pass through LDS: each wave holds the
      // whole list in its lanes (members q and q + 64 per lane; the padding ranks behind every
      // member) and ranks the members c = wave, wave + 16, ...: g = members above c, e = equal
      // members at lower positions, both by ballot.  The member with g + e = krem - 1 is the last
      // element taken; exactly one member is, so exactly one wave writes.
      const uint32_t d0 = L.cd[lane], d1 = L.cd[lane + 64];
      const int32_t i0 = L.ci[lane], i1 = L.ci[lane + 64];
      const bool two = n_in > 64u;
      for (int c = wave; c < (int)n_in; c += kTopkWaves) {
        const uint32_t dc = (uint32_t)__builtin_amdgcn_readlane((int)(c < 64 ? d0 : d1), c & 63);
        const int32_t ic = __builtin_amdgcn_readlane(c < 64 ? i0 : i1, c & 63);
        uint32_t g = (uint32_t)__popcll(__ballot(d0 < dc));
        uint32_t e = (uint32_t)__popcll(__ballot(d0 == dc && i0 < ic));
        if (two) {
          g += (uint32_t)__popcll(__ballot(d1 < dc));
          e += (uint32_t)__popcll(__ballot(d1 == dc && i1 < ic));
        }
        if (g + e == krem - 1u && lane == 0) {
          L.sh[0] = dc;
          L.sh[1] = e + 1u;
        }
      }
      __syncthreads();
      thr = __builtin_amdgcn_readfirstlane(L.sh[0]);
      r = __builtin_amdgcn_readfirstlane(L.sh[1]);
    } else {
      // the list stays as it is: every level narrows the window on it
      const int n_list = (int)n_in;
      uint32_t range = width;
      while (s > 0) {
        const int s2 = s > 13 ? s - 13 : 0;
        slice_level(
            L, [&](auto f) { for (int i = tid; i < n_list; i += kTopkThreads) f(L.cd[i]); }, lo, s2,
            range, krem, tb, n_in, tid, lane, wave);
        lo += tb << s2;
        range = 1u << s2;
        s = s2;
      }
      thr = lo;
      r = krem;
    }
  }

  // ---- 5. selected elements in front of this slice and per run of it -----------------------------
  // selected: d < thr, and the first r (in position order) of d == thr
  uint32_t bgt = 0, beq = 0;
  for_runs(0, j_lo, some_runs, [&](int, uint32_t d) {
    bgt += (uint32_t)__popcll(__ballot(d < thr));
    beq += (uint32_t)__popcll(__ballot(d == thr));
  });
  // wa / wb still hold the waves' extremes from step 1: a row of one value (dmax == 0) comes here
  // without passing another barrier, and a slow wave may not have read them yet
  __syncthreads();
  if (lane == 0) {
    L.wa[wave] = bgt;
    L.wb[wave] = beq;
  }
  int32_t* out_idx = p.out_idx + (int64_t)row * p.out_stride;
  elem_t* out_val =
      p.out_values ? reinterpret_cast<elem_t*>(p.out_values) + (int64_t)row * p.out_stride : nullptr;
  if (n_own <= kOwn) {
    // the slice's runs from registers; every wave turns the (run, wave) counts into the offsets of
    // its own 64-element pieces by itself: run jj, wave w is entry 16 jj + w, two entries per lane
    uint32_t od[kOwn];
    if (mode != kCanon) {  // (uniform: one formula per loop, not both and a select per element)
#pragma unroll
      for (int jj = 0; jj < kOwn; ++jj) od[jj] = (int32_t)own[jj] >= 0 ? top - own[jj] : own[jj] + neg_add;
    } else {
#pragma unroll
      for (int jj = 0; jj < kOwn; ++jj)
        od[jj] = top - KeyTraits<F32>::key(__builtin_bit_cast(float, own[jj]));
    }
#pragma unroll
    for (int jj = 0; jj < kOwn; ++jj) {
      if (jj >= n_own) {  // uniform
        od[jj] = kNoElement;
      } else if ((j_lo + jj + 1) * kTopkThreads > len) {  // uniform: the row's last run
        asm volatile("");
        od[jj] = (j_lo + jj) * kTopkThreads + tid < len ? od[jj] : kNoElement;
      }
      const uint32_t ng = (uint32_t)__popcll(__ballot(od[jj] < thr));
      const uint32_t ne = (uint32_t)__popcll(__ballot(od[jj] == thr));
      if (lane == 0) {
        L.run_gt[jj * kTopkWaves + wave] = ng;
        L.run_eq[jj * kTopkWaves + wave] = ne;
      }
    }
    __syncthreads();
    const uint32_t slice_gt = sum_first(L.wa, kTopkWaves, lane);
    const uint32_t slice_eq = sum_first(L.wb, kTopkWaves, lane);
    const uint2 g2 = reinterpret_cast<const uint2*>(L.run_gt)[lane];
    const uint2 e2 = reinterpret_cast<const uint2*>(L.run_eq)[lane];
    // exclusive prefix of the entry this wave reads from the lane: entry 2 lane + (wave & 1)
    uint32_t xg = wave_prefix_sum_dpp(g2.x + g2.y, lane) - g2.y - ((wave & 1) ? 0u : g2.x);
    uint32_t xe = wave_prefix_sum_dpp(e2.x + e2.y, lane) - e2.y - ((wave & 1) ? 0u : e2.x);
#pragma unroll
    for (int jj = 0; jj < kOwn; ++jj) {
      if (jj >= n_own) break;
      const int src = jj * (kTopkWaves / 2) + (wave >> 1);
      const uint32_t eq_before = slice_eq + __builtin_amdgcn_readlane(xe, src);
      const uint32_t out_before =
          slice_gt + __builtin_amdgcn_readlane(xg, src) + (eq_before < r ? eq_before : r);
      const bool eq = od[jj] == thr;
      const uint32_t eq_rank = eq_before + lanes_below(__ballot(eq));
      const bool sel = od[jj] < thr || (eq && eq_rank < r);
      const uint32_t pos = out_before + lanes_below(__ballot(sel));
      if (sel && pos < (uint32_t)k) {
        const int i = (j_lo + jj) * kTopkThreads + tid;
        out_idx[pos] = payload_of(i);
        if (out_val) out_val[pos] = vals[i];
      }
    }
    return;
  }
  // longer slices: counts per (run, wave), one thread per entry for the offsets
  for_runs(j_lo, j_hi, some_runs, [&](int j, uint32_t d) {
    const uint32_t ng = (uint32_t)__popcll(__ballot(d < thr));
    const uint32_t ne = (uint32_t)__popcll(__ballot(d == thr));
    if (lane == 0) {
      L.run_gt[(j - j_lo) * kTopkWaves + wave] = ng;
      L.run_eq[(j - j_lo) * kTopkWaves + wave] = ne;
    }
  });
  __syncthreads();
  {
    const uint32_t slice_gt = sum_first(L.wa, kTopkWaves, lane);
    const uint32_t slice_eq = sum_first(L.wb, kTopkWaves, lane);
    const bool has = tid < n_own * kTopkWaves;
    const uint32_t e = has ? L.run_eq[tid] : 0u, g = has ? L.run_gt[tid] : 0u;
    const uint32_t ie = wave_prefix_sum_dpp(e, lane), ig = wave_prefix_sum_dpp(g, lane);
    __syncthreads();  // wa, wb have been read
    if (lane == 63) {
      L.wa[wave] = ig;
      L.wb[wave] = ie;
    }
    __syncthreads();
    const uint32_t eq_before = slice_eq + sum_first(L.wb, wave, lane) + ie - e;
    const uint32_t gt_before = slice_gt + sum_first(L.wa, wave, lane) + ig - g;
    if (has) {
      L.run_eq[tid] = eq_before;
      L.run_gt[tid] = gt_before + (eq_before < r ? eq_before : r);  // output offset of the run
    }
  }
  __syncthreads();
  for_runs(j_lo, j_hi, some_runs, [&](int j, uint32_t d) {
    const bool eq = d == thr;
    const uint32_t eq_rank = L.run_eq[(j - j_lo) * kTopkWaves + wave] + lanes_below(__ballot(eq));
    const bool sel = d < thr || (eq && eq_rank < r);
    const uint32_t pos = L.run_gt[(j - j_lo) * kTopkWaves + wave] + lanes_below(__ballot(sel));
    if (sel && pos < (uint32_t)k) {
      const int i = j * kTopkThreads + tid;
      out_idx[pos] = payload_of(i);
      if (out_val) out_val[pos] = vals[i];
    }
  });
}

// Slices of a row for the sliced variant: enough workgroups to fill the chip when there are few
// rows, one workgroup per row when there are many (every workgroup of a row repeats the selection
// work on the whole row), whole 1024-element runs per slice.
static void slice_shape(int len, int rows, int& n_slices, int& rps) {
  const int nruns = (len + kTopkThreads - 1) / kTopkThreads;
  int want = 256 / (rows < 1 ? 1 : rows);  // a 1024-thread workgroup has a compute unit to itself
  if (want > nruns / 4) want = nruns / 4;  // at least 4 runs (4096 elements) per slice
  if (want > kCoopMaxSlices) want = kCoopMaxSlices;
  if (want < 1) want = 1;
  rps = (nruns + want - 1) / want;
  if (rps > kSliceMaxRuns) rps = kSliceMaxRuns;  // many long rows: more slices than wanted
  n_slices = (nruns + rps - 1) / rps;
}

template <typename T>
static void launch_topk_sliced(const TopkParams& p, int rows, hipStream_t st) {
  int n_slices, rps;
  slice_shape(p.len, rows, n_slices, rps);
  const dim3 grid((rows + kXcds - 1) / kXcds * n_slices * kXcds), block(kTopkThreads);
  if (p.len <= 8 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 8>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 16 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 16>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 24 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 24>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 32 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 32>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 40 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 40>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 48 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 48>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 56 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 56>), grid, block, 0, st, p, n_slices, rps, rows);
  else if (p.len <= 64 * kTopkThreads)
    hipLaunchKernelGGL((topk_slice_kernel<T, 64>), grid, block, 0, st, p, n_slices, rps, rows);
  else  // longer rows would not fit the registers of a 1024-thread workgroup: re-read per pass
    hipLaunchKernelGGL((topk_slice_kernel<T, 0>), grid, block, 0, st, p, n_slices, rps, rows);
}

// workgroups per row for the cooperative path, 0 if it does not apply
static int coop_slices(int len, int rows) {
  const int g = (len + kCoopSlice - 1) / kCoopSlice;
  if (g < 2 || g > kCoopMaxSlices) return 0;  // short rows: one workgroup is as fast
  return g;
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

extern "C" int td_topk_bounded(const void* values, int32_t values_dtype, int64_t values_stride,
                               int32_t rows, int32_t len, int32_t k, const int32_t* in_idx,
                               int64_t in_idx_stride, const int32_t* page_table,
                               int64_t page_table_stride, int32_t rows_per_table,
                               const int32_t* len_arr, int32_t page_size, const float* row_bound,
                               void* out_values, int32_t* out_idx, int64_t out_stride,
                               void* workspace, int64_t workspace_bytes, void* stream) {
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
  p.row_bound = row_bound;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  TD_REQUIRE(values_dtype == TD_F32 || values_dtype == TD_F16 || values_dtype == TD_BF16,
             "Top-k filtering failed to dispatch with dtype %d", values_dtype);
  // A few long rows: the three cooperative launches split each row over workgroups that share the
  // work through the scratch.  Everything else: one launch in which every workgroup of a row goes
  // through the whole row (rows up to 64K elements from registers) and emits its slice.
  const int slices = coop_slices(len, rows);
  if (len > 64 * kTopkThreads && slices && rows * slices <= 1024 && workspace &&
      workspace_bytes >= (int64_t)rows * kCoopRowWords * 4) {
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
  } else if (values_dtype == TD_F32) {
    launch_topk_sliced<F32>(p, rows, st);
  } else if (values_dtype == TD_F16) {
    launch_topk_sliced<F16>(p, rows, st);
  } else {
    launch_topk_sliced<BF16>(p, rows, st);
  }
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_topk(const void* values, int32_t values_dtype, int64_t values_stride,
                       int32_t rows, int32_t len, int32_t k, const int32_t* in_idx,
                       int64_t in_idx_stride, const int32_t* page_table,
                       int64_t page_table_stride, int32_t rows_per_table, const int32_t* len_arr,
                       int32_t page_size, void* out_values, int32_t* out_idx, int64_t out_stride,
                       void* workspace, int64_t workspace_bytes, void* stream) {
  return td_topk_bounded(values, values_dtype, values_stride, rows, len, k, in_idx, in_idx_stride,
                         page_table, page_table_stride, rows_per_table, len_arr, page_size, nullptr,
                         out_values, out_idx, out_stride, workspace, workspace_bytes, stream);
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
