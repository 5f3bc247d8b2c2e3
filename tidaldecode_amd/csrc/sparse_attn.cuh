// Sparse-layer decode attention for gfx950 (MI355X): the short-list form of decode_attn_kernel,
// for head_dim 128, one query head per head row, token-slot lists, power-of-two pages and a pool
// below 4 GiB.  Same arguments, same split workspace and the same results as decode_attn_kernel;
// what differs is the shape of the work, chosen for launches that move a few tens of MiB and are
// bound by dependent round trips and instruction issue rather than by bandwidth:
//
//   * a wave owns 4 U tokens (U = 8 or 16 K rows and as many V rows per lane: 64 or 128 VGPRs of
//     loads), all of them in flight at once, K rows first so that q.k runs while V arrives;
//   * the list entry of a token is loaded once, by the lane that owns the token; its byte offset
//     reaches the 16 lanes of a row through DPP row broadcasts (one instruction per row);
//   * q.k partial sums are reduce-scattered over the 16 lanes of a row, so that after U partial
//     dot products a lane holds the complete logit of ONE token and the softmax arithmetic runs
//     once per token instead of once per lane; the probabilities go back through row broadcasts;
//   * the maximum is wave-uniform per tile, so the four lane groups add up without rescaling;
//   * the workgroup's waves meet once in LDS, then wave 0 alone publishes the partial, takes the
//     ticket and, if it is the last of its head row, merges the partials (no further barrier).
//
// Semantics follow kernels/include/decode/decode_attn.cuh:432-658 of the reference
// (BatchDecodeWithPagedKVCacheKernel) including the forced last page (decode_page.cuh:320-346).

#pragma once

#include "decode_attn.cuh"

namespace tidal {

// value of lane N of this lane's 16-lane row (DPP row_newbcast)
template <int N>
__device__ __forceinline__ uint32_t row_bcast_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x150 + N, 0xf, 0xf, true);
}
template <int N>
__device__ __forceinline__ float row_bcast_f32(float x) {
  return __builtin_bit_cast(float, row_bcast_u32<N>(__builtin_bit_cast(uint32_t, x)));
}

// a[u] = this lane's partial sum for row u (U rows, U = 8 or 16) over its 8 of the 128 dimensions;
// returns the sum over the 16 lanes of the row group for row (lane % U).  Each butterfly step
// halves the rows a lane keeps and hands the other half to a partner whose lane index differs in
// the step's bit (any partner of the opposite class does, as long as every lane's contribution is
// counted once: xor 1, xor 2, rotate by 4, rotate by 8).
template <int U>
__device__ __forceinline__ float reduce_scatter_rows(float (&a)[U], int li) {
  static_assert(U == 8 || U == 16, "rows per lane group");
  float c1[U / 2], c2[U / 4], c3[U / 8];
  {
    const bool hi = li & 1;
#pragma unroll
    for (int i = 0; i < U / 2; ++i) {
      const float keep = hi ? a[2 * i + 1] : a[2 * i];
      const float send = hi ? a[2 * i] : a[2 * i + 1];
      c1[i] = keep + dpp_move<0xB1>(send);  // quad_perm [1,0,3,2]
    }
  }
  {
    const bool hi = li & 2;
#pragma unroll
    for (int i = 0; i < U / 4; ++i) {
      const float keep = hi ? c1[2 * i + 1] : c1[2 * i];
      const float send = hi ? c1[2 * i] : c1[2 * i + 1];
      c2[i] = keep + dpp_move<0x4E>(send);  // quad_perm [2,3,0,1]
    }
  }
  {
    const bool hi = li & 4;
#pragma unroll
    for (int i = 0; i < U / 8; ++i) {
      const float keep = hi ? c2[2 * i + 1] : c2[2 * i];
      const float send = hi ? c2[2 * i] : c2[2 * i + 1];
      c3[i] = keep + dpp_move<0x124>(send);  // row_ror:4: the sender sits in the other quad class
    }
  }
  if constexpr (U == 16) {
    const bool hi = li & 8;
    const float keep = hi ? c3[1] : c3[0];
    const float send = hi ? c3[0] : c3[1];
    return keep + dpp_move<0x128>(send);  // row_ror:8
  } else {
    return c3[0] + dpp_move<0x128>(c3[0]);  // lanes li and li ^ 8 hold the same row
  }
}

// maximum / sum over the 16 lanes of a row, result in every lane
__device__ __forceinline__ float row16_max(float x) {
  x = fmaxf(x, dpp_move<0xB1>(x));
  x = fmaxf(x, dpp_move<0x4E>(x));
  x = fmaxf(x, dpp_move<0x141>(x));
  x = fmaxf(x, dpp_move<0x140>(x));
  return x;
}

// exchange between the halves / the odd and even 16-lane rows of a wavefront: (a, b) -> x, y with
//   swap32: x = [a.lower | b.lower], y = [a.upper | b.upper]
//   swap16: x = [a.row0 | b.row0 | a.row2 | b.row2], y = [a.row1 | b.row1 | a.row3 | b.row3]
__device__ __forceinline__ void swap32(float a, float b, float& x, float& y) {
  const u32pair r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, a),
                                                     __builtin_bit_cast(uint32_t, b), false, false);
  const uint32_t lo = r.x, hi = r.y;
  x = __builtin_bit_cast(float, lo);
  y = __builtin_bit_cast(float, hi);
}
__device__ __forceinline__ void swap16(float a, float b, float& x, float& y) {
  const u32pair r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, a),
                                                     __builtin_bit_cast(uint32_t, b), false, false);
  const uint32_t lo = r.x, hi = r.y;
  x = __builtin_bit_cast(float, lo);
  y = __builtin_bit_cast(float, hi);
}

// Wave-uniform words of device-resident state, fetched through the scalar cache in one round trip
// (the compiler cannot: the kernel also writes memory, so it would use a vector load and a full
// wait for each word).  The words were written by earlier launches; a launch starts with a clean
// scalar cache.
__device__ __forceinline__ void scalar_load2(const int32_t* a0, const int32_t* a1, int32_t& v0,
                                             int32_t& v1) {
  asm volatile(
      "s_load_dword %0, %2, 0x0\n\t"
      "s_load_dword %1, %3, 0x0\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(v0), "=&s"(v1)
      : "s"(a0), "s"(a1)
      : "memory");
}
__device__ __forceinline__ void scalar_load4(const int32_t* a0, const int32_t* a1, const int32_t* a2,
                                             const int32_t* a3, int32_t& v0, int32_t& v1, int32_t& v2,
                                             int32_t& v3) {
  asm volatile(
      "s_load_dword %0, %4, 0x0\n\t"
      "s_load_dword %1, %5, 0x0\n\t"
      "s_load_dword %2, %6, 0x0\n\t"
      "s_load_dword %3, %7, 0x0\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(v0), "=&s"(v1), "=&s"(v2), "=&s"(v3)
      : "s"(a0), "s"(a1), "s"(a2), "s"(a3)
      : "memory");
}

// The tail of a head's computation, run by ONE wave that holds the workgroup's partial result of
// that head (lane: dimensions 2 lane, 2 lane + 1; M, L uniform): write the result if the head was
// not split, else publish the partial, take the head's ticket and, as the last of the splits to
// arrive, merge all partials.
template <typename T>
__device__ __forceinline__ void finish_head(const DecodeParams& p, int lane, int n_splits, int split,
                                            int64_t part0, int32_t* ticket, uint32_t* o32,
                                            float* lse_out, float o0, float o1, float M, float L) {
  constexpr int D = 128;
  if (n_splits == 1) {
    const float inv = L > 0.f ? 1.f / L : 0.f;
    *o32 = pack2<T>(o0 * inv, o1 * inv);
    if (lse_out && lane == 0) *lse_out = L > 0.f ? (M + fast_log2(L)) * kLn2 : -INFINITY;
    return;
  }
  store_coherent(p.ws_o + (part0 + split) * D + 2 * lane, o0, o1);
  if (lane == 0) store_coherent(p.ws_ml + (part0 + split) * 2, M, L);
  if (!p.fused_merge) return;  // a second launch (merge_partials_kernel) reduces the partials

  // Ordering.  The partial was stored by this wave alone, with device-scope write-through stores
  // (sc1): such a store is acknowledged -- vmcnt decremented -- only once it has reached memory, the
  // point where all XCDs meet, so after s_waitcnt vmcnt(0) the partial is visible device-wide.
  // Only then is the ticket taken; the increment is a device-scope atomic performed at memory,
  // so a wave that draws the last ticket knows that every other partial of the head had been
  // acknowledged before its own ticket was even issued.  It reads them with device-scope loads
  // (sc1), which do not hit lines a non-coherent cache level may still hold from earlier
  // launches.  What would break this: a plain (non-sc1) store or load on ws_o / ws_ml, a compiler
  // that moved the ticket above the wait (hence asm volatile with a memory clobber), or partials
  // stored by several waves without a barrier between their waits and the ticket.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  int tk = 0;
  if (lane == 0) tk = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  tk = __builtin_amdgcn_readfirstlane(tk);
  if (tk != n_splits - 1) return;

  float pm = kNegBig, pl = 0.f;  // (m, l) of split `lane`
  {
    const int sidx = lane < n_splits ? lane : n_splits - 1;
    float a, c;
    load_coherent(p.ws_ml + (part0 + sidx) * 2, a, c);
    if (lane < n_splits) { pm = a; pl = c; }
  }
  constexpr int PRE = 16;  // partial loads in flight
  float pa[PRE], pb[PRE];
  auto issue = [&](int base) {
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
      int sidx = base + u;
      sidx = sidx < n_splits ? sidx : n_splits - 1;
      load_coherent(p.ws_o + (part0 + sidx) * D + 2 * lane, pa[u], pb[u]);
    }
  };
  issue(0);
  const float Mx = rows_max(row16_max(pm));
  const float pf = fast_exp2(pm - Mx);  // scale of split `lane` (0 for lanes past the splits: pl = 0)
  const float Lx = rows_sum(group_sum<16>(pl * pf));
  float ra = 0.f, rb = 0.f;
  for (int base = 0; base < n_splits; base += PRE) {
    if (base) issue(base);
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
      const int sidx = base + u;  // uniform
      if (sidx < n_splits) {
        const float f = __builtin_bit_cast(
            float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pf), sidx));
        ra = fmaf(pa[u], f, ra);
        rb = fmaf(pb[u], f, rb);
      }
    }
  }
  const float inv = Lx > 0.f ? 1.f / Lx : 0.f;
  *o32 = pack2<T>(ra * inv, rb * inv);
  if (lse_out && lane == 0) *lse_out = Lx > 0.f ? (Mx + fast_log2(Lx)) * kLn2 : -INFINITY;
  if (lane == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// QPG query heads per loaded K/V row: 1 (every head row is a query head with its own walk of a
// list) or the 2, 4 or 8 query heads of a KV head that share one list (a head row is a KV head).
template <typename T, int NW, int U, bool FRESH, bool PROBE = false, int QPG = 1, bool WIDE = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(1, U == 16 ? 2 : 4))) void sparse_attn_kernel(const DecodeParams p) {
  static_assert(QPG == 1 || U == 8, "shared KV rows: 8 rows per lane");
  constexpr int D = 128;
  constexpr int LPR = 16;       // lanes per K/V row
  constexpr int TILE = 4 * U;   // tokens of a wave tile: lane group g holds tokens g U .. g U + U - 1
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, li = lane & 15;
  const int hrow = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
  // One batch of scalar loads for every kernel argument the main path uses: the compiler would
  // otherwise fetch them where they are first needed, a dependent round trip each time.
#define TD_TOUCH(x) asm volatile("" ::"s"(x))
  TD_TOUCH(p.q); TD_TOUCH(p.kv); TD_TOUCH(p.v_offset); TD_TOUCH(p.idx); TD_TOUCH(p.indptr);
  TD_TOUCH(p.count_arr); TD_TOUCH(p.last_len_arr); TD_TOUCH(p.last_idx_arr);
  TD_TOUCH(p.idx_row_stride); TD_TOUCH(p.idx_cols); TD_TOUCH(p.n_list_host); TD_TOUCH(p.qpk_shift);
  TD_TOUCH(p.chunk_shift); TD_TOUCH(p.max_splits); TD_TOUCH(p.page_shift); TD_TOUCH(p.max_slot);
  TD_TOUCH(p.page_stride_b); TD_TOUCH(p.entry_stride_b); TD_TOUCH(p.head_stride);
  TD_TOUCH(p.last_len); TD_TOUCH(p.last_idx); TD_TOUCH(p.scale_log2); TD_TOUCH(p.num_qo_heads);
  if constexpr (FRESH) {
    TD_TOUCH(p.fresh_k); TD_TOUCH(p.fresh_v); TD_TOUCH(p.fresh_cos); TD_TOUCH(p.fresh_sin);
    TD_TOUCH(p.fresh_slot);
  }
#undef TD_TOUCH
  // the host sends only power-of-two group sizes here
  const int kv_head = QPG > 1 ? hrow : hrow >> p.qpk_shift;
  const int rq0 = hrow * QPG;              // first query head of the head row
  const int own = g * U + (li & (U - 1));  // the token of the tile this lane owns

  // ---- everything that depends on the kernel arguments only is requested at once ---------------
  // The list entries of the first tile are read before the length of the list is known.  The
  // position is clamped to what the sequence's segment of the row is known to hold whatever the
  // device-resident count says: at most n_list_host columns (which the host has checked against
  // the row stride for a segment that starts at column 0), no further than the segment's end
  // indptr[b + 1], and never beyond the row itself.
  const int t0 = (split * NW + wave) * TILE;
  const int idx_row = (QPG > 1 || p.idx_per_kv) ? kv_head : hrow;
  int list_beg = 0, list_end = 0;
  if (p.indptr) scalar_load2(p.indptr + b, p.indptr + b + 1, list_beg, list_end);
  const int32_t* row = p.idx + (int64_t)idx_row * p.idx_row_stride + list_beg;
  const int cap = list_capacity(p.n_list_host, p.indptr != nullptr, list_beg, list_end, p.idx_cols);
  auto fetch_entry = [&](int t) -> int32_t {
    int pos = t + own;
    pos = pos < cap ? pos : cap - 1;
    return cap > 0 ? row[pos] : 0;
  };
  int32_t ent = fetch_entry(t0);

  // ---- q, and in the fused decode step (FRESH) what the workgroup's first wave prepares ----------
  // FRESH: q arrives un-rotated.  Wave 0 of the workgroup alone loads q, the step's cos / sin and
  // the new token's k and v, rotates q and k once, and leaves rotated q, rotated k and v in LDS for
  // the other waves (which then issue no global load besides their list entry and K/V rows: eight
  // waves per workgroup asking the same few cache lines for cos / sin cost the launch 0.5 us).
  uint32_t qp[QPG][4];
  const bool prep = FRESH && wave == 0;  // scalar
  if constexpr (!FRESH) {
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
      const u32x4 v =
          reinterpret_cast<const u32x4*>(p.q)[((int64_t)b * p.num_qo_heads + rq0 + j) * LPR + li];
      qp[j][0] = v.x; qp[j][1] = v.y; qp[j][2] = v.z; qp[j][3] = v.w;
    }
  }
  // What wave 0 loads for the fused step.  Defined in that wave only and read in that wave only:
  // giving the other waves a value here would make them wait for their list entry first (the
  // registers are the destination of loads in flight on the other side of the branch).
  u32x4 q_raw[QPG], kn_raw, vn_raw;
  f32x4 cos_lo, cos_hi, sin_lo, sin_hi;
  if constexpr (FRESH) {
    if (prep) {
#pragma unroll
      for (int j = 0; j < QPG; ++j)
        q_raw[j] = reinterpret_cast<const u32x4*>(p.q)[((int64_t)b * p.num_qo_heads + rq0 + j) * LPR + li];
      constexpr int HALF = LPR / 2;
      const f32x4* cp = reinterpret_cast<const f32x4*>(p.fresh_cos + (int64_t)b * (D / 2) + (li % HALF) * 8);
      const f32x4* sp = reinterpret_cast<const f32x4*>(p.fresh_sin + (int64_t)b * (D / 2) + (li % HALF) * 8);
      cos_lo = cp[0]; cos_hi = cp[1]; sin_lo = sp[0]; sin_hi = sp[1];
      const int n_kv = QPG > 1 ? p.num_qo_heads / QPG : p.num_qo_heads >> p.qpk_shift;
      const int64_t fresh_off = ((int64_t)b * n_kv + kv_head) * LPR + li;
      kn_raw = reinterpret_cast<const u32x4*>(p.fresh_k)[fresh_off];
      vn_raw = reinterpret_cast<const u32x4*>(p.fresh_v)[fresh_off];
    }
  }

  // ---- the sequence: listed entries, forced last page, splits ------------------------------------
  // (seq_items of decode_attn.cuh with the division by the chunk size as a shift)
  SeqList s;
  s.n_list = p.n_list_host;
  s.last_len = p.last_len;
  s.last_idx = p.last_idx;
  // slot of the token being decoded (FRESH): it travels with the other state words, load and wait
  // inside one asm statement, so that no register allocation can read it before it has landed; the
  // list entry, which the row loads wait for anyway, is in flight over the same round trip
  uint32_t new_slot = 0xffffffffu;
  if (FRESH || p.count_arr || p.last_len_arr || p.last_idx_arr) {
    // absent arrays read a dummy word (q is never NULL) and keep the host value
    const int32_t* dummy = reinterpret_cast<const int32_t*>(p.q);
    int32_t cnt, ll, lx, ns;
    scalar_load4(p.count_arr ? p.count_arr + b : dummy, p.last_len_arr ? p.last_len_arr + b : dummy,
                 p.last_idx_arr ? p.last_idx_arr + b : dummy, FRESH ? p.fresh_slot + b : dummy, cnt, ll,
                 lx, ns);
    if (p.indptr) s.n_list = p.count_arr ? cnt : list_end - list_beg;
    if (p.last_len_arr) s.last_len = ll;
    if (p.last_idx_arr) s.last_idx = lx;
    if constexpr (FRESH) new_slot = (uint32_t)ns;
  } else if (p.indptr) {
    s.n_list = list_end - list_beg;
  }
  // a count beyond what the first fetch was clamped to would pair tokens with the wrong entries
  s.n_list = s.n_list < 0 ? 0 : (s.n_list > cap ? cap : s.n_list);
  s.last_len = s.last_len < 0 ? 0 : (s.last_len > p.page_size ? p.page_size : s.last_len);
  const int c1 = s.n_list + s.last_len;
  int n_splits = (c1 + p.chunk_tokens - 1) >> p.chunk_shift;
  n_splits = n_splits > p.max_splits ? p.max_splits : n_splits;
  n_splits = n_splits < 1 ? 1 : n_splits;
  if (split >= n_splits) return;  // uniform for the workgroup
  const uint32_t last_base = (uint32_t)s.last_idx * (uint32_t)p.page_size;

  const char* kbase = reinterpret_cast<const char*>(p.kv);
  const char* vbase = kbase + p.v_offset * 2;
  const uint32_t head_byte_off = (uint32_t)(kv_head * p.head_stride + li * 8) * 2u;
  const uint32_t entry_mask = (1u << (p.page_shift & 31)) - 1u;
  // Byte offset of a token slot's K row of head 0 in the pool.  Lean form: power-of-two pages, a
  // pool below 4 GiB and strides that fit the 24-bit multiplier.  Wide form: any page size (one
  // division per lane and tile) and 64-bit offsets.
  using off_t = typename std::conditional<WIDE, uint64_t, uint32_t>::type;
  auto slot_offset = [&](uint32_t slot) -> off_t {
    if constexpr (WIDE) {
      uint32_t page, entry;
      if (p.page_shift >= 0) {
        page = slot >> p.page_shift;
        entry = slot & entry_mask;
      } else {
        page = slot / (uint32_t)p.page_size;
        entry = slot - page * (uint32_t)p.page_size;
      }
      return (uint64_t)page * (uint64_t)p.page_stride_b + (uint64_t)(entry * p.entry_stride_b);
    } else {
      return __umul24(slot >> p.page_shift, p.page_stride_b) + __umul24(slot & entry_mask, p.entry_stride_b);
    }
  };

  float m_run = kNegBig;  // wave-uniform running maximum (base-2 logits)
  float l_lane = 0.f;     // this lane's share of the denominator
  float acc[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) acc[d] = 0.f;
  // Shared KV rows (QPG > 1): per-head maxima and denominators, and p.V on the matrix cores:
  // accm[e][r] = o[head 4 g + r][li 8 + e], already summed over the four lane groups.
  float mh[QPG], lh[QPG];
#pragma unroll
  for (int j = 0; j < QPG; ++j) { mh[j] = kNegBig; lh[j] = 0.f; }
  f32x4 accm[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) accm[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  __shared__ __attribute__((aligned(16))) float sm_p[QPG > 1 ? NW * QPG * TILE : 4];
  // fused decode step: rotated q rows, the new token's rotated key and its value, 256 bytes each
  __shared__ __attribute__((aligned(16))) uint32_t sm_fresh[FRESH ? (QPG + 2) * 64 : 4];
  uint32_t* const sm_knew = sm_fresh + (FRESH ? QPG * 64 : 0);
  uint32_t* const sm_vnew = sm_knew + (FRESH ? 64 : 0);

  // ---- one tile of the wave: slot and row offset of the lane's own token, then every K and V row ----
  u32x4 kb[U], vb[U];
  uint32_t slot = 0;   // of this lane's token
  bool valid = false;  // the token exists
  auto issue = [&](int t, int32_t entry_raw) {
    const int i = t + own;
    valid = i < c1;
    // entry_raw was read at min(i, capacity - 1), which is i for every listed token (n_list <= capacity)
    slot = i < s.n_list ? (uint32_t)entry_raw : last_base + (uint32_t)(i - s.n_list);
    slot = slot > p.max_slot ? p.max_slot : slot;
    off_t off_own = slot_offset(slot);
    // lanes past the end of the list repeat the first token of the tile (which exists: t < c1)
    // with weight 0: a row that holds real data, whatever the unused list entries say
    if constexpr (WIDE) {
      const uint32_t lo = (uint32_t)off_own, hi = (uint32_t)(off_own >> 32);
      const uint32_t lo0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)lo);
      const uint32_t hi0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)hi);
      const uint32_t lo_own = valid ? lo : lo0, hi_own = valid ? hi : hi0;
      const char* ka[U];
#define TD_ROW_OFF(N)                                                                              \
  if constexpr (N < U)                                                                             \
    ka[N] = kbase + ((((uint64_t)row_bcast_u32<N>(hi_own)) << 32) | (uint64_t)row_bcast_u32<N>(lo_own)) + \
            head_byte_off;
      TD_ROW_OFF(0) TD_ROW_OFF(1) TD_ROW_OFF(2) TD_ROW_OFF(3) TD_ROW_OFF(4) TD_ROW_OFF(5)
      TD_ROW_OFF(6) TD_ROW_OFF(7) TD_ROW_OFF(8) TD_ROW_OFF(9) TD_ROW_OFF(10) TD_ROW_OFF(11)
      TD_ROW_OFF(12) TD_ROW_OFF(13) TD_ROW_OFF(14) TD_ROW_OFF(15)
#undef TD_ROW_OFF
#pragma unroll
      for (int u = 0; u < U; ++u)
        kb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ka[u]));
#pragma unroll
      for (int u = 0; u < U; ++u)
        vb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ka[u] + p.v_offset * 2));
    } else {
      off_own = valid ? off_own : (uint32_t)__builtin_amdgcn_readfirstlane((int)off_own);
      uint32_t offs[U];
#define TD_ROW_OFF(N) \
  if constexpr (N < U) offs[N] = row_bcast_u32<N>(off_own) + head_byte_off;
      TD_ROW_OFF(0) TD_ROW_OFF(1) TD_ROW_OFF(2) TD_ROW_OFF(3) TD_ROW_OFF(4) TD_ROW_OFF(5)
      TD_ROW_OFF(6) TD_ROW_OFF(7) TD_ROW_OFF(8) TD_ROW_OFF(9) TD_ROW_OFF(10) TD_ROW_OFF(11)
      TD_ROW_OFF(12) TD_ROW_OFF(13) TD_ROW_OFF(14) TD_ROW_OFF(15)
#undef TD_ROW_OFF
#pragma unroll
      for (int u = 0; u < U; ++u)
        kb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + offs[u]));
#pragma unroll
      for (int u = 0; u < U; ++u)
        vb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + offs[u]));
    }
  };

  // ---- arithmetic of the tile whose rows `issue` asked for ----------------------------------------
  auto compute = [&](bool first_tile) {
    if constexpr (PROBE) {  // measurement: the loads alone, no arithmetic and no merge
      u32x4 fold = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int u = 0; u < U; ++u) fold ^= kb[u] ^ vb[u];
      uint32_t w = fold.x ^ fold.y ^ fold.z ^ fold.w;
      if (w == 0x12345678u) reinterpret_cast<uint32_t*>(p.o)[0] = w;
      return;
    }
    // The token being decoded is used from LDS (where wave 0 left it) wherever the list names its
    // slot: what the pool holds there is being written by another workgroup of this launch.
    if constexpr (FRESH) {
      bool hit = slot == new_slot;
      const uint32_t hit_first = __builtin_amdgcn_readfirstlane(hit ? 1u : 0u);
      hit = valid ? hit : (hit_first != 0);  // lanes without a token hold a copy of the first lane's rows
      if (__ballot(hit)) {
        const u32x4 kn = *reinterpret_cast<const u32x4*>(sm_knew + li * 4);
        const u32x4 vn = *reinterpret_cast<const u32x4*>(sm_vnew + li * 4);
        const uint32_t hm = hit ? 1u : 0u;
#define TD_ROW_FIX(N)                   \
  if constexpr (N < U) {                \
    if (row_bcast_u32<N>(hm)) {         \
      kb[N] = kn;                       \
      vb[N] = vn;                       \
    }                                   \
  }
        TD_ROW_FIX(0) TD_ROW_FIX(1) TD_ROW_FIX(2) TD_ROW_FIX(3) TD_ROW_FIX(4) TD_ROW_FIX(5)
        TD_ROW_FIX(6) TD_ROW_FIX(7) TD_ROW_FIX(8) TD_ROW_FIX(9) TD_ROW_FIX(10) TD_ROW_FIX(11)
        TD_ROW_FIX(12) TD_ROW_FIX(13) TD_ROW_FIX(14) TD_ROW_FIX(15)
#undef TD_ROW_FIX
      }
    }

    if constexpr (QPG > 1) {
      // The lane ends with the logits of ITS token for all QPG heads; maxima per head are made
      // wave-uniform.  The weights then go through a strip of LDS private to the wave into the
      // A-operand layout of a 16x16x16 matrix product (row = head, inner index = the 16 tokens
      // 4c..4c+3 of the four lane groups), B = the four V rows a lane holds, one 16-bit element each.
      constexpr bool kSplit = std::is_same<T, BF16>::value;  // bf16 weights travel as value + remainder
      float* sp = sm_p + wave * (QPG * TILE);
      float alpha[QPG];
#pragma unroll
      for (int j = 0; j < QPG; ++j) {
        float part[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float a = dot2<T>(qp[j][0], kb[u].x, 0.f);
          a = dot2<T>(qp[j][1], kb[u].y, a);
          a = dot2<T>(qp[j][2], kb[u].z, a);
          part[u] = dot2<T>(qp[j][3], kb[u].w, a);
        }
        const float red = reduce_scatter_rows<U>(part, li);
        const float sv = valid ? red * p.scale_log2 : kNegBig;
        const float m_new = fmaxf(mh[j], rows_max(row16_max(sv)));
        alpha[j] = fast_exp2(mh[j] - m_new);
        mh[j] = m_new;
        const float pr = valid ? fast_exp2(sv - m_new) : 0.f;
        lh[j] = lh[j] * alpha[j] + (li < 8 ? pr : 0.f);  // lanes li and li ^ 8 hold the same token
        if (li < 8) sp[j * TILE + own] = pr;
      }
      if (!first_tile) {  // later tiles: rescale what the earlier ones left (row r of group g: head 4 g + r)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float f = (QPG == 8 && g == 1) ? alpha[(4 + r) % QPG] : alpha[r % QPG];
#pragma unroll
          for (int e = 0; e < 8; ++e) accm[e][r] *= f;
        }
      }
      // the strip was written by other lanes of this wave: LDS accesses of a wave complete in
      // issue order; the wait and the wave barrier pin that order for the compiler too
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int c = 0; c < U / 4; ++c) {
        f32x4 pa = *reinterpret_cast<const f32x4*>(sp + (li < QPG ? li : 0) * TILE + g * U + 4 * c);
        if (li >= QPG) pa = f32x4{0.f, 0.f, 0.f, 0.f};  // rows past the heads of the group
        const uint32_t ah0 = pack2<T>(pa.x, pa.y), ah1 = pack2<T>(pa.z, pa.w);
        uint32_t al0 = 0, al1 = 0;
        if constexpr (kSplit) {
          float r0, r1, r2, r3;
          unpack2<T>(ah0, r0, r1);
          unpack2<T>(ah1, r2, r3);
          al0 = pack2<T>(pa.x - r0, pa.y - r1);
          al1 = pack2<T>(pa.z - r2, pa.w - r3);
        }
        const uint32_t vw[4][4] = {
            {vb[4 * c].x, vb[4 * c].y, vb[4 * c].z, vb[4 * c].w},
            {vb[4 * c + 1].x, vb[4 * c + 1].y, vb[4 * c + 1].z, vb[4 * c + 1].w},
            {vb[4 * c + 2].x, vb[4 * c + 2].y, vb[4 * c + 2].z, vb[4 * c + 2].w},
            {vb[4 * c + 3].x, vb[4 * c + 3].y, vb[4 * c + 3].z, vb[4 * c + 3].w}};
#pragma unroll
        for (int w2 = 0; w2 < 4; ++w2) {
          const uint32_t lo0 = __builtin_amdgcn_perm(vw[1][w2], vw[0][w2], 0x05040100u);
          const uint32_t lo1 = __builtin_amdgcn_perm(vw[3][w2], vw[2][w2], 0x05040100u);
          const uint32_t hi0 = __builtin_amdgcn_perm(vw[1][w2], vw[0][w2], 0x07060302u);
          const uint32_t hi1 = __builtin_amdgcn_perm(vw[3][w2], vw[2][w2], 0x07060302u);
          accm[2 * w2] = mfma_16x16x16<T>(ah0, ah1, lo0, lo1, accm[2 * w2]);
          accm[2 * w2 + 1] = mfma_16x16x16<T>(ah0, ah1, hi0, hi1, accm[2 * w2 + 1]);
          if constexpr (kSplit) {
            accm[2 * w2] = mfma_16x16x16<T>(al0, al1, lo0, lo1, accm[2 * w2]);
            accm[2 * w2 + 1] = mfma_16x16x16<T>(al0, al1, hi0, hi1, accm[2 * w2 + 1]);
          }
        }
      }
      asm volatile("" ::: "memory");  // the strip is rewritten by the next tile only after these reads
      return;
    }
    // q.k: U partial sums per lane, reduce-scattered so that the lane ends with its own token
    float part[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float a = dot2<T>(qp[0][0], kb[u].x, 0.f);
      a = dot2<T>(qp[0][1], kb[u].y, a);
      a = dot2<T>(qp[0][2], kb[u].z, a);
      part[u] = dot2<T>(qp[0][3], kb[u].w, a);
    }
    const float red = reduce_scatter_rows<U>(part, li);  // every lane takes part: no branch around it
    const float sv = valid ? red * p.scale_log2 : kNegBig;
    const float m_new = fmaxf(m_run, rows_max(row16_max(sv)));
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    const float pr = valid ? fast_exp2(sv - m_new) : 0.f;
    // with U == 8 the lanes li and li ^ 8 hold the same token: it counts once
    l_lane = l_lane * alpha + ((U == 16 || li < 8) ? pr : 0.f);
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[d] *= alpha;
#define TD_ROW_PV(N)                                        \
  if constexpr (N < U) {                                    \
    const float pu = row_bcast_f32<N>(pr);                  \
    float v0, v1, v2, v3, v4, v5, v6, v7;                   \
    unpack2<T>(vb[N].x, v0, v1);                            \
    unpack2<T>(vb[N].y, v2, v3);                            \
    unpack2<T>(vb[N].z, v4, v5);                            \
    unpack2<T>(vb[N].w, v6, v7);                            \
    acc[0] = fmaf(pu, v0, acc[0]);                          \
    acc[1] = fmaf(pu, v1, acc[1]);                          \
    acc[2] = fmaf(pu, v2, acc[2]);                          \
    acc[3] = fmaf(pu, v3, acc[3]);                          \
    acc[4] = fmaf(pu, v4, acc[4]);                          \
    acc[5] = fmaf(pu, v5, acc[5]);                          \
    acc[6] = fmaf(pu, v6, acc[6]);                          \
    acc[7] = fmaf(pu, v7, acc[7]);                          \
  }
    TD_ROW_PV(0) TD_ROW_PV(1) TD_ROW_PV(2) TD_ROW_PV(3) TD_ROW_PV(4) TD_ROW_PV(5) TD_ROW_PV(6)
    TD_ROW_PV(7) TD_ROW_PV(8) TD_ROW_PV(9) TD_ROW_PV(10) TD_ROW_PV(11) TD_ROW_PV(12)
    TD_ROW_PV(13) TD_ROW_PV(14) TD_ROW_PV(15)
#undef TD_ROW_PV
  };

  // ---- the wave's tiles: rows of the first one are asked for before anything else happens --------
  const int STEP = n_splits * NW * TILE;
  int t = t0;
  bool live = t < c1;  // wave-uniform
  if (!prep && live) issue(t, ent);

  if constexpr (FRESH) {
    // Wave 0 rotates q and the new key while the other waves' rows are in flight (its own are asked
    // for right after: what it loaded for the rotation has arrived with its list entry, and the
    // registers are free again before its K/V rows need them) and leaves them and the new value in
    // LDS; the cache write of the new token follows after the tiles, from LDS.
    if (prep) {
      const float rcs[8] = {cos_lo.x, cos_lo.y, cos_lo.z, cos_lo.w, cos_hi.x, cos_hi.y, cos_hi.z, cos_hi.w};
      const float sgn = li < LPR / 2 ? -1.f : 1.f;  // y_lo = x_lo c - x_hi s,  y_hi = x_hi c + x_lo s
      const float rsn[8] = {sgn * sin_lo.x, sgn * sin_lo.y, sgn * sin_lo.z, sgn * sin_lo.w,
                            sgn * sin_hi.x, sgn * sin_hi.y, sgn * sin_hi.z, sgn * sin_hi.w};
      // rotate-half RoPE of 8 elements per lane; the partner dimension (+- 64) sits 8 lanes away
      auto rotate = [&](uint32_t(&w)[4]) {
        float x[8], y[8];
#pragma unroll
        for (int c = 0; c < 4; ++c) unpack2<T>(w[c], x[2 * c], x[2 * c + 1]);
#pragma unroll
        for (int d = 0; d < 8; ++d) y[d] = x[d] * rcs[d] + dpp_move<0x128>(x[d]) * rsn[d];
#pragma unroll
        for (int c = 0; c < 4; ++c) w[c] = pack2<T>(y[2 * c], y[2 * c + 1]);
      };
      uint32_t knew[4] = {kn_raw.x, kn_raw.y, kn_raw.z, kn_raw.w};
      rotate(knew);
      if (g == 0) {
        *reinterpret_cast<u32x4*>(sm_knew + li * 4) = u32x4{knew[0], knew[1], knew[2], knew[3]};
        *reinterpret_cast<u32x4*>(sm_vnew + li * 4) = vn_raw;
      }
#pragma unroll
      for (int j = 0; j < QPG; ++j) {
        uint32_t qj[4] = {q_raw[j].x, q_raw[j].y, q_raw[j].z, q_raw[j].w};
        rotate(qj);
        if (g == 0) *reinterpret_cast<u32x4*>(sm_fresh + j * 64 + li * 4) = u32x4{qj[0], qj[1], qj[2], qj[3]};
      }
      if (live) issue(t, ent);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the LDS writes have landed
    }
    // a bare barrier: the fence of __syncthreads would wait for the rows in flight
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // every wave, the first included: registers that no global load of either branch is still
    // writing to, so that the wait the compiler puts in front of this read is for LDS only
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(sm_fresh + j * 64 + li * 4);
      qp[j][0] = v.x; qp[j][1] = v.y; qp[j][2] = v.z; qp[j][3] = v.w;
    }
  }

  // the first tile apart from the loop: its rows were asked for above, and the loop then keeps no
  // K/V registers alive from one pass to the next
  if (live) {
    compute(true);
    for (t += STEP; t < c1; t += STEP) {
      issue(t, fetch_entry(t));
      compute(false);
    }
  }
  if constexpr (FRESH) {
    // One workgroup per KV head writes the new token into the cache, from the copy in LDS and after
    // the tiles: a store in front of them would have the tiles' first register writes wait for it.
    // Nobody in this launch reads that slot from memory.
    if (prep && split == 0 && (QPG > 1 || hrow == (kv_head << p.qpk_shift)) && g == 0) {
      const uint32_t ns = new_slot > p.max_slot ? p.max_slot : new_slot;
      char* dst = reinterpret_cast<char*>(const_cast<void*>(p.kv)) + slot_offset(ns) + head_byte_off;
      *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(sm_knew + li * 4);
      *reinterpret_cast<u32x4*>(dst + p.v_offset * 2) = *reinterpret_cast<const u32x4*>(sm_vnew + li * 4);
    }
  }

  if constexpr (PROBE) return;
  __shared__ __attribute__((aligned(16))) float sm_o[NW][QPG][D];
  __shared__ float sm_ml[NW][QPG][2];
  if constexpr (QPG > 1) {
    // the matrix product already summed the lane groups: the lanes of group g hold heads 4g..4g+3
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int head = 4 * g + r;
      if (head < QPG) {
        *reinterpret_cast<f32x4*>(&sm_o[wave][head][li * 8]) =
            f32x4{accm[0][r], accm[1][r], accm[2][r], accm[3][r]};
        *reinterpret_cast<f32x4*>(&sm_o[wave][head][li * 8 + 4]) =
            f32x4{accm[4][r], accm[5][r], accm[6][r], accm[7][r]};
      }
    }
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
      const float lw = rows_sum(group_sum<16>(lh[j]));
      if (lane == 0) {
        sm_ml[wave][j][0] = mh[j];
        sm_ml[wave][j][1] = lw;
      }
    }
  } else {
    // ---- the four lane groups of the wave: the maximum is shared, so the sums simply add --------
    // reduce-scatter over the groups: lane (g, li) ends with dimensions li 8 + g 2 + {0, 1}
    float r0, r1;
    {
      float x, y, h[4];
#pragma unroll
      for (int i2 = 0; i2 < 4; ++i2) {
        swap32(acc[i2], acc[i2 + 4], x, y);
        h[i2] = x + y;  // lower half: dimension i2, upper half: dimension i2 + 4
      }
      swap16(h[0], h[2], x, y);
      r0 = x + y;
      swap16(h[1], h[3], x, y);
      r1 = x + y;
    }
    const float l_w = rows_sum(group_sum<16>(l_lane));
    *reinterpret_cast<f32x2*>(&sm_o[wave][0][li * 8 + g * 2]) = f32x2{r0, r1};
    if (lane == 0) {
      sm_ml[wave][0][0] = m_run;
      sm_ml[wave][0][1] = l_w;
    }
  }
  // ---- the waves of the workgroup meet in LDS; wave j carries on alone with head j --------------
  __syncthreads();
  for (int j = wave; j < QPG; j += NW) {
    float M = kNegBig;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_ml[w][j][0]);
    float L = 0.f, o0 = 0.f, o1 = 0.f;  // this lane: dimensions 2 lane, 2 lane + 1
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = fast_exp2(sm_ml[w][j][0] - M);
      L = fmaf(sm_ml[w][j][1], f, L);
      const f32x2 v = *reinterpret_cast<const f32x2*>(&sm_o[w][j][2 * lane]);
      o0 = fmaf(v.x, f, o0);
      o1 = fmaf(v.y, f, o1);
    }
    const int qh = rq0 + j;
    uint32_t* o32 = reinterpret_cast<uint32_t*>(p.o) + ((int64_t)b * p.num_qo_heads + qh) * (D / 2) + lane;
    float* lse_out = p.lse ? p.lse + (int64_t)b * p.num_qo_heads + qh : nullptr;
    const int64_t part0 = ((int64_t)b * p.vheads + qh) * p.max_splits;
    int32_t* ticket = p.ws_cnt + (((int64_t)b * gridDim.x + hrow) * QPG + j) * p.ticket_stride;
    finish_head<T>(p, lane, n_splits, split, part0, ticket, o32, lse_out, o0, o1, M, L);
  }
}

// Shapes of the sparse-layer kernel: waves per workgroup x K (and V) rows per lane; with shared
// KV rows (2, 4 or 8 query heads per list walk) 8 rows per lane.
static bool sparse_shape_supported(int nw, int rows, int qpg = 1) {
  if (qpg == 1) return (nw == 4 || nw == 8) && (rows == 8 || rows == 16);
  return (qpg == 2 || qpg == 4 || qpg == 8) && (nw == 4 || nw == 8) && rows == 8;
}

// `wide`: 64-bit row offsets and pages of any size (8 rows per lane only)
template <typename T>
static int launch_sparse(const DecodeParams& p, int nw, int rows, bool probe, bool wide, dim3 grid,
                         hipStream_t st) {
#define TD_SPARSE_CASE(N_, U_)                                                                   \
  if (nw == N_ && rows == U_ && !wide) {                                                         \
    if (probe)                                                                                   \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, U_, false, true>), grid, dim3(N_ * 64), 0,   \
                         st, p);                                                                 \
    else if (p.fresh_k)                                                                          \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, U_, true>), grid, dim3(N_ * 64), 0, st, p);  \
    else                                                                                         \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, U_, false>), grid, dim3(N_ * 64), 0, st, p); \
    return TD_OK;                                                                                \
  }
  TD_SPARSE_CASE(8, 8)
  TD_SPARSE_CASE(4, 8)
  TD_SPARSE_CASE(4, 16)
  TD_SPARSE_CASE(8, 16)
#undef TD_SPARSE_CASE
#define TD_SPARSE_CASE(N_)                                                                          \
  if (nw == N_ && rows == 8 && wide) {                                                              \
    if (probe)                                                                                      \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, 8, false, true, 1, true>), grid, dim3(N_ * 64), \
                         0, st, p);                                                                 \
    else if (p.fresh_k)                                                                             \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, 8, true, false, 1, true>), grid, dim3(N_ * 64), \
                         0, st, p);                                                                 \
    else                                                                                            \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, 8, false, false, 1, true>), grid,               \
                         dim3(N_ * 64), 0, st, p);                                                  \
    return TD_OK;                                                                                   \
  }
  TD_SPARSE_CASE(8)
  TD_SPARSE_CASE(4)
#undef TD_SPARSE_CASE
  return fail(TD_ERR_UNSUPPORTED, "sparse decode attention: no kernel for %d waves x %d rows%s", nw, rows,
              wide ? " with 64-bit offsets" : "");
}

// shared KV rows: QPG query heads per list walk
template <typename T>
static int launch_sparse_shared(const DecodeParams& p, int nw, int qpg, bool wide, dim3 grid, hipStream_t st) {
#define TD_SPARSE_CASE(N_, Q_, W_)                                                                  \
  if (nw == N_ && qpg == Q_ && wide == W_) {                                                        \
    if (p.fresh_k)                                                                                  \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, 8, true, false, Q_, W_>), grid, dim3(N_ * 64),  \
                         0, st, p);                                                                 \
    else                                                                                            \
      hipLaunchKernelGGL((sparse_attn_kernel<T, N_, 8, false, false, Q_, W_>), grid, dim3(N_ * 64), \
                         0, st, p);                                                                 \
    return TD_OK;                                                                                   \
  }
  TD_SPARSE_CASE(4, 2, false)
  TD_SPARSE_CASE(4, 4, false)
  TD_SPARSE_CASE(4, 8, false)
  TD_SPARSE_CASE(8, 2, false)
  TD_SPARSE_CASE(8, 4, false)
  TD_SPARSE_CASE(8, 8, false)
  TD_SPARSE_CASE(4, 2, true)
  TD_SPARSE_CASE(4, 4, true)
  TD_SPARSE_CASE(4, 8, true)
  TD_SPARSE_CASE(8, 2, true)
  TD_SPARSE_CASE(8, 4, true)
  TD_SPARSE_CASE(8, 8, true)
#undef TD_SPARSE_CASE
  return fail(TD_ERR_UNSUPPORTED,
              "sparse decode attention: no kernel for %d waves with %d query heads per shared row", nw, qpg);
}

// Launches the sparse-layer kernel (and, when the plan asks for it, the second-launch merge);
// defined once per element type (and once more for shared KV rows) in sparse_attn_*.hip.
int launch_sparse_f16(const DecodeParams& p, int nw, int rows, bool probe, bool wide, bool merge_kernel,
                      dim3 grid, hipStream_t st);
int launch_sparse_bf16(const DecodeParams& p, int nw, int rows, bool probe, bool wide, bool merge_kernel,
                       dim3 grid, hipStream_t st);
int launch_sparse_shared_f16(const DecodeParams& p, int nw, int qpg, bool wide, bool merge_kernel, dim3 grid,
                             hipStream_t st);
int launch_sparse_shared_bf16(const DecodeParams& p, int nw, int qpg, bool wide, bool merge_kernel, dim3 grid,
                              hipStream_t st);

}  // namespace tidal
