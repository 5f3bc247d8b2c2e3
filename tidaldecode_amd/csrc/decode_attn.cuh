// Decode attention over a paged KV pool for gfx950 (MI355X): one new query token per sequence
// attends to a listed subset of the cache (sparse layers), or to the whole cache while emitting
// per-token logits (token-selection layers).
//
// Mapping.  A K or V row of one head is head_dim two-byte elements; LPR = head_dim/8 adjacent
// lanes hold it, 16 bytes (one global_load_dwordx4) per lane, so a 64-wide wavefront carries
// HPW = 64/LPR "head rows" at once and never reduces across more than one DPP row for
// head_dim 128.  A workgroup owns one group of HPW head rows and one chunk of the token list;
// its waves take interleaved tiles of U tokens, each wave keeping a private online-softmax
// state in base 2.  Wave states are merged through LDS, workgroup results through a fp32
// partial buffer that the last-arriving workgroup of a head group reduces (ticket counter), or
// that a second small kernel reduces when the plan asks for it.
//
// With grouped-query attention and an index list shared by the query heads of a KV head
// (QPG > 1) each lane group loads the KV row once and scores it against QPG query heads.
// QPG is 2, 4 or 8; other group sizes are padded up (3 -> 4, 5..7 -> 8) or cut into head rows of
// 8 (groups above 8), the padding heads scoring with q = 0 and never being written.
//
// Semantics follow kernels/include/decode/decode_attn.cuh:432-658 of the reference
// (BatchDecodeWithPagedKVCacheKernel) including the forced last page
// (decode_page.cuh:320-346) and the logits output (decode_attn.cuh:107-109).

#pragma once

#include <type_traits>

#include "common.cuh"

namespace tidal {

struct DecodeParams {
  const void* q;
  void* o;
  const void* kv;
  int64_t page_stride;   // elements from page p to page p+1  (2 * P * H_kv * D)
  int64_t v_offset;      // elements from a K row to its V row (P * H_kv * D)
  int32_t entry_stride;  // elements between consecutive tokens of a page
  int32_t head_stride;   // elements between consecutive KV heads of a token
  int32_t page_size;
  int32_t page_shift;  // log2(page_size) or -1
  uint32_t max_slot;   // max_pages * page_size - 1
  int32_t lean;        // 1: power-of-two pages and a pool below 4 GiB (32-bit byte offsets)
  uint32_t page_stride_b, entry_stride_b;  // byte strides for the lean path
  uint32_t max_page;   // max_pages - 1
  int32_t page_mode;   // 1: list entries are pages, 0: token slots
  int32_t num_qo_heads;
  int32_t n_hrows;   // head rows: num_qo_heads (QPG == 1) or num_kv_heads * subs (QPG > 1)
  int32_t q_per_kv;  // query heads per KV head
  int32_t vheads;    // head slots of the split workspace: n_hrows * QPG (QPG may be padded: a group
                     // of 3 runs as 4, 5-7 as 8; the padding heads have q = 0 and are never stored)
  int32_t subs;      // head rows per KV head on the shared-row kernels: groups above 8 are cut
                     // into rows of 8 query heads (the last one padded)
  // index list
  const int32_t* idx;
  int32_t idx_row_stride;  // 0 for a shared row
  int32_t idx_cols;        // elements a row holds (the caller's row stride; 0: unknown): reads stop there
  int32_t idx_per_kv;      // 1: rows are per KV head while QPG == 1
  const int32_t* indptr;
  const int32_t* count_arr;  // per-sequence entry counts of a padded table (else indptr differences)
  int32_t n_list_host;
  const int32_t* last_len_arr;
  const int32_t* last_idx_arr;
  int32_t last_len;
  int32_t last_idx;
  // split
  int32_t chunk_tokens;
  int32_t chunk_shift;  // log2(chunk_tokens) or -1
  int32_t qpk_shift;    // log2(q_per_kv) or -1
  int32_t max_splits;
  int32_t fused_merge;
  float scale_log2;  // sm_scale * log2(e)
  // outputs
  void* scores;
  int32_t scores_f32;
  int64_t score_stride;
  float* lse;
  float* ws_o;      // [batch * H_q * max_splits, D]
  float* ws_ml;     // [batch * H_q * max_splits, 2]
  int32_t* ws_cnt;  // [batch * head rows] ticket counters, ticket_stride words apart
  int32_t ticket_stride;
  // the token being decoded (FRESH kernels): un-rotated k, v, its rotary cos/sin and its slot
  const void* fresh_k;
  const void* fresh_v;
  const float* fresh_cos;
  const float* fresh_sin;
  const int32_t* fresh_slot;
};

template <bool LEAN>
__device__ __forceinline__ void divmod_page(const DecodeParams& p, uint32_t x, uint32_t& page,
                                            uint32_t& entry) {
  if (LEAN || p.page_shift >= 0) {
    page = x >> p.page_shift;
    entry = x & ((1u << p.page_shift) - 1u);
  } else {
    page = x / (uint32_t)p.page_size;
    entry = x - page * (uint32_t)p.page_size;
  }
}

// Per-sequence view of the token list.
struct SeqList {
  const int32_t* row;  // this lane group's index row, already offset to the sequence
  int32_t n_list;      // listed entries (pages or slots)
  int32_t n_items;     // tokens attended
  int32_t last_len;
  int32_t last_idx;
};

// 8-byte device-coherent accesses for the split partials: they are written by one workgroup and
// read by another that may sit on a different XCD (own L2), so they go to memory (sc1) instead
// of relying on an L2-wide write-back fence.
__device__ __forceinline__ void store_coherent(float* dst, float a, float b) {
  const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, a) |
                     ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
  __hip_atomic_store(reinterpret_cast<uint64_t*>(dst), v, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void load_coherent(const float* src, float& a, float& b) {
  const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(src), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
  a = __builtin_bit_cast(float, (uint32_t)v);
  b = __builtin_bit_cast(float, (uint32_t)(v >> 32));
}

// Reduce the n_splits partial results of the QPG query heads of one head row and write o (and
// lse).  Runs in one workgroup of NT threads: NT / (QPG * D / 2) "slots" of threads each own a
// float2 column and a subset of the splits; slots are combined through LDS.
template <typename T, int D, int QPG, int NT>
__device__ __forceinline__ void merge_splits(const DecodeParams& p, int b, int qh0, int rq0, int gsz,
                                             int n_splits) {
  constexpr int COLS = QPG * D / 2;
  constexpr int SLOTS = NT / COLS;
  constexpr int PRE = SLOTS >= 8 ? 4 : (SLOTS >= 4 ? 8 : 16);  // partial loads in flight per thread
  static_assert(SLOTS >= 1, "workgroup too small for the merge");
  __shared__ float mg_m[QPG][64], mg_l[QPG][64];
  __shared__ float mg_part[SLOTS][COLS][2];
  const int tid = threadIdx.x;
  const int c = tid % COLS, slot = tid / COLS;
  const int j = c / (D / 2), d2 = c % (D / 2);
  const int64_t part0 = ((int64_t)b * p.vheads + qh0 + j) * p.max_splits;

  // (m, l) of every split and head: one pair per thread; the load is unconditional (clamped
  // thread index) so that it is in flight together with the partial loads below
  float ml_m, ml_l;
  const bool has_ml = tid < n_splits * QPG;
  {
    const int tc = has_ml ? tid : 0;
    const int jj = tc / n_splits, ss = tc % n_splits;
    load_coherent(p.ws_ml + (((int64_t)b * p.vheads + qh0 + jj) * p.max_splits + ss) * 2,
                  ml_m, ml_l);
  }
  // Loads are unconditional (index clamped, contribution zeroed) so that a batch of PRE of them
  // is in flight per thread; a branch around a load makes the compiler wait for each one.
  float pa[PRE], pb[PRE];
  auto issue = [&](int base) {
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
      int sidx = base + u * SLOTS;
      sidx = sidx < n_splits ? sidx : n_splits - 1;
      load_coherent(p.ws_o + (part0 + sidx) * D + d2 * 2, pa[u], pb[u]);
    }
  };
  if (slot < SLOTS) issue(slot);
  if (has_ml) {
    mg_m[tid / n_splits][tid % n_splits] = ml_m;
    mg_l[tid / n_splits][tid % n_splits] = ml_l;
  }
  __syncthreads();
  float M = kNegBig;
  for (int sidx = 0; sidx < n_splits; ++sidx) M = fmaxf(M, mg_m[j][sidx]);
  float ra = 0.f, rb = 0.f;
  if (slot < SLOTS) {
    for (int base = slot; base < n_splits; base += PRE * SLOTS) {
      if (base != slot) issue(base);
#pragma unroll
      for (int u = 0; u < PRE; ++u) {
        const int sidx = base + u * SLOTS;
        const int sc = sidx < n_splits ? sidx : n_splits - 1;
        const bool live = sidx < n_splits;
        const float f = fast_exp2(mg_m[j][sc] - M);
        ra = fmaf(live ? pa[u] : 0.f, f, ra);
        rb = fmaf(live ? pb[u] : 0.f, f, rb);
      }
    }
    mg_part[slot][c][0] = ra;
    mg_part[slot][c][1] = rb;
  }
  __syncthreads();
  if (tid < COLS && j < gsz) {
    float L = 0.f;
    for (int sidx = 0; sidx < n_splits; ++sidx)
      L = fmaf(mg_l[j][sidx], fast_exp2(mg_m[j][sidx] - M), L);
    float oa = 0.f, ob = 0.f;
#pragma unroll
    for (int sl = 0; sl < SLOTS; ++sl) {
      oa += mg_part[sl][c][0];
      ob += mg_part[sl][c][1];
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    const int qh = rq0 + j;
    reinterpret_cast<uint32_t*>(p.o)[((int64_t)b * p.num_qo_heads + qh) * (D / 2) + d2] =
        pack2<T>(oa * inv, ob * inv);
    if (p.lse && d2 == 0)
      p.lse[(int64_t)b * p.num_qo_heads + qh] = L > 0.f ? (M + fast_log2(L)) * kLn2 : -INFINITY;
  }
}

// Which query heads a head row of a shared-row kernel (QPG > 1) stands for: its KV head, its first
// query head and how many of its QPG head slots are real.
template <int QPG>
__device__ __forceinline__ void head_row_geom(const DecodeParams& p, int hrow, int& kv_head, int& rq0,
                                              int& gsz) {
  if constexpr (QPG > 1) {
    kv_head = hrow / p.subs;
    const int sub = hrow - kv_head * p.subs;
    rq0 = kv_head * p.q_per_kv + sub * QPG;
    const int left = p.q_per_kv - sub * QPG;
    gsz = left < QPG ? left : QPG;
  } else {
    kv_head = hrow / p.q_per_kv;
    rq0 = hrow;
    gsz = 1;
  }
}

// Columns of a sequence's list segment that a kernel may read: the host's bound, cut to the segment
// [list_beg, list_end) when the call has an indptr and to what is left of the row (row_cols columns;
// 0: a row of unknown length).  Device-resident counts are clamped to it.
__device__ __forceinline__ int list_capacity(int n_list_host, bool has_indptr, int list_beg,
                                             int list_end, int row_cols) {
  int cap = n_list_host;
  if (has_indptr) cap = list_end - list_beg < cap ? list_end - list_beg : cap;
  if (row_cols > 0) cap = row_cols - list_beg < cap ? row_cols - list_beg : cap;
  return cap < 0 ? 0 : cap;
}

__device__ __forceinline__ int seq_items(const DecodeParams& p, int b, SeqList& s, int& list_beg) {
  list_beg = 0;
  int list_end = 0;
  if (p.indptr) {
    list_beg = p.indptr[b];
    list_end = p.indptr[b + 1];
    s.n_list = p.count_arr ? p.count_arr[b] : list_end - list_beg;
  } else {
    s.n_list = p.n_list_host;
  }
  const int cap = list_capacity(p.n_list_host, p.indptr != nullptr, list_beg, list_end, p.idx_cols);
  s.n_list = s.n_list < 0 ? 0 : (s.n_list > cap ? cap : s.n_list);
  s.last_len = p.last_len_arr ? p.last_len_arr[b] : p.last_len;
  s.last_idx = p.last_idx_arr ? p.last_idx_arr[b] : p.last_idx;
  // device-resident lengths are not trusted: a fill beyond the page, or more splits than the
  // grid holds, would leave tickets that no workgroup ever takes
  s.last_len = s.last_len < 0 ? 0 : (s.last_len > p.page_size ? p.page_size : s.last_len);
  s.n_items = (p.page_mode ? s.n_list * p.page_size : s.n_list) + s.last_len;
  int n_splits = (s.n_items + p.chunk_tokens - 1) / p.chunk_tokens;
  n_splits = n_splits > p.max_splits ? p.max_splits : n_splits;
  return n_splits < 1 ? 1 : n_splits;
}

template <typename T, int D, int QPG, int U, int NW, bool PAGE_MODE, bool EMIT, bool LEAN, bool FRESH>
__global__ __launch_bounds__(NW * 64) void decode_attn_kernel(const DecodeParams p) {
  static_assert(!FRESH || LEAN, "the fused decode step exists for the lean addressing only");
  constexpr int LPR = D / 8;     // lanes per K/V row
  constexpr int TPI = 64 / LPR;  // tokens one wave instruction covers
  constexpr int TILE = U * TPI;  // tokens per wave tile
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // scalar on purpose: control flow that depends on the wave index must be a real branch, because
  // matrix instructions do not honour the EXEC mask of a masked-off region
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane / LPR;   // lane group = token slot inside the instruction
  const int li = lane % LPR;  // 16-byte column of the row
  // Splits are the slowest grid dimension: a sequence shorter than the planned maximum leaves its
  // last splits without work, and those workgroups then reach the dispatcher after all the others
  // instead of between them (where each one that ends at once hands its place to a workgroup that
  // should have gone to an empty compute unit).
  const int hrow = blockIdx.x;
  const int b = blockIdx.y;
  const int split = blockIdx.z;
  const int qh0 = hrow * QPG;  // first head slot of this head row in the split workspace
  int kv_head, rq0, gsz;       // KV head, first query head, query heads that really exist in the row
  head_row_geom<QPG>(p, hrow, kv_head, rq0, gsz);

  SeqList s;
  int list_beg;
  const int n_splits = seq_items(p, b, s, list_beg);
  if (split >= n_splits) return;  // uniform for the whole workgroup
  const int idx_row = (QPG > 1 || p.idx_per_kv) ? kv_head : hrow;
  s.row = p.idx + (int64_t)idx_row * p.idx_row_stride + list_beg;

  // The splits of a head row interleave: split s takes the workgroup-wide tiles s, s + n_splits,
  // s + 2 n_splits, ... so that all workgroups sweep the sequence together as one moving window
  // (DRAM row locality of a streaming read) instead of as n_splits distant streams.
  const int c1 = s.n_items;

  // query: QPG heads x 8 elements per lane, kept packed in the KV dtype
  uint32_t qp[QPG][4];
  {
    const u32x4* qptr =
        reinterpret_cast<const u32x4*>(p.q) + ((int64_t)b * p.num_qo_heads + rq0) * LPR + li;
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
      const u32x4 v = qptr[(j < gsz ? j : gsz - 1) * LPR];  // unconditional load, clamped row
      const bool real = j < gsz;                            // padding heads score with q = 0
      qp[j][0] = real ? v.x : 0u;
      qp[j][1] = real ? v.y : 0u;
      qp[j][2] = real ? v.z : 0u;
      qp[j][3] = real ? v.w : 0u;
    }
  }

  // Decode-step fusion: q arrives un-rotated and is rotated in registers; the new token's k is
  // rotated here as well, written to its cache slot by one workgroup per KV head, and used from
  // registers wherever the list refers to that slot (the cache write races with nobody: no lane
  // consumes what it loaded from that slot).
  uint32_t knew[4] = {0, 0, 0, 0}, vnew[4] = {0, 0, 0, 0};
  uint32_t new_page = 0xffffffffu, new_entry = 0;
  float rcs[8], rsn[8];  // cos and signed sin of this lane's 8 dimensions
  if constexpr (FRESH) {
    constexpr int HALF = LPR / 2;  // lanes holding the first half of the head dimension
    const uint32_t ns = (uint32_t)p.fresh_slot[b];
    new_page = ns >> p.page_shift;
    new_entry = ns & ((1u << p.page_shift) - 1u);
    const f32x4* cp = reinterpret_cast<const f32x4*>(p.fresh_cos + (int64_t)b * (D / 2) + (li % HALF) * 8);
    const f32x4* sp = reinterpret_cast<const f32x4*>(p.fresh_sin + (int64_t)b * (D / 2) + (li % HALF) * 8);
    const f32x4 c0 = cp[0], c1v = cp[1], s0 = sp[0], s1 = sp[1];
    rcs[0] = c0.x; rcs[1] = c0.y; rcs[2] = c0.z; rcs[3] = c0.w;
    rcs[4] = c1v.x; rcs[5] = c1v.y; rcs[6] = c1v.z; rcs[7] = c1v.w;
    const float sgn = li < HALF ? -1.f : 1.f;  // y_lo = x_lo c - x_hi s,  y_hi = x_hi c + x_lo s
    rsn[0] = sgn * s0.x; rsn[1] = sgn * s0.y; rsn[2] = sgn * s0.z; rsn[3] = sgn * s0.w;
    rsn[4] = sgn * s1.x; rsn[5] = sgn * s1.y; rsn[6] = sgn * s1.z; rsn[7] = sgn * s1.w;
    const int64_t fresh_off =
        ((int64_t)b * (p.num_qo_heads / p.q_per_kv) + kv_head) * LPR + li;
    const u32x4 kn = reinterpret_cast<const u32x4*>(p.fresh_k)[fresh_off];
    const u32x4 vn = reinterpret_cast<const u32x4*>(p.fresh_v)[fresh_off];
    knew[0] = kn.x; knew[1] = kn.y; knew[2] = kn.z; knew[3] = kn.w;
    vnew[0] = vn.x; vnew[1] = vn.y; vnew[2] = vn.z; vnew[3] = vn.w;
  }
  // Rotation of q and of the new key, and the cache write; called once the first K/V tile of
  // the wave is in flight so that these few loads and shuffles hide behind it.
  // rotate-half RoPE of 8 elements per lane; the partner dimension (+- D/2) sits LPR/2 lanes away
  auto rotate = [&](uint32_t(&w)[4]) {
    float x[8], y[8];
#pragma unroll
    for (int c = 0; c < 4; ++c) unpack2<T>(w[c], x[2 * c], x[2 * c + 1]);
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      float partner;
      if constexpr (LPR == 16)
        partner = dpp_move<0x128>(x[d]);  // row_ror:8 == lane ^ 8 inside the 16-lane row
      else if constexpr (LPR == 8)
        partner = lane_xor16<4>(x[d]);
      else
        partner = __shfl_xor(x[d], LPR / 2, 64);
      y[d] = x[d] * rcs[d] + partner * rsn[d];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) w[c] = pack2<T>(y[2 * c], y[2 * c + 1]);
  };
  // (Rotating the new key lazily, only where the list meets the new slot, keeps cos/sin alive
  // through the main loop and costs more registers than it saves instructions.)
  auto finish_fresh = [&]() {
    if constexpr (FRESH) {
#pragma unroll
      for (int j = 0; j < QPG; ++j) rotate(qp[j]);
      rotate(knew);
      const bool writer_row = rq0 == kv_head * p.q_per_kv;  // the KV head's first head row
      if (split == 0 && wave == 0 && g == 0 && writer_row) {
        const uint32_t page_c = new_page > p.max_page ? p.max_page : new_page;
        char* dst = reinterpret_cast<char*>(const_cast<void*>(p.kv)) + page_c * p.page_stride_b +
                    new_entry * p.entry_stride_b + (uint32_t)(kv_head * p.head_stride + li * 8) * 2u;
        u32x4 ko = {knew[0], knew[1], knew[2], knew[3]};
        u32x4 vo = {vnew[0], vnew[1], vnew[2], vnew[3]};
        *reinterpret_cast<u32x4*>(dst) = ko;
        *reinterpret_cast<u32x4*>(dst + p.v_offset * 2) = vo;
      }
    }
  };

  // Shared-row path (QPG > 1): after the reduce-scatter of q.k a lane works on ONE query head,
  // hsel = li % QPG; the running maximum mh of a head is kept equal in all lanes of the wave, lh
  // is the lane group's share of the denominator, and p.V runs on the matrix cores with the 16
  // tokens of a tile as the inner dimension: accm[dd][i] = o[head (4g + i) % QPG][li * 8 + dd].
  // MMA: that path, for head_dim 128 (rows of 16 lanes, tiles of 16 tokens: 4 rows x 4 groups).
  // Other head sizes score their QPG query heads per loaded KV row on the vector ALU throughout.
  constexpr bool MMA = QPG > 1 && LPR == 16;
  static_assert(!MMA || (U == 4 && TPI == 4), "shared-row tiles are 16 tokens: 4 rows x 4 groups");
  float mh = kNegBig, lh = 0.f;
  f32x4 accm[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) accm[d] = f32x4{0.f, 0.f, 0.f, 0.f};

  float m[QPG], l[QPG], acc[QPG][8];
#pragma unroll
  for (int j = 0; j < QPG; ++j) {
    m[j] = kNegBig;
    l[j] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[j][d] = 0.f;
  }

  const int kv_head_off = kv_head * p.head_stride + li * 8;
  const uint16_t* kv16 = reinterpret_cast<const uint16_t*>(p.kv);

  // ---- software pipeline over this wave's tiles ------------------------------------------------
  // program order per iteration: list entries of tile t+2, K/V rows of tile t+1, arithmetic of
  // tile t.  Waiting for older list entries never waits for younger K/V loads, so two tiles of
  // K/V stay in flight per wave.
  u32x4 kA[U], vA[U], kB[U], vB[U];
  int32_t rawA[U], rawB[U];
  uint32_t hitA = 0, hitB = 0;

  // Address generation is branch-free: an item past the end of the chunk is redirected to the
  // chunk's last item (a valid address; its contribution is masked out in the arithmetic) and
  // list reads are clamped into the list.  With power-of-two pages and a pool below 4 GiB
  // (LEAN) the offsets are 32-bit byte offsets from a uniform base and pages are shifts.
  const char* kbase = reinterpret_cast<const char*>(p.kv);
  const char* vbase = kbase + p.v_offset * 2;
  const uint32_t head_byte_off = (uint32_t)kv_head_off * 2u;
  const bool has_list = s.n_list > 0;

  auto fetch_list = [&](int base, int32_t(&raw)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int i = base + u * TPI + g;
      i = i < c1 ? i : c1 - 1;
      uint32_t pos = (uint32_t)i;
      if constexpr (PAGE_MODE) {
        uint32_t e;
        divmod_page<LEAN>(p, (uint32_t)i, pos, e);
      }
      pos = (int32_t)pos < s.n_list ? pos : (uint32_t)(s.n_list - 1);
      raw[u] = has_list ? *reinterpret_cast<const int32_t*>(
                              reinterpret_cast<const char*>(s.row) + (pos << 2))
                        : 0;
    }
  };
  auto issue = [&](int base, const int32_t(&raw)[U], u32x4(&kb)[U], u32x4(&vb)[U], uint32_t& hit) {
    uint32_t page[U], entry[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int i = base + u * TPI + g;
      i = i < c1 ? i : c1 - 1;
      if constexpr (PAGE_MODE) {
        uint32_t pg;
        divmod_page<LEAN>(p, (uint32_t)i, pg, entry[u]);
        page[u] = (int32_t)pg < s.n_list ? (uint32_t)raw[u] : (uint32_t)s.last_idx;
      } else {
        uint32_t slot = i < s.n_list ? (uint32_t)raw[u]
                                     : (uint32_t)s.last_idx * (uint32_t)p.page_size +
                                           (uint32_t)(i - s.n_list);
        slot = slot > p.max_slot ? p.max_slot : slot;
        divmod_page<LEAN>(p, slot, page[u], entry[u]);
      }
      page[u] = page[u] > p.max_page ? p.max_page : page[u];
    }
    hit = 0;
    if constexpr (FRESH) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        hit |= (page[u] == new_page && entry[u] == new_entry) ? (1u << u) : 0u;
    }
    if constexpr (LEAN) {
      uint32_t offs[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        offs[u] = page[u] * p.page_stride_b + entry[u] * p.entry_stride_b + head_byte_off;
        kb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + offs[u]));
      }
      // V after all K: the q.k arithmetic of a tile starts while its V rows are still in flight.
      // K/V rows are read once per launch: non-temporal loads keep them from displacing the lists,
      // q and the split partials in L2 / Infinity Cache (measured: +15 % on the streaming layer).
#pragma unroll
      for (int u = 0; u < U; ++u)
        vb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + offs[u]));
    } else {
      int64_t offs[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        offs[u] = (int64_t)page[u] * p.page_stride + (int64_t)entry[u] * p.entry_stride + kv_head_off;
        kb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kv16 + offs[u]));
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        vb[u] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4*>(kv16 + offs[u] + p.v_offset));
    }
  };
  // ---- logits (EMIT) ------------------------------------------------------------------------------
  // Vector stores and loads share one in-order completion counter, so a store issued per tile
  // holds back the wait for every younger K/V or list load until its write is acknowledged.  The
  // logits are therefore collected in a per-wave LDS strip and written EMIT_TILES tiles at a
  // time: the stores enter the memory queue once per batch (once per launch for most shapes).
  // The later the better: what the writes cost is their HBM traffic in the middle of the read
  // stream (8 sequences x 32 heads x 32K tokens: 33.5 MB of logits beside 4.3 GB of K/V add 87 us to
  // 665; the same stores aimed at one 16 KB window add 5; write-through, non-temporal or
  // contiguous stores change nothing), and a workgroup that writes once, at its end, writes when
  // the others of its round do.  The shared-row kernels have the LDS for that (one workgroup per
  // compute unit): 12 KB per wave hold the 4 x 3328 logits of a 100K-token plan (32/8 heads at
  // 100K tokens: 86 -> 80.6 us with 12 KB per wave instead of 4; 8 x 32K: 214 -> 204).
  constexpr int EMIT_FLOATS = EMIT ? (NW == 16 ? 512 : (QPG > 1 ? 3072 : 1024)) : 1;  // per wave
  constexpr int EMIT_TILES = EMIT ? EMIT_FLOATS / (QPG * TILE) : 1;
  static_assert(EMIT_TILES >= 1, "logit strip too small for one tile");
  __shared__ float emit_buf[EMIT ? NW * EMIT_FLOATS : 1];
  int emit_n = 0;       // tiles waiting in the strip
  int emit_first = 0;   // first token of the oldest waiting tile
  const int emit_step = n_splits * NW * TILE;  // tokens between two tiles of this wave
  auto emit_flush = [&]() {
    if constexpr (EMIT) {
      // The strip was written by other lanes of this wave than the ones that now read it.  LDS
      // accesses of one wave complete in issue order, so the reads below see those writes; the
      // explicit wait and the wave barrier say so to the reader and pin the order for the
      // compiler as well (one wait per flush, that is per 16-64 tiles).
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      // a store instruction covers 64 / TILE tiles of one head: lane -> (tile, token)
      constexpr int TPS = 64 / TILE >= 1 ? 64 / TILE : 1;  // tiles per store (TILE <= 64)
      const int lt = lane / TILE, ltok = lane % TILE;
      for (int n0 = 0; n0 < emit_n; n0 += TPS) {
        const int n = n0 + lt;
        const int i = emit_first + n * emit_step + ltok;
#pragma unroll
        for (int j = 0; j < QPG; ++j) {
          if (n < emit_n && i < c1 && j < gsz) {
            const float nat = emit_buf[((wave * EMIT_TILES + n) * QPG + j) * TILE + ltok];
            const int64_t at = ((int64_t)b * p.num_qo_heads + rq0 + j) * p.score_stride + i;
            if (p.scores_f32)
              reinterpret_cast<float*>(p.scores)[at] = nat;
            else
              reinterpret_cast<uint16_t*>(p.scores)[at] = from_float<T>(nat);
          }
        }
      }
      emit_n = 0;
    }
  };
  auto emit_push = [&](int base) {  // the tile that starts at token `base` is in the strip
    if (emit_n == 0) emit_first = base;
    if (++emit_n == EMIT_TILES) emit_flush();
  };

  auto reduce = [&](u32x4(&kb)[U], u32x4(&vb)[U], int base, uint32_t hit) {
    if constexpr (FRESH) {
      if (__ballot(hit != 0)) {  // rare: some lane group of this wave meets the new token
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if ((hit >> u) & 1u) {
            kb[u].x = knew[0]; kb[u].y = knew[1]; kb[u].z = knew[2]; kb[u].w = knew[3];
            vb[u].x = vnew[0]; vb[u].y = vnew[1]; vb[u].z = vnew[2]; vb[u].w = vnew[3];
          }
        }
      }
    }
    if constexpr (MMA) {
      float sv[U], xe[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float a[QPG];
#pragma unroll
        for (int j = 0; j < QPG; ++j) {
          a[j] = dot2<T>(qp[j][0], kb[u].x, 0.f);
          a[j] = dot2<T>(qp[j][1], kb[u].y, a[j]);
          a[j] = dot2<T>(qp[j][2], kb[u].z, a[j]);
          a[j] = dot2<T>(qp[j][3], kb[u].w, a[j]);
        }
        const float x = reduce_scatter16<QPG>(a, li) * p.scale_log2;  // head li % QPG
        xe[u] = x;
        sv[u] = (base + u * TPI + g < c1) ? x : kNegBig;
      }
      if constexpr (EMIT) {
        // The 16 / QPG lanes of a row that hold the same head hold the same sums, so no value has
        // to move between lanes: copy c = li / QPG of head li % QPG keeps the logit of the tile's
        // row c (token base + c TPI + g).  The logits wait in the wave's LDS strip, laid out
        // [tile][head][token], and leave in batches (see emit_flush).
        constexpr int COPIES = 16 / QPG;
        const int head = li % QPG, c = li / QPG;
        float* strip = emit_buf + (wave * EMIT_TILES + emit_n) * (QPG * TILE);
#pragma unroll
        for (int u0 = 0; u0 < U; u0 += COPIES) {
          float e = xe[u0];
#pragma unroll
          for (int x = 1; x < COPIES; ++x)
            if (u0 + x < U) e = (c == x) ? xe[u0 + x] : e;
          if (u0 + c < U) strip[head * TILE + (u0 + c) * TPI + g] = e * kLn2;
        }
        emit_push(base);
      }
      float mt = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      mt = rows_max(mt);  // the tile's maximum over all four lane groups
      const float m_new = fmaxf(mh, mt);
      const float alpha = fast_exp2(mh - m_new);
      mh = m_new;
      float pr[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        pr[u] = (base + u * TPI + g < c1) ? fast_exp2(sv[u] - m_new) : 0.f;
      // The probabilities enter the matrix product in the KV type; the denominator, which also
      // gives the log-sum-exp, stays in fp32.  bf16 keeps 8 bits of a weight (fp16 11): against an
      // exact denominator that is an error of 2^-9 |v| (2^-12 |v|) in o, which with few selected
      // tokens and |v| of 3-4 reached the tolerance together with the rounding of o itself.  The
      // weights are therefore split into a rounded part and the (rounded) remainder, two products
      // instead of one: twice the bits, and the matrix pipeline has the room.
      const uint32_t p01 = pack2<T>(pr[0], pr[1]), p23 = pack2<T>(pr[2], pr[3]);
      constexpr bool kSplitP = true;
      uint32_t e01 = 0, e23 = 0;
      if constexpr (kSplitP) {
        float r0, r1, r2, r3;
        unpack2<T>(p01, r0, r1);
        unpack2<T>(p23, r2, r3);
        e01 = pack2<T>(pr[0] - r0, pr[1] - r1);
        e23 = pack2<T>(pr[2] - r2, pr[3] - r3);
      }
      lh = fmaf(lh, alpha, (pr[0] + pr[1]) + (pr[2] + pr[3]));
      // rescale the accumulators: row 4g + i belongs to head (4g + i) % QPG; the factors are
      // wave-uniform per head (lane x < QPG holds head x), so they travel through SGPRs
      float ah[QPG];
      bool any = false;
#pragma unroll
      for (int x = 0; x < QPG; ++x) {
        ah[x] = __builtin_bit_cast(
            float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, alpha), x));
        any |= ah[x] != 1.f;
      }
      if (any) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float f;
          if constexpr (QPG == 8)
            f = (g & 1) ? ah[4 + i] : ah[i];
          else
            f = ah[i % QPG];
#pragma unroll
          for (int d = 0; d < 8; ++d) accm[d][i] *= f;
        }
      }
      // B operand of dimension dd: the four rows of the tile held by this lane, one 16-bit value
      // each (v_perm picks the low or the high halves of two dwords)
      const uint32_t vw[U][4] = {{vb[0].x, vb[0].y, vb[0].z, vb[0].w},
                                 {vb[1].x, vb[1].y, vb[1].z, vb[1].w},
                                 {vb[2].x, vb[2].y, vb[2].z, vb[2].w},
                                 {vb[3].x, vb[3].y, vb[3].z, vb[3].w}};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t lo0 = __builtin_amdgcn_perm(vw[1][c], vw[0][c], 0x05040100u);
        const uint32_t lo1 = __builtin_amdgcn_perm(vw[3][c], vw[2][c], 0x05040100u);
        const uint32_t hi0 = __builtin_amdgcn_perm(vw[1][c], vw[0][c], 0x07060302u);
        const uint32_t hi1 = __builtin_amdgcn_perm(vw[3][c], vw[2][c], 0x07060302u);
        accm[2 * c] = mfma_16x16x16<T>(p01, p23, lo0, lo1, accm[2 * c]);
        accm[2 * c + 1] = mfma_16x16x16<T>(p01, p23, hi0, hi1, accm[2 * c + 1]);
        if constexpr (kSplitP) {
          accm[2 * c] = mfma_16x16x16<T>(e01, e23, lo0, lo1, accm[2 * c]);
          accm[2 * c + 1] = mfma_16x16x16<T>(e01, e23, hi0, hi1, accm[2 * c + 1]);
        }
      }
      return;
    }
    float sc[QPG][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + u * TPI + g;
      const bool valid = i < c1;
#pragma unroll
      for (int j = 0; j < QPG; ++j) {
        float a = dot2<T>(qp[j][0], kb[u].x, 0.f);
        a = dot2<T>(qp[j][1], kb[u].y, a);
        a = dot2<T>(qp[j][2], kb[u].z, a);
        a = dot2<T>(qp[j][3], kb[u].w, a);
        a = group_sum<LPR>(a) * p.scale_log2;
        sc[j][u] = valid ? a : kNegBig;
      }
    }
    if constexpr (EMIT) {
      // every lane of a lane group holds the group's U logits, so lane li < U of group g keeps
      // row li (token base + li TPI + g) and nothing moves between lanes; the logits wait in the
      // wave's LDS strip and leave in batches (see emit_flush)
      static_assert(U <= LPR, "one lane of the group per row of the tile");
#pragma unroll
      for (int j = 0; j < QPG; ++j) {  // strip layout [tile][head][token]
        float e = sc[j][0];
#pragma unroll
        for (int u = 1; u < U; ++u) e = (li == u) ? sc[j][u] : e;
        if (li < U)
          emit_buf[((wave * EMIT_TILES + emit_n) * QPG + j) * TILE + li * TPI + g] = e * kLn2;
      }
      emit_push(base);
    }
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
      float mt = sc[j][0];
#pragma unroll
      for (int u = 1; u < U; ++u) mt = fmaxf(mt, sc[j][u]);
      const float m_new = fmaxf(m[j], mt);
      const float alpha = fast_exp2(m[j] - m_new);
      m[j] = m_new;
      float pr[U];
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        pr[u] = (base + u * TPI + g < c1) ? fast_exp2(sc[j][u] - m_new) : 0.f;
        ps += pr[u];
      }
      l[j] = l[j] * alpha + ps;
#pragma unroll
      for (int d = 0; d < 8; ++d) acc[j][d] *= alpha;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float v0, v1, v2, v3, v4, v5, v6, v7;
        unpack2<T>(vb[u].x, v0, v1);
        unpack2<T>(vb[u].y, v2, v3);
        unpack2<T>(vb[u].z, v4, v5);
        unpack2<T>(vb[u].w, v6, v7);
        acc[j][0] = fmaf(pr[u], v0, acc[j][0]);
        acc[j][1] = fmaf(pr[u], v1, acc[j][1]);
        acc[j][2] = fmaf(pr[u], v2, acc[j][2]);
        acc[j][3] = fmaf(pr[u], v3, acc[j][3]);
        acc[j][4] = fmaf(pr[u], v4, acc[j][4]);
        acc[j][5] = fmaf(pr[u], v5, acc[j][5]);
        acc[j][6] = fmaf(pr[u], v6, acc[j][6]);
        acc[j][7] = fmaf(pr[u], v7, acc[j][7]);
      }
    }
  };

  const int STEP = n_splits * NW * TILE;  // tokens between two tiles of one wave
  int t = (split * NW + wave) * TILE;     // first token of this wave's current tile
  if (t < c1) {
    fetch_list(t, rawA);
    if (t + STEP < c1) fetch_list(t + STEP, rawB);
    issue(t, rawA, kA, vA, hitA);
    finish_fresh();
    while (true) {
      // A: K/V of tile t in flight; rawB: list entries of tile t+STEP in flight
      const int tn = t + STEP;
      const int tnn = tn + STEP;
      if (tnn < c1) fetch_list(tnn, rawA);
      if (tn < c1) issue(tn, rawB, kB, vB, hitB);
      reduce(kA, vA, t, hitA);
      if (tn >= c1) break;
      const int tnnn = tnn + STEP;
      if (tnnn < c1) fetch_list(tnnn, rawB);
      if (tnn < c1) issue(tnn, rawA, kA, vA, hitA);
      reduce(kB, vB, tn, hitB);
      if (tnn >= c1) break;
      t = tnn;
    }
  } else {
    finish_fresh();  // a wave without tokens still takes part in the shuffles and the write
  }
  emit_flush();

  // ---- combine the TPI token slots of the wave (butterfly over lane groups) ---------------------
  if constexpr (MMA) {  // the matrix product already summed the groups; only lh is per group
    lh += __shfl_xor(lh, 16, 64);
    lh += __shfl_xor(lh, 32, 64);
  }
#pragma unroll
  for (int j = 0; j < (MMA ? 0 : QPG); ++j) {
    float mw = m[j];
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
    const float f = fast_exp2(m[j] - mw);
    m[j] = mw;
    l[j] *= f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[j][d] *= f;
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
      l[j] += __shfl_xor(l[j], off, 64);
#pragma unroll
      for (int d = 0; d < 8; ++d) acc[j][d] += __shfl_xor(acc[j][d], off, 64);
    }
  }

  // ---- merge the NW wave states of the workgroup through LDS ------------------------------------
  // every wave publishes its QPG states, one barrier, then wave j reduces query head j
  // (QPG <= NW; heads beyond the waves are handled by the waves again in a second trip)
  __shared__ float sm_o[QPG][NW][8][LPR];
  __shared__ float sm_ml[QPG][NW][2];
  __shared__ int sm_ticket;
  if constexpr (MMA) {
#pragma unroll
    for (int j = 0; j < QPG; ++j) {  // head j is row j of the accumulator tile: group j / 4, i = j % 4
      if (g == j / 4) {
#pragma unroll
        for (int d = 0; d < 8; ++d) sm_o[j][wave][d][li] = accm[d][j % 4];
      }
    }
    if (lane < QPG) {
      sm_ml[lane][wave][0] = mh;
      sm_ml[lane][wave][1] = lh;
    }
  } else if (lane < LPR) {
#pragma unroll
    for (int j = 0; j < QPG; ++j) {
#pragma unroll
      for (int d = 0; d < 8; ++d) sm_o[j][wave][d][lane] = acc[j][d];
      if (lane == 0) {
        sm_ml[j][wave][0] = m[j];
        sm_ml[j][wave][1] = l[j];
      }
    }
  }
  __syncthreads();
  for (int j = wave; j < QPG; j += NW) {
    if (lane < LPR) {
      float M = kNegBig;
#pragma unroll
      for (int w = 0; w < NW; ++w) M = fmaxf(M, sm_ml[j][w][0]);
      float L = 0.f, r[8];
#pragma unroll
      for (int d = 0; d < 8; ++d) r[d] = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float f = fast_exp2(sm_ml[j][w][0] - M);
        L = fmaf(sm_ml[j][w][1], f, L);
#pragma unroll
        for (int d = 0; d < 8; ++d) r[d] = fmaf(sm_o[j][w][d][lane], f, r[d]);
      }
      const int qh = rq0 + j;
      if (n_splits == 1) {
        if (j >= gsz) continue;  // a padding head: nothing to write
        const float inv = L > 0.f ? 1.f / L : 0.f;
        u32x4 out;
        out.x = pack2<T>(r[0] * inv, r[1] * inv);
        out.y = pack2<T>(r[2] * inv, r[3] * inv);
        out.z = pack2<T>(r[4] * inv, r[5] * inv);
        out.w = pack2<T>(r[6] * inv, r[7] * inv);
        reinterpret_cast<u32x4*>(p.o)[((int64_t)b * p.num_qo_heads + qh) * LPR + lane] = out;
        if (p.lse && lane == 0)
          p.lse[(int64_t)b * p.num_qo_heads + qh] = L > 0.f ? (M + fast_log2(L)) * kLn2 : -INFINITY;
      } else {
        const int64_t part = ((int64_t)b * p.vheads + qh0 + j) * p.max_splits + split;
        float* dst = p.ws_o + part * D + lane * 8;
        store_coherent(dst + 0, r[0], r[1]);
        store_coherent(dst + 2, r[2], r[3]);
        store_coherent(dst + 4, r[4], r[5]);
        store_coherent(dst + 6, r[6], r[7]);
        if (lane == 0) store_coherent(p.ws_ml + part * 2, M, L);
      }
    }
  }

  if (n_splits == 1 || !p.fused_merge) return;

  // ---- the last workgroup of this (sequence, head row) to arrive reduces the partials ----------
  // Ordering.  The partials were stored with device-scope write-through stores (store_coherent,
  // sc1): such a store is acknowledged -- vmcnt decremented -- only once it has reached memory, the
  // point where all XCDs meet.  Every wave waits for its own stores, the barrier collects the
  // waves, and only then does one thread take the ticket, a device-scope atomic performed at
  // memory.  The workgroup that draws the last ticket therefore knows that every other partial of
  // the head row was acknowledged before its writer's ticket was issued, and it reads them with
  // device-scope loads (load_coherent, sc1) that a cache level private to one XCD cannot serve
  // from a stale line.  What would break this: a plain store or load on ws_o / ws_ml (a test greps
  // for that), the compiler moving the ticket above the wait (hence asm volatile with a memory
  // clobber), or dropping the barrier between the waves' waits and the ticket.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int32_t* ticket = p.ws_cnt + ((int64_t)b * gridDim.x + hrow) * p.ticket_stride;
  if (tid == 0)
    sm_ticket = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (sm_ticket != n_splits - 1) return;
  merge_splits<T, D, QPG, NW * 64>(p, b, qh0, rq0, gsz, n_splits);
  if (tid == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Second-kernel merge (plan.fused_merge == 0): one workgroup per (head row, sequence).
template <typename T, int D, int QPG, int NT>
__global__ __launch_bounds__(NT) void merge_partials_kernel(const DecodeParams p) {
  const int hrow = blockIdx.x;
  const int b = blockIdx.y;
  SeqList s;
  int list_beg;
  const int n_splits = seq_items(p, b, s, list_beg);
  if (n_splits <= 1) return;  // the attention kernel already wrote the final result
  int kv_head, rq0, gsz;
  head_row_geom<QPG>(p, hrow, kv_head, rq0, gsz);
  merge_splits<T, D, QPG, NT>(p, b, hrow * QPG, rq0, gsz, n_splits);
}

// ---------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------

// Instantiated shapes (tile_rows = K/V load instructions per wave tile):
//   one query head per head row: head_dim 64/128/256, 8 waves x {2, 4} rows or 16 waves x 4 rows;
//   2, 4 or 8 query heads per head row (KV rows shared inside a GQA group): head_dim 64 and 128
//   (256: 2 or 4), 8 waves x 4 rows; head_dim 128 on the matrix cores, the others on the vector ALU.
static bool shape_supported(int head_dim, int qpg, int nw, int rows = 4) {
  if (qpg == 1)
    return (head_dim == 64 || head_dim == 128 || head_dim == 256) &&
           ((nw == 8 && (rows == 2 || rows == 4)) || (nw == 16 && rows == 4));
  if (nw != 8 || rows != 4) return false;
  if (head_dim == 256) return qpg == 2 || qpg == 4;  // the split merge holds qpg * head_dim <= 1024
  return (head_dim == 64 || head_dim == 128) && (qpg == 2 || qpg == 4 || qpg == 8);
}

// Query heads scored per loaded KV row.  KV rows are shared between the query heads of a GQA
// group only when the group shares its list and a kernel for that shape exists; otherwise every
// query head walks the list on its own (same result, the KV rows are read once per query head).
static int qpg_for(int num_qo_heads, int num_kv_heads, int idx_rows, int head_dim) {
  const int group = num_qo_heads / num_kv_heads;
  if (group <= 1 || idx_rows == num_qo_heads) return 1;
  // groups of 3 run on the 4-head kernel, 5 to 7 on the 8-head kernel, larger ones as several head
  // rows of 8 (of 4 for head_dim 256): the padding heads cost arithmetic, not memory traffic,
  // which is what bounds these kernels
  int padded = group <= 2 ? 2 : (group <= 4 ? 4 : 8);
  if (head_dim == 256 && padded > 4) padded = 4;
  return shape_supported(head_dim, padded, 8) ? padded : 1;
}

template <typename T, int D, int QPG, int NW, int U, bool PAGE_MODE, bool EMIT>
static void launch_lean(const DecodeParams& p, dim3 grid, hipStream_t st) {
  if (p.lean && p.fresh_k)
    hipLaunchKernelGGL((decode_attn_kernel<T, D, QPG, U, NW, PAGE_MODE, EMIT, true, true>), grid,
                       dim3(NW * 64), 0, st, p);
  else if (p.lean)
    hipLaunchKernelGGL((decode_attn_kernel<T, D, QPG, U, NW, PAGE_MODE, EMIT, true, false>), grid,
                       dim3(NW * 64), 0, st, p);
  else
    hipLaunchKernelGGL((decode_attn_kernel<T, D, QPG, U, NW, PAGE_MODE, EMIT, false, false>), grid,
                       dim3(NW * 64), 0, st, p);
}

template <typename T, int D, int QPG, int NW, int U>
static void launch_variant(const DecodeParams& p, bool page_mode, bool emit, bool merge_kernel,
                           dim3 grid, hipStream_t st) {
  if (page_mode) {
    if (emit)
      launch_lean<T, D, QPG, NW, U, true, true>(p, grid, st);
    else
      launch_lean<T, D, QPG, NW, U, true, false>(p, grid, st);
  } else {
    if (emit)
      launch_lean<T, D, QPG, NW, U, false, true>(p, grid, st);
    else
      launch_lean<T, D, QPG, NW, U, false, false>(p, grid, st);
  }
  if (merge_kernel)
    hipLaunchKernelGGL((merge_partials_kernel<T, D, QPG, 512>), dim3(grid.x, grid.y), dim3(512), 0,
                       st, p);
}

template <typename T>
static int launch_shape(const DecodeParams& p, int head_dim, int qpg, int nw, int rows,
                        bool page_mode, bool emit, bool merge_kernel, dim3 grid, hipStream_t st) {
#define TD_CASE(D_, Q_, N_, U_)                                                    \
  if (head_dim == D_ && qpg == Q_ && nw == N_ && rows == U_) {                     \
    launch_variant<T, D_, Q_, N_, U_>(p, page_mode, emit, merge_kernel, grid, st); \
    return TD_OK;                                                                  \
  }
  TD_CASE(64, 1, 8, 4)
  TD_CASE(64, 1, 8, 2)
  TD_CASE(64, 1, 16, 4)
  TD_CASE(128, 1, 8, 4)
  TD_CASE(128, 1, 8, 2)
  TD_CASE(128, 1, 16, 4)
  TD_CASE(256, 1, 8, 4)
  TD_CASE(256, 1, 8, 2)
  TD_CASE(256, 1, 16, 4)
  TD_CASE(128, 2, 8, 4)
  TD_CASE(128, 4, 8, 4)
  TD_CASE(128, 8, 8, 4)
  TD_CASE(64, 2, 8, 4)
  TD_CASE(64, 4, 8, 4)
  TD_CASE(64, 8, 8, 4)
  TD_CASE(256, 2, 8, 4)
  TD_CASE(256, 4, 8, 4)
#undef TD_CASE
  return fail(TD_ERR_UNSUPPORTED,
              "BatchDecodeWithPagedKVCache failed to dispatch: head_dim %d with %d query heads per "
              "shared KV row and %d waves (supported: head_dim 64/128/256 with per-head lists; "
              "shared lists with 2, 4 or 8 heads per row, 2 or 4 for head_dim 256)",
              head_dim, qpg, nw);
}

// Launches the instantiation for (head_dim, qpg, nw, page_mode, emit); defined once per element
// type in decode_attn_f16.hip / decode_attn_bf16.hip so that the two halves compile in parallel.
int launch_decode_f16(const DecodeParams& p, int head_dim, int qpg, int nw, int rows, bool page_mode,
                      bool emit, bool merge_kernel, dim3 grid, hipStream_t st);
int launch_decode_bf16(const DecodeParams& p, int head_dim, int qpg, int nw, int rows,
                       bool page_mode, bool emit, bool merge_kernel, dim3 grid, hipStream_t st);

}  // namespace tidal
