// Host side of the decode-attention entry points: split planning and argument checks.  The
// kernels live in decode_attn.cuh and are instantiated in decode_attn_{f16,bf16}.hip.
#include "sparse_attn.cuh"

namespace tidal {

static int g_num_cus = 0;

static int num_cus() {
  if (g_num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        n > 0)
      g_num_cus = n;
    else
      g_num_cus = 256;  // MI355X
  }
  return g_num_cus;
}

static int64_t align256(int64_t x) { return (x + 255) & ~(int64_t)255; }

// Workspace layout: [ticket counters, fixed size | partial o | partial (m, l)].  The counters sit
// at a fixed place so that plans of different shapes sharing one workspace never find another
// plan's partial results where they expect zeroed tickets.  A counter has 64 bytes to itself: the
// tickets of a launch are all taken within a microsecond, and counters that share a line queue up
// behind one another at the memory channel (measured: 0.4 us of a 9.7 us launch).
constexpr int kTicketStride = 16;  // int32 words between counters
constexpr int64_t kTicketBytes = (int64_t)16384 * kTicketStride * 4;

// The short-list kernel (sparse_attn.cuh) covers a list in one pass of at most 64 workgroups per
// head; longer lists go to the streaming kernel, whose waves pipeline several tiles.
constexpr int64_t kSparseMaxItems = 64 * 256;

static bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

}  // namespace tidal

// Scratch of td_decode_attn_noalloc: ticket counters and split partials in device memory that
// belongs to the library image, for callers that must not allocate.  Zero when the image is
// loaded; every launch leaves the ticket counters zero again.
static __device__ __align__(256) unsigned char scratch[TD_STATIC_SCRATCH_BYTES];

namespace tidal {

// Device address of `scratch` on the current device.  The array's name is a host-side handle, not
// a device address: the address is looked up once per device (each device holds its own copy)
// and that pointer is what the launches get.
static int static_scratch(void** out) {
  constexpr int kMaxDevices = 64;
  static void* ptr_of[kMaxDevices] = {};
  int dev = 0;
  TD_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(TD_ERR_UNSUPPORTED, "td_decode_attn_noalloc: device %d (at most %d devices)", dev, kMaxDevices);
  void* ptr = __atomic_load_n(&ptr_of[dev], __ATOMIC_ACQUIRE);
  if (ptr == nullptr) {
    TD_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(TD_ERR_HIP, "hipGetSymbolAddress returned a NULL scratch address");
    __atomic_store_n(&ptr_of[dev], ptr, __ATOMIC_RELEASE);
  }
  *out = ptr;
  return TD_OK;
}

}  // namespace tidal

using namespace tidal;

// kernel family that served this thread's last td_decode_attn call
static thread_local const char* g_last_kernel = "none";

extern "C" const char* td_last_decode_kernel(void) { return g_last_kernel; }

extern "C" int td_num_cus(void) { return num_cus(); }

extern "C" int td_decode_make_plan(int32_t batch, int32_t num_qo_heads, int32_t num_kv_heads,
                              int32_t head_dim, int32_t idx_rows, int64_t max_items,
                              td_decode_plan* plan) {
  TD_REQUIRE(plan != nullptr, "td_decode_make_plan: plan is NULL");
  TD_REQUIRE(batch >= 1, "td_decode_make_plan: batch %d < 1", batch);
  TD_REQUIRE(num_kv_heads >= 1 && num_qo_heads >= num_kv_heads && num_qo_heads % num_kv_heads == 0,
             "td_decode_make_plan: num_qo_heads %d must be a positive multiple of num_kv_heads %d",
             num_qo_heads, num_kv_heads);
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(TD_ERR_UNSUPPORTED, "td_decode_make_plan: head_dim %d (supported: 64, 128, 256)",
                head_dim);
  TD_REQUIRE(idx_rows == 1 || idx_rows == num_kv_heads || idx_rows == num_qo_heads,
             "td_decode_make_plan: idx_rows %d must be 1, num_kv_heads (%d) or num_qo_heads (%d)",
             idx_rows, num_kv_heads, num_qo_heads);
  TD_REQUIRE(max_items >= 0 && max_items < ((int64_t)1 << 30), "td_decode_make_plan: max_items %lld",
             (long long)max_items);

  const int qpg = qpg_for(num_qo_heads, num_kv_heads, idx_rows, head_dim);
  const int subs = qpg > 1 ? (num_qo_heads / num_kv_heads + qpg - 1) / qpg : 1;
  const int n_hrows = qpg > 1 ? num_kv_heads * subs : num_qo_heads;
  {
    // Planning happens before the launches it serves (and outside any stream capture): a good
    // moment to look up this device's static scratch for td_decode_attn_noalloc.  Without a
    // device the lookup fails and is simply tried again by that entry point.
    void* unused = nullptr;
    (void)static_scratch(&unused);
  }

  // ---- short lists: the sparse-layer kernel -------------------------------------------------------
  // Chunks are a power of two (the kernel divides by shifting) and a multiple of the workgroup
  // tile; the streaming kernel at 8 waves x 4 rows (tile 128) can run the same plan when a call
  // turns out not to fit the short-list kernel (page lists, score output, large pools).
  int sw = plan->sparse_waves, sr = plan->sparse_rows;
  // one query head per list walk with a power-of-two group size, or exactly 2, 4 or 8 query heads
  // sharing their KV head's list (no padding heads)
  const int group = num_qo_heads / num_kv_heads;
  const bool heads_fit = qpg == 1 ? is_pow2(group) : (qpg == group && subs == 1);
  bool sparse = sw >= 0 && sr >= 0 && head_dim == 128 && heads_fit && max_items > 0 &&
                max_items <= kSparseMaxItems &&
                (plan->chunk_tokens == 0 || is_pow2(plan->chunk_tokens));
  if (qpg > 1 && sr == 16) sparse = false;  // shared rows: 8 rows per lane only
  if (sparse) {
    // Chunk: the smallest power of two from 128 tokens up that leaves at most 9/8 workgroups per
    // compute unit.  Where even 512 tokens leave more than that (batches), the chunk grows on for
    // as long as a full round of workgroups remains: fewer, longer workgroups then beat more
    // partials to merge (8 sequences x 32 heads, lists of 1024: 27.0 us at 512 tokens, 25.3 at
    // 1024; lists of 2048: 50.3 -> 47.5 at 2048; lists of 4096: 94.2 -> 90.4 at 4096; 16 sequences
    // x 1024: 51.0 -> 49.4; a round that is not full loses: 4 sequences x 1024 at 1024 tokens are
    // 128 workgroups and 20.3 us against 16.7).  Workgroup shape: 4 waves for 128-token chunks, 8
    // waves otherwise, 8 K rows per lane.
    int64_t chunk = plan->chunk_tokens;
    if (chunk == 0) {
      chunk = 128;
      const int64_t rows_all = (int64_t)n_hrows * batch;
      while (chunk < 512 && rows_all * ceil_div64(max_items, chunk) > num_cus() * 9 / 8) chunk <<= 1;
      while (rows_all * ceil_div64(max_items, chunk) > num_cus() * 9 / 8 && chunk < max_items &&
             rows_all * ceil_div64(max_items, chunk * 2) >= num_cus())
        chunk <<= 1;
      // Between one and 1.75 eight-wave workgroups of 256 tokens per compute unit neither 256 nor
      // 512 tokens fill the chip evenly (36 heads x 2048 tokens: 288 workgroups, 32 compute units
      // get a second one; 40 and 48 heads at 512 tokens: 160 and 192 workgroups for 256 compute
      // units).  Four-wave workgroups of 128 tokens spread better there (measured, 2048 tokens:
      // 36 heads 13.4 -> 12.0 us, 40 heads 12.95 -> 12.4, 48 heads 13.8 -> 13.2; no gain at 24,
      // 32, 56 and 64 heads, which keep their plan).
      const int64_t w256 = (int64_t)n_hrows * batch * ceil_div64(max_items, 256);
      if (sw == 0 && (sr == 0 || sr == 8) && w256 > num_cus() && w256 * 4 < (int64_t)num_cus() * 7 &&
          ceil_div64(max_items, 128) <= 64)
        chunk = 128;
    }
    while (ceil_div64(max_items, chunk) > 64) chunk <<= 1;
    if (sr == 0) sr = 8;
    if (sw == 0) sw = (chunk < 256 || sr == 16) ? 4 : 8;
    if (!sparse_shape_supported(sw, sr, qpg))
      return fail(TD_ERR_UNSUPPORTED,
                  "td_decode_make_plan: no short-list kernel with %d waves x %d rows (4 or 8 waves, 8 or "
                  "16 rows)", sw, sr);
    const int stile = sw * 4 * sr;
    if (plan->chunk_tokens == 0 && chunk < stile) chunk = stile;  // a preset shape with a larger tile
    if (chunk % stile != 0 || chunk % 128 != 0) {
      sparse = false;
    } else {
      plan->chunk_tokens = (int32_t)chunk;
      plan->max_splits = (int32_t)ceil_div64(max_items, chunk);
      plan->waves_per_block = 8;
      plan->tile_rows = 4;
      plan->sparse_waves = sw;
      plan->sparse_rows = sr;
    }
  }
  if (sparse) {
    if (plan->fused_merge < 0) plan->fused_merge = 1;
    plan->fused_merge = plan->fused_merge ? 1 : 0;
    TD_REQUIRE((int64_t)batch * n_hrows * qpg * kTicketStride * 4 <= kTicketBytes,
               "td_decode_make_plan: batch %d x %d heads exceeds the %lld ticket counters", batch,
               n_hrows * qpg, (long long)(kTicketBytes / (kTicketStride * 4)));
    const int64_t n_part = (int64_t)batch * n_hrows * qpg * plan->max_splits;
    plan->workspace_bytes = kTicketBytes + align256(n_part * head_dim * 4) + align256(n_part * 2 * 4);
    return TD_OK;
  }
  plan->sparse_waves = plan->sparse_rows = 0;

  int nw = plan->waves_per_block;
  if (nw == 0) nw = 8;
  if (qpg > 1) nw = 8;  // the shared-row kernels exist for 8 waves only
  // K/V rows per lane group and tile of the streaming kernel: 4 unless the caller presets 2
  // (short token-slot lists have a kernel of their own, above).
  int rows = plan->tile_rows;
  if (rows == 0) rows = 4;
  if (!shape_supported(head_dim, qpg, nw, rows))
    return fail(TD_ERR_UNSUPPORTED,
                "td_decode_make_plan: no kernel for head_dim %d, %d query heads per shared KV row, %d "
                "waves per block, %d rows per tile",
                head_dim, qpg, nw, rows);
  // tokens one pass of the workgroup covers: waves x instructions x rows per instruction
  const int tile = nw * rows * (64 / (head_dim / 8));

  // Aim at one round of workgroups that fills the chip, never less than one pass per workgroup,
  // never more than 64 partials per head.  The one-head-per-row kernels fit two 8-wave workgroups
  // on a compute unit (128 registers: four waves per SIMD), so their round is 2 per compute unit.
  // The shared-row kernels (141-256 registers) fit ONE: with twice as many workgroups the second
  // half waits for the first, and a few workgroups over one round double the launch (32/8 heads
  // x 128 at 100K tokens: 31 splits = 248 workgroups 84 us, 62 splits = 496 workgroups 90 us,
  // 34 splits = 272 workgroups 120 us; at 32K 33 us against 41, at 10K 18 against 26).  Their
  // round is kept a little under the compute-unit count: 256 workgroups on 256 compute units
  // measured like a round and a bit (124 us), 248 and fewer did not.
  const int64_t target_blocks = qpg > 1 ? (int64_t)num_cus() - num_cus() / 32 : (int64_t)num_cus() * 2;
  int64_t splits = target_blocks / ((int64_t)n_hrows * batch);
  if (splits < 1) splits = 1;
  if (splits > 64) splits = 64;
  int64_t chunk = max_items > 0 ? ceil_div64(max_items, splits) : tile;
  // A batch is planned from its longest sequence: chunks of that size leave the short sequences
  // with one long-running workgroup per head and the launch waits for the longest.  Finer chunks
  // balance a ragged batch (8 sequences of 14K-63K tokens: 935 -> 769 us).
  if (batch > 1 && qpg == 1 && chunk > 4096) chunk = 4096;
  // Shared rows in a batch: whole rounds of one workgroup per compute unit.  The split count with
  // the fewest rounds per split wins, chunks of 1024 tokens at least
  // (32/8 heads, 16 sequences x 8192 tokens: 2 splits = 256 workgroups 94 us, 3 splits 110, 1
  // split 130; 8 x 32768: 4 splits 172 us, 3 splits 187, 8 splits of 4096 tokens 182; 12 x 16384:
  // 5 splits = 2 rounds 136 us, 8 splits = 3 rounds 136, 4 splits 151, 3 splits 187).
  if (batch > 1 && qpg > 1 && max_items > 0) {
    const int64_t r = (int64_t)n_hrows * batch, cus = num_cus();
    int64_t s_max = max_items / 1024;
    s_max = s_max < 1 ? 1 : (s_max > 64 ? 64 : s_max);
    int64_t best_s = 1, best_rounds = ceil_div64(r, cus);
    for (int64_t s_try = 2; s_try <= s_max; ++s_try) {
      const int64_t rounds = ceil_div64(r * s_try, cus);
      // more splits in as many rounds always gain; more rounds have to gain 1/16 per split
      const bool better = rounds <= best_rounds ? rounds * best_s < best_rounds * s_try
                                                : rounds * best_s * 16 < best_rounds * s_try * 15;
      if (better) {
        best_s = s_try;
        best_rounds = rounds;
      }
    }
    chunk = ceil_div64(max_items, best_s);
  }
  if (plan->chunk_tokens > 0) chunk = plan->chunk_tokens;
  chunk = ceil_div64(chunk, tile) * tile;
  int64_t max_splits = max_items > 0 ? ceil_div64(max_items, chunk) : 1;
  if (max_splits > 64) {  // keep the merge bounded: widen the chunks
    chunk = ceil_div64(ceil_div64(max_items, 64), tile) * tile;
    max_splits = ceil_div64(max_items, chunk);
  }
  if (max_splits < 1) max_splits = 1;

  plan->chunk_tokens = (int32_t)chunk;
  plan->max_splits = (int32_t)max_splits;
  plan->waves_per_block = nw;
  plan->tile_rows = rows;
  if (plan->fused_merge < 0) plan->fused_merge = 1;
  plan->fused_merge = plan->fused_merge ? 1 : 0;
  TD_REQUIRE((int64_t)batch * n_hrows * kTicketStride * 4 <= kTicketBytes,
             "td_decode_make_plan: batch %d x %d head rows exceeds the %lld ticket counters", batch,
             n_hrows, (long long)(kTicketBytes / (kTicketStride * 4)));
  const int64_t n_part = (int64_t)batch * n_hrows * qpg * max_splits;  // head slots incl. padding
  plan->workspace_bytes = kTicketBytes + align256(n_part * head_dim * 4) + align256(n_part * 2 * 4);
  return TD_OK;
}

// Argument checks and the kernel parameter block shared by td_decode_attn and td_gather_probe.
static int build_params(const td_paged_kv* kv, const td_index_list* list, const td_decode_plan* plan,
                        const void* q, void* o, int32_t batch, int32_t num_qo_heads, float sm_scale,
                        void* scores, int32_t scores_dtype, int64_t score_stride, float* lse,
                        const td_fresh_token* fresh, void* workspace, int64_t workspace_bytes,
                        DecodeParams& p, int& qpg_out, int& n_hrows_out) {
  TD_REQUIRE(kv && list && plan && q && o, "td_decode_attn: NULL argument");
  TD_REQUIRE(kv->data != nullptr, "td_decode_attn: kv->data is NULL");
  TD_REQUIRE(batch >= 1, "td_decode_attn: batch %d < 1", batch);
  const int Hkv = kv->num_kv_heads, D = kv->head_dim, P = kv->page_size;
  if (D != 64 && D != 128 && D != 256)
    return fail(TD_ERR_UNSUPPORTED,
                "BatchDecodeWithPagedKVCache failed to dispatch: head_dim %d (supported: 64, 128, 256)",
                D);
  TD_REQUIRE(Hkv >= 1 && num_qo_heads >= Hkv && num_qo_heads % Hkv == 0,
             "td_decode_attn: num_qo_heads %d must be a positive multiple of num_kv_heads %d",
             num_qo_heads, Hkv);
  TD_REQUIRE(P >= 1 && kv->max_pages >= 1, "td_decode_attn: page_size %d / max_pages %lld", P,
             (long long)kv->max_pages);
  TD_REQUIRE(kv->max_pages * P < ((int64_t)1 << 31), "td_decode_attn: pool too large for int32 slots");
  TD_REQUIRE(kv->layout == TD_NHD || kv->layout == TD_HND, "td_decode_attn: layout %d", kv->layout);
  if (kv->dtype != TD_F16 && kv->dtype != TD_BF16)
    return fail(TD_ERR_UNSUPPORTED,
                "BatchDecodeWithPagedKVCache failed to dispatch with dtype %d (supported: fp16, bf16)",
                kv->dtype);
  TD_REQUIRE(list->idx_rows == 1 || list->idx_rows == Hkv || list->idx_rows == num_qo_heads,
             "td_decode_attn: idx_rows %d must be 1, %d or %d", list->idx_rows, Hkv, num_qo_heads);
  TD_REQUIRE(list->kind == TD_IDX_PAGES || list->kind == TD_IDX_SLOTS, "td_decode_attn: kind %d",
             list->kind);
  TD_REQUIRE(list->n_list_host >= 0, "td_decode_attn: n_list_host %d", list->n_list_host);
  TD_REQUIRE(list->count_arr == nullptr || list->indptr != nullptr,
             "td_decode_attn: count_arr needs indptr (the first column of every sequence)");
  TD_REQUIRE(list->idx != nullptr || list->n_list_host == 0,
             "td_decode_attn: idx is NULL but n_list_host is %d", list->n_list_host);
  TD_REQUIRE(list->idx_rows == 1 || list->idx_row_stride >= list->n_list_host,
             "td_decode_attn: idx_row_stride %d < n_list_host %d", list->idx_row_stride,
             list->n_list_host);
  TD_REQUIRE(list->last_page_len >= 0 && list->last_page_len <= P,
             "td_decode_attn: last_page_len %d not in [0, %d]", list->last_page_len, P);
  TD_REQUIRE(list->last_page_idx >= 0 && list->last_page_idx < kv->max_pages,
             "td_decode_attn: last_page_idx %d outside the pool of %lld pages", list->last_page_idx,
             (long long)kv->max_pages);
  TD_REQUIRE(plan->chunk_tokens > 0 && plan->max_splits >= 1 && plan->waves_per_block > 0 &&
                 plan->tile_rows > 0 &&
                 plan->chunk_tokens % (plan->waves_per_block * plan->tile_rows * (64 / (D / 8))) == 0,
             "td_decode_attn: plan not produced by td_decode_make_plan");
  // the planned split must cover every token the list can describe
  const int64_t max_items = (int64_t)list->n_list_host * (list->kind == TD_IDX_PAGES ? P : 1) +
                            (list->last_page_len_arr ? P : list->last_page_len);
  if (max_items > (int64_t)plan->chunk_tokens * plan->max_splits)
    return fail(TD_ERR_STATE,
                "td_decode_attn: the list describes up to %lld tokens but the plan covers %lld "
                "(call td_decode_make_plan / begin_forward for this budget first)",
                (long long)max_items, (long long)plan->chunk_tokens * plan->max_splits);
  if (scores) {
    TD_REQUIRE(scores_dtype == TD_F32 || scores_dtype == kv->dtype,
               "td_decode_attn: scores dtype %d must be fp32 or the KV dtype", scores_dtype);
    TD_REQUIRE(score_stride > 0, "td_decode_attn: score_stride %lld", (long long)score_stride);
  }

  const int qpg = qpg_for(num_qo_heads, Hkv, list->idx_rows, D);
  const int subs = qpg > 1 ? (num_qo_heads / Hkv + qpg - 1) / qpg : 1;
  const int n_hrows = qpg > 1 ? Hkv * subs : num_qo_heads;
  qpg_out = qpg;
  n_hrows_out = n_hrows;

  const int64_t n_part = (int64_t)batch * n_hrows * qpg * plan->max_splits;
  const int64_t off_o = kTicketBytes;
  const int64_t off_ml = off_o + align256(n_part * D * 4);
  const int64_t need = off_ml + align256(n_part * 2 * 4);
  TD_REQUIRE((int64_t)batch * n_hrows * kTicketStride * 4 <= kTicketBytes,
             "td_decode_attn: batch %d x %d head rows exceeds the ticket counters", batch, n_hrows);
  TD_REQUIRE(plan->max_splits <= 64, "td_decode_attn: plan has %d splits (limit 64)",
             plan->max_splits);
  if (plan->max_splits > 1) {
    if (workspace == nullptr || workspace_bytes < need)
      return fail(TD_ERR_STATE,
                  "td_decode_attn: workspace of %lld bytes is smaller than the %lld the plan needs "
                  "(call td_decode_make_plan / begin_forward first)",
                  (long long)workspace_bytes, (long long)need);
  }

  p.q = q;
  p.o = o;
  p.kv = kv->data;
  p.page_stride = (int64_t)2 * P * Hkv * D;
  p.v_offset = (int64_t)P * Hkv * D;
  if (kv->layout == TD_NHD) {
    p.entry_stride = Hkv * D;
    p.head_stride = D;
  } else {
    p.entry_stride = D;
    p.head_stride = P * D;
  }
  p.page_size = P;
  p.page_shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == P) p.page_shift = sft;
  p.max_slot = (uint32_t)(kv->max_pages * P - 1);
  p.page_stride_b = (uint32_t)(p.page_stride * 2);
  p.entry_stride_b = (uint32_t)(p.entry_stride * 2);
  p.lean = (p.page_shift >= 0 && (int64_t)kv->max_pages * p.page_stride * 2 < ((int64_t)1 << 32)) ? 1 : 0;
  p.fresh_k = p.fresh_v = nullptr;
  p.fresh_cos = p.fresh_sin = nullptr;
  p.fresh_slot = nullptr;
  if (fresh) {
    TD_REQUIRE(fresh->k && fresh->v && fresh->cos && fresh->sin && fresh->dst_slot,
               "td_decode_attn: fresh token with a NULL member");
    p.fresh_k = fresh->k;
    p.fresh_v = fresh->v;
    p.fresh_cos = fresh->cos;
    p.fresh_sin = fresh->sin;
    p.fresh_slot = fresh->dst_slot;
  }
  p.num_qo_heads = num_qo_heads;
  p.n_hrows = n_hrows;
  p.vheads = n_hrows * qpg;
  p.subs = subs;
  p.q_per_kv = num_qo_heads / Hkv;
  p.idx = list->idx;
  p.idx_row_stride = list->idx_rows == 1 ? 0 : list->idx_row_stride;
  p.idx_cols = list->idx_row_stride > 0 ? list->idx_row_stride : 0;
  p.idx_per_kv = (qpg == 1 && list->idx_rows == Hkv && Hkv != num_qo_heads) ? 1 : 0;
  p.page_mode = list->kind == TD_IDX_PAGES ? 1 : 0;
  p.max_page = (uint32_t)(kv->max_pages - 1);
  p.indptr = list->indptr;
  p.count_arr = list->count_arr;
  p.n_list_host = list->n_list_host;
  p.last_len_arr = list->last_page_len_arr;
  p.last_idx_arr = list->last_page_idx_arr;
  p.last_len = list->last_page_len;
  p.last_idx = list->last_page_idx;
  p.chunk_tokens = plan->chunk_tokens;
  p.chunk_shift = p.qpk_shift = -1;
  for (int sft = 0; sft < 31; ++sft) {
    if ((1 << sft) == plan->chunk_tokens) p.chunk_shift = sft;
    if ((1 << sft) == p.q_per_kv) p.qpk_shift = sft;
  }
  p.max_splits = plan->max_splits;
  p.fused_merge = plan->fused_merge;
  p.scale_log2 = sm_scale * kLog2e;
  p.scores = scores;
  p.scores_f32 = scores_dtype == TD_F32 ? 1 : 0;
  p.score_stride = score_stride;
  p.lse = lse;
  char* ws = reinterpret_cast<char*>(workspace);
  p.ws_cnt = reinterpret_cast<int32_t*>(ws);
  p.ticket_stride = kTicketStride;
  p.ws_o = reinterpret_cast<float*>(ws ? ws + off_o : nullptr);
  p.ws_ml = reinterpret_cast<float*>(ws ? ws + off_ml : nullptr);

  return TD_OK;
}

// Whether a call can run on the short-list kernel of its plan: token-slot lists, head_dim 128, one
// query head per list walk or a whole group per shared list, no score output, chunks that are a
// power-of-two multiple of the kernel's workgroup tile.  Returns 0 (no), kSparseLean (power-of-two
// pages, pool below 4 GiB, strides within the 24-bit multiplier: 32-bit row offsets) or kSparseWide
// (any page size, 64-bit row offsets; 8 rows per lane only).
enum { kSparseNo = 0, kSparseLean = 1, kSparseWide = 2 };
static int sparse_kernel_fits(const DecodeParams& p, const td_decode_plan* plan,
                              const td_index_list* list, int qpg, int head_dim, bool emit) {
  if (plan->sparse_waves <= 0 || !sparse_shape_supported(plan->sparse_waves, plan->sparse_rows, qpg))
    return kSparseNo;
  const int stile = plan->sparse_waves * 4 * plan->sparse_rows;
  const bool heads_fit = qpg == 1 ? p.qpk_shift >= 0 : (p.q_per_kv == qpg && p.subs == 1);
  if (!(list->kind == TD_IDX_SLOTS && !emit && heads_fit && head_dim == 128 && p.chunk_shift >= 0 &&
        plan->chunk_tokens % stile == 0))
    return kSparseNo;
  if (p.lean && p.page_stride_b < (1u << 24) && p.entry_stride_b < (1u << 24)) return kSparseLean;
  // a page's bytes and an entry's offset inside it stay 32-bit; the page base is a 64-bit product
  if (plan->sparse_rows == 8 && p.page_stride * 2 < ((int64_t)1 << 32)) return kSparseWide;
  return kSparseNo;
}

extern "C" int td_decode_attn(const td_paged_kv* kv, const td_index_list* list,
                              const td_decode_plan* plan, const void* q, void* o, int32_t batch,
                              int32_t num_qo_heads, float sm_scale, void* scores,
                              int32_t scores_dtype, int64_t score_stride, float* lse,
                              const td_fresh_token* fresh, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  DecodeParams p;
  int qpg, n_hrows;
  const int prc = build_params(kv, list, plan, q, o, batch, num_qo_heads, sm_scale, scores, scores_dtype,
                               score_stride, lse, fresh, workspace, workspace_bytes, p, qpg, n_hrows);
  if (prc != TD_OK) return prc;
  const int D = kv->head_dim;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool page_mode = list->kind == TD_IDX_PAGES;
  dim3 grid(n_hrows, batch, plan->max_splits);
  const bool merge_kernel = plan->max_splits > 1 && !plan->fused_merge;
  int rc;
  const int fits = sparse_kernel_fits(p, plan, list, qpg, D, scores != nullptr);
  if (fits != kSparseNo) {
    const bool wide = fits == kSparseWide;
    TD_REQUIRE((int64_t)batch * n_hrows * qpg * kTicketStride * 4 <= kTicketBytes,
               "td_decode_attn: batch %d x %d heads exceeds the ticket counters", batch, n_hrows * qpg);
    if (qpg > 1)
      rc = kv->dtype == TD_F16
               ? launch_sparse_shared_f16(p, plan->sparse_waves, qpg, wide, merge_kernel, grid, st)
               : launch_sparse_shared_bf16(p, plan->sparse_waves, qpg, wide, merge_kernel, grid, st);
    else if (kv->dtype == TD_F16)
      rc = launch_sparse_f16(p, plan->sparse_waves, plan->sparse_rows, false, wide, merge_kernel, grid, st);
    else
      rc = launch_sparse_bf16(p, plan->sparse_waves, plan->sparse_rows, false, wide, merge_kernel, grid, st);
    if (rc != TD_OK) return rc;
    TD_HIP_CHECK(hipGetLastError());
    g_last_kernel = wide ? "short-list, 64-bit offsets" : "short-list";
    return TD_OK;
  }
  if (fresh && !p.lean)
    return fail(TD_ERR_UNSUPPORTED,
                "td_decode_attn: outside the short-list kernel (token-slot lists of up to %lld entries, "
                "head_dim 128, no score output) the fused decode step needs a power-of-two page_size and "
                "a pool below 4 GiB (page_size %d, pool %lld bytes); use td_rope_append_decode first",
                (long long)kSparseMaxItems, kv->page_size, (long long)(kv->max_pages * p.page_stride * 2));
  if (kv->dtype == TD_F16)
    rc = launch_decode_f16(p, D, qpg, plan->waves_per_block, plan->tile_rows, page_mode, scores != nullptr,
                           merge_kernel, grid, st);
  else
    rc = launch_decode_bf16(p, D, qpg, plan->waves_per_block, plan->tile_rows, page_mode, scores != nullptr,
                            merge_kernel, grid, st);
  if (rc != TD_OK) return rc;
  TD_HIP_CHECK(hipGetLastError());
  g_last_kernel = p.lean ? "streaming" : "streaming, 64-bit offsets";
  return TD_OK;
}

extern "C" int td_decode_attn_noalloc(const td_paged_kv* kv, const td_index_list* list,
                                      const td_decode_plan* plan, const void* q, void* o,
                                      int32_t batch, int32_t num_qo_heads, float sm_scale,
                                      void* scores, int32_t scores_dtype, int64_t score_stride,
                                      float* lse, const td_fresh_token* fresh, void* stream) {
  TD_REQUIRE(plan != nullptr, "td_decode_attn_noalloc: plan is NULL");
  if (plan->workspace_bytes > (int64_t)TD_STATIC_SCRATCH_BYTES)
    return fail(TD_ERR_STATE,
                "td_decode_attn_noalloc: the plan needs %lld bytes of scratch, the built-in scratch holds "
                "%lld (fewer sequences, heads or splits, or td_decode_attn with a workspace)",
                (long long)plan->workspace_bytes, (long long)TD_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != TD_OK) return rc;
  return td_decode_attn(kv, list, plan, q, o, batch, num_qo_heads, sm_scale, scores, scores_dtype,
                        score_stride, lse, fresh, ws, (int64_t)TD_STATIC_SCRATCH_BYTES, stream);
}

// ---------------------------------------------------------------------------------------------
// Measurement aid: the memory side of a sparse layer alone.  Same grid, same interleaved tiles,
// same list -> slot -> K row / V row non-temporal 16-byte loads as decode_attn_kernel for token
// -slot lists, but no arithmetic, no merge: every wave folds what it loaded into one word and
// stores it.  Its duration is the floor that the attention launch is compared with.
// ---------------------------------------------------------------------------------------------
template <int D, int U, int NW>
__global__ __launch_bounds__(NW * 64) void gather_probe_kernel(const DecodeParams p, uint32_t* out) {
  constexpr int LPR = D / 8, TPI = 64 / LPR, TILE = U * TPI;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane / LPR, li = lane % LPR;
  const int hrow = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
  const int kv_head = hrow / p.q_per_kv;
  SeqList s;
  int list_beg;
  const int n_splits = seq_items(p, b, s, list_beg);
  if (split >= n_splits) return;
  const int idx_row = p.idx_per_kv ? kv_head : hrow;
  s.row = p.idx + (int64_t)idx_row * p.idx_row_stride + list_beg;
  const int c1 = s.n_list;  // listed slots only
  const char* kbase = reinterpret_cast<const char*>(p.kv);
  const char* vbase = kbase + p.v_offset * 2;
  const uint32_t head_byte_off = (uint32_t)(kv_head * p.head_stride + li * 8) * 2u;
  const int STEP = n_splits * NW * TILE;
  u32x4 fold = {0u, 0u, 0u, 0u};
  for (int t = (split * NW + wave) * TILE; t < c1; t += STEP) {
    u32x4 kb[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int i = t + u * TPI + g;
      i = i < c1 ? i : c1 - 1;
      uint32_t slot = (uint32_t)s.row[i];
      slot = slot > p.max_slot ? p.max_slot : slot;
      const uint32_t page = slot >> p.page_shift, entry = slot & ((1u << p.page_shift) - 1u);
      const uint32_t off = page * p.page_stride_b + entry * p.entry_stride_b + head_byte_off;
      kb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kbase + off));
      vb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vbase + off));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) fold ^= kb[u] ^ vb[u];
  }
  uint32_t w = fold.x ^ fold.y ^ fold.z ^ fold.w;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) w ^= (uint32_t)__shfl_xor((int)w, off, 64);
  if (lane == 0)
    out[(((int64_t)b * gridDim.x + hrow) * gridDim.z + split) * NW + wave] = w;
}

extern "C" int td_gather_probe(const td_paged_kv* kv, const td_index_list* list,
                               const td_decode_plan* plan, int32_t batch, int32_t num_qo_heads,
                               void* out, int64_t out_bytes, void* stream) {
  TD_REQUIRE(out != nullptr, "td_gather_probe: NULL out");
  DecodeParams p;
  int qpg, n_hrows;
  const int prc = build_params(kv, list, plan, out, out, batch, num_qo_heads, 1.f, nullptr, TD_F32, 0,
                               nullptr, nullptr, out, (int64_t)1 << 40, p, qpg, n_hrows);
  if (prc != TD_OK) return prc;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int fits = qpg == 1 ? sparse_kernel_fits(p, plan, list, qpg, kv->head_dim, false) : kSparseNo;
  if (fits != kSparseNo && list->last_page_len == 0 && !list->last_page_len_arr) {
    // the short-list kernel's own loads-only form; it reads `out` as q and writes nothing
    TD_REQUIRE(out_bytes >= (int64_t)batch * num_qo_heads * kv->head_dim * 2,
               "td_gather_probe: out holds %lld bytes, %lld needed", (long long)out_bytes,
               (long long)batch * num_qo_heads * kv->head_dim * 2);
    const dim3 sgrid(n_hrows, batch, plan->max_splits);
    const bool wide = fits == kSparseWide;
    const int src =
        kv->dtype == TD_F16
            ? launch_sparse_f16(p, plan->sparse_waves, plan->sparse_rows, true, wide, false, sgrid, st)
            : launch_sparse_bf16(p, plan->sparse_waves, plan->sparse_rows, true, wide, false, sgrid, st);
    if (src != TD_OK) return src;
    TD_HIP_CHECK(hipGetLastError());
    return TD_OK;
  }
  const int nw = plan->waves_per_block, rows = plan->tile_rows;
  if (!(list->kind == TD_IDX_SLOTS && p.lean && qpg == 1 && kv->head_dim == 128 &&
        ((nw == 8 && (rows == 4 || rows == 2)) || (nw == 16 && rows == 4)) &&
        list->last_page_len == 0 && !list->last_page_len_arr))
    return fail(TD_ERR_UNSUPPORTED,
                "td_gather_probe: token-slot lists without a forced last page, one query head per "
                "row, head_dim 128, power-of-two pages, pool below 4 GiB only");
  TD_REQUIRE(out_bytes >= (int64_t)batch * n_hrows * plan->max_splits * nw * 4,
             "td_gather_probe: out holds %lld bytes, %lld needed", (long long)out_bytes,
             (long long)batch * n_hrows * plan->max_splits * nw * 4);
  const dim3 grid(n_hrows, batch, plan->max_splits);
  uint32_t* outw = reinterpret_cast<uint32_t*>(out);
  if (nw == 16)
    hipLaunchKernelGGL((gather_probe_kernel<128, 4, 16>), grid, dim3(1024), 0, st, p, outw);
  else if (rows == 2)
    hipLaunchKernelGGL((gather_probe_kernel<128, 2, 8>), grid, dim3(512), 0, st, p, outw);
  else
    hipLaunchKernelGGL((gather_probe_kernel<128, 4, 8>), grid, dim3(512), 0, st, p, outw);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
