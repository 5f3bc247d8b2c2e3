/*
 * tidal_hip.h -- C ABI of libtidal_hip.so, the gfx950 (MI355X) implementation of the
 * TidalDecode decode-attention path.
 *
 * Every entry point takes raw device pointers, plain integer sizes and a hipStream_t passed as
 * void*.  No torch types cross this boundary.  All functions return 0 (TD_OK) on success and a
 * non-zero td_status otherwise; td_last_error() then holds a human-readable message for the
 * calling thread.  Nothing here synchronises the stream and nothing copies device -> host.
 *
 * Each declaration cites the interface of the reference (DerrickYLJ/TidalDecode) that it
 * replaces; paths are relative to the reference checkout.
 */
#ifndef TIDAL_HIP_H_
#define TIDAL_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  TD_OK = 0,
  TD_ERR_INVALID_ARG = 1, /* shape / pointer / range check failed */
  TD_ERR_UNSUPPORTED = 2, /* dtype, head_dim or group size has no kernel ("failed to dispatch") */
  TD_ERR_STATE = 3,       /* workspace too small for the plan */
  TD_ERR_HIP = 4          /* a HIP runtime call failed */
} td_status;

/* Element types.  KV cache, q, k, v, o are TD_F16 or TD_BF16; scores may be TD_F32 as well. */
typedef enum { TD_F16 = 0, TD_BF16 = 1, TD_F32 = 2 } td_dtype;

/* Layout of the last three page dimensions, tidal/utils/utils.py:1-5. */
typedef enum { TD_NHD = 0, TD_HND = 1 } td_layout;

/* How one row of the sparse index list is interpreted by td_decode_attn. */
typedef enum {
  /* Entries are physical page ids; every listed page contributes page_size tokens.  This is the
   * reference's meaning (kernels/include/decode/decode_page.cuh:320-346). */
  TD_IDX_PAGES = 0,
  /* Entries are physical token slots, slot = page_id * page_size + entry.  Extension for
   * token-granular selection with page_size > 1. */
  TD_IDX_SLOTS = 1
} td_idx_kind;

/* How scores are reduced before selection (td_score_reduce). */
typedef enum {
  TD_REDUCE_HEAD_SUM = 0, /* softmax probabilities summed over all query heads -> 1 row   */
  TD_REDUCE_GROUP_SUM = 1 /* summed over the query heads of each KV head      -> H_kv rows */
} td_reduce_mode;

/*
 * Paged KV pool of one layer.
 * data: [max_pages, 2, page_size, num_kv_heads, head_dim] (TD_NHD) or
 *       [max_pages, 2, num_kv_heads, page_size, head_dim] (TD_HND), index 1 = 0 for K, 1 for V.
 * Mirrors paged_kv_t, kernels/include/decode/decode_page.cuh:73-252.
 */
typedef struct {
  void* data;
  int64_t max_pages; /* capacity; slots are clamped to it inside the kernels */
  int32_t num_kv_heads;
  int32_t head_dim; /* 64, 128 or 256 */
  int32_t page_size;
  int32_t layout; /* td_layout */
  int32_t dtype;  /* td_dtype: TD_F16 or TD_BF16 */
} td_paged_kv;

/*
 * Per-call description of which tokens each sequence attends to.
 *
 * idx is a 2-D int32 array with `idx_rows` rows of `idx_row_stride` elements (a single row:
 * the number of elements it holds, or 0 if unknown).  Sequence b uses
 * columns [indptr[b], indptr[b+1]) of every row (indptr lives on the device; if indptr is NULL
 * the call is for one sequence that uses columns [0, n_list_host)).  With count_arr (device,
 * [batch]) sequence b uses count_arr[b] columns starting at indptr[b] instead: the rows of a
 * padded table, one fixed-width segment per sequence, which can grow in place.  Row r belongs to query
 * head r (idx_rows == num_qo_heads), to KV head r (idx_rows == num_kv_heads) or to everybody
 * (idx_rows == 1).  The kernels read no column of a row outside the sequence's segment
 * [indptr[b], indptr[b+1]), beyond n_list_host columns from its start, or at idx_row_stride and
 * beyond; a device-resident count that says otherwise is cut to that.
 *
 * After the listed entries every sequence may attend to one more, partially filled page: the
 * first last_page_len entries of page last_page_idx ("forced last page",
 * decode_page.cuh:326-329, decode_attn.cuh:726-730).  The *_arr pointers (device, [batch]) take
 * precedence over the scalars; last_page_len == 0 disables it.
 */
typedef struct {
  const int32_t* idx;
  int32_t idx_rows;
  int32_t idx_row_stride;
  int32_t kind; /* td_idx_kind */
  const int32_t* indptr; /* device [batch+1] or NULL */
  int32_t n_list_host;   /* used when indptr == NULL; else an upper bound of the per-sequence count */
  const int32_t* last_page_len_arr; /* device [batch] or NULL */
  const int32_t* last_page_idx_arr; /* device [batch] or NULL */
  int32_t last_page_len;
  int32_t last_page_idx;
  const int32_t* count_arr; /* device [batch] or NULL; needs indptr */
} td_index_list;

/*
 * Split plan of one decode-attention call: how many tokens one workgroup covers and how many
 * partial results per head that makes.  Filled by td_decode_make_plan on the host (no launch, no
 * allocation, no device memory is read; see there for the two runtime queries it makes); replaces
 * BatchDecodeHandler::BeginForward + BatchDecodeWithPagedKVCacheWorkEstimation +
 * PartitionPagedKVCacheComputeAuxiliaryInfo (kernels/include/decode/decode_handler.cuh:39-175,
 * decode_attn.cuh:687-906; binding tidal/ops/csrc/approx_attn.cu:27-66).
 */
typedef struct {
  int32_t chunk_tokens;    /* tokens per workgroup and head group */
  int32_t max_splits;      /* upper bound of partial results per head */
  int32_t waves_per_block; /* 8 or 16 */
  int32_t tile_rows;       /* K/V load instructions per wave tile: 2 or 4 */
  int32_t fused_merge;     /* 1: last workgroup merges in-kernel; 0: second kernel */
  /* Shape of the short-list kernel that serves calls with token-slot lists, head_dim 128, one
   * list row per query head (or one shared row without grouped queries) and no score output:
   * waves per workgroup (4 or 8) x K rows per lane (8 or 16; pools of 4 GiB and more and pages
   * that are not a power of two: 8).  0 on input: the planner decides; -1 on input: never use
   * that kernel.  On output 0 means the streaming kernel (waves_per_block x tile_rows) serves
   * every call of this plan. */
  int32_t sparse_waves;
  int32_t sparse_rows;
  int64_t workspace_bytes; /* device scratch the call needs (partials + tickets) */
} td_decode_plan;

/*
 * The token being decoded, for the fused decode step of td_decode_attn: its un-rotated key and
 * value rows, the cosines / sines of its rotary angles (td_rope_table) and the physical slot it
 * occupies.  All device pointers.
 */
typedef struct {
  const void* k;           /* [batch, num_kv_heads, head_dim] */
  const void* v;           /* [batch, num_kv_heads, head_dim] */
  const float* cos;        /* [batch, head_dim / 2] */
  const float* sin;        /* [batch, head_dim / 2] */
  const int32_t* dst_slot; /* [batch]: page_id * page_size + entry */
} td_fresh_token;

/* Thread-local message of the last failing call. */
const char* td_last_error(void);

/* Library ABI version (bumped on any signature change). */
int td_version(void);

/* Number of compute units of the current device (used by the planner; cached). */
int td_num_cus(void);

/*
 * Rotate-half (Llama) RoPE applied in place to q [n_tokens, num_qo_heads, head_dim] and
 * k [n_tokens, num_kv_heads, head_dim]; token i sits at position past_kv_len + i; angle =
 * position / rope_scale * rope_theta^(-2(j mod D/2)/D).
 * Replaces apply_rope_in_place (tidal/ops/csrc/bsk_ops.h:23-27, page.cu:212-253) and
 * QKApplyRotaryInPlace (kernels/include/decode/decode_page.cuh:639-723).
 */
int td_rope_in_place(void* q, void* k, int32_t n_tokens, int32_t num_qo_heads,
                     int32_t num_kv_heads, int32_t head_dim, int64_t past_kv_len, float rope_scale,
                     float rope_theta, int32_t dtype, void* stream);

/*
 * Append n_tokens new (k, v) rows [n_tokens, num_kv_heads, head_dim] to one sequence.
 * The sequence owns pages kv_indices[kv_indptr[0] .. kv_indptr[1]) and, after the append, holds
 * seq_len = (n_pages - 1) * page_size + last_page_len tokens; the new rows are its last
 * n_tokens.  n_tokens == 1 is the decode case.  kv_indices / kv_indptr are device arrays.
 * If meta != NULL, meta_indices/meta_indptr/meta_last_page_len describe a second paged pool
 * that keeps, per KV page, the running element-wise max (K plane) and min (V plane) of the keys
 * of that page (one metadata entry per KV page), as the reference does for its page estimator.
 * Replaces append_kv_cache_decode / append_kv_cache_prefill (bsk_ops.h:52-78, page.cu:6-210),
 * AppendPagedKVCacheDecode/Prefill (decode_page.cuh:387-627).
 */
int td_append_kv(const td_paged_kv* kv, const void* k, const void* v, int32_t n_tokens,
                 const int32_t* kv_indices, const int32_t* kv_indptr, int32_t last_page_len,
                 const td_paged_kv* meta, const int32_t* meta_indices, const int32_t* meta_indptr,
                 int32_t meta_last_page_len, void* stream);

/*
 * Decode-step fusion of the two calls above for a batch of sequences: rotates q [batch,
 * num_qo_heads, D] in place, rotates k [batch, num_kv_heads, D] and writes it together with
 * v into physical slot dst_slot[b] (= page_id * page_size + entry) of the pool.  positions[b]
 * is the token position of sequence b.  dst_slot and positions are device int32 [batch].
 * No counterpart as one call in the reference; it fuses apply_rope_in_place + append_kv_cache_decode
 * (tidal/models/SearchAttention.py:131-150).
 */
int td_rope_append_decode(const td_paged_kv* kv, void* q, const void* k, const void* v,
                          int32_t batch, int32_t num_qo_heads, const int32_t* positions,
                          const int32_t* dst_slot, float rope_scale, float rope_theta,
                          void* stream);

/*
 * Choose the split of a decode-attention call.  max_items is an upper bound of the tokens any
 * sequence attends to; idx_rows as in td_index_list.  chunk_tokens / waves_per_block / tile_rows /
 * sparse_waves / sparse_rows (non-zero) and fused_merge (non-negative) may be preset in *plan to
 * override the heuristics; pass a zero-initialised struct with fused_merge = -1 for defaults.
 * The plan itself is host arithmetic: no launch, no allocation, no synchronisation.  Two read-only
 * runtime queries ride along, each made once per process and device: the compute-unit count of
 * the current device (hipDeviceGetAttribute; 256 is assumed when there is no device) and the
 * device address of the static scratch of td_decode_attn_noalloc (hipGetSymbolAddress, so that
 * the entry point that must not allocate finds it resolved; a failure here is ignored and the
 * lookup is tried again there).  Call it outside stream capture.
 * Replaces BatchDecodeWithPagedKVCacheWorkEstimation and PartitionPagedKVCacheComputeAuxiliaryInfo
 * (kernels/include/decode/decode_attn.cuh:815-906, :687-748), reached through
 * BatchDecodeHandler::BeginForward (decode_handler.cuh:39-121, binding approx_attn.cu:27-62).
 */
int td_decode_make_plan(int32_t batch, int32_t num_qo_heads, int32_t num_kv_heads, int32_t head_dim,
                   int32_t idx_rows, int64_t max_items, td_decode_plan* plan);

/*
 * Decode attention of one new token per sequence over the listed tokens of a paged KV pool:
 * o[b,h,:] = softmax(q[b,h,:] . K_sel^T / sqrt(D)) V_sel, online softmax in base 2, fp32
 * accumulation, split over tokens and merged by log-sum-exp.
 *   q, o       [batch, num_qo_heads, head_dim], dtype of the pool
 *   scores     optional [batch, num_qo_heads, score_stride]: element i = q . k_i / sqrt(D) of the
 *              i-th attended token in list order (td_dtype scores_dtype); NULL to skip
 *   lse        optional float [batch, num_qo_heads]: natural-log sum of exp of the logits
 *   fresh      optional (NULL = off) decode-step fusion: q is then the UN-rotated query; the
 *              kernel rotates it in registers (q in memory is left as it was), rotates fresh->k,
 *              writes it and fresh->v into the cache at fresh->dst_slot, and attends to that
 *              token wherever the list names its slot -- one launch instead of
 *              td_rope_append_decode + td_decode_attn (tidal/models/SearchAttention.py:131-176 runs
 *              three).  Calls served by the streaming kernel (page lists, score output, lists of
 *              more than 16384 entries, head_dim 64 / 256) need a power-of-two page_size and a
 *              pool below 4 GiB for it (TD_ERR_UNSUPPORTED otherwise).
 *   workspace  device scratch of at least plan->workspace_bytes whose first 1 MiB (ticket
 *              counters, 64 bytes apart) was zero-filled once before first use; every call
 *              leaves them zero again, so one workspace serves plans of any shape.  Calls that
 *              share a workspace must be ordered on one stream.
 * Replaces BatchDecodeWithPagedKVCachePyTorchWrapper::Forward (bsk_ops.h:104-113,
 * tidal/ops/csrc/approx_attn.cu:68-151), BatchDecodeWithPagedKVCacheKernel
 * (kernels/include/decode/decode_attn.cuh:432-658) including its score output
 * (decode_attn.cuh:107-109) and VariableLengthMergeStates (decode_attn.cuh:1011-1020).
 */
int td_decode_attn(const td_paged_kv* kv, const td_index_list* list, const td_decode_plan* plan,
                   const void* q, void* o, int32_t batch, int32_t num_qo_heads, float sm_scale,
                   void* scores, int32_t scores_dtype, int64_t score_stride, float* lse,
                   const td_fresh_token* fresh, void* workspace, int64_t workspace_bytes,
                   void* stream);

/*
 * Which kernel family served the calling thread's last successful td_decode_attn call:
 * "short-list" (the sparse layer's kernel: token-slot lists of up to 16384 entries, head_dim 128, no
 * score output), "streaming" (everything else), each with ", 64-bit offsets" for pools of 4 GiB and
 * more or pages that are not a power of two; "none" before the first call.  No counterpart in the
 * reference (one kernel there, dispatched by SWITCH_HEAD_DIM,
 * kernels/include/decode/decode_attn.cuh:1150-1154); tests and benchmarks use it to say which code
 * they measured.
 */
const char* td_last_decode_kernel(void);

/*
 * td_decode_attn for callers that cannot allocate device memory or be handed a workspace -- code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc: the ticket
 * counters and split partials live in TD_STATIC_SCRATCH_BYTES of device memory inside the library
 * image (one copy per GPU, held until the process ends).  Same arguments, kernels and results as
 * td_decode_attn without `workspace` / `workspace_bytes`; a plan whose workspace_bytes exceeds
 * TD_STATIC_SCRATCH_BYTES is rejected with TD_ERR_STATE.  Calls no hipMalloc / hipFree.  All calls
 * on one GPU share that GPU's scratch: they must be ordered on one stream (calls that overlap
 * race), and they must not be mixed on another stream with in-flight calls of this entry point.
 * The scratch starts zeroed and every launch leaves its counters zeroed, so nothing is cleared per
 * call.  No counterpart in the reference, whose handler allocates its scratch in every
 * BeginForward (kernels/include/decode/decode_handler.cuh:39-121).
 */
#define TD_STATIC_SCRATCH_BYTES (4 << 20)
int td_decode_attn_noalloc(const td_paged_kv* kv, const td_index_list* list,
                           const td_decode_plan* plan, const void* q, void* o, int32_t batch,
                           int32_t num_qo_heads, float sm_scale, void* scores, int32_t scores_dtype,
                           int64_t score_stride, float* lse, const td_fresh_token* fresh,
                           void* stream);

/*
 * cos[b, j] / sin[b, j] of positions[b] / rope_scale * rope_theta^(-2j/head_dim), j < head_dim/2
 * (angles formed in double precision, as td_rope_in_place does).  One launch per decode step
 * serves every layer's fused td_decode_attn.
 */
int td_rope_table(const int32_t* positions, int32_t batch, int32_t head_dim, float rope_scale,
                  float rope_theta, float* cos, float* sin, void* stream);

/*
 * Device-resident state of one decoding sequence: everything the launches of a decode step need to
 * know about the sequence, as int32 words that td_step_advance keeps current, so that a decode
 * step captured in a HIP graph stays valid while the sequence grows (td_index_list.count_arr,
 * last_page_len_arr, last_page_idx_arr, td_fresh_token.dst_slot, td_rope_table's positions and
 * td_topk's len_arr all point into it).  No counterpart in the reference, whose controller
 * rebuilds and re-uploads this on the host every step (tidal/utils/controller.py:89-147).
 */
enum {
  TD_STEP_SEQ_LEN = 0,           /* tokens in the cache, the one being decoded included */
  TD_STEP_PAGES_BEFORE_LAST = 1, /* full pages before the page being filled */
  TD_STEP_LAST_PAGE_LEN = 2,     /* entries in use in the page being filled, 1..page_size */
  TD_STEP_LAST_PAGE_IDX = 3,     /* its physical page id */
  TD_STEP_DST_SLOT = 4,          /* physical slot of the token being decoded */
  TD_STEP_POSITION = 5,          /* its position, seq_len - 1 */
  TD_STEP_N_SELECTED = 6,        /* min(budget, seq_len): entries of the persisted token lists */
  TD_STEP_COUNT = 7,             /* steps taken */
  TD_STEP_WORDS = 8
};

/*
 * Advance the state by one token (one tiny launch, graph-safe): seq_len += 1 and the other words
 * follow from page_table [n_pages] (the pages of the sequence in order; the caller has reserved
 * pages for every token it will decode).  If token / tokens_out are given, the token id the step
 * consumes (*token) is first recorded at tokens_out[steps taken] (ignored beyond tokens_cap).
 */
int td_step_advance(int32_t* state, const int32_t* page_table, int32_t n_pages, int32_t page_size,
                    int32_t budget, const int64_t* token, int64_t* tokens_out, int32_t tokens_cap,
                    void* stream);

/*
 * Merge of attention states over disjoint token subsets: o_parts [n_parts, rows, head_dim] (dtype:
 * td_dtype, also the type of o) are the attention outputs of the parts, lse_parts [n_parts, rows]
 * the natural-log sums of exponentials of their logits (as td_decode_attn writes to `lse`);
 * o [rows, head_dim] = sum_i o_i e^(lse_i - lse), lse [rows] (optional) = log sum_i e^(lse_i).  A
 * part with lse = -inf is empty and ignored.  The stand-alone form of the split merge that
 * td_decode_attn runs inside its launch; replaces VariableLengthMergeStates of the reference's
 * FlashInfer dependency (call site kernels/include/decode/decode_attn.cuh:1011-1020) for callers
 * that split a sequence themselves, e.g. across devices.
 */
int td_merge_states(const void* o_parts, int32_t dtype, const float* lse_parts, int32_t n_parts,
                    int32_t rows, int32_t head_dim, void* o, float* lse, void* stream);

/*
 * td_step_advance for a batch decoding in lock step: word w of sequence b is state[w * stride + b]
 * (so every word is a contiguous [batch] array, the form the *_arr arguments take), sequence b's
 * pages are row b of page_table [batch, table_stride].
 */
int td_step_advance_batch(int32_t* state, int32_t stride, int32_t batch, const int32_t* page_table,
                          int32_t table_stride, int32_t page_size, int32_t budget, void* stream);

/*
 * out[0] = index of the largest of the n values of x (dtype: td_dtype; NaN counts as largest, ties
 * go to the lower index).  The greedy choice of the next token without leaving the device: a plain
 * one-workgroup launch with no scratch, so that it can sit in a captured decode step.  No
 * counterpart in the reference (its driver takes torch.argmax on the host side of each step).
 */
int td_argmax(const void* x, int32_t dtype, int32_t n, int64_t* out, void* stream);

/*
 * Cross-head reduction of selection-layer scores: out[r, i] = sum over the query heads h of
 * row r of exp(logits[h, i] - lse[h]) (i < n), fp32.  rows = 1 (TD_REDUCE_HEAD_SUM) or
 * num_kv_heads (TD_REDUCE_GROUP_SUM).  logits is float [num_qo_heads, logits_stride].
 * No counterpart in the reference (its selection is per head); implements the cross-head sum
 * of the benchmark configuration.
 */
int td_score_reduce(const float* logits, int64_t logits_stride, const float* lse,
                    int32_t num_qo_heads, int32_t num_kv_heads, int32_t n, int32_t mode,
                    float* out, int64_t out_stride, void* stream);

/*
 * Row-wise top-k: for each of `rows` rows of `values` (length len, row stride values_stride)
 * select the k largest elements; ties at the threshold go to the lower position.  Outputs, per
 * row, sorted by ascending position: out_values[r, j] (same dtype as values, may be NULL) and
 * out_idx[r, j] = payload of the selected position p:
 *     in_idx != NULL              -> in_idx[r * in_idx_stride + p]   (reference meaning)
 *     page_table != NULL          -> table[p / page_size] * page_size + p % page_size, where
 *                                    table = page_table + (r / rows_per_table) * page_table_stride
 *                                    (rows_per_table == 0: one table for all rows)
 *     both NULL                   -> p
 * k is clamped to len.  NaNs order above +inf.  out rows have stride out_stride.
 * len_arr (device, one entry per group of rows_per_table rows, or NULL): row r takes only its
 * first len_arr[r / rows_per_table] elements (clamped to 1..len) and selects min(k, that many);
 * the rest of its output row is left untouched.  Lengths that live on the device let a batch of
 * sequences of different lengths, or a captured graph whose sequence grows, use one call.
 * workspace: see td_topk_workspace_bytes (optional).
 * Replaces topk_filtering (bsk_ops.h:34-39, tidal/ops/csrc/topk.cu:7-44) and decode_select_k
 * (kernels/include/topk/decode_select_k.cuh:25-62; RAFT radix_topk_one_block_kernel).
 */
int td_topk(const void* values, int32_t values_dtype, int64_t values_stride, int32_t rows,
            int32_t len, int32_t k, const int32_t* in_idx, int64_t in_idx_stride,
            const int32_t* page_table, int64_t page_table_stride, int32_t rows_per_table,
            const int32_t* len_arr, int32_t page_size, void* out_values, int32_t* out_idx, int64_t out_stride,
            void* workspace, int64_t workspace_bytes, void* stream);

/*
 * td_topk with a per-row upper bound of the scores: row_bound[r] (float, device, or NULL) is a
 * value that no score of row r exceeds -- for the logits of a selection layer, the row's
 * log-sum-exp as td_decode_attn writes it; for td_score_reduce's sums, the number of heads summed.
 * The selection then measures every score from that bound instead of from the row's maximum and
 * needs no pass to find the maximum: the row is counted while its loads arrive.  Same result as
 * td_topk, bit for bit.  A NaN or infinite bound is ignored (td_decode_attn's lse is NaN whenever a
 * logit is NaN or +inf, so such rows take the exact path and NaNs still rank first).  A finite
 * bound below a score of the row, or above a NaN, gives an unspecified selection (never an access
 * out of bounds).  No counterpart in the reference.
 */
int td_topk_bounded(const void* values, int32_t values_dtype, int64_t values_stride, int32_t rows,
                    int32_t len, int32_t k, const int32_t* in_idx, int64_t in_idx_stride,
                    const int32_t* page_table, int64_t page_table_stride, int32_t rows_per_table,
                    const int32_t* len_arr, int32_t page_size, const float* row_bound,
                    void* out_values, int32_t* out_idx, int64_t out_stride, void* workspace,
                    int64_t workspace_bytes, void* stream);

/*
 * Bytes of device scratch for td_topk.  Rows of up to 65536 elements never touch it (one launch,
 * every workgroup of a row selects on the whole row and emits a slice).  A few longer rows are
 * shared between workgroups through it (three launches; about 56 KiB per row); without it (NULL),
 * or with many long rows, the one-launch kernel re-reads such rows from L2 in every pass.  The
 * scratch must be zero-filled once before its first use; every call leaves it ready for the next.
 * Plays the part of the `buf` argument of topk_filtering (tidal/utils/controller.py:164-168).
 */
int64_t td_topk_workspace_bytes(int32_t rows);

/*
 * Page-level upper bound of the attention logits from the per-page key max / min metadata that
 * td_append_kv maintains: o[h, e] = sum_d max(q[h,d] * max[e,d], q[h,d] * min[e,d]) for every
 * metadata entry e but the newest ((n_meta_pages - 1) * page_size + meta_last_page_len - 1
 * entries; o rows have stride o_stride, o in the pool's dtype).  Replaces estimate_attn_score
 * (bsk_ops.h:41-48, tidal/ops/csrc/estimate.cu:6-88, MaxPossibleSampleWithPagedKVCacheKernel,
 * kernels/include/decode/decode_attn.cuh:142-172,236-405).
 */
int td_estimate_score(const td_paged_kv* meta, const int32_t* meta_indices, int32_t n_meta_pages,
                      int32_t meta_last_page_len, const void* q, int32_t num_qo_heads, void* o,
                      int64_t o_stride, void* stream);

/*
 * RMSNorm: out[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight, fp32 math.
 * Replaces rms_norm_forward (bsk_ops.h:29-32, tidal/ops/csrc/rms_norm.cu:160-212).
 */
int td_rms_norm(const void* x, const void* weight, void* out, int32_t rows, int32_t cols,
                float eps, int32_t dtype, void* stream);

/*
 * Measurement aid without a counterpart in the reference: the memory side of a sparse layer
 * alone.  Same grid and the same list -> slot -> K / V row loads as td_decode_attn for
 * token-slot lists (the launch that replaces BatchDecodeWithPagedKVCacheKernel,
 * kernels/include/decode/decode_attn.cuh:432-658), no arithmetic and no merge; one word per
 * wavefront is written to out (batch * head rows * plan->max_splits * plan->waves_per_block words).  bench.py times
 * it next to the attention launch.
 */
int td_gather_probe(const td_paged_kv* kv, const td_index_list* list, const td_decode_plan* plan,
                    int32_t batch, int32_t num_qo_heads, void* out, int64_t out_bytes,
                    void* stream);

/*
 * Prefill: attention of the n_q newest tokens of one sequence (q, o: [n_q, num_qo_heads, head_dim])
 * over its kv_len cached tokens, whose pages are page_table[0 .. n_pages) in order (K/V of the
 * new tokens already appended).  causal != 0: query row i sees positions <= kv_len - n_q + i.
 * head_dim 64, 128 or 256, fp16 / bf16.  Replaces prefill_with_paged_kv_cache (bsk_ops.h:80-88,
 * tidal/ops/csrc/batch_prefill.cu:27-117, kernels/include/prefill/prefill.cuh:674-870).
 */
int td_prefill_attn(const td_paged_kv* kv, const int32_t* page_table, int32_t n_pages,
                    int32_t kv_len, const void* q, void* o, int32_t n_q, int32_t num_qo_heads,
                    float sm_scale, int32_t causal, void* stream);

/*
 * Matrix-vector product of a batch-1 decode step: y[rows] = W[rows, cols] . f(x) (+ residual),
 * 16-bit storage, fp32 accumulation.  x_mode 0: f(x) = x[cols]; 1: f(x) = RMSNorm(x) * norm_weight
 * (eps); 2: f(x) = silu(x[:cols]) * x[cols:2 cols] (gated MLP).  residual (or NULL) is added to
 * the result and may alias y.  pair_gated != 0: rows is even and y has rows/2 entries,
 * y[i] = silu(W[i] . f(x)) * (W[i + rows/2] . f(x)) (gate and up projections stacked in W).
 * cols: multiple of 8, at most 30720; w and x 16-byte aligned.
 * Serves the decoder harness around the attention path, where the reference calls torch's
 * nn.Linear, LlamaRMSNorm and act_fn one by one (tidal/models/SparseAttention.py:122-124,216,
 * tidal/models/llama.py:99,108-122,563-578).
 */
int td_gemv(const void* w, int64_t w_row_stride, int32_t rows, int32_t cols, const void* x,
            int32_t x_mode, const void* norm_weight, float eps, const void* residual,
            int32_t pair_gated, void* y, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TIDAL_HIP_H_ */
