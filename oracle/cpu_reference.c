/*
 * CPU oracle, C part.  TEST INFRASTRUCTURE ONLY: linked by tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py, never by the product.
 *
 * Plain-C restatement of the reference's own CPU checker, kernels/src/include/cpu_reference.h,
 * whose original cannot be compiled here (it includes <flashinfer/rope.cuh> and CUDA headers,
 * cpu_reference.h:25-29).  All arithmetic is float32 on float32 arrays; callers round inputs to
 * fp16 / bf16 beforehand.
 *
 *   ref_apply_llama_rope        cpu_reference.h:36-53
 *   ref_single_mha              cpu_reference.h:55-159   (qo_len == 1, no in-kernel RoPE)
 *   ref_selected_single_mha     cpu_reference.h:161-292
 *   ref_append_paged_kv_cache   cpu_reference.h:294-327
 *   ref_k_elem_offset / ref_v_elem_offset   kernels/include/decode/decode_page.cuh:191-234
 *   ref_stable_topk             selection rule of the benchmark configuration: k largest,
 *                               ties to the lower index (no reference source; pinned against
 *                               torch.topk and brute force in tests/test_oracle.py)
 *
 * Pinned in tests/test_oracle.py against torch's scaled_dot_product_attention, against the
 * independent torch restatement in oracle/tidal_oracle.py and against hand-computed cases.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { REF_NHD = 0, REF_HND = 1 };

/* contiguous (non-paged) tensors: [len, H, D] for NHD, [H, len, D] for HND */
static size_t kv_elem_offset(int layout, size_t len, size_t num_heads, size_t head_dim, size_t pos,
                             size_t head, size_t feat) {
  return layout == REF_HND ? (head * len + pos) * head_dim + feat
                           : (pos * num_heads + head) * head_dim + feat;
}

int64_t ref_k_elem_offset(int64_t page, int64_t head, int64_t entry, int64_t feat,
                          int64_t num_heads, int64_t page_size, int64_t head_dim, int layout) {
  return layout == REF_HND
             ? ((page * 2 * num_heads + head) * page_size + entry) * head_dim + feat
             : ((page * 2 * page_size + entry) * num_heads + head) * head_dim + feat;
}

int64_t ref_v_elem_offset(int64_t page, int64_t head, int64_t entry, int64_t feat,
                          int64_t num_heads, int64_t page_size, int64_t head_dim, int layout) {
  return layout == REF_HND
             ? (((page * 2 + 1) * num_heads + head) * page_size + entry) * head_dim + feat
             : (((page * 2 + 1) * page_size + entry) * num_heads + head) * head_dim + feat;
}

/* out[k] = cos(a_k) in[k] + sin(a_k) perm[k], perm = (-in[D/2:], in[:D/2]),
 * a_k = (offset / scale) / theta^(2 (k mod D/2) / D), all in float as the reference does. */
void ref_apply_llama_rope(const float* in, int64_t D, int64_t offset, float rope_scale,
                          float rope_theta, float* out) {
  for (int64_t k = 0; k < D; ++k) {
    float perm = (k < D / 2) ? -in[k + D / 2] : in[k - D / 2];
    float inv_freq =
        ((float)offset / rope_scale) / powf(rope_theta, (float)(2 * (k % (D / 2))) / (float)D);
    out[k] = cosf(inv_freq) * in[k] + sinf(inv_freq) * perm;
  }
}

/* decode attention of one query token over a contiguous cache; o [Hq, D] */
void ref_single_mha(const float* q, const float* k, const float* v, int64_t kv_len,
                    int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int layout,
                    float* o) {
  const float sm_scale = 1.f / sqrtf((float)head_dim);
  const int64_t group = num_q_heads / num_kv_heads;
  float* att = (float*)malloc(sizeof(float) * (size_t)(kv_len > 0 ? kv_len : 1));
  for (int64_t qh = 0; qh < num_q_heads; ++qh) {
    const int64_t kvh = qh / group;
    float max_val = -5e4f;
    for (int64_t i = 0; i < kv_len; ++i) {
      float s = 0.f;
      for (int64_t f = 0; f < head_dim; ++f)
        s += q[qh * head_dim + f] *
             k[kv_elem_offset(layout, kv_len, num_kv_heads, head_dim, i, kvh, f)] * sm_scale;
      att[i] = s;
      if (s > max_val) max_val = s;
    }
    float denom = 0.f;
    for (int64_t i = 0; i < kv_len; ++i) {
      att[i] = expf(att[i] - max_val);
      denom += att[i];
    }
    for (int64_t i = 0; i < kv_len; ++i) att[i] /= denom;
    for (int64_t f = 0; f < head_dim; ++f) {
      float acc = 0.f;
      for (int64_t i = 0; i < kv_len; ++i)
        acc += att[i] * v[kv_elem_offset(layout, kv_len, num_kv_heads, head_dim, i, kvh, f)];
      o[qh * head_dim + f] = acc;
    }
  }
  free(att);
}

/*
 * Attention over selected pages of a contiguous cache.  selected [num_q_heads, page_budget]:
 * logical page numbers (page p covers tokens p*page_size ...); the LAST entry of every row is the
 * partially filled last page with last_len tokens, all others are full.  num_q_heads must equal
 * num_kv_heads (the reference asserts it, cpu_reference.h:181-182).
 */
void ref_selected_single_mha(const float* q, const float* k, const float* v,
                             const int32_t* selected, int64_t page_budget, int64_t last_len,
                             int64_t kv_len, int64_t page_size, int64_t num_heads,
                             int64_t head_dim, int layout, float* o) {
  const float sm_scale = 1.f / sqrtf((float)head_dim);
  const int64_t sel_len = (page_budget - 1) * page_size + last_len;
  float* att = (float*)malloc(sizeof(float) * (size_t)(sel_len > 0 ? sel_len : 1));
  int64_t* pos = (int64_t*)malloc(sizeof(int64_t) * (size_t)(sel_len > 0 ? sel_len : 1));
  for (int64_t h = 0; h < num_heads; ++h) {
    int64_t n = 0;
    float max_val = -5e4f;
    for (int64_t j = 0; j < page_budget; ++j) {
      const int64_t start = (int64_t)selected[h * page_budget + j] * page_size;
      const int64_t cur = (j == page_budget - 1) ? last_len : page_size;
      for (int64_t e = 0; e < cur; ++e) {
        const int64_t kv_idx = start + e;
        float s = 0.f;
        for (int64_t f = 0; f < head_dim; ++f)
          s += q[h * head_dim + f] *
               k[kv_elem_offset(layout, kv_len, num_heads, head_dim, kv_idx, h, f)] * sm_scale;
        att[n] = s;
        pos[n] = kv_idx;
        if (s > max_val) max_val = s;
        ++n;
      }
    }
    float denom = 0.f;
    for (int64_t i = 0; i < n; ++i) {
      att[i] = expf(att[i] - max_val);
      denom += att[i];
    }
    for (int64_t i = 0; i < n; ++i) att[i] /= denom;
    for (int64_t f = 0; f < head_dim; ++f) {
      float acc = 0.f;
      for (int64_t i = 0; i < n; ++i)
        acc += att[i] * v[kv_elem_offset(layout, kv_len, num_heads, head_dim, pos[i], h, f)];
      o[h * head_dim + f] = acc;
    }
  }
  free(att);
  free(pos);
}

/*
 * Append the last n_append tokens of a sequence that then holds seq_len tokens into a paged pool
 * (float32 stand-in of the pool, same shape as the device pool).  keys/values [n_append, H, D].
 */
void ref_append_paged_kv_cache(float* pool, const int32_t* page_indices, int64_t seq_len,
                               const float* keys, const float* values, int64_t n_append,
                               int64_t num_heads, int64_t page_size, int64_t head_dim, int layout) {
  const int64_t start = seq_len - n_append;
  for (int64_t j = 0; j < n_append; ++j) {
    const int64_t p = start + j;
    const int64_t page = page_indices[p / page_size];
    const int64_t entry = p % page_size;
    for (int64_t h = 0; h < num_heads; ++h) {
      memcpy(pool + ref_k_elem_offset(page, h, entry, 0, num_heads, page_size, head_dim, layout),
             keys + (j * num_heads + h) * head_dim, sizeof(float) * (size_t)head_dim);
      memcpy(pool + ref_v_elem_offset(page, h, entry, 0, num_heads, page_size, head_dim, layout),
             values + (j * num_heads + h) * head_dim, sizeof(float) * (size_t)head_dim);
    }
  }
}

typedef struct {
  float v;
  int32_t i;
} ref_pair;

static int pair_cmp(const void* a, const void* b) {
  const ref_pair* x = (const ref_pair*)a;
  const ref_pair* y = (const ref_pair*)b;
  /* NaN orders above everything, like torch.sort / torch.topk */
  const int xn = isnan(x->v), yn = isnan(y->v);
  if (xn != yn) return xn ? -1 : 1;
  if (!xn) {
    if (x->v > y->v) return -1;
    if (x->v < y->v) return 1;
  }
  return (x->i > y->i) - (x->i < y->i);
}

static int idx_cmp(const void* a, const void* b) {
  const int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
  return (x > y) - (x < y);
}

/* per row: indices of the k largest values, ties to the lower index, output ascending */
void ref_stable_topk(const float* values, int64_t rows, int64_t len, int64_t k, int32_t* out) {
  ref_pair* buf = (ref_pair*)malloc(sizeof(ref_pair) * (size_t)(len > 0 ? len : 1));
  if (k > len) k = len;
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t i = 0; i < len; ++i) {
      buf[i].v = values[r * len + i];
      buf[i].i = (int32_t)i;
    }
    qsort(buf, (size_t)len, sizeof(ref_pair), pair_cmp);
    for (int64_t j = 0; j < k; ++j) out[r * k + j] = buf[j].i;
    qsort(out + r * k, (size_t)k, sizeof(int32_t), idx_cmp);
  }
  free(buf);
}
