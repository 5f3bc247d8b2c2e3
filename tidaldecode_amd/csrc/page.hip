// Rotary embedding, paged KV append, their decode-step fusion, and RMSNorm for gfx950.
//
// RoPE is the rotate-half (Llama) form of kernels/include/decode/decode_page.cuh:639-687 of the
// reference; angles are formed in double precision (position * theta^(-2j/D) / scale) and only
// the sine / cosine are rounded to fp32, so positions of 1e5 and beyond lose nothing to the
// fp32 product the reference forms.  Append follows AppendPagedKVCacheDecode/Prefill
// (decode_page.cuh:387-557) including the per-page key max/min metadata.

#include "common.cuh"

namespace tidal {

struct PoolGeom {
  void* data;
  int64_t page_stride;
  int64_t v_offset;
  int32_t entry_stride;
  int32_t head_stride;
  int32_t page_size;
  int32_t num_heads;
  uint32_t max_page;
};

static PoolGeom geom_of(const td_paged_kv* kv) {
  PoolGeom g;
  const int P = kv->page_size, H = kv->num_kv_heads, D = kv->head_dim;
  g.data = kv->data;
  g.page_stride = (int64_t)2 * P * H * D;
  g.v_offset = (int64_t)P * H * D;
  if (kv->layout == TD_NHD) {
    g.entry_stride = H * D;
    g.head_stride = D;
  } else {
    g.entry_stride = D;
    g.head_stride = P * D;
  }
  g.page_size = P;
  g.num_heads = H;
  g.max_page = (uint32_t)(kv->max_pages - 1);
  return g;
}

__device__ __forceinline__ int64_t k_offset(const PoolGeom& g, uint32_t page, int entry, int head) {
  page = page > g.max_page ? g.max_page : page;
  return (int64_t)page * g.page_stride + (int64_t)entry * g.entry_stride +
         (int64_t)head * g.head_stride;
}

// sin / cos of position * theta^(-2j/D) / scale.  The angle is formed and reduced to a fraction
// of a turn in double precision (exact to ~1e-10 rad at positions of 1e6); only the reduced
// argument, |x| <= 1, goes through the fp32 sincospi.
__device__ __forceinline__ void rope_sincos(double pos_over_scale, double log2_theta, int j, int D,
                                            float& sn, float& cs) {
  const double inv_freq = exp2(-log2_theta * (double)(2 * j) / (double)D);
  double turns = pos_over_scale * inv_freq * 0.15915494309189535;  // / (2 pi)
  turns -= rint(turns);                                            // [-0.5, 0.5]
  sincospif((float)(2.0 * turns), &sn, &cs);
}

template <typename T>
__device__ __forceinline__ void rotate_pair(uint16_t* row, int j, int half, float sn, float cs) {
  const float lo = to_float<T>(row[j]);
  const float hi = to_float<T>(row[j + half]);
  row[j] = from_float<T>(lo * cs - hi * sn);
  row[j + half] = from_float<T>(hi * cs + lo * sn);
}

// grid: n_tokens; block: 256 threads = (D/2 pair columns) x (512/D head slots)
template <typename T>
__global__ __launch_bounds__(256) void rope_kernel(uint16_t* q, uint16_t* k, int n_tokens, int Hq,
                                                   int Hkv, int D, double past_len,
                                                   double inv_scale, double log2_theta) {
  const int tok = blockIdx.x;
  const int half = D / 2;
  const int j = threadIdx.x % half;
  const int slot = threadIdx.x / half;
  const int slots = 256 / half;
  if (slot >= slots) return;
  float sn, cs;
  rope_sincos((past_len + (double)tok) * inv_scale, log2_theta, j, D, sn, cs);
  for (int h = slot; h < Hq + Hkv; h += slots) {
    uint16_t* row = h < Hq ? q + ((int64_t)tok * Hq + h) * D : k + ((int64_t)tok * Hkv + (h - Hq)) * D;
    rotate_pair<T>(row, j, half, sn, cs);
  }
}

// grid: batch; block: D/2 threads.  cos/sin of one token's rotary angles
__global__ void rope_table_kernel(const int32_t* positions, int D, double inv_scale,
                                  double log2_theta, float* cos_out, float* sin_out) {
  const int b = blockIdx.x, j = threadIdx.x;
  float sn, cs;
  rope_sincos((double)positions[b] * inv_scale, log2_theta, j, D, sn, cs);
  cos_out[(int64_t)b * (D / 2) + j] = cs;
  sin_out[(int64_t)b * (D / 2) + j] = sn;
}

// grid: batch; rotates q in place, rotates k into the cache slot, copies v into the cache slot
template <typename T>
__global__ __launch_bounds__(256) void rope_append_decode_kernel(
    PoolGeom g, uint16_t* q, const uint16_t* k, const uint16_t* v, int Hq, int D,
    const int32_t* positions, const int32_t* dst_slot, double inv_scale, double log2_theta) {
  const int b = blockIdx.x;
  const int Hkv = g.num_heads;
  const int half = D / 2;
  const int j = threadIdx.x % half;
  const int slot = threadIdx.x / half;
  const int slots = 256 / half;
  if (slot >= slots) return;
  const uint32_t dst = (uint32_t)dst_slot[b];
  uint32_t page = dst / (uint32_t)g.page_size;
  const int entry = (int)(dst - page * (uint32_t)g.page_size);
  page = page > g.max_page ? g.max_page : page;  // a bad slot lands inside the pool, as in the fused step
  float sn, cs;
  rope_sincos((double)positions[b] * inv_scale, log2_theta, j, D, sn, cs);
  uint16_t* pool = reinterpret_cast<uint16_t*>(g.data);
  for (int h = slot; h < Hq + Hkv; h += slots) {
    if (h < Hq) {
      rotate_pair<T>(q + ((int64_t)b * Hq + h) * D, j, half, sn, cs);
    } else {
      const int hk = h - Hq;
      const uint16_t* krow = k + ((int64_t)b * Hkv + hk) * D;
      const uint16_t* vrow = v + ((int64_t)b * Hkv + hk) * D;
      uint16_t* kdst = pool + k_offset(g, page, entry, hk);
      const float lo = to_float<T>(krow[j]);
      const float hi = to_float<T>(krow[j + half]);
      kdst[j] = from_float<T>(lo * cs - hi * sn);
      kdst[j + half] = from_float<T>(hi * cs + lo * sn);
      kdst[g.v_offset + j] = vrow[j];
      kdst[g.v_offset + j + half] = vrow[j + half];
    }
  }
}

// grid: n_tokens; copies one token's K and V rows (all heads) into its page slot, 16 B per lane
__global__ __launch_bounds__(256) void append_copy_kernel(PoolGeom g, const uint16_t* k,
                                                          const uint16_t* v, int n_tokens, int D,
                                                          const int32_t* indices,
                                                          const int32_t* indptr, int last_page_len) {
  const int tok = blockIdx.x;
  const int H = g.num_heads;
  const int n_pages = indptr[1] - indptr[0];
  const int seq_len = (n_pages - 1) * g.page_size + last_page_len;
  const int pos = seq_len - n_tokens + tok;
  if (pos < 0 || n_pages <= 0) return;
  const int pg = pos / g.page_size;
  const int entry = pos - pg * g.page_size;
  const uint32_t page = (uint32_t)indices[indptr[0] + pg];
  uint16_t* pool = reinterpret_cast<uint16_t*>(g.data);
  const int vec_per_row = D / 8;
  for (int x = threadIdx.x; x < H * vec_per_row; x += 256) {
    const int h = x / vec_per_row;
    const int c = (x - h * vec_per_row) * 8;
    const int64_t src = ((int64_t)tok * H + h) * D + c;
    uint16_t* dst = pool + k_offset(g, page, entry, h) + c;
    *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(k + src);
    *reinterpret_cast<u32x4*>(dst + g.v_offset) = *reinterpret_cast<const u32x4*>(v + src);
  }
}

// Per KV page touched by the append: element-wise running max (K plane) / min (V plane) of the
// page's keys, kept at entry (page ordinal) of the metadata pool.  grid: (touched pages, heads)
template <typename T>
__global__ void append_meta_kernel(PoolGeom kvg, PoolGeom mg, const uint16_t* k, int n_tokens,
                                   int D, const int32_t* kv_indptr, int last_page_len,
                                   const int32_t* meta_indices, const int32_t* meta_indptr,
                                   float type_max) {
  const int h = blockIdx.y;
  const int d = threadIdx.x;  // one element per thread, D threads
  const int H = kvg.num_heads;
  const int P = kvg.page_size;
  const int n_pages = kv_indptr[1] - kv_indptr[0];
  const int seq_len = (n_pages - 1) * P + last_page_len;
  const int start = seq_len - n_tokens;
  if (start < 0 || n_pages <= 0) return;
  const int pg = start / P + blockIdx.x;  // ordinal of the KV page inside the sequence
  if (pg >= n_pages) return;
  int e0 = start - pg * P;
  e0 = e0 < 0 ? 0 : e0;
  int e1 = seq_len - pg * P;
  e1 = e1 > P ? P : e1;
  const int mP = mg.page_size;
  const uint32_t mpage = (uint32_t)meta_indices[meta_indptr[0] + pg / mP];
  uint16_t* mrow = reinterpret_cast<uint16_t*>(mg.data) + k_offset(mg, mpage, pg % mP, h);
  float mx = -type_max, mn = type_max;
  if (e0 > 0) {
    mx = to_float<T>(mrow[d]);
    mn = to_float<T>(mrow[mg.v_offset + d]);
  }
  for (int e = e0; e < e1; ++e) {
    const int tok = pg * P + e - start;
    const float x = to_float<T>(k[((int64_t)tok * H + h) * D + d]);
    mx = fmaxf(mx, x);
    mn = fminf(mn, x);
  }
  mrow[d] = from_float<T>(mx);
  mrow[mg.v_offset + d] = from_float<T>(mn);
}

// Upper bound of q.k over the keys of a page from the page's element-wise max / min metadata:
// o[h, e] = sum_d max(q[h, d] * max[e, d], q[h, d] * min[e, d]).  A 16-byte lane group per
// metadata entry; grid: (ceil(entries / entries per workgroup), query heads).
template <typename T, int D>
__global__ __launch_bounds__(256) void estimate_kernel(PoolGeom mg, const int32_t* meta_indices,
                                                       int n_entries, const uint16_t* q,
                                                       int q_per_kv, uint16_t* o, int64_t o_stride) {
  constexpr int LPR = D / 8;
  constexpr int EPB = 256 / LPR;  // entries per workgroup
  const int tid = threadIdx.x;
  const int li = tid % LPR;
  const int e = blockIdx.x * EPB + tid / LPR;
  const int h = blockIdx.y;
  const int ec = e < n_entries ? e : n_entries - 1;  // clamped: loads stay unconditional
  const uint32_t page = (uint32_t)meta_indices[ec / mg.page_size];
  const uint16_t* row = reinterpret_cast<const uint16_t*>(mg.data) +
                        k_offset(mg, page, ec % mg.page_size, h / q_per_kv) + li * 8;
  const u32x4 mx = *reinterpret_cast<const u32x4*>(row);
  const u32x4 mn = *reinterpret_cast<const u32x4*>(row + mg.v_offset);
  const u32x4 qv = *reinterpret_cast<const u32x4*>(q + (int64_t)h * D + li * 8);
  const uint32_t mxw[4] = {mx.x, mx.y, mx.z, mx.w}, mnw[4] = {mn.x, mn.y, mn.z, mn.w},
                 qw[4] = {qv.x, qv.y, qv.z, qv.w};
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    float q0, q1, a0, a1, b0, b1;
    unpack2<T>(qw[c], q0, q1);
    unpack2<T>(mxw[c], a0, a1);
    unpack2<T>(mnw[c], b0, b1);
    acc += fmaxf(q0 * a0, q0 * b0);
    acc += fmaxf(q1 * a1, q1 * b1);
  }
  acc = group_sum<LPR>(acc);
  if (li == 0 && e < n_entries) o[(int64_t)h * o_stride + e] = from_float<T>(acc);
}

// RMSNorm, one 256-thread workgroup per row, fp32 accumulation.
// Sum of squares over the workgroup: every wave reduces by butterfly, four partials through LDS.
__device__ __forceinline__ float rms_block_sum(float ss) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  __shared__ float part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  return part[0] + part[1] + part[2] + part[3];
}

// Rows of up to CH*2048 elements with 16-byte alignment: the row is read once, as CH independent
// 16-byte loads per thread issued back to back, and stays in registers between the two passes.
// Threads past the end of the row reload the row's last chunk (an unconditional load keeps all
// loads in flight together; a predicated one is waited for inside its branch) and drop it.
template <typename T, int CH>
__global__ __launch_bounds__(256) void rms_norm_vec_kernel(const uint16_t* x, const uint16_t* w,
                                                           uint16_t* out, int cols, float eps) {
  const int64_t base = (int64_t)blockIdx.x * cols;
  uint4 xv[CH], wv[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = min((i * 256 + (int)threadIdx.x) * 8, cols - 8);
    xv[i] = *reinterpret_cast<const uint4*>(x + base + c);
  }
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = min((i * 256 + (int)threadIdx.x) * 8, cols - 8);
    wv[i] = *reinterpret_cast<const uint4*>(w + c);
  }
  float xf[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const uint32_t xw[4] = {xv[i].x, xv[i].y, xv[i].z, xv[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) unpack2<T>(xw[j], xf[i][2 * j], xf[i][2 * j + 1]);
    if ((i * 256 + (int)threadIdx.x) * 8 < cols) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(xf[i][j], xf[i][j], ss);
    }
  }
  const float inv = rsqrtf(rms_block_sum(ss) / (float)cols + eps);
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = (i * 256 + (int)threadIdx.x) * 8;
    if (c < cols) {
      const uint32_t ww[4] = {wv[i].x, wv[i].y, wv[i].z, wv[i].w};
      uint32_t ow[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float w0, w1;
        unpack2<T>(ww[j], w0, w1);
        ow[j] = pack2<T>(xf[i][2 * j] * inv * w0, xf[i][2 * j + 1] * inv * w1);
      }
      *reinterpret_cast<uint4*>(out + base + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
  }
}

// Any other row length or alignment: two passes of 2-byte accesses.
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_kernel(const uint16_t* x, const uint16_t* w,
                                                       uint16_t* out, int cols, float eps) {
  const int row = blockIdx.x;
  const uint16_t* xr = x + (int64_t)row * cols;
  uint16_t* orow = out + (int64_t)row * cols;
  float ss = 0.f;
#pragma unroll 4
  for (int c = threadIdx.x; c < cols; c += 256) {
    const float f = to_float<T>(xr[c]);
    ss = fmaf(f, f, ss);
  }
  const float inv = rsqrtf(rms_block_sum(ss) / (float)cols + eps);
#pragma unroll 4
  for (int c = threadIdx.x; c < cols; c += 256)
    orow[c] = from_float<T>(to_float<T>(xr[c]) * inv * to_float<T>(w[c]));
}

template <typename T>
static void launch_rms_norm(const void* x, const void* weight, void* out, int rows, int cols,
                            float eps, hipStream_t st) {
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)weight;
  uint16_t* op = (uint16_t*)out;
  const bool vec = cols % 8 == 0 && cols <= 8 * 2048 &&
                   (((uintptr_t)x | (uintptr_t)weight | (uintptr_t)out) & 15) == 0;
#define TD_RMS(CH) \
  hipLaunchKernelGGL((rms_norm_vec_kernel<T, CH>), dim3(rows), dim3(256), 0, st, xp, wp, op, cols, eps)
  if (!vec) hipLaunchKernelGGL(rms_norm_kernel<T>, dim3(rows), dim3(256), 0, st, xp, wp, op, cols, eps);
  else if (cols <= 2048) TD_RMS(1);
  else if (cols <= 2 * 2048) TD_RMS(2);
  else if (cols <= 4 * 2048) TD_RMS(4);
  else TD_RMS(8);
#undef TD_RMS
}

static int check_pool(const td_paged_kv* kv, const char* who) {
  TD_REQUIRE(kv && kv->data, "%s: pool is NULL", who);
  TD_REQUIRE(kv->num_kv_heads >= 1 && kv->page_size >= 1 && kv->max_pages >= 1,
             "%s: pool heads %d page_size %d max_pages %lld", who, kv->num_kv_heads, kv->page_size,
             (long long)kv->max_pages);
  TD_REQUIRE(kv->layout == TD_NHD || kv->layout == TD_HND, "%s: layout %d", who, kv->layout);
  TD_REQUIRE(kv->max_pages * kv->page_size < ((int64_t)1 << 31), "%s: pool too large for int32 slots",
             who);
  return TD_OK;
}

}  // namespace tidal

using namespace tidal;

extern "C" int td_rope_in_place(void* q, void* k, int32_t n_tokens, int32_t num_qo_heads,
                                int32_t num_kv_heads, int32_t head_dim, int64_t past_kv_len,
                                float rope_scale, float rope_theta, int32_t dtype, void* stream) {
  TD_REQUIRE(q && k, "apply_rope_in_place: NULL q or k");
  TD_REQUIRE(n_tokens >= 0 && num_qo_heads >= 1 && num_kv_heads >= 1,
             "apply_rope_in_place: n_tokens %d heads %d/%d", n_tokens, num_qo_heads, num_kv_heads);
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(TD_ERR_UNSUPPORTED, "apply_rope_in_place: head_dim %d (supported: 64, 128, 256)",
                head_dim);
  TD_REQUIRE(rope_scale > 0.f && rope_theta > 0.f, "apply_rope_in_place: scale %g theta %g",
             rope_scale, rope_theta);
  TD_REQUIRE(past_kv_len >= 0, "apply_rope_in_place: past_kv_len %lld", (long long)past_kv_len);
  if (n_tokens == 0) return TD_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const double inv_scale = 1.0 / (double)rope_scale;
  const double log2_theta = log2((double)rope_theta);
  if (dtype == TD_F16)
    hipLaunchKernelGGL(rope_kernel<F16>, dim3(n_tokens), dim3(256), 0, st, (uint16_t*)q,
                       (uint16_t*)k, n_tokens, num_qo_heads, num_kv_heads, head_dim,
                       (double)past_kv_len, inv_scale, log2_theta);
  else if (dtype == TD_BF16)
    hipLaunchKernelGGL(rope_kernel<BF16>, dim3(n_tokens), dim3(256), 0, st, (uint16_t*)q,
                       (uint16_t*)k, n_tokens, num_qo_heads, num_kv_heads, head_dim,
                       (double)past_kv_len, inv_scale, log2_theta);
  else
    return fail(TD_ERR_UNSUPPORTED, "apply_rope_in_place failed to dispatch with dtype %d", dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_append_kv(const td_paged_kv* kv, const void* k, const void* v, int32_t n_tokens,
                            const int32_t* kv_indices, const int32_t* kv_indptr,
                            int32_t last_page_len, const td_paged_kv* meta,
                            const int32_t* meta_indices, const int32_t* meta_indptr,
                            int32_t meta_last_page_len, void* stream) {
  (void)meta_last_page_len;
  int rc = check_pool(kv, "append_kv_cache");
  if (rc) return rc;
  TD_REQUIRE(k && v && kv_indices && kv_indptr, "append_kv_cache: NULL argument");
  TD_REQUIRE(n_tokens >= 0, "append_kv_cache: n_tokens %d", n_tokens);
  TD_REQUIRE(last_page_len >= 1 && last_page_len <= kv->page_size,
             "append_kv_cache: last_page_len %d not in [1, %d]", last_page_len, kv->page_size);
  const int D = kv->head_dim;
  if (D != 64 && D != 128 && D != 256)
    return fail(TD_ERR_UNSUPPORTED, "append_kv_cache: head_dim %d (supported: 64, 128, 256)", D);
  if (kv->dtype != TD_F16 && kv->dtype != TD_BF16)
    return fail(TD_ERR_UNSUPPORTED, "Append_kv_cache failed to dispatch with dtype %d", kv->dtype);
  if (n_tokens == 0) return TD_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const PoolGeom g = geom_of(kv);
  hipLaunchKernelGGL(append_copy_kernel, dim3(n_tokens), dim3(256), 0, st, g, (const uint16_t*)k,
                     (const uint16_t*)v, n_tokens, D, kv_indices, kv_indptr, last_page_len);
  TD_HIP_CHECK(hipGetLastError());
  if (meta && meta->data) {
    rc = check_pool(meta, "append_kv_cache(metadata)");
    if (rc) return rc;
    TD_REQUIRE(meta_indices && meta_indptr, "append_kv_cache: NULL metadata indices");
    TD_REQUIRE(meta->num_kv_heads == kv->num_kv_heads && meta->head_dim == D &&
                   meta->dtype == kv->dtype,
               "append_kv_cache: metadata pool shape differs from the KV pool");
    const PoolGeom mg = geom_of(meta);
    // pages touched by n_tokens appended tokens: at most ceil(n/P) + 1
    const int touched = (n_tokens + kv->page_size - 1) / kv->page_size + 1;
    dim3 grid(touched, kv->num_kv_heads);
    if (kv->dtype == TD_F16)
      hipLaunchKernelGGL(append_meta_kernel<F16>, grid, dim3(D), 0, st, g, mg, (const uint16_t*)k,
                         n_tokens, D, kv_indptr, last_page_len, meta_indices, meta_indptr, 65504.f);
    else
      hipLaunchKernelGGL(append_meta_kernel<BF16>, grid, dim3(D), 0, st, g, mg, (const uint16_t*)k,
                         n_tokens, D, kv_indptr, last_page_len, meta_indices, meta_indptr,
                         3.3895313892515355e38f);
    TD_HIP_CHECK(hipGetLastError());
  }
  return TD_OK;
}

extern "C" int td_rope_append_decode(const td_paged_kv* kv, void* q, const void* k, const void* v,
                                     int32_t batch, int32_t num_qo_heads, const int32_t* positions,
                                     const int32_t* dst_slot, float rope_scale, float rope_theta,
                                     void* stream) {
  int rc = check_pool(kv, "td_rope_append_decode");
  if (rc) return rc;
  TD_REQUIRE(q && k && v && positions && dst_slot, "td_rope_append_decode: NULL argument");
  TD_REQUIRE(batch >= 1 && num_qo_heads >= 1, "td_rope_append_decode: batch %d heads %d", batch,
             num_qo_heads);
  TD_REQUIRE(rope_scale > 0.f && rope_theta > 0.f, "td_rope_append_decode: scale %g theta %g",
             rope_scale, rope_theta);
  const int D = kv->head_dim;
  if (D != 64 && D != 128 && D != 256)
    return fail(TD_ERR_UNSUPPORTED, "td_rope_append_decode: head_dim %d (supported: 64, 128, 256)",
                D);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const PoolGeom g = geom_of(kv);
  const double inv_scale = 1.0 / (double)rope_scale;
  const double log2_theta = log2((double)rope_theta);
  if (kv->dtype == TD_F16)
    hipLaunchKernelGGL(rope_append_decode_kernel<F16>, dim3(batch), dim3(256), 0, st, g,
                       (uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, num_qo_heads, D,
                       positions, dst_slot, inv_scale, log2_theta);
  else if (kv->dtype == TD_BF16)
    hipLaunchKernelGGL(rope_append_decode_kernel<BF16>, dim3(batch), dim3(256), 0, st, g,
                       (uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, num_qo_heads, D,
                       positions, dst_slot, inv_scale, log2_theta);
  else
    return fail(TD_ERR_UNSUPPORTED, "td_rope_append_decode failed to dispatch with dtype %d",
                kv->dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_rope_table(const int32_t* positions, int32_t batch, int32_t head_dim,
                             float rope_scale, float rope_theta, float* cos, float* sin,
                             void* stream) {
  TD_REQUIRE(positions && cos && sin, "td_rope_table: NULL argument");
  TD_REQUIRE(batch >= 1, "td_rope_table: batch %d", batch);
  TD_REQUIRE(rope_scale > 0.f && rope_theta > 0.f, "td_rope_table: scale %g theta %g", rope_scale,
             rope_theta);
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(TD_ERR_UNSUPPORTED, "td_rope_table: head_dim %d (supported: 64, 128, 256)", head_dim);
  hipLaunchKernelGGL(rope_table_kernel, dim3(batch), dim3(head_dim / 2), 0,
                     reinterpret_cast<hipStream_t>(stream), positions, head_dim,
                     1.0 / (double)rope_scale, log2((double)rope_theta), cos, sin);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

// Merge of attention states: part i of a row holds the attention output o_i over its own subset of
// the tokens and the log-sum-exp lse_i of that subset's logits; the attention over the union is
// o = sum_i o_i e^(lse_i - lse), lse = log sum_i e^(lse_i).  One workgroup of D/2 threads per row.
// DT: 0 f16, 1 bf16, 2 f32 (parts and result share the type; the arithmetic is fp32).
template <int DT>
__global__ void merge_states_kernel(const void* o_parts, const float* lse_parts, int32_t n_parts,
                                    int32_t rows, int32_t head_dim, void* o, float* lse) {
  const int row = blockIdx.x;
  const int d2 = threadIdx.x;  // pair of dimensions
  float mx = -INFINITY;
  for (int i = 0; i < n_parts; ++i) mx = fmaxf(mx, lse_parts[(int64_t)i * rows + row]);
  float wsum = 0.f, a = 0.f, b = 0.f;
  if (mx > -INFINITY) {
    for (int i = 0; i < n_parts; ++i) {
      const float w = __expf(lse_parts[(int64_t)i * rows + row] - mx);  // 0 for an empty part
      const int64_t at = ((int64_t)i * rows + row) * head_dim + 2 * d2;
      float x, y;
      if constexpr (DT == 2) {
        x = reinterpret_cast<const float*>(o_parts)[at];
        y = reinterpret_cast<const float*>(o_parts)[at + 1];
      } else if constexpr (DT == 0) {
        unpack2<F16>(reinterpret_cast<const uint32_t*>(o_parts)[at / 2], x, y);
      } else {
        unpack2<BF16>(reinterpret_cast<const uint32_t*>(o_parts)[at / 2], x, y);
      }
      if (w > 0.f) {  // an empty part may hold anything, NaN included
        wsum += w;
        a = fmaf(w, x, a);
        b = fmaf(w, y, b);
      }
    }
  }
  const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
  const int64_t out = (int64_t)row * head_dim + 2 * d2;
  if constexpr (DT == 2) {
    reinterpret_cast<float*>(o)[out] = a * inv;
    reinterpret_cast<float*>(o)[out + 1] = b * inv;
  } else if constexpr (DT == 0) {
    reinterpret_cast<uint32_t*>(o)[out / 2] = pack2<F16>(a * inv, b * inv);
  } else {
    reinterpret_cast<uint32_t*>(o)[out / 2] = pack2<BF16>(a * inv, b * inv);
  }
  if (lse && d2 == 0) lse[row] = wsum > 0.f ? mx + __logf(wsum) : -INFINITY;
}

extern "C" int td_merge_states(const void* o_parts, int32_t dtype, const float* lse_parts,
                               int32_t n_parts, int32_t rows, int32_t head_dim, void* o, float* lse,
                               void* stream) {
  TD_REQUIRE(o_parts && lse_parts && o, "td_merge_states: NULL argument");
  TD_REQUIRE(n_parts >= 1 && rows >= 1, "td_merge_states: %d parts, %d rows", n_parts, rows);
  TD_REQUIRE(head_dim >= 2 && head_dim % 2 == 0 && head_dim <= 2048,
             "td_merge_states: head_dim %d (even, at most 2048)", head_dim);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(rows), block(head_dim / 2);
  if (dtype == TD_F16)
    hipLaunchKernelGGL(merge_states_kernel<0>, grid, block, 0, st, o_parts, lse_parts, n_parts, rows,
                       head_dim, o, lse);
  else if (dtype == TD_BF16)
    hipLaunchKernelGGL(merge_states_kernel<1>, grid, block, 0, st, o_parts, lse_parts, n_parts, rows,
                       head_dim, o, lse);
  else if (dtype == TD_F32)
    hipLaunchKernelGGL(merge_states_kernel<2>, grid, block, 0, st, o_parts, lse_parts, n_parts, rows,
                       head_dim, o, lse);
  else
    return fail(TD_ERR_UNSUPPORTED, "td_merge_states failed to dispatch with dtype %d", dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

// Index of the largest of n values (NaN counts as largest, ties go to the lower index): the
// greedy choice of the next token, kept on the device.  One workgroup; DT: 0 f16, 1 bf16, 2 f32.
template <int DT>
__global__ __launch_bounds__(1024) void argmax_kernel(const void* x, int32_t n, int64_t* out) {
  __shared__ float sv[16];
  __shared__ int32_t si[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float best = -INFINITY;
  int32_t at = 0x7fffffff;
  for (int i = tid; i < n; i += 1024) {
    float v;
    if constexpr (DT == 0)
      v = to_float<F16>(reinterpret_cast<const uint16_t*>(x)[i]);
    else if constexpr (DT == 1)
      v = to_float<BF16>(reinterpret_cast<const uint16_t*>(x)[i]);
    else
      v = reinterpret_cast<const float*>(x)[i];
    v = (v != v) ? INFINITY : v;  // NaN ranks with +inf; the lower index wins among equals
    if (v > best || (v == best && i < at)) { best = v; at = i; }
  }
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int32_t oi = __shfl_xor(at, off, 64);
    if (ov > best || (ov == best && oi < at)) { best = ov; at = oi; }
  }
  if (lane == 0) { sv[wave] = best; si[wave] = at; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < at)) { best = sv[w]; at = si[w]; }
    out[0] = at == 0x7fffffff ? 0 : at;
  }
}

extern "C" int td_argmax(const void* x, int32_t dtype, int32_t n, int64_t* out, void* stream) {
  TD_REQUIRE(x && out, "td_argmax: NULL argument");
  TD_REQUIRE(n >= 1, "td_argmax: n %d < 1", n);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == TD_F16)
    hipLaunchKernelGGL(argmax_kernel<0>, dim3(1), dim3(1024), 0, st, x, n, out);
  else if (dtype == TD_BF16)
    hipLaunchKernelGGL(argmax_kernel<1>, dim3(1), dim3(1024), 0, st, x, n, out);
  else if (dtype == TD_F32)
    hipLaunchKernelGGL(argmax_kernel<2>, dim3(1), dim3(1024), 0, st, x, n, out);
  else
    return fail(TD_ERR_UNSUPPORTED, "td_argmax failed to dispatch with dtype %d", dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

// One thread: the sequence grows by one token; everything a decode step's launches read about the
// sequence is recomputed from the new length and the page table.
__global__ void step_advance_kernel(int32_t* state, const int32_t* page_table, int32_t n_pages,
                                    int32_t page_size, int32_t budget, const int64_t* token,
                                    int64_t* tokens_out, int32_t tokens_cap) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const int32_t step = state[TD_STEP_COUNT];
  if (token && tokens_out && step < tokens_cap) tokens_out[step] = *token;
  const int32_t n = state[TD_STEP_SEQ_LEN] + 1;
  const int32_t pos = n - 1;
  int32_t pi = pos / page_size;
  pi = pi < n_pages ? pi : n_pages - 1;  // a length beyond the table cannot index past it
  const int32_t entry = pos - (pos / page_size) * page_size;
  const int32_t page = page_table[pi];
  state[TD_STEP_SEQ_LEN] = n;
  state[TD_STEP_PAGES_BEFORE_LAST] = pi;
  state[TD_STEP_LAST_PAGE_LEN] = entry + 1;
  state[TD_STEP_LAST_PAGE_IDX] = page;
  state[TD_STEP_DST_SLOT] = page * page_size + entry;
  state[TD_STEP_POSITION] = pos;
  state[TD_STEP_N_SELECTED] = n < budget ? n : budget;
  state[TD_STEP_COUNT] = step + 1;
}

// The same for a batch: word w of sequence b is state[w * stride + b], sequence b's pages are row
// b of page_table.  One thread per sequence.
__global__ void step_advance_batch_kernel(int32_t* state, int32_t stride, int32_t batch,
                                          const int32_t* page_table, int32_t table_stride,
                                          int32_t page_size, int32_t budget) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  int32_t* st = state + b;
  const int32_t n = st[TD_STEP_SEQ_LEN * stride] + 1;
  const int32_t pos = n - 1;
  int32_t pi = pos / page_size;
  pi = pi < table_stride ? pi : table_stride - 1;
  const int32_t entry = pos - (pos / page_size) * page_size;
  const int32_t page = page_table[(int64_t)b * table_stride + pi];
  st[TD_STEP_SEQ_LEN * stride] = n;
  st[TD_STEP_PAGES_BEFORE_LAST * stride] = pi;
  st[TD_STEP_LAST_PAGE_LEN * stride] = entry + 1;
  st[TD_STEP_LAST_PAGE_IDX * stride] = page;
  st[TD_STEP_DST_SLOT * stride] = page * page_size + entry;
  st[TD_STEP_POSITION * stride] = pos;
  st[TD_STEP_N_SELECTED * stride] = n < budget ? n : budget;
  st[TD_STEP_COUNT * stride] += 1;
}

extern "C" int td_step_advance_batch(int32_t* state, int32_t stride, int32_t batch,
                                     const int32_t* page_table, int32_t table_stride,
                                     int32_t page_size, int32_t budget, void* stream) {
  TD_REQUIRE(state && page_table, "td_step_advance_batch: NULL argument");
  TD_REQUIRE(batch >= 1 && stride >= batch, "td_step_advance_batch: batch %d, stride %d", batch, stride);
  TD_REQUIRE(table_stride >= 1 && page_size >= 1 && budget >= 0,
             "td_step_advance_batch: %d pages of %d per sequence, budget %d", table_stride, page_size,
             budget);
  hipLaunchKernelGGL(step_advance_batch_kernel, dim3((batch + 63) / 64), dim3(64), 0,
                     reinterpret_cast<hipStream_t>(stream), state, stride, batch, page_table,
                     table_stride, page_size, budget);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_step_advance(int32_t* state, const int32_t* page_table, int32_t n_pages,
                               int32_t page_size, int32_t budget, const int64_t* token,
                               int64_t* tokens_out, int32_t tokens_cap, void* stream) {
  TD_REQUIRE(state && page_table, "td_step_advance: NULL argument");
  TD_REQUIRE(n_pages >= 1 && page_size >= 1 && budget >= 0,
             "td_step_advance: %d pages of %d, budget %d", n_pages, page_size, budget);
  TD_REQUIRE((token == nullptr) == (tokens_out == nullptr) && tokens_cap >= 0,
             "td_step_advance: token and tokens_out go together");
  hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(64), 0,
                     reinterpret_cast<hipStream_t>(stream), state, page_table, n_pages, page_size,
                     budget, token, tokens_out, tokens_cap);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_estimate_score(const td_paged_kv* meta, const int32_t* meta_indices,
                                 int32_t n_meta_pages, int32_t meta_last_page_len, const void* q,
                                 int32_t num_qo_heads, void* o, int64_t o_stride, void* stream) {
  int rc = check_pool(meta, "td_estimate_score");
  if (rc) return rc;
  TD_REQUIRE(meta_indices && q && o, "td_estimate_score: NULL argument");
  TD_REQUIRE(num_qo_heads >= meta->num_kv_heads && num_qo_heads % meta->num_kv_heads == 0,
             "td_estimate_score: num_qo_heads %d is not a multiple of num_kv_heads %d",
             num_qo_heads, meta->num_kv_heads);
  TD_REQUIRE(n_meta_pages >= 1 && meta_last_page_len >= 1 && meta_last_page_len <= meta->page_size,
             "td_estimate_score: %d pages, last page length %d", n_meta_pages, meta_last_page_len);
  // the newest entry describes the page still being filled and is left out, as in the reference
  const int n_entries = (n_meta_pages - 1) * meta->page_size + meta_last_page_len - 1;
  TD_REQUIRE(o_stride >= n_entries, "td_estimate_score: o_stride %lld < %d entries",
             (long long)o_stride, n_entries);
  if (n_entries == 0) return TD_OK;
  const PoolGeom mg = geom_of(meta);
  const int D = meta->head_dim;
  const int qpk = num_qo_heads / meta->num_kv_heads;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const uint16_t* qp = reinterpret_cast<const uint16_t*>(q);
  uint16_t* op = reinterpret_cast<uint16_t*>(o);
#define TD_EST(T, DD)                                                                            \
  hipLaunchKernelGGL((estimate_kernel<T, DD>), dim3((n_entries + 2048 / DD - 1) / (2048 / DD),   \
                                                    num_qo_heads),                               \
                     dim3(256), 0, st, mg, meta_indices, n_entries, qp, qpk, op, o_stride)
  if (meta->dtype == TD_F16) {
    if (D == 64) TD_EST(F16, 64);
    else if (D == 128) TD_EST(F16, 128);
    else if (D == 256) TD_EST(F16, 256);
    else return fail(TD_ERR_UNSUPPORTED, "estimate_attn_score failed to dispatch with head_dim %d", D);
  } else if (meta->dtype == TD_BF16) {
    if (D == 64) TD_EST(BF16, 64);
    else if (D == 128) TD_EST(BF16, 128);
    else if (D == 256) TD_EST(BF16, 256);
    else return fail(TD_ERR_UNSUPPORTED, "estimate_attn_score failed to dispatch with head_dim %d", D);
  } else {
    return fail(TD_ERR_UNSUPPORTED, "estimate_attn_score failed to dispatch with dtype %d", meta->dtype);
  }
#undef TD_EST
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}

extern "C" int td_rms_norm(const void* x, const void* weight, void* out, int32_t rows,
                           int32_t cols, float eps, int32_t dtype, void* stream) {
  TD_REQUIRE(x && weight && out, "rms_norm_forward: NULL argument");
  TD_REQUIRE(rows >= 0 && cols >= 1, "rms_norm_forward: rows %d cols %d", rows, cols);
  if (rows == 0) return TD_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == TD_F16)
    launch_rms_norm<F16>(x, weight, out, rows, cols, eps, st);
  else if (dtype == TD_BF16)
    launch_rms_norm<BF16>(x, weight, out, rows, cols, eps, st);
  else
    return fail(TD_ERR_UNSUPPORTED, "rms_norm_forward failed to dispatch with dtype %d", dtype);
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
