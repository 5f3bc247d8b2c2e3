// Causal attention of the n_q newest tokens of a sequence over its paged KV cache (prefill) for
// gfx950 (MI355X), on the matrix cores.  Replaces BatchPrefillWithPagedKVCache of the reference
// (kernels/include/prefill/prefill.cuh:674-870, bound in tidal/ops/csrc/batch_prefill.cu:27-117).
//
// One workgroup of NW = 4 or 8 wavefronts per (16 MT NW query rows, query head); a wavefront owns
// 16 MT query rows as MT = 2 16-row tiles: every K/V operand read from LDS feeds two matrix
// instructions (head_dim 256: MT = 1, key tiles of 32 tokens).  The loop walks
// the keys in tiles of 64 tokens that the workgroup stages in LDS, two buffers per matrix (one
// barrier per tile) and two tiles in flight in registers.  LDS rows are padded by 32 bytes
// (288 for head_dim 128): gfx950 serves a 16-byte LDS read of lane 0 in one cycle with lanes
// 1-3, 12-15 and 20-27 (measured), and with that grouping a pitch of 16 (4k + 2) bytes is free of
// bank conflicts for the K operand reads and for the transposed V reads.  Per key tile:
//   S^T = K Q^T   mfma_f32_16x16x32, A = K rows from LDS, B = Q rows kept in registers: an operand
//                 is a 16-byte piece of a row;
//   softmax       base-2, online; the result tile has the query row in lane % 16 and four
//                 tokens per lane, which is the A-operand layout of the next product; the row
//                 maximum crosses the four lane groups with v_permlane16/32_swap;
//   O += P V      per 32 tokens: A = P (rounded to the KV type), B = V read with
//                 ds_read_b64_tr_b16, which hands lane r dimension 16 a + r of four tokens.
// Pages are looked up per staged row, one tile ahead; rows past the end of the sequence are
// clamped (never out of the pool) and masked.  All query tiles of the heads that share a KV head
// are placed on one XCD (see the block-index mapping in the kernel).

#include "common.cuh"
#include "../../include/tidal_hip.h"

namespace tidal {


// LDS read with transpose (gfx950): within every 16 lanes, lane 4a + b receives element b of the
// four 8-byte pieces addressed by lanes a, a + 4, a + 8, a + 12.
typedef short i16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* at) {
  const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) i16x4*)(at));
  return __builtin_bit_cast(u32x2, v);
}

struct PrefillParams {
  const uint16_t* kv;
  int64_t page_stride, v_offset;  // elements
  int32_t entry_stride, head_stride, page_size, page_shift;
  uint32_t max_page;
  const int32_t* page_table;
  int32_t n_pages, kv_len;
  const uint16_t* q;
  uint16_t* o;
  int32_t n_q, num_qo_heads, q_per_kv;
  float scale_log2;
  int32_t causal;
};

// BN tokens per key tile (a multiple of 32), NW wavefronts per workgroup (4 or 8: a staged K/V
// tile serves 16 MT NW query rows, so eight waves halve the global -> LDS traffic per flop)
template <typename T, int D, int MT, int BN, int NW>
__global__ __launch_bounds__(64 * NW, MT == 2 ? 2 : 1) void prefill_attn_kernel(const PrefillParams p) {
  constexpr int kThreads = 64 * NW;
  constexpr int kPfBM = 16 * MT * NW;  // query rows per workgroup
  constexpr int WR = 16 * MT;       // query rows per wavefront
  constexpr int NS = D / 32;        // 16-byte pieces of a Q/K row per lane (one MFMA each)
  constexpr int DC = D / 16;        // head dimensions per lane in the P.V product
  constexpr int PITCH = D + 16;     // LDS row pitch in elements: +32 bytes (see the layout note)
  constexpr int CPR = D / 8;        // 16-byte chunks per row
  constexpr int kPfBN = BN;
  constexpr int NSUB = BN / 16;     // 16-token sub-tiles per key tile
  constexpr int SR = kThreads / 8;  // staging: rows per pass (8 lanes per row piece)
  constexpr int RPT = BN / SR;      // staging: rows per thread (row = tid / 8 + SR jr)
  constexpr int CCT = CPR / 8;      // staging: chunks per thread and row (chunk = tid % 8 + 8 jc)
  constexpr int CPT = RPT * CCT;    // chunks a thread stages per tile and matrix
  static_assert(D == 64 || D == 128 || D == 256, "head dimensions of the prefill kernel");
  static_assert(BN % 32 == 0 && RPT >= 1 && CPT * kThreads == BN * CPR, "key tile");
  // two buffers per matrix: tile t + 1 is written while tile t is still being read
  constexpr int TILE = kPfBN * PITCH;
  __shared__ __attribute__((aligned(16))) uint16_t ks[2 * TILE];
  __shared__ __attribute__((aligned(16))) uint16_t vs[2 * TILE];

  // the wave index is made scalar: the per-tile activity tests below must be real branches, because
  // matrix instructions do not honour the EXEC mask of a masked-off region
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  // Workgroups go to the eight XCDs round-robin by linear id, and each XCD has its own L2.  When
  // the KV heads divide evenly, all query tiles of the heads that share a KV head are given to one
  // XCD, so that its L2 streams one head's K/V instead of every head's.  (Placement only decides
  // what the L2 holds; results do not depend on it.)  Longest rows first in either order.
  int qtile, qh;
  {
    const int n_tiles = gridDim.x, n_heads = gridDim.y;
    const int lin = blockIdx.x + n_tiles * blockIdx.y;
    const int n_kv = n_heads / p.q_per_kv;
    if (n_kv % 8 == 0) {
      const int xcd = lin & 7, slot = lin >> 3;
      const int idx = slot / n_tiles;  // which of this XCD's heads
      qtile = n_tiles - 1 - slot % n_tiles;
      qh = ((idx / p.q_per_kv) * 8 + xcd) * p.q_per_kv + idx % p.q_per_kv;
    } else {
      qtile = n_tiles - 1 - blockIdx.x;
      qh = blockIdx.y;
    }
  }
  const int kvh = qh / p.q_per_kv;
  const int q0 = qtile * kPfBM;
  const int q_off = p.kv_len - p.n_q;  // position of query row 0

  // ---- Q operands: row (q0 + WR wave + 16 mt + r), pieces [32 s + 8 g, +8) ----------------------
  u32x4 qb[MT][NS];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = q0 + wave * WR + mt * 16 + r;
    row = row < p.n_q ? row : p.n_q - 1;
    const u32x4* src =
        reinterpret_cast<const u32x4*>(p.q + ((int64_t)row * p.num_qo_heads + qh) * D);
#pragma unroll
    for (int s = 0; s < NS; ++s) qb[mt][s] = src[4 * s + g];
  }

  f32x4 oacc[MT][DC];
  float m_run[MT], l_run[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    m_run[mt] = kNegBig;
    l_run[mt] = 0.f;
#pragma unroll
    for (int d = 0; d < DC; ++d) oacc[mt][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // keys this workgroup needs: up to the position of its last query row
  int last_row = q0 + kPfBM - 1;
  last_row = last_row < p.n_q ? last_row : p.n_q - 1;
  const int kv_end = p.causal ? (q_off + last_row + 1) : p.kv_len;

  // ---- staging: thread -> CPT chunks of K and of V per tile --------------------------------------
  // eight adjacent lanes move 128 contiguous bytes of one row (one cache line in, one conflict-free
  // LDS write out); a thread looks up the page of each of its RPT rows once
  // Two register sets: the loads of tile t + 2 are issued while tile t + 1 still waits in the
  // other set for its turn to be written to LDS, so a tile has two iterations to arrive.
  u32x4 kreg_a[CPT], vreg_a[CPT], kreg_b[CPT], vreg_b[CPT];
  const int srow = tid >> 3, sl8 = tid & 7;
  // page ids are looked up one tile ahead of the rows they address, so that a tile's K/V loads
  // never wait for a page-table load issued in the same iteration
  uint32_t pg[RPT];
  auto split_tok = [&](int kt, int jr, int& pg_i, int& entry) {
    int tok = kt + srow + SR * jr;
    tok = tok < p.kv_len ? tok : p.kv_len - 1;
    if (p.page_shift >= 0) {
      pg_i = tok >> p.page_shift;
      entry = tok & (p.page_size - 1);
    } else {
      pg_i = tok / p.page_size;
      entry = tok - pg_i * p.page_size;
    }
  };
  auto lookup = [&](int kt) {
#pragma unroll
    for (int jr = 0; jr < RPT; ++jr) {
      int pg_i, entry;
      split_tok(kt, jr, pg_i, entry);
      pg[jr] = (uint32_t)p.page_table[pg_i];
    }
  };
  auto fetch = [&](int kt, u32x4 (&kreg)[CPT], u32x4 (&vreg)[CPT]) {  // needs lookup(kt) before it
#pragma unroll
    for (int jr = 0; jr < RPT; ++jr) {
      int pg_i, entry;
      split_tok(kt, jr, pg_i, entry);
      const uint32_t page = pg[jr] > p.max_page ? p.max_page : pg[jr];
      const uint16_t* src = p.kv + ((int64_t)page * p.page_stride + (int64_t)entry * p.entry_stride +
                                    (int64_t)kvh * p.head_stride + sl8 * 8);
#pragma unroll
      for (int jc = 0; jc < CCT; ++jc) {
        kreg[jr * CCT + jc] = *reinterpret_cast<const u32x4*>(src + jc * 64);
        vreg[jr * CCT + jc] = *reinterpret_cast<const u32x4*>(src + jc * 64 + p.v_offset);
      }
    }
  };
  auto stash = [&](int buf, const u32x4 (&kreg)[CPT], const u32x4 (&vreg)[CPT]) {
#pragma unroll
    for (int jr = 0; jr < RPT; ++jr)
#pragma unroll
      for (int jc = 0; jc < CCT; ++jc) {
        const int at = buf * TILE + (srow + SR * jr) * PITCH + (sl8 + 8 * jc) * 8;
        *reinterpret_cast<u32x4*>(&ks[at]) = kreg[jr * CCT + jc];
        *reinterpret_cast<u32x4*>(&vs[at]) = vreg[jr * CCT + jc];
      }
  };

  const int wave_first_pos = q_off + q0 + wave * WR;  // position of the wave's first query row
  auto compute = [&](int kt, int buf) {
    // A wave whose last query row lies before the key tile sees none of it (causal).  Inside an
    // active wave every query tile is computed: a tile that lies wholly before the key tile is
    // masked to zero weight below, which happens once per wave, and the loop body stays free of
    // branches around the matrix instructions.
    if (!p.causal || kt <= wave_first_pos + WR - 1) {
      // ---- S^T: each K operand is read once and used by every active query tile -----------------
      // (the two matrix phases run at raised wave priority: while one wave of a SIMD is in its
      // softmax arithmetic, the other's matrix instructions are issued first and keep the matrix
      // pipeline busy)
      __builtin_amdgcn_s_setprio(2);
      f32x4 st[MT][NSUB];
#pragma unroll
      for (int sub = 0; sub < NSUB; ++sub) {
        u32x4 ka[NS];
        const uint16_t* krow = &ks[buf * TILE + (sub * 16 + r) * PITCH + 8 * g];
#pragma unroll
        for (int s = 0; s < NS; ++s) ka[s] = *reinterpret_cast<const u32x4*>(krow + 32 * s);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < NS; ++s) acc = mfma_16x16x32<T>(ka[s], qb[mt][s], acc);
          st[mt][sub] = acc;  // raw q.k; the softmax scale is folded into the exponent below
        }
      }
      __builtin_amdgcn_s_setprio(0);
      // ---- online softmax of query row r (lanes r, r+16, r+32, r+48 share the row) ---------------
      uint32_t pa[MT][NSUB][2];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int qpos = wave_first_pos + mt * 16 + r;  // position of this lane's query row
        // the test of the wave's first query tile covers the second: masking a tile that does
        // not need it changes nothing, and one rare branch keeps the position arithmetic out of
        // the common path
        const bool need_mask =
            (p.causal && kt + kPfBN - 1 > wave_first_pos) || kt + kPfBN > p.kv_len;
        if (need_mask) {
#pragma unroll
          for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int tpos = kt + sub * 16 + 4 * g + i;
              const bool ok = tpos < p.kv_len && (!p.causal || tpos <= qpos);
              st[mt][sub][i] = ok ? st[mt][sub][i] : kNegBig;
            }
        }
        float mt_max = kNegBig;
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
          for (int i = 0; i < 4; ++i) mt_max = fmaxf(mt_max, st[mt][sub][i]);
        mt_max = rows_max(mt_max);
        // m_run is kept in the scaled base-2 domain.  A masked entry (kNegBig) gives exp2(-huge) = 0
        // by itself: every query row sees token 0 in its first tile, so m_new is a real maximum.
        // The running maximum only moves when the tile's maximum exceeds it by more than 2^8:
        // softmax does not depend on the reference point, weights up to 256 are exact to the same
        // relative precision, and the accumulator rescale below becomes rare.
        const float m_tile = mt_max * p.scale_log2;
        const float m_new = m_tile > m_run[mt] + 8.f ? m_tile : m_run[mt];
        const float alpha = fast_exp2(m_run[mt] - m_new);
        m_run[mt] = m_new;
        float psum = 0.f;
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub) {
          float pr[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            pr[i] = fast_exp2(fmaf(st[mt][sub][i], p.scale_log2, -m_new));
            psum += pr[i];
          }
          pa[mt][sub][0] = pack2<T>(pr[0], pr[1]);
          pa[mt][sub][1] = pack2<T>(pr[2], pr[3]);
        }
        l_run[mt] = fmaf(l_run[mt], alpha, psum);
        // rescale: accumulator row 4g + i is query row 4g + i, whose factor sits in lane 4g + i
        if (__ballot(alpha != 1.f)) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float f = __shfl(alpha, 4 * g + i, 64);
#pragma unroll
            for (int d = 0; d < DC; ++d) oacc[mt][d][i] *= f;
          }
        }
      }
      __builtin_amdgcn_s_setprio(2);
      // ---- O += P V, 32 tokens (two sub-tiles) per matrix instruction ------------------------------
      // B operand of head dimensions [16 a, 16 a + 16): lane (r, g) needs dimension 16 a + r of the
      // tokens 4g..4g+3 of both sub-tiles.  ds_read_b64_tr_b16 transposes a 4 token x 16 dimension
      // block inside every 16 lanes: lane r points at the 8-byte piece r % 4 of token row r / 4
      // and receives dimension r of the four rows.
      const uint16_t* vlane = &vs[buf * TILE + (4 * g + (r >> 2)) * PITCH + 4 * (r & 3)];
#pragma unroll
      for (int pair = 0; pair < NSUB / 2; ++pair) {
#pragma unroll
        for (int a = 0; a < DC; ++a) {
          const u32x2 t0 = lds_read_tr16(vlane + (32 * pair) * PITCH + 16 * a);
          const u32x2 t1 = lds_read_tr16(vlane + (32 * pair + 16) * PITCH + 16 * a);
          const u32x4 vb = {t0.x, t0.y, t1.x, t1.y};
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const u32x4 pp = {pa[mt][2 * pair][0], pa[mt][2 * pair][1], pa[mt][2 * pair + 1][0],
                              pa[mt][2 * pair + 1][1]};
            oacc[mt][a] = mfma_16x16x32<T>(pp, vb, oacc[mt][a]);
          }
        }
      }
      __builtin_amdgcn_s_setprio(0);
    }
  };

  // tile 0 into buffer 0, tile 1 into register set a
  lookup(0);
  fetch(0, kreg_a, vreg_a);
  lookup(kPfBN);
  stash(0, kreg_a, vreg_a);
  if (kPfBN < kv_end) {
    fetch(kPfBN, kreg_a, vreg_a);
    lookup(2 * kPfBN);
  }
  // One barrier per tile: it makes tile kt visible in its buffer, and it tells that every wave has
  // finished reading the other buffer, which the end of the step overwrites with tile kt + BN.
  for (int kt = 0; kt < kv_end; kt += 2 * kPfBN) {
    __syncthreads();
    if (kt + 2 * kPfBN < kv_end) {
      fetch(kt + 2 * kPfBN, kreg_b, vreg_b);
      lookup(kt + 3 * kPfBN);
    }
    compute(kt, 0);
    if (kt + kPfBN >= kv_end) break;
    stash(1, kreg_a, vreg_a);
    __syncthreads();
    if (kt + 3 * kPfBN < kv_end) {
      fetch(kt + 3 * kPfBN, kreg_a, vreg_a);
      lookup(kt + 4 * kPfBN);
    }
    compute(kt + kPfBN, 1);
    if (kt + 2 * kPfBN < kv_end) stash(0, kreg_b, vreg_b);
  }

  // ---- normalise and store: lane holds rows 4g + i, dimensions 16 a + r ---------------------------
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const float l = rows_sum(l_run[mt]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float li = __shfl(l, 4 * g + i, 64);
      const float inv = li > 0.f ? 1.f / li : 0.f;
      const int row = q0 + wave * WR + mt * 16 + 4 * g + i;
      if (row < p.n_q) {
        uint16_t* dst = p.o + ((int64_t)row * p.num_qo_heads + qh) * D + r;
#pragma unroll
        for (int a = 0; a < DC; ++a) dst[16 * a] = from_float<T>(oacc[mt][a][i] * inv);
      }
    }
  }
}

template <typename T>
static int launch_prefill(const PrefillParams& p, int head_dim, hipStream_t st) {
  // Two query tiles per wavefront and 64-token key tiles keep the kernel within 256 registers
  // (two waves per SIMD).  Staging a K/V tile (global loads, page lookups, LDS stores) costs a
  // quarter of the kernel's time, so head_dim 128 runs eight waves per workgroup: one staged tile
  // serves 256 query rows (8.9 -> 8.4 ms per layer at 32K x 32 heads); prompts of up to 128 rows
  // keep four.  (Four query tiles per wavefront halve the LDS traffic per flop but need twice
  // the registers: one wave per SIMD with every latency exposed, 2.5x slower.)  head_dim 256 has
  // twice the accumulators and twice the LDS per token: one query tile per wavefront, 32-token
  // key tiles.
  const dim3 block(256);
  if (head_dim == 128 && p.n_q > 128)
    hipLaunchKernelGGL((prefill_attn_kernel<T, 128, 2, 64, 8>), dim3((p.n_q + 255) / 256, p.num_qo_heads),
                       dim3(512), 0, st, p);
  else if (head_dim == 128)
    hipLaunchKernelGGL((prefill_attn_kernel<T, 128, 2, 64, 4>), dim3((p.n_q + 127) / 128, p.num_qo_heads),
                       block, 0, st, p);
  else if (head_dim == 64)
    hipLaunchKernelGGL((prefill_attn_kernel<T, 64, 2, 64, 4>), dim3((p.n_q + 127) / 128, p.num_qo_heads),
                       block, 0, st, p);
  else if (head_dim == 256)
    hipLaunchKernelGGL((prefill_attn_kernel<T, 256, 1, 32, 4>), dim3((p.n_q + 63) / 64, p.num_qo_heads),
                       block, 0, st, p);
  else
    return fail(TD_ERR_UNSUPPORTED,
                "BatchPrefillWithPagedKVCache failed to dispatch with head_dim %d (supported: 64, 128, 256)",
                head_dim);
  return TD_OK;
}

}  // namespace tidal

using namespace tidal;

extern "C" int td_prefill_attn(const td_paged_kv* kv, const int32_t* page_table, int32_t n_pages,
                               int32_t kv_len, const void* q, void* o, int32_t n_q,
                               int32_t num_qo_heads, float sm_scale, int32_t causal, void* stream) {
  TD_REQUIRE(kv && kv->data && page_table && q && o, "td_prefill_attn: NULL argument");
  TD_REQUIRE(kv->page_size >= 1 && kv->num_kv_heads >= 1 && kv->max_pages >= 1,
             "td_prefill_attn: bad pool geometry");
  TD_REQUIRE(num_qo_heads >= kv->num_kv_heads && num_qo_heads % kv->num_kv_heads == 0,
             "td_prefill_attn: num_qo_heads %d is not a multiple of num_kv_heads %d", num_qo_heads,
             kv->num_kv_heads);
  TD_REQUIRE(n_q >= 0 && kv_len >= n_q, "td_prefill_attn: n_q %d, kv_len %d", n_q, kv_len);
  TD_REQUIRE((int64_t)n_pages * kv->page_size >= kv_len,
             "td_prefill_attn: %d pages of %d entries do not hold %d tokens", n_pages,
             kv->page_size, kv_len);
  TD_REQUIRE(kv->layout == TD_NHD || kv->layout == TD_HND, "td_prefill_attn: layout %d", kv->layout);
  if (n_q == 0) return TD_OK;
  const int P = kv->page_size, H = kv->num_kv_heads, D = kv->head_dim;
  PrefillParams p;
  p.kv = reinterpret_cast<const uint16_t*>(kv->data);
  p.page_stride = (int64_t)2 * P * H * D;
  p.v_offset = (int64_t)P * H * D;
  p.entry_stride = kv->layout == TD_NHD ? H * D : D;
  p.head_stride = kv->layout == TD_NHD ? D : P * D;
  p.page_size = P;
  p.page_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;
  p.max_page = (uint32_t)(kv->max_pages - 1);
  p.page_table = page_table;
  p.n_pages = n_pages;
  p.kv_len = kv_len;
  p.q = reinterpret_cast<const uint16_t*>(q);
  p.o = reinterpret_cast<uint16_t*>(o);
  p.n_q = n_q;
  p.num_qo_heads = num_qo_heads;
  p.q_per_kv = num_qo_heads / H;
  p.scale_log2 = sm_scale * 1.4426950408889634f;
  p.causal = causal;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  int rc;
  if (kv->dtype == TD_F16)
    rc = launch_prefill<F16>(p, D, st);
  else if (kv->dtype == TD_BF16)
    rc = launch_prefill<BF16>(p, D, st);
  else
    return fail(TD_ERR_UNSUPPORTED, "BatchPrefillWithPagedKVCache failed to dispatch with dtype %d",
                kv->dtype);
  if (rc != TD_OK) return rc;
  TD_HIP_CHECK(hipGetLastError());
  return TD_OK;
}
