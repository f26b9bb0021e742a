// Decode attention on the matrix cores: one query a sequence over the pages of the cache (see attention_mfma.h for the
// products' layout).
#include "attention_mfma.h"

// attention_simple.hip; base2: the partial results' maxima are exponents of 2, not of e
int yalm_attn_decode_combine_bf16(const float* partial, void* out, float* lse, int B, int n_heads, int head_dim,
                                  int n_splits, int base2, const SinkArgs& sinks, hipStream_t stream);

namespace {

// ---------------------------------------------------------------------------
// decode: grid (split, kv head, sequence); NW waves take the pages of the split in turn.
// The keys of a wave's next page stay in flight while this page is mixed: the loop's loads stand
// under no branch (the last page is done by a copy of the body without them), else the compiler
// waits for every load in flight at each use.
// ---------------------------------------------------------------------------
// BLOCKS: the pages are laid out in blocks (YALM_PAGE_BLOCKS): every load instruction reads 1 KB of consecutive
// bytes, and asks for them non-temporally (a step reads a page once; with pieces of lines the hint costs more
// than it gains: the other half of a line would be fetched again).
// BIAS: a term is added to every score by the distance of query and key, bias[head][min(distance, n_bias - 1)].
template <int HD, int NW, bool BLOCKS, bool BIAS>
__global__ __launch_bounds__(NW * WAVE, NW == 4 ? 2 : 1) void attn_decode_mfma_kernel(   // 2 waves a SIMD: head size 128 needs their registers
    const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, int ring_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_len, float* __restrict__ partial, bf16* __restrict__ out, float* __restrict__ lse,
    int n_heads, int n_kv_heads, int window, int n_splits, int n_pages, const int* __restrict__ step_max_len,
    const int* __restrict__ seq_order, const float* __restrict__ bias, int n_bias) {
  // A head size that is no multiple of 32 (pages in rows then): the last step of the scores' product is half empty.
  // The query's lanes of that half hold zeros; the keys' lanes read the row's last 8 elements again (an address
  // inside the row, finite values for every row that counts).
  constexpr int KS = (HD + 31) / 32, DT = HD / 16;
  static_assert(HD % 16 == 0 && (!BLOCKS || HD % 32 == 0), "head sizes in steps of 16; pages in blocks in steps of 32");
  __shared__ float sm_m[NW][16];
  __shared__ float sm_l[NW][16];
  __shared__ f32x4 sm_o[NW][DT][WAVE];
  // seq_order: the rows in the order of their cost (only which workgroup takes which row changes)
  // a group of more than 16 query heads is taken 16 heads (a tile's columns) a workgroup: blockIdx.y = (KV head, part)
  const int Gall = n_heads / n_kv_heads, parts_g = (Gall + 15) / 16;
  const int split = blockIdx.x, g = (int)blockIdx.y / parts_g, h0 = g * Gall + ((int)blockIdx.y % parts_g) * 16;
  const int b = seq_order != nullptr ? min(max(seq_order[blockIdx.z], 0), (int)gridDim.z - 1) : (int)blockIdx.z;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE, qd = lane / 16,
            j = lane % 16;
  const int G = min(16, (g + 1) * Gall - h0);      // heads of this workgroup, the first being head h0
  const int slot = seq_slot[b];
  const int L = slot >= 0 ? seq_len[b] : 0;

  float m = -FLT_MAX, l = 0.f;
  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  if (L > 0) {
    const int lo = window > 0 ? max(0, L - window) : 0;
    const int first_page = lo / PAGE, last_page = (L - 1) / PAGE;
    const int total = last_page - first_page + 1;
    int per = (total + n_splits - 1) / n_splits;
    if (step_max_len != nullptr) {
      // Sequences of unequal lengths: a split is as many pages as the longest sequence's split, so that every working
      // workgroup has the same work and a short sequence uses fewer of its splits (the others find nothing to do),
      // instead of every sequence cutting its own length into n_splits pieces of unequal cost.  Whatever the value
      // says, the sequence's own pages are all covered.
      const int Lm = max(step_max_len[0], 1);
      const int total_m = (Lm - 1) / PAGE - (window > 0 ? max(0, Lm - window) / PAGE : 0) + 1;
      per = max(per, (total_m + n_splits - 1) / n_splits);
    }
    const int p_begin = first_page + split * per;
    const int p_end = min(last_page + 1, p_begin + per);
    // scores and the running maximum are kept in units of log2(e) / sqrt(head_dim): one multiply, and 2^x is one instruction
    const float score_scale = 1.4426950408889634f / sqrtf((float)HD);
    const size_t page_elems = (size_t)n_kv_heads * PAGE * HD;
    const int* table = block_table + (size_t)slot * table_stride;

    bf16x8 qv[KS];
    {
      const bool head_ok = j < G;
      const bf16* qrow = q + ((size_t)b * n_heads + h0 + (head_ok ? j : 0)) * HD;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qv[ks] = head_ok && ks * 32 + qd * 8 < HD ? ld8(qrow + ks * 32 + qd * 8) : zero8();
    }

    const float* bias_row = BIAS ? bias + (size_t)(h0 + min(j, G - 1)) * n_bias : nullptr;   // the column's head
    bf16x8 kreg[4][KS];
    auto page_of = [&](int a) { return min(max(table[a % ring_pages], 0), n_pages - 1); };
    auto load_keys = [&](int phys) {
      const bf16* kp = k_pages + phys * page_elems + (size_t)g * PAGE * HD;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          kreg[t][ks] = BLOCKS ? ld8_once(kp + ((ks * PAGE + t * 16 + j) * 32 + qd * 8))
                               : ld8(kp + key_row(t, j) * HD + min(ks * 32 + qd * 8, HD - 8));
    };
    int ap = p_begin + wave;
    int phys = ap < p_end ? page_of(ap) : 0;
    if (ap < p_end) load_keys(phys);

    // one page: has_next is a compile-time tag (std::true_type: the next page's keys are asked for)
    auto one_page = [&](auto has_next) {
      const bf16* vp = v_pages + phys * page_elems + (size_t)g * PAGE * HD;
      bf16x8 vreg[DT][2];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int s = 0; s < 2; ++s)
          vreg[dt][s] = BLOCKS ? ld8_once(vp + ((s * HD + dt * 16 + j) * 32 + qd * 8))
                               : ld8(vp + (dt * 16 + j) * PAGE + s * 32 + qd * 8);
      int physn = 0;
      if constexpr (decltype(has_next)::value) physn = page_of(ap + NW);
      __builtin_amdgcn_sched_barrier(0);         // the values are asked for before the keys are waited for

      f32x4 sc[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        sc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[t][ks], qv[ks], sc[t], 0, 0, 0);
      }
      if constexpr (decltype(has_next)::value) {
        load_keys(physn);                        // they stay in flight while this page is mixed
        phys = physn;
        __builtin_amdgcn_sched_barrier(0);
      }

      const int base = ap * PAGE;
      const bool edge = base < lo || base + PAGE > L;
      float mx = -FLT_MAX;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = sc[t][r] * score_scale;
          if constexpr (BIAS) {                    // in the same units as the scores: exponents of 2
            const int dist = L - 1 - (base + 32 * (t >> 1) + 8 * qd + 4 * (t & 1) + r);
            v = fmaf(bias_row[min(max(dist, 0), n_bias - 1)], 1.4426950408889634f, v);
          }
          if (edge) {
            int pos = base + 32 * (t >> 1) + 8 * qd + 4 * (t & 1) + r;
            if (pos < lo || pos >= L) v = -INFINITY;
          }
          sc[t][r] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      const float m_new = fmaxf(m, mx);
      const float corr = __builtin_amdgcn_exp2f(m - m_new);
      float psum = 0.f;
      bf16x8 pb[2];
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float p = __builtin_amdgcn_exp2f(sc[2 * s + (e >> 2)][e & 3] - m_new);
          psum += p;
          pb[s][e] = static_cast<bf16>(p);
        }
      l = l * corr + psum;
      m = m_new;
      if (base + PAGE > L) {                     // rows behind the length may hold anything: 0 * NaN must not happen
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (base + 32 * s + 8 * qd + e >= L) {
#pragma unroll
              for (int dt = 0; dt < DT; ++dt) vreg[dt][s][e] = static_cast<bf16>(0.f);
            }
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        o[dt] *= corr;
#pragma unroll
        for (int s = 0; s < 2; ++s)
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg[dt][s], pb[s], o[dt], 0, 0, 0);
      }
    };
    for (; ap + NW < p_end; ap += NW) one_page(std::true_type{});
    if (ap < p_end) one_page(std::false_type{});
  }

  // the four lanes of a column hold parts of its sum; then the waves merge
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (qd == 0) sm_m[wave][j] = m;
  __syncthreads();
  float m_all = sm_m[0][j];
#pragma unroll
  for (int w = 1; w < NW; ++w) m_all = fmaxf(m_all, sm_m[w][j]);
  const float scale = __builtin_amdgcn_exp2f(m - m_all);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) sm_o[wave][dt][lane] = o[dt] * scale;
  if (qd == 0) sm_l[wave][j] = l * scale;
  __syncthreads();
  if (j < G) {
    float lt = sm_l[0][j];
#pragma unroll
    for (int w = 1; w < NW; ++w) lt += sm_l[w][j];
    if (n_splits == 1 && out != nullptr) {        // nothing to merge with: this is the result
      bf16* orow = out + ((size_t)b * n_heads + h0 + j) * HD;
      const float inv_l = lt > 0.f ? 1.0f / lt : 0.f;
      for (int dt = wave; dt < DT; dt += NW) {
        f32x4 v = sm_o[0][dt][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) v += sm_o[w][dt][lane];
#pragma unroll
        for (int r = 0; r < 4; ++r) orow[dt * 16 + 4 * qd + r] = static_cast<bf16>(v[r] * inv_l);
      }
      if (lse != nullptr && wave == 0 && qd == 0)  // natural logarithm of the sum of exp(score): for a later mix with further keys
        lse[(size_t)b * n_heads + h0 + j] = lt > 0.f ? m_all * LN2 + logf(lt) : -FLT_MAX;
    } else {
      float* part = partial + (((size_t)b * n_heads + h0 + j) * n_splits + split) * (HD + 2);
      for (int dt = wave; dt < DT; dt += NW) {
        f32x4 v = sm_o[0][dt][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) v += sm_o[w][dt][lane];
#pragma unroll
        for (int r = 0; r < 4; ++r) part[dt * 16 + 4 * qd + r] = v[r];
      }
      if (wave == 0 && qd == 0) {
        part[HD] = m_all;
        part[HD + 1] = lt;
      }
    }
  }
}

}  // namespace

int yalm_attn_decode_bf16_mfma(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                               int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                               float* lse, float* partial, int B, int n_heads, int n_kv_heads, int head_dim, int window,
                               int n_splits, int n_pages, int page_layout, const SinkArgs& sinks,
                               const int* step_max_len, const int* seq_order, const float* bias, int n_bias,
                               hipStream_t stream) {
  // with sinks the merge kernel always runs: it takes them in, also where there is one split
  const bool merge = n_splits > 1 || sinks.n_sinks > 0;
  if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim)) return YALM_ERR_ARG;
  // a score bias: the engine's layout of the pages only (blocks where the head size allows), and no sinks (they are
  // scored without it)
  if (bias != nullptr && (n_bias <= 0 || (page_layout != YALM_PAGE_BLOCKS && head_dim % 32 == 0) || sinks.n_sinks > 0))
    return YALM_ERR_ARG;
  const int parts_g = (n_heads / n_kv_heads + 15) / 16;      // workgroups a KV head: 16 query heads each
  if ((long)n_kv_heads * parts_g > 65535) return YALM_ERR_ARG;
  dim3 grid(n_splits, n_kv_heads * parts_g, B);
#define YALM_DECODE(HD_, NW_, BLOCKS_, BIAS_)                                                                       \
  attn_decode_mfma_kernel<HD_, NW_, BLOCKS_, BIAS_><<<grid, NW_ * WAVE, 0, stream>>>(                               \
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, block_table, table_stride, ring_pages, seq_slot, \
      seq_len, partial, merge ? nullptr : (bf16*)out, lse, n_heads, n_kv_heads, window, n_splits, n_pages, \
      step_max_len, seq_order, bias, n_bias)
  // 4 waves a workgroup: 8 measured no faster with one split and slower with more (a CU draws about
  // 33 GB/s whatever its number of waves, so a small batch needs its workgroups spread over all CUs)
  // pages in blocks for the head sizes that are multiples of 32, in rows for the others (and for yalm_attn_decode)
  const bool blocks = page_layout == YALM_PAGE_BLOCKS;
  if (blocks && head_dim % 32 != 0) return YALM_ERR_ARG;
#define YALM_DECODE_HD32(HD_)                                                       \
  case HD_:                                                                         \
    if (bias != nullptr) YALM_DECODE(HD_, 4, true, true);                           \
    else if (blocks) YALM_DECODE(HD_, 4, true, false);                              \
    else YALM_DECODE(HD_, 4, false, false);                                         \
    break
#define YALM_DECODE_HD16(HD_)                                                       \
  case HD_:                                                                         \
    if (bias != nullptr) YALM_DECODE(HD_, 4, false, true);                          \
    else YALM_DECODE(HD_, 4, false, false);                                         \
    break
  switch (head_dim) {
    YALM_DECODE_HD16(16);
    YALM_DECODE_HD32(32);
    YALM_DECODE_HD16(48);
    YALM_DECODE_HD32(64);
    YALM_DECODE_HD16(80);
    YALM_DECODE_HD32(96);
    YALM_DECODE_HD16(112);
    YALM_DECODE_HD32(128);
  }
#undef YALM_DECODE_HD32
#undef YALM_DECODE_HD16
#undef YALM_DECODE
  int rc = launch_status();
  if (rc != YALM_OK || !merge) return rc;          // one split writes the result itself
  return yalm_attn_decode_combine_bf16(partial, out, lse, B, n_heads, head_dim, n_splits, 1, sinks, stream);
}
