// Attention in float32 arithmetic for every storage type: the kernels of the
// true 32-bit path and the fallback of the bfloat16 path.  One wave per
// (query, head); keys are taken 64 at a time, a lane per key for the scores
// and a lane per output element for the mix; softmax state in float32.
#include <float.h>
#include <mutex>
#include "common.h"
#include "sinks.h"
#include "yalm_hip.h"

int yalm_attn_prefill_bf16_mfma(const void* q, const void* k_stage, const void* v_stage, void* out, float* out_f32,
                                float* lse,
                                const int* cu_seqlens, const int* seq_tile0, const int* tile_order, int n_order,
                                int T, int B, int n_tiles, int n_heads, int n_kv_heads, int head_dim, int window,
                                const float* bias, int n_bias, hipStream_t stream);
int yalm_attn_decode_bf16_mfma(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                               int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                               float* lse, float* partial, int B, int n_heads, int n_kv_heads, int head_dim, int window,
                               int n_splits, int n_pages, int page_layout, const SinkArgs& sinks,
                               const int* step_max_len, const int* seq_order, const float* bias, int n_bias,
                               hipStream_t stream);

namespace {
// A term added to every score by the distance between query and key: table[head][min(distance, n - 1)] (float32), or
// nothing.  What a position encoding that is no rotation needs (a slope per head times the distance, a learned table).
struct ScoreBias {
  const float* table;
  int n;
  __device__ __forceinline__ float at(int head, int distance) const {
    return table != nullptr ? table[(size_t)head * n + min(max(distance, 0), n - 1)] : 0.f;
  }
};

constexpr int MAX_HD = 256;              // head sizes up to 256 (4 output elements per lane)
constexpr int ACC = MAX_HD / WAVE;
constexpr int COMBINE_THREADS = 256;

// ---------------------------------------------------------------------------
// prefill: a step's tokens over the same step's keys
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void attn_prefill_simple_kernel(
    const T* __restrict__ q, const T* __restrict__ k_stage, const T* __restrict__ v_stage, T* __restrict__ out,
    float* __restrict__ out_f32, float* __restrict__ lse, const int* __restrict__ seq_tile0,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int n_heads, int n_kv_heads, int hd, int window,
    ScoreBias sb) {
  __shared__ float qs[MAX_HD];
  __shared__ float ps[WAVE];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int b = tok_seq[t], pos = tok_pos[t];
  const int g = h / (n_heads / n_kv_heads);
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const float inv = sqrtf((float)hd);
  const size_t tile0 = (size_t)seq_tile0[b];

  for (int i = lane; i < hd; i += WAVE) qs[i] = to_f32(q[((size_t)t * n_heads + h) * hd + i]);
  __syncthreads();

  float m = -FLT_MAX, l = 0.f;
  float acc[ACC];
#pragma unroll
  for (int a = 0; a < ACC; ++a) acc[a] = 0.f;

  for (int tile = lo / PAGE; tile <= pos / PAGE; ++tile) {
    const T* kp = k_stage + ((tile0 + tile) * n_kv_heads + g) * PAGE * hd;
    const T* vp = v_stage + ((tile0 + tile) * n_kv_heads + g) * PAGE * hd;
    int j = tile * PAGE + lane;
    bool valid = j >= lo && j <= pos;
    float s = -FLT_MAX;
    if (valid) {
      const T* kr = kp + (size_t)lane * hd;
      float d = 0.f;
      for (int i = 0; i < hd; ++i) d = fmaf(qs[i], to_f32(kr[i]), d);
      s = d / inv + sb.at(h, pos - j);
    }
    float m_new = fmaxf(m, wave_max(s));
    float p = valid ? expf(s - m_new) : 0.f;
    float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
#pragma unroll
    for (int a = 0; a < ACC; ++a) {
      int d = lane + a * WAVE;
      if (d < hd) {
        const T* vr = vp + (size_t)d * PAGE;
        float s2 = 0.f;
        for (int jj = 0; jj < PAGE; ++jj) {
          float pj = ps[jj];
          if (pj != 0.f) s2 = fmaf(pj, to_f32(vr[jj]), s2);     // rows outside the mask may hold anything
        }
        acc[a] = acc[a] * corr + s2;
      }
    }
  }
#pragma unroll
  for (int a = 0; a < ACC; ++a) {
    int d = lane + a * WAVE;
    if (d < hd) {
      out[((size_t)t * n_heads + h) * hd + d] = from_f32<T>(acc[a] / l);
      if (out_f32 != nullptr) out_f32[((size_t)t * n_heads + h) * hd + d] = acc[a] / l;
    }
  }
  // natural logarithm of the sum of exp(score) over the keys seen: for a later mix with further keys
  if (lse != nullptr && lane == 0) lse[(size_t)t * n_heads + h] = m + logf(l);
}

// ---------------------------------------------------------------------------
// decode: one query per sequence over the pages of the cache, split over pages
// partial layout: [B, n_heads, n_splits, hd + 2] = (acc[hd], m, l)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WAVE) void attn_decode_simple_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, int ring_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_len, float* __restrict__ partial, int n_heads, int n_kv_heads, int hd, int window,
    int n_splits, int n_pages, int page_layout, ScoreBias sb) {
  __shared__ float qs[MAX_HD];
  __shared__ float ps[WAVE];
  const int b = blockIdx.x, h = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
  float* part = partial + (((size_t)b * n_heads + h) * n_splits + split) * (hd + 2);
  const int slot = seq_slot[b];
  const int L = slot >= 0 ? seq_len[b] : 0;
  float m = -FLT_MAX, l = 0.f;
  float acc[ACC];
#pragma unroll
  for (int a = 0; a < ACC; ++a) acc[a] = 0.f;

  if (L > 0) {
    const int g = h / (n_heads / n_kv_heads);
    const int lo = window > 0 ? max(0, L - window) : 0;       // first visible position
    const int first_page = lo / PAGE, last_page = (L - 1) / PAGE;
    const int total = last_page - first_page + 1;
    const int per = (total + n_splits - 1) / n_splits;
    const int p_begin = first_page + split * per;
    const int p_end = min(last_page + 1, p_begin + per);
    const float inv = sqrtf((float)hd);
    for (int i = lane; i < hd; i += WAVE) qs[i] = to_f32(q[((size_t)b * n_heads + h) * hd + i]);
    __syncthreads();
    for (int ap = p_begin; ap < p_end; ++ap) {
      int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys < 0 || phys >= n_pages) continue;               // never the case for a live sequence
      const T* kp = k_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
      const T* vp = v_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
      int pos = ap * PAGE + lane;
      bool valid = pos >= lo && pos < L;
      float s = -FLT_MAX;
      if (valid) {
        float d = 0.f;
        for (int i = 0; i < hd; ++i) d = fmaf(qs[i], to_f32(kp[page_k_offset(page_layout, lane, i, hd)]), d);
        s = d / inv + sb.at(h, L - 1 - pos);
      }
      float m_new = fmaxf(m, wave_max(s));
      float p = valid ? expf(s - m_new) : 0.f;
      float corr = expf(m - m_new);
      l = l * corr + wave_sum(p);
      m = m_new;
      __syncthreads();
      ps[lane] = p;
      __syncthreads();
#pragma unroll
      for (int a = 0; a < ACC; ++a) {
        int d = lane + a * WAVE;
        if (d < hd) {
          float s2 = 0.f;
          for (int jj = 0; jj < PAGE; ++jj) {
            float pj = ps[jj];                                   // rows outside the mask may hold anything
            if (pj != 0.f) s2 = fmaf(pj, to_f32(vp[page_v_offset(page_layout, jj, d, hd)]), s2);
          }
          acc[a] = acc[a] * corr + s2;
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < ACC; ++a) {
    int d = lane + a * WAVE;
    if (d < hd) part[d] = acc[a];
  }
  if (lane == 0) {
    part[hd] = m;
    part[hd + 1] = l;
  }
}

// BASE2: the maxima of the partial results are exponents of 2 (the matrix-core kernel's), else of e.
// With sk.n_sinks > 0 the attention sinks that the query's window no longer covers count as further
// splits of one key each (maximum = score, denominator 1, sum = value): their scores are worked out
// here, with the keys turned, while the splits' loads are in flight; and a token at one of its
// sequence's first positions stores its key and value as a sink (no query of the launch reads it: one
// token a sequence, and the window, at least n_sinks wide, still covers it).
template <typename T, bool BASE2 = false>
__global__ __launch_bounds__(COMBINE_THREADS) void attn_decode_combine_kernel(const float* __restrict__ partial,
                                                                             T* __restrict__ out,
                                                                             float* __restrict__ lse, int n_heads,
                                                                             int hd, int n_splits, SinkArgs sk) {
  // One trip to memory: every wave asks for the maxima and denominators of all splits (lanes over
  // splits) and, before it waits for them, for the sums of its own first splits (waves share the
  // splits of the weighted sum and add their parts in a fixed order).
  constexpr int NWV = COMBINE_THREADS / WAVE;
  constexpr int PRE = 4;                          // splits a wave asks for ahead
  __shared__ float accs[NWV][MAX_HD];
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & (WAVE - 1), g = threadIdx.x / WAVE;
  const int stride = hd + 2;
  const float* part = partial + ((size_t)b * n_heads + h) * n_splits * stride;
  auto weight = [](float d) { return BASE2 ? exp2f(d) : expf(d); };
  float pre[PRE][ACC];
#pragma unroll
  for (int u = 0; u < PRE; ++u) {
    const int sp = min(g + u * NWV, n_splits - 1);
#pragma unroll
    for (int j = 0; j < ACC; ++j) {
      pre[u][j] = part[(size_t)sp * stride + min(lane + j * WAVE, hd - 1)];   // elements beyond hd are never stored
    }
  }
  const int s0 = min(lane, n_splits - 1);
  const float m0 = part[(size_t)s0 * stride + hd], l0 = part[(size_t)s0 * stride + hd + 1];
  __shared__ float sink_score[YALM_MAX_SINKS];
  int n_behind = 0;                               // sinks behind the window of this query
  const T* sv = nullptr;
  if (sk.n_sinks > 0) {                           // the same for the whole launch
    const int slot = sk.seq_slot[b];
    const int pos = sk.seq_len[b] - 1;
    if (slot >= 0 && slot < sk.n_slots) {
      const int kvh = h / (n_heads / sk.n_kv_heads);
      if (sk.k_pages != nullptr && pos < sk.n_sinks && h < sk.n_kv_heads) {
        const int page = sk.block_table[(size_t)slot * sk.table_stride];
        if (page >= 0 && page < sk.n_pages)
          copy_sink((const T*)sk.k_pages, (const T*)sk.v_pages, sk.page_layout, page, h, pos, slot, (T*)sk.sink_k,
                    (T*)sk.sink_v, sk.n_kv_heads, hd, sk.n_sinks, (int)threadIdx.x, COMBINE_THREADS);
      }
      n_behind = max(0, min(sk.n_sinks, pos - sk.window + 1));
      if (n_behind > 0) {
        const int turn = max(0, pos - sk.window - sk.n_sinks + 1);
        const int half_rot = sk.rotary_dim / 2;
        const float2* cs = sk.cos_sin != nullptr && turn > 0 && turn < sk.n_positions
                               ? sk.cos_sin + (size_t)turn * half_rot : nullptr;
        const T* qr = (const T*)sk.q + ((size_t)b * n_heads + h) * hd;
        const T* kbase = (const T*)sk.sink_k + ((size_t)slot * sk.n_kv_heads + kvh) * sk.n_sinks * hd;
        sv = (const T*)sk.sink_v + ((size_t)slot * sk.n_kv_heads + kvh) * sk.n_sinks * hd;
        const float to_exponent = (BASE2 ? 1.4426950408889634f : 1.0f) / sqrtf((float)hd);
        for (int j = g; j < n_behind; j += NWV) {
          const float d = sink_dot(qr, kbase + (size_t)j * hd, cs, hd, half_rot, lane);
          if (lane == 0) sink_score[j] = d * to_exponent;
        }
      }
    }
    __syncthreads();
  }
  float m = lane < n_splits ? m0 : -FLT_MAX;
  for (int sp = lane + WAVE; sp < n_splits; sp += WAVE) m = fmaxf(m, part[(size_t)sp * stride + hd]);
  m = wave_max(m);
  for (int j = 0; j < n_behind; ++j) m = fmaxf(m, sink_score[j]);
  float l = lane < n_splits ? l0 * weight(m0 - m) : 0.f;
  for (int sp = lane + WAVE; sp < n_splits; sp += WAVE) {
    const float* ps = part + (size_t)sp * stride;
    l += ps[hd + 1] * weight(ps[hd] - m);
  }
  l = wave_sum(l);
  for (int j = 0; j < n_behind; ++j) l += weight(sink_score[j] - m);
  const float inv_l = l > 0.f ? 1.0f / l : 0.f;
  if (lse != nullptr && threadIdx.x == 0)
    lse[(size_t)b * n_heads + h] = l > 0.f ? (BASE2 ? m * 0.6931471805599453f : m) + logf(l) : -FLT_MAX;
  float a[ACC];
#pragma unroll
  for (int j = 0; j < ACC; ++j) a[j] = 0.f;
#pragma unroll
  for (int u = 0; u < PRE; ++u) {
    const int sp = g + u * NWV;
    if (sp < n_splits) {
      const float w = weight(part[(size_t)sp * stride + hd] - m);
#pragma unroll
      for (int j = 0; j < ACC; ++j) a[j] += pre[u][j] * w;
    }
  }
  for (int sp = g + PRE * NWV; sp < n_splits; sp += NWV) {
    const float* ps = part + (size_t)sp * stride;
    const float w = weight(ps[hd] - m);
#pragma unroll
    for (int j = 0; j < ACC; ++j) {
      const int d = lane + j * WAVE;
      if (d < hd) a[j] += ps[d] * w;
    }
  }
#pragma unroll
  for (int j = 0; j < ACC; ++j) accs[g][lane + j * WAVE] = a[j];
  __syncthreads();
  if (g == 0) {
#pragma unroll
    for (int j = 0; j < ACC; ++j) {
      const int d = lane + j * WAVE;
      if (d >= hd) continue;
      float t = accs[0][d];
#pragma unroll
      for (int w = 1; w < NWV; ++w) t += accs[w][d];
      for (int s = 0; s < n_behind; ++s) t = fmaf(weight(sink_score[s] - m), to_f32(sv[(size_t)s * hd + d]), t);
      out[((size_t)b * n_heads + h) * hd + d] = from_f32<T>(t * inv_l);
    }
  }
}

bool bad_heads(int n_heads, int n_kv_heads, int hd) {
  return n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || hd <= 0 || hd > MAX_HD;
}
}  // namespace

extern "C" int yalm_attn_prefill_lse(const void* q, const void* k_stage, const void* v_stage, void* out, float* out_f32,
                                     float* lse,
                                     const int* cu_seqlens, const int* seq_tile0, const int* tok_seq, const int* tok_pos,
                                 const int* tile_order, int n_order, int T, int B, int n_tiles, int n_heads,
                                 int n_kv_heads, int head_dim, int window, int dtype, int force_simple,
                                 const float* score_bias, int n_bias, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (bad_heads(n_heads, n_kv_heads, head_dim) || window < 0 || n_tiles <= 0) return YALM_ERR_ARG;
  if (score_bias != nullptr && n_bias <= 0) return YALM_ERR_ARG;
  const ScoreBias sb = {score_bias, n_bias};
  dim3 grid(T, n_heads);
  if (dtype == YALM_F32) {
    attn_prefill_simple_kernel<float><<<grid, WAVE, 0, stream>>>((const float*)q, (const float*)k_stage,
                                                                 (const float*)v_stage, (float*)out, out_f32, lse, seq_tile0,
                                                                 tok_seq, tok_pos, n_heads, n_kv_heads, head_dim,
                                                                 window, sb);
    return launch_status();
  }
  if (dtype != YALM_BF16) return YALM_ERR_DTYPE;
  if (!force_simple) {
    int rc = yalm_attn_prefill_bf16_mfma(q, k_stage, v_stage, out, out_f32, lse, cu_seqlens, seq_tile0, tile_order, n_order, T, B,
                                         n_tiles, n_heads, n_kv_heads, head_dim, window, score_bias, n_bias, stream);
    if (rc != YALM_ERR_ARG) return rc;
  }
  attn_prefill_simple_kernel<bf16><<<grid, WAVE, 0, stream>>>((const bf16*)q, (const bf16*)k_stage,
                                                              (const bf16*)v_stage, (bf16*)out, out_f32, lse, seq_tile0, tok_seq,
                                                              tok_pos, n_heads, n_kv_heads, head_dim, window, sb);
  return launch_status();
}

extern "C" int yalm_attn_prefill(const void* q, const void* k_stage, const void* v_stage, void* out,
                                 const int* cu_seqlens, const int* seq_tile0, const int* tok_seq, const int* tok_pos,
                                 const int* tile_order, int n_order, int T, int B, int n_tiles, int n_heads,
                                 int n_kv_heads, int head_dim, int window, int dtype, int force_simple,
                                 hipStream_t stream) {
  return yalm_attn_prefill_lse(q, k_stage, v_stage, out, nullptr, nullptr, cu_seqlens, seq_tile0, tok_seq, tok_pos, tile_order,
                               n_order, T, B, n_tiles, n_heads, n_kv_heads, head_dim, window, dtype, force_simple,
                               nullptr, 0, stream);
}

// merges the partial results of the splits (also used by the MFMA kernel)
int yalm_attn_decode_combine_bf16(const float* partial, void* out, float* lse, int B, int n_heads, int head_dim,
                                  int n_splits, int base2, const SinkArgs& sinks, hipStream_t stream) {
  dim3 cgrid(B, n_heads);
  if (base2)
    attn_decode_combine_kernel<bf16, true><<<cgrid, COMBINE_THREADS, 0, stream>>>(partial, (bf16*)out, lse, n_heads,
                                                                                  head_dim, n_splits, sinks);
  else
    attn_decode_combine_kernel<bf16><<<cgrid, COMBINE_THREADS, 0, stream>>>(partial, (bf16*)out, lse, n_heads,
                                                                            head_dim, n_splits, sinks);
  return launch_status();
}

extern "C" long yalm_attn_decode_workspace(int B, int n_heads, int head_dim, int n_splits) {
  return (long)B * n_heads * n_splits * (head_dim + 2) * (long)sizeof(float);
}

namespace {
int attn_decode_any(const void* q, const void* k_pages, const void* v_pages, const int* block_table, int table_stride,
                    int ring_pages, const int* seq_slot, const int* seq_len, void* out, float* lse, float* partial,
                    int B, int n_heads, int n_kv_heads, int head_dim, int window, int n_splits, int n_pages,
                    int page_layout, int dtype, int force_simple, const SinkArgs& sinks, const int* step_max_len,
                    const int* seq_order, const float* score_bias, int n_bias, hipStream_t stream) {
  if (B <= 0) return YALM_OK;
  if (score_bias != nullptr && (n_bias <= 0 || sinks.n_sinks > 0)) return YALM_ERR_ARG;   // sinks are scored without it
  const ScoreBias sb = {score_bias, n_bias};
  if (bad_heads(n_heads, n_kv_heads, head_dim) || window < 0 || n_splits <= 0 || ring_pages <= 0 ||
      !page_layout_ok(page_layout, head_dim))
    return YALM_ERR_ARG;
  dim3 grid(B, n_heads, n_splits), cgrid(B, n_heads);
  if (dtype == YALM_F32) {
    attn_decode_simple_kernel<float><<<grid, WAVE, 0, stream>>>(
        (const float*)q, (const float*)k_pages, (const float*)v_pages, block_table, table_stride, ring_pages,
        seq_slot, seq_len, partial, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages, page_layout, sb);
    attn_decode_combine_kernel<float><<<cgrid, COMBINE_THREADS, 0, stream>>>(partial, (float*)out, lse, n_heads,
                                                                             head_dim, n_splits, sinks);
    return launch_status();
  }
  if (dtype != YALM_BF16) return YALM_ERR_DTYPE;
  if (!force_simple) {
    int rc = yalm_attn_decode_bf16_mfma(q, k_pages, v_pages, block_table, table_stride, ring_pages, seq_slot, seq_len,
                                        out, lse, partial, B, n_heads, n_kv_heads, head_dim, window, n_splits,
                                        n_pages, page_layout, sinks, step_max_len, seq_order, score_bias, n_bias, stream);
    if (rc != YALM_ERR_ARG) return rc;
  }
  attn_decode_simple_kernel<bf16><<<grid, WAVE, 0, stream>>>(
      (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, block_table, table_stride, ring_pages, seq_slot,
      seq_len, partial, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages, page_layout, sb);
  attn_decode_combine_kernel<bf16><<<cgrid, COMBINE_THREADS, 0, stream>>>(partial, (bf16*)out, lse, n_heads, head_dim,
                                                                          n_splits, sinks);
  return launch_status();
}
}  // namespace

extern "C" int yalm_attn_decode_lse(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                    int table_stride, int ring_pages, const int* seq_slot, const int* seq_len,
                                    void* out, float* lse, float* partial, int B, int n_heads, int n_kv_heads,
                                    int head_dim, int window, int n_splits, int n_pages, int page_layout, int dtype,
                                    int force_simple, const int* step_max_len, const int* seq_order,
                                    const float* score_bias, int n_bias, hipStream_t stream) {
  SinkArgs none = {};
  return attn_decode_any(q, k_pages, v_pages, block_table, table_stride, ring_pages, seq_slot, seq_len, out, lse,
                         partial, B, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages, page_layout, dtype,
                         force_simple, none, step_max_len, seq_order, score_bias, n_bias, stream);
}

extern "C" int yalm_attn_decode(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                int table_stride, int ring_pages, const int* seq_slot, const int* seq_len, void* out,
                                float* partial, int B, int n_heads, int n_kv_heads, int head_dim, int window,
                                int n_splits, int n_pages, int dtype, int force_simple, hipStream_t stream) {
  return yalm_attn_decode_lse(q, k_pages, v_pages, block_table, table_stride, ring_pages, seq_slot, seq_len, out,
                              nullptr, partial, B, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages,
                              YALM_PAGE_ROWS, dtype, force_simple, nullptr, nullptr, nullptr, 0, stream);
}

extern "C" int yalm_attn_decode_sinks(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                      int table_stride, int ring_pages, const int* seq_slot, const int* seq_len,
                                      void* out, float* partial, void* sink_k, void* sink_v, int store,
                                      const float* cos_sin, int n_positions, int n_slots, int rotary_dim, int n_sinks,
                                      int B, int n_heads, int n_kv_heads, int head_dim, int window, int n_splits,
                                      int n_pages, int page_layout, int dtype, int force_simple,
                                      const int* step_max_len, const int* seq_order, hipStream_t stream) {
  if (n_sinks <= 0 || n_sinks > YALM_MAX_SINKS || window < n_sinks || n_slots <= 0 || sink_k == nullptr ||
      sink_v == nullptr || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2 || head_dim % 2)
    return YALM_ERR_ARG;
  SinkArgs sk = {};
  sk.q = q;
  sk.sink_k = sink_k;
  sk.sink_v = sink_v;
  if (store) {
    sk.k_pages = k_pages;
    sk.v_pages = v_pages;
    sk.block_table = block_table;
    sk.table_stride = table_stride;
    sk.n_pages = n_pages;
    sk.page_layout = page_layout;
  }
  sk.seq_slot = seq_slot;
  sk.seq_len = seq_len;
  sk.cos_sin = rotary_dim > 0 ? (const float2*)cos_sin : nullptr;
  sk.n_positions = n_positions;
  sk.n_slots = n_slots;
  sk.n_kv_heads = n_kv_heads;
  sk.rotary_dim = rotary_dim;
  sk.window = window;
  sk.n_sinks = n_sinks;
  return attn_decode_any(q, k_pages, v_pages, block_table, table_stride, ring_pages, seq_slot, seq_len, out, nullptr,
                         partial, B, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages, page_layout, dtype,
                         force_simple, sk, step_max_len, seq_order, nullptr, 0, stream);
}

// ---------------------------------------------------------------------------
// yalm_attn_decode for callers that cannot allocate: the partial results of the splits go to a
// fixed array in device memory instead of a workspace of the caller's.  Every GPU that the library
// runs on holds its own copy of the array, at its own address, until the process ends.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float scratch[YALM_ATTN_DECODE_STATIC_BYTES / sizeof(float)];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
float* scratch_of_device[MAX_DEVICES];      // the array's address on each device, asked for once

// The address of `scratch` on the current device (in host code the array's name is no device address).
int scratch_pointer(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return YALM_ERR_ARG;
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (scratch_of_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return YALM_ERR_ARG;
    scratch_of_device[dev] = (float*)p;
  }
  *ptr = scratch_of_device[dev];
  return YALM_OK;
}
}  // namespace

extern "C" int yalm_attn_decode_static(const void* q, const void* k_pages, const void* v_pages,
                                       const int* block_table, int table_stride, int ring_pages,
                                       const int* seq_slot, const int* seq_len, void* out, int B, int n_heads,
                                       int n_kv_heads, int head_dim, int window, int n_splits, int n_pages, int dtype,
                                       int force_simple, hipStream_t stream) {
  if (B <= 0) return YALM_OK;
  if (bad_heads(n_heads, n_kv_heads, head_dim) || window < 0 || n_splits <= 0 || ring_pages <= 0)
    return YALM_ERR_ARG;
  if (yalm_attn_decode_workspace(B, n_heads, head_dim, n_splits) > (long)YALM_ATTN_DECODE_STATIC_BYTES)
    return YALM_ERR_SCRATCH;
  float* partial = nullptr;
  int rc = scratch_pointer(&partial);
  if (rc != YALM_OK) return rc;
  // nothing in the array has to start at zero: every split of every (sequence, head) writes its
  // sums, maximum and denominator before the merge reads them, also for padding rows
  return yalm_attn_decode(q, k_pages, v_pages, block_table, table_stride, ring_pages, seq_slot, seq_len, out, partial,
                          B, n_heads, n_kv_heads, head_dim, window, n_splits, n_pages, dtype, force_simple, stream);
}
