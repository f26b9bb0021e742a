// Attention of whole prompts on the matrix cores (see attention_mfma.h for the products' layout).
#include "attention_mfma.h"

namespace {

// ---------------------------------------------------------------------------
// prefill: a workgroup takes 64 * NC query positions of one head (4 waves x NC 16-position
// column tiles); key/value tiles of 64 rows go through LDS once per workgroup, double-
// buffered, rows stored in the order the MFMA operands read them.  grid (head, 64-position
// tile): with NC = 2 (the one in use: each key tile read from LDS serves more queries; NC = 1
// measured no faster at 2,048 tokens and slower beyond) the workgroup of every second tile of
// a sequence works.  The heads of a tile are neighbours in the launch order, so that the
// workgroups running together cost the same and the heads of a group share their keys in the
// cache; the tiles that see the most keys start first.  With tile_order (the working tiles,
// those that see the most keys first) only these are launched, and from workgroup fold_at on
// the order is turned round: when every compute unit gets two workgroups, the second of the
// one that began with the longest is the shortest.
// ---------------------------------------------------------------------------
//
// KSPL = 2: two groups of four waves share the queries and take every second key tile each, with
// LDS buffers of their own, and merge their results through LDS at the end.  A workgroup then fills a
// compute unit alone and is done in half the time, so that the compute units are no longer held by
// the few workgroups that see the most keys (with KSPL = 1 the launch lasts as long as its longest
// workgroup, 32 key tiles at 2,048 tokens, while the mean is 17).
// BIAS: a term is added to every score by the distance of query and key, bias[head][min(distance, n_bias - 1)].
template <int HD, int NC, int KSPL, bool BIAS>
__global__ __launch_bounds__(256 * KSPL, KSPL == 1 ? 2 : 1) void attn_prefill_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_stage, const bf16* __restrict__ v_stage,
    bf16* __restrict__ out, float* __restrict__ out_f32, float* __restrict__ lse, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_tile0, const int* __restrict__ tile_order, int fold_at, int B, int n_heads,
    int n_kv_heads, int window, const float* __restrict__ bias, int n_bias) {
  // A head size that is no multiple of 32: the last step of the scores' product is half empty (zeros in the query's
  // lanes, the row's last 8 elements once more in the keys'), and the tile's chunks do not divide evenly over the threads.
  constexpr int KS = (HD + 31) / 32, DT = HD / 16;
  static_assert(HD % 16 == 0, "head sizes in steps of 16");
  constexpr int KROW = HD + 8;                    // LDS row strides (elements): 16 bytes of padding
  constexpr int VROW = PAGE + 8;
  constexpr int KTILE = PAGE * KROW, VTILE = HD * VROW;
  constexpr int CHUNKS = PAGE * HD / 8;           // 16-byte chunks of a tile
  constexpr int NLOAD = (CHUNKS + 255) / 256;     // chunks per thread and tile
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* smem = reinterpret_cast<bf16*>(smem_raw);   // [2][KSPL][KTILE + VTILE]

  // heads run fastest and tiles from the last to the first: within a sequence the last tiles see
  // the most keys, and workgroups that start first should be the long ones
  int h = blockIdx.x, gt = (int)gridDim.y - 1 - (int)blockIdx.y;
  if (tile_order) {
    int lin = (int)blockIdx.y * n_heads + h;
    const int total = (int)gridDim.y * n_heads;
    if (lin >= fold_at) lin = total - 1 - (lin - fold_at);
    h = lin % n_heads;
    gt = tile_order[lin / n_heads];
    if ((unsigned)gt >= (unsigned)seq_tile0[B]) return;
  }
  // half: which group of four waves (which key tiles); tid, wave: the thread's place inside its group
  const int half = __builtin_amdgcn_readfirstlane((int)threadIdx.x / 256), tid = threadIdx.x % 256;
  const int wave = tid / WAVE, lane = tid % WAVE, qd = lane / 16, j = lane % 16;
  int b = 0;
  {
    int lo_b = 0, hi_b = B - 1;
    while (lo_b < hi_b) {
      int mid = (lo_b + hi_b + 1) >> 1;
      if (seq_tile0[mid] <= gt) lo_b = mid; else hi_b = mid - 1;
    }
    b = lo_b;
  }
  const int tile0 = seq_tile0[b];
  const int tq = gt - tile0;
  if (NC == 2 && (tq & 1)) return;                // the workgroup of the even tile covers this one too
  const int start = cu_seqlens[b], len = cu_seqlens[b + 1] - start;
  const int g = h / (n_heads / n_kv_heads);
  const float score_scale = 1.4426950408889634f / sqrtf((float)HD);   // log2(e) / sqrt(head_dim)
  const float* bias_row = BIAS ? bias + (size_t)h * n_bias : nullptr;

  const int blk0 = tq * PAGE;                     // first position of the workgroup
  const int pos0 = blk0 + wave * 16 * NC;         // first position of the wave
  const bool wave_live = pos0 < len;
  bf16x8 qv[NC][KS];
  bool q_ok[NC];
  int pos_q[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    pos_q[c] = pos0 + c * 16 + j;
    q_ok[c] = pos_q[c] < len;
    const bf16* qrow = q + ((size_t)(start + (q_ok[c] ? pos_q[c] : 0)) * n_heads + h) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qv[c][ks] = q_ok[c] && ks * 32 + qd * 8 < HD ? ld8(qrow + ks * 32 + qd * 8) : zero8();
  }
  float m[NC], l[NC];
  f32x4 o[NC][DT];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    m[c] = -FLT_MAX;
    l[c] = 0.f;
  }
#pragma unroll
  for (int c = 0; c < NC; ++c)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[c][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int blk_last = min(blk0 + NC * PAGE - 1, len - 1);
  const int kt_hi = blk_last / PAGE;
  const int kt_lo = window > 0 ? max(0, blk0 - window + 1) / PAGE : 0;
  const int wave_last = min(pos0 + 16 * NC - 1, len - 1);
  const size_t tile_elems = (size_t)n_kv_heads * PAGE * HD;

  // global -> registers -> LDS; key rows are stored at the index the MFMA row reads them at
  bf16x8 rk[NLOAD], rv[NLOAD];
  auto load_tile = [&](int kt) {
    const bf16* kp = k_stage + (tile0 + kt) * tile_elems + (size_t)g * PAGE * HD;
    const bf16* vp = v_stage + (tile0 + kt) * tile_elems + (size_t)g * PAGE * HD;
#pragma unroll
    for (int p = 0; p < NLOAD; ++p) {
      int c = min(tid + p * 256, CHUNKS - 1);       // a thread beyond the tile reads its last chunk and stores nothing
      rk[p] = ld8(kp + (size_t)c * 8);
      rv[p] = ld8(vp + (size_t)c * 8);
    }
  };
  auto store_tile = [&](int buf) {
    bf16* ks_l = smem + (buf * KSPL + half) * (KTILE + VTILE);
    bf16* vs_l = ks_l + KTILE;
#pragma unroll
    for (int p = 0; p < NLOAD; ++p) {
      int c = tid + p * 256;
      if (CHUNKS % 256 != 0 && c >= CHUNKS) break;
      int row = c / (HD / 8), col = (c % (HD / 8)) * 8;              // key tile: [row][element]
      int t = 2 * (row >> 5) + ((row >> 2) & 1), i = 4 * ((row >> 3) & 3) + (row & 3);
      *reinterpret_cast<bf16x8*>(ks_l + (t * 16 + i) * KROW + col) = rk[p];
      int vrow = c / 8, vcol = (c % 8) * 8;                            // value tile: [element][row]
      *reinterpret_cast<bf16x8*>(vs_l + vrow * VROW + vcol) = rv[p];
    }
  };

  if (kt_lo + half <= kt_hi) {
    load_tile(kt_lo + half);
    store_tile(0);
  }
  __syncthreads();
  for (int kt0 = kt_lo; kt0 <= kt_hi; kt0 += KSPL) {        // every group its own tile of the round
    const int kt = kt0 + half;
    const int cur = ((kt0 - kt_lo) / KSPL) & 1;
    const bool next = kt + KSPL <= kt_hi;
    if (next) load_tile(kt + KSPL);
    const int base = kt * PAGE;
    const bool visible = kt <= kt_hi && wave_live && base <= wave_last &&
                         (window == 0 || base + PAGE - 1 > pos0 - window);
    if (visible) {
      const bf16* ks_l = smem + (cur * KSPL + half) * (KTILE + VTILE);
      const bf16* vs_l = ks_l + KTILE;
      f32x4 sc[NC][4];
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int t = 0; t < 4; ++t) sc[c][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks_l + (t * 16 + j) * KROW + min(ks * 32 + qd * 8, HD - 8));
#pragma unroll
          for (int c = 0; c < NC; ++c)
            sc[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qv[c][ks], sc[c][t], 0, 0, 0);
        }
      const bool edge = base + PAGE - 1 > pos0 || (window > 0 && base < pos0 + 16 * NC - 1 - window + 1);
      bf16x8 pb[NC][2];
      float corr[NC];
      // scores in the base-2 domain: p = 2^(s * log2(e) / sqrt(hd) - m)
      auto softmax_tile = [&](auto masked) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          // the maximum is taken over the raw dot products and scaled once (the scale is positive); every
          // score is then scaled and has the maximum taken off in one fused multiply-add
          float mx = -FLT_MAX;
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float v = sc[c][t][r];
              if constexpr (BIAS) {               // scaled here, with the distance's term in the same units (exponents of 2)
                const int dist = pos_q[c] - (base + 32 * (t >> 1) + 8 * qd + 4 * (t & 1) + r);
                v = fmaf(v, score_scale, bias_row[min(max(dist, 0), n_bias - 1)] * 1.4426950408889634f);
                sc[c][t][r] = v;
              }
              if (decltype(masked)::value) {
                int kpos = base + 32 * (t >> 1) + 8 * qd + 4 * (t & 1) + r;
                bool vis = kpos <= pos_q[c] && (window == 0 || pos_q[c] - kpos < window) && q_ok[c];
                v = vis ? v : -INFINITY;
                sc[c][t][r] = v;
              }
              mx = fmaxf(mx, v);
            }
          mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
          mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
          const float m_new = fmaxf(m[c], BIAS ? mx : mx * score_scale);
          corr[c] = __builtin_amdgcn_exp2f(m[c] - m_new);
          float psum = 0.f;
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float sv = sc[c][2 * s2 + (e >> 2)][e & 3];
              float p = __builtin_amdgcn_exp2f(BIAS ? sv - m_new : fmaf(sv, score_scale, -m_new));
              psum += p;
              pb[c][s2][e] = static_cast<bf16>(p);
            }
          l[c] = l[c] * corr[c] + psum;
          m[c] = m_new;
        }
      };
      if (edge)
        softmax_tile(std::true_type{});
      else
        softmax_tile(std::false_type{});
      bool settled = true;                        // the maxima settle after a few tiles
#pragma unroll
      for (int c = 0; c < NC; ++c) settled = settled && corr[c] == 1.0f;
      const bool rescale = !__all(settled);
      const bool tail = base + PAGE > len;        // rows behind the sequence's end may hold anything
      if (rescale) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int c = 0; c < NC; ++c) o[c][dt] *= corr[c];
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          bf16x8 vf = *reinterpret_cast<const bf16x8*>(vs_l + (dt * 16 + j) * VROW + s2 * 32 + qd * 8);
          if (tail) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (base + 32 * s2 + 8 * qd + e >= len) vf[e] = static_cast<bf16>(0.f);
          }
#pragma unroll
          for (int c = 0; c < NC; ++c)
            o[c][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[c][s2], o[c][dt], 0, 0, 0);
        }
      }
    }
    if (next) store_tile(cur ^ 1);
    __syncthreads();
  }
  if constexpr (KSPL == 2) {
    // the second group hands its maxima, denominators and sums to the first, which merges and writes
    f32x4* mo = reinterpret_cast<f32x4*>(smem_raw);            // [NC][DT][256]
    float* ml = reinterpret_cast<float*>(mo + NC * DT * 256);   // [NC][2][256]
    if (half == 1) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) mo[(c * DT + dt) * 256 + tid] = o[c][dt];
        ml[(c * 2) * 256 + tid] = m[c];
        ml[(c * 2 + 1) * 256 + tid] = l[c];
      }
    }
    __syncthreads();
    if (half == 1) return;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const float m2 = ml[(c * 2) * 256 + tid], l2 = ml[(c * 2 + 1) * 256 + tid];
      const float m_new = fmaxf(m[c], m2);
      const float f1 = __builtin_amdgcn_exp2f(m[c] - m_new), f2 = __builtin_amdgcn_exp2f(m2 - m_new);
      l[c] = l[c] * f1 + l2 * f2;
      m[c] = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[c][dt] = o[c][dt] * f1 + mo[(c * DT + dt) * 256 + tid] * f2;
    }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    float lt = l[c];
    lt += __shfl_xor(lt, 16, WAVE);
    lt += __shfl_xor(lt, 32, WAVE);
    if (q_ok[c]) {
      bf16* orow = out + ((size_t)(start + pos_q[c]) * n_heads + h) * HD;
      const float inv_l = 1.0f / lt;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) orow[dt * 16 + 4 * qd + r] = static_cast<bf16>(o[c][dt][r] * inv_l);
      if (out_f32 != nullptr) {                   // the unrounded row too, for whoever mixes further keys in
        float* frow = out_f32 + ((size_t)(start + pos_q[c]) * n_heads + h) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) frow[dt * 16 + 4 * qd + r] = o[c][dt][r] * inv_l;
      }
      if (lse != nullptr && qd == 0) lse[(size_t)(start + pos_q[c]) * n_heads + h] = m[c] * LN2 + logf(lt);
    }
  }
}

// compute units of the current device (asked once: this library drives one device a process)
int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    n = v;
  }
  return n;
}

// launches attn_prefill_mfma_kernel<head_dim, NC, KSPL> (more than 64 KB of LDS is asked for once a device)
template <int HD, int NC, int KSPL, bool BIAS>
int launch_prefill(dim3 grid, int threads, size_t lds, hipStream_t stream, const bf16* qp, const bf16* kp, const bf16* vp,
                   bf16* out, float* out_f32, float* lse, const int* cu_seqlens, const int* seq_tile0,
                   const int* tile_order, int fold_at, int B, int n_heads, int n_kv_heads, int window,
                   const float* bias, int n_bias) {
  auto kernel = &attn_prefill_mfma_kernel<HD, NC, KSPL, BIAS>;
  if (lds > 64 * 1024) {
    static LdsAllowance allowed;
    if (int rc = allow_dynamic_lds(allowed, (const void*)kernel, 150 * 1024); rc != YALM_OK) return rc;
  }
  kernel<<<grid, threads, lds, stream>>>(qp, kp, vp, out, out_f32, lse, cu_seqlens, seq_tile0, tile_order, fold_at, B,
                                         n_heads, n_kv_heads, window, bias, n_bias);
  return launch_status();
}
template <int NC, int KSPL, typename... Args>
int launch_prefill_hd(int head_dim, bool biased, Args... args) {
#define YALM_PREFILL_HD(HD_)                                                        \
  case HD_:                                                                         \
    return biased ? launch_prefill<HD_, NC, KSPL, true>(args...) : launch_prefill<HD_, NC, KSPL, false>(args...)
  switch (head_dim) {
    YALM_PREFILL_HD(16);
    YALM_PREFILL_HD(32);
    YALM_PREFILL_HD(48);
    YALM_PREFILL_HD(64);
    YALM_PREFILL_HD(80);
    YALM_PREFILL_HD(96);
    YALM_PREFILL_HD(112);
    YALM_PREFILL_HD(128);
  }
#undef YALM_PREFILL_HD
  return YALM_ERR_ARG;
}
}  // namespace

int yalm_attn_prefill_bf16_mfma(const void* q, const void* k_stage, const void* v_stage, void* out, float* out_f32,
                                float* lse,
                                const int* cu_seqlens, const int* seq_tile0, const int* tile_order, int n_order,
                                int T, int B, int n_tiles, int n_heads, int n_kv_heads, int head_dim, int window,
                                const float* bias, int n_bias, hipStream_t stream) {
  if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim) || n_tiles > 65535) return YALM_ERR_ARG;
  if (bias != nullptr && n_bias <= 0) return YALM_ERR_ARG;
  const bool biased = bias != nullptr;
  if (tile_order && (n_order <= 0 || n_order > n_tiles)) return YALM_ERR_ARG;
  dim3 grid(n_heads, tile_order ? n_order : n_tiles);
  const long total = (long)grid.x * grid.y;
  const size_t tile_bytes = ((size_t)PAGE * (head_dim + 8) + (size_t)head_dim * (PAGE + 8)) * sizeof(bf16);
  const bf16 *qp = (const bf16*)q, *kp = (const bf16*)k_stage, *vp = (const bf16*)v_stage;
  // Few workgroups (at most two a compute unit, as a prompt of 2,048 tokens with 32 heads makes): the launch
  // would last as long as the workgroup that sees the most keys, so eight waves take each workgroup's keys
  // in two halves (2,048 tokens: 72 against 78 us; 512 tokens 1.6 % of the prompt step).  More workgroups
  // keep the compute units busy anyway, and two independent workgroups of four waves a compute unit are
  // the faster way then (8,192 tokens: 3 % of the step, 16,384: 5 %).
  const long working = (long)n_heads * (tile_order ? n_order : (n_tiles + 1) / 2);
  if ((long)n_heads * n_tiles <= compute_units()) {
    // a short step: a workgroup of eight waves for every tile of 64 queries (not 128), so that twice as many
    // compute units work (512 tokens with 32 heads: 19.6 -> 15.9 us a layer); all of them run at once, so their order
    // does not matter
    return launch_prefill_hd<1, 2>(head_dim, biased, dim3(n_heads, n_tiles), 512, 4 * tile_bytes, stream, qp, kp, vp,
                                   (bf16*)out, out_f32, lse, cu_seqlens, seq_tile0, (const int*)nullptr, 0, B, n_heads,
                                   n_kv_heads, window, bias, n_bias);
  }
  if (working <= 2L * compute_units()) {
    // a workgroup of eight waves a compute unit, the workgroups that see the most keys first
    return launch_prefill_hd<2, 2>(head_dim, biased, grid, 512, 4 * tile_bytes, stream, qp, kp, vp, (bf16*)out, out_f32,
                                   lse, cu_seqlens, seq_tile0, tile_order, (int)total, B, n_heads, n_kv_heads, window,
                                   bias, n_bias);
  }
  // two workgroups fit a compute unit: with more than one and at most two each, the second
  // half of the launch runs from the shortest workgroup up
  const int cus = compute_units();
  const int fold_at = total > cus && total <= 2 * cus ? cus : (int)total;
  return launch_prefill_hd<2, 1>(head_dim, biased, grid, 256, 2 * tile_bytes, stream, qp, kp, vp, (bf16*)out, out_f32,
                                 lse, cu_seqlens, seq_tile0, tile_order, fold_at, B, n_heads, n_kv_heads, window, bias,
                                 n_bias);
}
