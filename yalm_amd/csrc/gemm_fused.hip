// Decode GEMMs (at most 8 rows) that start from the float32 residual stream:
//
//   out = epilogue( rmsnorm(x, w_norm, eps) * W^T )
//
// The norm is folded into the product: every workgroup first puts bfloat16(x * w_norm)
// into LDS and computes rsqrt(mean(x^2) + eps) per row (x is small and sits in L2),
// while its first weights are already on their way; the activations then enter the
// matrix cores from LDS and the float32 sums are scaled afterwards.  That saves a
// kernel and a round trip of the activations per norm.  Epilogues: float32 store (LM head), gated SiLU (feed-forward), and for
// the fused q/k/v projection the rotation of q and k at each row's position and
// the write of k and v into the pages of the cache.
// Same structure as gemm_skinny_kernel: 16 or 32 weight rows a workgroup, the
// waves split K in chunks of 128, partial sums meet in LDS.
#include "common.h"
#include "skinny_gemm.h"
#include "yalm_hip.h"

namespace {

using namespace skinny;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

constexpr int MAX_ROWS = 8;                      // rows of the step (sequences of a decode batch)

// LDS: the normalised activations xs[M][K + 8] as bfloat16 (dynamic), then the partial sums.
template <int NT, int NWAVES, int EPI>
__global__ __launch_bounds__(NWAVES * WAVE) void gemm_norm_kernel(const float* __restrict__ X,
                                                                   const float* __restrict__ norm_w, float eps,
                                                                   const bf16* __restrict__ W, void* __restrict__ Cv,
                                                                   int M, int N, int K, int H, RopeArgs ra) {
  constexpr int KC = 128;
  constexpr int NTHREADS = NWAVES * WAVE;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ f32x4 red[NWAVES][NT][WAVE];
  __shared__ float sm_part[NWAVES][MAX_ROWS];
  __shared__ float sm_scale[16];
  bf16* xs = reinterpret_cast<bf16*>(smem);
  const int xs_row = K + 8;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int q = lane / 16, j = lane % 16;
  const int n0 = blockIdx.x * 16 * NT;

  const bf16* wrow[NT];
  bool wok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int n = n0 + t * 16 + j;
    wok[t] = n < N;
    wrow[t] = W + (size_t)(wok[t] ? n : 0) * K;
  }
  const bf16x8 z8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // the wave's first chunk of weights goes on its way before the activations are prepared
  bf16x8 wv[NT][4];
  int kc = wave * KC;
  if (kc < K) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      int k = kc + s * 32 + q * 8;
      bool ok = k < K;
#pragma unroll
      for (int t = 0; t < NT; ++t) wv[t][s] = (ok && wok[t]) ? *reinterpret_cast<const bf16x8*>(wrow[t] + k) : z8;
    }
  }

  // xs[m][k] = bfloat16(x[m][k] * norm_w[k]); scale[m] = rsqrt(mean(x[m]^2) + eps)
  {
    float ss[MAX_ROWS];
#pragma unroll
    for (int m = 0; m < MAX_ROWS; ++m) ss[m] = 0.f;
#pragma unroll 2
    for (int k = threadIdx.x * 4; k < K; k += NTHREADS * 4) {
      const float4 w4 = *reinterpret_cast<const float4*>(norm_w + k);
#pragma unroll
      for (int m = 0; m < MAX_ROWS; ++m) {
        if (m < M) {
          const float4 a = *reinterpret_cast<const float4*>(X + (size_t)m * K + k);
          ss[m] += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
          bf16x4 d;
          d[0] = static_cast<bf16>(a.x * w4.x);
          d[1] = static_cast<bf16>(a.y * w4.y);
          d[2] = static_cast<bf16>(a.z * w4.z);
          d[3] = static_cast<bf16>(a.w * w4.w);
          *reinterpret_cast<bf16x4*>(xs + (size_t)m * xs_row + k) = d;
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MAX_ROWS; ++m) {
      float v = wave_sum(ss[m]);
      if (lane == 0) sm_part[wave][m] = v;
    }
    __syncthreads();
    if (threadIdx.x < 16) {
      float tot = 0.f;
      if (threadIdx.x < MAX_ROWS)
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) tot += sm_part[w][threadIdx.x];
      sm_scale[threadIdx.x] = 1.0f / sqrtf(tot / (float)K + eps);
    }
    __syncthreads();
  }

  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bool xok = j < M;
  const bf16* xrow = xs + (size_t)(xok ? j : 0) * xs_row;

  for (; kc < K; kc += NWAVES * KC) {
    bf16x8 wn[NT][4];
    const int kn = kc + NWAVES * KC;
    if (kn < K) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        int k = kn + s * 32 + q * 8;
        bool ok = k < K;
#pragma unroll
        for (int t = 0; t < NT; ++t) wn[t][s] = (ok && wok[t]) ? *reinterpret_cast<const bf16x8*>(wrow[t] + k) : z8;
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int k = kc + s * 32 + q * 8;
      const bf16x8 xv = (xok && k < K) ? *reinterpret_cast<const bf16x8*>(xrow + k) : z8;
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv, wv[t][s], acc[t], 0, 0, 0);
    }
    if (kn < K) {
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < NT; ++t) wv[t][s] = wn[t][s];
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();

  constexpr int NTP = (gated(EPI)) ? NT / 2 : NT;
  for (int tp = wave; tp < NTP; tp += NWAVES) {
    float scale[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) scale[r] = sm_scale[4 * q + r];
    if (gated(EPI)) {
      f32x4 g = (f32x4){0.f, 0.f, 0.f, 0.f}, u = g;
#pragma unroll
      for (int w = 0; w < NWAVES; ++w) {
        g += red[w][2 * tp][lane];
        u += red[w][2 * tp + 1][lane];
      }
      const int hcol = (n0 / 32 + tp) * 16 + j;
      bf16* C = (bf16*)Cv;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int m = 4 * q + r;
        if (m < M && hcol < H)
          C[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(g[r] * scale[r]) * (u[r] * scale[r]));
      }
    } else {
      f32x4 v = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NWAVES; ++w) v += red[w][tp][lane];
      const int n = n0 + tp * 16 + j;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] *= scale[r];
      if (EPI == EPI_F32) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int m = 4 * q + r;
          if (m < M && n < N) ((float*)Cv)[(size_t)m * N + n] = v[r];
        }
      } else {                                    // EPI_ROPE: n runs over [q heads | k heads | v heads]
        f32x4 other;
#pragma unroll
        for (int r = 0; r < 4; ++r) other[r] = __shfl_xor(v[r], 1, WAVE);   // the pair partner sits in the next lane
        const int Q = ra.n_heads * ra.hd, KV = ra.n_kv_heads * ra.hd;
        if (n < N) {
          const int region = n < Q ? 0 : (n < Q + KV ? 1 : 2);
          const int nn = n - (region == 0 ? 0 : (region == 1 ? Q : Q + KV));
          const int head = nn / ra.hd, i = nn % ra.hd, p = i >> 1;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = 4 * q + r;
            if (m >= M) continue;
            const int pos = ra.tok_pos[m];
            float y = v[r];
            if (region < 2 && ra.cos_sin != nullptr && p < ra.rotary_dim / 2 && pos >= 0 && pos < ra.n_positions) {
              const float2 c = ra.cos_sin[(size_t)pos * (ra.rotary_dim / 2) + p];
              y = (i & 1) ? other[r] * c.y + v[r] * c.x : v[r] * c.x - other[r] * c.y;
            }
            const bf16 yb = static_cast<bf16>(y);
            if (region == 0) {
              ra.q_out[(size_t)m * Q + n] = yb;
            } else {
              const int slot = ra.seq_slot[m];
              if (slot < 0 || pos < 0) continue;
              const int phys = ra.block_table[(size_t)slot * ra.table_stride + (pos / PAGE) % ra.ring_pages];
              if (phys < 0 || phys >= ra.n_pages) continue;
              const size_t base = ((size_t)phys * ra.n_kv_heads + head) * PAGE * ra.hd;
              const int row = pos & (PAGE - 1);
              if (region == 1)
                ra.k_pages[base + page_k_offset(ra.page_layout, row, i, ra.hd)] = yb;
              else
                ra.v_pages[base + page_v_offset(ra.page_layout, row, i, ra.hd)] = yb;
            }
          }
        }
      }
    }
  }
}

template <int EPI>
int launch_norm(const float* X, const float* norm_w, float eps, const bf16* W, void* C, int M, int N, int K, int H,
           const RopeArgs& ra, hipStream_t stream) {
  bool wide = gated(EPI) || N >= 16384;
  size_t lds = (size_t)M * (K + 8) * sizeof(bf16);
  if (wide)
    gemm_norm_kernel<4, 4, EPI><<<ceil_div(N, 64), 4 * WAVE, lds, stream>>>(X, norm_w, eps, W, C, M, N, K, H, ra);
  else
    gemm_norm_kernel<1, 8, (gated(EPI) ? EPI_F32 : EPI)><<<ceil_div(N, 16), 8 * WAVE, lds, stream>>>(
        X, norm_w, eps, W, C, M, N, K, H, ra);
  return launch_status();
}

bool shape_ok(const void* X, const void* norm_w, const void* W, int M, int N, int K) {
  return M >= 1 && M <= MAX_ROWS && N > 0 && K > 0 && K % 8 == 0 && (size_t)M * (K + 8) * sizeof(bf16) <= 72 * 1024 &&
         !((uintptr_t)X & 15) && !((uintptr_t)norm_w & 15) && !((uintptr_t)W & 15);
}
}  // namespace

extern "C" int yalm_gemm_norm(const float* x, const float* norm_w, float eps, const void* W, void* C, int M, int N,
                              int K, int epilogue, int H, hipStream_t stream) {
  if (!shape_ok(x, norm_w, W, M, N, K)) return YALM_ERR_ARG;
  RopeArgs ra = {};
  if (epilogue == EPI_F32) return launch_norm<EPI_F32>(x, norm_w, eps, (const bf16*)W, C, M, N, K, H, ra, stream);
  if (gated(epilogue)) {
    if (H <= 0 || N != 32 * ((H + 15) / 16)) return YALM_ERR_ARG;
    if (epilogue == EPI_GATED_GELU)
      return launch_norm<EPI_GATED_GELU>(x, norm_w, eps, (const bf16*)W, C, M, N, K, H, ra, stream);
    return launch_norm<EPI_GATED>(x, norm_w, eps, (const bf16*)W, C, M, N, K, H, ra, stream);
  }
  return YALM_ERR_ARG;
}

extern "C" int yalm_gemm_norm_qkv_rope(const float* x, const float* norm_w, float eps, const void* Wqkv, void* q_out,
                                       void* k_pages, void* v_pages, const int* block_table, int table_stride,
                                       int ring_pages, const int* tok_pos, const int* seq_slot, const float* cos_sin,
                                       int n_positions, int M, int K, int n_heads, int n_kv_heads, int head_dim,
                                       int rotary_dim, int n_pages, int page_layout, hipStream_t stream) {
  const int N = (n_heads + 2 * n_kv_heads) * head_dim;
  if (!shape_ok(x, norm_w, Wqkv, M, N, K)) return YALM_ERR_ARG;
  if (head_dim <= 0 || head_dim % 16 != 0 || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > head_dim ||
      n_heads <= 0 || n_kv_heads <= 0 || ring_pages <= 0 || n_pages <= 0 || !page_layout_ok(page_layout, head_dim))
    return YALM_ERR_ARG;
  RopeArgs ra;
  ra.q_out = (bf16*)q_out;
  ra.k_pages = (bf16*)k_pages;
  ra.v_pages = (bf16*)v_pages;
  ra.block_table = block_table;
  ra.tok_pos = tok_pos;
  ra.seq_slot = seq_slot;
  ra.cos_sin = (const float2*)cos_sin;
  ra.table_stride = table_stride;
  ra.ring_pages = ring_pages;
  ra.n_positions = n_positions;
  ra.n_heads = n_heads;
  ra.n_kv_heads = n_kv_heads;
  ra.hd = head_dim;
  ra.rotary_dim = rotary_dim;
  ra.n_pages = n_pages;
  ra.page_layout = page_layout;
  return launch_norm<EPI_ROPE>(x, norm_w, eps, (const bf16*)Wqkv, nullptr, M, N, K, 0, ra, stream);
}

// ---------------------------------------------------------------------------
// chained decode GEMMs (skinny_gemm.h): bfloat16 activations that a producer emitted
// already multiplied by the norm weights, scaled here per row; and the producer side
// ---------------------------------------------------------------------------
extern "C" int yalm_gemm_chain(const void* X, const void* W, void* C, int M, int N, int K, int epilogue, int H,
                               const float* ss_in, int n_parts_in, float eps, const float* emit_nw, void* emit_xn,
                               float* emit_ss, hipStream_t stream) {
  if (M < 1 || M > 64 || N <= 0 || K <= 0 || K % 8 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)W & 15))
    return YALM_ERR_ARG;
  if (ss_in != nullptr && n_parts_in <= 0) return YALM_ERR_ARG;
  ChainArgs ca = {};
  ca.ss_in = ss_in;
  ca.n_parts_in = n_parts_in;
  ca.eps = eps;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  if (epilogue == EPI_ADD) {
    if (emit_nw != nullptr) {
      if (emit_xn == nullptr || emit_ss == nullptr || N >= 16384) return YALM_ERR_ARG;
      ca.emit_nw = emit_nw;
      ca.emit_xn = (bf16*)emit_xn;
      ca.emit_ss = emit_ss;
    }
    return skinny::launch<EPI_ADD>(x, w, C, M, N, K, H, ca, stream);
  }
  if (emit_nw != nullptr) return YALM_ERR_ARG;
  if (epilogue == EPI_F32) return skinny::launch<EPI_F32>(x, w, C, M, N, K, H, ca, stream);
  if (gated(epilogue)) {
    if (H <= 0 || N != 32 * ((H + 15) / 16)) return YALM_ERR_ARG;
    if (epilogue == EPI_GATED_GELU) return skinny::launch<EPI_GATED_GELU>(x, w, C, M, N, K, H, ca, stream);
    return skinny::launch<EPI_GATED>(x, w, C, M, N, K, H, ca, stream);
  }
  return YALM_ERR_ARG;
}

extern "C" int yalm_gemm_chain_qkv_rope(const void* X, const float* ss_in, int n_parts_in, float eps,
                                        const void* Wqkv, void* q_out, void* k_pages, void* v_pages,
                                        const int* block_table, int table_stride, int ring_pages,
                                        const int* tok_pos, const int* seq_slot, const float* cos_sin,
                                        int n_positions, int M, int K, int n_heads, int n_kv_heads, int head_dim,
                                        int rotary_dim, int n_pages, int page_layout, hipStream_t stream) {
  const int N = (n_heads + 2 * n_kv_heads) * head_dim;
  if (M < 1 || M > 64 || K <= 0 || K % 8 != 0 || ((uintptr_t)X & 15) || ((uintptr_t)Wqkv & 15) || ss_in == nullptr ||
      n_parts_in <= 0 || block_table == nullptr || tok_pos == nullptr || seq_slot == nullptr)
    return YALM_ERR_ARG;
  if (head_dim <= 0 || head_dim % 16 != 0 || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > head_dim ||
      n_heads <= 0 || n_kv_heads <= 0 || ring_pages <= 0 || n_pages <= 0 || !page_layout_ok(page_layout, head_dim))
    return YALM_ERR_ARG;
  ChainArgs ca = {};
  ca.ss_in = ss_in;
  ca.n_parts_in = n_parts_in;
  ca.eps = eps;
  RopeArgs& ra = ca.ra;
  ra.q_out = (bf16*)q_out;
  ra.k_pages = (bf16*)k_pages;
  ra.v_pages = (bf16*)v_pages;
  ra.block_table = block_table;
  ra.tok_pos = tok_pos;
  ra.seq_slot = seq_slot;
  ra.cos_sin = (const float2*)cos_sin;
  ra.table_stride = table_stride;
  ra.ring_pages = ring_pages;
  ra.n_positions = n_positions;
  ra.n_heads = n_heads;
  ra.n_kv_heads = n_kv_heads;
  ra.hd = head_dim;
  ra.rotary_dim = rotary_dim;
  ra.n_pages = n_pages;
  ra.page_layout = page_layout;
  return skinny::launch<EPI_ROPE>((const bf16*)X, (const bf16*)Wqkv, nullptr, M, N, K, 0, ca, stream);
}

extern "C" int yalm_gemm_chain_parts(int N) { return skinny::parts_of(N); }
