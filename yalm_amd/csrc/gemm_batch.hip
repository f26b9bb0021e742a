// Decode GEMM for 17..64 rows (to 128 with K a multiple of 64), bfloat16: C = epilogue(X[M,K] * W[N,K]^T).
//
// With more than 16 rows the activations outweigh a workgroup's share of the weights,
// so reading them once per 16 weight rows (as gemm_skinny does) makes the first-level cache,
// not HBM, the limit.  Here K is split across workgroups and N across the waves of a
// workgroup: every wave owns 16 (32 for the gated epilogue) weight rows, and the workgroup's
// chunk of the activations goes through LDS once and all waves read it from there.  Two
// kernels: with K a multiple of 64 both operands are staged in LDS by DMA (2 or 4 waves, see
// gemm_batch_dma_kernel); else the activations go through registers into LDS and the weights
// straight to registers, prefetched one chunk ahead (8 waves).  Each K slice writes its
// float32 partial product; a second kernel adds the slices in a fixed order and applies the
// epilogue (one slice: the first kernel applies it itself).
#include "common.h"
#include "yalm_hip.h"

int yalm_gemm_bf16_dma_partial(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N,
                               int K, int* slices_out, int residual, hipStream_t stream);   // gemm_dma.hip

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// The norm chain for more than 16 rows: the activations came as bfloat16(x * w_norm) from a producer that also left
// partial sums of squares of every row (yalm_gemm_add_emit); the sums of this product are scaled by
// rsqrt(sum(ss[m, :]) / K + eps) per row before they are stored (as slices or through the epilogue: the scale is the
// same for every slice of a row, so the sum of the scaled slices is the scaled sum).  ss null: no scale.
struct RowScale {
  const float* ss;                               // [M][n_parts]
  int n_parts;
  float eps;
};

// A thread per row adds the row's parts (row_sum: asked for BEFORE the first stages of the operands, so that waiting
// for it does not mean waiting for them: loads return in order) and leaves the scale in LDS; the epilogue reads it
// from there.  The workgroups have at least 16 * MT threads.
__device__ __forceinline__ float row_sum(const RowScale& rs, int M, int rows) {
  float t = 0.f;
  if (rs.ss != nullptr && (int)threadIdx.x < rows && (int)threadIdx.x < M) {
    const float* p = rs.ss + (size_t)threadIdx.x * rs.n_parts;
    int i = 0;
    for (; i + 4 <= rs.n_parts; i += 4) {
      const float a = p[i], b = p[i + 1], c = p[i + 2], d = p[i + 3];
      t += a; t += b; t += c; t += d;
    }
    for (; i < rs.n_parts; ++i) t += p[i];
  }
  return t;
}
__device__ __forceinline__ void row_scale_store(const RowScale& rs, float sum, int K, int rows, float* sm_scale) {
  if (rs.ss != nullptr && (int)threadIdx.x < rows) sm_scale[threadIdx.x] = 1.0f / sqrtf(sum / (float)K + rs.eps);
}
template <int MT, int NTW>
__device__ __forceinline__ void row_scales_apply(const RowScale& rs, const float* sm_scale, int q, f32x4 (&acc)[MT][NTW]) {
  if (rs.ss == nullptr) return;
  __syncthreads();
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sc = sm_scale[mt * 16 + 4 * q + r];
#pragma unroll
      for (int t = 0; t < NTW; ++t) acc[mt][t][r] *= sc;
    }
}

constexpr int NWAVES = 8;
constexpr int KC = 128;                          // k per chunk
constexpr int XROW = KC + 8;                     // LDS row stride (elements): 16 bytes of padding

__device__ __forceinline__ bf16x8 load8(const bf16* p, bool ok) {
  bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? *reinterpret_cast<const bf16x8*>(p) : z;
}

// epilogue codes as in yalm_gemm: 0 float32 store, 1 bfloat16 store, 2 float32 add, 3 and 5 gated
template <int EPI>
__device__ __forceinline__ void store_tile(void* Cv, const f32x4& v, const f32x4& u, int m_base, int n, int hcol,
                                           int M, int N, int H) {
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int m = m_base + r;
    if (m >= M) continue;
    if (gated(EPI)) {
      if (hcol < H) ((bf16*)Cv)[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(v[r]) * u[r]);
    } else if (n < N) {
      size_t o = (size_t)m * N + n;
      if (EPI == 0) ((float*)Cv)[o] = v[r];
      if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(v[r]);
      if (EPI == 2) ((float*)Cv)[o] += v[r];
    }
  }
}

// grid (row blocks of 128 * NTW weight rows, K slices).  partial: [slices][M][N] float32 when slices > 1.
template <int MT, int NTW, int EPI>
__global__ __launch_bounds__(NWAVES * WAVE) void gemm_batch_kernel(const bf16* __restrict__ X,
                                                                    const bf16* __restrict__ W,
                                                                    void* __restrict__ Cv,
                                                                    float* __restrict__ partial, int M, int N, int K,
                                                                    int H, int k_per_slice, int always_partial,
                                                                    RowScale rs) {
  __shared__ __attribute__((aligned(16))) bf16 xs[2][MT * 16 * XROW];
  constexpr int NTHREADS = NWAVES * WAVE;
  constexpr int XCHUNKS = MT * 16 * (KC / 8);    // 16-byte pieces of an activation chunk
  constexpr int XPT = (XCHUNKS + NTHREADS - 1) / NTHREADS;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int q = lane / 16, j = lane % 16;
  const int n0 = (blockIdx.x * NWAVES + wave) * 16 * NTW;
  const int k_begin = blockIdx.y * k_per_slice, k_end = min(K, k_begin + k_per_slice);

  const bf16* wrow[NTW];
  bool wok[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) {
    int n = n0 + t * 16 + j;
    wok[t] = n < N;
    wrow[t] = W + (size_t)(wok[t] ? n : 0) * K;
  }
  f32x4 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) acc[mt][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  bf16x8 wv[NTW][4], xr[XPT];
  auto load_w = [&](int kc, bf16x8 (&dst)[NTW][4]) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      int k = kc + s * 32 + q * 8;
      bool ok = k < k_end;
#pragma unroll
      for (int t = 0; t < NTW; ++t) dst[t][s] = load8(wrow[t] + k, ok && wok[t]);
    }
  };
  auto load_x = [&](int kc) {
#pragma unroll
    for (int p = 0; p < XPT; ++p) {
      int c = tid + p * NTHREADS;
      int row = c / (KC / 8), k = kc + (c % (KC / 8)) * 8;
      xr[p] = load8(X + (size_t)min(row, M - 1) * K + k, c < XCHUNKS && row < M && k < k_end);
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int p = 0; p < XPT; ++p) {
      int c = tid + p * NTHREADS;
      if (c < XCHUNKS) *reinterpret_cast<bf16x8*>(&xs[buf][(c / (KC / 8)) * XROW + (c % (KC / 8)) * 8]) = xr[p];
    }
  };

  __shared__ float sm_scale[MT * 16];
  static_assert(NTHREADS >= MT * 16, "a thread per batch row");
  row_scale_store(rs, row_sum(rs, M, MT * 16), K, MT * 16, sm_scale);
  if (k_begin < k_end) {
    load_w(k_begin, wv);
    load_x(k_begin);
    store_x(0);
  }
  __syncthreads();
  int it = 0;
  for (int kc = k_begin; kc < k_end; kc += KC, ++it) {
    const int cur = it & 1;
    const int kn = kc + KC;
    bf16x8 wn[NTW][4];
    if (kn < k_end) {
      load_w(kn, wn);
      load_x(kn);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 xf = *reinterpret_cast<const bf16x8*>(&xs[cur][(mt * 16 + j) * XROW + s * 32 + q * 8]);
#pragma unroll
        for (int t = 0; t < NTW; ++t)
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wv[t][s], acc[mt][t], 0, 0, 0);
      }
    if (kn < k_end) {
      store_x(cur ^ 1);
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < NTW; ++t) wv[t][s] = wn[t][s];
    }
    __syncthreads();
  }

  // C[m][n]: lane (q, j) holds rows 4q..4q+3 of column j of every tile
  row_scales_apply<MT, NTW>(rs, sm_scale, q, acc);
  if (gridDim.y == 1 && !always_partial) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (gated(EPI)) {
        store_tile<EPI>(Cv, acc[mt][0], acc[mt][NTW - 1], mt * 16 + 4 * q, 0, n0 / 2 + j, M, N, H);
      } else {
#pragma unroll
        for (int t = 0; t < NTW; ++t)
          store_tile<EPI>(Cv, acc[mt][t], acc[mt][t], mt * 16 + 4 * q, n0 + t * 16 + j, 0, M, N, H);
      }
    }
  } else {
    float* part = partial + (size_t)blockIdx.y * M * N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        int n = n0 + t * 16 + j;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int m = mt * 16 + 4 * q + r;
          if (m < M && n < N) part[(size_t)m * N + n] = acc[mt][t][r];
        }
      }
  }
}

template <int N_>
__device__ __forceinline__ void wait_vmcnt() {   // vmcnt only: expcnt and lgkmcnt fields at their maxima
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// The same product with both operands going from global memory straight into LDS
// (global_load_lds_dwordx4), for K and K slices that are multiples of 64: a stage is 64 k, every wave
// keeps a ring of S stages of its own weight rows, and the workgroup one ring of the activations, of
// which every wave fetches 8 rows.  Every request to the second-level cache is a whole 128-byte line
// (8 lanes a row), where the register path's lanes ask for 64-byte pieces and a CU's requests a clock
// are what limits it; the 16-byte chunks of a row are XOR-swizzled by the row number in the global
// address, so that the fragment reads of 8 rows fall on different banks.  One bare s_barrier a
// stage: after it everyone's part of the stage's activations is there and everyone has read the
// stage before.
template <int MT, int NTW, int EPI, int S, int NW>
__global__ __launch_bounds__(NW * WAVE) void gemm_batch_dma_kernel(const bf16* __restrict__ X,
                                                                        const bf16* __restrict__ W,
                                                                        void* __restrict__ Cv,
                                                                        float* __restrict__ partial, int M, int N,
                                                                        int K, int H, int k_per_slice,
                                                                        int always_partial, RowScale rs) {
  constexpr int KD = 64;
  constexpr int WSTAGE = NTW * 2048;             // a wave's weight rows of a stage
  constexpr int XG0 = MT <= 2 ? 4 : (MT <= 4 ? 8 : 16);  // DMA instructions for the activations: 8 rows each, 32, 64 or
  constexpr int XG = XG0 < NW ? NW : XG0;        // 128 rows (and at least one instruction a wave)
  static_assert(XG % NW == 0, "the activations' instructions divide over the waves");
  constexpr int XSTAGE = XG * 1024;
  constexpr int XI = XG / NW;                    // of which every wave issues this many
  constexpr int L = 2 * NTW + XI;                // DMA instructions a wave and stage
  static_assert(S >= 3 && S <= 4, "3 or 4 stages");
  extern __shared__ __attribute__((aligned(1024))) unsigned char ring[];   // [NW][S][WSTAGE], then [S][XSTAGE]
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int q = lane / 16, j = lane % 16;
  unsigned char* wring = ring + (size_t)wave * S * WSTAGE;
  unsigned char* xring = ring + (size_t)NW * S * WSTAGE;
  const int n0 = (blockIdx.x * NW + wave) * 16 * NTW;
  const int k_begin = blockIdx.y * k_per_slice, k_end = min(K, k_begin + k_per_slice);
  const int n_st = max(0, k_end - k_begin) / KD;

  const int r8 = lane / 8, chunk = (lane % 8) ^ r8;   // this lane's row of an instruction and the chunk it asks for
  const bf16* gw[2 * NTW];
#pragma unroll
  for (int u = 0; u < 2 * NTW; ++u)
    gw[u] = W + (size_t)min(n0 + (u / 2) * 16 + (u % 2) * 8 + r8, N - 1) * K + k_begin + chunk * 8;
  const bf16* gx[XI];
#pragma unroll
  for (int u = 0; u < XI; ++u) gx[u] = X + (size_t)min((wave * XI + u) * 8 + r8, M - 1) * K + k_begin + chunk * 8;
  // The workgroups do not walk K from the same end: workgroup b begins at k tile b (mod the slice's tiles) and
  // wraps round.  Rows lie a power of two apart (8 KB at K = 4,096), so workgroups in step would all ask for the
  // same few address bits at a time, and with them for the same memory channels (gate/up at 64 rows: 4.9 TB/s
  // with K = 4,096 against 5.7 with K = 4,160 before this, 6.0 with it).
  int tile = n_st > 0 ? (int)(blockIdx.x % (unsigned)n_st) : 0;
  auto issue = [&](int buf) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass drops a template that names this builtin, and its launch stub with it
#pragma unroll
    for (int u = 0; u < 2 * NTW; ++u)
      __builtin_amdgcn_global_load_lds(gw[u] + (size_t)tile * KD, wring + buf * WSTAGE + u * 1024, 16, 0, YALM_READ_ONCE);
#pragma unroll
    for (int u = 0; u < XI; ++u)
      __builtin_amdgcn_global_load_lds(gx[u] + (size_t)tile * KD, xring + buf * XSTAGE + (wave * XI + u) * 1024, 16, 0, 0);
#endif
    if (++tile == n_st) tile = 0;
  };

  f32x4 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) acc[mt][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  __shared__ float sm_scale[MT * 16];
  static_assert(NW * WAVE >= MT * 16, "a thread per batch row");
  const float rsum = row_sum(rs, M, MT * 16);
#pragma unroll
  for (int i = 0; i < S - 1; ++i)
    if (i < n_st) issue(i);
  row_scale_store(rs, rsum, K, MT * 16, sm_scale);
  // fragment reads: lane (q, j) of step s wants chunk 4 s + q of row j, which lies at (4 s + q) ^ (j & 7)
  const int rd = j * 128, swz = j & 7;
  int buf = 0;
  for (int i = 0; i < n_st; ++i) {
    const int ahead = n_st - 1 - i;               // stages behind this one that are in flight
    if (ahead >= S - 2) wait_vmcnt<(S - 2) * L>();
    else if (ahead == 1) wait_vmcnt<L>();
    else wait_vmcnt<0>();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (i + S - 1 < n_st) {
      int nb = buf + S - 1;
      if (nb >= S) nb -= S;
      issue(nb);                                  // into the buffer that everyone read in the round before
    }
    const unsigned char* wcur = wring + buf * WSTAGE;
    const unsigned char* xcur = xring + buf * XSTAGE;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int off = ((4 * s + q) ^ swz) << 4;
      bf16x8 wf[NTW];
#pragma unroll
      for (int t = 0; t < NTW; ++t) wf[t] = *reinterpret_cast<const bf16x8*>(wcur + t * 2048 + rd + off);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 xf = *reinterpret_cast<const bf16x8*>(xcur + mt * 2048 + rd + off);
#pragma unroll
        for (int t = 0; t < NTW; ++t)
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wf[t], acc[mt][t], 0, 0, 0);
      }
    }
    if (++buf == S) buf = 0;
  }

  row_scales_apply<MT, NTW>(rs, sm_scale, q, acc);
  if (gridDim.y == 1 && !always_partial) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (gated(EPI)) {
        store_tile<EPI>(Cv, acc[mt][0], acc[mt][NTW - 1], mt * 16 + 4 * q, 0, n0 / 2 + j, M, N, H);
      } else {
#pragma unroll
        for (int t = 0; t < NTW; ++t)
          store_tile<EPI>(Cv, acc[mt][t], acc[mt][t], mt * 16 + 4 * q, n0 + t * 16 + j, 0, M, N, H);
      }
    }
  } else {
    float* part = partial + (size_t)blockIdx.y * M * N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        int n = n0 + t * 16 + j;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int m = mt * 16 + 4 * q + r;
          if (m < M && n < N) part[(size_t)m * N + n] = acc[mt][t][r];
        }
      }
  }
}

// launches one of the two kernels: the DMA one (NW waves; up to 128 rows) where K and the slices are
// multiples of 64, else the register one (8 waves; up to 64 rows)
template <int MT, int NTW, int EPI, int NW>
int launch_kernel(dim3 grid, const bf16* X, const bf16* W, void* C, float* ws, int M, int N, int K, int H,
                  int k_per_slice, int always_partial, const RowScale& rs, hipStream_t stream) {
  if (K % 64 == 0 && k_per_slice % 64 == 0) {
    constexpr int XG0 = MT <= 2 ? 4 : (MT <= 4 ? 8 : 16);
    constexpr int XG = XG0 < NW ? NW : XG0;
    constexpr int S = (NW * NTW <= 8 && XG <= 8) || (NW * NTW <= 4) ? 4 : 3;
    constexpr size_t lds = (size_t)NW * S * NTW * 2048 + (size_t)S * XG * 1024;
    static_assert(lds <= 128 * 1024, "the rings fit the LDS of a CU");
    auto kernel = &gemm_batch_dma_kernel<MT, NTW, EPI, S, NW>;
    static LdsAllowance allowed;                   // more than 64 KB of LDS has to be asked for once a device
    if (int rc = allow_dynamic_lds(allowed, (const void*)kernel, (int)lds); rc != YALM_OK) return rc;
    kernel<<<grid, NW * WAVE, lds, stream>>>(X, W, C, ws, M, N, K, H, k_per_slice, always_partial, rs);
    return launch_status();
  }
  if constexpr (MT <= 4 && NW == NWAVES) {
    gemm_batch_kernel<MT, NTW, EPI><<<grid, NWAVES * WAVE, 0, stream>>>(X, W, C, ws, M, N, K, H, k_per_slice,
                                                                        always_partial, rs);
    return launch_status();
  }
  return YALM_ERR_ARG;
}

// adds the K slices in order and applies the epilogue; a thread per (row, 4 columns)
template <int EPI>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ Cv, int M, int N, int H,
                                     int slices) {
  const int cols4 = (gated(EPI)) ? (N / 2) / 4 : (N + 3) / 4;     // gated: N = 32 * blocks, a thread per 4 hidden columns
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)M * cols4) return;
  const int m = (int)(idx / cols4), c4 = (int)(idx % cols4) * 4;
  const size_t plane = (size_t)M * N;
  if (gated(EPI)) {
    const int blk = c4 / 16, off = c4 % 16;      // hidden column c4 = blk * 16 + off; gate at blk*32+off, up 16 further
    const float* pg = partial + (size_t)m * N + blk * 32 + off;
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f), u = g;
    for (int s = 0; s < slices; ++s) {
      const float4 a = *reinterpret_cast<const float4*>(pg + s * plane);
      const float4 b = *reinterpret_cast<const float4*>(pg + s * plane + 16);
      g.x += a.x; g.y += a.y; g.z += a.z; g.w += a.w;
      u.x += b.x; u.y += b.y; u.z += b.z; u.w += b.w;
    }
    bf16* C = (bf16*)Cv + (size_t)m * H;
    const float gv[4] = {g.x, g.y, g.z, g.w}, uv[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (c4 + e < H) C[c4 + e] = static_cast<bf16>(gate_act<EPI>(gv[e]) * uv[e]);
  } else {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    const float* p = partial + (size_t)m * N + c4;
    if (c4 + 3 < N && (N & 3) == 0) {
      for (int s = 0; s < slices; ++s) {
        const float4 a = *reinterpret_cast<const float4*>(p + s * plane);
        v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w;
      }
    } else {
      for (int s = 0; s < slices; ++s)
        for (int e = 0; e < 4; ++e)
          if (c4 + e < N) v[e] += p[s * plane + e];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (c4 + e >= N) continue;
      size_t o = (size_t)m * N + c4 + e;
      if (EPI == 0) ((float*)Cv)[o] = v[e];
      if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(v[e]);
      if (EPI == 2) ((float*)Cv)[o] += v[e];
    }
  }
}

// K slices wanted for n_blocks row blocks: until every CU has a workgroup, while the partial sums stay small
// beside the weights (slices * M * N * 4 bytes against N * K * 2) and a slice keeps at least 2 chunks
int wanted_slices(int n_blocks, int M, int K) {
  const int chunks = ceil_div(K, KC);
  int slices = 1;
  // more than 64 rows: a workgroup's rings fill the LDS of a CU, so that workgroups beyond one a CU wait for a
  // second round; 192 workgroups in one round beat 384 in two (batch 96 / 128: +0.7 %)
  const int target = M > 64 ? 130 : 200;
  while (n_blocks * slices < target && slices * 2 <= K / (8 * M) && slices * 2 <= chunks / 2 && slices < 16)
    slices *= 2;
  return slices;
}
// k a slice covers (whole chunks), and how many slices that makes
void slice_k(int K, int wanted, int* k_per_slice, int* slices) {
  *k_per_slice = ceil_div(ceil_div(K, KC), wanted) * KC;
  *slices = ceil_div(K, *k_per_slice);
}

template <int MT, int EPI, int NW, int NTW_ = 0>
int launch_nw(const bf16* X, const bf16* W, void* C, float* ws, long ws_floats, int M, int N, int K, int H,
              const RowScale& rs, hipStream_t stream) {
  constexpr int NTW = NTW_ ? NTW_ : (gated(EPI) ? 2 : 1);
  if constexpr (NTW_ == 0 && !gated(EPI) && MT <= 4 && NW <= 4) {
    // a matrix with rows enough (the head): workgroups of 128 rows fill the chip by themselves, K unsplit
    if (K % 64 == 0 && ceil_div(N, NW * 32) >= 200)
      return launch_nw<MT, EPI, NW, 2>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
  }
  const int rows_per_wg = NW * 16 * NTW;
  const int n_blocks = ceil_div(N, rows_per_wg);
  int slices = wanted_slices(n_blocks, M, K), k_per_slice;
  if (ws == nullptr || (long)slices * M * N > ws_floats) slices = 1;
  slice_k(K, slices, &k_per_slice, &slices);
  dim3 grid(n_blocks, slices);
  int rc = launch_kernel<MT, NTW, EPI, NW>(grid, X, W, C, ws, M, N, K, H, k_per_slice, 0, rs, stream);
  if (rc != YALM_OK || slices == 1) return rc;
  const long items = (long)M * (gated(EPI) ? (N / 2) / 4 : (N + 3) / 4);
  splitk_reduce_kernel<EPI><<<ceil_div(items, 256), 256, 0, stream>>>(ws, C, M, N, H, slices);
  return launch_status();
}

template <int MT, int EPI>
int launch_mt(const bf16* X, const bf16* W, void* C, float* ws, long ws_floats, int M, int N, int K, int H,
              const RowScale& rs, hipStream_t stream) {
  // waves a workgroup of the DMA kernel (they share the activations' stage): measured at batch 64
  // 8 waves 8120, 4 waves 8580, 2 waves 8410 tokens a second; at batch 32 5490, 5740 and 5870; with more than 64
  // rows 8 waves where their rings fit (not the gated product's): batch 96 8,950 -> 9,060, batch 128 9,540 -> 9,590
  constexpr int NW = MT <= 2 ? 2 : (MT > 4 && !gated(EPI) ? 8 : 4);
  if (K % 64 == 0) return launch_nw<MT, EPI, NW>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
  if constexpr (MT > 4) return YALM_ERR_ARG;
  else return launch_nw<MT, EPI, 8>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
}

// The residual add that also does the NEXT RMSNorm: a workgroup per row adds the K slices to
// the float32 residual stream, sums the squares of the new row, and writes the normalised
// activations h = bfloat16(x * rsqrt(mean(x^2) + eps) * w).  No norm kernel runs afterwards.
constexpr int RN_THREADS = 1024;
__global__ __launch_bounds__(RN_THREADS) void reduce_add_norm_kernel(const float* __restrict__ partial,
                                                                     float* __restrict__ C,
                                                                     const float* __restrict__ norm_w, float eps,
                                                                     bf16* __restrict__ h, int M, int N, int slices) {
  __shared__ float red[RN_THREADS / WAVE];
  const int m = blockIdx.x;
  const size_t plane = (size_t)M * N;
  float* row = C + (size_t)m * N;
  const float* prow = partial + (size_t)m * N;
  float ss = 0.f;
  if ((N & 3) == 0) {                             // four columns a thread, the slices' loads four at a time
    for (int c = threadIdx.x * 4; c < N; c += RN_THREADS * 4) {
      float4 y = *reinterpret_cast<const float4*>(row + c);
      int s = 0;
      for (; s + 4 <= slices; s += 4) {
        float4 p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) p[u] = *reinterpret_cast<const float4*>(prow + (size_t)(s + u) * plane + c);
#pragma unroll
        for (int u = 0; u < 4; ++u) {             // added in the order of the slices
          y.x += p[u].x; y.y += p[u].y; y.z += p[u].z; y.w += p[u].w;
        }
      }
      for (; s < slices; ++s) {
        const float4 p = *reinterpret_cast<const float4*>(prow + (size_t)s * plane + c);
        y.x += p.x; y.y += p.y; y.z += p.z; y.w += p.w;
      }
      *reinterpret_cast<float4*>(row + c) = y;
      ss += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
    }
  } else {
    for (int c = threadIdx.x; c < N; c += RN_THREADS) {
      float y = row[c];
      for (int s = 0; s < slices; ++s) y += prow[(size_t)s * plane + c];
      row[c] = y;
      ss += y * y;
    }
  }
  ss = block_sum<RN_THREADS / WAVE>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)N + eps);
  // every thread reads back what it wrote itself
  if ((N & 3) == 0) {
    for (int c = threadIdx.x * 4; c < N; c += RN_THREADS * 4) {
      const float4 y = *reinterpret_cast<const float4*>(row + c);
      const float4 w = *reinterpret_cast<const float4*>(norm_w + c);
      typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
      bf16x4 o = {static_cast<bf16>(y.x * scale * w.x), static_cast<bf16>(y.y * scale * w.y),
                  static_cast<bf16>(y.z * scale * w.z), static_cast<bf16>(y.w * scale * w.w)};
      *reinterpret_cast<bf16x4*>(h + (size_t)m * N + c) = o;
    }
  } else {
    for (int c = threadIdx.x; c < N; c += RN_THREADS)
      h[(size_t)m * N + c] = static_cast<bf16>(row[c] * scale * norm_w[c]);
  }
}

// Workgroups of 32 weight rows a wave instead of 16 (twice the rows for the same stage of activations): what a CU
// takes in is bounded (about 37 GB/s, whether the bytes come from memory or from the second-level cache), so the
// activations' share is taken from the weights'; at 64 batch rows a workgroup of 64 weight rows spends half of it on
// activations, one of 128 a third.  Such a workgroup's rings allow one workgroup a CU, so K is cut into as many slices
// as bring the launch to at most 256 workgroups, and a slice must stay long enough to be worth its start (12 stages).
// Measured at 64 rows of the 7B shape: down projection 31.4 -> 27.9 us, q/k/v 16.0 -> 12.7 (5 slices of 13 stages);
// the output projection (8 slices of 8 stages) 15.3 -> 16.5, which the rule leaves out.  Returns the slices, 0: no.
int wide_slices(int n_blocks_wide, int K) {
  int s = 256 / (n_blocks_wide > 0 ? n_blocks_wide : 1);
  if (s > 16) s = 16;
  if (s < 1 || n_blocks_wide * s < 192 || K % 64 != 0 || K / s < 768) return 0;
  return s;
}

// The same with a row's columns kept in registers between the two halves (N a multiple of 4, at most
// THREADS * VPT * 4): the new row is written and never read again, and the norm's weights are asked for before the
// sum of squares is known.  64 rows of 4,096 columns: 4.85 -> see the launcher.
template <int THREADS, int VPT>
__global__ __launch_bounds__(THREADS) void reduce_add_norm_reg_kernel(const float* __restrict__ partial,
                                                                      float* __restrict__ C,
                                                                      const float* __restrict__ norm_w, float eps,
                                                                      bf16* __restrict__ h, int M, int N, int slices) {
  __shared__ float red[THREADS / WAVE];
  const int m = blockIdx.x;
  const size_t plane = (size_t)M * N;
  float* row = C + (size_t)m * N;
  const float* prow = partial + (size_t)m * N;
  float4 y[VPT], w[VPT];
  int col[VPT];
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    col[v] = (threadIdx.x + v * THREADS) * 4;
    const bool ok = col[v] < N;
    const int c = ok ? col[v] : 0;                  // every lane loads (a load under a branch holds up the others)
    y[v] = *reinterpret_cast<const float4*>(row + c);
    w[v] = *reinterpret_cast<const float4*>(norm_w + c);
  }
  int s = 0;
  for (; s + 4 <= slices; s += 4) {
    float4 p[4][VPT];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int v = 0; v < VPT; ++v)
        p[u][v] = *reinterpret_cast<const float4*>(prow + (size_t)(s + u) * plane + (col[v] < N ? col[v] : 0));
#pragma unroll
    for (int u = 0; u < 4; ++u)                     // added in the order of the slices
#pragma unroll
      for (int v = 0; v < VPT; ++v) {
        y[v].x += p[u][v].x; y[v].y += p[u][v].y; y[v].z += p[u][v].z; y[v].w += p[u][v].w;
      }
  }
  for (; s < slices; ++s) {
    float4 p[VPT];
#pragma unroll
    for (int v = 0; v < VPT; ++v)
      p[v] = *reinterpret_cast<const float4*>(prow + (size_t)s * plane + (col[v] < N ? col[v] : 0));
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
      y[v].x += p[v].x; y[v].y += p[v].y; y[v].z += p[v].z; y[v].w += p[v].w;
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v)
    if (col[v] < N) {
      *reinterpret_cast<float4*>(row + col[v]) = y[v];
      ss += y[v].x * y[v].x + y[v].y * y[v].y + y[v].z * y[v].z + y[v].w * y[v].w;
    }
  ss = block_sum<THREADS / WAVE>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)N + eps);
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
#pragma unroll
  for (int v = 0; v < VPT; ++v)
    if (col[v] < N) {
      bf16x4 o = {static_cast<bf16>(y[v].x * scale * w[v].x), static_cast<bf16>(y[v].y * scale * w[v].y),
                  static_cast<bf16>(y[v].z * scale * w[v].z), static_cast<bf16>(y[v].w * scale * w[v].w)};
      *reinterpret_cast<bf16x4*>(h + (size_t)m * N + col[v]) = o;
    }
}

// The residual add that prepares the next norm without waiting for it: a workgroup takes EMIT_COLS columns of a row,
// adds the K slices to the residual stream, and writes xn = bfloat16(x_new * norm_w) and the sum of the squares of its
// columns, ss[row][part].  The consumer scales its sums by rsqrt(sum(ss[row, :]) / N + eps) (RowScale).  No workgroup
// waits for a whole row, so a batch of 64 rows is 256 small workgroups instead of 64 that each walk a row twice.
constexpr int EMIT_THREADS = 256, EMIT_COLS = EMIT_THREADS * 4;
__global__ __launch_bounds__(EMIT_THREADS) void reduce_add_emit_kernel(const float* __restrict__ partial,
                                                                       float* __restrict__ C,
                                                                       const float* __restrict__ norm_w,
                                                                       bf16* __restrict__ xn, float* __restrict__ ss_out,
                                                                       int M, int N, int slices) {
  __shared__ float red[EMIT_THREADS / WAVE];
  const int m = blockIdx.x, part = blockIdx.y, n_parts = gridDim.y;
  const size_t plane = (size_t)M * N;
  const int c = part * EMIT_COLS + threadIdx.x * 4;
  float ss = 0.f;
  {                                               // N is a multiple of 8 (the launcher sees to it)
    const bool ok = c < N;
    const int cc = ok ? c : 0;
    float* row = C + (size_t)m * N + cc;
    const float* prow = partial + (size_t)m * N + cc;
    float4 y = *reinterpret_cast<const float4*>(row);
    const float4 w = *reinterpret_cast<const float4*>(norm_w + cc);
    int s = 0;
    for (; s + 4 <= slices; s += 4) {
      float4 p[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) p[u] = *reinterpret_cast<const float4*>(prow + (size_t)(s + u) * plane);
#pragma unroll
      for (int u = 0; u < 4; ++u) {                // added in the order of the slices
        y.x += p[u].x; y.y += p[u].y; y.z += p[u].z; y.w += p[u].w;
      }
    }
    for (; s < slices; ++s) {
      const float4 p = *reinterpret_cast<const float4*>(prow + (size_t)s * plane);
      y.x += p.x; y.y += p.y; y.z += p.z; y.w += p.w;
    }
    if (ok) {
      *reinterpret_cast<float4*>(row) = y;
      typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
      bf16x4 o = {static_cast<bf16>(y.x * w.x), static_cast<bf16>(y.y * w.y), static_cast<bf16>(y.z * w.z),
                  static_cast<bf16>(y.w * w.w)};
      *reinterpret_cast<bf16x4*>(xn + (size_t)m * N + c) = o;
      ss = y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
    }
  }
  ss = block_sum<EMIT_THREADS / WAVE>(ss, red);
  if (threadIdx.x == 0) ss_out[(size_t)m * n_parts + part] = ss;
}

int emit_parts(int N) { return ceil_div(N, EMIT_COLS); }

// emit_ss null: the new row's norm is finished here (h = its output); else h = bfloat16(x_new * norm_w) and emit_ss
// receives the parts of the rows' sums of squares
int launch_reduce_add_norm(const float* ws, float* C, const float* norm_w, float eps, bf16* h, int M, int N, int slices,
                           hipStream_t stream, float* emit_ss = nullptr) {
  if (emit_ss != nullptr) {
    reduce_add_emit_kernel<<<dim3(M, emit_parts(N)), EMIT_THREADS, 0, stream>>>(ws, C, norm_w, h, emit_ss, M, N, slices);
    return launch_status();
  }
  if ((N & 3) == 0 && N <= 1024 * 4 && !((uintptr_t)norm_w & 15))
    reduce_add_norm_reg_kernel<1024, 1><<<M, 1024, 0, stream>>>(ws, C, norm_w, eps, h, M, N, slices);
  else if ((N & 3) == 0 && N <= 1024 * 4 * 4 && !((uintptr_t)norm_w & 15))
    reduce_add_norm_reg_kernel<1024, 4><<<M, 1024, 0, stream>>>(ws, C, norm_w, eps, h, M, N, slices);
  else
    reduce_add_norm_kernel<<<M, RN_THREADS, 0, stream>>>(ws, C, norm_w, eps, h, M, N, slices);
  return launch_status();
}

template <int MT, int NW, int NTW = 1>
int launch_add_norm_nw(const bf16* X, const bf16* W, float* C, float* ws, long ws_floats, int M, int N, int K,
                       const float* norm_w, float eps, bf16* h, hipStream_t stream, float* emit_ss = nullptr) {
  if constexpr (NTW == 1 && MT <= 4 && NW <= 4) {
    const int wide = wide_slices(ceil_div(N, NW * 32), K);
    if (wide > 0 && ws != nullptr && (long)wide * M * N <= ws_floats)
      return launch_add_norm_nw<MT, NW, 2>(X, W, C, ws, ws_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
  }
  const int n_blocks = ceil_div(N, NW * 16 * NTW);
  int slices = NTW == 2 ? wide_slices(n_blocks, K) : wanted_slices(n_blocks, M, K), k_per_slice;
  while (slices > 1 && (long)slices * M * N > ws_floats) slices /= 2;
  if (ws == nullptr || (long)slices * M * N > ws_floats) return YALM_ERR_ARG;
  slice_k(K, slices, &k_per_slice, &slices);
  dim3 grid(n_blocks, slices);
  int rc = launch_kernel<MT, NTW, 2, NW>(grid, X, W, C, ws, M, N, K, 0, k_per_slice, 1, RowScale{nullptr, 0, 0.f}, stream);
  if (rc != YALM_OK) return rc;
  return launch_reduce_add_norm(ws, C, norm_w, eps, h, M, N, slices, stream, emit_ss);
}

template <int MT>
int launch_add_norm(const bf16* X, const bf16* W, float* C, float* ws, long ws_floats, int M, int N, int K,
                    const float* norm_w, float eps, bf16* h, hipStream_t stream, float* emit_ss = nullptr) {
  if (K % 64 == 0 && MT > 2)
    return launch_add_norm_nw<MT, (MT > 4 ? 8 : 4)>(X, W, C, ws, ws_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
  if constexpr (MT > 4) return YALM_ERR_ARG;
  else return launch_add_norm_nw<MT, NWAVES>(X, W, C, ws, ws_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
}

// the K slices only: [slices][M][N] in ws, for a consumer that adds them
template <int MT, int NW, int NTW = 1>
int launch_partial_nw(const bf16* X, const bf16* W, float* ws, long ws_floats, int M, int N, int K, int* slices_out,
                      const RowScale& rs, hipStream_t stream) {
  if constexpr (NTW == 1 && MT <= 4 && NW <= 4) {
    const int wide = wide_slices(ceil_div(N, NW * 32), K);
    if (wide > 0 && ws != nullptr && (long)wide * M * N <= ws_floats)
      return launch_partial_nw<MT, NW, 2>(X, W, ws, ws_floats, M, N, K, slices_out, rs, stream);
  }
  const int n_blocks = ceil_div(N, NW * 16 * NTW);
  int slices = NTW == 2 ? wide_slices(n_blocks, K) : wanted_slices(n_blocks, M, K), k_per_slice;
  while (slices > 1 && (long)slices * M * N > ws_floats) slices /= 2;
  if (ws == nullptr || (long)slices * M * N > ws_floats) return YALM_ERR_ARG;
  slice_k(K, slices, &k_per_slice, &slices);
  *slices_out = slices;
  dim3 grid(n_blocks, slices);
  return launch_kernel<MT, NTW, 0, NW>(grid, X, W, ws, ws, M, N, K, 0, k_per_slice, 1, rs, stream);
}

template <int MT>
int launch_partial(const bf16* X, const bf16* W, float* ws, long ws_floats, int M, int N, int K, int* slices_out,
                   const RowScale& rs, hipStream_t stream) {
  if (K % 64 == 0)
    return launch_partial_nw<MT, (MT > 4 ? 8 : 4)>(X, W, ws, ws_floats, M, N, K, slices_out, rs, stream);
  if constexpr (MT > 4) return YALM_ERR_ARG;
  else return launch_partial_nw<MT, NWAVES>(X, W, ws, ws_floats, M, N, K, slices_out, rs, stream);
}

template <int EPI>
int dispatch(const bf16* X, const bf16* W, void* C, float* ws, long ws_floats, int M, int N, int K, int H,
             const RowScale& rs, hipStream_t stream) {
  switch ((M + 15) / 16) {
    case 2: return launch_mt<2, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 3: return launch_mt<3, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 4: return launch_mt<4, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 5: return launch_mt<5, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 6: return launch_mt<6, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 7: return launch_mt<7, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
    case 8: return launch_mt<8, EPI>(X, W, C, ws, ws_floats, M, N, K, H, rs, stream);
  }
  return YALM_ERR_ARG;
}
}  // namespace

// 17..64 rows, and up to 128 with K a multiple of 64; workspace: float32 scratch for the K slices (may be
// null: one slice then).  ss (may be null): the producer's partial sums of squares [M][n_parts] for the row scale.
// Refuses (YALM_ERR_ARG) what it does not take.
static int gemm_batch_scaled(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M,
                             int N, int K, int epilogue, int H, const float* ss, int n_parts, float eps,
                             hipStream_t stream) {
  if (M <= 16 || M > (K % 64 == 0 ? 128 : 64) || K % 8 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15))
    return YALM_ERR_ARG;
  if (ss != nullptr && n_parts <= 0) return YALM_ERR_ARG;
  const RowScale rs = {ss, n_parts, eps};
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  switch (epilogue) {
    case 0: return dispatch<0>(a, w, C, workspace, workspace_floats, M, N, K, H, rs, stream);
    case 1: return dispatch<1>(a, w, C, workspace, workspace_floats, M, N, K, H, rs, stream);
    case 2: return dispatch<2>(a, w, C, workspace, workspace_floats, M, N, K, H, rs, stream);
    case 3: return dispatch<3>(a, w, C, workspace, workspace_floats, M, N, K, H, rs, stream);
    case 5: return dispatch<5>(a, w, C, workspace, workspace_floats, M, N, K, H, rs, stream);
  }
  return YALM_ERR_ARG;
}

int yalm_gemm_bf16_batch(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                         int K, int epilogue, int H, hipStream_t stream) {
  return gemm_batch_scaled(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, nullptr, 0, 0.f, stream);
}

// yalm_gemm for 17..128 bfloat16 rows (more than 64: K a multiple of 64) whose activations came from yalm_gemm_add_emit:
// the sums are scaled per row by rsqrt(sum(ss[m, :]) / K + eps).  Refuses (YALM_ERR_ARG) other shapes.
extern "C" int yalm_gemm_scaled(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M,
                                int N, int K, int epilogue, int H, const float* ss, int n_parts, float eps,
                                hipStream_t stream) {
  if (ss == nullptr) return YALM_ERR_ARG;
  if (gated(epilogue) && (H <= 0 || N != 32 * ((H + 15) / 16))) return YALM_ERR_ARG;
  return gemm_batch_scaled(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, ss, n_parts, eps, stream);
}

static int gemm_partial_scaled(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N,
                               int K, int* slices, const float* ss, int n_parts, float eps, hipStream_t stream) {
  if (M <= 16 || M > (K % 64 == 0 ? 128 : 64) || K % 8 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15) ||
      slices == nullptr || (ss != nullptr && n_parts <= 0))
    return YALM_ERR_ARG;
  const RowScale rs = {ss, n_parts, eps};
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  switch ((M + 15) / 16) {
    case 2: return launch_partial<2>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 3: return launch_partial<3>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 4: return launch_partial<4>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 5: return launch_partial<5>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 6: return launch_partial<6>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 7: return launch_partial<7>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
    case 8: return launch_partial<8>(a, w, workspace, workspace_floats, M, N, K, slices, rs, stream);
  }
  return YALM_ERR_ARG;
}

extern "C" int yalm_gemm_partial(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N,
                                 int K, int* slices, hipStream_t stream) {
  if (M > 128 || (M > 64 && K % 64 != 0))
    return yalm_gemm_bf16_dma_partial(A, W, workspace, workspace_floats, M, N, K, slices, 0, stream);
  return gemm_partial_scaled(A, W, workspace, workspace_floats, M, N, K, slices, nullptr, 0, 0.f, stream);
}

// yalm_gemm_partial with the row scale of yalm_gemm_scaled applied to every slice (17..128 rows only).
extern "C" int yalm_gemm_partial_scaled(const void* A, const void* W, float* workspace, long workspace_floats, int M,
                                        int N, int K, int* slices, const float* ss, int n_parts, float eps,
                                        hipStream_t stream) {
  if (ss == nullptr) return YALM_ERR_ARG;
  return gemm_partial_scaled(A, W, workspace, workspace_floats, M, N, K, slices, ss, n_parts, eps, stream);
}

// C (float32 residual stream) += A * W^T for more than 16 rows, and h = RMSNorm(C_new) * norm_w in bfloat16
// for the next consumer.  Needs scratch for at least M * N floats; refuses (YALM_ERR_ARG) other shapes.
static int gemm_add_norm_or_emit(const void* A, const void* W, float* C, float* workspace, long workspace_floats,
                                 int M, int N, int K, const float* norm_w, float eps, void* h_out, float* emit_ss,
                                 hipStream_t stream) {
  if (norm_w == nullptr || h_out == nullptr) return YALM_ERR_ARG;
  if (M > 128 || (M > 64 && K % 64 != 0)) {        // the tiled kernel's slices, then the same reduction
    int slices = 0;
    int rc = yalm_gemm_bf16_dma_partial(A, W, workspace, workspace_floats, M, N, K, &slices, 1, stream);
    if (rc != YALM_OK) return rc;
    return launch_reduce_add_norm(workspace, C, norm_w, eps, (bf16*)h_out, M, N, slices, stream, emit_ss);
  }
  if (M <= 16 || K % 8 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return YALM_ERR_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  bf16* h = (bf16*)h_out;
  switch ((M + 15) / 16) {
    case 2: return launch_add_norm<2>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 3: return launch_add_norm<3>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 4: return launch_add_norm<4>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 5: return launch_add_norm<5>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 6: return launch_add_norm<6>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 7: return launch_add_norm<7>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
    case 8: return launch_add_norm<8>(a, w, C, workspace, workspace_floats, M, N, K, norm_w, eps, h, stream, emit_ss);
  }
  return YALM_ERR_ARG;
}

extern "C" int yalm_gemm_add_norm(const void* A, const void* W, float* C, float* workspace, long workspace_floats,
                                  int M, int N, int K, const float* norm_w, float eps, void* h_out,
                                  hipStream_t stream) {
  return gemm_add_norm_or_emit(A, W, C, workspace, workspace_floats, M, N, K, norm_w, eps, h_out, nullptr, stream);
}

// The same product and residual add, but the next norm is only prepared: xn_out bfloat16 [M,N] = C_new * norm_w and
// ss_out float32 [M, yalm_gemm_add_emit_parts(N)] = sums of squares of C_new over the columns of each part; the
// consumer (yalm_gemm_scaled, yalm_gemm_partial_scaled) scales its sums.  Same shapes as yalm_gemm_add_norm.
extern "C" int yalm_gemm_add_emit(const void* A, const void* W, float* C, float* workspace, long workspace_floats,
                                  int M, int N, int K, const float* norm_w, void* xn_out, float* ss_out,
                                  hipStream_t stream) {
  if (ss_out == nullptr || N % 8 != 0 || ((uintptr_t)norm_w & 15)) return YALM_ERR_ARG;   // a consumer's K is this N
  return gemm_add_norm_or_emit(A, W, C, workspace, workspace_floats, M, N, K, norm_w, 0.f, xn_out, ss_out, stream);
}
extern "C" int yalm_gemm_add_emit_parts(int N) { return emit_parts(N); }

// Adds `slices` float32 partial products [slices][M][N] in order and applies the epilogue (for the
// kernels that split K: this file's and the tiled one of gemm_dma.hip).
int yalm_splitk_reduce(const float* partial, void* C, int M, int N, int H, int slices, int epilogue,
                       hipStream_t stream) {
  const long items = (long)M * (gated(epilogue) ? (N / 2) / 4 : (N + 3) / 4);
  const int blocks = ceil_div(items, 256);
  switch (epilogue) {
    case 0: splitk_reduce_kernel<0><<<blocks, 256, 0, stream>>>(partial, C, M, N, H, slices); break;
    case 1: splitk_reduce_kernel<1><<<blocks, 256, 0, stream>>>(partial, C, M, N, H, slices); break;
    case 2: splitk_reduce_kernel<2><<<blocks, 256, 0, stream>>>(partial, C, M, N, H, slices); break;
    case 3: splitk_reduce_kernel<3><<<blocks, 256, 0, stream>>>(partial, C, M, N, H, slices); break;
    case 5: splitk_reduce_kernel<5><<<blocks, 256, 0, stream>>>(partial, C, M, N, H, slices); break;
    default: return YALM_ERR_ARG;
  }
  return launch_status();
}
