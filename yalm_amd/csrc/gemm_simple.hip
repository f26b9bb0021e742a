// C = A[M,K] * W[N,K]^T, float32 arithmetic for every storage type: the kernels of the
// true 32-bit path and the fallback of the bfloat16 path for shapes the MFMA kernels
// refuse.  gemm_simple: 64x64 tile, 16-deep k steps through LDS, 256 threads with a 4x4
// register tile each; any M, N, K.  gemm_rows_f32: at most 64 rows of float32, a pass over
// the weights for every 16 of them (below).
#include "common.h"
#include "yalm_hip.h"

int yalm_gemm_bf16_mfma(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                        int K, int epilogue, int H, hipStream_t stream);   // gemm_mfma.hip; YALM_ERR_ARG: shape refused

namespace {
constexpr int BM = 64, BN = 64, BK = 16;


template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemm_simple_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                          void* __restrict__ Cv, int M, int N, int K, int H) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int ty = tid / 16, tx = tid % 16;
  const int lr = tid / 4, lk = (tid % 4) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const bool a_row_ok = m0 + lr < M, w_row_ok = n0 + lr < N;
  const T* a_row = A + (size_t)(a_row_ok ? m0 + lr : 0) * K;
  const T* w_row = W + (size_t)(w_row_ok ? n0 + lr : 0) * K;

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      int k = k0 + lk + e;
      As[lk + e][lr] = (a_row_ok && k < K) ? to_f32(a_row[k]) : 0.f;
      Ws[lk + e][lr] = (w_row_ok && k < K) ? to_f32(w_row[k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    if (gated(EPI)) {
      T* C = (T*)Cv;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        int hcol = (n0 / 32 + jj) * 16 + tx;
        if (hcol < H) C[(size_t)m * H + hcol] = from_f32<T>(gate_act<EPI>(acc[i][2 * jj]) * acc[i][2 * jj + 1]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int n = n0 + tx + 16 * j;
        if (n >= N) continue;
        size_t o = (size_t)m * N + n;
        if (EPI == 0) ((float*)Cv)[o] = acc[i][j];
        if (EPI == 1) ((T*)Cv)[o] = from_f32<T>(acc[i][j]);
        if (EPI == 2) ((float*)Cv)[o] += acc[i][j];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Float32 weights and at most 16 rows (a decode step of the 32-bit path): one pass over the weights
// at the speed of memory instead of 64x64 tiles that are mostly padding.  A wave owns 4 weight rows
// and walks K in chunks of 256: every lane takes 4 consecutive k of each of its rows (16-byte loads,
// a row's chunk is 1 KB contiguous for the wave) and multiplies them with the same 4 k of all batch
// rows, which the workgroup keeps in LDS.  The lanes' partial sums are added by a wave reduction at
// the end, so the order of the additions is fixed.  The gated epilogue takes a workgroup of 8 waves:
// 16 gate rows and their 16 up rows.
// ---------------------------------------------------------------------------
constexpr int RK = 256;                            // k a chunk: 64 lanes x 4

template <int MB, int EPI>
__global__ __launch_bounds__(gated(EPI) ? 512 : 256) void gemm_rows_f32_kernel(const float* __restrict__ A,
                                                                             const float* __restrict__ W,
                                                                             void* __restrict__ Cv, int M, int N, int K,
                                                                             int H) {
  constexpr int NWV = gated(EPI) ? 8 : 4;
  __shared__ __attribute__((aligned(16))) float xs[2][MB][RK];
  __shared__ float sums[NWV * 4][MB];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int n0 = blockIdx.x * NWV * 4 + wave * 4;
  const float* wrow[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wrow[r] = W + (size_t)min(n0 + r, N - 1) * K;
  float acc[4][MB];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0.f;

  const int n_chunks = (K + RK - 1) / RK;
  auto stage_x = [&](int c, int buf) {             // the workgroup's copy of chunk c of the batch rows (zeros beyond M and K)
    for (int e = tid; e < MB * (RK / 4); e += NWV * WAVE) {
      const int m = e / (RK / 4), k = c * RK + (e % (RK / 4)) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (m < M && k < K) v = *reinterpret_cast<const float4*>(A + (size_t)m * K + k);
      *reinterpret_cast<float4*>(&xs[buf][m][(e % (RK / 4)) * 4]) = v;
    }
  };
  auto load_w = [&](int c, float4 (&w)[4]) {
    const int k = c * RK + lane * 4;
    const int kk = k < K ? k : 0;                  // lanes beyond K read the row's start, and it counts as zeros
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      w[r] = *reinterpret_cast<const float4*>(wrow[r] + kk);
      if (k >= K) w[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  float4 wv[4];
  stage_x(0, 0);
  load_w(0, wv);
  __syncthreads();
  for (int c = 0; c < n_chunks; ++c) {
    const int cur = c & 1;
    float4 wn[4];
    if (c + 1 < n_chunks) {
      load_w(c + 1, wn);
      stage_x(c + 1, cur ^ 1);
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float4 x = *reinterpret_cast<const float4*>(&xs[cur][m][lane * 4]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc[r][m] = fmaf(wv[r].x, x.x, acc[r][m]);
        acc[r][m] = fmaf(wv[r].y, x.y, acc[r][m]);
        acc[r][m] = fmaf(wv[r].z, x.z, acc[r][m]);
        acc[r][m] = fmaf(wv[r].w, x.w, acc[r][m]);
      }
    }
    if (c + 1 < n_chunks) {
#pragma unroll
      for (int r = 0; r < 4; ++r) wv[r] = wn[r];
    }
    __syncthreads();                               // the next chunk of the batch rows is there; this one is read
  }

#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      const float t = wave_sum(acc[r][m]);
      if (lane == 0) sums[wave * 4 + r][m] = t;
    }
  __syncthreads();
  if (gated(EPI)) {                                  // rows 0..15 of the workgroup are gate rows, 16..31 their up rows
    const int base = blockIdx.x * 16;
    for (int e = tid; e < 16 * MB; e += NWV * WAVE) {
      const int j = e % 16, m = e / 16, hcol = base + j;
      if (m < M && hcol < H)
        ((float*)Cv)[(size_t)m * H + hcol] = gate_act<EPI>(sums[j][m]) * sums[16 + j][m];
    }
  } else {
    const int nb = blockIdx.x * NWV * 4;
    for (int e = tid; e < NWV * 4 * MB; e += NWV * WAVE) {
      const int j = e % (NWV * 4), m = e / (NWV * 4), n = nb + j;
      if (m >= M || n >= N) continue;
      const size_t o = (size_t)m * N + n;
      if (EPI == 0 || EPI == 1) ((float*)Cv)[o] = sums[j][m];
      if (EPI == 2) ((float*)Cv)[o] += sums[j][m];
    }
  }
}

template <int MB>
int launch_rows_f32(const float* A, const float* W, void* C, int M, int N, int K, int epilogue, int H,
                    hipStream_t stream) {
  switch (epilogue) {
    case 0: gemm_rows_f32_kernel<MB, 0><<<ceil_div(N, 16), 256, 0, stream>>>(A, W, C, M, N, K, H); break;
    case 1: gemm_rows_f32_kernel<MB, 1><<<ceil_div(N, 16), 256, 0, stream>>>(A, W, C, M, N, K, H); break;
    case 2: gemm_rows_f32_kernel<MB, 2><<<ceil_div(N, 16), 256, 0, stream>>>(A, W, C, M, N, K, H); break;
    case 3: gemm_rows_f32_kernel<MB, 3><<<ceil_div(N, 32), 512, 0, stream>>>(A, W, C, M, N, K, H); break;
    case 5: gemm_rows_f32_kernel<MB, 5><<<ceil_div(N, 32), 512, 0, stream>>>(A, W, C, M, N, K, H); break;
    default: return YALM_ERR_ARG;
  }
  return launch_status();
}

// float32, at most 64 rows (16 a pass over the weights: up to four passes still beat the tiles, which
// are mostly padding then), K a multiple of 4 and 16-byte aligned operands; YALM_ERR_ARG: not taken
int gemm_rows_f32(const void* A, const void* W, void* C, int M, int N, int K, int epilogue, int H, hipStream_t stream) {
  if (M > 64 || K % 4 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return YALM_ERR_ARG;
  const float* w = (const float*)W;
  const int out_cols = gated(epilogue) ? H : N;
  for (int m0 = 0; m0 < M; m0 += 16) {
    const float* a = (const float*)A + (size_t)m0 * K;
    float* c = (float*)C + (size_t)m0 * out_cols;
    const int rows = min(16, M - m0);
    int rc;
    if (rows <= 4) rc = launch_rows_f32<4>(a, w, c, rows, N, K, epilogue, H, stream);
    else if (rows <= 8) rc = launch_rows_f32<8>(a, w, c, rows, N, K, epilogue, H, stream);
    else rc = launch_rows_f32<16>(a, w, c, rows, N, K, epilogue, H, stream);
    if (rc != YALM_OK) return rc;
  }
  return YALM_OK;
}

template <typename T>
int gemm_simple(const void* A, const void* W, void* C, int M, int N, int K, int epilogue, int H, hipStream_t stream) {
  dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
  const T* a = (const T*)A;
  const T* w = (const T*)W;
  switch (epilogue) {
    case 0: gemm_simple_kernel<T, 0><<<grid, 256, 0, stream>>>(a, w, C, M, N, K, H); break;
    case 1: gemm_simple_kernel<T, 1><<<grid, 256, 0, stream>>>(a, w, C, M, N, K, H); break;
    case 2: gemm_simple_kernel<T, 2><<<grid, 256, 0, stream>>>(a, w, C, M, N, K, H); break;
    case 3: gemm_simple_kernel<T, 3><<<grid, 256, 0, stream>>>(a, w, C, M, N, K, H); break;
    case 5: gemm_simple_kernel<T, 5><<<grid, 256, 0, stream>>>(a, w, C, M, N, K, H); break;
    default: return YALM_ERR_ARG;
  }
  return launch_status();
}
}  // namespace

extern "C" int yalm_gemm(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                         int K, int dtype, int epilogue, int H, int force_simple, hipStream_t stream) {
  if (M <= 0) return YALM_OK;
  if (N <= 0 || K <= 0 || epilogue < 0 || (epilogue > 3 && epilogue != EPI_GATED_GELU)) return YALM_ERR_ARG;
  if (gated(epilogue) && (H <= 0 || N != 32 * ((H + 15) / 16))) return YALM_ERR_ARG;
  if (dtype == YALM_F32) {
    if (!force_simple) {
      int rc = gemm_rows_f32(A, W, C, M, N, K, epilogue, H, stream);
      if (rc != YALM_ERR_ARG) return rc;
    }
    return gemm_simple<float>(A, W, C, M, N, K, epilogue, H, stream);
  }
  if (dtype != YALM_BF16) return YALM_ERR_DTYPE;
  if (!force_simple) {
    int rc = yalm_gemm_bf16_mfma(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, stream);
    if (rc != YALM_ERR_ARG) return rc;
  }
  return gemm_simple<bf16>(A, W, C, M, N, K, epilogue, H, stream);
}
