// C = A[M,K] * W[N,K]^T, float32 arithmetic for every storage type.  This is the
// kernel of the true 32-bit path and the fallback of the bfloat16 path for
// shapes the MFMA kernels refuse.  64x64 tile, 16-deep k steps through LDS,
// 256 threads with a 4x4 register tile each; any M, N, K.
#include "common.h"
#include "yalm_hip.h"

int yalm_gemm_bf16_mfma(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                        int K, int epilogue, int H, hipStream_t stream);   // gemm_mfma.hip; YALM_ERR_ARG: shape refused

namespace {
constexpr int BM = 64, BN = 64, BK = 16;

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

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
    if (EPI == 3) {
      T* C = (T*)Cv;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        int hcol = (n0 / 32 + jj) * 16 + tx;
        if (hcol < H) C[(size_t)m * H + hcol] = from_f32<T>(silu_f(acc[i][2 * jj]) * acc[i][2 * jj + 1]);
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
    default: return YALM_ERR_ARG;
  }
  return launch_status();
}
}  // namespace

extern "C" int yalm_gemm(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                         int K, int dtype, int epilogue, int H, int force_simple, hipStream_t stream) {
  if (M <= 0) return YALM_OK;
  if (N <= 0 || K <= 0 || epilogue < 0 || epilogue > 3) return YALM_ERR_ARG;
  if (epilogue == 3 && (H <= 0 || N != 32 * ((H + 15) / 16))) return YALM_ERR_ARG;
  if (dtype == YALM_F32) return gemm_simple<float>(A, W, C, M, N, K, epilogue, H, stream);
  if (dtype != YALM_BF16) return YALM_ERR_DTYPE;
  if (!force_simple) {
    int rc = yalm_gemm_bf16_mfma(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, stream);
    if (rc != YALM_ERR_ARG) return rc;
  }
  return gemm_simple<bf16>(A, W, C, M, N, K, epilogue, H, stream);
}
