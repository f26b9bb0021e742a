// bfloat16 GEMMs on the matrix cores: C = A[M,K] * W[N,K]^T, float32 accumulation.
//
//  * gemm_skinny  (M <= 64, decode): bound by the one pass over the weights.  A
//    workgroup owns 16 or 32 weight rows and all of K; its waves split K in
//    chunks of 128, every lane streaming 64 contiguous bytes of a weight row per
//    chunk; the batch is the other MFMA operand (16 rows a tile, up to 4 tiles);
//    partial sums of the waves meet in LDS, then the epilogue runs once.
//  * gemm_tiled   (M > 64, prefill, K not a multiple of 64; otherwise gemm_dma.hip runs):
//    128x128x64 or 256x128x64 tiles through LDS with a register prefetch of the next
//    tile, 4 waves, v_mfma_f32_32x32x16_bf16.
//
// Both take any M and N and any K that is a multiple of 8 (rows must be 16-byte
// aligned); other shapes are refused so that the caller runs the float32-arithmetic kernel.
#include "common.h"
#include "skinny_gemm.h"
#include "yalm_hip.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;


__device__ __forceinline__ bf16x8 load8(const bf16* p, bool ok) {
  bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? *reinterpret_cast<const bf16x8*>(p) : z;
}

// ---------------------------------------------------------------------------
// skinny GEMM: see skinny_gemm.h
// ---------------------------------------------------------------------------
template <int EPI>
int skinny_dispatch(const bf16* X, const bf16* W, void* C, int M, int N, int K, int H, hipStream_t stream) {
  skinny::ChainArgs ca = {};
  return skinny::launch<EPI>(X, W, C, M, N, K, H, ca, stream);
}

// ---------------------------------------------------------------------------
// tiled GEMM
// ---------------------------------------------------------------------------
constexpr int TK = 64;
constexpr int LDS_ROW = TK + 8;                  // bf16 elements; 16 bytes of padding keep b128 reads off each other's banks

// MFMA 32x32x16: operand rows i/j = lane % 32, 8 k per lane at k offset 8 * (lane / 32);
// C: lane holds column j = lane % 32 and rows 8 * (r / 4) + 4 * (lane / 32) + r % 4 for r < 16.
// A workgroup of 4 waves (2 x 2) owns a TM x TN tile; a wave owns (TM/2) x (TN/2).
// One LDS buffer: the next k tile waits in registers while this one is multiplied.
template <int EPI, int TM, int TN, int NWM, int NWN, int MINW>
__global__ __launch_bounds__(NWM * NWN * WAVE, MINW) void gemm_tiled_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                            void* __restrict__ Cv, int M, int N, int K, int H) {
  constexpr int NT = NWM * NWN * WAVE;
  constexpr int WM = TM / NWM, WN = TN / NWN, FA = WM / 32, FB = WN / 32;
  constexpr int RPP = NT / 8;                    // rows covered by one pass of all threads
  constexpr int LA = TM / RPP, LB = TN / RPP;    // 16-byte chunks per thread and k tile
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16* As = reinterpret_cast<bf16*>(smem_raw);  // [TM][LDS_ROW]
  bf16* Ws = As + TM * LDS_ROW;                  // [TN][LDS_ROW]
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int wm = wave / NWN, wn = wave % NWN;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int li = lane % 32, lh = lane / 32;

  // global -> LDS: thread t carries 16 bytes of row (t / 8) + RPP p at k offset 8 * (t % 8)
  const int lrow = tid / 8, lk = (tid % 8) * 8;
  const bf16* ap[LA];
  const bf16* wp[LB];
  bool aok[LA], wok[LB];
#pragma unroll
  for (int p = 0; p < LA; ++p) {
    int m = m0 + lrow + RPP * p;
    aok[p] = m < M;
    ap[p] = A + (size_t)(aok[p] ? m : 0) * K + lk;
  }
#pragma unroll
  for (int p = 0; p < LB; ++p) {
    int n = n0 + lrow + RPP * p;
    wok[p] = n < N;
    wp[p] = W + (size_t)(wok[p] ? n : 0) * K + lk;
  }

  f32x16 acc[FA][FB];
#pragma unroll
  for (int a = 0; a < FA; ++a)
#pragma unroll
    for (int b = 0; b < FB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // rows of the W tile that feed the wave's column tiles: plain, or for the gated epilogue
  // even tiles = the gate rows and odd tiles = the up rows of two 16-row blocks
  int wrow_lds[FB];
#pragma unroll
  for (int b = 0; b < FB; ++b) {
    if (gated(EPI))
      wrow_lds[b] = wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16);
    else
      wrow_lds[b] = wn * WN + b * 32 + li;
  }

  bf16x8 ra[LA], rw[LB];
  const int nk = (K + TK - 1) / TK;
  {
    bool kok = lk < K;
#pragma unroll
    for (int p = 0; p < LA; ++p) ra[p] = load8(ap[p], aok[p] && kok);
#pragma unroll
    for (int p = 0; p < LB; ++p) rw[p] = load8(wp[p], wok[p] && kok);
  }
  for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
    for (int p = 0; p < LA; ++p) *reinterpret_cast<bf16x8*>(&As[(lrow + RPP * p) * LDS_ROW + lk]) = ra[p];
#pragma unroll
    for (int p = 0; p < LB; ++p) *reinterpret_cast<bf16x8*>(&Ws[(lrow + RPP * p) * LDS_ROW + lk]) = rw[p];
    __syncthreads();
    if (kt + 1 < nk) {
      bool kok = (kt + 1) * TK + lk < K;
#pragma unroll
      for (int p = 0; p < LA; ++p) ra[p] = load8(ap[p] + (size_t)(kt + 1) * TK, aok[p] && kok);
#pragma unroll
      for (int p = 0; p < LB; ++p) rw[p] = load8(wp[p] + (size_t)(kt + 1) * TK, wok[p] && kok);
    }
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) {
      bf16x8 fa[FA], fw[FB];
#pragma unroll
      for (int a = 0; a < FA; ++a)
        fa[a] = *reinterpret_cast<const bf16x8*>(&As[(wm * WM + a * 32 + li) * LDS_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int b = 0; b < FB; ++b)
        fw[b] = *reinterpret_cast<const bf16x8*>(&Ws[wrow_lds[b] * LDS_ROW + ks * 16 + lh * 8]);
#pragma unroll
      for (int a = 0; a < FA; ++a)
#pragma unroll
        for (int b = 0; b < FB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[a], fw[b], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }

  // epilogue
#pragma unroll
  for (int a = 0; a < FA; ++a) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      int m = m0 + wm * WM + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
      if (m >= M) continue;
      if (gated(EPI)) {
#pragma unroll
        for (int pp = 0; pp < FB / 2; ++pp) {
          int hcol = (n0 + wn * WN + pp * 64) / 2 + li;
          if (hcol < H)
            ((bf16*)Cv)[(size_t)m * H + hcol] =
                static_cast<bf16>(gate_act<EPI>(acc[a][2 * pp][r]) * acc[a][2 * pp + 1][r]);
        }
      } else {
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          int n = n0 + wn * WN + b * 32 + li;
          if (n >= N) continue;
          size_t o = (size_t)m * N + n;
          if (EPI == 0) ((float*)Cv)[o] = acc[a][b][r];
          if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(acc[a][b][r]);
          if (EPI == 2) ((float*)Cv)[o] += acc[a][b][r];
        }
      }
    }
  }
}

template <int EPI, int TM, int TN, int NWM, int NWN, int MINW>
int tiled_launch_shape(const bf16* A, const bf16* W, void* C, int M, int N, int K, int H, hipStream_t stream) {
  dim3 grid(ceil_div(N, TN), ceil_div(M, TM));
  size_t lds = (size_t)(TM + TN) * LDS_ROW * sizeof(bf16);
  gemm_tiled_kernel<EPI, TM, TN, NWM, NWN, MINW><<<grid, NWM * NWN * WAVE, lds, stream>>>(A, W, C, M, N, K, H);
  return launch_status();
}

template <int EPI>
int tiled_launch(const bf16* A, const bf16* W, void* C, int M, int N, int K, int H, hipStream_t stream) {
  // 256x128 tiles move fewer bytes per flop; 128x128 tiles where those would not fill the chip
  if ((long)ceil_div(M, 256) * ceil_div(N, 128) > 1024)
    return tiled_launch_shape<EPI, 256, 128, 2, 2, 2>(A, W, C, M, N, K, H, stream);
  return tiled_launch_shape<EPI, 128, 128, 2, 2, 2>(A, W, C, M, N, K, H, stream);
}

}  // namespace

int yalm_gemm_bf16_batch(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                         int K, int epilogue, int H, hipStream_t stream);   // gemm_batch.hip

int yalm_gemm_bf16_dma(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                       int K, int epilogue, int H, hipStream_t stream);      // gemm_dma.hip

int yalm_gemm_bf16_mfma(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                        int K, int epilogue, int H, hipStream_t stream) {
  if (K % 8 != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return YALM_ERR_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if (M > 16 && M <= 128) {                        // (more than 64 rows: only with K a multiple of 64)
    int rc = yalm_gemm_bf16_batch(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, stream);
    if (rc != YALM_ERR_ARG) return rc;
  }
  if (M <= 64) {
    switch (epilogue) {
      case 0: return skinny_dispatch<0>(a, w, C, M, N, K, H, stream);
      case 1: return skinny_dispatch<1>(a, w, C, M, N, K, H, stream);
      case 2: return skinny_dispatch<2>(a, w, C, M, N, K, H, stream);
      case 3: return skinny_dispatch<3>(a, w, C, M, N, K, H, stream);
      case 5: return skinny_dispatch<5>(a, w, C, M, N, K, H, stream);
    }
    return YALM_ERR_ARG;
  }
  {
    int rc = yalm_gemm_bf16_dma(A, W, C, workspace, workspace_floats, M, N, K, epilogue, H, stream);   // K % 64 == 0
    if (rc != YALM_ERR_ARG) return rc;
  }
  switch (epilogue) {
    case 0: return tiled_launch<0>(a, w, C, M, N, K, H, stream);
    case 1: return tiled_launch<1>(a, w, C, M, N, K, H, stream);
    case 2: return tiled_launch<2>(a, w, C, M, N, K, H, stream);
    case 3: return tiled_launch<3>(a, w, C, M, N, K, H, stream);
    case 5: return tiled_launch<5>(a, w, C, M, N, K, H, stream);
  }
  return YALM_ERR_ARG;
}
