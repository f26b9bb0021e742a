// Prefill GEMM whose k tiles go from global memory straight into LDS:
// C = epilogue(A[M,K] * W[N,K]^T), bfloat16 operands, float32 accumulation, more than 64 rows.
//
// A workgroup owns a TM x TN tile of C.  Its waves issue global_load_lds_dwordx4 (16 bytes a
// lane, a wave's 64 lanes land as 1 KB contiguous in LDS) for k tile kt + S - 1 into a ring
// of S stages while they multiply k tile kt; no register or LDS write instruction stands
// between memory and the matrix cores.  Rows are kept unpadded (128 bytes for 64 k) and the
// 16-byte chunks of a row are XOR-swizzled by the row number, which every lane applies to
// the GLOBAL address it asks for, so that the b128 fragment reads of 16 consecutive rows
// fall on different banks.  The compiler does not know that these loads write LDS: the
// kernel waits for them itself (s_waitcnt vmcnt) and uses the bare s_barrier, because
// __syncthreads() carries a fence that would wait for the loads of all stages.
//
// With few tiles (a decode batch of more than 64 rows) K is split over grid z as well: every slice
// writes its float32 partial product and yalm_splitk_reduce adds them in order and applies the epilogue.
//
// Takes any M and N and K % 64 == 0; other shapes are refused (YALM_ERR_ARG) and the
// caller runs the kernel of gemm_mfma.hip.  Sums are in a fixed order for a given shape.
#include "common.h"
#include "yalm_hip.h"

int yalm_splitk_reduce(const float* partial, void* C, int M, int N, int H, int slices, int epilogue,
                       hipStream_t stream);                                  // gemm_batch.hip

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int TK = 64;
constexpr int ROWB = TK * 2;                     // bytes a row of a stage
constexpr int CPR = ROWB / 16;                   // 16-byte chunks a row
constexpr int RPI = WAVE / CPR;                  // rows one wave instruction brings

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }
__device__ __forceinline__ int swizzle_of(int row) { return (row >> 1) & (CPR - 1); }

template <int N_>
__device__ __forceinline__ void wait_vmcnt() {   // vmcnt only: expcnt and lgkmcnt fields at their maxima
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// MFMA 32x32x16: operand rows i/j = lane % 32, 8 k per lane at k offset 8 * (lane / 32);
// C: lane holds column j = lane % 32 and rows 8 * (r / 4) + 4 * (lane / 32) + r % 4 for r < 16.
template <int EPI, int TM, int TN, int S, int NWM, int NWN, int MINW>
__global__ __launch_bounds__(NWM * NWN * WAVE, MINW) void gemm_dma_kernel(const bf16* __restrict__ A,
                                                                         const bf16* __restrict__ W,
                                                                         void* __restrict__ Cv, int M, int N, int K,
                                                                         int H, float* __restrict__ partial,
                                                                         int tiles_per_slice, int n_tile0) {
  constexpr int NW = NWM * NWN;
  constexpr int ROWS = TM + TN;                    // A rows, then W rows
  constexpr int STAGE_B = ROWS * ROWB;
  constexpr int L = ROWS / (RPI * NW);             // load instructions a wave and stage
  static_assert(ROWS % (RPI * NW) == 0, "the rows of a stage must divide over the waves");
  static_assert((S - 2) * L < 64, "vmcnt holds 6 bits");
  constexpr int WM = TM / NWM, WN = TN / NWN, FA = WM / 32, FB = WN / 32;
  constexpr int KS = TK / 16;
  extern __shared__ __attribute__((aligned(1024))) unsigned char stages[];
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  const int wm = wave / NWN, wn = wave % NWN;
  const int m0 = blockIdx.y * TM, n0 = (blockIdx.x + n_tile0) * TN;   // a launch may own a range of the columns
  const int li = lane % 32, lh = lane / 32;

  // instruction i of this wave fills rows (i * NW + wave) * RPI ... of a stage; the lane's
  // place there is (row, slot), and it asks memory for the chunk that belongs in that slot
  const bf16* gp[L];
#pragma unroll
  for (int i = 0; i < L; ++i) {
    const int row = (i * NW + wave) * RPI + lane / CPR;
    const int chunk = (lane % CPR) ^ swizzle_of(row);
    const bf16* base = row < TM ? A + (size_t)min(m0 + row, M - 1) * K          // rows past the edge repeat the last
                                : W + (size_t)min(n0 + row - TM, N - 1) * K;    // one and are never stored
    gp[i] = base + chunk * 8;
  }
  auto issue = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < L; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass drops a template that names this builtin, and its launch stub with it
      __builtin_amdgcn_global_load_lds(gp[i] + (size_t)kt * TK, stages + stage * STAGE_B + (i * NW + wave) * 1024, 16, 0,
                                       0);
#endif
    }
  };

  f32x16 acc[FA][FB];
#pragma unroll
  for (int a = 0; a < FA; ++a)
#pragma unroll
    for (int b = 0; b < FB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // fragment rows of this lane: A rows of the wave's row tiles; W rows of its column tiles, where
  // for the gated epilogue even tiles are the gate rows and odd tiles the up rows of two 16-row blocks
  int a_base[FA], a_swz[FA], w_base[FB], w_swz[FB];
#pragma unroll
  for (int a = 0; a < FA; ++a) {
    const int row = wm * WM + a * 32 + li;
    a_base[a] = row * ROWB;
    a_swz[a] = swizzle_of(row);
  }
#pragma unroll
  for (int b = 0; b < FB; ++b) {
    const int r = (EPI == 3) ? wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16) : wn * WN + b * 32 + li;
    const int row = TM + r;
    w_base[b] = row * ROWB;
    w_swz[b] = swizzle_of(row);
  }

  // grid z: slices of K (each writes its float32 partial product; a second kernel adds them)
  const int kt0 = blockIdx.z * tiles_per_slice;
  const int nk = min(K / TK - kt0, tiles_per_slice);
#pragma unroll
  for (int i = 0; i < L; ++i) gp[i] += (size_t)kt0 * TK;
#pragma unroll
  for (int s = 0; s < S - 1; ++s)
    if (s < nk) issue(s, s);
  for (int kt = 0; kt < nk; ++kt) {
    // stage kt has landed when at most the loads of the S - 2 stages behind it are in flight
    if (kt + S - 2 < nk) wait_vmcnt<(S - 2) * L>(); else wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();                  // everyone's part of stage kt is there, and everyone has read stage kt - 1
    asm volatile("" ::: "memory");
    if (kt + S - 1 < nk) issue(kt + S - 1, (kt + S - 1) % S);      // into the buffer that iteration kt - 1 read
    const unsigned char* cur = stages + (kt % S) * STAGE_B;
    bf16x8 fa[2][FA], fw[2][FB];
#pragma unroll
    for (int a = 0; a < FA; ++a) fa[0][a] = *reinterpret_cast<const bf16x8*>(cur + a_base[a] + ((lh ^ a_swz[a]) << 4));
#pragma unroll
    for (int b = 0; b < FB; ++b) fw[0][b] = *reinterpret_cast<const bf16x8*>(cur + w_base[b] + ((lh ^ w_swz[b]) << 4));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = ks & 1, n = c ^ 1;
      if (ks + 1 < KS) {                           // the next fragments are read while these are multiplied
        const int ch = (ks + 1) * 2 + lh;
#pragma unroll
        for (int a = 0; a < FA; ++a) fa[n][a] = *reinterpret_cast<const bf16x8*>(cur + a_base[a] + ((ch ^ a_swz[a]) << 4));
#pragma unroll
        for (int b = 0; b < FB; ++b) fw[n][b] = *reinterpret_cast<const bf16x8*>(cur + w_base[b] + ((ch ^ w_swz[b]) << 4));
      }
#pragma unroll
      for (int a = 0; a < FA; ++a)
#pragma unroll
        for (int b = 0; b < FB; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[c][a], fw[c][b], acc[a][b], 0, 0, 0);
    }
  }

  if (gridDim.z > 1) {                             // a slice of K: the plain sums, column n = weight row n
    float* plane = partial + (size_t)blockIdx.z * M * N;
#pragma unroll
    for (int a = 0; a < FA; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
        if (m >= M) continue;
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int wr = (EPI == 3) ? wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16) : wn * WN + b * 32 + li;
          const int n = n0 + wr;
          if (n < N) plane[(size_t)m * N + n] = acc[a][b][r];
        }
      }
    return;
  }
#pragma unroll
  for (int a = 0; a < FA; ++a) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * WM + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
      if (m >= M) continue;
      if (EPI == 3) {
#pragma unroll
        for (int pp = 0; pp < FB / 2; ++pp) {
          const int hcol = (n0 + wn * WN + pp * 64) / 2 + li;
          if (hcol < H)
            ((bf16*)Cv)[(size_t)m * H + hcol] = static_cast<bf16>(silu_f(acc[a][2 * pp][r]) * acc[a][2 * pp + 1][r]);
        }
      } else {
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int n = n0 + wn * WN + b * 32 + li;
          if (n >= N) continue;
          const size_t o = (size_t)m * N + n;
          if (EPI == 0) ((float*)Cv)[o] = acc[a][b][r];
          if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(acc[a][b][r]);
          if (EPI == 2) ((float*)Cv)[o] += acc[a][b][r];
        }
      }
    }
  }
}

template <int EPI, int TM, int TN, int S, int NWM, int NWN, int MINW>
int launch_shape(const bf16* A, const bf16* W, void* C, int M, int N, int K, int H, float* partial, int slices,
                 hipStream_t stream, bool add_slices = true, int n_tile0 = 0, int n_tiles = -1) {
  const int tiles_per_slice = ceil_div(K / TK, slices);
  if (n_tiles < 0) n_tiles = ceil_div(N, TN) - n_tile0;     // column tiles n_tile0 ... of this launch
  const dim3 grid(n_tiles, ceil_div(M, TM), ceil_div(K / TK, tiles_per_slice));
  const size_t lds = (size_t)S * (TM + TN) * ROWB;
  static bool allowed = false;                     // more than 64 KB of LDS has to be asked for once
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)&gemm_dma_kernel<EPI, TM, TN, S, NWM, NWN, MINW>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    allowed = true;
  }
  gemm_dma_kernel<EPI, TM, TN, S, NWM, NWN, MINW><<<grid, NWM * NWN * WAVE, lds, stream>>>(A, W, C, M, N, K, H, partial,
                                                                                       tiles_per_slice, n_tile0);
  int rc = launch_status();
  if (rc != YALM_OK || grid.z == 1 || !add_slices) return rc;
  return yalm_splitk_reduce(partial, C, M, N, H, (int)grid.z, EPI, stream);
}

// slices of K for the 128x128 tiles: with few rows (a big decode batch) the tiles alone leave most CUs
// without work and the weights would stream through a few of them
int slices_for(int M, int N, int K, long workspace_floats) {
  const long tiles = (long)ceil_div(M, 128) * ceil_div(N, 128);
  int slices = 1;
  while (tiles * slices < 384 && slices * 2 <= (K / TK) / 8 && slices < 16 &&
         (long)slices * 2 * M * N <= workspace_floats)
    slices *= 2;
  return slices;
}

// 256x256 tiles (8 waves, two stages of 64 KB, one workgroup a CU) ask the caches for the
// fewest bytes per product; 128x128 tiles (4 waves, two workgroups a CU) where those would
// leave CUs without work.
template <int EPI>
int launch(const bf16* A, const bf16* W, void* C, float* ws, long ws_floats, int M, int N, int K, int H,
           hipStream_t stream) {
  const long t256 = (long)ceil_div(M, 256) * ceil_div(N, 256);
  if (t256 >= 160) {
    // 256x192 tiles where they fill the last round of workgroups so much better that it outweighs their
    // fewer products per byte (2,048 x 6,144: 256 tiles for 256 CUs instead of 192; 100 against 123 us)
    if (EPI != 3) {
      const long t192 = (long)ceil_div(M, 256) * ceil_div(N, 192);
      auto filled = [](long tiles) { return (double)tiles / (double)(ceil_div(tiles, 256L) * 256L); };
      if (filled(t192) * 0.93 > filled(t256))
        return launch_shape<EPI, 256, 192, 2, 4, 2, 1>(A, W, C, M, N, K, H, nullptr, 1, stream);
    }
    // A last round of workgroups that is at most half full: its columns go to a second launch of
    // 256x128 tiles, which fills the chip with them (2,048 x 28,672: 3 rounds + 1 of half-wide tiles
    // instead of 3.5 that cost 4).
    const int mt = ceil_div(M, 256), nt = ceil_div(N, 256);
    const long rounds = t256 / 256, rest = t256 % 256;
    const int nt_main = (int)(rounds * 256 / mt);
    if (rounds >= 1 && rest > 0 && rest <= 128 && nt_main > 0 && nt_main < nt) {
      int rc = launch_shape<EPI, 256, 256, 2, 4, 2, 1>(A, W, C, M, N, K, H, nullptr, 1, stream, true, 0, nt_main);
      if (rc != YALM_OK) return rc;
      return launch_shape<EPI, 256, 128, 2, 4, 2, 1>(A, W, C, M, N, K, H, nullptr, 1, stream, true, 2 * nt_main);
    }
    return launch_shape<EPI, 256, 256, 2, 4, 2, 1>(A, W, C, M, N, K, H, nullptr, 1, stream);
  }
  const int slices = ws != nullptr ? slices_for(M, N, K, ws_floats) : 1;
  return launch_shape<EPI, 128, 128, 2, 2, 2, 2>(A, W, C, M, N, K, H, ws, slices, stream);
}

}  // namespace

// floats of scratch with which yalm_gemm_bf16_dma would split K (0: it would not)
long yalm_gemm_bf16_dma_workspace(int M, int N, int K) {
  if (M <= 64 || K < TK || K % TK != 0 || (long)ceil_div(M, 256) * ceil_div(N, 256) >= 160) return 0;
  const int slices = slices_for(M, N, K, (long)1 << 40);
  return slices > 1 ? (long)slices * M * N : 0;
}

// The product's K slices, left unadded, as [*slices][M][N] float32 in the workspace (one slice: the product
// itself), for a consumer that adds them.  More than 64 rows, K a multiple of 64, at least M * N floats.
int yalm_gemm_bf16_dma_partial(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N,
                               int K, int* slices_out, hipStream_t stream) {
  if (M <= 64 || K < TK || K % TK != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15) || workspace == nullptr ||
      workspace_floats < (long)M * N || slices_out == nullptr)
    return YALM_ERR_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if ((long)ceil_div(M, 256) * ceil_div(N, 256) >= 160) {
    *slices_out = 1;
    return launch_shape<0, 256, 256, 2, 4, 2, 1>(a, w, workspace, M, N, K, 0, nullptr, 1, stream);
  }
  int slices = slices_for(M, N, K, workspace_floats);
  const int tiles_per_slice = ceil_div(K / TK, slices);
  slices = ceil_div(K / TK, tiles_per_slice);          // what the launch makes of it
  *slices_out = slices;
  return launch_shape<0, 128, 128, 2, 2, 2, 2>(a, w, workspace, M, N, K, 0, workspace, slices, stream, false);
}

int yalm_gemm_bf16_dma(const void* A, const void* W, void* C, float* workspace, long workspace_floats, int M, int N,
                       int K, int epilogue, int H, hipStream_t stream) {
  if (M <= 64 || K < TK || K % TK != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return YALM_ERR_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  switch (epilogue) {
    case 0: return launch<0>(a, w, C, workspace, workspace_floats, M, N, K, H, stream);
    case 1: return launch<1>(a, w, C, workspace, workspace_floats, M, N, K, H, stream);
    case 2: return launch<2>(a, w, C, workspace, workspace_floats, M, N, K, H, stream);
    case 3: return launch<3>(a, w, C, workspace, workspace_floats, M, N, K, H, stream);
  }
  return YALM_ERR_ARG;
}
