// GEMMs of more than 64 rows whose k tiles go from global memory straight into LDS:
// C = epilogue(A[M,K] * W[N,K]^T), bfloat16 operands, float32 accumulation.
//
// A workgroup owns a tile of C.  Its waves issue global_load_lds_dwordx4 (16 bytes a lane, a
// wave's 64 lanes land as 1 KB contiguous in LDS) for later k tiles while they multiply the
// current one; no register or LDS write instruction stands between memory and the matrix
// cores.  Rows are kept unpadded (128 bytes for 64 k) and the 16-byte chunks of a row are
// XOR-swizzled by the row number, which every lane applies to the GLOBAL address it asks
// for, so that the b128 fragment reads of 16 consecutive rows fall on different banks.  The
// compiler does not know that these loads write LDS: the kernels wait for them themselves
// (s_waitcnt vmcnt) and use the bare s_barrier, because __syncthreads() carries a fence that
// would wait for the loads of all stages.
//
// gemm_dma_kernel (128x128 tiles, two stages, two workgroups a CU) serves decode batches of 65 to 159
// rows: with few tiles K is split over grid z as well, every slice writes its float32 partial product and
// yalm_splitk_reduce adds them in order and applies the epilogue.  gemm_ring_kernel and gemm_ring16_kernel
// (256-row tiles, five slots in turn, loads issued between the products; K split the same way for short
// prompts) serve prompt steps and the biggest decode batches.
//
// Takes any M and N and K % 64 == 0; other shapes are refused (YALM_ERR_ARG) and the
// caller runs the kernel of gemm_mfma.hip.  Sums are in a fixed order for a given shape.
#include "common.h"
#include "yalm_hip.h"
#include <type_traits>

int yalm_splitk_reduce(const float* partial, void* C, int M, int N, int H, int slices, int epilogue,
                       hipStream_t stream);                                  // gemm_batch.hip

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int TK = 64;
constexpr int ROWB = TK * 2;                     // bytes a row of a stage
constexpr int CPR = ROWB / 16;                   // 16-byte chunks a row
constexpr int RPI = WAVE / CPR;                  // rows one wave instruction brings

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
    const int r = (gated(EPI)) ? wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16) : wn * WN + b * 32 + li;
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
          const int wr = (gated(EPI)) ? wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16) : wn * WN + b * 32 + li;
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
      if (gated(EPI)) {
#pragma unroll
        for (int pp = 0; pp < FB / 2; ++pp) {
          const int hcol = (n0 + wn * WN + pp * 64) / 2 + li;
          if (hcol < H)
            ((bf16*)Cv)[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(acc[a][2 * pp][r]) * acc[a][2 * pp + 1][r]);
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
  static LdsAllowance allowed;                     // more than 64 KB of LDS has to be asked for once a device
  if (int rc = allow_dynamic_lds(allowed, (const void*)&gemm_dma_kernel<EPI, TM, TN, S, NWM, NWN, MINW>, (int)lds);
      rc != YALM_OK)
    return rc;
  gemm_dma_kernel<EPI, TM, TN, S, NWM, NWN, MINW><<<grid, NWM * NWN * WAVE, lds, stream>>>(A, W, C, M, N, K, H, partial,
                                                                                       tiles_per_slice, n_tile0);
  int rc = launch_status();
  if (rc != YALM_OK || grid.z == 1 || !add_slices) return rc;
  return yalm_splitk_reduce(partial, C, M, N, H, (int)grid.z, EPI, stream);
}

// ---------------------------------------------------------------------------
// The kernel for many tiles: 256 x TN tiles, 8 waves, and a ring of five 32 KB slots that holds the k tiles of
// W and of A in turn (W0 A0 W1 A1 W2 ...; tile t has W in slot 2t mod 5 and A in slot (2t + 1) mod 5), so that
// two and a half k tiles are in flight or in use.  What it does differently from the kernel above, each measured:
//  * a vector memory instruction holds its wave for tens of clocks, more while the memory system is busy; issued
//    as a burst behind the barrier they stall every wave at once and the matrix cores idle.  Here a wave issues
//    one DMA instruction in every few products, all through the iteration, and each has a k step or more to land;
//  * the barrier stands between k steps 2 and 3 of a tile: the fragments of the last k step are in registers by
//    then, so nobody reads the tile's slots any more and they are refilled at once, and the first fragments
//    of the next tile are read while the last products of this one run;
//  * the fragments of a k step are read during the products of the one before (two register sets);
//  * the DMA takes its base from scalar registers and a 32-bit offset a lane (inline asm: the compiler would
//    add a 64-bit pair a lane for every instruction).
// The order of statements in the loop is the order of the instructions: a scheduling fence follows each.
// ---------------------------------------------------------------------------
constexpr int RING_SLOT = 32768, RING_SLOTS = 5, RING_TM = 256;

__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0x3F | (0x7 << 4) | (0x0 << 8) | (0x3 << 14)); }

// the product index of a k step (of n_products) behind which DMA instruction d of n_dma is issued
// (evenly spread: 2 of 8 go behind products 1 and 4)
__host__ __device__ constexpr int dma_place(int d, int n_dma, int n_products) {
  const int at = (d + 1) * n_products / (n_dma + 1) - 1;
  return at < 0 ? 0 : at;
}

template <int EPI, int TN, int MAP>
__global__ __launch_bounds__(512, 1) void gemm_ring_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                           void* __restrict__ Cv, int M, int N, int K, int H, int n_tile0,
                                                           int n_tiles, float* __restrict__ partial,
                                                           int tiles_per_slice) {
  constexpr int TM = RING_TM, NW = 8, NWM = 4, NWN = 2, WM = TM / NWM, WN = TN / NWN, FA = WM / 32, FB = WN / 32;
  constexpr int KS = TK / 16;
  constexpr int DA = (TM / 8) / NW, DW = (TN / 8) / NW;     // DMA instructions (8 rows each) a wave and slot
  constexpr int DA1 = DA / 2, DW1 = (DW + 1) / 2;           // of them in the first of the two k steps that issue them
  constexpr int NMF = FA * FB;                              // products a k step
  static_assert(TM % (8 * NW) == 0 && TN % (8 * NW) == 0 && DA % 2 == 0, "the rows of a slot must divide over the waves");
  static_assert(FA + FB <= NMF, "a fragment read follows a product");
  static_assert(!gated(EPI) || FB % 2 == 0, "the gated epilogue pairs column tiles");
  extern __shared__ __attribute__((aligned(1024))) unsigned char stages[];
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int wm = wave / NWN, wn = wave % NWN;
  const int li = lane % 32, lh = lane / 32;
  int tile_m, tile_n;
  if (MAP == 0) {
    tile_m = blockIdx.y;
    tile_n = blockIdx.x + n_tile0;
  } else {
    // Workgroup L runs on XCD L mod 8.  Every XCD takes a run of the tile sequence (groups of MAP tile columns;
    // in a group the rows fastest, then the columns), so that the tiles it works on at a time share rows and
    // columns in its second-level cache.
    const int mt = (M + TM - 1) / TM, T = mt * n_tiles, chunk = (T + 7) / 8;
    const int L = blockIdx.x, t = (L % 8) * chunk + L / 8;
    if (t >= T || L / 8 >= chunk) return;
    const int per_group = mt * MAP, g = t / per_group, r = t % per_group;
    const int width = min(MAP, n_tiles - g * MAP);        // the last group may be narrower
    tile_n = n_tile0 + g * MAP + r % width;
    tile_m = r / width;
  }
  const int m0 = tile_m * TM, n0 = tile_n * TN;
  // slices of K (grid z without the XCD mapping, grid y with it): each writes its float32 partial product
  const int slice = MAP == 0 ? blockIdx.z : blockIdx.y, n_slices = MAP == 0 ? gridDim.z : gridDim.y;
  const int kt0 = slice * tiles_per_slice;
  const int nk = min(K / TK - kt0, tiles_per_slice);

  // DMA instruction i of a wave fills rows (i * 8 + wave) * 8 ... + 7 of a slot; a lane's place there is (row,
  // 16-byte slot of the row), and it asks memory for the chunk that belongs there (rows past the edge repeat the
  // last one and are never stored)
  unsigned off_a[DA], off_w[DW];
  const char* a_base = (const char*)(A + (size_t)m0 * K + (size_t)kt0 * TK);
  const char* w_base = (const char*)(W + (size_t)n0 * K + (size_t)kt0 * TK);
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int row = (i * NW + wave) * RPI + lane / CPR;
    off_a[i] = (unsigned)(((size_t)min(row, M - 1 - m0) * K + ((lane % CPR) ^ swizzle_of(row)) * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < DW; ++i) {
    const int row = (i * NW + wave) * RPI + lane / CPR;
    off_w[i] = (unsigned)(((size_t)min(row, N - 1 - n0) * K + ((lane % CPR) ^ swizzle_of(row)) * 8) * 2);
  }
  auto dma = [&](const char* base, unsigned off, int slot, int i) {
    const unsigned lds_addr = (unsigned)(uintptr_t)(stages + slot * RING_SLOT + (i * NW + wave) * 1024);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
  };

  f32x16 acc[FA][FB];
#pragma unroll
  for (int a = 0; a < FA; ++a)
#pragma unroll
    for (int b = 0; b < FB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // fragments: A rows of the wave's row tiles; W rows of its column tiles, where for the gated epilogue even tiles
  // are the gate rows and odd tiles the up rows of two 16-row blocks.  Address in a slot: row * 128 + ((2 ks + lh)
  // ^ swizzle) * 16; tiles 32 (16, 64) rows apart share the swizzle.
  const int a_row = wm * WM + li;
  const int w_row = (gated(EPI)) ? wn * WN + (li / 16) * 32 + (li % 16) : wn * WN + li;
  int a_at[KS], w_at[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    a_at[ks] = a_row * ROWB + (((2 * ks + lh) ^ swizzle_of(a_row)) << 4);
    w_at[ks] = w_row * ROWB + (((2 * ks + lh) ^ swizzle_of(w_row)) << 4);
  }
  auto frag_a = [&](int slot, int ks, int a) {
    return *reinterpret_cast<const bf16x8*>(stages + slot * RING_SLOT + a_at[ks] + a * 32 * ROWB);
  };
  auto frag_w = [&](int slot, int ks, int b) {
    const int rows = (gated(EPI)) ? (b / 2) * 64 + (b % 2) * 16 : b * 32;
    return *reinterpret_cast<const bf16x8*>(stages + slot * RING_SLOT + w_at[ks] + rows * ROWB);
  };

  // before the loop: W0 A0 W1 and the first half of A1 (what iterations -2 and -1 would have issued)
#pragma unroll
  for (int i = 0; i < DW; ++i) dma(w_base, off_w[i], 0, i);
#pragma unroll
  for (int i = 0; i < DA; ++i) dma(a_base, off_a[i], 1, i);
  if (nk > 1) {
#pragma unroll
    for (int i = 0; i < DW; ++i) dma(w_base + ROWB, off_w[i], 2, i);
#pragma unroll
    for (int i = 0; i < DA1; ++i) dma(a_base + ROWB, off_a[i], 3, i);
    wait_vmcnt<DW + DA1>();
  } else {
    wait_vmcnt<0>();
  }
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 fa[2][FA], fw[2][FB];
#pragma unroll
  for (int a = 0; a < FA; ++a) fa[0][a] = frag_a(1, 0, a);
#pragma unroll
  for (int b = 0; b < FB; ++b) fw[0][b] = frag_w(0, 0, b);

  int ws = 0, as = 1;                              // slots of the tile that is multiplied
  for (int kt = 0; kt < nk; ++kt) {
    const int ws1 = ws + 2 >= RING_SLOTS ? ws + 2 - RING_SLOTS : ws + 2;          // of tile kt + 1
    const int as1 = as + 2 >= RING_SLOTS ? as + 2 - RING_SLOTS : as + 2;
    const int ws2 = ws1 + 2 >= RING_SLOTS ? ws1 + 2 - RING_SLOTS : ws1 + 2;       // of tile kt + 2
    const int as2 = as1 + 2 >= RING_SLOTS ? as1 + 2 - RING_SLOTS : as1 + 2;
    const bool t1 = kt + 1 < nk, t2 = kt + 2 < nk;
    const char* a1 = a_base + (size_t)(kt + 1) * ROWB;
    const char* a2 = a_base + (size_t)(kt + 2) * ROWB;
    const char* w2 = w_base + (size_t)(kt + 2) * ROWB;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = ks & 1, n = c ^ 1;
      if (ks == KS - 1) {
        // The last fragments of tile kt are in registers; this wave's share of tile kt + 1 has landed (the second
        // half of A(kt + 1) from k step 0, and everything older; W(kt + 2) may still be on its way).  Behind the
        // barrier that holds for all waves: tile kt + 1 can be read and the slots of tile kt written.
        wait_lgkmcnt0();
        if (t2) wait_vmcnt<DW>(); else wait_vmcnt<0>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < NMF; ++j) {
        const int a = j / FB, b = j % FB;
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[c][a], fw[c][b], acc[a][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (ks < KS - 1) {                           // a fragment of k step ks + 1 of this tile
          if (j < FA) fa[n][j] = frag_a(as, ks + 1, j);
          else if (j < FA + FB) fw[n][j - FA] = frag_w(ws, ks + 1, j - FA);
        } else {                                     // of k step 0 of the next tile (behind the last tile: read, never used)
          if (j < FA) fa[n][j] = frag_a(as1, 0, j);
          else if (j < FA + FB) fw[n][j - FA] = frag_w(ws1, 0, j - FA);
        }
        // k step 0: the second half of A(kt + 1); 1 and 2: W(kt + 2); 3, behind the barrier: the first half of A(kt + 2)
        if (ks == 0) {
#pragma unroll
          for (int d = 0; d < DA - DA1; ++d)
            if (j == dma_place(d, DA - DA1, NMF) && t1) dma(a1, off_a[DA1 + d], as1, DA1 + d);
        } else if (ks == 1) {
#pragma unroll
          for (int d = 0; d < DW1; ++d)
            if (j == dma_place(d, DW1, NMF) && t2) dma(w2, off_w[d], ws2, d);
        } else if (ks == 2) {
#pragma unroll
          for (int d = 0; d < DW - DW1; ++d)
            if (j == dma_place(d, DW - DW1, NMF) && t2) dma(w2, off_w[DW1 + d], ws2, DW1 + d);
        } else {
#pragma unroll
          for (int d = 0; d < DA1; ++d)
            if (j == dma_place(d, DA1, NMF) && t2) dma(a2, off_a[d], as2, d);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    ws = ws1;
    as = as1;
  }
  wait_vmcnt<0>();                                 // nothing of this workgroup is on its way into LDS when it ends

  if (n_slices > 1) {                              // a slice of K: the plain sums, column n = weight row n
    float* plane = partial + (size_t)slice * M * N;
#pragma unroll
    for (int a = 0; a < FA; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + a * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
        if (m >= M) continue;
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int wr = (gated(EPI)) ? wn * WN + (b / 2) * 64 + (li / 16) * 32 + (b % 2) * 16 + (li % 16) : wn * WN + b * 32 + li;
          if (n0 + wr < N) plane[(size_t)m * N + n0 + wr] = acc[a][b][r];
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
      if (gated(EPI)) {
#pragma unroll
        for (int pp = 0; pp < FB / 2; ++pp) {
          const int hcol = (n0 + wn * WN + pp * 64) / 2 + li;
          if (hcol < H)
            ((bf16*)Cv)[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(acc[a][2 * pp][r]) * acc[a][2 * pp + 1][r]);
        }
      } else {
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int nn = n0 + wn * WN + b * 32 + li;
          if (nn >= N) continue;
          const size_t o = (size_t)m * N + nn;
          if (EPI == 0) ((float*)Cv)[o] = acc[a][b][r];
          if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(acc[a][b][r]);
          if (EPI == 2) ((float*)Cv)[o] += acc[a][b][r];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same ring with v_mfma_f32_16x16x32_bf16, for tiles of 256 and 192 columns.  The chip is power-bound under
// this loop (the shader clock falls to 1.5-1.8 GHz), and on random operands the 16x16x32 instruction does about a
// sixth more products for the same power than 32x32x16 (2.16 against 1.83 PFLOP/s out of registers: it moves a
// quarter of the accumulator registers per product); the whole GEMM gains 5-10 %.  (Tiles of 128 columns, 64x64 a
// wave, are 2-9 % slower this way and stay with the kernel above.)
// A wave owns 64 rows x TN/2 columns: 4 x FB tiles of 16x16.  A tile's 64 k are two k steps of 32; a k step is FB
// groups of four products that share one W fragment.  The W fragments come from LDS through a ring of four, three
// groups ahead of their use; the A fragments of a k step are read during the one before.  The barrier stands in
// front of the group behind which no fragment of the tile is read any more (the ring holds the last three); behind
// it the first fragments of the next tile are read.
// ---------------------------------------------------------------------------
template <int EPI, int TN, int MAP>
__global__ __launch_bounds__(512, 1) void gemm_ring16_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                             void* __restrict__ Cv, int M, int N, int K, int H,
                                                             int n_tile0, int n_tiles, float* __restrict__ partial,
                                                             int tiles_per_slice) {
  constexpr int TM = RING_TM, NW = 8, NWM = 4, NWN = 2, WM = TM / NWM, WN = TN / NWN, FA = WM / 16, FB = WN / 16;
  constexpr int DA = (TM / 8) / NW, DW = (TN / 8) / NW;     // DMA instructions (8 rows each) a wave and slot
  constexpr int DA1 = DA / 2, DW1 = (DW + 1) / 2;           // of them in the first of the two quarters that issue them
  constexpr int RB = 4;                                     // the ring of W fragments
  constexpr int NG = 2 * FB;                                // groups a tile
  constexpr int GB = NG - (RB - 1);                         // the barrier stands in front of this group
  constexpr int QG = NG / 4;                                // groups a quarter of the tile (the DMA's timetable)
  constexpr int G3 = GB > 3 * QG ? GB : 3 * QG;             // the first group of the last quarter behind the barrier
  static_assert(FA == 4 && NG % RB == 0 && NG % 4 == 0, "64 rows a wave; the ring goes round whole times a tile");
  static_assert(2 * QG <= GB && NG - G3 >= 1, "W(kt + 2) is issued in front of the barrier, half of A(kt + 2) behind it");
  static_assert(!gated(EPI) || FB % 2 == 0, "the gated epilogue pairs column tiles");
  extern __shared__ __attribute__((aligned(1024))) unsigned char stages[];
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int wm = wave / NWN, wn = wave % NWN;
  const int l16 = lane % 16, lq = lane / 16;
  int tile_m, tile_n;
  if (MAP == 0) {
    tile_m = blockIdx.y;
    tile_n = blockIdx.x + n_tile0;
  } else {                                                  // blocks of tiles for every XCD, as in gemm_ring_kernel
    const int mt = (M + TM - 1) / TM, T = mt * n_tiles, chunk = (T + 7) / 8;
    const int L = blockIdx.x, t = (L % 8) * chunk + L / 8;
    if (t >= T || L / 8 >= chunk) return;
    const int per_group = mt * MAP, g = t / per_group, r = t % per_group;
    const int width = min(MAP, n_tiles - g * MAP);
    tile_n = n_tile0 + g * MAP + r % width;
    tile_m = r / width;
  }
  const int m0 = tile_m * TM, n0 = tile_n * TN;
  const int slice = MAP == 0 ? blockIdx.z : blockIdx.y, n_slices = MAP == 0 ? gridDim.z : gridDim.y;
  const int kt0 = slice * tiles_per_slice;
  const int nk = min(K / TK - kt0, tiles_per_slice);

  unsigned off_a[DA], off_w[DW];
  const char* a_base = (const char*)(A + (size_t)m0 * K + (size_t)kt0 * TK);
  const char* w_base = (const char*)(W + (size_t)n0 * K + (size_t)kt0 * TK);
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int row = (i * NW + wave) * RPI + lane / CPR;
    off_a[i] = (unsigned)(((size_t)min(row, M - 1 - m0) * K + ((lane % CPR) ^ swizzle_of(row)) * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < DW; ++i) {
    const int row = (i * NW + wave) * RPI + lane / CPR;
    off_w[i] = (unsigned)(((size_t)min(row, N - 1 - n0) * K + ((lane % CPR) ^ swizzle_of(row)) * 8) * 2);
  }
  // the LDS address of this wave's first row block of a slot (scalar); instruction i lies i * 8 KB further
  const unsigned lds0 = (unsigned)(uintptr_t)stages + (unsigned)(wave * 1024);
  auto slot_addr = [&](int slot) { return lds0 + (unsigned)slot * RING_SLOT; };
  auto dma = [&](const char* base, unsigned off, unsigned lds_slot, int i) {
    const unsigned add = (unsigned)(i * NW * 1024);
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 : : "s"(lds_slot), "v"(off), "s"(base), "s"(add) : "memory", "m0", "scc");
  };

  f32x4 acc[FA][FB];
#pragma unroll
  for (int a = 0; a < FA; ++a)
#pragma unroll
    for (int b = 0; b < FB; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // fragments (operand rows = lane % 16, 8 k at k offset 8 * (lane / 16)): address in a slot row * 128 +
  // ((4 s + lq) ^ swizzle) * 16 for k step s; tiles 16 rows apart share the swizzle
  const int a_row = wm * WM + l16, w_row = wn * WN + l16;
  int a_at[2], w_at[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    a_at[s] = a_row * ROWB + (((4 * s + lq) ^ swizzle_of(a_row)) << 4);
    w_at[s] = w_row * ROWB + (((4 * s + lq) ^ swizzle_of(w_row)) << 4);
  }
  auto frag_a = [&](int slot, int s, int a) {
    return *reinterpret_cast<const bf16x8*>(stages + slot * RING_SLOT + a_at[s] + a * 16 * ROWB);
  };
  auto frag_w = [&](int slot, int s, int b) {
    return *reinterpret_cast<const bf16x8*>(stages + slot * RING_SLOT + w_at[s] + b * 16 * ROWB);
  };

  // before the loop: W0 A0 W1 and the first half of A1 (what iterations -2 and -1 would have issued)
#pragma unroll
  for (int i = 0; i < DW; ++i) dma(w_base, off_w[i], slot_addr(0), i);
#pragma unroll
  for (int i = 0; i < DA; ++i) dma(a_base, off_a[i], slot_addr(1), i);
  if (nk > 1) {
#pragma unroll
    for (int i = 0; i < DW; ++i) dma(w_base + ROWB, off_w[i], slot_addr(2), i);
#pragma unroll
    for (int i = 0; i < DA1; ++i) dma(a_base + ROWB, off_a[i], slot_addr(3), i);
    wait_vmcnt<DW + DA1>();
  } else {
    wait_vmcnt<0>();
  }
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 fa[2][FA], fb[RB];
#pragma unroll
  for (int a = 0; a < FA; ++a) fa[0][a] = frag_a(1, 0, a);
#pragma unroll
  for (int g = 0; g < RB - 1; ++g) fb[g] = frag_w(0, g / FB, g % FB);

  int ws = 0, as = 1;                              // slots of the tile that is multiplied
  // one k tile; T1 / T2: tiles kt + 1 / kt + 2 exist (the loop's last two iterations stand apart, so that the
  // others carry no branch)
  auto iteration = [&](int kt, auto t1_, auto t2_) {
    constexpr bool T1 = decltype(t1_)::value, T2 = decltype(t2_)::value;
    const int ws1 = ws + 2 >= RING_SLOTS ? ws + 2 - RING_SLOTS : ws + 2;          // of tile kt + 1
    const int as1 = as + 2 >= RING_SLOTS ? as + 2 - RING_SLOTS : as + 2;
    const int ws2 = ws1 + 2 >= RING_SLOTS ? ws1 + 2 - RING_SLOTS : ws1 + 2;       // of tile kt + 2
    const int as2 = as1 + 2 >= RING_SLOTS ? as1 + 2 - RING_SLOTS : as1 + 2;
    const unsigned l_as1 = slot_addr(as1), l_ws2 = slot_addr(ws2), l_as2 = slot_addr(as2);
    const char* a1 = a_base + (size_t)(kt + 1) * ROWB;
    const char* a2 = a_base + (size_t)(kt + 2) * ROWB;
    const char* w2 = w_base + (size_t)(kt + 2) * ROWB;
#pragma unroll
    for (int g = 0; g < NG; ++g) {                 // group g: W fragment b of k step s against the four A fragments
      const int s = g / FB, b = g % FB;
      if (g == GB) {
        // No fragment of tile kt is read from here on; this wave's share of tile kt + 1 has landed (W(kt + 2) may
        // still be on its way).  Behind the barrier that holds for all waves.
        wait_lgkmcnt0();
        if (T2) wait_vmcnt<DW>(); else wait_vmcnt<0>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int a = 0; a < FA; ++a) {
        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[s][a], fb[g % RB], acc[a][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (a == 0) {                                // the W fragment RB - 1 groups ahead (behind the barrier: of the next tile;
          const int gn = g + RB - 1;                 // behind the last tile: read, never used)
          if (gn < NG) fb[gn % RB] = frag_w(ws, gn / FB, gn % FB);
          else fb[gn % RB] = frag_w(ws1, (gn - NG) / FB, (gn - NG) % FB);
        }
        if (a == 2 && s == 0 && b >= FB - FA)        // the A fragments of k step 1, in the last four groups of k step 0
          fa[1][b - (FB - FA)] = frag_a(as, 1, b - (FB - FA));
        if (a >= 2 && g >= GB && (g - GB) * 2 + (a - 2) < FA)      // those of the next tile behind the barrier, two a group
          fa[0][(g - GB) * 2 + (a - 2)] = frag_a(as1, 0, (g - GB) * 2 + (a - 2));
        // DMA by quarters of the tile: the second half of A(kt + 1); W(kt + 2) in two halves; behind the barrier the
        // first half of A(kt + 2); behind the second and the fourth product of a group
        if (a == 1 || a == 3) {
          const int q = g / QG, d = (g % QG) * 2 + (a == 3);
          if (q == 0) { if (T1 && d < DA - DA1) dma(a1, off_a[DA1 + d], l_as1, DA1 + d); }
          else if (q == 1) { if (T2 && d < DW1) dma(w2, off_w[d], l_ws2, d); }
          else if (q == 2) { if (T2 && d < DW - DW1) dma(w2, off_w[DW1 + d], l_ws2, DW1 + d); }
          if (g >= G3) {
            const int d2 = (g - G3) * 2 + (a == 3);
            if (T2 && d2 < DA1) dma(a2, off_a[d2], l_as2, d2);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    ws = ws1;
    as = as1;
  };
  int kt = 0;
  for (; kt + 2 < nk; ++kt) iteration(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < nk) { iteration(kt, std::true_type{}, std::false_type{}); ++kt; }
  if (kt < nk) iteration(kt, std::false_type{}, std::false_type{});
  wait_vmcnt<0>();                                 // nothing of this workgroup is on its way into LDS when it ends

  // C: lane (lq, l16) holds rows 4 lq .. 4 lq + 3 of column l16 of every tile
  if (n_slices > 1) {                              // a slice of K: the plain sums, column n = weight row n
    float* plane = partial + (size_t)slice * M * N;
#pragma unroll
    for (int a = 0; a < FA; ++a)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + wm * WM + a * 16 + 4 * lq + r;
        if (m >= M) continue;
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int nn = n0 + wn * WN + b * 16 + l16;
          if (nn < N) plane[(size_t)m * N + nn] = acc[a][b][r];
        }
      }
    return;
  }
#pragma unroll
  for (int a = 0; a < FA; ++a) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + wm * WM + a * 16 + 4 * lq + r;
      if (m >= M) continue;
      if (gated(EPI)) {                              // weight rows: 16 gate rows, 16 up rows, ...: even tiles gate, odd tiles up
#pragma unroll
        for (int pp = 0; pp < FB / 2; ++pp) {
          const int hcol = (n0 + wn * WN) / 2 + pp * 16 + l16;
          if (hcol < H)
            ((bf16*)Cv)[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(acc[a][2 * pp][r]) * acc[a][2 * pp + 1][r]);
        }
      } else {
#pragma unroll
        for (int b = 0; b < FB; ++b) {
          const int nn = n0 + wn * WN + b * 16 + l16;
          if (nn >= N) continue;
          const size_t o = (size_t)m * N + nn;
          if (EPI == 0) ((float*)Cv)[o] = acc[a][b][r];
          if (EPI == 1) ((bf16*)Cv)[o] = static_cast<bf16>(acc[a][b][r]);
          if (EPI == 2) ((float*)Cv)[o] += acc[a][b][r];
        }
      }
    }
  }
}

// column tiles n_tile0 ... n_tile0 + n_tiles - 1 (n_tiles < 0: to the last) of a 256 x TN tiling
// (slices > 1: the slices of K go to `partial` as [slices][M][N], unadded)
template <int EPI, int TN, int MAP>
int launch_ring(const bf16* A, const bf16* W, void* C, int M, int N, int K, int H, hipStream_t stream, int n_tile0 = 0,
                int n_tiles = -1, float* partial = nullptr, int slices = 1) {
  if (n_tiles < 0) n_tiles = ceil_div(N, TN) - n_tile0;
  const int mt = ceil_div(M, RING_TM);
  const int tiles_per_slice = ceil_div(K / TK, slices);
  slices = ceil_div(K / TK, tiles_per_slice);
  const dim3 grid = MAP == 0 ? dim3(n_tiles, mt, slices) : dim3(8 * ceil_div(mt * n_tiles, 8), slices, 1);
  const size_t lds = (size_t)RING_SLOTS * RING_SLOT;
  // tiles of 256 and 192 columns: the kernel with the 16x16x32 products; of 128: the one with 32x32x16
  void (*kernel)(const bf16*, const bf16*, void*, int, int, int, int, int, int, float*, int);
  if constexpr (TN == 128) kernel = &gemm_ring_kernel<EPI, TN, MAP>;
  else kernel = &gemm_ring16_kernel<EPI, TN, MAP>;
  static LdsAllowance allowed;                     // more than 64 KB of LDS has to be asked for once a device
  if (int rc = allow_dynamic_lds(allowed, (const void*)kernel, (int)lds); rc != YALM_OK) return rc;
  kernel<<<grid, 512, lds, stream>>>(A, W, C, M, N, K, H, n_tile0, n_tiles, partial, tiles_per_slice);
  return launch_status();
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

// Which kernel takes a shape.  160 rows and more (prompt steps, big decode batches) go to the ring kernel; fewer
// to 128x128 tiles with K split over workgroups (a layer's four products at 160 / 256 / 383 rows: 161 / 170 /
// 250 us against 182 / 180 / 259).
bool takes_ring(int M) { return M >= 160; }

// What a prompt step's GEMM is launched as: the tile width, the slices of K, and whether whole rounds of 256x256
// tiles are followed by a second launch of 256x128 tiles for the remaining columns.
struct RingPlan {
  int tn = 256, slices = 1, nt_main = 0;         // nt_main > 0: two launches, the first over nt_main tile columns
};

// Estimated time in us of `tiles` workgroups of `iters` k tiles each.  An iteration of a 256x256 tile takes about
// 1.47 us with all CUs at work, of a tile of 192 columns 1.30 and of 128 columns 1.00 (8,192 x 4,096 x 14,336: 329,
// 291 and 225 us a round of 224 iterations); a last round on the fraction f of the CUs
// costs about 0.55 + 0.45 f of a full one (the chip clocks higher with fewer CUs at work); a workgroup's first loads
// and its epilogue take some 6 us.
double ring_time(long tiles, int iters, int tn) {
  const double per_iter = tn == 256 ? 1.47 : (tn == 192 ? 1.30 : 1.00);
  const long rounds = tiles / 256, rest = tiles % 256;
  const double f = (double)rest / 256.0;
  return ((double)rounds + (rest ? 0.55 + 0.45 * f : 0.0)) * iters * per_iter + 6.0;
}

// Splits K where the tiles alone leave most CUs without work (short prompts, narrow outputs): a second kernel then
// adds the slices (about (slices + 2) * M * N * 4 bytes at 4 TB/s).  residual: the product is added to the float32
// residual stream.  Unsplit, the tiles read and write that stream in their epilogue, M * N * 8 bytes that no loop
// hides (2,048 x 4,096 x 4,096 on tiles of 128 columns: 87 us, the same tiles with the gated epilogue 65); split,
// the kernel that adds the slices also does the norm behind them, whose own pass (M * N * 6 bytes) is saved.
// consumer: who takes the product.  RING_PLAIN: the epilogue, or a kernel that adds the slices; RING_RESIDUAL:
// as described above; RING_READER: a kernel that reads the product anyway adds the slices as it reads (the
// rotation kernel behind q/k/v), a slice more is M * N * 4 bytes more for it to read.
enum { RING_PLAIN = 0, RING_RESIDUAL = 1, RING_READER = 2 };
RingPlan ring_plan(int M, int N, int K, long workspace_floats, int consumer) {
  const bool residual = consumer == RING_RESIDUAL;
  const int mt = ceil_div(M, 256), nk = K / TK;
  RingPlan best;
  double best_t = 1e30;
  const double in_epilogue = residual ? (double)M * N * 8.0 / 4.0e6 : 0.0;
  const double norm_saved = residual ? (double)M * N * 6.0 / 5.0e6 : 0.0;
  for (int tn : {256, 192, 128}) {
    const long tiles = (long)mt * ceil_div(N, tn);
    for (int s = 1; s <= 8; s *= 2) {
      if (s > 1 && (tiles * s > 256 || nk / s < 8 || (long)s * M * N > workspace_floats)) break;
      const int iters = ceil_div(nk, s);
      const double adding = consumer == RING_READER ? (double)(s - 1) * M * N * 4.0 / 5.0e6
                                                    : 3.0 + (double)(s + 2) * M * N * 4.0 / 4.0e6 - norm_saved;
      const double t = ring_time(tiles * s, iters, tn) + (s > 1 ? adding : in_epilogue);
      if (t < best_t) { best_t = t; best.tn = tn; best.slices = s; best.nt_main = 0; }
    }
  }
  const int nt = ceil_div(N, 256);
  const int nt_main = (int)(((long)mt * nt / 256) * 256 / mt);
  if (nt_main > 0 && nt_main < nt) {
    const double t = ring_time((long)mt * nt_main, nk, 256) +
                     ring_time((long)mt * (ceil_div(N, 128) - 2 * nt_main), nk, 128) + in_epilogue;
    if (t < best_t) { best_t = t; best.tn = 256; best.slices = 1; best.nt_main = nt_main; }
  }
  return best;
}

// partial: scratch for the slices of K (the plan was made with its size); with always_partial the product's slices
// stay there unadded (one slice: the product itself), *slices_out says how many
template <int EPI>
int launch_ring_shape(const bf16* A, const bf16* W, void* C, float* partial, long partial_floats, int M, int N, int K,
                      int H, hipStream_t stream, int* slices_out = nullptr,
                      int consumer = EPI == 2 ? RING_RESIDUAL : RING_PLAIN) {
  const bool keep = slices_out != nullptr;
  const RingPlan p = ring_plan(M, N, K, partial != nullptr ? partial_floats : 0, consumer);
  if (p.nt_main > 0) {
    if (keep) *slices_out = 1;
    int rc = launch_ring<EPI, 256, 4>(A, W, C, M, N, K, H, stream, 0, p.nt_main);
    if (rc != YALM_OK) return rc;
    return launch_ring<EPI, 128, 4>(A, W, C, M, N, K, H, stream, 2 * p.nt_main);
  }
  int slices = p.slices;
  if (slices > 1) {                                // what the launch makes of it
    const int per = ceil_div(K / TK, slices);
    slices = ceil_div(K / TK, per);
  }
  if (keep) *slices_out = slices;
  int rc;
  if (p.tn == 192) {
    rc = launch_ring<EPI, 192, 0>(A, W, C, M, N, K, H, stream, 0, -1, partial, slices);
  } else if (p.tn == 128) {
    rc = launch_ring<EPI, 128, 4>(A, W, C, M, N, K, H, stream, 0, -1, partial, slices);
  } else {
    rc = launch_ring<EPI, 256, 4>(A, W, C, M, N, K, H, stream, 0, -1, partial, slices);
  }
  if (rc != YALM_OK || slices == 1 || keep) return rc;
  return yalm_splitk_reduce(partial, C, M, N, H, slices, EPI, stream);
}

template <int EPI>
int launch(const bf16* A, const bf16* W, void* C, float* ws, long ws_floats, int M, int N, int K, int H,
           hipStream_t stream) {
  if (takes_ring(M)) return launch_ring_shape<EPI>(A, W, C, ws, ws_floats, M, N, K, H, stream);
  const int slices = ws != nullptr ? slices_for(M, N, K, ws_floats) : 1;
  return launch_shape<EPI, 128, 128, 2, 2, 2, 2>(A, W, C, M, N, K, H, ws, slices, stream);
}

}  // namespace

// floats of scratch with which yalm_gemm_bf16_dma would split K (0: it would not) as a product that is added to
// the residual stream; other products split as much or less
long yalm_gemm_bf16_dma_workspace(int M, int N, int K) {
  if (M <= 64 || K < TK || K % TK != 0) return 0;
  if (takes_ring(M)) {
    const int s = max(ring_plan(M, N, K, (long)1 << 40, RING_RESIDUAL).slices,
                      ring_plan(M, N, K, (long)1 << 40, RING_READER).slices);
    return s > 1 ? (long)s * M * N : 0;
  }
  const int slices = slices_for(M, N, K, (long)1 << 40);
  return slices > 1 ? (long)slices * M * N : 0;
}

// The product's K slices, left unadded, as [*slices][M][N] float32 in the workspace (one slice: the product
// itself), for a consumer that adds them.  More than 64 rows, K a multiple of 64, at least M * N floats.
// residual: the consumer adds them to the residual stream; else it is a kernel that reads the product anyway
// (see ring_plan).
int yalm_gemm_bf16_dma_partial(const void* A, const void* W, float* workspace, long workspace_floats, int M, int N,
                               int K, int* slices_out, int residual, hipStream_t stream) {
  if (M <= 64 || K < TK || K % TK != 0 || ((uintptr_t)A & 15) || ((uintptr_t)W & 15) || workspace == nullptr ||
      workspace_floats < (long)M * N || slices_out == nullptr)
    return YALM_ERR_ARG;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if (takes_ring(M)) {              // one slice: the ring kernel stores the product itself, to the workspace
    const int consumer = residual ? RING_RESIDUAL : RING_READER;
    const RingPlan p = ring_plan(M, N, K, workspace_floats, consumer);
    if (p.slices == 1) {
      *slices_out = 1;
      return launch_ring_shape<0>(a, w, workspace, nullptr, 0, M, N, K, 0, stream);
    }
    return launch_ring_shape<0>(a, w, nullptr, workspace, workspace_floats, M, N, K, 0, stream, slices_out,
                                consumer);
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
    case 5: return launch<5>(a, w, C, workspace, workspace_floats, M, N, K, H, stream);
  }
  return YALM_ERR_ARG;
}
