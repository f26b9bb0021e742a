// The decode GEMM (at most 64 rows) on the matrix cores, shared by gemm_mfma.hip and
// gemm_fused.hip:  C = epilogue(row_scale * (X[M,K] * W[N,K]^T)), bfloat16 operands,
// float32 accumulation.  It is bound by the one pass over the weights.  A workgroup owns
// 16 * NT weight rows and all of K and its waves split K; the batch is the other MFMA
// operand (16 rows a tile, MT tiles); partial sums of the waves meet in LDS, then the
// epilogue runs once.  Two ways from memory to the matrix cores: with K a multiple of 64
// and one batch tile, through LDS by DMA in whole 128-byte lines (see DMA_S below); else
// straight into registers, chunks of 32 * KS, every lane 16 bytes of a weight row per load
// (the four lane groups of a row read 64 contiguous bytes).
//
// Chaining norms through the GEMMs of a decode step: a producer with the residual-add
// epilogue can also emit, for the NEXT RMSNorm, the activations bfloat16(x * w_norm) and
// the partial sums of squares of its columns; a consumer given those scales its float32
// sums by rsqrt(mean(x^2) + eps) per row.  No norm kernel runs in between, and the sums
// are added in a fixed order.
#pragma once
#include <type_traits>
#include "common.h"

namespace skinny {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 load8(const bf16* p, bool ok) {
  bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? *reinterpret_cast<const bf16x8*>(p) : z;
}
// A load that every lane makes (from an address kept inside the matrix), zeroed afterwards
// where it does not count.  Loads under a branch make the compiler wait for all loads in
// flight before the next arithmetic, which undoes the prefetch.
__device__ __forceinline__ bf16x8 load8_always(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero_unless(bf16x8 v, bool ok) {
  bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? v : z;
}

template <int N_>
__device__ __forceinline__ void skinny_wait_vmcnt() {   // vmcnt only: expcnt and lgkmcnt fields at their maxima
  __builtin_amdgcn_s_waitcnt((N_ & 0xF) | ((N_ >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

constexpr int EPI_F32 = 0, EPI_STORE = 1, EPI_ADD = 2, EPI_GATED = EPI_GATED_SILU, EPI_ROPE = 4;   // and EPI_GATED_GELU = 5

struct RopeArgs {                                // epilogue of the fused q/k/v projection
  bf16* q_out;
  bf16* k_pages;
  bf16* v_pages;
  const int* block_table;
  const int* tok_pos;
  const int* seq_slot;
  const float2* cos_sin;
  int table_stride, ring_pages, n_positions, n_heads, n_kv_heads, hd, rotary_dim, n_pages, page_layout;
};

struct ChainArgs {
  const float* ss_in;                            // [M][n_parts_in] partial sums of squares, or null: no row scale
  int n_parts_in;
  float eps;
  const float* emit_nw;                          // EPI_ADD only: float32 norm weights [N], or null
  bf16* emit_xn;                                 // [M][N] = bfloat16(x_new * emit_nw)
  float* emit_ss;                                // [M][gridDim.x] sums of squares of this workgroup's columns
  RopeArgs ra;
};

// MFMA 16x16x32: operand A = activations (row i = batch row, 8 k per lane), operand
// B = weights (column j = weight row, 8 k per lane); C[i][j]: lane (q = lane/16,
// j = lane%16) holds batch rows 4q..4q+3 of weight row j.  Which k a lane's slot
// holds is the same for both operands, so any assignment of k to slots is right;
// here step s of a chunk takes k = kc + 32 s + 8 q ... + 8.
//
// A wave multiplies TW of the workgroup's NT tiles: with TW < NT the waves form NT / TW groups, each
// with its own tiles and the chunks of K split over the waves of the group (less to keep in flight per
// wave and more waves, at the price of one more load of the activations per group).
//
// DMA_S > 0 (one batch tile, K a multiple of 64): the operands go from global memory straight into
// LDS (global_load_lds_dwordx4), every wave into a ring of DMA_S stages of its own, 64 k a stage, and
// from there to the matrix cores.  A CU can only send so many requests a clock to the second-level
// cache (measured from memory: about 37 GB/s a CU with the 64-byte row pieces that the register path's
// lanes ask for, 90 GB/s with whole 128-byte lines), and the activations' loads, though they hit that cache,
// come out of the same budget.  Here every request is a whole line: 8 lanes read the 128 bytes of
// one row, 8 rows an instruction; the 16-byte chunks of a row are XOR-swizzled by the row number in
// the global address each lane asks for, so that the fragment reads of 8 rows fall on different
// banks.  XR (8 or 16) rows of the activations are staged.  No wave waits for another before the
// partial sums meet.
//
// RW < 16 * NT (one tile a wave, DMA path): the workgroup owns RW weight rows, its last tile only the first 8 of its
// 16 (the waves of that tile ask for one instruction of weights a stage instead of two, and the tile's other columns,
// which hold whatever was in LDS, are never stored).  6,144 rows are 256 workgroups of 24, one for every compute unit,
// where 192 of 32 left a quarter of the units idle.
template <int MT, int NT, int NWAVES, int EPI, int KS, bool PREFETCH = true, int TW = NT, int DMA_S = 0, int XR = 16,
          int RW = 16 * NT>
__global__ __launch_bounds__(NWAVES * WAVE) void gemm_skinny_kernel(const bf16* __restrict__ X,
                                                                     const bf16* __restrict__ W,
                                                                     void* __restrict__ Cv, int M, int N, int K,
                                                                     int H, ChainArgs ca) {
  constexpr int KC = 32 * KS;                    // k per wave iteration
  constexpr int G = NT / TW;                     // groups of waves, each with TW tiles
  constexpr int KW = NWAVES / G;                 // waves of a group: they split K
  static_assert(NT % TW == 0 && NWAVES % G == 0, "tiles and waves divide evenly");
  static_assert(RW == 16 * NT || (RW == 16 * NT - 8 && TW == 1 && DMA_S > 0 && !gated(EPI)),
                "a last tile of 8 rows: one tile a wave, the DMA path, no gated pairs");
  __shared__ f32x4 red[NWAVES][MT * TW][WAVE];
  __shared__ float sm_scale[MT * 16];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int q = lane / 16, j = lane % 16;
  const int n0 = blockIdx.x * RW;

  const int grp = wave % G, kw = wave / G;
  const bf16* wrow[TW];
  bool wok[TW];
#pragma unroll
  for (int t = 0; t < TW; ++t) {
    int n = n0 + (grp * TW + t) * 16 + j;
    wok[t] = n < N;
    wrow[t] = W + (size_t)(wok[t] ? n : 0) * K;
  }
  const bf16* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + j;
    xok[mt] = m < M;
    xrow[mt] = X + (size_t)(xok[mt] ? m : 0) * K;
  }

  f32x4 acc[MT][TW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < TW; ++t) acc[mt][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // Workgroups start at different chunks of K (and wrap around): with all of them on the
  // same columns at the same time, the rows' 8 KB-strided pieces crowd few memory channels.
  const int n_chunks = (K + KC - 1) / KC;
  const int rot = (int)((blockIdx.x * 5u) % (unsigned)n_chunks);
  auto chunk_k = [&](int c) {
    int cc = c + rot;
    if (cc >= n_chunks) cc -= n_chunks;
    return cc * KC;
  };
  // the residual values of the epilogue's first tile are asked for now, not after the sums
  f32x4 c_old = (f32x4){0.f, 0.f, 0.f, 0.f};
  if (EPI == EPI_ADD && wave < MT * NT) {
    const int n = min(n0 + (wave % NT) * 16 + j, N - 1);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = min((wave / NT) * 16 + 4 * q + r, M - 1);
      c_old[r] = ((const float*)Cv)[(size_t)m * N + n];
    }
  }

  auto load_chunk = [&](int c, bf16x8 (&w)[TW][KS], bf16x8 (&x)[MT][KS]) {
    const int kc = chunk_k(c);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k = kc + s * 32 + q * 8;
      const bool ok = k < K;
      const int kk = ok ? k : K - 8;               // rows beyond N or M are clamped too and never stored
#pragma unroll
      for (int t = 0; t < TW; ++t) w[t][s] = load8_always(wrow[t] + kk);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) x[mt][s] = zero_unless(load8_always(xrow[mt] + kk), ok);
    }
  };
  auto row_scales = [&]() {   // from the producer's partial sums of squares (a wave per row, lanes over the parts)
    if (ca.ss_in == nullptr) return;
    for (int m = wave; m < MT * 16; m += NWAVES) {
      float s = 0.f;
      if (m < M)
        for (int p = lane; p < ca.n_parts_in; p += WAVE) s += ca.ss_in[(size_t)m * ca.n_parts_in + p];
      s = wave_sum(s);
      if (lane == 0) sm_scale[m] = 1.0f / sqrtf(s / (float)K + ca.eps);
    }
  };

  if constexpr (DMA_S > 0) {
    static_assert(MT == 1 && (XR == 8 || XR == 16) && DMA_S >= 2 && DMA_S <= 4, "one batch tile; 8 or 16 staged rows; 2..4 stages");
    constexpr int KD = 64;                         // k a stage: one 128-byte line of every row
    constexpr int XI = XR / 8;                     // DMA instructions a stage: 8 rows each
    constexpr int STAGE_B = (16 * TW + XR) * 128;
    extern __shared__ __attribute__((aligned(1024))) unsigned char dma_ring[];   // [NWAVES][DMA_S][STAGE_B]
    unsigned char* ring = dma_ring + (size_t)wave * DMA_S * STAGE_B;
    const int r8 = lane / 8, chunk = (lane % 8) ^ r8;          // this lane's row of an instruction and the chunk it asks for
    // NWI: instructions of weights a stage (8 rows each): 2 * TW, or 1 for the waves of a last tile of 8 rows
    auto run = [&](auto nwi_tag) {
    constexpr int NWI = decltype(nwi_tag)::value;
    constexpr int L = NWI + XI;
    const bf16* gw[NWI];
#pragma unroll
    for (int i = 0; i < NWI; ++i) {
      const int n = min(n0 + (grp * TW + i / 2) * 16 + (i % 2) * 8 + r8, N - 1);
      gw[i] = W + (size_t)n * K + chunk * 8;
    }
    const bf16* gx[XI];
#pragma unroll
    for (int i = 0; i < XI; ++i) gx[i] = X + (size_t)min(i * 8 + r8, M - 1) * K + chunk * 8;
    const int nd = K / KD;                         // stages in all; this wave takes kw, kw + KW, ...
    const int rotd = (int)((blockIdx.x * 5u) % (unsigned)nd);
    const int mine = kw < nd ? (nd - kw + KW - 1) / KW : 0;
    auto issue = [&](int i, int buf) {
      int c = kw + i * KW + rotd;
      if (c >= nd) c -= nd;
      unsigned char* dst = ring + buf * STAGE_B;
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass drops a template that names this builtin, and its launch stub with it
#pragma unroll
      for (int u = 0; u < NWI; ++u)
        __builtin_amdgcn_global_load_lds(gw[u] + (size_t)c * KD, dst + u * 1024, 16, 0, YALM_READ_ONCE);
#pragma unroll
      for (int u = 0; u < XI; ++u)
        __builtin_amdgcn_global_load_lds(gx[u] + (size_t)c * KD, dst + (2 * TW + u) * 1024, 16, 0, 0);
#endif
    };
#pragma unroll
    for (int i = 0; i < DMA_S - 1; ++i)
      if (i < mine) issue(i, i);
    row_scales();
    // fragment reads: lane (q, j) of step s wants chunk 4 s + q of row j, which lies at (4 s + q) ^ (j & 7)
    const int rd_w = j * 128, rd_x = (16 * TW + (j % XR)) * 128, swz = j & 7;
    int buf = 0;
    for (int i = 0; i < mine; ++i) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the fragment reads of the buffer that is filled next are done
      const int ahead = mine - 1 - i;              // stages behind this one that are (or now get) in flight
      if (ahead >= DMA_S - 1) {
        int nb = buf + DMA_S - 1;
        if (nb >= DMA_S) nb -= DMA_S;
        issue(i + DMA_S - 1, nb);
        skinny_wait_vmcnt<(DMA_S - 1) * L>();
      } else if (ahead == 2) {                     // the last stages: nothing more to ask for
        skinny_wait_vmcnt<2 * L>();
      } else if (ahead == 1) {
        skinny_wait_vmcnt<L>();
      } else {
        skinny_wait_vmcnt<0>();
      }
      asm volatile("" ::: "memory");
      const unsigned char* cur = ring + buf * STAGE_B;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int off = ((4 * s + q) ^ swz) << 4;
        const bf16x8 xf = *reinterpret_cast<const bf16x8*>(cur + rd_x + off);
#pragma unroll
        for (int t = 0; t < TW; ++t) {
          const bf16x8 wf = *reinterpret_cast<const bf16x8*>(cur + t * 2048 + rd_w + off);
          acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wf, acc[0][t], 0, 0, 0);
        }
      }
      if (++buf == DMA_S) buf = 0;
    }
    };
    if constexpr (RW < 16 * NT) {
      if (grp == G - 1)
        run(std::integral_constant<int, 1>{});
      else
        run(std::integral_constant<int, 2 * TW>{});
    } else {
      run(std::integral_constant<int, 2 * TW>{});
    }
  } else {
    bf16x8 wv[TW][KS], xv[MT][KS];
    if (!PREFETCH) {
      // few, large chunks: all loads of a chunk are in flight at once and the products
      // start as the first arrive (K <= 512 * NWAVES is one round trip to memory)
      bool first = true;
      for (int c = kw; c < n_chunks; c += KW) {
        load_chunk(c, wv, xv);
        if (first) row_scales();
        first = false;
  #pragma unroll
        for (int s = 0; s < KS; ++s)
  #pragma unroll
          for (int mt = 0; mt < MT; ++mt)
  #pragma unroll
            for (int t = 0; t < TW; ++t)
              acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv[mt][s], wv[t][s], acc[mt][t], 0, 0, 0);
      }
      if (first) row_scales();
    } else {
      int c = kw;
      if (c < n_chunks) load_chunk(c, wv, xv);
      row_scales();
      for (; c < n_chunks; c += KW) {
        bf16x8 wn[TW][KS], xn[MT][KS];
        const bool more = c + KW < n_chunks;
        if (more) load_chunk(c + KW, wn, xn);        // prefetch the wave's next chunk
  #pragma unroll
        for (int s = 0; s < KS; ++s)
  #pragma unroll
          for (int mt = 0; mt < MT; ++mt)
  #pragma unroll
            for (int t = 0; t < TW; ++t)
              acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv[mt][s], wv[t][s], acc[mt][t], 0, 0, 0);
        if (more) {
  #pragma unroll
          for (int s = 0; s < KS; ++s) {
  #pragma unroll
            for (int t = 0; t < TW; ++t) wv[t][s] = wn[t][s];
  #pragma unroll
            for (int mt = 0; mt < MT; ++mt) xv[mt][s] = xn[mt][s];
          }
        }
      }
    }

  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < TW; ++t) red[wave][mt * TW + t][lane] = acc[mt][t];
  __syncthreads();
  // tile t of the workgroup: the sums of the waves of group t / TW, in their slot t % TW
  auto tile_sum = [&](int mt, int t) {
    f32x4 v = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < KW; ++w) v += red[w * G + t / TW][mt * TW + t % TW][lane];
    return v;
  };

  const bool scaled = ca.ss_in != nullptr;
  constexpr int NTP = (gated(EPI)) ? NT / 2 : NT;  // gated: a gate tile and its up tile finish together
  for (int idx = wave; idx < MT * NTP; idx += NWAVES) {
    const int mt = idx / NTP, tp = idx % NTP;
    float scale[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) scale[r] = scaled ? sm_scale[mt * 16 + 4 * q + r] : 1.0f;
    if (gated(EPI)) {
      const f32x4 g = tile_sum(mt, 2 * tp), u = tile_sum(mt, 2 * tp + 1);
      int hcol = (n0 / 32 + tp) * 16 + j;
      bf16* C = (bf16*)Cv;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int m = mt * 16 + 4 * q + r;
        if (m < M && hcol < H)
          C[(size_t)m * H + hcol] = static_cast<bf16>(gate_act<EPI>(g[r] * scale[r]) * (u[r] * scale[r]));
      }
      continue;
    }
    f32x4 v = tile_sum(mt, tp);
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] *= scale[r];
    const int n = (tp * 16 + j < RW) ? n0 + tp * 16 + j : N;        // a column beyond the workgroup's rows counts as beyond N
    if (EPI == EPI_F32 || EPI == EPI_STORE) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int m = mt * 16 + 4 * q + r;
        if (m < M && n < N) {
          size_t o = (size_t)m * N + n;
          if (EPI == EPI_F32) ((float*)Cv)[o] = v[r];
          if (EPI == EPI_STORE) ((bf16*)Cv)[o] = static_cast<bf16>(v[r]);
        }
      }
    } else if (EPI == EPI_ADD) {
      const bool emit = ca.emit_nw != nullptr;   // NT == 1 then (the launcher sees to it)
      const float nw = (emit && n < N) ? ca.emit_nw[n] : 0.f;
      float sq[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int m = mt * 16 + 4 * q + r;
        sq[r] = 0.f;
        if (m < M && n < N) {
          size_t o = (size_t)m * N + n;
          float y = (idx == wave ? c_old[r] : ((float*)Cv)[o]) + v[r];
          ((float*)Cv)[o] = y;
          if (emit) {
            ca.emit_xn[o] = static_cast<bf16>(y * nw);
            sq[r] = y * y;
          }
        }
      }
      if (emit) {                                // sums over the 16 columns of the tile: lanes j of one lane group
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t = sq[r];
          t += __shfl_xor(t, 1, WAVE);
          t += __shfl_xor(t, 2, WAVE);
          t += __shfl_xor(t, 4, WAVE);
          t += __shfl_xor(t, 8, WAVE);
          int m = mt * 16 + 4 * q + r;
          if (j == 0 && m < M) ca.emit_ss[(size_t)m * gridDim.x + blockIdx.x] = t;
        }
      }
    } else {                                      // EPI_ROPE: n runs over [q heads | k heads | v heads]
      const RopeArgs& ra = ca.ra;
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
          const int m = mt * 16 + 4 * q + r;
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

// Up to 16 batch rows.  K a multiple of 64 goes through LDS (DMA_S > 0): wide matrices (the gated
// epilogue, or more than 4096 weight rows without a norm to prepare) in workgroups of 128, 64 or
// 32 weight rows, as many as still make some 200 workgroups; the others 16 rows and 8 waves that
// split K.  A producer of the norm chain always owns 16 rows (one emitted part a workgroup).
// Other K keep the register path (measured at 4096..32000 weight rows, K 4096 and 14336): the
// gated epilogue 32 rows and 4 waves with all loads of a 256-wide chunk in flight at once; other
// wide matrices 32 rows and 16 waves, a tile each for half of them; a long K 16 rows, 8 waves and
// 512-wide chunks; the small projections 16 rows, 8 waves and prefetched 128-wide chunks.  More
// batch rows (only when the split-K kernel refused the shape) keep 128-wide chunks for the registers.
// the LDS-DMA variant: its ring of stages is dynamic LDS, which has to be allowed once beyond 64 KB
template <int NT, int NWAVES, int EPI, int TW, int S, int XR, int RW = 16 * NT>
int launch_dma(const bf16* X, const bf16* W, void* C, int M, int N, int K, int H, const ChainArgs& ca,
               hipStream_t stream) {
  constexpr size_t lds = (size_t)NWAVES * S * (16 * TW + XR) * 128;
  static_assert(lds + NWAVES * TW * WAVE * 16 + 1024 <= 160 * 1024, "the ring and the partial sums fit the LDS of a CU");
  auto kernel = &gemm_skinny_kernel<1, NT, NWAVES, EPI, 1, false, TW, S, XR, RW>;
  static LdsAllowance allowed;                     // once a device
  if (int rc = allow_dynamic_lds(allowed, (const void*)kernel, (int)lds); rc != YALM_OK) return rc;
  kernel<<<ceil_div(N, RW), NWAVES * WAVE, lds, stream>>>(X, W, C, M, N, K, H, ca);
  return launch_status();
}

template <int MT, int EPI>
int launch_mt(const bf16* X, const bf16* W, void* C, int M, int N, int K, int H, const ChainArgs& ca,
              hipStream_t stream) {
  constexpr int E = gated(EPI) ? EPI_F32 : EPI;   // the gated epilogue needs pairs of tiles
  const bool emit = ca.emit_nw != nullptr;
  if constexpr (MT == 1) {
    if (K % 64 == 0) {                            // through LDS; measured at 8 rows against the register path:
      const bool few = M <= 8;                     // gate/up 41.9 against 52.6 us, q/k/v 11.0 against 15.3,
      if (gated(EPI) || (!emit && N > 4096 && K < 8192)) {   // down 21.3 against 25.2, o 7.0 against 8.3
        if (N >= 200 * 128)                        // workgroups of 128 weight rows while they still fill the chip
          return few ? launch_dma<8, 8, EPI, 2, 3, 8>(X, W, C, M, N, K, H, ca, stream)
                     : launch_dma<8, 8, EPI, 2, 2, 16>(X, W, C, M, N, K, H, ca, stream);
        if (N >= 200 * 64)                         // (9..16 rows: a wave with two row tiles stages the activations once
          return few ? launch_dma<4, 16, EPI, 1, 2, 8>(X, W, C, M, N, K, H, ca, stream)   // for both; gate/up at 16
                     : launch_dma<4, 8, EPI, 2, 2, 16>(X, W, C, M, N, K, H, ca, stream);  // rows 41.6 -> 37.8 us)
        if constexpr (!gated(EPI)) {
          // workgroups of 24 rows where they are at most one a compute unit (6,144 rows: 256 workgroups instead of
          // 192 of 32 rows, which leave a quarter of the chip idle)
          if (ceil_div(N, 24) <= 256)
            return few ? launch_dma<2, 16, EPI, 1, 2, 8, 24>(X, W, C, M, N, K, H, ca, stream)
                       : launch_dma<2, 16, EPI, 1, 2, 16, 24>(X, W, C, M, N, K, H, ca, stream);
        }
        return few ? launch_dma<2, 16, EPI, 1, 2, 8>(X, W, C, M, N, K, H, ca, stream)
                   : launch_dma<2, 16, EPI, 1, 2, 16>(X, W, C, M, N, K, H, ca, stream);
      }
      return few ? launch_dma<1, 8, E, 1, 3, 8>(X, W, C, M, N, K, H, ca, stream)
                 : launch_dma<1, 8, E, 1, 3, 16>(X, W, C, M, N, K, H, ca, stream);
    }
    if (gated(EPI))
      gemm_skinny_kernel<1, 2, 4, EPI, 8, false><<<ceil_div(N, 32), 4 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
    else if (!emit && N > 4096 && K < 8192)
      gemm_skinny_kernel<1, 2, 16, EPI, 8, false, 1><<<ceil_div(N, 32), 16 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
    else if (K >= 8192)
      gemm_skinny_kernel<1, 1, 8, E, 16, false><<<ceil_div(N, 16), 8 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
    else
      gemm_skinny_kernel<1, 1, 8, E, 4><<<ceil_div(N, 16), 8 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
  } else {
    const bool wide = gated(EPI) || (N >= 16384 && !emit);
    if (wide && MT <= 2)
      gemm_skinny_kernel<MT, 4, 4, EPI, 4><<<ceil_div(N, 64), 4 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
    else if (wide)
      gemm_skinny_kernel<MT, 2, 4, EPI, 4><<<ceil_div(N, 32), 4 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
    else
      gemm_skinny_kernel<MT, 1, 8, E, 4><<<ceil_div(N, 16), 8 * WAVE, 0, stream>>>(X, W, C, M, N, K, H, ca);
  }
  return launch_status();
}

template <int EPI>
int launch(const bf16* X, const bf16* W, void* C, int M, int N, int K, int H, const ChainArgs& ca,
           hipStream_t stream) {
  switch ((M + 15) / 16) {
    case 1: return launch_mt<1, EPI>(X, W, C, M, N, K, H, ca, stream);
    case 2: return launch_mt<2, EPI>(X, W, C, M, N, K, H, ca, stream);
    case 3: return launch_mt<3, EPI>(X, W, C, M, N, K, H, ca, stream);
    case 4: return launch_mt<4, EPI>(X, W, C, M, N, K, H, ca, stream);
  }
  return YALM_ERR_ARG;
}

// workgroups along N of a launch without the gated epilogue (the number of emitted parts)
inline int parts_of(int N) { return ceil_div(N, 16); }

}  // namespace skinny
