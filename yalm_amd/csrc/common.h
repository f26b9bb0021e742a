// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave64 reductions and the launch-error convention of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <mutex>

#define YALM_OK 0
#define YALM_ERR_ARG 1001          // an argument the kernel family refuses
#define YALM_ERR_DTYPE 1002        // unknown dtype code
#define YALM_ERR_SCRATCH 1003      // the sizes need more scratch than the fixed array of the entry point holds

// dtype codes shared with the Python side
#define YALM_F32 0
#define YALM_BF16 1

#define WAVE 64
#define PAGE 64                    // tokens per cache page; equals the wave width on purpose

typedef __bf16 bf16;

// Cache policy bits of a global load (the `aux` operand of the load-to-LDS builtin).  READ_ONCE marks data
// that a launch reads once and nobody reads again soon (a decode step's weights): non-temporal, so that it
// does not push out of the second-level cache what is read again (the activations).  Measured on the decode
// GEMMs: gate/up at 8 rows 41.1 -> 37.0 us (5.7 -> 6.4 TB/s), at 64 rows 53.7 -> 49.7.
#ifndef YALM_READ_ONCE
#define YALM_READ_ONCE 2
#endif

// Where the key and the value of row r (0..63) lie inside a cache page of one KV head (elements from the
// page's start).
//   YALM_PAGE_ROWS:   keys [row][element], values [element][row] (the staging area of a prompt step always).
//   YALM_PAGE_BLOCKS: head sizes that are multiples of 32.  Keys [element / 32][place(row)][element % 32],
//     place(row) being the row's place in the order in which the matrix-core decode attention takes the
//     rows of a page (16 rows an instruction: rows 8a + b (+4) (+32) for a, b < 4); values
//     [row / 32][element][row % 32].  Each of that kernel's load instructions then reads 1 KB of
//     consecutive bytes, whole 128-byte lines, instead of 16 pieces of 64 bytes.
#define YALM_PAGE_ROWS 0
#define YALM_PAGE_BLOCKS 1
__host__ __device__ __forceinline__ int page_row_place(int r) {
  return 16 * (2 * (r >> 5) + ((r >> 2) & 1)) + 4 * ((r >> 3) & 3) + (r & 3);
}
__host__ __device__ __forceinline__ int page_k_offset(int layout, int r, int e, int hd) {
  return layout == YALM_PAGE_BLOCKS ? ((e >> 5) * PAGE + page_row_place(r)) * 32 + (e & 31) : r * hd + e;
}
__host__ __device__ __forceinline__ int page_v_offset(int layout, int r, int e, int hd) {
  return layout == YALM_PAGE_BLOCKS ? ((r >> 5) * hd + e) * 32 + (r & 31) : e * PAGE + r;
}
__host__ __device__ __forceinline__ bool page_layout_ok(int layout, int hd) {
  return layout == YALM_PAGE_ROWS || (layout == YALM_PAGE_BLOCKS && hd % 32 == 0);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return static_cast<bf16>(v); }

// Epilogue codes of the GEMMs (yalm_hip.h).  The two gated ones differ in the gate's activation
// (src/infer.cpp:189-195): silu(z) = z / (1 + exp(-z)); gelu(z) = z/2 (1 + tanh(0.797885 (z + 0.044715 z^3))).
constexpr int EPI_GATED_SILU = 3, EPI_GATED_GELU = 5;
constexpr bool gated(int epilogue) { return epilogue == EPI_GATED_SILU || epilogue == EPI_GATED_GELU; }
template <int EPI>
__device__ __forceinline__ float gate_act(float z) {
  if constexpr (EPI == EPI_GATED_GELU) return 0.5f * z * (1.0f + tanhf(0.797885f * (z + 0.044715f * z * z * z)));
  return z / (1.0f + expf(-z));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of NW waves; every thread gets the result.  `red` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if (NW == 1) return v;
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) s += red[i];
  return s;
}
template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  if (NW == 1) return v;
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = v;
  __syncthreads();
  float s = red[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) s = fmaxf(s, red[i]);
  return s;
}

// More than 64 KB of dynamic LDS has to be allowed for a kernel before its first launch, on every device it is
// launched on.  One LdsAllowance (a static of the launcher) per kernel: a bit per device, set under a lock.
struct LdsAllowance {
  std::mutex lock;
  unsigned long long devices = 0;
};
static inline int allow_dynamic_lds(LdsAllowance& a, const void* kernel, int bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return YALM_ERR_ARG;
  std::lock_guard<std::mutex> hold(a.lock);
  if ((a.devices >> dev) & 1ull) return YALM_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return (int)e;
  a.devices |= 1ull << dev;
  return YALM_OK;
}

static inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? YALM_OK : (int)e;
}

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }
