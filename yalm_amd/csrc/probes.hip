// Measured peaks for the bench's roofline figures: what a kernel that only reads memory reaches, and what a
// loop of matrix-core instructions on registers reaches.  The reference prints the bandwidth of a run
// (src/main.cpp:133-147) and times single kernels at model sizes (src/test.cpp:340-405); these two loops
// give the yardsticks beside the vendor's peaks.
#include "common.h"
#include "yalm_hip.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

// Every workgroup reads whole pieces of PIECE bytes, 16 bytes a lane and instruction, 4 KB a workgroup and
// instruction, non-temporal (the data is read once); the pieces of a workgroup lie `gridDim.x` pieces apart.
// What it reads is xor-ed into one word a lane so that no load can be dropped; one word a workgroup is kept.
#define PROBE_THREADS 256
#define PROBE_UNROLL 8
__global__ __launch_bounds__(PROBE_THREADS) void probe_read_kernel(const u32x4_t* __restrict__ src, long n16,
                                                                   unsigned int* __restrict__ out) {
  const long per_pass = (long)PROBE_THREADS * PROBE_UNROLL;          // 16-byte words of a piece
  const long n_pieces = n16 / per_pass;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (long piece = blockIdx.x; piece < n_pieces; piece += gridDim.x) {
    const u32x4_t* p = src + piece * per_pass + threadIdx.x;
    u32x4_t v[PROBE_UNROLL];
#pragma unroll
    for (int u = 0; u < PROBE_UNROLL; ++u) v[u] = __builtin_nontemporal_load(p + u * PROBE_THREADS);
#pragma unroll
    for (int u = 0; u < PROBE_UNROLL; ++u) acc ^= v[u];
  }
  unsigned int w = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) w ^= __shfl_xor(w, o, WAVE);
  if ((threadIdx.x & (WAVE - 1)) == 0) atomicXor(out + (blockIdx.x & 1023), w);
}

// Eight waves a workgroup, two a SIMD; every wave keeps four independent 32x32 (or eight 16x16) accumulators
// and feeds them from registers.  The operands are small non-zero values that differ from lane to lane (the
// power the matrix cores draw, and with it the clock, depends on the data: zeros run faster than any real
// product does).
template <int SHAPE>
__global__ __launch_bounds__(512) void probe_mfma_kernel(int iters, float* __restrict__ out) {
  bf16x8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(0.001f * (float)(((threadIdx.x * 8 + i) * 37 + blockIdx.x) % 61 - 30));
    b[i] = static_cast<__bf16>(0.001f * (float)(((threadIdx.x * 8 + i) * 53 + blockIdx.x) % 59 - 29));
  }
  float sum = 0.f;
  if (SHAPE == 32) {
    f32x16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int it = 0; it < iters; ++it) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, a, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, b, c3, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) sum += c0[i] + c1[i] + c2[i] + c3[i];
  } else {
    f32x4_t c[8] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        c[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16((j & 1) ? b : a, (j & 2) ? a : b, c[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) sum += c[j][0] + c[j][1] + c[j][2] + c[j][3];
  }
  if (sum == 12345.678f) out[0] = sum;          // keeps the products alive; practically never true
}

// Reads `bytes` bytes (rounded down to whole pieces of 32 KB) of src once; `out` needs 1,024 words.
extern "C" int yalm_probe_read(const void* src, long bytes, unsigned int* out, int workgroups, hipStream_t stream) {
  if (!src || !out || bytes < (long)PROBE_THREADS * PROBE_UNROLL * 16 || workgroups < 1) return YALM_ERR_ARG;
  hipLaunchKernelGGL(probe_read_kernel, dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (const u32x4_t*)src,
                     bytes / 16, out);
  return launch_status();
}

// `iters` rounds of matrix-core instructions in each of 8 waves of `workgroups` workgroups; shape 32:
// v_mfma_f32_32x32x16_bf16 (four a round), shape 16: v_mfma_f32_16x16x32_bf16 (eight a round).  *flops
// (host memory, may be null) receives the floating-point operations of the launch.
extern "C" int yalm_probe_mfma(int shape, int iters, int workgroups, float* out, double* flops, hipStream_t stream) {
  if ((shape != 16 && shape != 32) || iters < 1 || workgroups < 1 || !out) return YALM_ERR_ARG;
  const double per_round = shape == 32 ? 4.0 * 2.0 * 32 * 32 * 16 : 8.0 * 2.0 * 16 * 16 * 32;
  if (flops) *flops = per_round * iters * 8.0 * workgroups;
  if (shape == 32)
    hipLaunchKernelGGL(probe_mfma_kernel<32>, dim3(workgroups), dim3(512), 0, stream, iters, out);
  else
    hipLaunchKernelGGL(probe_mfma_kernel<16>, dim3(workgroups), dim3(512), 0, stream, iters, out);
  return launch_status();
}
