// bfloat16 attention on the matrix cores (v_mfma_f32_16x16x32_bf16), softmax state
// in float32.  Keys are kept [row][element] and values transposed [element][row] in
// pages of 64 rows, so every operand is a 16-byte load:
//
//   scores^T[key, col] = K[key, :] . Q[col, :]     A = 16 key rows x 32 elements, B = queries
//   out^T[elem, col]  += V^T[elem, key] P^T[key, col]   A = 16 elements x 32 keys, B = P^T
//
// The C layout of the first product (a lane holds 4 consecutive rows of one column)
// feeds the second product's B operand directly: key tile t reads the page rows
// key_row(t, i), chosen so that a lane ends up with 8 consecutive keys per 32-key
// step, the same keys its 16-byte load of V^T covers.  No shuffles, no LDS.
//
// A column is a query head of the group (decode: up to 16 heads share one pass over
// the keys of their KV head) or a query position (prefill: 16 positions a wave).
#pragma once
#include <float.h>
#include <math.h>
#include <type_traits>
#include "common.h"
#include "sinks.h"
#include "yalm_hip.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr float LN2 = 0.6931471805599453f;      // the kernels' maxima are exponents of 2

__device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() { return (bf16x8){0, 0, 0, 0, 0, 0, 0, 0}; }
// a load of data that the launch reads once: non-temporal
__device__ __forceinline__ bf16x8 ld8_once(const bf16* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
}

// page row that MFMA row i (0..15) of key tile t (0..3) reads
__device__ __forceinline__ int key_row(int t, int i) { return 32 * (t >> 1) + 8 * (i >> 2) + 4 * (t & 1) + (i & 3); }

// head sizes the kernels are built for: 16 to 128 in steps of 16
bool mfma_shape_ok(int n_heads, int n_kv_heads, int head_dim) {
  return head_dim >= 16 && head_dim <= 128 && head_dim % 16 == 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0;
}

}  // namespace
