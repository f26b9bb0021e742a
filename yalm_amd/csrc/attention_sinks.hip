// Attention sinks beside a window, for a step of whole prompts: the first positions of a sequence
// stay visible after the window has moved past them.  Their keys and values live in a small
// per-slot store of their own (the ring of pages overwrites their places); a pass behind the
// attention kernel mixes them into its result with the log-sum-exp that the attention kernel left.
// Few keys (two in the reference, src/model.h:12), so a wave per (token, head) in float32 arithmetic
// does for every storage type.  (A decode step takes its sinks in where it merges the attention's
// splits, attention_simple.hip.)
#include <float.h>
#include "common.h"
#include "sinks.h"
#include "yalm_hip.h"

namespace {
constexpr int MAX_HD = 256;
constexpr int MAX_SINKS = YALM_MAX_SINKS;

// a step of whole prompts; grid (sequence, kv head, sink); a wave copies one key row and one value column
template <typename T>
__global__ __launch_bounds__(WAVE) void sink_store_kernel(const T* __restrict__ k_stage, const T* __restrict__ v_stage,
                                                          const int* __restrict__ seq_tile0,
                                                          const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_len, T* __restrict__ sink_k,
                                                          T* __restrict__ sink_v, int n_tiles, int n_slots,
                                                          int n_kv_heads, int hd, int n_sinks) {
  const int b = blockIdx.x, g = blockIdx.y, j = blockIdx.z;
  const int slot = seq_slot[b];
  if (slot < 0 || slot >= n_slots || j >= seq_len[b]) return;
  const int tile = seq_tile0[b];
  if (tile < 0 || tile >= n_tiles) return;
  copy_sink(k_stage, v_stage, YALM_PAGE_ROWS, tile, g, j, slot, sink_k, sink_v, n_kv_heads, hd, n_sinks,
            (int)threadIdx.x, WAVE);
}

// grid (token, head); lanes over the head's elements, pairs (2p, 2p + 1) in one lane
template <typename T>
__global__ __launch_bounds__(WAVE) void attn_sink_mix_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                             const float* __restrict__ src_f32,
                                                             const float* __restrict__ lse,
                                                             const T* __restrict__ sink_k,
                                                             const T* __restrict__ sink_v,
                                                             const int* __restrict__ tok_seq,
                                                             const int* __restrict__ tok_pos,
                                                             const int* __restrict__ seq_slot,
                                                             const float2* __restrict__ cos_sin, int n_positions,
                                                             int n_slots, int n_heads, int n_kv_heads, int hd,
                                                             int rotary_dim, int window, int n_sinks) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int slot = seq_slot[tok_seq[t]];
  if (slot < 0 || slot >= n_slots) return;
  const int pos = tok_pos[t];
  const int n_out = min(n_sinks, pos - window + 1);    // sinks j <= pos - window lie behind the window
  if (n_out <= 0) return;
  const int shift = max(0, pos - window - n_sinks + 1);
  const int g = h / (n_heads / n_kv_heads);
  const int half_rot = rotary_dim / 2;
  const bool turn = cos_sin != nullptr && shift > 0 && shift < n_positions;
  const T* qr = q + ((size_t)t * n_heads + h) * hd;
  T* orow = out + ((size_t)t * n_heads + h) * hd;
  const float inv = sqrtf((float)hd);

  __shared__ float w[MAX_SINKS];
  const float seen = lse[(size_t)t * n_heads + h];
  float top = seen;
  for (int j = 0; j < n_out; ++j) {
    const T* kr = sink_k + (((size_t)slot * n_kv_heads + g) * n_sinks + j) * hd;
    const float d = sink_dot(qr, kr, turn ? cos_sin + (size_t)shift * half_rot : nullptr, hd, half_rot, lane) / inv;
    if (lane == 0) w[j] = d;
    top = fmaxf(top, d);
  }
  __syncthreads();
  const float w0 = expf(seen - top);
  float denom = w0;
  for (int j = 0; j < n_out; ++j) denom += expf(w[j] - top);
  for (int i = lane; i < hd; i += WAVE) {
    // the attention's result before it was rounded to the storage type, where the caller kept it: the mixed row is
    // then rounded once, as a decode step's is
    float acc = w0 * (src_f32 != nullptr ? src_f32[((size_t)t * n_heads + h) * hd + i] : to_f32(orow[i]));
    for (int j = 0; j < n_out; ++j)
      acc = fmaf(expf(w[j] - top), to_f32(sink_v[(((size_t)slot * n_kv_heads + g) * n_sinks + j) * hd + i]), acc);
    orow[i] = from_f32<T>(acc / denom);
  }
}

bool bad_shape(int n_kv_heads, int hd, int n_sinks) {
  return n_kv_heads <= 0 || hd <= 0 || hd > MAX_HD || hd % 2 || n_sinks <= 0 || n_sinks > MAX_SINKS;
}
}  // namespace

extern "C" int yalm_sink_store(const void* k_stage, const void* v_stage, const int* seq_tile0, const int* seq_slot,
                               const int* seq_len, void* sink_k, void* sink_v, int B, int n_tiles, int n_slots,
                               int n_kv_heads, int head_dim, int n_sinks, int dtype, hipStream_t stream) {
  if (B <= 0) return YALM_OK;
  if (bad_shape(n_kv_heads, head_dim, n_sinks) || n_sinks > PAGE || n_tiles <= 0 || n_slots <= 0) return YALM_ERR_ARG;
  dim3 grid(B, n_kv_heads, n_sinks);
  if (dtype == YALM_F32)
    sink_store_kernel<float><<<grid, WAVE, 0, stream>>>((const float*)k_stage, (const float*)v_stage, seq_tile0,
                                                        seq_slot, seq_len, (float*)sink_k, (float*)sink_v, n_tiles,
                                                        n_slots, n_kv_heads, head_dim, n_sinks);
  else if (dtype == YALM_BF16)
    sink_store_kernel<bf16><<<grid, WAVE, 0, stream>>>((const bf16*)k_stage, (const bf16*)v_stage, seq_tile0,
                                                       seq_slot, seq_len, (bf16*)sink_k, (bf16*)sink_v, n_tiles,
                                                       n_slots, n_kv_heads, head_dim, n_sinks);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_attn_sink_mix(const void* q, void* out, const float* src_f32, const float* lse, const void* sink_k,
                                  const void* sink_v,
                                  const int* tok_seq, const int* tok_pos, const int* seq_slot, const float* cos_sin,
                                  int n_positions, int T, int n_slots, int n_heads, int n_kv_heads, int head_dim,
                                  int rotary_dim, int window, int n_sinks, int dtype, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (bad_shape(n_kv_heads, head_dim, n_sinks) || n_heads <= 0 || n_heads % n_kv_heads || window < n_sinks ||
      n_slots <= 0 || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2)
    return YALM_ERR_ARG;
  dim3 grid(T, n_heads);
  if (dtype == YALM_F32)
    attn_sink_mix_kernel<float><<<grid, WAVE, 0, stream>>>(
        (const float*)q, (float*)out, src_f32, lse, (const float*)sink_k, (const float*)sink_v, tok_seq, tok_pos, seq_slot,
        (const float2*)cos_sin, n_positions, n_slots, n_heads, n_kv_heads, head_dim, rotary_dim, window, n_sinks);
  else if (dtype == YALM_BF16)
    attn_sink_mix_kernel<bf16><<<grid, WAVE, 0, stream>>>(
        (const bf16*)q, (bf16*)out, src_f32, lse, (const bf16*)sink_k, (const bf16*)sink_v, tok_seq, tok_pos, seq_slot,
        (const float2*)cos_sin, n_positions, n_slots, n_heads, n_kv_heads, head_dim, rotary_dim, window, n_sinks);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}
