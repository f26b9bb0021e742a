// Attention sinks beside a window: what the kernels that handle them share.  A sink is one of
// the first n_sinks positions of a sequence; its key and value are kept per slot as
// [slot][kv head][sink][element], the key as it was rotated at its own position.
#pragma once
#include "common.h"

#define YALM_MAX_SINKS 16

// What a decode step's merge of the attention splits needs to take the sinks in (n_sinks 0: none).
struct SinkArgs {
  const void* q;              // [B, n_heads, hd], rotated at each token's position
  void* sink_k;               // [n_slots, n_kv_heads, n_sinks, hd]
  void* sink_v;
  const void* k_pages;        // not null: a token at a position < n_sinks stores its key and value from its page
  const void* v_pages;
  const int* block_table;
  int table_stride;
  int n_pages;
  int page_layout;            // of k_pages, v_pages
  const int* seq_slot;        // [B]
  const int* seq_len;         // [B], the new token included: its position is seq_len - 1
  const float2* cos_sin;      // (cos, sin) [n_positions, rotary_dim / 2], or null
  int n_positions;
  int n_slots;
  int n_kv_heads;
  int rotary_dim;
  int window;
  int n_sinks;
};

// copies the key and the value of row j of a page (of the given layout) into the store of `slot`; threads
// tid, tid + n_threads, ...
template <typename T>
__device__ __forceinline__ void copy_sink(const T* __restrict__ k_src, const T* __restrict__ v_src, int layout,
                                          int page, int g, int j, int slot, T* __restrict__ sink_k,
                                          T* __restrict__ sink_v, int n_kv_heads, int hd, int n_sinks, int tid,
                                          int n_threads) {
  const T* kp = k_src + ((size_t)page * n_kv_heads + g) * PAGE * hd;
  const T* vp = v_src + ((size_t)page * n_kv_heads + g) * PAGE * hd;
  T* dk = sink_k + (((size_t)slot * n_kv_heads + g) * n_sinks + j) * hd;
  T* dv = sink_v + (((size_t)slot * n_kv_heads + g) * n_sinks + j) * hd;
  for (int i = tid; i < hd; i += n_threads) {
    dk[i] = kp[page_k_offset(layout, j, i, hd)];
    dv[i] = vp[page_v_offset(layout, j, i, hd)];
  }
}

// q . turned(k) over a head, by one wave (every lane gets the sum): pairs (2p, 2p + 1) of k are turned by the
// angles of cs (the table's row of the distance; null: not turned) for p < half_rot
template <typename T>
__device__ __forceinline__ float sink_dot(const T* __restrict__ qr, const T* __restrict__ kr,
                                          const float2* __restrict__ cs, int hd, int half_rot, int lane) {
  float d = 0.f;
  for (int p = lane; p < hd / 2; p += WAVE) {
    float k0 = to_f32(kr[2 * p]), k1 = to_f32(kr[2 * p + 1]);
    if (cs != nullptr && p < half_rot) {
      const float2 c = cs[p];
      const float y0 = k0 * c.x - k1 * c.y, y1 = k0 * c.y + k1 * c.x;
      k0 = y0;
      k1 = y1;
    }
    d = fmaf(to_f32(qr[2 * p]), k0, d);
    d = fmaf(to_f32(qr[2 * p + 1]), k1, d);
  }
  return wave_sum(d);
}
