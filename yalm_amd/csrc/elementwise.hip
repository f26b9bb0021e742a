// Embedding gather, RMSNorm and the fused rotation + cache write.
#include "common.h"
#include "yalm_hip.h"

// ---------------------------------------------------------------------------
// embedding
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ out,
                             int D, int V) {
  int t = blockIdx.x;
  int tok = tokens[t];
  float* o = out + (size_t)t * D;
  if (tok < 0 || tok >= V) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + (size_t)tok * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = to_f32(row[i]);
}

extern "C" int yalm_embed(const void* table, int table_dtype, const int* tokens, float* out, int T, int D, int V,
                          hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || V <= 0) return YALM_ERR_ARG;
  int threads = D >= 1024 ? 1024 : (D >= 256 ? 256 : 64);
  if (table_dtype == YALM_F32)
    embed_kernel<float><<<T, threads, 0, stream>>>((const float*)table, tokens, out, D, V);
  else if (table_dtype == YALM_BF16)
    embed_kernel<bf16><<<T, threads, 0, stream>>>((const bf16*)table, tokens, out, D, V);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

// ---------------------------------------------------------------------------
// RMSNorm: one block per row, sum of squares in float32
// ---------------------------------------------------------------------------
template <typename TW, typename TO, int NW>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w, TO* __restrict__ out,
                               const int* __restrict__ row_index, int D, float eps) {
  __shared__ float red[NW];
  int r = blockIdx.x;
  int src = row_index ? row_index[r] : r;
  TO* o = out + (size_t)r * D;
  if (src < 0) {
    for (int i = threadIdx.x; i < D; i += NW * WAVE) o[i] = from_f32<TO>(0.f);
    return;
  }
  const float* xr = x + (size_t)src * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += NW * WAVE) {
    float v = xr[i];
    ss += v * v;
  }
  ss = block_sum<NW>(ss, red);
  float scale = 1.0f / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += NW * WAVE) o[i] = from_f32<TO>(xr[i] * scale * to_f32(w[i]));
}

template <typename TW, typename TO>
static int rmsnorm_launch(const float* x, const void* w, void* out, const int* row_index, int R, int D, float eps,
                          hipStream_t stream) {
  if (D > 1024)
    rmsnorm_kernel<TW, TO, 4><<<R, 256, 0, stream>>>(x, (const TW*)w, (TO*)out, row_index, D, eps);
  else
    rmsnorm_kernel<TW, TO, 1><<<R, 64, 0, stream>>>(x, (const TW*)w, (TO*)out, row_index, D, eps);
  return launch_status();
}

extern "C" int yalm_rmsnorm(const float* x, const void* w, int w_dtype, void* out, int out_dtype,
                            const int* row_index, int R, int D, float eps, hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (D <= 0) return YALM_ERR_ARG;
  if (w_dtype == YALM_F32 && out_dtype == YALM_F32) return rmsnorm_launch<float, float>(x, w, out, row_index, R, D, eps, stream);
  if (w_dtype == YALM_F32 && out_dtype == YALM_BF16) return rmsnorm_launch<float, bf16>(x, w, out, row_index, R, D, eps, stream);
  if (w_dtype == YALM_BF16 && out_dtype == YALM_F32) return rmsnorm_launch<bf16, float>(x, w, out, row_index, R, D, eps, stream);
  if (w_dtype == YALM_BF16 && out_dtype == YALM_BF16) return rmsnorm_launch<bf16, bf16>(x, w, out, row_index, R, D, eps, stream);
  return YALM_ERR_DTYPE;
}

// ---------------------------------------------------------------------------
// rotation of q and k + write of k and v into the pages of the cache
// grid (T, n_heads + 2 n_kv_heads); one wave per (token, head); a lane per pair
// ---------------------------------------------------------------------------
template <typename T>
__global__ void rope_kv_write_kernel(const float* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_stage,
                                     T* __restrict__ v_stage, const int* __restrict__ seq_tile0,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const int* __restrict__ block_table, int table_stride, int ring_pages,
                                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                     const int* __restrict__ seq_slot, const int* __restrict__ seq_len,
                                     const float2* __restrict__ cos_sin, int n_positions, int n_heads,
                                     int n_kv_heads, int hd, int rotary_dim, int n_pages) {
  int t = blockIdx.x;
  int job = blockIdx.y;
  int pos = tok_pos[t];
  int Q = n_heads * hd, KV = n_kv_heads * hd;
  const float* row = qkv + (size_t)t * (Q + 2 * KV);
  int half_rot = rotary_dim / 2;
  bool rotate = cos_sin != nullptr && pos >= 0 && pos < n_positions;
  const float2* cs = rotate ? cos_sin + (size_t)pos * half_rot : nullptr;

  if (job < n_heads) {                       // a query head
    const float* src = row + job * hd;
    T* dst = q_out + (size_t)t * Q + job * hd;
    for (int p = threadIdx.x; p < hd / 2; p += WAVE) {
      float x0 = src[2 * p], x1 = src[2 * p + 1];
      if (rotate && p < half_rot) {
        float2 c = cs[p];
        float y0 = x0 * c.x - x1 * c.y;
        float y1 = x0 * c.y + x1 * c.x;
        x0 = y0;
        x1 = y1;
      }
      dst[2 * p] = from_f32<T>(x0);
      dst[2 * p + 1] = from_f32<T>(x1);
    }
    return;
  }

  // where this token's key and value go in the cache (or nowhere)
  int b = tok_seq[t];
  int slot = b >= 0 ? seq_slot[b] : -1;
  T* kpage = nullptr;
  T* vpage = nullptr;
  int g = (job - n_heads) % n_kv_heads;
  bool is_k = (job - n_heads) < n_kv_heads;
  int r = pos & (PAGE - 1);
  if (slot >= 0 && pos >= 0 && k_pages != nullptr) {
    int ap = pos / PAGE;
    int last_ap = (seq_len[b] - 1) / PAGE;
    if (ap > last_ap - ring_pages) {
      int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys >= 0 && phys < n_pages) {
        kpage = k_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
        vpage = v_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
      }
    }
  }

  // the step's own keys and values, in page format, for attention over the step's tokens
  T* kst = nullptr;
  T* vst = nullptr;
  if (k_stage != nullptr && b >= 0 && pos >= 0) {
    size_t tile = (size_t)seq_tile0[b] + pos / PAGE;
    kst = k_stage + (tile * n_kv_heads + g) * PAGE * hd;
    vst = v_stage + (tile * n_kv_heads + g) * PAGE * hd;
  }

  if (is_k) {
    const float* src = row + Q + g * hd;
    for (int p = threadIdx.x; p < hd / 2; p += WAVE) {
      float x0 = src[2 * p], x1 = src[2 * p + 1];
      if (rotate && p < half_rot) {
        float2 c = cs[p];
        float y0 = x0 * c.x - x1 * c.y;
        float y1 = x0 * c.y + x1 * c.x;
        x0 = y0;
        x1 = y1;
      }
      T a = from_f32<T>(x0), bb = from_f32<T>(x1);
      if (kst) {
        kst[r * hd + 2 * p] = a;
        kst[r * hd + 2 * p + 1] = bb;
      }
      if (kpage) {
        kpage[r * hd + 2 * p] = a;
        kpage[r * hd + 2 * p + 1] = bb;
      }
    }
  } else {
    const float* src = row + Q + KV + g * hd;
    for (int i = threadIdx.x; i < hd; i += WAVE) {
      T a = from_f32<T>(src[i]);
      if (vst) vst[(size_t)i * PAGE + r] = a;
      if (vpage) vpage[(size_t)i * PAGE + r] = a;      // values are kept transposed inside a page
    }
  }
}

extern "C" int yalm_rope_kv_write(const float* qkv, void* q_out, void* k_stage, void* v_stage,
                                  const int* seq_tile0, void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages,
                                  const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_len,
                                  const float* cos_sin, int n_positions, int T, int n_heads, int n_kv_heads,
                                  int head_dim, int rotary_dim, int n_pages, int dtype, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (head_dim <= 0 || (head_dim & 1) || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > head_dim ||
      n_heads <= 0 || n_kv_heads <= 0 || ring_pages <= 0)
    return YALM_ERR_ARG;
  dim3 grid(T, n_heads + 2 * n_kv_heads);
  if (dtype == YALM_F32)
    rope_kv_write_kernel<float><<<grid, WAVE, 0, stream>>>(
        qkv, (float*)q_out, (float*)k_stage, (float*)v_stage, seq_tile0, (float*)k_pages, (float*)v_pages, block_table,
        table_stride, ring_pages, tok_seq, tok_pos, seq_slot, seq_len, (const float2*)cos_sin, n_positions, n_heads,
        n_kv_heads, head_dim, rotary_dim, n_pages);
  else if (dtype == YALM_BF16)
    rope_kv_write_kernel<bf16><<<grid, WAVE, 0, stream>>>(
        qkv, (bf16*)q_out, (bf16*)k_stage, (bf16*)v_stage, seq_tile0, (bf16*)k_pages, (bf16*)v_pages, block_table, table_stride,
        ring_pages, tok_seq, tok_pos, seq_slot, seq_len, (const float2*)cos_sin, n_positions, n_heads, n_kv_heads,
        head_dim, rotary_dim, n_pages);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}
