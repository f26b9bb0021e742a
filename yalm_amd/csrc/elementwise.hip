// Embedding gather, RMSNorm and the fused rotation + cache write.
#include <type_traits>

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

// The same with the row kept in registers between the two passes (read once, 16 bytes a load):
// D a multiple of 4, at most 256 threads x 8 x 4 elements.
constexpr int RMS_VEC_MAX = 8;
__device__ __forceinline__ void store4(float* o, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(o) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16* o, float a, float b, float c, float d) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  bf16x4 v = {static_cast<bf16>(a), static_cast<bf16>(b), static_cast<bf16>(c), static_cast<bf16>(d)};
  *reinterpret_cast<bf16x4*>(o) = v;
}
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                                          TO* __restrict__ out, const int* __restrict__ row_index,
                                                          int D, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const int src = row_index ? row_index[r] : r;
  TO* o = out + (size_t)r * D;
  const int n4 = D / 4;
  if (src < 0) {
    for (int i = threadIdx.x; i < n4; i += 256) store4(o + 4 * i, 0.f, 0.f, 0.f, 0.f);
    return;
  }
  const float4* xr = reinterpret_cast<const float4*>(x + (size_t)src * D);
  float4 v[RMS_VEC_MAX];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < RMS_VEC_MAX; ++u) {
    const int i = threadIdx.x + u * 256;
    v[u] = i < n4 ? xr[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    ss += v[u].x * v[u].x + v[u].y * v[u].y + v[u].z * v[u].z + v[u].w * v[u].w;
  }
  ss = block_sum<4>(ss, red);
  const float scale = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
  for (int u = 0; u < RMS_VEC_MAX; ++u) {
    const int i = threadIdx.x + u * 256;
    if (i >= n4) continue;
    const TW* wp = w + 4 * i;
    store4(o + 4 * i, v[u].x * scale * to_f32(wp[0]), v[u].y * scale * to_f32(wp[1]), v[u].z * scale * to_f32(wp[2]),
           v[u].w * scale * to_f32(wp[3]));
  }
}

template <typename TW, typename TO>
static int rmsnorm_launch(const float* x, const void* w, void* out, const int* row_index, int R, int D, float eps,
                          hipStream_t stream) {
  const bool vec = D % 4 == 0 && D > 1024 && D <= 256 * 4 * RMS_VEC_MAX && !((uintptr_t)x & 15) &&
                   !((uintptr_t)out & 15);
  if (vec)
    rmsnorm_vec_kernel<TW, TO><<<R, 256, 0, stream>>>(x, (const TW*)w, (TO*)out, row_index, D, eps);
  else if (D > 1024)
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

__device__ __forceinline__ void store_pair(float* dst, float a, float b) {
  *reinterpret_cast<float2*>(dst) = make_float2(a, b);
}
__device__ __forceinline__ void store_pair(bf16* dst, float a, float b) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 v = {static_cast<bf16>(a), static_cast<bf16>(b)};
  *reinterpret_cast<bf16x2*>(dst) = v;
}

// ---------------------------------------------------------------------------
// rotation of q and k + write of k and v into the pages of the cache
// grid (T, ceil((n_heads + 2 n_kv_heads) / ROPE_JOBS)); one wave per (token, head); a lane per pair
// ---------------------------------------------------------------------------
constexpr int ROPE_JOBS = 1;                     // (token, head) jobs a workgroup: a wave each
template <typename T>
__global__ __launch_bounds__(ROPE_JOBS * WAVE) void rope_kv_write_kernel(const float* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_stage,
                                     T* __restrict__ v_stage, const int* __restrict__ seq_tile0,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const int* __restrict__ block_table, int table_stride, int ring_pages,
                                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                     const int* __restrict__ seq_slot, const int* __restrict__ seq_len,
                                     const float2* __restrict__ cos_sin, int n_positions, int n_heads,
                                     int n_kv_heads, int hd, int rotary_dim, int n_pages, int page_layout, int slices,
                                     long plane) {
  // qkv may be `slices` partial products [slices][T][Q + 2 KV] of a GEMM that split K: added here, in order;
  // the loads of four slices are asked for together
  auto rd = [&](const float* p) {
    float v = p[0];
    int s = 1;
    for (; s + 4 <= slices; s += 4) {
      const float a = p[(size_t)s * plane], b = p[(size_t)(s + 1) * plane], c = p[(size_t)(s + 2) * plane],
                  d = p[(size_t)(s + 3) * plane];
      v += a; v += b; v += c; v += d;
    }
    for (; s < slices; ++s) v += p[(size_t)s * plane];
    return v;
  };
  const bool pairs_aligned = ((((uintptr_t)qkv) | ((uintptr_t)q_out)) & 7) == 0;
  auto rd2 = [&](const float* p) {                // an adjacent pair (head sizes are even)
    if (!pairs_aligned) return make_float2(rd(p), rd(p + 1));
    float2 v = *reinterpret_cast<const float2*>(p);
    int s = 1;
    for (; s + 4 <= slices; s += 4) {
      const float2 a = *reinterpret_cast<const float2*>(p + (size_t)s * plane),
                   b = *reinterpret_cast<const float2*>(p + (size_t)(s + 1) * plane),
                   c = *reinterpret_cast<const float2*>(p + (size_t)(s + 2) * plane),
                   d = *reinterpret_cast<const float2*>(p + (size_t)(s + 3) * plane);
      v.x += a.x; v.y += a.y; v.x += b.x; v.y += b.y; v.x += c.x; v.y += c.y; v.x += d.x; v.y += d.y;
    }
    for (; s < slices; ++s) {
      const float2 a = *reinterpret_cast<const float2*>(p + (size_t)s * plane);
      v.x += a.x; v.y += a.y;
    }
    return v;
  };
  const int t = blockIdx.x;
  const int job = blockIdx.y * ROPE_JOBS + threadIdx.x / WAVE;       // a wave per (token, head)
  const int lane = threadIdx.x % WAVE;
  if (job >= n_heads + 2 * n_kv_heads) return;
  int pos = tok_pos[t];
  int Q = n_heads * hd, KV = n_kv_heads * hd;
  const float* row = qkv + (size_t)t * (Q + 2 * KV);
  int half_rot = rotary_dim / 2;
  bool rotate = cos_sin != nullptr && pos >= 0 && pos < n_positions;
  const float2* cs = rotate ? cos_sin + (size_t)pos * half_rot : nullptr;

  if (job < n_heads) {                       // a query head
    const float* src = row + job * hd;
    T* dst = q_out + (size_t)t * Q + job * hd;
    for (int p = lane; p < hd / 2; p += WAVE) {
      const float2 x = rd2(src + 2 * p);
      float x0 = x.x, x1 = x.y;
      if (rotate && p < half_rot) {
        float2 c = cs[p];
        float y0 = x0 * c.x - x1 * c.y;
        float y1 = x0 * c.y + x1 * c.x;
        x0 = y0;
        x1 = y1;
      }
      if (pairs_aligned) {
        store_pair(dst + 2 * p, x0, x1);
      } else {
        dst[2 * p] = from_f32<T>(x0);
        dst[2 * p + 1] = from_f32<T>(x1);
      }
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
    for (int p = lane; p < hd / 2; p += WAVE) {
      const float2 x = rd2(src + 2 * p);
      float x0 = x.x, x1 = x.y;
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
        const int o = page_k_offset(page_layout, r, 2 * p, hd);     // a pair never straddles a block of 32
        kpage[o] = a;
        kpage[o + 1] = bb;
      }
    }
  } else {
    const float* src = row + Q + KV + g * hd;
    for (int i = lane; i < hd; i += WAVE) {
      T a = from_f32<T>(rd(src + i));
      if (vst) vst[(size_t)i * PAGE + r] = a;
      if (vpage) vpage[page_v_offset(page_layout, r, i, hd)] = a;      // values are kept transposed inside a page
    }
  }
}

// ---------------------------------------------------------------------------
// The same for whole prompts (every sequence from position 0), a workgroup per
// (64-position tile, job): job < n_kv_heads: the keys and values of one KV head, whole
// page-shaped tiles at once (the values transposed through LDS, so that staging area and
// cache page are written in 16-byte pieces); the other jobs: one query head of the tile's
// positions.  A thread takes a pair of a row at a time: 512 contiguous bytes a wave.
// ---------------------------------------------------------------------------
constexpr int VT_ROW = PAGE + 8;                  // LDS row of the transposed values (elements)


// 2 * PP consecutive values
template <int PP>
__device__ __forceinline__ void store_values(float* dst, const float* v) {
  if constexpr (PP == 2) *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
  else store_pair(dst, v[0], v[1]);
}
template <int PP>
__device__ __forceinline__ void store_values(bf16* dst, const float* v) {
  if constexpr (PP == 2) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 o = {static_cast<bf16>(v[0]), static_cast<bf16>(v[1]), static_cast<bf16>(v[2]), static_cast<bf16>(v[3])};
    *reinterpret_cast<bf16x4*>(dst) = o;
  } else {
    store_pair(dst, v[0], v[1]);
  }
}

// 2 * PP consecutive floats at `at`, or the sum of the `slices` planes that hold them as the K slices of a
// product, added in order (four loads asked for before the first is added: a slice more costs no trip to
// memory of its own)
template <int PP>
__device__ __forceinline__ void load_slices(const float* at, int slices, long plane, float* v) {
  typedef typename std::conditional<PP == 2, float4, float2>::type V;
  V x = *reinterpret_cast<const V*>(at);
  float* xs = reinterpret_cast<float*>(&x);
  for (int s = 1; s < slices; s += 4) {
    V y[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (s + u < slices) {
        y[u] = *reinterpret_cast<const V*>(at + (size_t)(s + u) * plane);
      } else {
#pragma unroll
        for (int c = 0; c < 2 * PP; ++c) reinterpret_cast<float*>(&y[u])[c] = 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int c = 0; c < 2 * PP; ++c) xs[c] += reinterpret_cast<const float*>(&y[u])[c];
  }
#pragma unroll
  for (int c = 0; c < 2 * PP; ++c) v[c] = xs[c];
}

// PP: pairs a thread takes at a time (2: 16-byte loads; head sizes that are multiples of 4)
template <typename T, int PP>
__global__ __launch_bounds__(256) void rope_kv_tiles_kernel(
    const float* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_stage, T* __restrict__ v_stage,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_tile0, T* __restrict__ k_pages,
    T* __restrict__ v_pages, const int* __restrict__ block_table, int table_stride, int ring_pages,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_len, const float2* __restrict__ cos_sin,
    int n_positions, int B, int n_heads, int n_kv_heads, int hd, int rotary_dim, int n_pages, int page_layout,
    int slices, long plane) {
  extern __shared__ __attribute__((aligned(16))) unsigned char vt_raw[];
  T* vt = reinterpret_cast<T*>(vt_raw);           // [hd][VT_ROW]
  const int gt = blockIdx.x, job = blockIdx.y, tid = threadIdx.x;
  int b = 0;
  {
    int lo = 0, hi = B - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (seq_tile0[mid] <= gt) lo = mid; else hi = mid - 1;
    }
    b = lo;
  }
  const int ap = gt - seq_tile0[b];               // page of the sequence
  const int start = cu_seqlens[b], len = cu_seqlens[b + 1] - start;
  const int p0 = ap * PAGE;
  const int rows = min(PAGE, len - p0);           // positions of this tile
  if (rows <= 0) return;
  const int Q = n_heads * hd, KV = n_kv_heads * hd, W = Q + 2 * KV;
  const int half_rot = rotary_dim / 2, pairs = hd / 2;
  const float* src0 = qkv + (size_t)(start + p0) * W;

  // qkv may come as the K slices of its product ([slices] planes of `plane` floats), added here in order
  auto rotate = [&](float* v, int pos, int p) {   // the pairs p .. p + PP - 1 of a head at position pos
#pragma unroll
    for (int u = 0; u < PP; ++u) {
      if (cos_sin != nullptr && p + u < half_rot && pos < n_positions) {
        const float2 c = cos_sin[(size_t)pos * half_rot + p + u];
        const float a = v[2 * u], b2 = v[2 * u + 1];
        v[2 * u] = a * c.x - b2 * c.y;
        v[2 * u + 1] = a * c.y + b2 * c.x;
      }
    }
  };
  const int groups = pairs / PP;

  if (job >= n_kv_heads) {                        // a query head
    const int h = job - n_kv_heads;
    for (int e = tid; e < rows * groups; e += 256) {
      const int r = e / groups, p = (e % groups) * PP;
      float v[2 * PP];
      load_slices<PP>(src0 + (size_t)r * W + h * hd + 2 * p, slices, plane, v);
      rotate(v, p0 + r, p);
      store_values<PP>(q_out + (size_t)(start + p0 + r) * Q + h * hd + 2 * p, v);
    }
    return;
  }

  const int g = job;
  T* kst = k_stage + ((size_t)gt * n_kv_heads + g) * PAGE * hd;
  T* vst = v_stage + ((size_t)gt * n_kv_heads + g) * PAGE * hd;
  T* kpage = nullptr;
  T* vpage = nullptr;
  const int slot = seq_slot[b];
  if (k_pages != nullptr && slot >= 0) {          // a page is kept iff it is among the last ring_pages of its sequence
    const int last_ap = (seq_len[b] - 1) / PAGE;
    if (ap > last_ap - ring_pages) {
      const int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys >= 0 && phys < n_pages) {
        kpage = k_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
        vpage = v_pages + ((size_t)phys * n_kv_heads + g) * PAGE * hd;
      }
    }
  }
  for (int e = tid; e < rows * groups; e += 256) {
    const int r = e / groups, p = (e % groups) * PP;
    float v[2 * PP];
    load_slices<PP>(src0 + (size_t)r * W + Q + g * hd + 2 * p, slices, plane, v);
    rotate(v, p0 + r, p);
    store_values<PP>(kst + r * hd + 2 * p, v);
    if (kpage) store_values<PP>(kpage + page_k_offset(page_layout, r, 2 * p, hd), v);   // 4 elements from a multiple of 4 lie together in either layout
    load_slices<PP>(src0 + (size_t)r * W + Q + KV + g * hd + 2 * p, slices, plane, v);
#pragma unroll
    for (int c = 0; c < 2 * PP; ++c) vt[(2 * p + c) * VT_ROW + r] = from_f32<T>(v[c]);
  }
  __syncthreads();
  // values, transposed: element i of the head is a row of 64 positions; positions behind the prompt's end get zeros
  constexpr int PER = 16 / sizeof(T);             // elements in 16 bytes
  for (int e = tid; e < hd * (PAGE / PER); e += 256) {
    const int i = e / (PAGE / PER), c0 = (e % (PAGE / PER)) * PER;
    T piece[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) piece[u] = c0 + u < rows ? vt[i * VT_ROW + c0 + u] : from_f32<T>(0.f);
    *reinterpret_cast<uint4*>(vst + (size_t)i * PAGE + c0) = *reinterpret_cast<const uint4*>(piece);
    if (vpage)       // 16 bytes of consecutive rows stay consecutive in either layout
      *reinterpret_cast<uint4*>(vpage + page_v_offset(page_layout, c0, i, hd)) = *reinterpret_cast<const uint4*>(piece);
  }
}

extern "C" int yalm_rope_kv_write_tiles(const float* qkv, void* q_out, void* k_stage, void* v_stage,
                                        const int* cu_seqlens, const int* seq_tile0, void* k_pages, void* v_pages,
                                        const int* block_table, int table_stride, int ring_pages,
                                        const int* seq_slot, const int* seq_len, const float* cos_sin,
                                        int n_positions, int T, int B, int n_tiles, int n_heads, int n_kv_heads,
                                        int head_dim, int rotary_dim, int n_pages, int page_layout, int slices,
                                        int dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0 || n_tiles <= 0) return YALM_OK;
  if (slices < 1) return YALM_ERR_ARG;
  const long plane = (long)T * (n_heads + 2 * n_kv_heads) * head_dim;
  if (head_dim <= 0 || (head_dim & 1) || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > head_dim ||
      n_heads <= 0 || n_kv_heads <= 0 || ring_pages <= 0 || k_stage == nullptr || v_stage == nullptr ||
      cu_seqlens == nullptr || seq_tile0 == nullptr || n_heads + n_kv_heads > 65535 ||
      ((n_heads + 2 * n_kv_heads) * head_dim) % 2 != 0 || !page_layout_ok(page_layout, head_dim))
    return YALM_ERR_ARG;
  const size_t esize = dtype == YALM_F32 ? 4 : 2;
  const size_t lds = (size_t)head_dim * VT_ROW * esize;
  if (lds > 64 * 1024) return YALM_ERR_ARG;
  dim3 grid(n_tiles, n_kv_heads + n_heads);
  // two pairs a thread where every address it touches is a multiple of 16 bytes (8 for bfloat16 stores)
  const bool wide = head_dim % 4 == 0 && ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)q_out & 15) == 0 &&
                    ((uintptr_t)k_stage & 15) == 0 && ((uintptr_t)k_pages & 15) == 0;
#define YALM_ROPE_TILES(T_)                                                                                         \
  do {                                                                                                              \
    if (wide)                                                                                                       \
      rope_kv_tiles_kernel<T_, 2><<<grid, 256, lds, stream>>>(                                                      \
          qkv, (T_*)q_out, (T_*)k_stage, (T_*)v_stage, cu_seqlens, seq_tile0, (T_*)k_pages, (T_*)v_pages,           \
          block_table, table_stride, ring_pages, seq_slot, seq_len, (const float2*)cos_sin, n_positions, B,         \
          n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, page_layout, slices, plane);                          \
    else                                                                                                            \
      rope_kv_tiles_kernel<T_, 1><<<grid, 256, lds, stream>>>(                                                      \
          qkv, (T_*)q_out, (T_*)k_stage, (T_*)v_stage, cu_seqlens, seq_tile0, (T_*)k_pages, (T_*)v_pages,           \
          block_table, table_stride, ring_pages, seq_slot, seq_len, (const float2*)cos_sin, n_positions, B,         \
          n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, page_layout, slices, plane);                          \
  } while (0)
  if (dtype == YALM_F32)
    YALM_ROPE_TILES(float);
  else if (dtype == YALM_BF16)
    YALM_ROPE_TILES(bf16);
  else
    return YALM_ERR_DTYPE;
#undef YALM_ROPE_TILES
  return launch_status();
}

extern "C" int yalm_rope_kv_write(const float* qkv, void* q_out, void* k_stage, void* v_stage,
                                  const int* seq_tile0, void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages,
                                  const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_len,
                                  const float* cos_sin, int n_positions, int T, int n_heads, int n_kv_heads,
                                  int head_dim, int rotary_dim, int n_pages, int page_layout, int slices, int dtype,
                                  hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (head_dim <= 0 || (head_dim & 1) || rotary_dim < 0 || (rotary_dim & 1) || rotary_dim > head_dim ||
      n_heads <= 0 || n_kv_heads <= 0 || ring_pages <= 0 || slices < 1 || !page_layout_ok(page_layout, head_dim))
    return YALM_ERR_ARG;
  const long plane = (long)T * (n_heads + 2 * n_kv_heads) * head_dim;
  dim3 grid(T, ceil_div(n_heads + 2 * n_kv_heads, ROPE_JOBS));
  if (dtype == YALM_F32)
    rope_kv_write_kernel<float><<<grid, ROPE_JOBS * WAVE, 0, stream>>>(
        qkv, (float*)q_out, (float*)k_stage, (float*)v_stage, seq_tile0, (float*)k_pages, (float*)v_pages, block_table,
        table_stride, ring_pages, tok_seq, tok_pos, seq_slot, seq_len, (const float2*)cos_sin, n_positions, n_heads,
        n_kv_heads, head_dim, rotary_dim, n_pages, page_layout, slices, plane);
  else if (dtype == YALM_BF16)
    rope_kv_write_kernel<bf16><<<grid, ROPE_JOBS * WAVE, 0, stream>>>(
        qkv, (bf16*)q_out, (bf16*)k_stage, (bf16*)v_stage, seq_tile0, (bf16*)k_pages, (bf16*)v_pages, block_table, table_stride,
        ring_pages, tok_seq, tok_pos, seq_slot, seq_len, (const float2*)cos_sin, n_positions, n_heads, n_kv_heads,
        head_dim, rotary_dim, n_pages, page_layout, slices, plane);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}
