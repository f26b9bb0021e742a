// Sampling over float32 logits: argmax, temperature sampling given the uniform
// number, and the probability of one token.  One block of 1024 threads per row,
// 16-byte loads where the row's address allows them.
#include <float.h>
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int NTA = 1024;                        // argmax: 1024 threads a row

// keeps (best, arg) the first maximum: a candidate wins only if it is larger, or as large at a lower index
__device__ __forceinline__ void take(float v, int i, float& best, int& arg) {
  if (v > best || (v == best && i < arg)) {
    best = v;
    arg = i;
  }
}

// A row is read in 16-byte pieces, four of them in flight per thread; the floats in front of the
// first aligned address and behind the last whole piece go one to a thread.
__global__ __launch_bounds__(NTA) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
  __shared__ float bv[NTA / WAVE];
  __shared__ int bi[NTA / WAVE];
  const float* l = logits + (size_t)blockIdx.x * V;
  const int t = threadIdx.x;
  float best = -FLT_MAX;
  int arg = V;                                   // "none": larger than every index
  const int head = min(V, (int)((4 - ((uintptr_t)l / sizeof(float)) % 4) % 4));
  const int n4 = (V - head) / 4;
  const float4* l4 = reinterpret_cast<const float4*>(l + head);
  if (t < head) take(l[t], t, best, arg);
  for (int i = t; i < n4; i += 4 * NTA) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = l4[min(i + u * NTA, n4 - 1)];   // every load unconditional
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = i + u * NTA;
      if (j < n4) {
        const int at = head + 4 * j;
        take(v[u].x, at, best, arg);
        take(v[u].y, at + 1, best, arg);
        take(v[u].z, at + 2, best, arg);
        take(v[u].w, at + 3, best, arg);
      }
    }
  }
  const int tail0 = head + 4 * n4;
  if (tail0 + t < V) take(l[tail0 + t], tail0 + t, best, arg);
  // the lowest index wins ties, in the wave and among the waves
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o, WAVE);
    int oi = __shfl_xor(arg, o, WAVE);
    take(ov, oi, best, arg);
  }
  if ((t & (WAVE - 1)) == 0) {
    bv[t / WAVE] = best;
    bi[t / WAVE] = arg;
  }
  __syncthreads();
  if (t == 0) {
    for (int w = 1; w < NTA / WAVE; ++w) take(bv[w], bi[w], best, arg);
    out[blockIdx.x] = arg < V ? arg : 0;
  }
}

// Four consecutive floats of a row from index i on; those at or behind V read as the lowest float.
// One 16-byte load where the row starts on a 16-byte boundary and the four are inside.
__device__ __forceinline__ float4 load4(const float* __restrict__ l, int i, int V, bool aligned) {
  if (aligned && i + 4 <= V) return *reinterpret_cast<const float4*>(l + i);
  float4 v;
  v.x = i < V ? l[i] : -FLT_MAX;
  v.y = i + 1 < V ? l[i + 1] : -FLT_MAX;
  v.z = i + 2 < V ? l[i + 2] : -FLT_MAX;
  v.w = i + 3 < V ? l[i + 3] : -FLT_MAX;
  return v;
}

constexpr int TILE = 4 * WAVE;                   // floats a wave takes with one load a lane

// the largest logit of a row, by all waves of the block
template <int NWB>
__device__ __forceinline__ float row_max(const float* __restrict__ l, int V, bool aligned, float* red) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n_tiles = (V + TILE - 1) / TILE;
  float mx = -FLT_MAX;
  for (int t = wave; t < n_tiles; t += 2 * NWB) {
    const float4 a = load4(l, t * TILE + 4 * lane, V, aligned);
    const float4 b = load4(l, min(t + NWB, n_tiles - 1) * TILE + 4 * lane, V, aligned);
    mx = fmaxf(fmaxf(fmaxf(mx, a.x), fmaxf(a.y, a.z)), fmaxf(fmaxf(a.w, b.x), fmaxf(fmaxf(b.y, b.z), b.w)));
  }
  return block_max<NWB>(mx, red);
}

// e((v - mx) / temperature) of the four, 0 behind the row's end
__device__ __forceinline__ float4 weights4(float4 v, int i, int V, float mx, float temperature) {
  float4 e;
  e.x = i < V ? expf((v.x - mx) / temperature) : 0.f;
  e.y = i + 1 < V ? expf((v.y - mx) / temperature) : 0.f;
  e.z = i + 2 < V ? expf((v.z - mx) / temperature) : 0.f;
  e.w = i + 3 < V ? expf((v.w - mx) / temperature) : 0.f;
  return e;
}

// Temperature sampling as sampler.cpp:40-65 walks it (the first index whose running sum reaches
// u times the total), with the walk cut in three: a wave owns a run of whole tiles and adds up its
// weights; every thread finds the wave whose run the target falls in; that wave goes through its
// tiles again, and in the tile that reaches the target a scan over the lanes and the lane's own four
// weights give the index.  Sums are added in index order at every level, so that rounding can only
// move the pick to a neighbour at an edge of the running sum.
__global__ __launch_bounds__(NTA) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ u,
                                                     float temperature, int* __restrict__ out, int V) {
  constexpr int NWB = NTA / WAVE;
  __shared__ float red[NWB];
  __shared__ float wsum[NWB];
  const float* l = logits + (size_t)blockIdx.x * V;
  const bool aligned = ((uintptr_t)l & 15) == 0;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n_tiles = (V + TILE - 1) / TILE;
  const int tpw = (n_tiles + NWB - 1) / NWB;     // tiles a wave owns, one after the other
  const int t0 = min(n_tiles, wave * tpw), t1 = min(n_tiles, t0 + tpw);
  const float mx = row_max<NWB>(l, V, aligned, red);

  float mine = 0.f;
  for (int t = t0; t < t1; ++t) {
    const int i = t * TILE + 4 * lane;
    const float4 e = weights4(load4(l, i, V, aligned), i, V, mx, temperature);
    mine += wave_sum((e.x + e.y) + (e.z + e.w));
  }
  if (lane == 0) wsum[wave] = mine;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < NWB; ++w) total += wsum[w];
  const float target = u[blockIdx.x] * total;
  float c = 0.f;
  int owner = -1;
#pragma unroll
  for (int w = 0; w < NWB; ++w) {
    if (owner < 0) {
      if (c + wsum[w] >= target && wsum[w] > 0.f) owner = w; else c += wsum[w];
    }
  }
  if (owner < 0) {                               // nothing reaches the target (NaN, or rounding at the very end)
    if (threadIdx.x == 0) out[blockIdx.x] = V - 1;
    return;
  }
  if (wave != owner) return;
  int pick = min(V, t1 * TILE) - 1;              // rounding may leave the walk just short of the run's sum
  for (int t = t0; t < t1; ++t) {
    const int i = t * TILE + 4 * lane;
    const float4 e = weights4(load4(l, i, V, aligned), i, V, mx, temperature);
    const float es = (e.x + e.y) + (e.z + e.w);
    const float tile_total = wave_sum(es);
    if (c + tile_total >= target && tile_total > 0.f) {
      float incl = es;                           // inclusive scan over the lanes
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
      }
      const unsigned long long reached = __ballot(c + incl >= target);
      pick = min(V, (t + 1) * TILE) - 1;
      if (reached != 0ull) {
        const int first = __ffsll((long long)reached) - 1;
        float cc = c + __shfl(incl - es, first, WAVE);
        const float4 ef = {__shfl(e.x, first, WAVE), __shfl(e.y, first, WAVE), __shfl(e.z, first, WAVE),
                           __shfl(e.w, first, WAVE)};
        const int at = t * TILE + 4 * first;
        pick = min(V, at + 4) - 1;
        if ((cc += ef.x) >= target) pick = at;
        else if ((cc += ef.y) >= target) pick = at + 1;
        else if ((cc += ef.z) >= target) pick = at + 2;
        pick = min(pick, V - 1);
      }
      break;
    }
    c += tile_total;
  }
  if (lane == 0) out[blockIdx.x] = pick;
}

// softmax probability (temperature 1) of one token a row, sampler.cpp:11-25
__global__ __launch_bounds__(NTA) void token_prob_kernel(const float* __restrict__ logits,
                                                         const int* __restrict__ index, float* __restrict__ prob,
                                                         int V) {
  constexpr int NWB = NTA / WAVE;
  __shared__ float red[NWB];
  const float* l = logits + (size_t)blockIdx.x * V;
  const bool aligned = ((uintptr_t)l & 15) == 0;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n_tiles = (V + TILE - 1) / TILE;
  const float mx = row_max<NWB>(l, V, aligned, red);
  float s = 0.f;
  for (int t = wave; t < n_tiles; t += NWB) {
    const int i = t * TILE + 4 * lane;
    const float4 e = weights4(load4(l, i, V, aligned), i, V, mx, 1.0f);
    s += (e.x + e.y) + (e.z + e.w);
  }
  s = block_sum<NWB>(s, red);
  if (threadIdx.x == 0) {
    int idx = index[blockIdx.x];
    prob[blockIdx.x] = (idx >= 0 && idx < V) ? expf(l[idx] - mx) / s : 0.f;
  }
}
}  // namespace

extern "C" int yalm_argmax(const float* logits, int* out, int R, int V, hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (V <= 0) return YALM_ERR_ARG;
  argmax_kernel<<<R, NTA, 0, stream>>>(logits, out, V);
  return launch_status();
}

extern "C" int yalm_sample(const float* logits, const float* u, float temperature, int* out, int R, int V,
                           hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (V <= 0 || !(temperature > 0.f)) return YALM_ERR_ARG;
  sample_kernel<<<R, NTA, 0, stream>>>(logits, u, temperature, out, V);
  return launch_status();
}

extern "C" int yalm_token_prob(const float* logits, const int* index, float* prob, int R, int V,
                               hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (V <= 0) return YALM_ERR_ARG;
  token_prob_kernel<<<R, NTA, 0, stream>>>(logits, index, prob, V);
  return launch_status();
}
