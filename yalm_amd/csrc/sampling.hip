// Sampling over float32 logits: argmax, temperature sampling given the uniform
// number, and the probability of one token.  One block of 256 threads per row;
// every thread owns one contiguous chunk of the vocabulary so that "first
// index" keeps its meaning.
#include <float.h>
#include "common.h"
#include "yalm_hip.h"

namespace {
constexpr int NT = 256;
constexpr int NW = NT / WAVE;

constexpr int NTA = 1024;                        // argmax: 1024 threads a row

__global__ __launch_bounds__(NTA) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
  __shared__ float bv[NTA / WAVE];
  __shared__ int bi[NTA / WAVE];
  const float* l = logits + (size_t)blockIdx.x * V;
  float best = -FLT_MAX;
  int arg = V;                                   // "none": larger than every index
  for (int i = threadIdx.x; i < V; i += NTA) {   // indices rise within a thread: strict '>' keeps its first maximum
    float v = l[i];
    if (v > best) {
      best = v;
      arg = i;
    }
  }
  // the lowest index wins ties, in the wave and among the waves
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o, WAVE);
    int oi = __shfl_xor(arg, o, WAVE);
    if (oi < V && (arg >= V || ov > best || (ov == best && oi < arg))) {
      best = ov;
      arg = oi;
    }
  }
  if ((threadIdx.x & (WAVE - 1)) == 0) {
    bv[threadIdx.x / WAVE] = best;
    bi[threadIdx.x / WAVE] = arg;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < NTA / WAVE; ++w) {
      float ov = bv[w];
      int oi = bi[w];
      if (oi < V && (arg >= V || ov > best || (ov == best && oi < arg))) {
        best = ov;
        arg = oi;
      }
    }
    out[blockIdx.x] = arg < V ? arg : 0;
  }
}

__global__ __launch_bounds__(NT) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ u,
                                                    float temperature, int* __restrict__ out, int V) {
  __shared__ float red[NW];
  __shared__ float sums[NT];
  const float* l = logits + (size_t)blockIdx.x * V;
  int chunk = (V + NT - 1) / NT;
  int lo = min(V, (int)threadIdx.x * chunk), hi = min(V, lo + chunk);
  float mx = -FLT_MAX;
  for (int i = lo; i < hi; ++i) mx = fmaxf(mx, l[i]);
  mx = block_max<NW>(mx, red);
  float s = 0.f;
  for (int i = lo; i < hi; ++i) s += expf((l[i] - mx) / temperature);
  sums[threadIdx.x] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int t = 0; t < NT; ++t) total += sums[t];
    float target = u[blockIdx.x] * total;
    float c = 0.f;
    int owner = -1;
    for (int t = 0; t < NT; ++t) {
      if (c + sums[t] >= target && sums[t] > 0.f) {
        owner = t;
        break;
      }
      c += sums[t];
    }
    int pick = V - 1;
    if (owner >= 0) {
      int a = min(V, owner * chunk), b = min(V, a + chunk);
      pick = b - 1;                              // rounding may leave the walk just short of the chunk's sum
      for (int i = a; i < b; ++i) {
        c += expf((l[i] - mx) / temperature);
        if (c >= target) {
          pick = i;
          break;
        }
      }
    }
    out[blockIdx.x] = pick;
  }
}

__global__ __launch_bounds__(NT) void token_prob_kernel(const float* __restrict__ logits,
                                                        const int* __restrict__ index, float* __restrict__ prob,
                                                        int V) {
  __shared__ float red[NW];
  const float* l = logits + (size_t)blockIdx.x * V;
  float mx = -FLT_MAX;
  for (int i = threadIdx.x; i < V; i += NT) mx = fmaxf(mx, l[i]);
  mx = block_max<NW>(mx, red);
  float s = 0.f;
  for (int i = threadIdx.x; i < V; i += NT) s += expf(l[i] - mx);
  s = block_sum<NW>(s, red);
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
  sample_kernel<<<R, NT, 0, stream>>>(logits, u, temperature, out, V);
  return launch_status();
}

extern "C" int yalm_token_prob(const float* logits, const int* index, float* prob, int R, int V,
                               hipStream_t stream) {
  if (R <= 0) return YALM_OK;
  if (V <= 0) return YALM_ERR_ARG;
  token_prob_kernel<<<R, NT, 0, stream>>>(logits, index, prob, V);
  return launch_status();
}
