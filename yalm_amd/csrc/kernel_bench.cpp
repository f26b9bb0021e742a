// Single kernels of the library at the sizes of a 7B decoder, timed with events, without Python:
//
//   kernel_bench <kernel> [rows] [copies]
//     matmul       the feed-forward's gate/up product with its gated epilogue, [rows, 4096] x [28672, 4096]
//     matmul-wide  the head, [rows, 4096] x [32000, 4096], float32 out
//     down         the down projection with the residual add, [rows, 14336] x [4096, 14336]
//     qkv          the q/k/v projection, float32 out, [rows, 4096] x [6144, 4096]
//     read         a kernel that only reads `copies` x 256 MB
//     mfma         a loop of matrix-core instructions on registers
//
// The role of the reference's `test -bk <kernel>` (src/test.cpp:340-405), which runs one kernel at these sizes for a
// profiler; here the bytes and the rate are printed as well.  Every product has `copies` weight matrices (default 8)
// that are used in turn, so that no launch finds its weights in a cache.  A run under `rocprofv3 --pmc` gives the
// memory traffic of each launch by counters, against which the printed byte count can be held.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <string>
#include <vector>
#include "yalm_hip.h"

#define CK(x)                                                                           \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                    \
      return 1;                                                                         \
    }                                                                                   \
  } while (0)

static unsigned short bf16_of(float v) {
  unsigned int u;
  memcpy(&u, &v, 4);
  return (unsigned short)((u + 0x7FFF + ((u >> 16) & 1)) >> 16);
}

// values in [-scale, scale), a different stream for every seed
static void fill(std::vector<unsigned short>& v, unsigned long long seed, float scale) {
  unsigned long long s = seed * 0x9E3779B97F4A7C15ull + 1;
  for (auto& x : v) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    x = bf16_of(((float)((s >> 40) & 0xFFFF) / 32768.0f - 1.0f) * scale);
  }
}

int main(int argc, char** argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: %s matmul|matmul-wide|down|qkv|read|mfma [rows] [copies]\n", argv[0]);
    return 2;
  }
  const std::string what = argv[1];
  const int M = argc > 2 ? atoi(argv[2]) : 1;
  const int copies = argc > 3 ? atoi(argv[3]) : 8;
  const int dim = 4096, hidden = 14336, vocab = 32000, qkv = 6144;
  hipStream_t stream;
  CK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));

  if (what == "read" || what == "mfma") {
    unsigned int* out;
    CK(hipMalloc(&out, 4096));
    CK(hipMemset(out, 0, 4096));
    double work = 0.0;
    void* buf = nullptr;
    const long bytes = (long)copies * (256l << 20);
    if (what == "read") {
      CK(hipMalloc(&buf, bytes));
      CK(hipMemset(buf, 1, bytes));
    }
    for (int rep = 0; rep < 4; ++rep) {
      CK(hipEventRecord(e0, stream));
      int rc = what == "read" ? yalm_probe_read(buf, bytes, out, 2048, stream)
                              : yalm_probe_mfma(16, 16384, 1024, (float*)out, &work, stream);
      if (rc != 0) {
        fprintf(stderr, "launch failed: %s\n", yalm_error_string(rc));
        return 1;
      }
      CK(hipEventRecord(e1, stream));
      CK(hipEventSynchronize(e1));
      float ms = 0.f;
      CK(hipEventElapsedTime(&ms, e0, e1));
      if (what == "read")
        printf("read %ld bytes in %.1f us: %.0f GB/s\n", bytes, ms * 1e3, bytes / (ms * 1e-3) / 1e9);
      else
        printf("mfma 16x16x32 %.3g flop in %.1f us: %.0f TFLOP/s\n", work, ms * 1e3, work / (ms * 1e-3) / 1e12);
    }
    return 0;
  }

  int N, K, epilogue, H = 0;
  if (what == "matmul") { N = 32 * ((hidden + 15) / 16); K = dim; epilogue = 3; H = hidden; }
  else if (what == "matmul-wide") { N = vocab; K = dim; epilogue = 0; }
  else if (what == "down") { N = dim; K = hidden; epilogue = 2; }
  else if (what == "qkv") { N = qkv; K = dim; epilogue = 0; }
  else {
    fprintf(stderr, "unknown kernel %s\n", what.c_str());
    return 2;
  }
  if (M < 1 || M > 4096 || copies < 1 || copies > 64) {
    fprintf(stderr, "rows 1..4096, copies 1..64\n");
    return 2;
  }
  std::vector<unsigned short> hw((size_t)N * K), hx((size_t)M * K);
  fill(hw, 1, 1.0f / 64.0f);
  fill(hx, 2, 1.0f);
  std::vector<void*> w(copies);
  for (int c = 0; c < copies; ++c) {
    CK(hipMalloc(&w[c], hw.size() * 2));
    CK(hipMemcpy(w[c], hw.data(), hw.size() * 2, hipMemcpyHostToDevice));
  }
  void *x, *out;
  float* ws;
  const long ws_floats = 16l * M * N;
  CK(hipMalloc(&x, hx.size() * 2));
  CK(hipMemcpy(x, hx.data(), hx.size() * 2, hipMemcpyHostToDevice));
  CK(hipMalloc(&out, (size_t)M * N * 4));
  CK(hipMemset(out, 0, (size_t)M * N * 4));
  CK(hipMalloc(&ws, ws_floats * 4));
  const double bytes = (double)N * K * 2 + (double)M * K * 2 + (double)M * (epilogue == 3 ? H * 2 : N * 4);
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0, stream));
    for (int c = 0; c < copies; ++c) {
      int rc = yalm_gemm(x, w[c], out, ws, ws_floats, M, N, K, 1, epilogue, H, 0, stream);
      if (rc != 0) {
        fprintf(stderr, "yalm_gemm failed: %s\n", yalm_error_string(rc));
        return 1;
      }
    }
    CK(hipEventRecord(e1, stream));
    CK(hipEventSynchronize(e1));
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / copies;
    printf("%s rows %d: [%d, %d] x [%d, %d]  %.2f us a launch, %.1f MB -> %.0f GB/s (%.3f of 8 TB/s), %.1f TFLOP/s\n",
           what.c_str(), M, M, K, N, K, us, bytes / 1e6, bytes / us / 1e3, bytes / us / 1e3 / 8000.0,
           2.0 * M * N * K / us / 1e6);
  }
  return 0;
}
