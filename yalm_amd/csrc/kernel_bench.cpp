// Single kernels of the library at the sizes of a 7B decoder, timed with events, without Python:
//
//   kernel_bench <kernel> [rows] [copies]
//     matmul       the feed-forward's gate/up product with its gated epilogue, [rows, 4096] x [28672, 4096]
//     matmul-wide  the head, [rows, 4096] x [32000, 4096], float32 out
//     down         the down projection with the residual add, [rows, 14336] x [4096, 14336]
//     qkv          the q/k/v projection, float32 out, [rows, 4096] x [6144, 4096]
//     ffn          the whole feed-forward: gate/up with the gated GELU epilogue, then down with the residual add
//     mha          decode attention of `rows` sequences over 4,096 cached positions each (32 heads in 8 groups of
//                  head size 128; `copies` splits of every sequence's pages, default 8)
//     read         a kernel that only reads `copies` x 256 MB
//     mfma         a loop of matrix-core instructions on registers
//
// The role of the reference's `test -bk <kernel>` (src/test.cpp:340-405: matmul, matmul-wide, mha, ffn), which runs
// one kernel at these sizes for a profiler; here the bytes and the rate are printed as well.  Every product has `copies` weight matrices (default 8)
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
    fprintf(stderr, "usage: %s matmul|matmul-wide|down|qkv|ffn|mha|read|mfma [rows] [copies]\n", argv[0]);
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

  if (what == "mha") {
    // the pages of every sequence lie one behind the other; what they hold does not matter to the clock
    const int n_heads = 32, n_kv = 8, hd = 128, kv_len = 4096, page = 64, pages_seq = kv_len / page;
    const int B = M, n_splits = argc > 3 ? copies : 8;
    if (B < 1 || B > 256 || n_splits < 1 || n_splits > 64) {
      fprintf(stderr, "sequences 1..256, splits 1..64\n");
      return 2;
    }
    const size_t page_elems = (size_t)n_kv * page * hd;
    std::vector<unsigned short> hk((size_t)B * pages_seq * page_elems), hq((size_t)B * n_heads * hd);
    fill(hk, 3, 1.0f);
    fill(hq, 4, 1.0f);
    std::vector<int> table((size_t)B * pages_seq), slot(B), len(B, kv_len);
    for (int b = 0; b < B; ++b) {
      slot[b] = b;
      for (int p = 0; p < pages_seq; ++p) table[(size_t)b * pages_seq + p] = p * B + b;   // handed out in turn, as the cache does
    }
    void *kp, *vp, *q, *out, *d_table, *d_slot, *d_len;
    float* partial;
    const long ws_bytes = yalm_attn_decode_workspace(B, n_heads, hd, n_splits);
    CK(hipMalloc(&kp, hk.size() * 2));
    CK(hipMalloc(&vp, hk.size() * 2));
    CK(hipMemcpy(kp, hk.data(), hk.size() * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(vp, hk.data(), hk.size() * 2, hipMemcpyHostToDevice));
    CK(hipMalloc(&q, hq.size() * 2));
    CK(hipMemcpy(q, hq.data(), hq.size() * 2, hipMemcpyHostToDevice));
    CK(hipMalloc(&out, hq.size() * 2));
    CK(hipMalloc(&d_table, table.size() * 4));
    CK(hipMemcpy(d_table, table.data(), table.size() * 4, hipMemcpyHostToDevice));
    CK(hipMalloc(&d_slot, B * 4));
    CK(hipMemcpy(d_slot, slot.data(), B * 4, hipMemcpyHostToDevice));
    CK(hipMalloc(&d_len, B * 4));
    CK(hipMemcpy(d_len, len.data(), B * 4, hipMemcpyHostToDevice));
    CK(hipMalloc(&partial, ws_bytes));
    const double bytes = 2.0 * hk.size() * 2;
    for (int rep = 0; rep < 3; ++rep) {
      const int launches = 8;
      CK(hipEventRecord(e0, stream));
      for (int c = 0; c < launches; ++c) {
        int rc = yalm_attn_decode_lse(q, kp, vp, (const int*)d_table, pages_seq, pages_seq, (const int*)d_slot,
                                      (const int*)d_len, out, nullptr, partial, B, n_heads, n_kv, hd, 0, n_splits,
                                      B * pages_seq, /* pages in blocks */ 1, /* bfloat16 */ 1, 0, nullptr, nullptr, nullptr, 0, stream);
        if (rc != 0) {
          fprintf(stderr, "yalm_attn_decode_lse failed: %s\n", yalm_error_string(rc));
          return 1;
        }
      }
      CK(hipEventRecord(e1, stream));
      CK(hipEventSynchronize(e1));
      float ms = 0.f;
      CK(hipEventElapsedTime(&ms, e0, e1));
      const double us = ms * 1e3 / launches;
      printf("mha %d sequences x %d positions, %d splits: %.2f us a launch (with the merge of the splits), %.1f MB -> %.0f GB/s "
             "(%.3f of 8 TB/s)\n", B, kv_len, n_splits, us, bytes / 1e6, bytes / us / 1e3, bytes / us / 1e3 / 8000.0);
    }
    return 0;
  }

  int N, K, epilogue, H = 0;
  const bool ffn = what == "ffn";
  if (ffn) { N = 32 * ((hidden + 15) / 16); K = dim; epilogue = 5; H = hidden; }
  else if (what == "matmul") { N = 32 * ((hidden + 15) / 16); K = dim; epilogue = 3; H = hidden; }
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
  // ffn: the down projection behind the gated product, whose bfloat16 [rows, hidden] result lies in `out`
  std::vector<void*> w2(ffn ? copies : 0);
  void* x_out = nullptr;
  if (ffn) {
    std::vector<unsigned short> hw2((size_t)dim * hidden);
    fill(hw2, 5, 1.0f / 128.0f);
    for (int c = 0; c < copies; ++c) {
      CK(hipMalloc(&w2[c], hw2.size() * 2));
      CK(hipMemcpy(w2[c], hw2.data(), hw2.size() * 2, hipMemcpyHostToDevice));
    }
    CK(hipMalloc(&x_out, (size_t)M * dim * 4));
    CK(hipMemset(x_out, 0, (size_t)M * dim * 4));
  }
  const double bytes = (double)N * K * 2 + (double)M * K * 2 + (double)M * (epilogue == 3 || epilogue == 5 ? H * 2 : N * 4) +
                       (ffn ? (double)dim * hidden * 2 + (double)M * hidden * 2 + (double)M * dim * 8 : 0.0);
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0, stream));
    for (int c = 0; c < copies; ++c) {
      int rc = yalm_gemm(x, w[c], out, ws, ws_floats, M, N, K, 1, epilogue, H, 0, stream);
      if (rc == 0 && ffn) rc = yalm_gemm(out, w2[c], x_out, ws, ws_floats, M, dim, hidden, 1, 2, 0, 0, stream);
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
    const double flop = 2.0 * M * N * K + (ffn ? 2.0 * M * dim * hidden : 0.0);
    printf("%s rows %d: [%d, %d] x [%d, %d]%s  %.2f us%s, %.1f MB -> %.0f GB/s (%.3f of 8 TB/s), %.1f TFLOP/s\n",
           what.c_str(), M, M, K, N, K, ffn ? ", gelu(gate) * up, x [4096, 14336] added to the residual" : "", us,
           ffn ? " for the two launches" : " a launch", bytes / 1e6, bytes / us / 1e3, bytes / us / 1e3 / 8000.0,
           flop / us / 1e6);
  }
  return 0;
}
