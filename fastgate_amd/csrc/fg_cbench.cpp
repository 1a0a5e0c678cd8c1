// Standalone C++ caller of the C ABI: no Python, no torch -- device memory from hipMalloc, the
// library through include/fastgate.h, timing with HIP events.  It doubles as the smallest complete
// example of the workspace protocol and as a profiling target whose trace holds nothing but the
// library's kernels.
//
//   fg_cbench [--m M] [--n N] [--k K] [--layout nk|kn] [--dtype f16|i8|i4] [--iters I] [--buffers R]
//
// Checks before timing (closed forms that need no CPU reference): activations of ones against
// weights whose row n (column n for [K,N]) holds the constant (n % 7) - 3 must give K * that
// constant in every row of C; for i8 the same with int8 weights, for i4 with nibbles (n % 15)
// and zero point 8.  Prints one JSON line; exit status 0 only when the check passed.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "fastgate.h"

#define HIP_OK(call)                                                                       \
  do {                                                                                     \
    hipError_t e_ = (call);                                                                \
    if (e_ != hipSuccess) {                                                                \
      std::fprintf(stderr, "%s failed: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__); \
      std::exit(2);                                                                        \
    }                                                                                      \
  } while (0)

#define FG_OK_OR_DIE(call)                                                          \
  do {                                                                              \
    int s_ = (call);                                                                \
    if (s_ != FG_OK) {                                                              \
      std::fprintf(stderr, "%s failed: %s (line %d)\n", #call, fg_strerror(s_), __LINE__); \
      std::exit(2);                                                                 \
    }                                                                               \
  } while (0)

namespace {

uint16_t f2h(float f) {  // exact for the small integers used here
  _Float16 h = static_cast<_Float16>(f);
  uint16_t b;
  std::memcpy(&b, &h, 2);
  return b;
}
float h2f(uint16_t b) {
  _Float16 h;
  std::memcpy(&h, &b, 2);
  return static_cast<float>(h);
}

struct Args {
  int M = 8, N = 8192, K = 8192, iters = 100, buffers = 0;
  std::string layout = "nk", dtype = "f16";
};

Args parse(int argc, char** argv) {
  Args a;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string k = argv[i], v = argv[i + 1];
    if (k == "--m") a.M = std::atoi(v.c_str());
    else if (k == "--n") a.N = std::atoi(v.c_str());
    else if (k == "--k") a.K = std::atoi(v.c_str());
    else if (k == "--iters") a.iters = std::atoi(v.c_str());
    else if (k == "--buffers") a.buffers = std::atoi(v.c_str());
    else if (k == "--layout") a.layout = v;
    else if (k == "--dtype") a.dtype = v;
    else {
      std::fprintf(stderr, "unknown option %s\n", k.c_str());
      std::exit(2);
    }
  }
  return a;
}

}  // namespace

int main(int argc, char** argv) {
  const Args a = parse(argc, argv);
  const int M = a.M, N = a.N, K = a.K;
  const bool nk = a.layout == "nk";
  const int layout = nk ? FG_W_NK : FG_W_KN;
  const bool f16 = a.dtype == "f16", i8 = a.dtype == "i8", i4 = a.dtype == "i4";
  if (!(f16 || i8 || i4) || (!f16 && !nk) || M < 1 || N < 1 || K < 1 || a.iters < 1) {
    std::fprintf(stderr, "bad arguments (int8 / int4 weights are [N,K] only)\n");
    return 2;
  }
  const size_t wbytes = f16 ? (size_t)N * K * 2 : (i8 ? (size_t)N * K : (size_t)N * K / 2);
  // rotate over enough weight buffers to exceed the 256 MB last-level cache
  int R = a.buffers > 0 ? a.buffers : (int)std::min<size_t>(64, (640u << 20) / wbytes + 2);

  // host images: weights constant per output column, activations all ones
  std::vector<uint8_t> w(wbytes);
  auto col_value = [&](int n) { return i4 ? (n % 15) : (n % 7) - 3; };
  if (f16) {
    uint16_t* p = reinterpret_cast<uint16_t*>(w.data());
    for (int r = 0; r < (nk ? N : K); ++r)
      for (int c = 0; c < (nk ? K : N); ++c) p[(size_t)r * (nk ? K : N) + c] = f2h((float)col_value(nk ? r : c));
  } else if (i8) {
    for (int n = 0; n < N; ++n) std::memset(w.data() + (size_t)n * K, (uint8_t)(int8_t)col_value(n), K);
  } else {
    for (int n = 0; n < N; ++n) std::memset(w.data() + (size_t)n * (K / 2), (uint8_t)(col_value(n) * 0x11), K / 2);
  }
  std::vector<uint16_t> ones((size_t)M * K, f2h(1.0f));

  std::vector<void*> W(R);
  for (auto& b : W) {
    HIP_OK(hipMalloc(&b, wbytes));
    HIP_OK(hipMemcpy(b, w.data(), wbytes, hipMemcpyHostToDevice));
  }
  void *A, *C;
  HIP_OK(hipMalloc(&A, (size_t)M * K * 2));
  HIP_OK(hipMemcpy(A, ones.data(), (size_t)M * K * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMalloc(&C, (size_t)M * N * 2));
  HIP_OK(hipMemset(C, 0xFF, (size_t)M * N * 2));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // split-K workspace: size from the library, counters cleared once
  fg_plan_t plan;
  std::memset(&plan, 0, sizeof(plan));
  void* ws = nullptr;
  size_t ws_bytes = 0;
  if (f16) {
    FG_OK_OR_DIE(fg_plan(M, N, K, layout, 0, &plan));
    ws_bytes = fg_workspace_bytes(M, N, K, layout, 0);
    if (ws_bytes) {
      HIP_OK(hipMalloc(&ws, ws_bytes));
      FG_OK_OR_DIE(fg_workspace_init(ws, ws_bytes, stream));
    }
  }
  auto call = [&](int i) {
    if (f16) return fg_gemm_f16(A, W[i % R], C, M, N, K, layout, 0, 0, ws, ws_bytes, stream);
    if (i8) return fg_gemv_w8a16(W[i % R], A, nullptr, 1.0f, 0.0f, C, M, N, K, stream);
    return fg_gemv_w4a16(W[i % R], A, nullptr, 1.0f, 8.0f, C, M, N, K, stream);
  };

  // check
  FG_OK_OR_DIE(call(0));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<uint16_t> c((size_t)M * N);
  HIP_OK(hipMemcpy(c.data(), C, c.size() * 2, hipMemcpyDeviceToHost));
  size_t bad = 0;
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      const float want = (float)K * (float)(col_value(n) - (i4 ? 8 : 0));
      const float got = h2f(c[(size_t)m * N + n]);
      // K * v is rounded once to fp16; compare against the same rounding
      if (got != h2f(f2h(want))) ++bad;
    }

  // time
  for (int i = 0; i < 10; ++i) FG_OK_OR_DIE(call(i));
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, stream));
  for (int i = 0; i < a.iters; ++i) FG_OK_OR_DIE(call(i));
  HIP_OK(hipEventRecord(e1, stream));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  const double us = ms * 1e3 / a.iters;
  const double bytes = (double)wbytes + 2.0 * M * K + 2.0 * M * N;
  std::printf(
      "{\"dtype\": \"%s\", \"layout\": \"%s\", \"M\": %d, \"N\": %d, \"K\": %d, \"buffers\": %d, "
      "\"kernel\": %d, \"splitk\": %d, \"waves\": %d, \"workspace_bytes\": %zu, \"us_per_call\": %.2f, "
      "\"GBps\": %.1f, \"mismatches\": %zu, \"ok\": %s}\n",
      a.dtype.c_str(), a.layout.c_str(), M, N, K, R, plan.kernel, plan.splitk, plan.waves, ws_bytes, us,
      bytes / us / 1e3, bad, bad == 0 ? "true" : "false");
  return bad == 0 ? 0 : 1;
}
