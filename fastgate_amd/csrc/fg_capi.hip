// C ABI of libfastgate: argument validation, launch planning, dispatch.  Host code only;
// the kernels live in fg_kernels_*.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "fg_internal.h"
#include "fg_plan.h"

// Split-K scratch of fg_gemm_f16_static: one copy per GPU, held until the process ends.  The name
// is a host-side stand-in for the symbol, never a device address: host code reaches the memory
// only through the per-device pointer that static_scratch() obtains with hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[FG_STATIC_SCRATCH_BYTES];
static_assert(FG_STATIC_SCRATCH_BYTES == fg::kWsHeaderBytes + (8u << 20), "the header documented in fastgate.h plus 8 MiB of partials");

namespace fg {
namespace {

int check_launch() { return hipGetLastError() == hipSuccess ? FG_OK : FG_ERR_LAUNCH; }

// The planner's rules and the [K,N] kernels' band spreading count compute units.  The entry points
// that launch read the current device's count once, before they plan; fg_plan and
// fg_workspace_bytes never call into the HIP runtime and plan for the count the library holds
// at that moment (MI355X's 256 until a launch or fg_set_compute_units changed it).
std::atomic<bool> g_cus_pinned{false};  // fg_set_compute_units was called: keep the caller's count
void read_compute_units() {
  static std::once_flag once;
  std::call_once(once, [] {
    if (g_cus_pinned.load()) return;
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) {
      set_compute_units(n);
      int x = 0;
      if (hipDeviceGetAttribute(&x, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && x > 0) set_xccs(x);
    }
    (void)hipGetLastError();
  });
}

// `tail`: bias and activation bits of the kernels' flag word (0 for a plain product).
int run_gemm(const void* A, const void* W, void* C, int M, int N, int K, int accumulate,
             const fg_plan_t& p, void* ws, size_t ws_bytes, hipStream_t s, int tail = 0,
             const void* bias = nullptr, int ldw = 0) {
  if (p.splitk > 1 && (ws == nullptr || ws_bytes < p.workspace_bytes)) return FG_ERR_WORKSPACE;
  read_compute_units();  // the [K,N] kernels take the count as an argument
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W) |
       reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(ws)) & 15) {
    return FG_ERR_INVALID_ARG;  // 16-byte loads and stores
  }
  const bool kn = p.kernel == FG_KERNEL_KN_DOT2 || p.kernel == FG_KERNEL_KN_MFMA;
  if (ldw == 0) ldw = kn ? N : K;
  if (ldw != (kn ? N : K) && (!kn || ldw < N || ldw % 8 != 0)) return FG_ERR_INVALID_ARG;
  GemmArgs a{A, W, C, nullptr, nullptr, M, N, K,
             (accumulate ? kFlagAccumulate : 0) | (p.stagger ? kFlagStagger : 0) | tail, bias, ldw,
             compute_units(), xccs()};
  if (p.splitk > 1) {
    a.ws = reinterpret_cast<float*>(static_cast<unsigned char*>(ws) + kWsHeaderBytes);
    a.counters = p.fused ? static_cast<int*>(ws) : nullptr;
    if (p.fused == 2) {
      if (p.splitk > kFixMaxSplit || (size_t)M * N > kWsAccElems) return FG_ERR_UNSUPPORTED;
      a.accumulate |= kFlagFixSplit;
    }
    if (p.fused == 3 || p.fused == 4) {
      if (p.kernel != FG_KERNEL_KN_MFMA || p.splitk > kMailboxMaxSplit ||
          (size_t)p.grid_x * p.grid_y * p.splitk * p.waves > kWsMailboxFlags) {
        return FG_ERR_UNSUPPORTED;
      }
      a.accumulate |= kFlagXcdLocal | (p.fused == 4 ? kFlagPretendForeign : 0);
    }
  }
  (void)hipGetLastError();
  bool ok = false;
  switch (p.kernel) {
    case FG_KERNEL_NK_DOT2: ok = launch_nk_dot2(p, a, s); break;
    case FG_KERNEL_NK_MFMA4: ok = launch_nk_mfma4(p, a, s); break;
    case FG_KERNEL_NK_MFMA_R: ok = launch_nk_mfma_r(p, a, s); break;
    case FG_KERNEL_KN_DOT2: ok = launch_kn_dot2(p, a, s); break;
    case FG_KERNEL_KN_MFMA: ok = launch_kn_mfma(p, a, s); break;
    default: break;
  }
  if (!ok) return FG_ERR_UNSUPPORTED;
  if (check_launch() != FG_OK) return FG_ERR_LAUNCH;
  if (p.splitk > 1 && !p.fused) {
    launch_splitk_reduce(a.ws, C, p.splitk, M, N, a.accumulate, a.bias, s);
    if (check_launch() != FG_OK) return FG_ERR_LAUNCH;
  }
  return FG_OK;
}

// Device address of `scratch` on the current device, resolved once per device (with that device
// current) and kept.  The first resolution also clears the counter header with a fill kernel on
// `s`; after that every call leaves the counters at zero by itself.  Returns null on failure.
constexpr int kMaxDevices = 64;
void* static_scratch(hipStream_t s) {
  static std::atomic<void*> ptrs[kMaxDevices];
  static std::mutex mu;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = ptrs[dev].load(std::memory_order_acquire);
  if (p != nullptr) return p;
  std::lock_guard<std::mutex> lock(mu);
  p = ptrs[dev].load(std::memory_order_acquire);
  if (p != nullptr) return p;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
    (void)hipGetLastError();
    return nullptr;
  }
  (void)hipGetLastError();
  launch_fill_zero(p, kWsHeaderBytes, s);
  if (check_launch() != FG_OK) return nullptr;
  ptrs[dev].store(p, std::memory_order_release);
  return p;
}

bool is_nk(int kernel) {
  return kernel == FG_KERNEL_NK_DOT2 || kernel == FG_KERNEL_NK_MFMA4 || kernel == FG_KERNEL_NK_MFMA_R;
}
bool is_kn(int kernel) { return kernel == FG_KERNEL_KN_DOT2 || kernel == FG_KERNEL_KN_MFMA; }

}  // namespace
}  // namespace fg

extern "C" {

int fg_version(void) { return FG_VERSION; }

const char* fg_strerror(int status) {
  switch (status) {
    case FG_OK: return "ok";
    case FG_ERR_INVALID_ARG: return "invalid argument (null or misaligned pointer, bad size or enum)";
    case FG_ERR_ALIGN128: return "K and N must be multiples of 128";
    case FG_ERR_WORKSPACE: return "split-K workspace missing or too small";
    case FG_ERR_LAUNCH: return "HIP kernel launch failed";
    case FG_ERR_UNSUPPORTED: return "plan names a kernel/tile combination that is not built";
    case FG_ERR_SCRATCH_LIMIT:
      return "shape needs more split-K scratch than the static buffer of fg_gemm_f16_static holds";
    default: return "unknown fastgate status";
  }
}

int fg_plan(int M, int N, int K, int w_layout, int splitk, fg_plan_t* out) {
  if (out == nullptr || splitk < 0) return FG_ERR_INVALID_ARG;
  int st = fg::plan_validate_shape(M, N, K, w_layout);
  if (st != FG_OK) return st;
  st = fg::plan_make(M, N, K, w_layout, splitk, out);
  if (st != FG_OK) return st;
  // FASTGATE_SPLITK_COMPLETION = two-pass | counter | atomic | xcd-local (read once) overrides how the
  // library's plans complete a split: a way back to the second kernel, whose only communication
  // is the kernel boundary, without rebuilding.
  static const int forced = [] {
    const char* e = std::getenv("FASTGATE_SPLITK_COMPLETION");
    if (e == nullptr || *e == 0) return -1;
    if (std::strcmp(e, "two-pass") == 0) return 0;
    if (std::strcmp(e, "counter") == 0) return 1;
    if (std::strcmp(e, "atomic") == 0) return 2;
    if (std::strcmp(e, "xcd-local") == 0) return 3;
    std::fprintf(stderr, "libfastgate: FASTGATE_SPLITK_COMPLETION=%s is not one of two-pass, counter, atomic, "
                         "xcd-local; ignored\n", e);
    return -1;
  }();
  if (forced >= 0 && out->splitk > 1) {
    // a plan the forced completion does not apply to keeps the planner's own
    const bool applies = forced <= 1 ||
                         (forced == 2 && out->splitk <= fg::kFixMaxSplit && (size_t)M * N <= fg::kWsAccElems) ||
                         (forced == 3 && out->kernel == FG_KERNEL_KN_MFMA && out->splitk <= fg::kMailboxMaxSplit &&
                          (size_t)out->grid_x * out->grid_y * out->splitk * out->waves <= fg::kWsMailboxFlags);
    if (applies) {
      fg_plan_t q = *out;
      q.fused = forced;
      if (fg::plan_finish(M, N, K, &q) == FG_OK) *out = q;
    }
  }
  return FG_OK;
}

size_t fg_workspace_bytes(int M, int N, int K, int w_layout, int splitk) {
  fg_plan_t p;
  if (fg_plan(M, N, K, w_layout, splitk, &p) != FG_OK) return 0;
  return p.workspace_bytes;
}

size_t fg_workspace_header_bytes(void) { return fg::kWsHeaderBytes; }

int fg_set_compute_units(int cus) {
  if (cus < 16 || cus > 4096) return FG_ERR_INVALID_ARG;
  fg::g_cus_pinned.store(true);
  fg::set_compute_units(cus);
  return FG_OK;
}

int fg_compute_units(void) { return fg::compute_units(); }

int fg_use_device_compute_units(void) {
  fg::read_compute_units();
  return fg::compute_units();
}

int fg_workspace_init(void* ws, size_t ws_bytes, void* stream) {
  if (ws == nullptr || ws_bytes < fg::kWsHeaderBytes || (reinterpret_cast<uintptr_t>(ws) & 15)) {
    return FG_ERR_INVALID_ARG;
  }
  (void)hipGetLastError();
  fg::launch_fill_zero(ws, fg::kWsHeaderBytes, static_cast<hipStream_t>(stream));
  return fg::check_launch();
}

int fg_gemm_f16(const void* A, const void* W, void* C, int M, int N, int K, int w_layout,
                int accumulate, int splitk, void* ws, size_t ws_bytes, void* stream) {
  if (A == nullptr || W == nullptr || C == nullptr) return FG_ERR_INVALID_ARG;
  fg::read_compute_units();
  fg_plan_t p;
  int st = fg_plan(M, N, K, w_layout, splitk, &p);
  if (st != FG_OK) return st;
  if (splitk == 0 && p.splitk > 1 && (ws == nullptr || ws_bytes < p.workspace_bytes)) {
    // the library's own choice of a split needs a workspace the caller did not bring: run
    // unsplit (slower where the grid then leaves CUs idle) instead of failing
    st = fg_plan(M, N, K, w_layout, 1, &p);
    if (st != FG_OK) return st;
  }
  return fg::run_gemm(A, W, C, M, N, K, accumulate, p, ws, ws_bytes,
                      static_cast<hipStream_t>(stream));
}

int fg_gemm_f16_static(const void* A, const void* W, void* C, int M, int N, int K, int w_layout,
                       int accumulate, int splitk, void* stream) {
  if (A == nullptr || W == nullptr || C == nullptr) return FG_ERR_INVALID_ARG;
  fg::read_compute_units();
  fg_plan_t p;
  const int st = fg_plan(M, N, K, w_layout, splitk, &p);
  if (st != FG_OK) return st;
  if (p.workspace_bytes > (size_t)FG_STATIC_SCRATCH_BYTES) return FG_ERR_SCRATCH_LIMIT;
  void* ws = nullptr;
  if (p.splitk > 1) {
    ws = fg::static_scratch(static_cast<hipStream_t>(stream));
    if (ws == nullptr) return FG_ERR_LAUNCH;
  }
  return fg::run_gemm(A, W, C, M, N, K, accumulate, p, ws, p.splitk > 1 ? (size_t)FG_STATIC_SCRATCH_BYTES : 0,
                      static_cast<hipStream_t>(stream));
}

int fg_gemm_f16_pitched(const void* A, const void* W, void* C, int M, int N, int K, int ldw,
                        int accumulate, int splitk, void* ws, size_t ws_bytes, void* stream) {
  if (A == nullptr || W == nullptr || C == nullptr) return FG_ERR_INVALID_ARG;
  if (ldw < N || ldw % 8 != 0) return FG_ERR_INVALID_ARG;
  fg::read_compute_units();
  fg_plan_t p;
  int st = fg_plan(M, N, K, FG_W_KN, splitk, &p);
  if (st != FG_OK) return st;
  if (splitk == 0 && p.splitk > 1 && (ws == nullptr || ws_bytes < p.workspace_bytes)) {
    st = fg_plan(M, N, K, FG_W_KN, 1, &p);
    if (st != FG_OK) return st;
  }
  return fg::run_gemm(A, W, C, M, N, K, accumulate, p, ws, ws_bytes, static_cast<hipStream_t>(stream),
                      0, nullptr, ldw);
}

int fg_gemm_f16_planned(const void* A, const void* W, void* C, int M, int N, int K, int w_layout,
                        int accumulate, fg_plan_t* plan, void* ws, size_t ws_bytes, void* stream) {
  if (A == nullptr || W == nullptr || C == nullptr || plan == nullptr) return FG_ERR_INVALID_ARG;
  int st = fg::plan_validate_shape(M, N, K, w_layout);
  if (st != FG_OK) return st;
  if ((w_layout == FG_W_NK && !fg::is_nk(plan->kernel)) ||
      (w_layout == FG_W_KN && !fg::is_kn(plan->kernel))) {
    return FG_ERR_UNSUPPORTED;
  }
  st = fg::plan_finish(M, N, K, plan);
  if (st != FG_OK) return st;
  return fg::run_gemm(A, W, C, M, N, K, accumulate, *plan, ws, ws_bytes,
                      static_cast<hipStream_t>(stream));
}

int fg_gemm_f16_bias_act(const void* A, const void* W, const void* bias, int act, void* C, int M,
                         int N, int K, int w_layout, int splitk, fg_plan_t* plan, void* ws,
                         size_t ws_bytes, void* stream) {
  if (A == nullptr || W == nullptr || C == nullptr) return FG_ERR_INVALID_ARG;
  if (act < FG_ACT_NONE || act > FG_ACT_SILU) return FG_ERR_INVALID_ARG;
  if (reinterpret_cast<uintptr_t>(bias) & 1) return FG_ERR_INVALID_ARG;
  const int tail = (bias != nullptr ? fg::kFlagBias : 0) | (act << fg::kFlagActShift);
  fg::read_compute_units();
  fg_plan_t p;
  int st;
  if (plan == nullptr) {
    st = fg_plan(M, N, K, w_layout, splitk, &p);
    if (st != FG_OK) return st;
    plan = &p;
  } else {
    st = fg::plan_validate_shape(M, N, K, w_layout);
    if (st != FG_OK) return st;
    if ((w_layout == FG_W_NK && !fg::is_nk(plan->kernel)) ||
        (w_layout == FG_W_KN && !fg::is_kn(plan->kernel))) {
      return FG_ERR_UNSUPPORTED;
    }
    st = fg::plan_finish(M, N, K, plan);
    if (st != FG_OK) return st;
  }
  return fg::run_gemm(A, W, C, M, N, K, 0, *plan, ws, ws_bytes, static_cast<hipStream_t>(stream),
                      tail, bias);
}

int fg_gemv_w8a16(const void* Wq, const void* x, const void* scale, float scalar_scale,
                  float zero_point, void* y, int M, int N, int K, void* stream) {
  if (Wq == nullptr || x == nullptr || y == nullptr) return FG_ERR_INVALID_ARG;
  if (M <= 0 || M > 16 || N <= 0 || K <= 0) return FG_ERR_INVALID_ARG;
  if (N % 128 != 0 || K % 128 != 0) return FG_ERR_ALIGN128;
  if ((reinterpret_cast<uintptr_t>(Wq) | reinterpret_cast<uintptr_t>(x)) & 15) {
    return FG_ERR_INVALID_ARG;
  }
  fg::W8A16Args a{Wq, x, scale, scalar_scale, zero_point, y, M, N, K};
  (void)hipGetLastError();
  if (!fg::launch_w8a16(a, static_cast<hipStream_t>(stream))) return FG_ERR_UNSUPPORTED;
  return fg::check_launch();
}

int fg_gemv_w4a16(const void* Wq4, const void* x, const void* scale, float scalar_scale,
                  float zero_point, void* y, int M, int N, int K, void* stream) {
  if (Wq4 == nullptr || x == nullptr || y == nullptr) return FG_ERR_INVALID_ARG;
  if (M <= 0 || M > 4 || N <= 0 || K <= 0) return FG_ERR_INVALID_ARG;
  if (N % 128 != 0 || K % 128 != 0) return FG_ERR_ALIGN128;
  if ((reinterpret_cast<uintptr_t>(Wq4) | reinterpret_cast<uintptr_t>(x)) & 15) {
    return FG_ERR_INVALID_ARG;
  }
  fg::W8A16Args a{Wq4, x, scale, scalar_scale, zero_point, y, M, N, K};
  (void)hipGetLastError();
  if (!fg::launch_w4a16(a, static_cast<hipStream_t>(stream))) return FG_ERR_UNSUPPORTED;
  return fg::check_launch();
}

int fg_gemv_i8i8_i32(const void* Wq, const void* xq, int32_t* acc, int M, int N, int K,
                     void* stream) {
  if (Wq == nullptr || xq == nullptr || acc == nullptr) return FG_ERR_INVALID_ARG;
  if (M <= 0 || M > 8 || N <= 0 || K <= 0) return FG_ERR_INVALID_ARG;
  if (N % 128 != 0 || K % 128 != 0) return FG_ERR_ALIGN128;
  if ((reinterpret_cast<uintptr_t>(Wq) | reinterpret_cast<uintptr_t>(xq)) & 15) {
    return FG_ERR_INVALID_ARG;
  }
  (void)hipGetLastError();
  if (!fg::launch_i8i8_i32(Wq, xq, acc, M, N, K, static_cast<hipStream_t>(stream))) {
    return FG_ERR_UNSUPPORTED;
  }
  return fg::check_launch();
}

int fg_dequant_i32_f16(const int32_t* acc, const void* scale, float x_scale, void* y, int M, int N,
                       void* stream) {
  if (acc == nullptr || y == nullptr || M <= 0 || N <= 0) return FG_ERR_INVALID_ARG;
  (void)hipGetLastError();
  fg::launch_dequant_i32_f16(acc, scale, x_scale, y, M, N, static_cast<hipStream_t>(stream));
  return fg::check_launch();
}

size_t fg_stream_read_sink_bytes(void) { return (size_t)fg::kStreamReadBlocks * sizeof(uint32_t); }

int fg_stream_read(const void* src, size_t bytes, void* sink, void* stream) {
  if (src == nullptr || sink == nullptr || bytes == 0 || (bytes & 15) ||
      (reinterpret_cast<uintptr_t>(src) & 15)) {
    return FG_ERR_INVALID_ARG;
  }
  (void)hipGetLastError();
  fg::launch_stream_read(src, bytes, sink, static_cast<hipStream_t>(stream));
  return fg::check_launch();
}

}  // extern "C"
