// pybind11 / ATen host layer: the reference's operator surface on top of libfastgate.
//
// Every function keeps the reference's name, argument order, argument meaning and C protocol
// (overwrite, or accumulate into a caller-zeroed C) and forwards to the C ABI in
// include/fastgate.h on the current HIP stream.  Tile sizes in the names are labels: all
// names route to the same shape-dispatched gfx950 kernels.  Reference files are cited
// relative to the root of chanzhennan/Fastgate:
//   backend/cuda/hk/edgemm.h:4-14, flatgemm.h:4-10, edgemm_tr.h:7-11, fastgemv.h:4-7,
//   backend/cuda/czn/fastgemm.h, backend/pybind.cpp:21-27.
//
// Error behaviour: K or N not a multiple of 128 -> std::invalid_argument (ValueError in
// Python) with the reference's wording, checked first as in the reference; everything the
// reference leaves unchecked (device, dtype, contiguity, shape agreement) -> c10::Error
// (RuntimeError) instead of undefined behaviour.  There is no CPU path.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <pybind11/pybind11.h>
#include <torch/extension.h>

#include <map>
#include <vector>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>

#include "fastgate.h"

namespace py = pybind11;

namespace {

void* current_stream(const at::Tensor& t) {
  return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

void raise_status(int st, const char* op) {
  if (st == FG_OK) return;
  const std::string msg = std::string(op) + ": " + fg_strerror(st);
  if (st == FG_ERR_ALIGN128 || st == FG_ERR_INVALID_ARG) throw std::invalid_argument(msg);
  throw std::runtime_error(msg);
}

void check_tensor(const at::Tensor& t, const char* name, at::ScalarType dtype, const char* op) {
  TORCH_CHECK(t.defined(), op, ": ", name, " is undefined");
  TORCH_CHECK(t.is_cuda(), op, ": ", name, " must live on a HIP device (got ", t.device(), ")");
  TORCH_CHECK(t.scalar_type() == dtype, op, ": ", name, " must be ", dtype, " (got ",
              t.scalar_type(), ")");
  TORCH_CHECK(t.is_contiguous(), op, ": ", name, " must be contiguous");
}

// Split-K scratch, one buffer per (device, stream), grown on demand through the caching
// allocator so that reuse is ordered on the stream that last used it.  Allocated zeroed: the
// header at its start (arrival counters and accumulator words) must be zero before the first
// call and every call leaves it zero.  The last buffer a thread used is remembered without a
// lock; only a change of device or stream, or growth, goes to the shared table.
struct Workspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};
Workspace workspace(int device, void* stream, const at::Tensor& like, size_t bytes) {
  struct Last {
    int device = -1;
    void* stream = nullptr;
    Workspace ws;
  };
  static thread_local Last last;
  if (last.device == device && last.stream == stream && last.ws.bytes >= bytes) return last.ws;
  static std::mutex mu;
  static std::map<std::pair<int, void*>, at::Tensor> cache;
  std::lock_guard<std::mutex> lock(mu);
  const auto key = std::make_pair(device, stream);
  auto it = cache.find(key);
  if (it == cache.end() || (size_t)it->second.numel() < bytes) {
    const size_t want = std::max<size_t>(bytes, (size_t)16 << 20);
    // a buffer that is outgrown stays allocated: another thread may still remember its address
    static std::vector<at::Tensor> outgrown;
    if (it != cache.end()) outgrown.push_back(it->second);
    cache[key] = at::zeros({(int64_t)want}, like.options().dtype(at::kByte));
    it = cache.find(key);
  }
  last.device = device;
  last.stream = stream;
  last.ws = Workspace{it->second.data_ptr(), (size_t)it->second.numel()};
  return last.ws;
}

// The library's plan for (M, N, K, layout), remembered per thread: planning walks a few hundred
// lines of rules, a call of a small shape takes a few microseconds in all.
const fg_plan_t& cached_plan(int M, int N, int K, int w_layout, int* status) {
  struct Entry {
    int M = 0, N = 0, K = 0, layout = -1, status = 0;
    fg_plan_t plan;
  };
  static thread_local Entry table[64];
  const unsigned h = ((unsigned)M * 2654435761u ^ (unsigned)N * 40503u ^ (unsigned)K * 2246822519u ^
                      (unsigned)w_layout) >> 7;
  Entry& e = table[h & 63];
  // plans are made for the compute units of the device the tensors live on (current here)
  static thread_local const int cus = fg_use_device_compute_units();
  (void)cus;
  if (e.M != M || e.N != N || e.K != K || e.layout != w_layout) {
    e.status = fg_plan(M, N, K, w_layout, 0, &e.plan);
    e.M = M, e.N = N, e.K = K, e.layout = w_layout;
  }
  *status = e.status;
  return e.plan;
}

// Plan of a GEMM operator call.  `bz` is the reference's split-K factor, tuned for another GPU
// (its scripts pass 1 and 2, which would leave three quarters of this one idle): it is accepted
// and does not enter the plan.  fg_gemm_f16's own `splitk` argument is the way to force a split.
const fg_plan_t& call_plan(int M, int N, int K, int w_layout, int bz, int* status) {
  (void)bz;
  return cached_plan(M, N, K, w_layout, status);
}

enum Protocol { kOverwrite = 0, kAccumulate = 1 };

// C = A·W or C += A·W for fp16 tensors; `msg128` is the reference's exception text.
// With `tail` set: C = act(A·W + bias) (bias may be undefined), always overwriting C.
void gemm(const char* op, const at::Tensor& A, const at::Tensor& W, at::Tensor& C, int w_layout,
          Protocol protocol, int bz, const char* msg128, bool tail = false,
          const at::Tensor& bias = at::Tensor(), int act = FG_ACT_NONE) {
  TORCH_CHECK(A.dim() == 2 && W.dim() == 2, op, ": A and B must be 2-D");
  const int64_t M = A.size(0), K = A.size(1);
  const int64_t N = w_layout == FG_W_KN ? W.size(1) : W.size(0);
  if (N % 128 || K % 128) throw std::invalid_argument(msg128);
  TORCH_CHECK(bz >= 0, op, ": bz must be non-negative");
  check_tensor(A, "A", at::kHalf, op);
  // B[K,N] may be a view of padded weights: rows W.stride(0) >= N elements apart (a multiple of 8),
  // unit stride along N.  The reference's tensors are dense; a pitch of N + 128 is about 9 % faster
  // where N is a multiple of 512.
  const bool pitched = w_layout == FG_W_KN && !tail && W.defined() && !W.is_contiguous() &&
                       W.stride(1) == 1 && W.stride(0) >= N && W.stride(0) % 8 == 0 &&
                       W.stride(0) <= INT32_MAX;
  if (pitched) {
    TORCH_CHECK(W.is_cuda(), op, ": B must live on a HIP device (got ", W.device(), ")");
    TORCH_CHECK(W.scalar_type() == at::kHalf, op, ": B must be Half (got ", W.scalar_type(), ")");
  } else {
    check_tensor(W, "B", at::kHalf, op);
  }
  check_tensor(C, "C", at::kHalf, op);
  const int64_t Kw = w_layout == FG_W_KN ? W.size(0) : W.size(1);
  TORCH_CHECK(Kw == K, op, ": inner dimensions differ (A has K=", K, ", B has K=", Kw, ")");
  TORCH_CHECK(C.numel() == M * N, op, ": C must hold M*N = ", M * N, " elements (got ", C.numel(),
              ")");
  TORCH_CHECK(A.device() == W.device() && A.device() == C.device(), op,
              ": tensors are on different devices");
  TORCH_CHECK(M > 0, op, ": A has no rows");
  TORCH_CHECK(M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX, op, ": size overflow");

  c10::hip::HIPGuardMasqueradingAsCUDA guard(A.device());
  int st;
  fg_plan_t plan = call_plan((int)M, (int)N, (int)K, w_layout, bz, &st);
  raise_status(st, op);
  void* stream = current_stream(A);
  Workspace ws;
  if (plan.workspace_bytes) ws = workspace((int)A.device().index(), stream, A, plan.workspace_bytes);
  if (tail) {
    const void* bias_ptr = nullptr;
    if (bias.defined()) {
      check_tensor(bias, "bias", at::kHalf, op);
      TORCH_CHECK(bias.numel() == N && bias.device() == A.device(), op,
                  ": bias must hold N = ", N, " elements on the device of A");
      bias_ptr = bias.data_ptr();
    }
    st = fg_gemm_f16_bias_act(A.data_ptr(), W.data_ptr(), bias_ptr, act, C.data_ptr(), (int)M,
                              (int)N, (int)K, w_layout, 0, &plan, ws.ptr, ws.bytes, stream);
  } else if (pitched) {
    st = fg_gemm_f16_pitched(A.data_ptr(), W.data_ptr(), C.data_ptr(), (int)M, (int)N, (int)K,
                             (int)W.stride(0), protocol == kAccumulate, 0, ws.ptr, ws.bytes, stream);
  } else {
    st = fg_gemm_f16_planned(A.data_ptr(), W.data_ptr(), C.data_ptr(), (int)M, (int)N, (int)K,
                             w_layout, protocol == kAccumulate, &plan, ws.ptr, ws.bytes, stream);
  }
  raise_status(st, op);
}

int act_id(const std::string& act, const char* op) {
  if (act == "none") return FG_ACT_NONE;
  if (act == "relu") return FG_ACT_RELU;
  if (act == "gelu") return FG_ACT_GELU;
  if (act == "gelu_tanh") return FG_ACT_GELU_TANH;
  if (act == "silu") return FG_ACT_SILU;
  throw std::invalid_argument(std::string(op) + ": act must be none, relu, gelu, gelu_tanh or silu");
}

at::Tensor optional_tensor(const py::object& o) {
  return o.is_none() ? at::Tensor() : o.cast<at::Tensor>();
}

const char* kMsgKN = "K(input column) & N(output column) must be multiple of 128!";
const char* kMsgNK = "K(input column) & N(transposed output row) must be multiple of 128!";

// --- name tables -----------------------------------------------------------------------
struct OpSpec {
  const char* name;
  int layout;
  Protocol protocol;
  const char* msg;
  const char* doc;
};

// (A[M,K], B, C[M,N]) operators without a split-K argument.
const OpSpec kOps3[] = {
    // backend/cuda/hk/edgemm.cu
    {"edgemm", FG_W_KN, kOverwrite, kMsgKN, "C = A @ B, B[K,N] (hk/edgemm.cu:12-39)"},
    {"edgemm_m8n256k64", FG_W_KN, kOverwrite, kMsgKN, "C = A @ B, B[K,N] (hk/edgemm.cu:41-70)"},
    {"edgemm_m8n128k64", FG_W_KN, kOverwrite, kMsgKN, "C = A @ B, B[K,N] (hk/edgemm.cu:72-99)"},
    {"edgemm_m8n128k128", FG_W_KN, kOverwrite, kMsgKN, "C = A @ B, B[K,N] (hk/edgemm.cu:327-354)"},
    {"edgemm_m8n128k64x4", FG_W_KN, kOverwrite, kMsgKN, "C = A @ B, B[K,N] (hk/edgemm.cu:102-156)"},
    {"edgemm_m8n128k64x4_amd", FG_W_KN, kOverwrite, kMsgKN,
     "C = A @ B, B[K,N], any M <= 16 in one block row (hk/edgemm.cu:159-213)"},
    {"edgemm_m8n128k64x4_tr_amd", FG_W_NK, kOverwrite, kMsgKN,
     "C = A @ B_t.T, B_t[N,K] (hk/edgemm.cu:216-270)"},
    {"edgemm_m8n128k64x4_bt", FG_W_NK, kOverwrite, kMsgNK,
     "C = A @ B_t.T, B_t[N,K] (hk/edgemm.cu:274-324)"},
    {"edgemm_m8n256k32x8", FG_W_KN, kAccumulate, kMsgKN,
     "C += A @ B, B[K,N]; C is not zeroed (hk/edgemm.cu:363-385)"},
    {"edgemv_m1n128k64x4", FG_W_KN, kAccumulate, kMsgKN,
     "C += A @ B, B[K,N]; C is not zeroed (hk/edgemm.cu:388-416)"},
    {"edgemv_m1n256k64x4", FG_W_KN, kAccumulate, kMsgKN,
     "C += A @ B, B[K,N]; C is not zeroed (hk/edgemm.cu:418-445)"},
    // backend/cuda/hk/flatgemm.cu
    {"flat_gemm_m8n256k32x8_bz1", FG_W_KN, kOverwrite, kMsgNK,
     "C = A @ B, B[K,N] (hk/flatgemm.cu:34-52)"},
    {"flat_gemm_m8n256k32x16", FG_W_KN, kOverwrite, kMsgKN,
     "C = A @ B, B[K,N] (hk/flatgemm.cu:81-104)"},
    // backend/cuda/hk/edgemm_tr.cu
    {"gemm_m8n128k64x4_bt", FG_W_NK, kOverwrite, kMsgKN,
     "C = A @ B_t.T, B_t[N,K], M <= 16 per block row (hk/edgemm_tr.cu:19-50)"},
    {"gemm_m8n32k128x8_bt", FG_W_NK, kAccumulate, kMsgNK,
     "C += A @ B_t.T, B_t[N,K]; C is not zeroed (hk/edgemm_tr.cu:55-72)"},
    {"gemm_m8n32k256x8_bt", FG_W_NK, kAccumulate, kMsgNK,
     "C += A @ B_t.T, B_t[N,K]; C is not zeroed (hk/edgemm_tr.cu:99-116)"},
};

// (A, B, C, bz) operators: bz, the reference's split-K factor, is accepted and not used.
const OpSpec kOps4[] = {
    {"flat_gemm_m8n128k64x4_bz1", FG_W_KN, kAccumulate, kMsgNK,
     "C += A @ B, B[K,N], split-K bz (hk/flatgemm.cu:13-32)"},
    {"flat_gemm_m8n256k64x8", FG_W_KN, kAccumulate, kMsgKN,
     "C += A @ B, B[K,N], split-K bz (hk/flatgemm.cu:55-79)"},
    {"flat_gemm_m8n512k32x16", FG_W_KN, kAccumulate, kMsgKN,
     "C += A @ B, B[K,N], split-K bz (hk/flatgemm.cu:106-129)"},
    {"flat_gemm_m8n64k128x8", FG_W_KN, kAccumulate, kMsgNK,
     "C += A @ B, B[K,N], split-K bz (hk/flatgemm.cu:132-149)"},
    {"flat_gemm_m8n32k256x8", FG_W_KN, kAccumulate, kMsgNK,
     "C += A @ B, B[K,N], split-K bz (hk/flatgemm.cu:152-169)"},
    {"gemm_m8n64k128x8_bt_exp", FG_W_NK, kAccumulate, kMsgNK,
     "C += A @ B_t.T, B_t[N,K], split-K bz (hk/edgemm_tr.cu:77-94)"},
    {"gemm_m8n32k256x8_bt_bz2", FG_W_NK, kAccumulate, kMsgNK,
     "C += A @ B_t.T, B_t[N,K], split-K bz (hk/edgemm_tr.cu:122-139)"},
};

// --- GEMV family: weight first ------------------------------------------------------------
// mat[N,K]; vec holds M*K contiguous elements ([1,K], [K,1], [K] for M = 1, [M,K] otherwise);
// res holds M*N elements, row-major [M,N].
void gemv_f16(const char* op, const at::Tensor& mat, const at::Tensor& vec, at::Tensor& res) {
  TORCH_CHECK(mat.dim() == 2, op, ": mat must be 2-D [N,K]");
  const int64_t N = mat.size(0), K = mat.size(1);
  if (N % 128 || K % 128) throw std::invalid_argument(kMsgNK);
  check_tensor(mat, "mat", at::kHalf, op);
  check_tensor(vec, "vec", at::kHalf, op);
  check_tensor(res, "res", at::kHalf, op);
  TORCH_CHECK(vec.numel() > 0 && vec.numel() % K == 0, op, ": vec must hold a multiple of K = ", K,
              " elements (got ", vec.numel(), ")");
  const int64_t M = vec.numel() / K;
  TORCH_CHECK(M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX, op, ": size overflow");
  TORCH_CHECK(M == 1 || (vec.dim() == 2 && vec.size(1) == K), op, ": batched vec must be [M,K]");
  TORCH_CHECK(res.numel() == M * N, op, ": res must hold M*N = ", M * N, " elements (got ",
              res.numel(), ")");
  TORCH_CHECK(mat.device() == vec.device() && mat.device() == res.device(), op,
              ": tensors are on different devices");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(mat.device());
  int st;
  fg_plan_t plan = cached_plan((int)M, (int)N, (int)K, FG_W_NK, &st);
  raise_status(st, op);
  void* stream = current_stream(mat);
  Workspace ws;
  if (plan.workspace_bytes) ws = workspace((int)mat.device().index(), stream, mat, plan.workspace_bytes);
  raise_status(fg_gemm_f16_planned(vec.data_ptr(), mat.data_ptr(), res.data_ptr(), (int)M, (int)N, (int)K,
                                   FG_W_NK, 0, &plan, ws.ptr, ws.bytes, stream),
               op);
}

void fastgemv(at::Tensor mat, at::Tensor vec, at::Tensor res) { gemv_f16("fastgemv", mat, vec, res); }
void fastgemv_tuned(at::Tensor mat, at::Tensor vec, at::Tensor res) {
  gemv_f16("fastgemv_tuned", mat, vec, res);
}
void fastgemv_extend(at::Tensor mat, at::Tensor vec, at::Tensor res) {
  gemv_f16("fastgemv_extend", mat, vec, res);
}
void fastgemm(at::Tensor mat, at::Tensor vec, at::Tensor res) { gemv_f16("fastgemm", mat, vec, res); }

// fastgemv_int8(mat_i8[N,K], vec_f16, res_f16): the reference's host passes (1.0, 0.0) into the
// kernel's (scale, zero_point) slots (hk/fastgemv.cu:50-60), so the defaults are scale 1 and
// zero point 0.  `scale` (fp16 [N]) is this library's per-output-channel extension.
void fastgemv_int8(at::Tensor mat, at::Tensor vec, at::Tensor res, c10::optional<at::Tensor> scale,
                   double scalar_scale, double zero_point) {
  const char* op = "fastgemv_int8";
  TORCH_CHECK(mat.dim() == 2, op, ": mat must be 2-D [N,K]");
  const int64_t N = mat.size(0), K = mat.size(1);
  if (N % 128 || K % 128) throw std::invalid_argument(kMsgNK);
  check_tensor(mat, "mat", at::kChar, op);
  check_tensor(vec, "vec", at::kHalf, op);
  check_tensor(res, "res", at::kHalf, op);
  TORCH_CHECK(vec.numel() > 0 && vec.numel() % K == 0, op, ": vec must hold a multiple of K = ", K,
              " elements");
  const int64_t M = vec.numel() / K;
  TORCH_CHECK(M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX, op, ": size overflow");
  TORCH_CHECK(M <= 16, op, ": at most 16 activation rows");
  TORCH_CHECK(res.numel() == M * N, op, ": res must hold M*N = ", M * N, " elements");
  const void* sp = nullptr;
  if (scale.has_value() && scale->defined()) {
    check_tensor(*scale, "scale", at::kHalf, op);
    TORCH_CHECK(scale->numel() == N, op, ": scale must hold N = ", N, " elements");
    TORCH_CHECK(scale->device() == mat.device(), op, ": scale is on a different device");
    sp = scale->data_ptr();
  }
  TORCH_CHECK(mat.device() == vec.device() && mat.device() == res.device(), op,
              ": tensors are on different devices");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(mat.device());
  raise_status(fg_gemv_w8a16(mat.data_ptr(), vec.data_ptr(), sp, (float)scalar_scale,
                             (float)zero_point, res.data_ptr(), (int)M, (int)N, (int)K,
                             current_stream(mat)),
               op);
}

// fastgemv_int4(mat_u8[N,K/2], vec_f16, res_f16): the formula of gemv_quantized_int4
// (hk/fastgemv.cuh:394-495), which the reference defines without a host function or binding.
// Two unsigned 4-bit weights per byte, even element in the low nibble (hk/utility.cuh:13-36).
void fastgemv_int4(at::Tensor mat, at::Tensor vec, at::Tensor res, c10::optional<at::Tensor> scale,
                   double scalar_scale, double zero_point) {
  const char* op = "fastgemv_int4";
  TORCH_CHECK(mat.dim() == 2, op, ": mat must be 2-D [N,K/2]");
  const int64_t N = mat.size(0), K = mat.size(1) * 2;
  if (N % 128 || K % 128) throw std::invalid_argument(kMsgNK);
  check_tensor(mat, "mat", at::kByte, op);
  check_tensor(vec, "vec", at::kHalf, op);
  check_tensor(res, "res", at::kHalf, op);
  TORCH_CHECK(vec.numel() > 0 && vec.numel() % K == 0, op, ": vec must hold a multiple of K = ", K,
              " elements");
  const int64_t M = vec.numel() / K;
  TORCH_CHECK(M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX, op, ": size overflow");
  TORCH_CHECK(M <= 4, op, ": at most 4 activation rows");
  TORCH_CHECK(res.numel() == M * N, op, ": res must hold M*N = ", M * N, " elements");
  const void* sp = nullptr;
  if (scale.has_value() && scale->defined()) {
    check_tensor(*scale, "scale", at::kHalf, op);
    TORCH_CHECK(scale->numel() == N, op, ": scale must hold N = ", N, " elements");
    TORCH_CHECK(scale->device() == mat.device(), op, ": scale is on a different device");
    sp = scale->data_ptr();
  }
  TORCH_CHECK(mat.device() == vec.device() && mat.device() == res.device(), op,
              ": tensors are on different devices");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(mat.device());
  raise_status(fg_gemv_w4a16(mat.data_ptr(), vec.data_ptr(), sp, (float)scalar_scale,
                             (float)zero_point, res.data_ptr(), (int)M, (int)N, (int)K,
                             current_stream(mat)),
               op);
}

// Integer stage: acc_i32[M,N] = xq_i8[M,K] · mat_i8[N,K]^T (exact).
void gemv_i8i8_i32(at::Tensor mat, at::Tensor xq, at::Tensor acc) {
  const char* op = "gemv_i8i8_i32";
  TORCH_CHECK(mat.dim() == 2, op, ": mat must be 2-D [N,K]");
  const int64_t N = mat.size(0), K = mat.size(1);
  if (N % 128 || K % 128) throw std::invalid_argument(kMsgNK);
  check_tensor(mat, "mat", at::kChar, op);
  check_tensor(xq, "xq", at::kChar, op);
  check_tensor(acc, "acc", at::kInt, op);
  TORCH_CHECK(xq.numel() > 0 && xq.numel() % K == 0, op, ": xq must hold a multiple of K elements");
  const int64_t M = xq.numel() / K;
  TORCH_CHECK(M <= 8, op, ": at most 8 activation rows");
  TORCH_CHECK(acc.numel() == M * N, op, ": acc must hold M*N elements");
  TORCH_CHECK(mat.device() == xq.device() && mat.device() == acc.device(), op,
              ": tensors are on different devices");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(mat.device());
  raise_status(fg_gemv_i8i8_i32(mat.data_ptr(), xq.data_ptr(), acc.data_ptr<int32_t>(), (int)M,
                                (int)N, (int)K, current_stream(mat)),
               op);
}

// y_f16[M,N] = acc_i32 * x_scale * scale[n]
void dequant_i32_f16(at::Tensor acc, c10::optional<at::Tensor> scale, double x_scale, at::Tensor y) {
  const char* op = "dequant_i32_f16";
  check_tensor(acc, "acc", at::kInt, op);
  check_tensor(y, "y", at::kHalf, op);
  TORCH_CHECK(acc.dim() == 2 && y.numel() == acc.numel(), op, ": acc must be [M,N], y M*N elements");
  const void* sp = nullptr;
  if (scale.has_value() && scale->defined()) {
    check_tensor(*scale, "scale", at::kHalf, op);
    TORCH_CHECK(scale->numel() == acc.size(1), op, ": scale must hold N elements");
    sp = scale->data_ptr();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(acc.device());
  raise_status(fg_dequant_i32_f16(acc.data_ptr<int32_t>(), sp, (float)x_scale, y.data_ptr(),
                                  (int)acc.size(0), (int)acc.size(1), current_stream(acc)),
               op);
}

// Vendor comparators the reference binds next to its own kernels: hgemm (hk/hgemm.cu:29-74,
// cuBLAS there, hipBLASLt through ATen here), hgemm_tr (hk/hgemm_tr.cu:30-75) and mma
// (czn/mma.cu:19-88, large-M GEMM with B[N,K]).
void hgemm(at::Tensor A, at::Tensor B, at::Tensor C) { at::matmul_out(C, A, B); }
void hgemm_tr(at::Tensor A, at::Tensor B, at::Tensor C) { at::matmul_out(C, A, B.t()); }
void mma(at::Tensor A, at::Tensor B, at::Tensor C) { at::matmul_out(C, A, B.t()); }

py::dict plan_dict(const fg_plan_t& p) {
  py::dict d;
  d["kernel"] = p.kernel;
  d["splitk"] = p.splitk;
  d["fused"] = p.fused;
  d["tile_n"] = p.tile_n;
  d["m_block"] = p.m_block;
  d["waves"] = p.waves;
  d["unroll"] = p.unroll;
  d["stream_w"] = p.stream_w;
  d["stagger"] = p.stagger;
  d["band"] = p.band;
  d["grid"] = py::make_tuple(p.grid_x, p.grid_y, p.grid_z);
  d["block"] = p.block;
  d["workspace_bytes"] = p.workspace_bytes;
  return d;
}

py::dict plan(int M, int N, int K, int w_layout, int splitk) {
  fg_plan_t p;
  const int st = fg_plan(M, N, K, w_layout, splitk, &p);
  raise_status(st, "plan");
  return plan_dict(p);
}

// The plan operator `name` runs for a shape and a `bz` argument (host only).
py::dict plan_dict(const fg_plan_t& p);
py::dict plan_for(const std::string& name, int M, int N, int K, int bz) {
  const OpSpec* spec = nullptr;
  for (const OpSpec& s : kOps3)
    if (name == s.name) spec = &s;
  for (const OpSpec& s : kOps4)
    if (name == s.name) spec = &s;
  if (spec == nullptr) throw std::invalid_argument("plan_for: unknown GEMM operator " + name);
  if (N % 128 || K % 128) throw std::invalid_argument(spec->msg);
  int st;
  const fg_plan_t p = call_plan(M, N, K, spec->layout, bz, &st);
  raise_status(st, "plan_for");
  return plan_dict(p);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "MI355X-native small-batch GEMM/GEMV operators with the Fastgate operator surface";
  for (const OpSpec& s : kOps3) {
    const OpSpec spec = s;
    m.def(
        spec.name,
        [spec](at::Tensor A, at::Tensor B, at::Tensor C) {
          gemm(spec.name, A, B, C, spec.layout, spec.protocol, 0, spec.msg);
        },
        py::arg("A"), py::arg("B"), py::arg("C"), spec.doc);
  }
  for (const OpSpec& s : kOps4) {
    const OpSpec spec = s;
    m.def(
        spec.name,
        [spec](at::Tensor A, at::Tensor B, at::Tensor C, int bz) {
          gemm(spec.name, A, B, C, spec.layout, spec.protocol, bz, spec.msg);
        },
        py::arg("A"), py::arg("B"), py::arg("C"), py::arg("bz"), spec.doc);
  }
  m.def("fastgemv", &fastgemv, py::arg("mat"), py::arg("vec"), py::arg("res"),
        "res[N] = mat[N,K] @ vec[K]; weight first (hk/fastgemv.cu:12-33)");
  m.def("fastgemv_tuned", &fastgemv_tuned, py::arg("mat"), py::arg("vec"), py::arg("res"),
        "as fastgemv (hk/fastgemv.cu:63-84); accumulates in fp32 here");
  m.def("fastgemv_extend", &fastgemv_extend, py::arg("mat"), py::arg("vec"), py::arg("res"),
        "res[M,N] = vec[M,K] @ mat[N,K].T (hk/fastgemv.cu:86-111)");
  m.def("fastgemm", &fastgemm, py::arg("mat"), py::arg("vec"), py::arg("res"),
        "res[M,N] = vec[M,K] @ mat[N,K].T, M in {1,2} in the reference (czn/fastgemm.cu:13-55)");
  m.def("fastgemv_int8", &fastgemv_int8, py::arg("mat"), py::arg("vec"), py::arg("res"),
        py::arg("scale") = py::none(), py::arg("scalar_scale") = 1.0, py::arg("zero_point") = 0.0,
        "res = (vec @ (mat_i8[N,K] - zero_point).T) * scalar_scale * scale[N] "
        "(hk/fastgemv.cu:35-61; per-channel scale is an extension)");
  m.def("fastgemv_int4", &fastgemv_int4, py::arg("mat"), py::arg("vec"), py::arg("res"),
        py::arg("scale") = py::none(), py::arg("scalar_scale") = 1.0, py::arg("zero_point") = 0.0,
        "res = (vec @ (mat_u4[N,K] - zero_point).T) * scalar_scale * scale[N]; mat is uint8 [N,K/2], "
        "even element in the low nibble (formula of hk/fastgemv.cuh:394-495)");
  m.def(
      "gemm_bias_act",
      [](at::Tensor A, at::Tensor B, at::Tensor C, py::object bias, const std::string& act) {
        gemm("gemm_bias_act", A, B, C, FG_W_KN, kOverwrite, 0, kMsgKN, true, optional_tensor(bias),
             act_id(act, "gemm_bias_act"));
      },
      py::arg("A"), py::arg("B"), py::arg("C"), py::arg("bias") = py::none(),
      py::arg("act") = "none",
      "C = act(A @ B + bias), B[K,N]; bias fp16 [N] or None; act in none, relu, gelu, gelu_tanh, "
      "silu (no counterpart in the reference: the tail of an FFN up-projection, fused)");
  m.def(
      "gemm_bias_act_bt",
      [](at::Tensor A, at::Tensor B_t, at::Tensor C, py::object bias, const std::string& act) {
        gemm("gemm_bias_act_bt", A, B_t, C, FG_W_NK, kOverwrite, 0, kMsgNK, true,
             optional_tensor(bias), act_id(act, "gemm_bias_act_bt"));
      },
      py::arg("A"), py::arg("B_t"), py::arg("C"), py::arg("bias") = py::none(),
      py::arg("act") = "none", "C = act(A @ B_t.T + bias), B_t[N,K]");
  m.def(
      "ffn_bt",
      [](at::Tensor A, at::Tensor W1_t, py::object b1, at::Tensor W2_t, py::object b2, at::Tensor H,
         at::Tensor C, const std::string& act) {
        const int a = act_id(act, "ffn_bt");
        gemm("ffn_bt (up)", A, W1_t, H, FG_W_NK, kOverwrite, 0, kMsgNK, true, optional_tensor(b1), a);
        gemm("ffn_bt (down)", H, W2_t, C, FG_W_NK, kOverwrite, 0, kMsgNK, true, optional_tensor(b2),
             FG_ACT_NONE);
      },
      py::arg("A"), py::arg("W1_t"), py::arg("b1"), py::arg("W2_t"), py::arg("b2"), py::arg("H"),
      py::arg("C"), py::arg("act") = "gelu",
      "feed-forward pair in two launches: H = act(A @ W1_t.T + b1), C = H @ W2_t.T + b2; "
      "W1_t[N1,K], W2_t[N2,N1], H[M,N1] and C[M,N2] caller allocated");
  m.def("gemv_i8i8_i32", &gemv_i8i8_i32, py::arg("mat"), py::arg("xq"), py::arg("acc"),
        "acc_i32[M,N] = xq_i8[M,K] @ mat_i8[N,K].T, exact");
  m.def("dequant_i32_f16", &dequant_i32_f16, py::arg("acc"), py::arg("scale"), py::arg("x_scale"),
        py::arg("y"), "y_f16 = acc_i32 * x_scale * scale[N]");
  m.def("hgemm", &hgemm, "C = A @ B through the vendor GEMM (hk/hgemm.cu:29-74)");
  m.def("hgemm_tr", &hgemm_tr, "C = A @ B_t.T through the vendor GEMM (hk/hgemm_tr.cu:30-75)");
  m.def("mma", &mma, "C = A @ B_t.T through the vendor GEMM (czn/mma.cu:19-88)");
  m.def("plan", &plan, py::arg("M"), py::arg("N"), py::arg("K"), py::arg("w_layout"),
        py::arg("splitk") = 0, "launch plan the library picks for a shape (host only)");
  m.def("plan_for", &plan_for, py::arg("name"), py::arg("M"), py::arg("N"), py::arg("K"), py::arg("bz") = 0,
        "launch plan operator `name` uses for a shape; bz is accepted and does not enter (host only)");
  m.attr("W_KN") = (int)FG_W_KN;
  m.attr("W_NK") = (int)FG_W_NK;
}
