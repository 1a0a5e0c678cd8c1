/*
 * libfastgate — C ABI of the MI355X (gfx950) small-batch GEMM / GEMV library.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its kernels on the
 * HIP stream it is given (a hipStream_t passed as void*; NULL = the null stream), returns
 * 0 or a negative fg_status, never throws and never allocates device memory.  The library
 * keeps no state.  There is no CPU path: without a HIP device every compute call fails
 * with FG_ERR_LAUNCH.
 *
 * The reference (chanzhennan/Fastgate, paths relative to its root) exposes this path as
 * C++ host functions `void f(at::Tensor A, at::Tensor B, at::Tensor C[, int bz])`; each
 * declaration below cites the host functions it services.  The pybind11 module `speedgate`
 * keeps those names and argument conventions and forwards to these entry points.
 *
 * Common conventions
 *   A      fp16 [M,K] row-major activations (contiguous)
 *   W      fp16 weights, w_layout FG_W_KN = [K,N] row-major, FG_W_NK = [N,K] row-major
 *   C      fp16 [M,N] row-major, caller allocated
 *   K, N   multiples of 128 (the reference's only documented constraint, README.md:6-12)
 *   M      any positive value; the kernels are meant for M = 1..16 (one pass over the weights up
 *          to 32 rows with [N,K] weights, one more pass per further 32 / 16 rows)
 *   arithmetic: fp16 products, fp32 accumulation, one rounding to fp16 at the end
 */
#ifndef FASTGATE_H_
#define FASTGATE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FG_VERSION 110

typedef enum fg_status {
  FG_OK = 0,
  FG_ERR_INVALID_ARG = -1, /* null pointer, non-positive size, bad enum value        */
  FG_ERR_ALIGN128 = -2,    /* K or N not a multiple of 128 (reference: invalid_argument) */
  FG_ERR_WORKSPACE = -3,   /* split-K requested/needed and workspace missing or small */
  FG_ERR_LAUNCH = -4,      /* HIP reported an error at launch (no device, bad stream) */
  FG_ERR_UNSUPPORTED = -5, /* plan names a kernel/tile combination that does not exist */
  FG_ERR_SCRATCH_LIMIT = -6 /* fg_gemm_f16_static: the shape's split-K partials exceed
                               FG_STATIC_SCRATCH_BYTES                                   */
} fg_status;

enum { FG_W_KN = 0, FG_W_NK = 1 };

/* Kernel families (fg_plan_t.kernel). */
enum {
  FG_KERNEL_AUTO = 0,
  FG_KERNEL_NK_DOT2 = 1, /* [N,K] weights, lanes along K, v_dot2_f32_f16                */
  FG_KERNEL_KN_DOT2 = 3, /* [K,N] weights, 8x8 register transpose + v_dot2_f32_f16       */
  FG_KERNEL_KN_MFMA = 4, /* [K,N] weights, 8x8 register transpose + MFMA                 */
  FG_KERNEL_NK_MFMA4 = 5, /* [N,K] weights, v_mfma_f32_4x4x4_16B_f16: 4 rows x 256 B a load */
  FG_KERNEL_NK_MFMA_R = 8  /* [N,K] weights, 16x16x32 MFMA, 16- to 64-column tiles, weights AND
                              activations loaded as contiguous row pieces and transposed in
                              wave-private LDS; fills the chip without split-K                */
};

/*
 * Launch plan for one fg_gemm_f16 call.  fg_plan() fills it with the library's choice;
 * fg_gemm_f16_planned() accepts a caller-edited copy (the shape sweep uses this to
 * compare kernels and split-K factors).  Fields a kernel family does not use are ignored.
 */
typedef struct fg_plan_t {
  int kernel;   /* FG_KERNEL_*                                                        */
  int splitk;   /* S >= 1: K is divided over S workgroups per output tile.  S > 1 needs the
                   workspace; how the S partial sums of an element meet is `fused`.  Every
                   completion is reproducible run to run (none depends on arrival order)  */
  int fused;    /* with S > 1, how the split completes:
                   0 = fp32 partials [S,M,N] go to the workspace and a second kernel sums them;
                   1 = same partials; the workgroup that finishes a tile last sums them in the
                       same launch (one counter atomic per workgroup);
                   2 = every workgroup adds its partial, in 2^-28 fixed point, to the element's
                       64-bit word of the workspace header with one atomic, and the arrival
                       that completes an element writes it (S <= 31, M*N <= 262144).  Partials
                       stay out of memory except those fixed point cannot hold (not finite, or
                       of magnitude 2^20 and more): these go to their [S,M,N] slot and are
                       added in fp32, in ascending order of S, when the element completes;
                   3 = FG_KERNEL_KN_MFMA only, S <= 32: the S workgroups of a tile run on one
                       XCD and hand their partials over through that XCD's L2, announced by
                       per-wave flag words in the workspace header that carry a tag unique to
                       the launch; the workgroup with the last K range sums them.  If the
                       partners are not on its XCD or stay silent it computes their K ranges
                       itself (same result, slower);
                   4 = as 3 with a fifth of the workgroups taking that fallback on purpose (for
                       tests).
                   0, 1, 3 and 4 sum in ascending order of S in fp32 and agree bit for bit; 2
                   sums exactly and may differ from them in the last bit                  */
  int tile_n;   /* output columns per workgroup; FG_KERNEL_NK_MFMA_R takes 16, 32, 48, 64 or,
                   with band = 128, 8 waves and no split, any divisor of N from 17 to 47  */
  int m_block;  /* rows of A per workgroup (grid.y = ceil(M / m_block))               */
  int waves;    /* wavefronts per workgroup; they interleave over K, reduced in LDS   */
  int unroll;   /* independent 16-byte load groups in flight per lane and step        */
  int stream_w; /* 1 = weight loads carry the non-temporal hint                       */
  int stagger;  /* K-interleaved [N,K] kernels start each workgroup at its own K step:
                   0 = (workgroup id / 8) % steps, spread within every XCD (default);
                   1 = workgroup id % steps, one K band per XCD (only with 8 steps)  */
  int band;     /* FG_KERNEL_NK_MFMA_R only: bytes of K per weight row and step, 128, 256 or
                   512 (0 = 256 * unroll); a narrower band halves the activation bytes a
                   32-column tile re-reads, a wider one halves the load instructions   */
  int grid_x, grid_y, grid_z, block; /* filled by fg_plan / fg_gemm_f16_planned       */
  size_t workspace_bytes;            /* 0 when splitk == 1                            */
} fg_plan_t;

/*
 * C = A·W (accumulate = 0) or C += A·W (accumulate = 1; C holds fp16 on entry and the sum
 * is formed in fp32 before the single rounding).
 *   splitk  0 = library heuristic, S >= 1 = forced.  (The reference's trailing `int bz` is a split
 *           factor tuned for another GPU; the pybind layer accepts it and passes 0 here.)  With 0 and
 *           no (or too small a) workspace the call runs unsplit instead of failing; a forced
 *           S > 1 without workspace is FG_ERR_WORKSPACE.
 *   ws      device scratch of at least fg_workspace_bytes() bytes when the plan's
 *           splitk > 1, else may be NULL.  Its first fg_workspace_header_bytes() bytes (64 KiB of
 *           arrival counters, 3 MiB of per-element accumulator words, 512 KiB of flag words)
 *           must be zero before the first call (a library older than FG_VERSION 110 had a
 *           shorter header: size the clear from fg_workspace_header_bytes(), never a
 *           constant): zero them once with fg_workspace_init() (or allocate zeroed memory).
 *           Every call leaves counters and accumulator words zero again; flag words keep the
 *           tag of the launch that wrote them, which no later launch takes for its own.
 *           Calls that share a workspace must not overlap: order them on one stream, or
 *           with events.
 * Services, with w_layout = FG_W_KN: edgemm_m8n128k64x4 (backend/cuda/hk/edgemm.cu:102-156),
 * edgemm_m8n128k64x4_amd (:159-213), edgemm_m8n256k32x8 (:363-385, accumulate),
 * flat_gemm_m8n128k64x4_bz1, flat_gemm_m8n256k32x8_bz1, flat_gemm_m8n256k64x8,
 * flat_gemm_m8n256k32x16, flat_gemm_m8n512k32x16, flat_gemm_m8n64k128x8,
 * flat_gemm_m8n32k256x8 (backend/cuda/hk/flatgemm.cu:13-169), hgemm (hk/hgemm.cu:29-74);
 * with w_layout = FG_W_NK: edgemm_m8n128k64x4_bt (hk/edgemm.cu:274-324),
 * edgemm_m8n128k64x4_tr_amd (:216-270), gemm_m8n128k64x4_bt, gemm_m8n32k128x8_bt,
 * gemm_m8n64k128x8_bt_exp, gemm_m8n32k256x8_bt, gemm_m8n32k256x8_bt_bz2
 * (backend/cuda/hk/edgemm_tr.cu:19-139), fastgemv, fastgemv_tuned, fastgemv_extend
 * (backend/cuda/hk/fastgemv.cu:12-33,63-111), fastgemm (backend/cuda/czn/fastgemm.cu:13-55).
 */
int fg_gemm_f16(const void* A, const void* W, void* C, int M, int N, int K, int w_layout,
                int accumulate, int splitk, void* ws, size_t ws_bytes, void* stream);

/*
 * fg_gemm_f16 without the workspace arguments, for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  The split-K workspace is a static device array of FG_STATIC_SCRATCH_BYTES (the
 * workspace header of fg_workspace_header_bytes() + 8 MiB of fp32 partials, twice what the
 * library's own plans need for up to 16 rows) that every GPU the library runs on holds until the process ends; the call allocates and
 * frees nothing.  A plan that needs more (S*M*N*4 bytes of partials > 8 MiB, e.g. a forced
 * 16-way split of 16 x 16384 outputs) is rejected with FG_ERR_SCRATCH_LIMIT; plans that do not
 * split have no limit.  `splitk` as in fg_gemm_f16.  Results are those of fg_gemm_f16, bit for bit.  All calls on one GPU share that GPU's array: calls that overlap in time on one
 * GPU (two streams, two threads) race, so order them on one stream.  The first call on a device
 * looks the array's address up and clears its workspace header; make that call outside graph
 * capture, with the device of `stream` current.
 */
#define FG_STATIC_SCRATCH_BYTES (65536 + 3145728 + 524288 + (8 << 20))
int fg_gemm_f16_static(const void* A, const void* W, void* C, int M, int N, int K, int w_layout,
                       int accumulate, int splitk, void* stream);

/*
 * fg_gemm_f16 for [K,N] weights whose rows are ldw >= N elements apart (ldw a multiple of 8):
 * W[k][n] at W + k*ldw + n.  No counterpart in the reference, whose tensors are contiguous.  It is
 * for callers that own the weights and can pad them once at load time: when N is a multiple of 512
 * every byte a wave has in flight sits at the same offset within 1 KB, and rows 256 bytes further
 * apart (ldw = N + 128) make the same call about 9 % faster (M = 16, K = N = 8192: 26.1 -> 23.5 us).
 * The result is the one fg_gemm_f16 gives on the dense copy, bit for bit.
 */
int fg_gemm_f16_pitched(const void* A, const void* W, void* C, int M, int N, int K, int ldw,
                        int accumulate, int splitk, void* ws, size_t ws_bytes, void* stream);

/* Same computation with an explicit plan (kernel family, tile, split-K, unroll).  Grid and
 * workspace fields of *plan are recomputed and written back. */
int fg_gemm_f16_planned(const void* A, const void* W, void* C, int M, int N, int K,
                        int w_layout, int accumulate, fg_plan_t* plan, void* ws,
                        size_t ws_bytes, void* stream);

/*
 * C = act(A·W + bias): the same kernels with the bias add and the activation applied in fp32 to
 * the finished sum (after the split-K reduction when there is one), before the single rounding
 * to fp16.  bias: fp16 [N], one value per output column, or NULL.  act: FG_ACT_*.  plan: NULL for
 * the library's choice (then `splitk` is honoured as in fg_gemm_f16), or a caller-edited plan as
 * in fg_gemm_f16_planned.  Always overwrites C.
 *
 * No counterpart in the reference, whose operators stop at the product: the up-projection of
 * its DiT feed-forward pair (16 x 3072 x 12288, then 16 x 12288 x 3072) would be followed by a
 * separate elementwise launch over C; here the up-projection writes act(A·W1 + b1) directly.
 */
enum {
  FG_ACT_NONE = 0,
  FG_ACT_RELU = 1,      /* max(x, 0)                                               */
  FG_ACT_GELU = 2,      /* 0.5 x (1 + erf(x / sqrt 2))                             */
  FG_ACT_GELU_TANH = 3, /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))         */
  FG_ACT_SILU = 4       /* x / (1 + exp(-x))                                       */
};
int fg_gemm_f16_bias_act(const void* A, const void* W, const void* bias, int act, void* C, int M,
                         int N, int K, int w_layout, int splitk, fg_plan_t* plan, void* ws,
                         size_t ws_bytes, void* stream);

/* The plan fg_gemm_f16 would use for this shape (splitk as above).  Pure host code: it never calls
 * into the HIP runtime, so a process that only sizes buffers (or plans and then starts workers)
 * leaves the GPU untouched.  The rules count compute units: the library plans for 256 (MI355X)
 * until an entry point that launches has read the current device's count, or the caller set one. */
int fg_plan(int M, int N, int K, int w_layout, int splitk, fg_plan_t* out);

/* Workspace bytes fg_gemm_f16 needs for this shape and splitk argument (0 when the plan
 * does not split across workgroups).  Pure host code, as fg_plan. */
size_t fg_workspace_bytes(int M, int N, int K, int w_layout, int splitk);

/* Compute units the plans are made for.  fg_set_compute_units (16..4096, pure host code) pins a
 * count, e.g. to plan on a machine without the GPU; fg_use_device_compute_units reads the count
 * of the current HIP device once (this one initialises the HIP runtime, as every launching entry
 * point does by itself) unless one was pinned, and returns the count in use. */
int fg_set_compute_units(int cus);
int fg_compute_units(void);
int fg_use_device_compute_units(void);

/* Size of the header (arrival counters, then accumulator and class words) at the start of a
 * split-K workspace, and the call that zeroes it (a fill kernel on `stream`, safe to capture in a HIP graph).  Needed once per workspace, not
 * per call.  The reference has no counterpart: its split-K adds fp16 atomically into a C the
 * host zeroed with an extra memset launch (backend/cuda/hk/edgemm.cu:138-142). */
size_t fg_workspace_header_bytes(void);
int fg_workspace_init(void* ws, size_t ws_bytes, void* stream);

/*
 * W8A16 GEMV: y[m,n] = s_n · ( Σ_k x[m,k]·float(Wq[n,k]) − zero_point·Σ_k x[m,k] ),
 * s_n = scalar_scale · (scale ? float(scale[n]) : 1).  Wq int8 [N,K] row-major, x fp16
 * [M,K], scale fp16 [N] or NULL, y fp16 [M,N].  fp32 accumulation, int8→fp16 conversion
 * is exact.  1 <= M <= 16.  An activation row that holds an infinity or a NaN gets the class the
 * reference's element-by-element sum of x·(float(Wq) − zero_point) has (±inf, or NaN where the
 * weight under the infinity equals the zero point or infinities of both signs meet), not the
 * NaN that inf − inf of the two-term form above would give; the same holds for fg_gemv_w4a16.
 * Services fastgemv_int8 (backend/cuda/hk/fastgemv.cu:35-61; kernel formula
 * hk/fastgemv.cuh:316-389, whose host passes scale = 1, zero_point = 0); the per-channel
 * scale vector is an extension the reference does not have.
 */
int fg_gemv_w8a16(const void* Wq, const void* x, const void* scale, float scalar_scale,
                  float zero_point, void* y, int M, int N, int K, void* stream);

/*
 * W4A16 GEMV: y[m,n] = s_n · ( Σ_k x[m,k]·float(u4[n,k]) − zero_point·Σ_k x[m,k] ), u4 the unsigned
 * 4-bit weights packed two per byte, element 2i in the low nibble of byte i (uint4_2,
 * backend/cuda/hk/utility.cuh:13-36).  Wq4 uint8 [N,K/2] row-major, x fp16 [M,K], scale fp16 [N]
 * or NULL, y fp16 [M,N].  fp32 accumulation, nibble→fp16 conversion exact.  1 <= M <= 4.
 * Services the formula of gemv_quantized_int4 (backend/cuda/hk/fastgemv.cuh:394-495), a kernel
 * the reference defines without a host entry point.
 */
int fg_gemv_w4a16(const void* Wq4, const void* x, const void* scale, float scalar_scale,
                  float zero_point, void* y, int M, int N, int K, void* stream);

/*
 * Integer dot stage: acc[m,n] = Σ_k int32(xq[m,k])·int32(Wq[n,k]) with v_dot4_i32_i8.
 * Wq int8 [N,K], xq int8 [M,K], acc int32 [M,N].  Exact for K <= 2^17.  1 <= M <= 8.
 * No counterpart in the reference (its int8 GEMV multiplies fp16 activations); this is the
 * stage whose result is compared bit for bit.
 */
int fg_gemv_i8i8_i32(const void* Wq, const void* xq, int32_t* acc, int M, int N, int K,
                     void* stream);

/*
 * Dequantising epilogue of the integer stage: y[m,n] = fp16( float(acc[m,n]) · x_scale ·
 * (scale ? float(scale[n]) : 1) ).  Together with fg_gemv_i8i8_i32 this is the W8A8 GEMV.
 */
int fg_dequant_i32_f16(const int32_t* acc, const void* scale, float x_scale, void* y, int M,
                       int N, void* stream);

/*
 * Roofline calibration: read `bytes` (multiple of 16) from src with 16-byte loads and
 * fold them into one 32-bit word per workgroup at sink (at least fg_stream_read_sink_bytes()
 * bytes).  Reports the read-only streaming ceiling the GEMV kernels are compared with.
 */
int fg_stream_read(const void* src, size_t bytes, void* sink, void* stream);
size_t fg_stream_read_sink_bytes(void);

/* Human-readable text for a status code; never NULL. */
const char* fg_strerror(int status);

/* FG_VERSION of the built library. */
int fg_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FASTGATE_H_ */
