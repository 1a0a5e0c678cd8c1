/*
 * CPU oracle for the small-batch GEMM / GEMV path.  TEST INFRASTRUCTURE ONLY: nothing under
 * fastgate_amd/ may include, link or call this file; only tests/, the smoke check and the
 * bench's cpu_baseline leg use it, and only as the checker or the reported CPU baseline.
 *
 * It restates, in plain C, what the reference (chanzhennan/Fastgate) computes on this path.
 * The reference's own check is torch.matmul (script/standard-test.py:152, script/gemv-test.py:
 * 20, script/ncu-gemv-test.py:39): C = A·W with fp16 inputs, results compared after rounding
 * to fp16.  The arithmetic contract used here is the one the task fixes: exact fp16 products,
 * fp32 accumulation in ascending k, one rounding to fp16 (fg_oracle_gemm_f16), with an fp64
 * accumulation twin (fg_oracle_gemm_f16_f64) used to bound the fp32 summation error.
 *
 *   function                      follows (reference file:line)
 *   fg_oracle_gemm_f16*           backend/cuda/hk/edgemm.cu:102-156 (A[M,K], B[K,N], N=B.size(1)),
 *                                 :274-324 (B_t[N,K], N=B.size(0)); hk/flatgemm.cu:13-169;
 *                                 hk/edgemm_tr.cu:19-139; hk/fastgemv.cu:12-33,86-111
 *                                 (res[m*N+n] = Σ_k mat[n,k]·vec[m,k], hk/fastgemv.cuh:244-311)
 *   fg_oracle_gemv_w8a16          hk/fastgemv.cuh:316-389: sum += x·(float(w) − zp); sum *= scale
 *   fg_oracle_gemv_w4a16          hk/fastgemv.cuh:394-495, nibble order hk/utility.cuh:13-36
 *   fg_oracle_gemv_i8i8_i32       none (integer stage added by this library); exact integer sum
 *   fg_oracle_bias_act            none (bias + activation tail added by this library; the
 *                                 reference's operators stop at the product): textbook formulas
 *
 * Pinning (tests/test_oracle.py): exact rational arithmetic on small cases, closed forms
 * (ones·ones = K from script/ncu-gemv-test.py:29-30, unit vectors, identity), the committed
 * vectors in tests/golden/, and torch.matmul on CPU.  The reference holds no golden vectors
 * for this path.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* IEEE binary16 -> binary32, every encoding (subnormals, inf, NaN). */
float fg_oracle_h2f(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* binary32 -> binary16, round to nearest even, overflow to inf, subnormal results kept. */
uint16_t fg_oracle_f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / NaN */
    return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u | ((absx >> 13) & 0x3ffu) : 0));
  }
  if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
    if (absx < 0x33000000u) return sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even 0) */
    const int e = (int)(absx >> 23);      /* biased fp32 exponent, 102..112 */
    const uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    const int shift = 126 - e; /* result = man >> shift, in units of 2^-24 */
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
  {
    uint32_t e = (absx >> 23) - 127 + 15;
    uint32_t man = absx & 0x7fffffu;
    uint32_t q = (e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry may bump the exponent */
    return (uint16_t)(sign | q);
  }
}

/* binary64 -> binary16 with a single rounding (no double rounding through fp32). */
uint16_t fg_oracle_d2h(double d) {
  if (d != d) return 0x7e00u;
  const uint16_t sign = signbit(d) ? 0x8000u : 0;
  double a = fabs(d);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);
  if (a < ldexp(1.0, -14)) {
    /* subnormal range: units of 2^-24, rint = round half even in the default mode */
    const double q = rint(ldexp(a, 24));
    return (uint16_t)(sign | (uint16_t)q);
  }
  int e;
  const double m = frexp(a, &e); /* a = m·2^e, m in [0.5,1) */
  /* 11 significant bits: scale so the integer part holds them */
  const double q = rint(ldexp(m, 11)); /* 1024..2048 */
  uint32_t qi = (uint32_t)q;
  int ee = e - 1; /* exponent of the leading bit */
  if (qi == 2048u) {
    qi = 1024u;
    ++ee;
  }
  if (ee > 15) return (uint16_t)(sign | 0x7c00u);
  return (uint16_t)(sign | ((uint32_t)(ee + 15) << 10) | (qi & 0x3ffu));
}

/* fp16 -> fp32 lookup built from fg_oracle_h2f: keeps the O(M·N·K) loops cheap. */
static float g_h2f[65536];
static int g_h2f_ready = 0;
static void ensure_table(void) {
  if (!g_h2f_ready) {
    for (uint32_t i = 0; i < 65536u; ++i) g_h2f[i] = fg_oracle_h2f((uint16_t)i);
    g_h2f_ready = 1;
  }
}

/*
 * C[m,n] = fp16( Σ_k A[m,k]·W(k,n) (+ C[m,n]) ), fp32 accumulation, k ascending for every
 * (m,n).  w_layout 0: W is [K,N] row-major; 1: W is [N,K] row-major.  C32 (optional)
 * receives the unrounded fp32 sums without the accumulate term.  `row` is caller scratch of
 * N floats.
 */
void fg_oracle_gemm_f16(const uint16_t* A, const uint16_t* W, uint16_t* C, float* C32, float* row,
                        int M, int N, int K, int w_layout, int accumulate) {
  ensure_table();
  for (int m = 0; m < M; ++m) {
    const uint16_t* a = A + (size_t)m * K;
    if (w_layout) {
      for (int n = 0; n < N; ++n) {
        const uint16_t* w = W + (size_t)n * K;
        float sum = 0.f;
        for (int k = 0; k < K; ++k) sum += g_h2f[a[k]] * g_h2f[w[k]];
        row[n] = sum;
      }
    } else {
      for (int n = 0; n < N; ++n) row[n] = 0.f;
      for (int k = 0; k < K; ++k) { /* every row[n] still sees k = 0,1,2,... in order */
        const float ak = g_h2f[a[k]];
        const uint16_t* w = W + (size_t)k * N;
        for (int n = 0; n < N; ++n) row[n] += ak * g_h2f[w[n]];
      }
    }
    for (int n = 0; n < N; ++n) {
      float sum = row[n];
      if (C32) C32[(size_t)m * N + n] = sum;
      if (accumulate) sum += g_h2f[C[(size_t)m * N + n]];
      C[(size_t)m * N + n] = fg_oracle_f2h(sum);
    }
  }
}

/* Same contraction with fp64 accumulation and a single fp64 -> fp16 rounding.  `row` is
 * caller scratch of N doubles. */
void fg_oracle_gemm_f16_f64(const uint16_t* A, const uint16_t* W, uint16_t* C, double* C64,
                            double* row, int M, int N, int K, int w_layout, int accumulate) {
  ensure_table();
  for (int m = 0; m < M; ++m) {
    const uint16_t* a = A + (size_t)m * K;
    if (w_layout) {
      for (int n = 0; n < N; ++n) {
        const uint16_t* w = W + (size_t)n * K;
        double sum = 0.0;
        for (int k = 0; k < K; ++k) sum += (double)g_h2f[a[k]] * (double)g_h2f[w[k]];
        row[n] = sum;
      }
    } else {
      for (int n = 0; n < N; ++n) row[n] = 0.0;
      for (int k = 0; k < K; ++k) {
        const double ak = (double)g_h2f[a[k]];
        const uint16_t* w = W + (size_t)k * N;
        for (int n = 0; n < N; ++n) row[n] += ak * (double)g_h2f[w[n]];
      }
    }
    for (int n = 0; n < N; ++n) {
      double sum = row[n];
      if (C64) C64[(size_t)m * N + n] = sum;
      if (accumulate) sum += (double)g_h2f[C[(size_t)m * N + n]];
      C[(size_t)m * N + n] = fg_oracle_d2h(sum);
    }
  }
}

/*
 * y[m,n] = fp16( ( Σ_k x[m,k]·(float(Wq[n,k]) − zp) ) · scalar_scale · (scale ? scale[n] : 1) ),
 * fp32 arithmetic in the order of hk/fastgemv.cuh:344-363 (subtract, multiply, add; scale last).
 * Y32 (optional) receives the unrounded values.
 */
void fg_oracle_gemv_w8a16(const int8_t* Wq, const uint16_t* X, const uint16_t* scale,
                          float scalar_scale, float zero_point, uint16_t* Y, float* Y32, int M, int N,
                          int K) {
  ensure_table();
  for (int m = 0; m < M; ++m) {
    const uint16_t* x = X + (size_t)m * K;
    for (int n = 0; n < N; ++n) {
      const int8_t* w = Wq + (size_t)n * K;
      float sum = 0.f;
      for (int k = 0; k < K; ++k) sum += g_h2f[x[k]] * ((float)w[k] - zero_point);
      sum *= scalar_scale;
      if (scale) sum *= g_h2f[scale[n]];
      if (Y32) Y32[(size_t)m * N + n] = sum;
      Y[(size_t)m * N + n] = fg_oracle_f2h(sum);
    }
  }
}

/*
 * W4A16 GEMV, hk/fastgemv.cuh:394-495 with the nibble order of hk/utility.cuh:13-36 (getX = low
 * nibble = even element, getY = high nibble = odd element): sum += x·(float(u4) − zp) in
 * ascending k, scale last.  Wq4 is [N][K/2] bytes.
 */
void fg_oracle_gemv_w4a16(const uint8_t* Wq4, const uint16_t* X, const uint16_t* scale,
                          float scalar_scale, float zero_point, uint16_t* Y, float* Y32, int M, int N,
                          int K) {
  ensure_table();
  for (int m = 0; m < M; ++m) {
    const uint16_t* x = X + (size_t)m * K;
    for (int n = 0; n < N; ++n) {
      const uint8_t* w = Wq4 + (size_t)n * (K / 2);
      float sum = 0.f;
      for (int k = 0; k < K; ++k) {
        const uint8_t b = w[k >> 1];
        const float u = (float)((k & 1) ? (b >> 4) : (b & 0x0f));
        sum += g_h2f[x[k]] * (u - zero_point);
      }
      sum *= scalar_scale;
      if (scale) sum *= g_h2f[scale[n]];
      if (Y32) Y32[(size_t)m * N + n] = sum;
      Y[(size_t)m * N + n] = fg_oracle_f2h(sum);
    }
  }
}

/* acc[m,n] = Σ_k int32(Xq[m,k])·int32(Wq[n,k]), summed in int64 and checked to fit int32. */
int fg_oracle_gemv_i8i8_i32(const int8_t* Wq, const int8_t* Xq, int32_t* acc, int M, int N, int K) {
  int overflow = 0;
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      int64_t sum = 0;
      for (int k = 0; k < K; ++k) sum += (int64_t)Xq[(size_t)m * K + k] * (int64_t)Wq[(size_t)n * K + k];
      if (sum > INT32_MAX || sum < INT32_MIN) overflow = 1;
      acc[(size_t)m * N + n] = (int32_t)sum;
    }
  }
  return overflow;
}

/* y[m,n] = fp16( float(acc[m,n]) · x_scale · (scale ? scale[n] : 1) ). */
void fg_oracle_dequant_i32_f16(const int32_t* acc, const uint16_t* scale, float x_scale, uint16_t* Y,
                               int M, int N) {
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      float s = x_scale;
      if (scale) s *= fg_oracle_h2f(scale[n]);
      Y[(size_t)m * N + n] = fg_oracle_f2h((float)acc[(size_t)m * N + n] * s);
    }
  }
}

/*
 * Y[m,n] = fp16( act( C32[m,n] + bias[n] ) ), fp32 arithmetic with libm; act: 0 none, 1 relu,
 * 2 gelu 0.5 x (1 + erf(x / sqrt 2)), 3 gelu-tanh 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))),
 * 4 silu x / (1 + exp(-x)).  bias: fp16 [N] or NULL.  Y32 (optional) receives the unrounded values.
 */
void fg_oracle_bias_act(const float* C32, const uint16_t* bias, int act, uint16_t* Y, float* Y32,
                        int M, int N) {
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      float v = C32[(size_t)m * N + n];
      if (bias) v += fg_oracle_h2f(bias[n]);
      switch (act) {
        case 1: v = v > 0.f ? v : 0.f; break;
        case 2: v = 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); break;
        case 3: v = 0.5f * v * (1.f + tanhf(0.79788456080286536f * (v + 0.044715f * v * v * v))); break;
        case 4: v = v / (1.f + expf(-v)); break;
        default: break;
      }
      if (Y32) Y32[(size_t)m * N + n] = v;
      Y[(size_t)m * N + n] = fg_oracle_f2h(v);
    }
  }
}
