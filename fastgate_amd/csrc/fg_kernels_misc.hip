// Second pass of split-K and the read-only streaming probe used to calibrate the roofline.
#include "fg_device.h"
#include "fg_internal.h"

namespace fg {

// C[m,n] = fp16( Σ_{s<S} ws[s,m,n] (+ C[m,n]) ), s ascending: the result does not depend on
// the order in which the first-pass workgroups finished.  Four columns per thread.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws,
                                                            half_t* __restrict__ C, int S,
                                                            size_t MN, int accumulate) {
  const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= MN) return;
  float4_t sum = *reinterpret_cast<const float4_t*>(ws + i);
  for (int s = 1; s < S; ++s) sum += *reinterpret_cast<const float4_t*>(ws + (size_t)s * MN + i);
  typedef half_t half4_t __attribute__((ext_vector_type(4)));
  half4_t* c = reinterpret_cast<half4_t*>(C + i);
  if (accumulate) {
    const half4_t old = *c;
#pragma unroll
    for (int k = 0; k < 4; ++k) sum[k] += static_cast<float>(old[k]);
  }
  half4_t out;
#pragma unroll
  for (int k = 0; k < 4; ++k) out[k] = static_cast<half_t>(sum[k]);
  *c = out;
}

void launch_splitk_reduce(const float* ws, void* C, int S, int M, int N, int accumulate,
                          hipStream_t s) {
  const size_t MN = (size_t)M * N;  // N % 128 == 0, so MN % 4 == 0
  const unsigned blocks = (unsigned)((MN / 4 + 255) / 256);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, ws,
                     static_cast<half_t*>(C), S, MN, accumulate);
}

// Grid-stride read of `n16` 16-byte words, 8 independent loads in flight per lane, xor-folded
// so the loads cannot be dropped; one word per workgroup is written to sink.
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ src,
                                                          size_t n16, uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (; i + 7 * stride < n16; i += 8 * stride) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
  x ^= (uint32_t)dpp_i32<0xB1>((int)x);
  x ^= (uint32_t)dpp_i32<0x4E>((int)x);
  x ^= (uint32_t)dpp_i32<0x141>((int)x);
  x ^= (uint32_t)dpp_i32<0x140>((int)x);
  __shared__ uint32_t part[16];
  if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t r = 0;
    for (int p = 0; p < 16; ++p) r ^= part[p];
    sink[blockIdx.x] = r;
  }
}

void launch_stream_read(const void* src, size_t bytes, void* sink, hipStream_t s) {
  hipLaunchKernelGGL(stream_read_kernel, dim3(kStreamReadBlocks), dim3(256), 0, s,
                     static_cast<const u32x4*>(src), bytes / 16, static_cast<uint32_t*>(sink));
}

}  // namespace fg
