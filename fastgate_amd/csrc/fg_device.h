// Device-side building blocks shared by the gfx950 kernels: vector types, 16-byte global
// loads, packed-fp16 dot products with fp32 accumulation, wave64 DPP reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fg {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// 16-byte global load.  STREAM marks data that is read exactly once (the weights) with the
// non-temporal hint so it does not displace the activation panel from the caches.
template <bool STREAM>
__device__ __forceinline__ u32x4 load16(const void* p) {
  if constexpr (STREAM) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  } else {
    return *reinterpret_cast<const u32x4*>(p);
  }
}

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ half8_t as_half8(u32x4 v) { return __builtin_bit_cast(half8_t, v); }

// acc + Σ_{i<8} w_i·x_i: four v_dot2_f32_f16, products and sum kept in fp32.
__device__ __forceinline__ float dot8(u32x4 w, u32x4 x, float acc) {
  acc = __builtin_amdgcn_fdot2(as_half2(w.x), as_half2(x.x), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.y), as_half2(x.y), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.z), as_half2(x.z), acc, false);
  acc = __builtin_amdgcn_fdot2(as_half2(w.w), as_half2(x.w), acc, false);
  return acc;
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// Sum over each DPP row (16 consecutive lanes); every lane of the row ends with the row sum.
// quad_perm[1,0,3,2], quad_perm[2,3,0,1], row_half_mirror, row_mirror.
__device__ __forceinline__ float row16_allreduce(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  return v;
}
__device__ __forceinline__ int row16_allreduce(int v) {
  v += dpp_i32<0xB1>(v);
  v += dpp_i32<0x4E>(v);
  v += dpp_i32<0x141>(v);
  v += dpp_i32<0x140>(v);
  return v;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<half_t>(v));
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return static_cast<float>(__builtin_bit_cast(half_t, b));
}

}  // namespace fg
