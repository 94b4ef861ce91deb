// Shared device helpers for the gfx950 WKV kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hiprwkv {

struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// round-to-nearest-even, NaN stays NaN: the hardware conversion (v_cvt_pk_bf16_f32), one instruction
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

__device__ __forceinline__ float ld_f(const float* p) { return *p; }
__device__ __forceinline__ float ld_f(const bf16_t* p) { return bf16_to_f32(p->bits); }
__device__ __forceinline__ void st_f(float* p, float x) { *p = x; }
__device__ __forceinline__ void st_f(bf16_t* p, float x) { p->bits = f32_to_bf16(x); }

// 8 consecutive elements <-> 8 floats (pointer must be 16-byte aligned for bf16, 32 for fp32)
__device__ __forceinline__ void ld8(const float* p, float (&o)[8]) {
  float4 a = *reinterpret_cast<const float4*>(p);
  float4 b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void ld8(const bf16_t* p, float (&o)[8]) {
  uint4 a = *reinterpret_cast<const uint4*>(p);
  uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void st8(float* p, const float (&o)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(o[4], o[5], o[6], o[7]);
}
__device__ __forceinline__ void st8(bf16_t* p, const float (&o)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (uint32_t)f32_to_bf16(o[2 * i]) | ((uint32_t)f32_to_bf16(o[2 * i + 1]) << 16);
  *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

// IEEE half: the forward residual sa of the bf16 paths (11 significant bits where bf16 has 8)
__device__ __forceinline__ void ld8(const _Float16* p, float (&o)[8]) {
  typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
  const h8_t a = *reinterpret_cast<const h8_t*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (float)a[i];
}
__device__ __forceinline__ void st8(_Float16* p, const float (&o)[8]) {
  typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
  h8_t a;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = (_Float16)o[i];
  *reinterpret_cast<h8_t*>(p) = a;
}

// 16 consecutive elements starting at element `el` of a typed array -> 16 floats
template <typename T>
__device__ __forceinline__ void ld16(const void* base, size_t el, float (&o)[16]) {
  const T* p = reinterpret_cast<const T*>(base) + el;
  float lo[8], hi[8];
  ld8(p, lo);
  ld8(p + 8, hi);
#pragma unroll
  for (int c = 0; c < 8; ++c) { o[c] = lo[c]; o[8 + c] = hi[c]; }
}

// sum over the 4 lanes of a quad (lanes 4m..4m+3); every lane gets the total
__device__ __forceinline__ float quad_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
  return x;
}

}  // namespace hiprwkv
