// Element-wise stages of RWKV-7 time mixing on either side of the WKV op, fused into two memory-bound kernels
// (reference: /root/reference/src/jaxrwkv/rwkv7.py:248-252 and :263-265).  Sixteen lanes (one DPP row) per
// (token, head), four consecutive channels per lane: a wavefront handles four (token, head) units with one 8- or
// 16-byte access per lane and array, and the per-head reductions (L2 norm, mean/variance, r.k.r_k) are four
// DPP row rotations each; nothing goes through LDS.  fp32 arithmetic, fp32 or bf16 I/O.
//
//   pre :  kk = normalize_head(k . k_k) ;  k' = k (1 + (a - 1) k_a) ;  a_i = -kk ;  b_i = kk . a
//   post:  out = ( group_norm_head(y; eps) . ln_w + ln_b + (sum_j r_j k'_j r_k_j) v ) . g
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

// sum over the 16 lanes of a DPP row, delivered to all of them
__device__ __forceinline__ float row_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, false));   // row_ror:8
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, false));   // row_ror:4
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x122, 0xf, 0xf, false));   // row_ror:2
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x121, 0xf, 0xf, false));   // row_ror:1
  return x;
}

// four consecutive elements <-> four floats (pointer 8-byte aligned for bf16, 16 for fp32)
__device__ __forceinline__ void ld4(const float* p, float (&o)[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  o[0] = x.x; o[1] = x.y; o[2] = x.z; o[3] = x.w;
}
__device__ __forceinline__ void ld4(const bf16_t* p, float (&o)[4]) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  o[0] = __uint_as_float(x.x << 16); o[1] = __uint_as_float(x.x & 0xffff0000u);
  o[2] = __uint_as_float(x.y << 16); o[3] = __uint_as_float(x.y & 0xffff0000u);
}
__device__ __forceinline__ void st4(float* p, const float (&o)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void st4(bf16_t* p, const float (&o)[4]) {
  const uint32_t lo = (uint32_t)f32_to_bf16(o[0]) | ((uint32_t)f32_to_bf16(o[1]) << 16);
  const uint32_t hi = (uint32_t)f32_to_bf16(o[2]) | ((uint32_t)f32_to_bf16(o[3]) << 16);
  *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
}

constexpr int MIX_THREADS = 256;        // 16 (token, head) units per workgroup

template <typename T>
__global__ __launch_bounds__(MIX_THREADS) void rwkv7_premix_kernel(int64_t rows, int64_t H, const T* __restrict__ k,
                                                                   const T* __restrict__ a, const T* __restrict__ k_k,
                                                                   const T* __restrict__ k_a, T* __restrict__ k_out,
                                                                   T* __restrict__ a_out, T* __restrict__ b_out) {
  // units beyond the end redo the last one (same loads, same stores): whole rows stay active for the reductions
  int64_t unit = (int64_t)blockIdx.x * (MIX_THREADS / 16) + (threadIdx.x >> 4);
  unit = unit < rows * H ? unit : rows * H - 1;
  const int c4 = 4 * (threadIdx.x & 15);
  const int64_t h = unit % H;
  const size_t el = (size_t)unit * 64 + c4, ch = (size_t)h * 64 + c4;
  float kv[4], av[4], kkw[4], kaw[4];
  ld4(k + el, kv); ld4(a + el, av); ld4(k_k + ch, kkw); ld4(k_a + ch, kaw);
  float kk[4], ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) { kk[i] = kv[i] * kkw[i]; ss = fmaf(kk[i], kk[i], ss); }
  const float inv = 1.f / fmaxf(sqrtf(row_sum(ss)), 1e-12f);   // rwkv7.py:250
  float ko[4], ao[4], bo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    kk[i] *= inv;
    ko[i] = kv[i] * (1.f + (av[i] - 1.f) * kaw[i]);              // :252
    ao[i] = -kk[i];                                              // :257
    bo[i] = kk[i] * av[i];
  }
  st4(k_out + el, ko); st4(a_out + el, ao); st4(b_out + el, bo);
}

template <typename T>
__global__ __launch_bounds__(MIX_THREADS) void rwkv7_postmix_kernel(int64_t rows, int64_t H, const T* __restrict__ y,
                                                                    const T* __restrict__ r, const T* __restrict__ k,
                                                                    const T* __restrict__ v, const T* __restrict__ g,
                                                                    const T* __restrict__ ln_w,
                                                                    const T* __restrict__ ln_b,
                                                                    const T* __restrict__ r_k, float eps,
                                                                    T* __restrict__ out) {
  int64_t unit = (int64_t)blockIdx.x * (MIX_THREADS / 16) + (threadIdx.x >> 4);
  unit = unit < rows * H ? unit : rows * H - 1;
  const int c4 = 4 * (threadIdx.x & 15);
  const int64_t h = unit % H;
  const size_t el = (size_t)unit * 64 + c4, ch = (size_t)h * 64 + c4;
  float yv[4], rv[4], kv[4], vv[4], gv[4], lw[4], lb[4], rk[4];
  ld4(y + el, yv); ld4(r + el, rv); ld4(k + el, kv); ld4(v + el, vv); ld4(g + el, gv);
  ld4(ln_w + ch, lw); ld4(ln_b + ch, lb); ld4(r_k + ch, rk);
  const float mean = row_sum(yv[0] + yv[1] + yv[2] + yv[3]) * (1.f / 64.f);
  float d[4], sq = 0.f, dot = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    d[i] = yv[i] - mean;
    sq = fmaf(d[i], d[i], sq);
    dot = fmaf(rv[i] * kv[i], rk[i], dot);
  }
  const float rstd = rsqrtf(row_sum(sq) * (1.f / 64.f) + eps);   // biased variance, rwkv7.py:19
  const float bonus = row_sum(dot);                              // :264
  float o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = (d[i] * rstd * lw[i] + lb[i] + bonus * vv[i]) * gv[i];
  st4(out + el, o);
}

}  // namespace

hipError_t launch_rwkv7_premix(int io_f32, int64_t rows, int64_t H, const void* k, const void* a, const void* k_k,
                               const void* k_a, void* k_out, void* a_out, void* b_out, hipStream_t stream) {
  const dim3 grid((unsigned)((rows * H + MIX_THREADS / 16 - 1) / (MIX_THREADS / 16))), block(MIX_THREADS);
  if (io_f32)
    hipLaunchKernelGGL(rwkv7_premix_kernel<float>, grid, block, 0, stream, rows, H, (const float*)k, (const float*)a,
                       (const float*)k_k, (const float*)k_a, (float*)k_out, (float*)a_out, (float*)b_out);
  else
    hipLaunchKernelGGL(rwkv7_premix_kernel<bf16_t>, grid, block, 0, stream, rows, H, (const bf16_t*)k, (const bf16_t*)a,
                       (const bf16_t*)k_k, (const bf16_t*)k_a, (bf16_t*)k_out, (bf16_t*)a_out, (bf16_t*)b_out);
  return hipGetLastError();
}

hipError_t launch_rwkv7_postmix(int io_f32, int64_t rows, int64_t H, const void* y, const void* r, const void* k,
                                const void* v, const void* g, const void* ln_w, const void* ln_b, const void* r_k,
                                float eps, void* out, hipStream_t stream) {
  const dim3 grid((unsigned)((rows * H + MIX_THREADS / 16 - 1) / (MIX_THREADS / 16))), block(MIX_THREADS);
  if (io_f32)
    hipLaunchKernelGGL(rwkv7_postmix_kernel<float>, grid, block, 0, stream, rows, H, (const float*)y, (const float*)r,
                       (const float*)k, (const float*)v, (const float*)g, (const float*)ln_w, (const float*)ln_b,
                       (const float*)r_k, eps, (float*)out);
  else
    hipLaunchKernelGGL(rwkv7_postmix_kernel<bf16_t>, grid, block, 0, stream, rows, H, (const bf16_t*)y,
                       (const bf16_t*)r, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)g, (const bf16_t*)ln_w,
                       (const bf16_t*)ln_b, (const bf16_t*)r_k, eps, (bf16_t*)out);
  return hipGetLastError();
}

}  // namespace hiprwkv
