// Element-wise stages of RWKV-7 time mixing on either side of the WKV op, fused into two memory-bound kernels
// (reference: /root/reference/src/jaxrwkv/rwkv7.py:248-252 and :263-265).  One wavefront per (token, head): lane j
// owns channel j of the 64-wide head, the per-head reductions (L2 norm, mean/variance, r.k.r_k) are DPP/permute
// wave reductions; nothing goes through LDS.  fp32 arithmetic, fp32 or bf16 I/O.
//
//   pre :  kk = normalize_head(k . k_k) ;  k' = k (1 + (a - 1) k_a) ;  a_i = -kk ;  b_i = kk . a
//   post:  out = ( group_norm_head(y; eps) . ln_w + ln_b + (sum_j r_j k'_j r_k_j) v ) . g
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

template <typename T>
__global__ __launch_bounds__(256) void rwkv7_premix_kernel(int64_t rows, int64_t H, const T* __restrict__ k,
                                                           const T* __restrict__ a, const T* __restrict__ k_k,
                                                           const T* __restrict__ k_a, T* __restrict__ k_out,
                                                           T* __restrict__ a_out, T* __restrict__ b_out) {
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // (token, head)
  if (unit >= rows * H) return;
  const int lane = threadIdx.x & 63;
  const int64_t h = unit % H;
  const size_t el = (size_t)unit * 64 + lane, ch = (size_t)h * 64 + lane;
  const float kv = ld_f(k + el), av = ld_f(a + el);
  float kk = kv * ld_f(k_k + ch);
  const float nrm = sqrtf(wave_sum(kk * kk));
  kk = kk / fmaxf(nrm, 1e-12f);                                  // rwkv7.py:250
  st_f(k_out + el, kv * (1.f + (av - 1.f) * ld_f(k_a + ch)));    // :252
  st_f(a_out + el, -kk);                                         // :257
  st_f(b_out + el, kk * av);
}

template <typename T>
__global__ __launch_bounds__(256) void rwkv7_postmix_kernel(int64_t rows, int64_t H, const T* __restrict__ y,
                                                            const T* __restrict__ r, const T* __restrict__ k,
                                                            const T* __restrict__ v, const T* __restrict__ g,
                                                            const T* __restrict__ ln_w, const T* __restrict__ ln_b,
                                                            const T* __restrict__ r_k, float eps, T* __restrict__ out) {
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= rows * H) return;
  const int lane = threadIdx.x & 63;
  const int64_t h = unit % H;
  const size_t el = (size_t)unit * 64 + lane, ch = (size_t)h * 64 + lane;
  const float yv = ld_f(y + el);
  const float mean = wave_sum(yv) * (1.f / 64.f);
  const float d = yv - mean;
  const float var = wave_sum(d * d) * (1.f / 64.f);              // biased variance, rwkv7.py:19
  const float yn = d * rsqrtf(var + eps) * ld_f(ln_w + ch) + ld_f(ln_b + ch);
  const float bonus = wave_sum(ld_f(r + el) * ld_f(k + el) * ld_f(r_k + ch));   // :264
  st_f(out + el, (yn + bonus * ld_f(v + el)) * ld_f(g + el));
}

}  // namespace

hipError_t launch_rwkv7_premix(int io_f32, int64_t rows, int64_t H, const void* k, const void* a, const void* k_k,
                               const void* k_a, void* k_out, void* a_out, void* b_out, hipStream_t stream) {
  const dim3 grid((unsigned)((rows * H + 3) / 4)), block(256);
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
  const dim3 grid((unsigned)((rows * H + 3) / 4)), block(256);
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
