// Three element-wise steps of RWKV-7 time mixing between the projections and the WKV op, one memory-bound kernel each
// way (reference: /root/reference/src/jaxrwkv/rwkv7.py:237, :241-242 and :244; jnp there, fused by XLA):
//     decay:  w  = -softplus(-(w0 + x)) - 0.5                 x = tanh(xw w1) w2, the low-rank decay term
//     vmix :  v' = v + (v_first - v) sigmoid(v0 + x)          x = (xv v1) v2, layers after the first
//     agate:  a  = sigmoid(a0 + x)                            x = (xa a1) a2
//     relusq: k  = relu(x)^2                                  channel mixing, rwkv7.py:196 (x = xk W_key)
// w0, v0, a0 are (C,) parameters, everything else (rows, C).  As separate tensor operations these are five to seven passes
// over a (T, C) tensor each.  A thread owns eight consecutive channels; fp32 arithmetic, one rounding per output.
//
// Backward, for a cotangent g of the output:
//     decay:  dx = g sigmoid(-(w0 + x)) ;                      dw0 = sum over rows of dx
//     vmix :  s = sigmoid(v0 + x) ;  dv = g (1 - s) ;  dv_first = g s ;  dx = g (v_first - v) s (1 - s) ;  dv0 = sum of dx
//     agate:  dx = g a (1 - a) ;                               da0 = sum of dx
//     relusq: dx = 2 g relu(x)
// A workgroup walks a run of rows with the partial sums of the parameter cotangent in registers (a thread's own
// channels) and ends with one fp32 atomic per channel; the launcher zeroes the result first with a fill kernel.
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

constexpr int GATE_THREADS = 256;

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + __expf(-z)); }
// softplus(z) = log(1 + e^z) = max(z, 0) + log(1 + e^-|z|): the argument of the logarithm lies in (1, 2], where the
// hardware logarithm is accurate to a few 1e-7 absolute (log1pf, a software routine, made this kernel three times slower)
__device__ __forceinline__ float softplusf(float z) { return fmaxf(z, 0.f) + __logf(1.f + __expf(-fabsf(z))); }

template <typename T, bool SIGMOID>   // SIGMOID: the gate a = sigmoid(a0 + x) instead of the decay
__global__ __launch_bounds__(GATE_THREADS) void rwkv7_decay_kernel(int64_t rows, int64_t C, const T* __restrict__ x,
                                                                    const T* __restrict__ w0, T* __restrict__ w) {
  const int64_t per_row = C / 8;
  const int64_t idx = (int64_t)blockIdx.x * GATE_THREADS + threadIdx.x;
  if (idx >= rows * per_row) return;
  const int c8 = (int)(idx % per_row) * 8;
  const size_t el = (size_t)(idx / per_row) * C + c8;
  float xv[8], p[8], o[8];
  ld8(x + el, xv); ld8(w0 + c8, p);
#pragma unroll
  for (int c = 0; c < 8; ++c) o[c] = SIGMOID ? sigmoidf(p[c] + xv[c]) : -softplusf(-(p[c] + xv[c])) - 0.5f;
  st8(w + el, o);
}

template <typename T>
__global__ __launch_bounds__(GATE_THREADS) void rwkv7_vmix_kernel(int64_t rows, int64_t C, const T* __restrict__ v,
                                                                   const T* __restrict__ vf, const T* __restrict__ x,
                                                                   const T* __restrict__ v0, T* __restrict__ out) {
  const int64_t per_row = C / 8;
  const int64_t idx = (int64_t)blockIdx.x * GATE_THREADS + threadIdx.x;
  if (idx >= rows * per_row) return;
  const int c8 = (int)(idx % per_row) * 8;
  const size_t el = (size_t)(idx / per_row) * C + c8;
  float vv[8], fv[8], xv[8], p[8], o[8];
  ld8(v + el, vv); ld8(vf + el, fv); ld8(x + el, xv); ld8(v0 + c8, p);
#pragma unroll
  for (int c = 0; c < 8; ++c) o[c] = fmaf(fv[c] - vv[c], sigmoidf(p[c] + xv[c]), vv[c]);
  st8(out + el, o);
}

// relu(x)^2 (BWD: 2 g relu(x)) over n8 groups of eight consecutive elements
template <typename T, bool BWD>
__global__ __launch_bounds__(GATE_THREADS) void rwkv7_relusq_kernel(int64_t n8, const T* __restrict__ x,
                                                                     const T* __restrict__ g, T* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * GATE_THREADS + threadIdx.x;
  if (idx >= n8) return;
  float xv[8], gv[8], o[8];
  ld8(x + idx * 8, xv);
  if (BWD) ld8(g + idx * 8, gv);
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const float r = fmaxf(xv[c], 0.f);
    o[c] = BWD ? 2.f * gv[c] * r : r * r;
  }
  st8(out + idx * 8, o);
}

// Workgroup (blockIdx.x = channel block, blockIdx.y = run of `run` consecutive rows)
template <typename T, bool SIGMOID>
__global__ __launch_bounds__(GATE_THREADS) void rwkv7_decay_bwd_kernel(int64_t rows, int64_t C, int64_t run,
                                                                        const T* __restrict__ x, const T* __restrict__ w0,
                                                                        const T* __restrict__ g, T* __restrict__ dx,
                                                                        float* __restrict__ dw0) {
  const int c8 = (blockIdx.x * GATE_THREADS + threadIdx.x) * 8;
  if (c8 >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * run, r1 = r0 + run < rows ? r0 + run : rows;
  float p[8], acc[8];
  ld8(w0 + c8, p);
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const size_t el = (size_t)r * C + c8;
    float xv[8], gv[8], o[8];
    ld8(x + el, xv); ld8(g + el, gv);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const float sg = sigmoidf(p[c] + xv[c]);
      o[c] = gv[c] * (SIGMOID ? sg * (1.f - sg) : 1.f - sg);      // sigmoid(-z) = 1 - sigmoid(z)
      acc[c] += o[c];
    }
    st8(dx + el, o);
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) atomicAdd(dw0 + c8 + c, acc[c]);
}

template <typename T>
__global__ __launch_bounds__(GATE_THREADS) void rwkv7_vmix_bwd_kernel(int64_t rows, int64_t C, int64_t run,
                                                                       const T* __restrict__ v, const T* __restrict__ vf,
                                                                       const T* __restrict__ x, const T* __restrict__ v0,
                                                                       const T* __restrict__ g, T* __restrict__ dv,
                                                                       T* __restrict__ dvf, T* __restrict__ dx,
                                                                       float* __restrict__ dv0) {
  const int c8 = (blockIdx.x * GATE_THREADS + threadIdx.x) * 8;
  if (c8 >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * run, r1 = r0 + run < rows ? r0 + run : rows;
  float p[8], acc[8];
  ld8(v0 + c8, p);
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const size_t el = (size_t)r * C + c8;
    float vv[8], fv[8], xv[8], gv[8], o1[8], o2[8], o3[8];
    ld8(v + el, vv); ld8(vf + el, fv); ld8(x + el, xv); ld8(g + el, gv);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const float s = sigmoidf(p[c] + xv[c]);
      o1[c] = gv[c] * (1.f - s);
      o2[c] = gv[c] * s;
      o3[c] = gv[c] * (fv[c] - vv[c]) * s * (1.f - s);
      acc[c] += o3[c];
    }
    st8(dv + el, o1); st8(dvf + el, o2); st8(dx + el, o3);
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) atomicAdd(dv0 + c8 + c, acc[c]);
}

__global__ void fill_zero_kernel(float* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// grid of the backward kernels: about two workgroups per CU (the closing atomics set the pace beyond that)
struct BwdGrid {
  dim3 grid;
  int64_t run;
};
BwdGrid bwd_grid(int64_t rows, int64_t C) {
  const unsigned cblocks = (unsigned)((C / 8 + GATE_THREADS - 1) / GATE_THREADS);
  int64_t run = (rows * cblocks + 511) / 512;
  run = run < 16 ? 16 : run;
  return {dim3(cblocks, (unsigned)((rows + run - 1) / run)), run};
}

}  // namespace

// sigmoid = 0: the decay w; 1: the gate a
hipError_t launch_rwkv7_decay(int io_f32, int sigmoid, int64_t rows, int64_t C, const void* x, const void* w0, void* w,
                              hipStream_t stream) {
  const dim3 grid((unsigned)((rows * (C / 8) + GATE_THREADS - 1) / GATE_THREADS)), block(GATE_THREADS);
#define HIPRWKV_GATE_LAUNCH(TY, SG) \
  hipLaunchKernelGGL((rwkv7_decay_kernel<TY, SG>), grid, block, 0, stream, rows, C, (const TY*)x, (const TY*)w0, (TY*)w)
  if (io_f32) { if (sigmoid) HIPRWKV_GATE_LAUNCH(float, true); else HIPRWKV_GATE_LAUNCH(float, false); }
  else { if (sigmoid) HIPRWKV_GATE_LAUNCH(bf16_t, true); else HIPRWKV_GATE_LAUNCH(bf16_t, false); }
#undef HIPRWKV_GATE_LAUNCH
  return hipGetLastError();
}

hipError_t launch_rwkv7_decay_bwd(int io_f32, int sigmoid, int64_t rows, int64_t C, const void* x, const void* w0,
                                  const void* g, void* dx, float* dw0, hipStream_t stream) {
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((C + 255) / 256)), dim3(256), 0, stream, dw0, C);
  const BwdGrid G = bwd_grid(rows, C);
  const dim3 block(GATE_THREADS);
#define HIPRWKV_GATE_LAUNCH(TY, SG)                                                                                \
  hipLaunchKernelGGL((rwkv7_decay_bwd_kernel<TY, SG>), G.grid, block, 0, stream, rows, C, G.run, (const TY*)x,     \
                     (const TY*)w0, (const TY*)g, (TY*)dx, dw0)
  if (io_f32) { if (sigmoid) HIPRWKV_GATE_LAUNCH(float, true); else HIPRWKV_GATE_LAUNCH(float, false); }
  else { if (sigmoid) HIPRWKV_GATE_LAUNCH(bf16_t, true); else HIPRWKV_GATE_LAUNCH(bf16_t, false); }
#undef HIPRWKV_GATE_LAUNCH
  return hipGetLastError();
}

// g == nullptr: forward (out = relu(x)^2); else backward (out = 2 g relu(x))
hipError_t launch_rwkv7_relusq(int io_f32, int64_t n, const void* x, const void* g, void* out, hipStream_t stream) {
  const int64_t n8 = n / 8;
  const dim3 grid((unsigned)((n8 + GATE_THREADS - 1) / GATE_THREADS)), block(GATE_THREADS);
#define HIPRWKV_GATE_LAUNCH(TY, BW) \
  hipLaunchKernelGGL((rwkv7_relusq_kernel<TY, BW>), grid, block, 0, stream, n8, (const TY*)x, (const TY*)g, (TY*)out)
  if (io_f32) { if (g) HIPRWKV_GATE_LAUNCH(float, true); else HIPRWKV_GATE_LAUNCH(float, false); }
  else { if (g) HIPRWKV_GATE_LAUNCH(bf16_t, true); else HIPRWKV_GATE_LAUNCH(bf16_t, false); }
#undef HIPRWKV_GATE_LAUNCH
  return hipGetLastError();
}

hipError_t launch_rwkv7_vmix(int io_f32, int64_t rows, int64_t C, const void* v, const void* v_first, const void* x,
                             const void* v0, void* out, hipStream_t stream) {
  const dim3 grid((unsigned)((rows * (C / 8) + GATE_THREADS - 1) / GATE_THREADS)), block(GATE_THREADS);
  if (io_f32) hipLaunchKernelGGL(rwkv7_vmix_kernel<float>, grid, block, 0, stream, rows, C, (const float*)v, (const float*)v_first, (const float*)x, (const float*)v0, (float*)out);
  else hipLaunchKernelGGL(rwkv7_vmix_kernel<bf16_t>, grid, block, 0, stream, rows, C, (const bf16_t*)v, (const bf16_t*)v_first, (const bf16_t*)x, (const bf16_t*)v0, (bf16_t*)out);
  return hipGetLastError();
}

hipError_t launch_rwkv7_vmix_bwd(int io_f32, int64_t rows, int64_t C, const void* v, const void* v_first, const void* x,
                                 const void* v0, const void* g, void* dv, void* dv_first, void* dx, float* dv0,
                                 hipStream_t stream) {
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((C + 255) / 256)), dim3(256), 0, stream, dv0, C);
  const BwdGrid G = bwd_grid(rows, C);
  const dim3 block(GATE_THREADS);
  if (io_f32) hipLaunchKernelGGL(rwkv7_vmix_bwd_kernel<float>, G.grid, block, 0, stream, rows, C, G.run, (const float*)v, (const float*)v_first, (const float*)x, (const float*)v0, (const float*)g, (float*)dv, (float*)dv_first, (float*)dx, dv0);
  else hipLaunchKernelGGL(rwkv7_vmix_bwd_kernel<bf16_t>, G.grid, block, 0, stream, rows, C, G.run, (const bf16_t*)v, (const bf16_t*)v_first, (const bf16_t*)x, (const bf16_t*)v0, (const bf16_t*)g, (bf16_t*)dv, (bf16_t*)dv_first, (bf16_t*)dx, dv0);
  return hipGetLastError();
}

}  // namespace hiprwkv
