// Element-wise stages of RWKV-7 time mixing on either side of the WKV op, fused into two memory-bound kernels
// (reference: /root/reference/src/jaxrwkv/rwkv7.py:248-252 and :263-265).  Sixteen lanes (one DPP row) per
// (token, head), four consecutive channels per lane: a wavefront handles four (token, head) units with one 8- or
// 16-byte access per lane and array, and the per-head reductions (L2 norm, mean/variance, r.k.r_k) are four
// DPP row rotations each; nothing goes through LDS.  fp32 arithmetic, fp32 or bf16 I/O.
//
//   pre :  kk = normalize_head(k . k_k) ;  k' = k (1 + (a - 1) k_a) ;  a_i = -kk ;  b_i = kk . a
//   post:  out = ( group_norm_head(y; eps) . ln_w + ln_b + (sum_j r_j k'_j r_k_j) v ) . g
//
// The backward kernels recompute the forward quantities from the same inputs (nothing is saved) and return the
// cotangents of every input.  Those of the per-head parameters are sums over all tokens: a workgroup works on one
// head, its sixteen lane rows walk over that head's tokens with the partial sums in registers, the rows are added
// through LDS and one fp32 atomic per channel and workgroup lands in the (H, 64) fp32 result, which the launcher
// zeroes first with a fill kernel on the same stream.
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

constexpr int BWD_ROWS = MIX_THREADS / 16;   // lane rows per workgroup

__global__ void zero_f32_kernel(float* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// adds NP per-lane partial sums (four channels each) over the workgroup's lane rows and into out[p][h][64]
template <int NP>
__device__ __forceinline__ void reduce_params(const float (&part)[NP][4], float* const (&out)[NP], int64_t h) {
  __shared__ float red[NP][BWD_ROWS][64];
  const int grp = threadIdx.x >> 4, c4 = 4 * (threadIdx.x & 15);
#pragma unroll
  for (int p = 0; p < NP; ++p)
    *reinterpret_cast<float4*>(&red[p][grp][c4]) = make_float4(part[p][0], part[p][1], part[p][2], part[p][3]);
  __syncthreads();
  for (int i = threadIdx.x; i < NP * 64; i += MIX_THREADS) {
    const int p = i >> 6, c = i & 63;
    float sum = 0.f;
#pragma unroll
    for (int g = 0; g < BWD_ROWS; ++g) sum += red[p][g][c];
    atomicAdd(out[p] + h * 64 + c, sum);
  }
}

// Workgroup b: head b % H, token rows (b / H) * 16 + lane row, stepping by 16 * (gridDim.x / H).
template <typename T>
__global__ __launch_bounds__(MIX_THREADS) void rwkv7_premix_bwd_kernel(
    int64_t rows, int64_t H, const T* __restrict__ k, const T* __restrict__ a, const T* __restrict__ k_k,
    const T* __restrict__ k_a, const T* __restrict__ gko, const T* __restrict__ gao, const T* __restrict__ gbo,
    T* __restrict__ gk, T* __restrict__ ga, float* __restrict__ gk_k, float* __restrict__ gk_a) {
  const int64_t h = blockIdx.x % H, rb = blockIdx.x / H, nrb = gridDim.x / H;
  const int grp = threadIdx.x >> 4, c4 = 4 * (threadIdx.x & 15);
  float kkw[4], kaw[4];
  ld4(k_k + h * 64 + c4, kkw); ld4(k_a + h * 64 + c4, kaw);
  float part[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  // every lane row runs the same number of rounds; rows beyond the end redo the last token without storing
  for (int64_t base = rb * BWD_ROWS; base < rows; base += nrb * BWD_ROWS) {
    const int64_t row = base + grp;
    const bool active = row < rows;
    const size_t el = (size_t)((active ? row : rows - 1) * H + h) * 64 + c4;
    float kv[4], av[4], dko[4], dao[4], dbo[4];
    ld4(k + el, kv); ld4(a + el, av); ld4(gko + el, dko); ld4(gao + el, dao); ld4(gbo + el, dbo);
    float kk[4], gkk[4], ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) { kk[i] = kv[i] * kkw[i]; ss = fmaf(kk[i], kk[i], ss); }
    const float nrm = sqrtf(row_sum(ss));
    const float inv = 1.f / fmaxf(nrm, 1e-12f);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      kk[i] *= inv;
      gkk[i] = dbo[i] * av[i] - dao[i];             // a_i = -kk, b_i = kk a
      dot = fmaf(kk[i], gkk[i], dot);
    }
    dot = nrm >= 1e-12f ? row_sum(dot) : 0.f;       // below the clamp the norm is a constant
    float ok[4], oa[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float graw = (gkk[i] - kk[i] * dot) * inv;            // cotangent of k . k_k
      ok[i] = dko[i] * (1.f + (av[i] - 1.f) * kaw[i]) + graw * kkw[i];
      oa[i] = dbo[i] * kk[i] + dko[i] * kv[i] * kaw[i];
      if (active) {
        part[0][i] = fmaf(graw, kv[i], part[0][i]);
        part[1][i] = fmaf(dko[i] * kv[i], av[i] - 1.f, part[1][i]);
      }
    }
    if (active) { st4(gk + el, ok); st4(ga + el, oa); }
  }
  float* const outs[2] = {gk_k, gk_a};
  reduce_params<2>(part, outs, h);
}

template <typename T>
__global__ __launch_bounds__(MIX_THREADS) void rwkv7_postmix_bwd_kernel(
    int64_t rows, int64_t H, const T* __restrict__ y, const T* __restrict__ r, const T* __restrict__ k,
    const T* __restrict__ v, const T* __restrict__ g, const T* __restrict__ ln_w, const T* __restrict__ ln_b,
    const T* __restrict__ r_k, float eps, const T* __restrict__ go, T* __restrict__ gy, T* __restrict__ gr,
    T* __restrict__ gk, T* __restrict__ gv, T* __restrict__ gg, float* __restrict__ gln_w, float* __restrict__ gln_b,
    float* __restrict__ gr_k) {
  const int64_t h = blockIdx.x % H, rb = blockIdx.x / H, nrb = gridDim.x / H;
  const int grp = threadIdx.x >> 4, c4 = 4 * (threadIdx.x & 15);
  float lw[4], lb[4], rk[4];
  ld4(ln_w + h * 64 + c4, lw); ld4(ln_b + h * 64 + c4, lb); ld4(r_k + h * 64 + c4, rk);
  float part[3][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int64_t base = rb * BWD_ROWS; base < rows; base += nrb * BWD_ROWS) {
    const int64_t row = base + grp;
    const bool active = row < rows;
    const size_t el = (size_t)((active ? row : rows - 1) * H + h) * 64 + c4;
    float yv[4], rv[4], kv[4], vv[4], gv_[4], dout[4];
    ld4(y + el, yv); ld4(r + el, rv); ld4(k + el, kv); ld4(v + el, vv); ld4(g + el, gv_); ld4(go + el, dout);
    const float mean = row_sum(yv[0] + yv[1] + yv[2] + yv[3]) * (1.f / 64.f);
    float xh[4], sq = 0.f, dot = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xh[i] = yv[i] - mean;
      sq = fmaf(xh[i], xh[i], sq);
      dot = fmaf(rv[i] * kv[i], rk[i], dot);
    }
    const float rstd = rsqrtf(row_sum(sq) * (1.f / 64.f) + eps);
    const float bonus = row_sum(dot);
    float t[4], gx[4], s1 = 0.f, s2 = 0.f, sv = 0.f, og[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xh[i] *= rstd;
      og[i] = dout[i] * (xh[i] * lw[i] + lb[i] + bonus * vv[i]);   // cotangent of the gate
      t[i] = dout[i] * gv_[i];                                    // cotangent of the gated sum
      gx[i] = t[i] * lw[i];
      s1 += gx[i];
      s2 = fmaf(gx[i], xh[i], s2);
      sv = fmaf(t[i], vv[i], sv);
    }
    s1 = row_sum(s1) * (1.f / 64.f);
    s2 = row_sum(s2) * (1.f / 64.f);
    const float gbonus = row_sum(sv);
    float oy[4], orr[4], okk[4], ov[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      oy[i] = rstd * (gx[i] - s1 - xh[i] * s2);
      orr[i] = gbonus * kv[i] * rk[i];
      okk[i] = gbonus * rv[i] * rk[i];
      ov[i] = t[i] * bonus;
      if (active) {
        part[0][i] = fmaf(t[i], xh[i], part[0][i]);
        part[1][i] += t[i];
        part[2][i] = fmaf(gbonus * rv[i], kv[i], part[2][i]);
      }
    }
    if (active) { st4(gy + el, oy); st4(gr + el, orr); st4(gk + el, okk); st4(gv + el, ov); st4(gg + el, og); }
  }
  float* const outs[3] = {gln_w, gln_b, gr_k};
  reduce_params<3>(part, outs, h);
}

// workgroups per head: enough to fill the GPU, never more than there are 16-token groups
inline unsigned bwd_row_blocks(int64_t rows, int64_t H) {
  const int64_t want = (4096 + H - 1) / H, have = (rows + BWD_ROWS - 1) / BWD_ROWS;
  const int64_t n = want < have ? want : have;
  return (unsigned)(n < 1 ? 1 : n);
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

hipError_t launch_rwkv7_premix_bwd(int io_f32, int64_t rows, int64_t H, const void* k, const void* a, const void* k_k,
                                   const void* k_a, const void* gko, const void* gao, const void* gbo, void* gk,
                                   void* ga, float* gk_k, float* gk_a, hipStream_t stream) {
  const int np = (int)(H * 64);
  hipLaunchKernelGGL(zero_f32_kernel, dim3((np + 255) / 256), dim3(256), 0, stream, gk_k, np);
  hipLaunchKernelGGL(zero_f32_kernel, dim3((np + 255) / 256), dim3(256), 0, stream, gk_a, np);
  const dim3 grid((unsigned)H * bwd_row_blocks(rows, H)), block(MIX_THREADS);
  if (io_f32)
    hipLaunchKernelGGL(rwkv7_premix_bwd_kernel<float>, grid, block, 0, stream, rows, H, (const float*)k,
                       (const float*)a, (const float*)k_k, (const float*)k_a, (const float*)gko, (const float*)gao,
                       (const float*)gbo, (float*)gk, (float*)ga, gk_k, gk_a);
  else
    hipLaunchKernelGGL(rwkv7_premix_bwd_kernel<bf16_t>, grid, block, 0, stream, rows, H, (const bf16_t*)k,
                       (const bf16_t*)a, (const bf16_t*)k_k, (const bf16_t*)k_a, (const bf16_t*)gko,
                       (const bf16_t*)gao, (const bf16_t*)gbo, (bf16_t*)gk, (bf16_t*)ga, gk_k, gk_a);
  return hipGetLastError();
}

hipError_t launch_rwkv7_postmix_bwd(int io_f32, int64_t rows, int64_t H, const void* y, const void* r, const void* k,
                                    const void* v, const void* g, const void* ln_w, const void* ln_b, const void* r_k,
                                    float eps, const void* go, void* gy, void* gr, void* gk, void* gv, void* gg,
                                    float* gln_w, float* gln_b, float* gr_k, hipStream_t stream) {
  const int np = (int)(H * 64);
  hipLaunchKernelGGL(zero_f32_kernel, dim3((np + 255) / 256), dim3(256), 0, stream, gln_w, np);
  hipLaunchKernelGGL(zero_f32_kernel, dim3((np + 255) / 256), dim3(256), 0, stream, gln_b, np);
  hipLaunchKernelGGL(zero_f32_kernel, dim3((np + 255) / 256), dim3(256), 0, stream, gr_k, np);
  const dim3 grid((unsigned)H * bwd_row_blocks(rows, H)), block(MIX_THREADS);
  if (io_f32)
    hipLaunchKernelGGL(rwkv7_postmix_bwd_kernel<float>, grid, block, 0, stream, rows, H, (const float*)y,
                       (const float*)r, (const float*)k, (const float*)v, (const float*)g, (const float*)ln_w,
                       (const float*)ln_b, (const float*)r_k, eps, (const float*)go, (float*)gy, (float*)gr,
                       (float*)gk, (float*)gv, (float*)gg, gln_w, gln_b, gr_k);
  else
    hipLaunchKernelGGL(rwkv7_postmix_bwd_kernel<bf16_t>, grid, block, 0, stream, rows, H, (const bf16_t*)y,
                       (const bf16_t*)r, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)g, (const bf16_t*)ln_w,
                       (const bf16_t*)ln_b, (const bf16_t*)r_k, eps, (const bf16_t*)go, (bf16_t*)gy, (bf16_t*)gr,
                       (bf16_t*)gk, (bf16_t*)gv, (bf16_t*)gg, gln_w, gln_b, gr_k);
  return hipGetLastError();
}

}  // namespace hiprwkv
