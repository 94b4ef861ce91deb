// Token shift and interpolation at the head of RWKV-7 time mixing and channel mixing, one memory-bound kernel each way
// (reference: /root/reference/src/jaxrwkv/rwkv7.py:226-235 and :192-195):
//     sx_t = (new_starts[t] ? 0 : x_{t-1}) - x_t        (x_{-1} = the layer's token-shift row of the model state)
//     out_i = x + sx . mix_i          i = 0 .. NOUT-1     (six interpolations in time mixing, one in channel mixing)
// The reference leaves these to XLA's fusion; as separate tensor operations they cost about forty passes over a (T, C)
// tensor per layer.  Here x is read once (the previous token's row comes from the cache) and every output written once.
// A thread owns eight consecutive channels (one 16-byte access in bf16); fp32 arithmetic, one rounding per output.
//
// Backward, for cotangents g_i of the outputs:
//     dx_t   = sum_i g_i,t (1 - mix_i) + (t+1 < T and not new_starts[t+1]) sum_i g_i,t+1 mix_i
//     dprev  = not new_starts[0] ? sum_i g_i,0 mix_i : 0
//     dmix_i = sum over sequences and tokens of g_i,t . sx_t
// A workgroup walks down a run of consecutive tokens with the sum_i g_i mix_i of the token after in registers, so
// every g is read once; a thread keeps the partial sums of dmix for its own channels and adds them to the fp32
// result with one atomic per channel and workgroup (the launcher zeroes the result first with a fill kernel).
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

constexpr int SHIFT_THREADS = 256;
constexpr int MAX_MIX = 6;

struct MixPtrs {
  const void* mix[MAX_MIX];   // (C,) each, I/O dtype
  void* out[MAX_MIX];         // forward: outputs (B,T,C); backward: unused
  const void* g[MAX_MIX];     // backward: cotangents of the outputs
};

template <typename T>
__device__ __forceinline__ void ld8z(const T* p, bool take, float (&o)[8]) {
  if (take) {
    ld8(p, o);
  } else {
#pragma unroll
    for (int c = 0; c < 8; ++c) o[c] = 0.f;
  }
}

// thread -> (token n = b*T + t, channels c8 .. c8+7)
template <typename T, int NOUT>
__global__ __launch_bounds__(SHIFT_THREADS) void rwkv7_shiftmix_kernel(int64_t B, int64_t Tn, int64_t C, const T* __restrict__ x,
                                                                       const T* __restrict__ prev, int64_t prev_bstride,
                                                                       const uint8_t* __restrict__ ns, MixPtrs P) {
  const int64_t per_tok = C / 8;
  const int64_t idx = (int64_t)blockIdx.x * SHIFT_THREADS + threadIdx.x;
  if (idx >= B * Tn * per_tok) return;
  const int64_t n = idx / per_tok;
  const int c8 = (int)(idx % per_tok) * 8;
  const int64_t b = n / Tn, t = n % Tn;
  float xv[8], pv[8];
  ld8(x + n * C + c8, xv);
  const bool reset = ns != nullptr && ns[n] != 0;
  ld8z(t == 0 ? prev + b * prev_bstride + c8 : x + (n - 1) * C + c8, !reset, pv);
#pragma unroll
  for (int i = 0; i < NOUT; ++i) {
    float m[8], o[8];
    ld8(reinterpret_cast<const T*>(P.mix[i]) + c8, m);
#pragma unroll
    for (int c = 0; c < 8; ++c) o[c] = fmaf(pv[c] - xv[c], m[c], xv[c]);
    st8(reinterpret_cast<T*>(P.out[i]) + n * C + c8, o);
  }
}

// Workgroup (blockIdx.x = channel block, blockIdx.y = run of `run` consecutive tokens), walking the run downwards.
template <typename T, int NOUT>
__global__ __launch_bounds__(SHIFT_THREADS) void rwkv7_shiftmix_bwd_kernel(int64_t B, int64_t Tn, int64_t C, int64_t run,
                                                                           const T* __restrict__ x, const T* __restrict__ prev,
                                                                           int64_t prev_bstride, const uint8_t* __restrict__ ns,
                                                                           MixPtrs P, T* __restrict__ dx, T* __restrict__ dprev,
                                                                           int64_t dprev_bstride, float* __restrict__ dmix) {
  const int c8 = (blockIdx.x * SHIFT_THREADS + threadIdx.x) * 8;
  if (c8 >= C) return;
  const int64_t total = B * Tn;
  const int64_t n0 = (int64_t)blockIdx.y * run;
  const int64_t n1 = (n0 + run < total ? n0 + run : total) - 1;       // last token of the run
  float m[NOUT][8], acc[NOUT][8];
#pragma unroll
  for (int i = 0; i < NOUT; ++i) {
    ld8(reinterpret_cast<const T*>(P.mix[i]) + c8, m[i]);
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[i][c] = 0.f;
  }
  // sum_i g_i mix_i of the token after the run, if that token takes its shifted value from the run's last token
  float gm_next[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) gm_next[c] = 0.f;
  if (n1 + 1 < total && (n1 + 1) % Tn != 0 && !(ns != nullptr && ns[n1 + 1] != 0)) {
#pragma unroll
    for (int i = 0; i < NOUT; ++i) {
      float g[8];
      ld8(reinterpret_cast<const T*>(P.g[i]) + (n1 + 1) * C + c8, g);
#pragma unroll
      for (int c = 0; c < 8; ++c) gm_next[c] = fmaf(g[c], m[i][c], gm_next[c]);
    }
  }
  for (int64_t n = n1; n >= n0; --n) {
    const int64_t b = n / Tn, t = n % Tn;
    const bool reset = ns != nullptr && ns[n] != 0;
    float xv[8], pv[8];
    ld8(x + n * C + c8, xv);
    ld8z(t == 0 ? prev + b * prev_bstride + c8 : x + (n - 1) * C + c8, !reset, pv);
    float gsum[8], gm[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) { gsum[c] = 0.f; gm[c] = 0.f; }
#pragma unroll
    for (int i = 0; i < NOUT; ++i) {
      float g[8];
      ld8(reinterpret_cast<const T*>(P.g[i]) + n * C + c8, g);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        gsum[c] += g[c];
        gm[c] = fmaf(g[c], m[i][c], gm[c]);
        acc[i][c] = fmaf(g[c], pv[c] - xv[c], acc[i][c]);
      }
    }
    float o[8];
    const bool last_of_seq = t == Tn - 1;
#pragma unroll
    for (int c = 0; c < 8; ++c) o[c] = gsum[c] - gm[c] + (last_of_seq ? 0.f : gm_next[c]);
    st8(dx + n * C + c8, o);
    // what this token hands to the one before it (or to the state row)
#pragma unroll
    for (int c = 0; c < 8; ++c) gm_next[c] = reset ? 0.f : gm[c];
    if (t == 0) st8(dprev + b * dprev_bstride + c8, gm_next);
  }
#pragma unroll
  for (int i = 0; i < NOUT; ++i)
#pragma unroll
    for (int c = 0; c < 8; ++c) atomicAdd(dmix + (size_t)i * C + c8 + c, acc[i][c]);
}

__global__ void fill_zero_kernel(float* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

MixPtrs pack(int n_out, const void* const* mix, void* const* out, const void* const* g) {
  MixPtrs P;
  for (int i = 0; i < MAX_MIX; ++i) {
    P.mix[i] = i < n_out ? mix[i] : nullptr;
    P.out[i] = (out && i < n_out) ? out[i] : nullptr;
    P.g[i] = (g && i < n_out) ? g[i] : nullptr;
  }
  return P;
}

}  // namespace

hipError_t launch_rwkv7_shiftmix(int io_f32, int64_t B, int64_t T, int64_t C, int n_out, const void* x, const void* prev,
                                 int64_t prev_bstride, const uint8_t* ns, const void* const* mix, void* const* out,
                                 hipStream_t stream) {
  const MixPtrs P = pack(n_out, mix, out, nullptr);
  const int64_t threads = B * T * (C / 8);
  const dim3 grid((unsigned)((threads + SHIFT_THREADS - 1) / SHIFT_THREADS)), block(SHIFT_THREADS);
#define HIPRWKV_SHIFT_LAUNCH(TY, NO)                                                                              \
  hipLaunchKernelGGL((rwkv7_shiftmix_kernel<TY, NO>), grid, block, 0, stream, B, T, C, (const TY*)x, (const TY*)prev, \
                     prev_bstride, ns, P)
  if (io_f32) { if (n_out == 1) HIPRWKV_SHIFT_LAUNCH(float, 1); else HIPRWKV_SHIFT_LAUNCH(float, 6); }
  else { if (n_out == 1) HIPRWKV_SHIFT_LAUNCH(bf16_t, 1); else HIPRWKV_SHIFT_LAUNCH(bf16_t, 6); }
#undef HIPRWKV_SHIFT_LAUNCH
  return hipGetLastError();
}

hipError_t launch_rwkv7_shiftmix_bwd(int io_f32, int64_t B, int64_t T, int64_t C, int n_out, const void* x,
                                     const void* prev, int64_t prev_bstride, const uint8_t* ns, const void* const* mix,
                                     const void* const* g, void* dx, void* dprev, int64_t dprev_bstride, float* dmix,
                                     hipStream_t stream) {
  const MixPtrs P = pack(n_out, mix, nullptr, g);
  const int64_t nz = (int64_t)n_out * C;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, stream, dmix, nz);
  // runs of tokens: about two workgroups per CU.  Every workgroup ends with one atomic per channel and output, and
  // those set the pace beyond that (B=16 T=4096 C=2048, six outputs: 0.66 ms with 512 workgroups, 0.84 with 1024,
  // 1.13 with 2048, 1.84 with 4096; 1.06 with 128)
  const int64_t total = B * T;
  const unsigned cblocks = (unsigned)((C / 8 + SHIFT_THREADS - 1) / SHIFT_THREADS);
  int64_t run = (total * cblocks + 511) / 512;
  run = run < 16 ? 16 : run;
  const dim3 grid(cblocks, (unsigned)((total + run - 1) / run)), block(SHIFT_THREADS);
#define HIPRWKV_SHIFT_LAUNCH(TY, NO)                                                                                   \
  hipLaunchKernelGGL((rwkv7_shiftmix_bwd_kernel<TY, NO>), grid, block, 0, stream, B, T, C, run, (const TY*)x,           \
                     (const TY*)prev, prev_bstride, ns, P, (TY*)dx, (TY*)dprev, dprev_bstride, dmix)
  if (io_f32) { if (n_out == 1) HIPRWKV_SHIFT_LAUNCH(float, 1); else HIPRWKV_SHIFT_LAUNCH(float, 6); }
  else { if (n_out == 1) HIPRWKV_SHIFT_LAUNCH(bf16_t, 1); else HIPRWKV_SHIFT_LAUNCH(bf16_t, 6); }
#undef HIPRWKV_SHIFT_LAUNCH
  return hipGetLastError();
}

}  // namespace hiprwkv
