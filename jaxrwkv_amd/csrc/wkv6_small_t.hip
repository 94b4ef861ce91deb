// WKV6 forward for very short sequences (decode: T = 1 .. 8), gfx950.
//
// At T = 1 the op is pure state traffic: read the 64x64 state of every (sequence, head), apply one step of
//     S' = new_starts[t] ? 0 : S ;  y_t[j] = sum_i r_i (u_i k_i v_j + S'[i][j]) ;  S = diag(exp(w_t)) S' + k_t v_t^T
// (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191; S[i][j] = key row i, value column j) and write it
// back: 2 x 16 KB per head in fp32 against 640 B of token vectors.  The chunked kernel (one 8-wave workgroup with an
// LDS ring per head) and the staged sequential kernel are workgroup-launch bound there; this kernel has no LDS, no
// barrier and no per-launch set-up: 256 threads per head, thread (column j = tid/4, quarter q = tid%4) keeps the 16
// state elements S[16q..16q+15][j] in registers.  One load instruction of a wave covers four 64-byte pieces of four
// state rows, and the other waves of the workgroup take the rest of those rows, so every fetched line is used
// whole.  The thread reads its 16 key channels of r, k, w, u straight from global memory (the 64 columns share
// them through the cache) and reduces the dot product over the quad with DPP.  fp32 arithmetic whatever the I/O and
// state dtypes.
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

template <typename ST>
__device__ __forceinline__ void st_col(void* base, size_t el, const float (&S)[16], bool zero) {
  ST* p = reinterpret_cast<ST*>(base) + el;
#pragma unroll
  for (int c = 0; c < 16; ++c) st_f(p + (size_t)c * 64, zero ? 0.f : S[c]);
}

template <typename IO, typename ST>
__global__ __launch_bounds__(256) void wkv6_small_t_kernel(Wkv6Args A) {
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  const int j = threadIdx.x >> 2, q = threadIdx.x & 3, c0 = 16 * q;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const uint8_t* ns = A.ns ? A.ns + b * A.T : nullptr;
  // the returned state is the reset state there (associative-scan rule)
  const bool q2drop = (A.flags & 1u) && L < A.T && ns != nullptr && ns[L] != 0;
  // a sequence's state is H*64*64 contiguous elements; consecutive sequences may lie further apart (a layer's rows of
  // a packed model state).  Every thread reads its 16 elements once, up front, and writes them once: s and new_s may
  // be the same memory.
  const size_t in_head = ((size_t)h * 64 + c0) * 64 + j;
  const size_t dense = (size_t)A.H * 4096;
  const size_t sel = (size_t)b * (A.s_bstride ? (size_t)A.s_bstride : dense) + in_head;
  const size_t sel_out = (size_t)b * (A.new_s_bstride ? (size_t)A.new_s_bstride : dense) + in_head;
  float S[16], u[16];
  {
    const ST* p = reinterpret_cast<const ST*>(A.s) + sel;
#pragma unroll
    for (int c = 0; c < 16; ++c) S[c] = ld_f(p + (size_t)c * 64);
  }
  ld16<IO>(A.u, (size_t)h * 64 + c0, u);
  if (L == 0) st_col<ST>(A.new_s, sel_out, S, q2drop);
  for (int64_t t = 0; t < A.T; ++t) {
    const size_t tel = (((size_t)b * A.T + t) * A.H + h) * 64;
    float w[16], r[16], k[16];
    ld16<IO>(A.w, ((A.flags & FLAG_W_PER_HEAD) ? (size_t)h * 64 : tel) + c0, w);
    ld16<IO>(A.k, tel + c0, k);
    ld16<IO>(A.r, tel + c0, r);
    const float vj = ld_f(reinterpret_cast<const IO*>(A.v) + tel + j);
    if (ns != nullptr && ns[t]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    float y0 = 0.f, y1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; c += 2) {
      // fp32 I/O keeps the accurate exponential of the sequential kernel; bf16 inputs do not need it
      const float d0 = sizeof(IO) == 4 ? expf(w[c]) : __expf(w[c]);
      const float d1 = sizeof(IO) == 4 ? expf(w[c + 1]) : __expf(w[c + 1]);
      const float kv0 = k[c] * vj, kv1 = k[c + 1] * vj;
      y0 = fmaf(r[c], fmaf(u[c], kv0, S[c]), y0);
      y1 = fmaf(r[c + 1], fmaf(u[c + 1], kv1, S[c + 1]), y1);
      S[c] = fmaf(d0, S[c], kv0);
      S[c + 1] = fmaf(d1, S[c + 1], kv1);
    }
    const float y = quad_sum(y0 + y1);
    if (q == 0) st_f(reinterpret_cast<IO*>(A.out) + tel + j, y);
    if (t == L - 1) st_col<ST>(A.new_s, sel_out, S, q2drop);
  }
}

}  // namespace

hipError_t launch_wkv6_small_t_fwd(const Wkv6Args& A, hipStream_t stream) {
  const dim3 grid((unsigned)(A.B * A.H)), block(256);
  if (A.io_f32) {
    if (A.st_f32) hipLaunchKernelGGL((wkv6_small_t_kernel<float, float>), grid, block, 0, stream, A);
    else hipLaunchKernelGGL((wkv6_small_t_kernel<float, bf16_t>), grid, block, 0, stream, A);
  } else {
    if (A.st_f32) hipLaunchKernelGGL((wkv6_small_t_kernel<bf16_t, float>), grid, block, 0, stream, A);
    else hipLaunchKernelGGL((wkv6_small_t_kernel<bf16_t, bf16_t>), grid, block, 0, stream, A);
  }
  return hipGetLastError();
}

}  // namespace hiprwkv
