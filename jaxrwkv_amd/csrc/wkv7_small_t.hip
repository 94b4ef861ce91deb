// WKV7 forward for very short sequences (decode: T = 1 .. 8), gfx950.
//
// At T = 1 the op is pure state traffic: read the 64x64 state of every (sequence, head), apply one step of
//     S' = new_starts[t] ? 0 : S ;  sa = S' a_t ;  S = S' diag(d_t) + v_t k_t^T + sa b_t^T ;  y_t = S r_t
// (reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220) and write it back: 2 x 16 KB per head in fp32 against
// 896 B of token vectors.  The chunked kernel (one 8-wave workgroup with a 128 KB LDS ring per head) and the staged
// sequential kernel are workgroup-launch bound there; this kernel has no LDS, no barrier and no per-launch set-up:
// 256 threads per head, thread (row i = tid/4, quarter q = tid%4) keeps 16 contiguous state elements of value
// row i in registers (64-byte coalesced pieces of a 256-byte row), reads its 16 key channels of w, r, k, a, b
// straight from global memory (the four quarters of a row share them through the cache) and reduces the two dot
// products over the quad with DPP.  fp32 arithmetic whatever the I/O and state dtypes.
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

template <typename T>
__device__ __forceinline__ void st16(void* base, size_t el, const float (&o)[16], bool zero) {
  T* p = reinterpret_cast<T*>(base) + el;
  float lo[8], hi[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) { lo[c] = zero ? 0.f : o[c]; hi[c] = zero ? 0.f : o[8 + c]; }
  st8(p, lo);
  st8(p + 8, hi);
}

template <typename IO, typename ST>
__global__ __launch_bounds__(256) void wkv7_small_t_kernel(Wkv7Args A) {
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  const int i = threadIdx.x >> 2, q = threadIdx.x & 3, c0 = 16 * q;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const bool compat = (A.flags & 1u) != 0;
  const uint8_t* ns = A.ns ? A.ns + b * A.T : nullptr;
  // the returned state is the reset state there (associative-scan rule)
  const bool q2drop = compat && L < A.T && ns != nullptr && ns[L] != 0;
  // a sequence's state is H*64*64 contiguous elements; consecutive sequences may lie further apart (a layer's rows of
  // a packed model state).  Every thread reads its 16 elements once, up front, and writes them once: s and new_s may
  // be the same memory.
  const size_t in_head = ((size_t)h * 64 + i) * 64 + c0;
  const size_t dense = (size_t)A.H * 4096;
  const size_t sel = (size_t)b * (A.s_bstride ? (size_t)A.s_bstride : dense) + in_head;
  const size_t sel_out = (size_t)b * (A.new_s_bstride ? (size_t)A.new_s_bstride : dense) + in_head;
  float S[16];
  ld16<ST>(A.s, sel, S);
  if (L == 0) st16<ST>(A.new_s, sel_out, S, q2drop);   // rwkv7.py:203
  for (int64_t t = 0; t < A.T; ++t) {
    const size_t tel = (((size_t)b * A.T + t) * A.H + h) * 64;
    float w[16], r[16], k[16], a[16], bb[16];
    ld16<IO>(A.w, tel + c0, w);
    ld16<IO>(A.a, tel + c0, a);
    ld16<IO>(A.k, tel + c0, k);
    ld16<IO>(A.b, tel + c0, bb);
    ld16<IO>(A.r, tel + c0, r);
    const float vi = ld_f(reinterpret_cast<const IO*>(A.v) + tel + i);
    if (ns != nullptr && ns[t]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    float p = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) p = fmaf(S[c], a[c], p);
    const float sa = quad_sum(p);
    float y = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      // fp32 I/O keeps the accurate exponentials of the sequential kernel; bf16 inputs do not need them
      const float d = sizeof(IO) == 4 ? expf(-expf(w[c])) : __expf(-__expf(w[c]));
      S[c] = fmaf(S[c], d, fmaf(vi, k[c], sa * bb[c]));
      y = fmaf(S[c], r[c], y);
    }
    y = quad_sum(y);
    if (compat && t + 1 < A.T && ns != nullptr && ns[t + 1]) y = 0.f;   // rwkv7.py:331-333, 344
    if (q == 0) {
      st_f(reinterpret_cast<IO*>(A.out) + tel + i, y);
      if (A.sa != nullptr) {      // fp32 beside fp32 I/O, IEEE half beside bf16 I/O
        if (sizeof(IO) == 4) reinterpret_cast<float*>(A.sa)[tel + i] = sa;
        else reinterpret_cast<_Float16*>(A.sa)[tel + i] = (_Float16)sa;
      }
    }
    if (t == L - 1) st16<ST>(A.new_s, sel_out, S, q2drop);
  }
}

}  // namespace

hipError_t launch_wkv7_small_t_fwd(const Wkv7Args& A, hipStream_t stream) {
  const dim3 grid((unsigned)(A.B * A.H)), block(256);
  if (A.io_f32) {
    if (A.st_f32) hipLaunchKernelGGL((wkv7_small_t_kernel<float, float>), grid, block, 0, stream, A);
    else hipLaunchKernelGGL((wkv7_small_t_kernel<float, bf16_t>), grid, block, 0, stream, A);
  } else {
    if (A.st_f32) hipLaunchKernelGGL((wkv7_small_t_kernel<bf16_t, float>), grid, block, 0, stream, A);
    else hipLaunchKernelGGL((wkv7_small_t_kernel<bf16_t, bf16_t>), grid, block, 0, stream, A);
  }
  return hipGetLastError();
}

}  // namespace hiprwkv
