// WKV4 forward: per-channel max-tracked recurrence, one thread per (sequence, channel).
//
// Reference: BaseRWKV.inner_loop, /root/reference/src/jaxrwkv/rwkv4.py:144-172, in the operand convention of the
// reference's native op (rwkv4.py:311-323): w = -exp(time_decay) is passed in, the receptance is applied outside.
//     ww = u + k_t ; q = max(pp, ww) ; y_t = (e^{pp-q} aa + e^{ww-q} v_t) / (e^{pp-q} bb + e^{ww-q})
//     ww = pp + w  ; q = max(ww, k_t) ; aa = e^{ww-q} aa + e^{k_t-q} v_t ; bb = e^{ww-q} bb + e^{k_t-q} ; pp = q
// In each pair of exponentials one argument is exactly 0, so a step costs two exp, not four.
// k and v are streamed with a register prefetch of TB steps per thread (coalesced across channels), which keeps
// enough bytes in flight to cover HBM latency with the few waves per CU this problem has.
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

constexpr int W4_THREADS = 64;
constexpr int W4_TB = 16;
constexpr float W4_RESET_PP = -1e30f;  // rwkv4.py:149-150

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_fwd_kernel(Wkv4Args A) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  if (c >= A.C) return;
  const IO* kp = reinterpret_cast<const IO*>(A.k) + (size_t)b * A.T * A.C + c;
  const IO* vp = reinterpret_cast<const IO*>(A.v) + (size_t)b * A.T * A.C + c;
  IO* yp = reinterpret_cast<IO*>(A.out) + (size_t)b * A.T * A.C + c;
  const IO* sp = reinterpret_cast<const IO*>(A.s) + (size_t)b * 3 * A.C + c;
  IO* nsp = reinterpret_cast<IO*>(A.new_s) + (size_t)b * 3 * A.C + c;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + c);
  const float u = ld_f(reinterpret_cast<const IO*>(A.u) + c);
  float aa = ld_f(sp), bb = ld_f(sp + A.C), pp = ld_f(sp + 2 * A.C);
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const bool q2drop = (A.flags & 1u) && L < A.T && ns != nullptr && ns[L] != 0;
  if (L == 0) {
    st_f(nsp, q2drop ? 0.f : aa);
    st_f(nsp + A.C, q2drop ? 0.f : bb);
    st_f(nsp + 2 * A.C, q2drop ? W4_RESET_PP : pp);
  }

  float kb[W4_TB], vb[W4_TB];
  auto fetch = [&](int64_t t0) {
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      const int64_t t = t0 + x;
      if (t < A.T) {
        kb[x] = ld_f(kp + (size_t)t * A.C);
        vb[x] = ld_f(vp + (size_t)t * A.C);
      } else {
        kb[x] = 0.f;
        vb[x] = 0.f;
      }
    }
  };
  fetch(0);
  for (int64_t t0 = 0; t0 < A.T; t0 += W4_TB) {
    float kc[W4_TB], vc[W4_TB];
    uint32_t rmask = 0;
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      kc[x] = kb[x];
      vc[x] = vb[x];
      if (ns != nullptr && t0 + x < A.T && ns[t0 + x]) rmask |= 1u << x;
    }
    if (t0 + W4_TB < A.T) fetch(t0 + W4_TB);
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      const int64_t t = t0 + x;
      if (t < A.T) {
      if (rmask & (1u << x)) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
      const float kt = kc[x], vt = vc[x];
      {
        const float diff = pp - (u + kt);                  // e1 = e^{pp-q}, e2 = e^{ww-q}
        const float e = __expf(-fabsf(diff));
        const float e1 = diff >= 0.f ? 1.f : e;
        const float e2 = diff >= 0.f ? e : 1.f;
        const float num = fmaf(e1, aa, e2 * vt);
        const float den = fmaf(e1, bb, e2);
        st_f(yp + (size_t)t * A.C, __fdividef(num, den));
      }
      {
        const float ww = pp + w;
        const float diff = ww - kt;                        // e1 = e^{ww-q}, e2 = e^{k-q}
        const float e = __expf(-fabsf(diff));
        const float e1 = diff >= 0.f ? 1.f : e;
        const float e2 = diff >= 0.f ? e : 1.f;
        aa = fmaf(e1, aa, e2 * vt);
        bb = fmaf(e1, bb, e2);
        pp = fmaxf(ww, kt);
      }
      if (t == L - 1) {
        st_f(nsp, q2drop ? 0.f : aa);
        st_f(nsp + A.C, q2drop ? 0.f : bb);
        st_f(nsp + 2 * A.C, q2drop ? W4_RESET_PP : pp);
      }
      }
    }
  }
}

hipError_t launch_wkv4_fwd(const Wkv4Args& A, hipStream_t stream) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const dim3 grid((unsigned)(A.B * cblocks)), block(W4_THREADS);
  if (A.io_f32) hipLaunchKernelGGL(wkv4_fwd_kernel<float>, grid, block, 0, stream, A);
  else hipLaunchKernelGGL(wkv4_fwd_kernel<bf16_t>, grid, block, 0, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
