// WKV4 forward: per-channel max-tracked recurrence, one thread per (sequence, channel).
//
// Reference: BaseRWKV.inner_loop, /root/reference/src/jaxrwkv/rwkv4.py:144-172, in the operand convention of the
// reference's native op (rwkv4.py:311-323): w = -exp(time_decay) is passed in, the receptance is applied outside.
//     ww = u + k_t ; q = max(pp, ww) ; y_t = (e^{pp-q} aa + e^{ww-q} v_t) / (e^{pp-q} bb + e^{ww-q})
//     ww = pp + w  ; q = max(ww, k_t) ; aa = e^{ww-q} aa + e^{k_t-q} v_t ; bb = e^{ww-q} bb + e^{k_t-q} ; pp = q
// In each pair of exponentials one argument is exactly 0, so a step costs two exp, not four.
// k and v are streamed with a register prefetch of TB steps per thread (coalesced across channels), which keeps
// enough bytes in flight to cover HBM latency with the few waves per CU this problem has.  A lone wave issues one
// instruction every ~4.6 cycles whatever its kind, so the step is kept short: blocks of TB steps without a reset,
// a sequence end or the token length-1 run a loop without per-step checks, the reset flags of a block are fetched
// by one load (a byte per lane, one block ahead) and turned into a uniform mask, and the quotient is num * rcp(den)
// (v_rcp_f32 is good to 1 ulp; the reference divides, the difference is ~1e-7 relative).
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

constexpr int W4_THREADS = 64;
constexpr int W4_TB = 32;
constexpr float W4_RESET_PP = -1e30f;  // rwkv4.py:149-150

namespace {

// y_t from the state entering step t, then the state after it
__device__ __forceinline__ float wkv4_step(float& aa, float& bb, float& pp, float kt, float vt, float w, float u) {
  float y;
  {
    const float diff = pp - (u + kt);                  // e1 = e^{pp-q}, e2 = e^{ww-q}
    const float e = __expf(-fabsf(diff));
    const float e1 = diff >= 0.f ? 1.f : e;
    const float e2 = diff >= 0.f ? e : 1.f;
    const float num = fmaf(e1, aa, e2 * vt);
    const float den = fmaf(e1, bb, e2);
    y = num * __builtin_amdgcn_rcpf(den);
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
  return y;
}

// Raw buffer access: address = descriptor base (scalar) + lane offset (one VGPR, loop-invariant) + scalar offset.
// Stepping through the tokens then costs one scalar add for k, v and y together, and no vector address arithmetic.
using rsrc_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ float buf_ld(const float*, rsrc_t r, int voff, int soff) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ float buf_ld(const bf16_t*, rsrc_t r, int voff, int soff) {
  return bf16_to_f32(__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0));
}
__device__ __forceinline__ void buf_st(float*, float x, rsrc_t r, int voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(x), r, voff, soff, 0);
}
__device__ __forceinline__ void buf_st(bf16_t*, float x, rsrc_t r, int voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b16(f32_to_bf16(x), r, voff, soff, 0);
}

}  // namespace

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_fwd_kernel(Wkv4Args A) {
  static_assert(W4_TB <= W4_THREADS, "one lane per reset flag of a block");
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  // lanes beyond C work on channel C-1 as well: they load the same values and store the same results to the same
  // places as that channel's own lane, so no access needs a predicate
  const int64_t cc = c < A.C ? c : A.C - 1;
  const IO* kseq = reinterpret_cast<const IO*>(A.k) + (size_t)b * A.T * A.C;
  const IO* vseq = reinterpret_cast<const IO*>(A.v) + (size_t)b * A.T * A.C;
  IO* yseq = reinterpret_cast<IO*>(A.out) + (size_t)b * A.T * A.C;
  const IO* sp = reinterpret_cast<const IO*>(A.s) + (size_t)b * 3 * A.C + cc;
  IO* nsp = reinterpret_cast<IO*>(A.new_s) + (size_t)b * 3 * A.C + cc;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + cc);
  const float u = ld_f(reinterpret_cast<const IO*>(A.u) + cc);
  float aa = ld_f(sp), bb = ld_f(sp + A.C), pp = ld_f(sp + 2 * A.C);
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const bool q2drop = (A.flags & 1u) && L < A.T && ns != nullptr && ns[L] != 0;
  auto snapshot = [&]() {
    st_f(nsp, q2drop ? 0.f : aa);
    st_f(nsp + A.C, q2drop ? 0.f : bb);
    st_f(nsp + 2 * A.C, q2drop ? W4_RESET_PP : pp);
  };
  if (L == 0) snapshot();

  const int lane = threadIdx.x;
  const int voff = (int)(cc * sizeof(IO));
  const int stride = (int)(A.C * sizeof(IO));        // bytes between consecutive tokens
  float kb[W4_TB], vb[W4_TB];
  uint8_t nsb = 0;                                    // this lane's reset flag of the block after the current one
  auto fetch = [&](int64_t t0) {
    const rsrc_t rk = make_rsrc(kseq + (size_t)t0 * A.C), rv = make_rsrc(vseq + (size_t)t0 * A.C);
    int soff = 0;
    if (t0 + W4_TB <= A.T) {
#pragma unroll
      for (int x = 0; x < W4_TB; ++x) {
        kb[x] = buf_ld(kseq, rk, voff, soff);
        vb[x] = buf_ld(vseq, rv, voff, soff);
        soff += stride;
      }
    } else {
#pragma unroll
      for (int x = 0; x < W4_TB; ++x) {
        const bool in = t0 + x < A.T;
        kb[x] = in ? buf_ld(kseq, rk, voff, soff) : 0.f;
        vb[x] = in ? buf_ld(vseq, rv, voff, soff) : 0.f;
        soff += stride;
      }
    }
    nsb = 0;
    if (ns != nullptr && lane < W4_TB && t0 + lane < A.T) nsb = ns[t0 + lane];
  };
  fetch(0);
  for (int64_t t0 = 0; t0 < A.T; t0 += W4_TB) {
    float kc[W4_TB], vc[W4_TB];
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      kc[x] = kb[x];
      vc[x] = vb[x];
    }
    const uint64_t rmask = ns != nullptr ? __ballot(nsb != 0) : 0ull;
    if (t0 + W4_TB < A.T) fetch(t0 + W4_TB);
    const rsrc_t ry = make_rsrc(yseq + (size_t)t0 * A.C);
    int soff = 0;
    const bool plain = rmask == 0ull && t0 + W4_TB <= A.T && (L - 1 < t0 || L - 1 >= t0 + W4_TB);
    if (plain) {
#pragma unroll
      for (int x = 0; x < W4_TB; ++x) {
        buf_st(yseq, wkv4_step(aa, bb, pp, kc[x], vc[x], w, u), ry, voff, soff);
        soff += stride;
      }
    } else {
#pragma unroll
      for (int x = 0; x < W4_TB; ++x) {
        const int64_t t = t0 + x;
        if (t < A.T) {
          if (rmask & (1ull << x)) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
          buf_st(yseq, wkv4_step(aa, bb, pp, kc[x], vc[x], w, u), ry, voff, soff);
          if (t == L - 1) snapshot();
        }
        soff += stride;
      }
    }
  }
}

// ------------------------------------------------------------------ backward
// Reverse-mode derivative of the recurrence above, step by step (so that it agrees with autodiff of the
// reference's scan implementation, including how max() routes its cotangent).  The states entering each step are
// needed in reverse order: a first kernel re-runs the recurrence and keeps the state entering every W4_SEG-th
// step; the second kernel walks the segments backwards, recomputes the W4_SEG states of a segment into registers
// and then differentiates its steps last to first.
constexpr int W4_SEG = 16;

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_ckpt_kernel(Wkv4Args A) {
  static_assert(W4_SEG <= W4_THREADS, "one lane per reset flag of a segment");
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c0 = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  // lanes beyond C redo channel C-1 (same loads, same stores of the same values): every lane stays active for the
  // ballot that gathers a segment's reset flags
  const int64_t c = c0 < A.C ? c0 : A.C - 1;
  const int lane = threadIdx.x;
  const IO* kp = reinterpret_cast<const IO*>(A.k) + (size_t)b * A.T * A.C + c;
  const IO* vp = reinterpret_cast<const IO*>(A.v) + (size_t)b * A.T * A.C + c;
  const IO* sp = reinterpret_cast<const IO*>(A.s) + (size_t)b * 3 * A.C + c;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const int64_t nseg = (A.T + W4_SEG - 1) / W4_SEG;
  float* ck = A.ckpt + (size_t)b * nseg * 3 * A.C + c;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + c);
  float aa = ld_f(sp), bb = ld_f(sp + A.C), pp = ld_f(sp + 2 * A.C);
  for (int64_t sg = 0; sg < nseg; ++sg) {
    ck[(sg * 3 + 0) * A.C] = aa;
    ck[(sg * 3 + 1) * A.C] = bb;
    ck[(sg * 3 + 2) * A.C] = pp;
    float kc[W4_SEG], vc[W4_SEG];
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      const int64_t t = sg * W4_SEG + x;
      kc[x] = t < A.T ? ld_f(kp + (size_t)t * A.C) : 0.f;
      vc[x] = t < A.T ? ld_f(vp + (size_t)t * A.C) : 0.f;
    }
    // one flag per lane, gathered into a uniform mask
    bool mine = false;
    if (ns != nullptr && lane < W4_SEG && sg * W4_SEG + lane < A.T) mine = ns[sg * W4_SEG + lane] != 0;
    const uint32_t rmask = (uint32_t)__ballot(mine);
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      const int64_t t = sg * W4_SEG + x;
      if (t < A.T) {
        if ((rmask >> x) & 1u) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
        const float ww = pp + w, diff = ww - kc[x];
        const float e = __expf(-fabsf(diff));
        const float e1 = diff >= 0.f ? 1.f : e, e2 = diff >= 0.f ? e : 1.f;
        aa = fmaf(e1, aa, e2 * vc[x]);
        bb = fmaf(e1, bb, e2);
        pp = fmaxf(ww, kc[x]);
      }
    }
  }
}

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_bwd_kernel(Wkv4Args A) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c0 = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  // lanes beyond C redo channel C-1 (same loads, same stores of the same values): every lane stays active for the
  // ballot that gathers a segment's reset flags
  const int64_t c = c0 < A.C ? c0 : A.C - 1;
  const int lane = threadIdx.x;
  const size_t tok0 = (size_t)b * A.T * A.C + c;
  const IO* kp = reinterpret_cast<const IO*>(A.k) + tok0;
  const IO* vp = reinterpret_cast<const IO*>(A.v) + tok0;
  const IO* gyp = reinterpret_cast<const IO*>(A.gy) + tok0;
  IO* gkp = reinterpret_cast<IO*>(A.gk) + tok0;
  IO* gvp = reinterpret_cast<IO*>(A.gv) + tok0;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const int64_t nseg = (A.T + W4_SEG - 1) / W4_SEG;
  const float* ck = A.ckpt + (size_t)b * nseg * 3 * A.C + c;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + c);
  const float u = ld_f(reinterpret_cast<const IO*>(A.u) + c);
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const bool q2drop = (A.flags & 1u) && L < A.T && ns != nullptr && ns[L] != 0;
  float inj_a = 0.f, inj_b = 0.f, inj_p = 0.f;   // cotangent of the returned state
  if (A.gs_new != nullptr && !q2drop) {
    const IO* gp = reinterpret_cast<const IO*>(A.gs_new) + (size_t)b * 3 * A.C + c;
    inj_a = ld_f(gp); inj_b = ld_f(gp + A.C); inj_p = ld_f(gp + 2 * A.C);
  }
  float g_aa = 0.f, g_bb = 0.f, g_pp = 0.f, gw = 0.f, gu = 0.f;
  for (int64_t sg = nseg - 1; sg >= 0; --sg) {
    const int64_t t0 = sg * W4_SEG;
    float kc[W4_SEG], vc[W4_SEG], gc[W4_SEG], sa[W4_SEG], sb[W4_SEG], spp[W4_SEG];
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      const int64_t t = t0 + x;
      const bool in = t < A.T;
      kc[x] = in ? ld_f(kp + (size_t)t * A.C) : 0.f;
      vc[x] = in ? ld_f(vp + (size_t)t * A.C) : 0.f;
      gc[x] = in ? ld_f(gyp + (size_t)t * A.C) : 0.f;
    }
    // one flag per lane, gathered into a uniform mask
    bool mine = false;
    if (ns != nullptr && lane < W4_SEG && t0 + lane < A.T) mine = ns[t0 + lane] != 0;
    const uint32_t rmask = (uint32_t)__ballot(mine);
    float aa = ck[(sg * 3 + 0) * A.C], bb = ck[(sg * 3 + 1) * A.C], pp = ck[(sg * 3 + 2) * A.C];
    // states entering each step of the segment
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      if (rmask & (1ull << x)) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
      sa[x] = aa; sb[x] = bb; spp[x] = pp;
      const float ww = pp + w, diff = ww - kc[x];
      const float e = __expf(-fabsf(diff));
      const float e1 = diff >= 0.f ? 1.f : e, e2 = diff >= 0.f ? e : 1.f;
      aa = fmaf(e1, aa, e2 * vc[x]);
      bb = fmaf(e1, bb, e2);
      pp = fmaxf(ww, kc[x]);
    }
#pragma unroll
    for (int x = W4_SEG - 1; x >= 0; --x) {
      const int64_t t = t0 + x;
      if (t < A.T) {
        if (t == L - 1) { g_aa += inj_a; g_bb += inj_b; g_pp += inj_p; }
        const float a0 = sa[x], b0 = sb[x], p0 = spp[x], kt = kc[x], vt = vc[x], gy = gc[x];
        // state update: aa' = f1 aa + f2 v, bb' = f1 bb + f2, pp' = max(pp + w, k)
        const float ww2 = p0 + w, d2 = ww2 - kt;
        const float ex2 = __expf(-fabsf(d2));
        const bool up2 = d2 >= 0.f;
        const float f1 = up2 ? 1.f : ex2, f2 = up2 ? ex2 : 1.f;
        const float gf1 = (g_aa * a0 + g_bb * b0) * f1, gf2 = (g_aa * vt + g_bb) * f2;
        float n_aa = g_aa * f1, n_bb = g_bb * f1;
        float gv = g_aa * f2;
        const float gq2 = g_pp - gf1 - gf2;
        const float gww2 = gf1 + (up2 ? gq2 : 0.f);
        float gk = gf2 + (up2 ? 0.f : gq2);
        float n_pp = gww2;
        gw += gww2;
        // output: y = (e1 aa + e2 v) / (e1 bb + e2) with q = max(pp, u + k)
        const float ww = u + kt, d1 = p0 - ww;
        const float ex1 = __expf(-fabsf(d1));
        const bool up1 = d1 >= 0.f;
        const float e1 = up1 ? 1.f : ex1, e2 = up1 ? ex1 : 1.f;
        const float An = fmaf(e1, a0, e2 * vt), Bd = fmaf(e1, b0, e2);
        const float rB = __frcp_rn(Bd);
        const float gA = gy * rB, gB = -gy * An * rB * rB;
        const float ge1 = (gA * a0 + gB * b0) * e1, ge2 = (gA * vt + gB) * e2;
        n_aa = fmaf(gA, e1, n_aa);
        n_bb = fmaf(gB, e1, n_bb);
        gv = fmaf(gA, e2, gv);
        const float gq = -ge1 - ge2;
        n_pp += ge1 + (up1 ? gq : 0.f);
        const float gww = ge2 + (up1 ? 0.f : gq);
        gu += gww;
        gk += gww;
        st_f(gkp + (size_t)t * A.C, gk);
        st_f(gvp + (size_t)t * A.C, gv);
        const bool reset = (rmask >> x) & 1u;
        g_aa = reset ? 0.f : n_aa;
        g_bb = reset ? 0.f : n_bb;
        g_pp = reset ? 0.f : n_pp;
      }
    }
  }
  if (L == 0) { g_aa += inj_a; g_bb += inj_b; g_pp += inj_p; }   // the returned state is the input state itself
  IO* gsp = reinterpret_cast<IO*>(A.gs) + (size_t)b * 3 * A.C + c;
  st_f(gsp, g_aa);
  st_f(gsp + A.C, g_bb);
  st_f(gsp + 2 * A.C, g_pp);
  A.gw[(size_t)b * A.C + c] = gw;
  A.gu[(size_t)b * A.C + c] = gu;
}

hipError_t launch_wkv4_bwd(const Wkv4Args& A, hipStream_t stream) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const dim3 grid((unsigned)(A.B * cblocks)), block(W4_THREADS);
  if (A.io_f32) {
    hipLaunchKernelGGL(wkv4_ckpt_kernel<float>, grid, block, 0, stream, A);
    hipLaunchKernelGGL(wkv4_bwd_kernel<float>, grid, block, 0, stream, A);
  } else {
    hipLaunchKernelGGL(wkv4_ckpt_kernel<bf16_t>, grid, block, 0, stream, A);
    hipLaunchKernelGGL(wkv4_bwd_kernel<bf16_t>, grid, block, 0, stream, A);
  }
  return hipGetLastError();
}

hipError_t launch_wkv4_fwd(const Wkv4Args& A, hipStream_t stream) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const dim3 grid((unsigned)(A.B * cblocks)), block(W4_THREADS);
  if (A.io_f32) hipLaunchKernelGGL(wkv4_fwd_kernel<float>, grid, block, 0, stream, A);
  else hipLaunchKernelGGL(wkv4_fwd_kernel<bf16_t>, grid, block, 0, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
