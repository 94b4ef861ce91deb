// WKV4 forward: per-channel max-tracked recurrence, one thread per (sequence, channel).
//
// Reference: BaseRWKV.inner_loop, /root/reference/src/jaxrwkv/rwkv4.py:144-172, in the operand convention of the
// reference's native op (rwkv4.py:311-323): w = -exp(time_decay) is passed in, the receptance is applied outside.
//     ww = u + k_t ; q = max(pp, ww) ; y_t = (e^{pp-q} aa + e^{ww-q} v_t) / (e^{pp-q} bb + e^{ww-q})
//     ww = pp + w  ; q = max(ww, k_t) ; aa = e^{ww-q} aa + e^{k_t-q} v_t ; bb = e^{ww-q} bb + e^{k_t-q} ; pp = q
// In each pair of exponentials one argument is exactly 0, so a step costs two exp, not four.
// k and v are streamed through a rolling register prefetch of TB steps per thread (coalesced across channels): a
// step's two operands are requested TB steps before their use, into the registers the step TB earlier has just
// read, so the requests stay in flight continuously and nothing is copied.  A short distance is the fast one here:
// with one wave per 64 channels the GPU holds 1280 streams of 256-byte pieces 10 KB apart at the benchmark shape,
// and HBM serves that pattern best (5.0 of the 6.0 TB/s a linear stream reaches) with 8-9 rows in flight per
// stream, 8 % better than with 20-32.  A lone wave issues one instruction every ~4.6 cycles whatever its kind, so
// the step is kept short: blocks of TB steps without a reset or the token length-1 skip the per-step checks, the
// reset flags of a block are fetched by one load (a byte per lane, one block ahead) and turned into a uniform
// mask, and the quotient is num * rcp(den) (v_rcp_f32 is good to 1 ulp; the reference divides, the difference is
// ~1e-7 relative).
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

constexpr int W4_THREADS = 64;
constexpr int W4_TB = 8;
constexpr int W4_SEG = 16;                // the backward pass wants the state entering every W4_SEG-th step
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

// this lane's reset flag of the run of tokens that starts at token tb (lane x: token tb + x, clamped into the
// sequence: lanes beyond it re-read its last flag and are masked by the caller); without flags every lane reads a
// byte of `dummy` that is then ignored
__device__ __forceinline__ uint32_t seg_flag(const uint8_t* ns, const void* dummy, int64_t tb, int64_t T, int lane) {
  const int64_t fb = tb < T - 1 ? tb : T - 1;
  const int room = (int)(T - 1 - fb < 63 ? T - 1 - fb : 63);
  const void* base = ns != nullptr ? static_cast<const void*>(ns + fb) : dummy;
  const int off = ns != nullptr ? (lane < room ? lane : room) : 0;
  return __builtin_amdgcn_raw_buffer_load_b8(make_rsrc(base), off, 0, 0);
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
  // k and v of the next W4_TB steps live in registers: register x holds step t0 + x until that step has used it,
  // then step t0 + W4_TB + x is requested into the same register.  2 W4_TB loads stay in flight all the time, a
  // step waits for exactly its own two (the oldest outstanding ones), and nothing is copied between registers.
  // Every block issues the same sequence of requests (flags, then per step: y store, k load, v load), which is
  // what lets the compiler count the requests that may stay outstanding at each wait.  Rows beyond the sequence
  // re-read row T-1 and are never used, so no request needs a predicate.
  float kr[W4_TB], vr[W4_TB];
  uint32_t nsb;                                      // this lane's reset flag of the block after the current one
  auto fetch_flags = [&](int64_t tb) { nsb = seg_flag(ns, kseq, tb, A.T, lane); };
  fetch_flags(0);
  {
    const rsrc_t rk = make_rsrc(kseq), rv = make_rsrc(vseq);
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      const int off = (x < A.T ? x : (int)(A.T - 1)) * stride;
      kr[x] = buf_ld(kseq, rk, voff, off);
      vr[x] = buf_ld(vseq, rv, voff, off);
      __builtin_amdgcn_sched_barrier(0);             // keep the request order of the main loop
    }
  }
  auto general_step = [&](int x, int64_t t, uint64_t rmask, rsrc_t ry, int soff) {
    if (rmask & (1ull << x)) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
    buf_st(yseq, wkv4_step(aa, bb, pp, kr[x], vr[x], w, u), ry, voff, soff);
    if (t == L - 1) snapshot();
  };
  const uint64_t block_lanes = (1ull << W4_TB) - 1ull;
  // with a checkpoint array (a forward pass whose backward will follow) the state entering every W4_SEG-th step is
  // kept, before that step's reset: what the backward's own first pass would recompute from k and v
  static_assert(W4_SEG % W4_TB == 0, "segments start at block starts");
  float* ck = A.ckpt ? A.ckpt + (size_t)b * ((A.T + W4_SEG - 1) / W4_SEG) * 3 * A.C + cc : nullptr;
  auto checkpoint = [&](int64_t t) {
    if (ck != nullptr && t % W4_SEG == 0) {
      const int64_t sg = t / W4_SEG;
      ck[(sg * 3 + 0) * A.C] = aa;
      ck[(sg * 3 + 1) * A.C] = bb;
      ck[(sg * 3 + 2) * A.C] = pp;
    }
  };
  int64_t t0 = 0;
  for (; t0 + W4_TB <= A.T; t0 += W4_TB) {
    checkpoint(t0);
    const uint64_t rmask = ns != nullptr ? (__ballot(nsb != 0) & block_lanes) : 0ull;
    fetch_flags(t0 + W4_TB);
    // descriptors of the block: offsets stay below 2 W4_TB rows whatever the sequence length
    const rsrc_t rk = make_rsrc(kseq + (size_t)t0 * A.C), rv = make_rsrc(vseq + (size_t)t0 * A.C);
    const rsrc_t ry = make_rsrc(yseq + (size_t)t0 * A.C);
    const bool plain = rmask == 0ull && (L - 1 < t0 || L - 1 >= t0 + W4_TB);
    const int64_t rows_left = A.T - 1 - t0;
    const int last_off = (int)(rows_left < 2 * W4_TB ? rows_left : 2 * W4_TB) * stride;
    int soff = 0;
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      if (plain) buf_st(yseq, wkv4_step(aa, bb, pp, kr[x], vr[x], w, u), ry, voff, soff);
      else general_step(x, t0 + x, rmask, ry, soff);
      const int noff = min(soff + W4_TB * stride, last_off);
      kr[x] = buf_ld(kseq, rk, voff, noff);
      vr[x] = buf_ld(vseq, rv, voff, noff);
      soff += stride;
    }
  }
  // the ragged end: fewer than W4_TB tokens, their operands are in the registers already
  if (t0 < A.T) {
    checkpoint(t0);
    const int left = (int)(A.T - t0);
    const uint64_t rmask = ns != nullptr ? (__ballot(nsb != 0) & ((1ull << left) - 1ull)) : 0ull;
    const rsrc_t ry = make_rsrc(yseq + (size_t)t0 * A.C);
    int soff = 0;
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      if (x < left) general_step(x, t0 + x, rmask, ry, soff);
      soff += stride;
    }
  }
}

// ------------------------------------------------------------------ backward
// Reverse-mode derivative of the recurrence above, step by step (so that it agrees with autodiff of the
// reference's scan implementation, including how max() routes its cotangent).  The states entering each step are
// needed in reverse order: a first kernel re-runs the recurrence and keeps the state entering every W4_SEG-th
// step; the second kernel walks the segments backwards, recomputes the W4_SEG states of a segment into registers
// and then differentiates its steps last to first.  Both stream their operands like the forward kernel: every
// segment issues the same sequence of requests, each for a row that is needed a fixed number of steps later.
namespace {

// the flags of a segment as a uniform mask, bit x = token t0 + x (tokens beyond the sequence have none)
__device__ __forceinline__ uint32_t seg_mask(const uint8_t* ns, uint32_t flag, int64_t t0, int64_t T) {
  if (ns == nullptr) return 0u;
  const int64_t left = T - t0;
  const uint32_t lanes = left >= W4_SEG ? (1u << W4_SEG) - 1u : (1u << (int)left) - 1u;
  return (uint32_t)__ballot(flag != 0) & lanes;
}
__device__ __forceinline__ void wkv4_advance(float& aa, float& bb, float& pp, float kt, float vt, float w) {
  const float ww = pp + w, diff = ww - kt;
  const float e = __expf(-fabsf(diff));
  const float e1 = diff >= 0.f ? 1.f : e, e2 = diff >= 0.f ? e : 1.f;
  aa = fmaf(e1, aa, e2 * vt);
  bb = fmaf(e1, bb, e2);
  pp = fmaxf(ww, kt);
}

}  // namespace

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_ckpt_kernel(Wkv4Args A) {
  static_assert(W4_SEG <= 32 && W4_SEG % W4_TB == 0, "a segment is a whole number of prefetch rounds");
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c0 = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  // lanes beyond C redo channel C-1 (same loads, same stores of the same values): every lane stays active for the
  // ballot that gathers a segment's reset flags
  const int64_t c = c0 < A.C ? c0 : A.C - 1;
  const int lane = threadIdx.x;
  const IO* kseq = reinterpret_cast<const IO*>(A.k) + (size_t)b * A.T * A.C;
  const IO* vseq = reinterpret_cast<const IO*>(A.v) + (size_t)b * A.T * A.C;
  const IO* sp = reinterpret_cast<const IO*>(A.s) + (size_t)b * 3 * A.C + c;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const int64_t nseg = (A.T + W4_SEG - 1) / W4_SEG;
  float* ck = A.ckpt + (size_t)b * nseg * 3 * A.C + c;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + c);
  const int voff = (int)(c * sizeof(IO));
  const int stride = (int)(A.C * sizeof(IO));
  float aa = ld_f(sp), bb = ld_f(sp + A.C), pp = ld_f(sp + 2 * A.C);
  // rolling prefetch as in the forward kernel; rows beyond the sequence re-read row T-1, and what the recurrence
  // makes of them is never stored
  float kr[W4_TB], vr[W4_TB];
  uint32_t flag = seg_flag(ns, kseq, 0, A.T, lane);
  {
    const rsrc_t rk = make_rsrc(kseq), rv = make_rsrc(vseq);
#pragma unroll
    for (int x = 0; x < W4_TB; ++x) {
      const int off = (x < A.T ? x : (int)(A.T - 1)) * stride;
      kr[x] = buf_ld(kseq, rk, voff, off);
      vr[x] = buf_ld(vseq, rv, voff, off);
      __builtin_amdgcn_sched_barrier(0);             // keep the request order of the main loop
    }
  }
  for (int64_t sg = 0; sg < nseg; ++sg) {
    const int64_t t0 = sg * W4_SEG;
    ck[(sg * 3 + 0) * A.C] = aa;
    ck[(sg * 3 + 1) * A.C] = bb;
    ck[(sg * 3 + 2) * A.C] = pp;
    const uint32_t rmask = seg_mask(ns, flag, t0, A.T);
    flag = seg_flag(ns, kseq, t0 + W4_SEG, A.T, lane);
    const rsrc_t rk = make_rsrc(kseq + (size_t)t0 * A.C), rv = make_rsrc(vseq + (size_t)t0 * A.C);
    const int64_t rows_left = A.T - 1 - t0;
    const int last_off = (int)(rows_left < 2 * W4_SEG ? rows_left : 2 * W4_SEG) * stride;
    int soff = 0;
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      if ((rmask >> x) & 1u) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
      wkv4_advance(aa, bb, pp, kr[x % W4_TB], vr[x % W4_TB], w);
      const int noff = min(soff + W4_TB * stride, last_off);
      kr[x % W4_TB] = buf_ld(kseq, rk, voff, noff);
      vr[x % W4_TB] = buf_ld(vseq, rv, voff, noff);
      soff += stride;
    }
  }
}

namespace {

// operands of one segment of the reverse pass
struct Seg4 {
  float k[W4_SEG], v[W4_SEG], g[W4_SEG];
  float aa, bb, pp;      // state entering the segment
  uint32_t flag;         // this lane's reset flag
};

}  // namespace

template <typename IO>
__global__ __launch_bounds__(W4_THREADS) void wkv4_bwd_kernel(Wkv4Args A) {
  const int64_t cblocks = (A.C + W4_THREADS - 1) / W4_THREADS;
  const int64_t b = blockIdx.x / cblocks;
  const int64_t c0 = (blockIdx.x % cblocks) * W4_THREADS + threadIdx.x;
  // lanes beyond C redo channel C-1 (same loads, same stores of the same values): every lane stays active for the
  // ballot that gathers a segment's reset flags
  const int64_t c = c0 < A.C ? c0 : A.C - 1;
  const int lane = threadIdx.x;
  const size_t seq0 = (size_t)b * A.T * A.C;
  const IO* kseq = reinterpret_cast<const IO*>(A.k) + seq0;
  const IO* vseq = reinterpret_cast<const IO*>(A.v) + seq0;
  const IO* gyseq = reinterpret_cast<const IO*>(A.gy) + seq0;
  IO* gkseq = reinterpret_cast<IO*>(A.gk) + seq0;
  IO* gvseq = reinterpret_cast<IO*>(A.gv) + seq0;
  const uint8_t* ns = A.ns ? A.ns + (size_t)b * A.T : nullptr;
  const int64_t nseg = (A.T + W4_SEG - 1) / W4_SEG;
  const float* ck = A.ckpt + (size_t)b * nseg * 3 * A.C + c;
  const float w = ld_f(reinterpret_cast<const IO*>(A.w) + c);
  const float u = ld_f(reinterpret_cast<const IO*>(A.u) + c);
  const int voff = (int)(c * sizeof(IO));
  const int stride = (int)(A.C * sizeof(IO));
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const bool q2drop = (A.flags & 1u) && L < A.T && ns != nullptr && ns[L] != 0;
  float inj_a = 0.f, inj_b = 0.f, inj_p = 0.f;   // cotangent of the returned state
  if (A.gs_new != nullptr && !q2drop) {
    const IO* gp = reinterpret_cast<const IO*>(A.gs_new) + (size_t)b * 3 * A.C + c;
    inj_a = ld_f(gp); inj_b = ld_f(gp + A.C); inj_p = ld_f(gp + 2 * A.C);
  }
  float g_aa = 0.f, g_bb = 0.f, g_pp = 0.f, gw = 0.f, gu = 0.f;

  // Requests of segment sg, spread over the steps of the segment handled before it (sg + 1) in the order of their
  // use: flags and state first, k and v of step x during the recomputation of step x, gy of step x during the
  // differentiation of step x.  Rows beyond the sequence re-read row T-1.
  auto row_off = [&](int64_t t0, int x) {
    const int64_t r = A.T - 1 - t0;
    return (int)(x < r ? x : r) * stride;
  };
  auto request_head = [&](Seg4& s, int64_t sg) {
    s.flag = seg_flag(ns, kseq, sg * W4_SEG, A.T, lane);
    s.aa = ck[(sg * 3 + 0) * A.C];
    s.bb = ck[(sg * 3 + 1) * A.C];
    s.pp = ck[(sg * 3 + 2) * A.C];
  };
  // One segment: `cur` holds its operands, `nxt` receives those of segment sg - 1, which is a whole one (when there
  // is none, row 0 is requested instead: never used).
  auto run = [&](Seg4& cur, Seg4& nxt, int64_t sg) {
    const int64_t t0 = sg * W4_SEG;
    const int64_t sn = sg > 0 ? sg - 1 : 0, tn = sn * W4_SEG;
    const int nstride = sg > 0 ? stride : 0;
    const uint32_t rmask = seg_mask(ns, cur.flag, t0, A.T);
    request_head(nxt, sn);
    const rsrc_t rk = make_rsrc(kseq + (size_t)tn * A.C), rv = make_rsrc(vseq + (size_t)tn * A.C);
    const rsrc_t rg = make_rsrc(gyseq + (size_t)tn * A.C);
    const rsrc_t rgk = make_rsrc(gkseq + (size_t)t0 * A.C), rgv = make_rsrc(gvseq + (size_t)t0 * A.C);
    float sa[W4_SEG], sb[W4_SEG], spp[W4_SEG];
    float aa = cur.aa, bb = cur.bb, pp = cur.pp;
    int noff = 0;
    // states entering each step of the segment
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      if ((rmask >> x) & 1u) { aa = 0.f; bb = 0.f; pp = W4_RESET_PP; }
      sa[x] = aa; sb[x] = bb; spp[x] = pp;
      wkv4_advance(aa, bb, pp, cur.k[x], cur.v[x], w);
      nxt.k[x] = buf_ld(kseq, rk, voff, noff);
      nxt.v[x] = buf_ld(vseq, rv, voff, noff);
      noff += nstride;
    }
    int soff = W4_SEG * stride;
#pragma unroll
    for (int x = W4_SEG - 1; x >= 0; --x) {
      noff -= nstride;
      soff -= stride;
      const int64_t t = t0 + x;
      if (t < A.T) {
        if (t == L - 1) { g_aa += inj_a; g_bb += inj_b; g_pp += inj_p; }
        const float a0 = sa[x], b0 = sb[x], p0 = spp[x], kt = cur.k[x], vt = cur.v[x], gy = cur.g[x];
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
        buf_st(gkseq, gk, rgk, voff, soff);
        buf_st(gvseq, gv, rgv, voff, soff);
        const bool reset = (rmask >> x) & 1u;
        g_aa = reset ? 0.f : n_aa;
        g_bb = reset ? 0.f : n_bb;
        g_pp = reset ? 0.f : n_pp;
      }
      nxt.g[x] = buf_ld(gyseq, rg, voff, noff);
    }
  };

  Seg4 s0, s1;
  {
    // operands of the last segment, in the request order of `run`
    const int64_t sg = nseg - 1, t0 = sg * W4_SEG;
    request_head(s0, sg);
    const rsrc_t rk = make_rsrc(kseq + (size_t)t0 * A.C), rv = make_rsrc(vseq + (size_t)t0 * A.C);
    const rsrc_t rg = make_rsrc(gyseq + (size_t)t0 * A.C);
#pragma unroll
    for (int x = 0; x < W4_SEG; ++x) {
      s0.k[x] = buf_ld(kseq, rk, voff, row_off(t0, x));
      s0.v[x] = buf_ld(vseq, rv, voff, row_off(t0, x));
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int x = W4_SEG - 1; x >= 0; --x) {
      s0.g[x] = buf_ld(gyseq, rg, voff, row_off(t0, x));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (int64_t sg = nseg - 1; sg >= 0; sg -= 2) {
    run(s0, s1, sg);
    if (sg >= 1) run(s1, s0, sg - 1);
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
  const bool have_ckpt = (A.flags & FLAG_CKPT_READY) != 0;   // written by the forward pass of the same inputs
  if (A.io_f32) {
    if (!have_ckpt) hipLaunchKernelGGL(wkv4_ckpt_kernel<float>, grid, block, 0, stream, A);
    hipLaunchKernelGGL(wkv4_bwd_kernel<float>, grid, block, 0, stream, A);
  } else {
    if (!have_ckpt) hipLaunchKernelGGL(wkv4_ckpt_kernel<bf16_t>, grid, block, 0, stream, A);
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
