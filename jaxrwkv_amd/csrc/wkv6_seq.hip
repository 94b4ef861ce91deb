// WKV6 sequential kernels (fp32 VALU, one token per step): forward and the two backward sweeps.
//
// Recurrence (reference: BaseRWKV.inner_loop, /root/reference/src/jaxrwkv/rwkv6.py:175-191), per head,
// S[i][j] = key row i, value column j, dec_t = exp(w_t) with w the log decay:
//     S' = new_starts[t] ? 0 : S ;  y_t[j] = sum_i r_i (u_i k_i v_j + S'[i][j]) ;  S = diag(dec_t) S' + k_t v_t^T
//
// Backward (G = dL/dS carried from t = T-1 down, c_t = v_t . dy_t):
//     G += dS_out at t = length-1
//     dk_t[i] = r_i u_i c_t + sum_j G[i][j] v_j        dv_t[j] = dy_j sum_i r_i u_i k_i + sum_i G[i][j] k_i
//     dr_t[i] = u_i k_i c_t + sum_j S'[i][j] dy_j       du[i]  += r_i k_i c_t
//     G = (diag(dec_t) G + r_t dy_t^T) * !new_starts[t]
// The decay gradient dw_t[i] = dec_t[i] <G_t[i][:], S'_t[i][:]> is obtained without stored states from
//     dw_t = D_t - k_t . (G_t v_t),  D_t = rowsum(G_t * S_t),
//     D_{t-1} = (new_starts[t] ? 0 : dw_t + r_t . (S'_t dy_t)) (+ rowsum(dS_out * S_{length-1}) at t-1 = length-1)
//     sweep F (forward, S by rows)                  -> gr, gu, er = r . (S' dy), eI = rowsum(dS_out * S_{length-1})
//     sweep R (reverse, G by rows and by columns)   -> gk, gv, gw, gs
#include "seq_skel.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

__device__ __forceinline__ float ld_state6(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}
__device__ __forceinline__ void st_state6(void* p, int f32, size_t off, float x) {
  if (f32) reinterpret_cast<float*>(p)[off] = x;
  else reinterpret_cast<uint16_t*>(p)[off] = f32_to_bf16(x);
}

struct Ids6 {
  int64_t b, h;
  int line, q;
  int64_t L;
  bool q2drop;
};

__device__ __forceinline__ Ids6 ids6(const Wkv6Args& A) {
  Ids6 id;
  id.b = blockIdx.x / A.H;
  id.h = blockIdx.x % A.H;
  id.line = threadIdx.x >> 2;
  id.q = threadIdx.x & 3;
  int64_t L = A.length ? (int64_t)A.length[id.b] : A.T;
  id.L = L < A.T ? L : A.T;
  id.q2drop = (A.flags & 1u) && id.L < A.T && A.ns != nullptr && A.ns[id.b * A.T + id.L] != 0;
  return id;
}

__device__ __forceinline__ float ld_u(const Wkv6Args& A, int64_t h, int i) {
  const size_t off = (size_t)h * N64 + i;
  return A.io_f32 ? reinterpret_cast<const float*>(A.u)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(A.u)[off]);
}

}  // namespace

// ------------------------------------------------------------------ forward: S by columns
// thread owns value column j = line, key rows i = 16q..16q+15.  inputs: 0 r, 1 k, 2 v, 3 dec ; outputs: 0 y
constexpr int F6_CH = 32;
struct Fwd6Step {
  float S[16], u[16];
  Ids6 id;
  const Wkv6Args* A;

  __device__ __forceinline__ void snapshot() {
    const size_t base = ((size_t)id.b * A->H + id.h) * N64 * N64;
#pragma unroll
    for (int c = 0; c < 16; ++c)
      st_state6(A->new_s, A->st_f32, base + (size_t)(id.q * 16 + c) * N64 + id.line, id.q2drop ? 0.f : S[c]);
  }
  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[F6_CH][N64], float (*sout)[F6_CH][N64],
                                       const uint8_t* sns) {
    float r[16], k[16], dec[16];
    const int r0 = id.q * 16;
    lds16(&sin[0][tl][r0], r);
    lds16(&sin[1][tl][r0], k);
    lds16(&sin[3][tl][r0], dec);
    const float vj = sin[2][tl][id.line];
    if (sns[tl]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    float y0 = 0.f, y1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; c += 2) {
      const float kv0 = k[c] * vj, kv1 = k[c + 1] * vj;
      y0 = fmaf(r[c], fmaf(u[c], kv0, S[c]), y0);
      y1 = fmaf(r[c + 1], fmaf(u[c + 1], kv1, S[c + 1]), y1);
      S[c] = fmaf(dec[c], S[c], kv0);
      S[c + 1] = fmaf(dec[c + 1], S[c + 1], kv1);
    }
    const float y = quad_sum(y0 + y1);
    if (id.q == 0) sout[0][tl][id.line] = y;
    if (t == id.L - 1) snapshot();
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv6_seq_fwd_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) float smem[];
  Fwd6Step st;
  st.id = ids6(A);
  st.A = &A;
  const size_t base = ((size_t)st.id.b * A.H + st.id.h) * N64 * N64;
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    st.S[c] = ld_state6(A.s, A.st_f32, base + (size_t)(st.id.q * 16 + c) * N64 + st.id.line);
    st.u[c] = ld_u(A, st.id.h, st.id.q * 16 + c);
  }
  if (st.id.L == 0) st.snapshot();
  const int io = A.io_f32;
  VecIn in[4] = {{A.r, io, VK_ID}, {A.k, io, VK_ID}, {A.v, io, VK_ID}, {A.w, io, VK_EXP, (int)((A.flags & FLAG_W_PER_HEAD) != 0)}};
  VecOut out[1] = {{A.out, io}};
  seq_run<4, 1, F6_CH, false>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
}

// ------------------------------------------------------------------ backward sweep F: S by rows (forward)
// thread owns key row i = line, value columns j = 16q..16q+15.  inputs: 0 r, 1 k, 2 v, 3 dec, 4 gy ; outputs: 0 gr, 1 er
constexpr int BF6_CH = 32;
struct BwdF6Step {
  float S[16];
  float ui, du;
  Ids6 id;
  const Wkv6Args* A;

  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[BF6_CH][N64], float (*sout)[BF6_CH][N64],
                                       const uint8_t* sns) {
    float v[16], dy[16];
    const int c0 = id.q * 16, i = id.line;
    lds16(&sin[2][tl][c0], v);
    lds16(&sin[4][tl][c0], dy);
    const float ri = sin[0][tl][i], ki = sin[1][tl][i], deci = sin[3][tl][i];
    if (sns[tl]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      p0 = fmaf(v[c], dy[c], p0);
      p1 = fmaf(S[c], dy[c], p1);
      S[c] = fmaf(deci, S[c], ki * v[c]);
    }
    const float cdy = quad_sum(p0);
    const float sdy = quad_sum(p1);
    du = fmaf(ri * ki, cdy, du);
    if (id.q == 0) {
      sout[0][tl][i] = fmaf(ui * ki, cdy, sdy);
      sout[1][tl][i] = ri * sdy;
    }
    if (t == id.L - 1 && A->gs_out != nullptr) {
      float p = 0.f;
      if (!id.q2drop) {
        const size_t base = (((size_t)id.b * A->H + id.h) * N64 + i) * N64 + c0;
#pragma unroll
        for (int c = 0; c < 16; ++c) p = fmaf(ld_state6(A->gs_out, A->st_f32, base + c), S[c], p);
      }
      p = quad_sum(p);
      if (id.q == 0) A->eI[((size_t)id.b * A->H + id.h) * N64 + i] = p;
    }
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv6_seq_bwd_f_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) float smem[];
  BwdF6Step st;
  st.id = ids6(A);
  st.A = &A;
  st.du = 0.f;
  st.ui = ld_u(A, st.id.h, st.id.line);
  const size_t base = (((size_t)st.id.b * A.H + st.id.h) * N64 + st.id.line) * N64 + st.id.q * 16;
#pragma unroll
  for (int c = 0; c < 16; ++c) st.S[c] = ld_state6(A.s, A.st_f32, base + c);
  const int io = A.io_f32;
  VecIn in[5] = {{A.r, io, VK_ID}, {A.k, io, VK_ID}, {A.v, io, VK_ID}, {A.w, io, VK_EXP, (int)((A.flags & FLAG_W_PER_HEAD) != 0)}, {A.gy, io, VK_ID}};
  VecOut out[2] = {{A.gr, io}, {A.er, 1}};
  seq_run<5, 2, BF6_CH, false>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
  if (st.id.q == 0) A.gu[((size_t)st.id.b * A.H + st.id.h) * N64 + st.id.line] = st.du;
}

// ------------------------------------------------------------------ backward sweep R: G by rows and by columns (reverse)
// Grow[c] = G[line][16q+c], Gcol[c] = G[16q+c][line].  inputs: 0 r, 1 k, 2 v, 3 dec, 4 gy, 5 er ; outputs: 0 gk, 1 gv, 2 gw
constexpr int BR6_CH = 32;
struct BwdR6Step {
  float Grow[16], Gcol[16], uq[16];
  float ui, carry;
  Ids6 id;
  const Wkv6Args* A;

  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[BR6_CH][N64], float (*sout)[BR6_CH][N64],
                                       const uint8_t* sns) {
    float r[16], k[16], v[16], dec[16], dy[16];
    const int c0 = id.q * 16, l = id.line;
    lds16(&sin[0][tl][c0], r);
    lds16(&sin[1][tl][c0], k);
    lds16(&sin[2][tl][c0], v);
    lds16(&sin[3][tl][c0], dec);
    lds16(&sin[4][tl][c0], dy);
    const float rl = sin[0][tl][l], kl = sin[1][tl][l], decl = sin[3][tl][l], dyl = sin[4][tl][l], erl = sin[5][tl][l];
    float eI = 0.f;
    if (t == id.L - 1 && A->gs_out != nullptr && !id.q2drop) {
      const size_t base = ((size_t)id.b * A->H + id.h) * N64 * N64;
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        Grow[c] += ld_state6(A->gs_out, A->st_f32, base + (size_t)l * N64 + c0 + c);
        Gcol[c] += ld_state6(A->gs_out, A->st_f32, base + (size_t)(c0 + c) * N64 + l);
      }
      eI = A->eI[((size_t)id.b * A->H + id.h) * N64 + l];
    }
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      p0 = fmaf(v[c], dy[c], p0);              // c_t = v . dy
      p1 = fmaf(Grow[c], v[c], p1);            // sum_j G[l][j] v_j
      p2 = fmaf(r[c] * uq[c], k[c], p2);       // sum_i r_i u_i k_i
      p3 = fmaf(Gcol[c], k[c], p3);            // sum_i G[i][l] k_i
    }
    const float cdy = quad_sum(p0), gv_ = quad_sum(p1), ruk = quad_sum(p2), gk_ = quad_sum(p3);
    const bool reset = sns[tl] != 0;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      Grow[c] = reset ? 0.f : fmaf(decl, Grow[c], rl * dy[c]);
      Gcol[c] = reset ? 0.f : fmaf(dec[c], Gcol[c], r[c] * dyl);
    }
    const float D = carry + eI;
    const float dl = reset ? 0.f : D - kl * gv_;
    carry = reset ? 0.f : dl + erl;
    if (id.q == 0) {
      sout[0][tl][l] = fmaf(rl * ui, cdy, gv_);   // dk_l
      sout[1][tl][l] = fmaf(dyl, ruk, gk_);       // dv_l
      sout[2][tl][l] = dl;                        // dw_l
    }
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv6_seq_bwd_r_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) float smem[];
  BwdR6Step st;
  st.id = ids6(A);
  st.A = &A;
  st.carry = 0.f;
  st.ui = ld_u(A, st.id.h, st.id.line);
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    st.Grow[c] = 0.f;
    st.Gcol[c] = 0.f;
    st.uq[c] = ld_u(A, st.id.h, st.id.q * 16 + c);
  }
  const int io = A.io_f32;
  VecIn in[6] = {{A.r, io, VK_ID}, {A.k, io, VK_ID}, {A.v, io, VK_ID}, {A.w, io, VK_EXP, (int)((A.flags & FLAG_W_PER_HEAD) != 0)}, {A.gy, io, VK_ID}, {A.er, 1, VK_ID}};
  VecOut out[3] = {{A.gk, io}, {A.gv, io}, {A.gw, io}};
  seq_run<6, 3, BR6_CH, true>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
  const size_t base = (((size_t)st.id.b * A.H + st.id.h) * N64 + st.id.line) * N64 + st.id.q * 16;
  const bool pass = st.id.L == 0 && A.gs_out != nullptr && !st.id.q2drop;
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    float g = st.Grow[c];
    if (pass) g += ld_state6(A.gs_out, A.st_f32, base + c);
    st_state6(A.gs, A.st_f32, base + c, g);
  }
}

// ------------------------------------------------------------------ host launchers
hipError_t launch_wkv6_seq_fwd(const Wkv6Args& A, hipStream_t stream) {
  constexpr size_t smem = seq_smem_bytes<4, 1, F6_CH>();
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_seq_fwd_kernel), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv6_seq_fwd_kernel, dim3((unsigned)(A.B * A.H)), dim3(SEQ_THREADS), smem, stream, A);
  return hipGetLastError();
}

hipError_t launch_wkv6_seq_bwd(const Wkv6Args& A, hipStream_t stream) {
  constexpr size_t sf = seq_smem_bytes<5, 2, BF6_CH>();
  constexpr size_t sr = seq_smem_bytes<6, 3, BR6_CH>();
  static LdsAttrOnce once_f, once_r;
  hipError_t e;
  if ((e = allow_dynamic_lds(once_f, reinterpret_cast<const void*>(wkv6_seq_bwd_f_kernel), sf)) != hipSuccess) return e;
  if ((e = allow_dynamic_lds(once_r, reinterpret_cast<const void*>(wkv6_seq_bwd_r_kernel), sr)) != hipSuccess) return e;
  const dim3 grid((unsigned)(A.B * A.H)), block(SEQ_THREADS);
  hipLaunchKernelGGL(wkv6_seq_bwd_f_kernel, grid, block, sf, stream, A);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  hipLaunchKernelGGL(wkv6_seq_bwd_r_kernel, grid, block, sr, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
