// WKV7 sequential kernels (fp32 VALU, one token per step): forward and the three backward sweeps.
//
// Recurrence (reference: BaseRWKV.inner_loop, /root/reference/src/jaxrwkv/rwkv7.py:200-220), per head,
// S[i][j] = value row i, key column j, d_t = exp(-exp(w_t)):
//     S' = new_starts[t] ? 0 : S ;  sa = S' a_t ;  S = S' diag(d_t) + v_t k_t^T + sa b_t^T ;  y_t = S r_t
//
// Backward (G = dL/dS, carried from t = T-1 down):
//     G += dy_t r_t^T (+ dS_out at t = length-1)
//     dv_t = G k_t, dk_t = G^T v_t, db_t = G^T sa_t, dsa = G b_t, da_t = S'^T dsa, dr_t = S_t^T dy_t
//     G = (G diag(d_t) + dsa a_t^T) * !new_starts[t]
// The decay gradient needs <G_t, S'_t> per key column; instead of keeping states it uses
//     dl_t = D_t - k_t.dk_t - b_t.db_t,   D_t = sum_i G_t[i][:] S_t[i][:],
//     D_{t-1} = (new_starts[t] ? 0 : dl_t + a_t.da_t) + r_{t-1}.dr_{t-1} (+ <dS_out, S_{length-1}> at t-1 = length-1)
// (. = elementwise), dw_t = dl_t * (-exp(w_t)).  Three sweeps, each a 64x64 fp32 recurrence of the same shape
// as the forward one:
//     sweep A (reverse, G by rows)     -> gv, dsa, gs
//     sweep B (forward, S by columns)  -> gr, ga, e2 = a.da, e3 = r.dr (+ <dS_out,S> term)
//     sweep C (reverse, G by columns)  -> gk, gb, gw (runs the D recursion)
#include "seq_skel.h"
#include "wkv_args.h"

namespace hiprwkv {

__device__ __forceinline__ float ld_state(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}
__device__ __forceinline__ void st_state(void* p, int f32, size_t off, float x) {
  if (f32) reinterpret_cast<float*>(p)[off] = x;
  else reinterpret_cast<uint16_t*>(p)[off] = f32_to_bf16(x);
}

struct SeqIds {
  int64_t b, h;
  int line, q;   // state line (row or column) and 16-element quarter owned by this thread
  int64_t L;     // min(length, T)
  bool compat;
  bool q2drop;   // compat && L < T && new_starts[L]: returned state is the reset state
};

__device__ __forceinline__ SeqIds seq_ids(const Wkv7Args& A) {
  SeqIds id;
  id.b = blockIdx.x / A.H;
  id.h = blockIdx.x % A.H;
  id.line = threadIdx.x >> 2;
  id.q = threadIdx.x & 3;
  int64_t L = A.length ? (int64_t)A.length[id.b] : A.T;
  id.L = L < A.T ? L : A.T;
  id.compat = (A.flags & 1u) != 0;
  id.q2drop = id.compat && id.L < A.T && A.ns != nullptr && A.ns[id.b * A.T + id.L] != 0;
  return id;
}

// ------------------------------------------------------------------ forward
constexpr int FWD_CH = 32;
struct FwdStep {
  float S[16];
  SeqIds id;
  const Wkv7Args* A;

  __device__ __forceinline__ void snapshot() {
    const size_t base = (((size_t)id.b * A->H + id.h) * N64 + id.line) * N64 + id.q * 16;
#pragma unroll
    for (int c = 0; c < 16; ++c) st_state(A->new_s, A->st_f32, base + c, id.q2drop ? 0.f : S[c]);
  }
  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[FWD_CH][N64], float (*sout)[FWD_CH][N64],
                                       const uint8_t* sns) {
    float d[16], r[16], k[16], a[16], b[16];
    const int c0 = id.q * 16;
    lds16(&sin[4][tl][c0], a);
    lds16(&sin[0][tl][c0], d);
    lds16(&sin[2][tl][c0], k);
    lds16(&sin[5][tl][c0], b);
    lds16(&sin[1][tl][c0], r);
    const float vi = sin[3][tl][id.line];
    if (sns[tl]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; c += 2) { p0 = fmaf(S[c], a[c], p0); p1 = fmaf(S[c + 1], a[c + 1], p1); }
    const float sa = quad_sum(p0 + p1);
    float y0 = 0.f, y1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; c += 2) {
      S[c] = fmaf(S[c], d[c], fmaf(sa, b[c], vi * k[c]));
      S[c + 1] = fmaf(S[c + 1], d[c + 1], fmaf(sa, b[c + 1], vi * k[c + 1]));
      y0 = fmaf(S[c], r[c], y0);
      y1 = fmaf(S[c + 1], r[c + 1], y1);
    }
    const float y = quad_sum(y0 + y1);
    if (id.q == 0) {
      sout[0][tl][id.line] = y;
      sout[1][tl][id.line] = sa;
    }
    if (t == id.L - 1) snapshot();
  }
  __device__ __forceinline__ void post(int o, int tl, int64_t t, float (&vals)[8], const uint8_t* sns) {
    // y[t] = 0 where the associative form zeroes scan element t+1 (rwkv7.py:331-333,344)
    if (o == 0 && id.compat && sns[tl + 1]) {
#pragma unroll
      for (int e = 0; e < 8; ++e) vals[e] = 0.f;
    }
  }
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv7_seq_fwd_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) float smem[];
  FwdStep st;
  st.id = seq_ids(A);
  st.A = &A;
  const size_t base = (((size_t)st.id.b * A.H + st.id.h) * N64 + st.id.line) * N64 + st.id.q * 16;
#pragma unroll
  for (int c = 0; c < 16; ++c) st.S[c] = ld_state(A.s, A.st_f32, base + c);
  if (st.id.L == 0) st.snapshot();  // rwkv7.py:203 (out_s starts as s); zero under compat if new_starts[0]
  const int io = A.io_f32;
  VecIn in[6] = {{A.w, io, VK_EXPNEGEXP}, {A.r, io, VK_ID}, {A.k, io, VK_ID},
                 {A.v, io, VK_ID},        {A.a, io, VK_ID}, {A.b, io, VK_ID}};
  VecOut out[2] = {{A.out, io}, {A.sa, io ? 1 : 2}};
  seq_run<6, 2, FWD_CH, false>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
}

// ------------------------------------------------------------------ backward sweep A: G by rows (reverse)
// inputs: 0 d, 1 r, 2 k, 3 a, 4 b, 5 gy ; outputs: 0 gv, 1 dsa
constexpr int BWA_CH = 32;
struct BwdAStep {
  float G[16];
  SeqIds id;
  const Wkv7Args* A;

  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[BWA_CH][N64], float (*sout)[BWA_CH][N64],
                                       const uint8_t* sns) {
    float d[16], r[16], k[16], a[16], b[16];
    const int c0 = id.q * 16;
    lds16(&sin[1][tl][c0], r);
    lds16(&sin[2][tl][c0], k);
    lds16(&sin[4][tl][c0], b);
    lds16(&sin[0][tl][c0], d);
    lds16(&sin[3][tl][c0], a);
    float dyi = sin[5][tl][id.line];
    if (id.compat && sns[tl + 1]) dyi = 0.f;  // y[t] is the constant 0 there
    if (t == id.L - 1 && A->gs_out != nullptr && !id.q2drop) {
      const size_t base = (((size_t)id.b * A->H + id.h) * N64 + id.line) * N64 + c0;
#pragma unroll
      for (int c = 0; c < 16; ++c) G[c] += ld_state(A->gs_out, A->st_f32, base + c);
    }
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      G[c] = fmaf(dyi, r[c], G[c]);
      p0 = fmaf(G[c], k[c], p0);
      p1 = fmaf(G[c], b[c], p1);
    }
    const float dv = quad_sum(p0);
    const float dsa = quad_sum(p1);
    const bool reset = sns[tl] != 0;
#pragma unroll
    for (int c = 0; c < 16; ++c) G[c] = reset ? 0.f : fmaf(G[c], d[c], dsa * a[c]);
    if (id.q == 0) {
      sout[0][tl][id.line] = dv;
      sout[1][tl][id.line] = dsa;
    }
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv7_seq_bwd_a_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) float smem[];
  BwdAStep st;
  st.id = seq_ids(A);
  st.A = &A;
#pragma unroll
  for (int c = 0; c < 16; ++c) st.G[c] = 0.f;
  const int io = A.io_f32;
  VecIn in[6] = {{A.w, io, VK_EXPNEGEXP}, {A.r, io, VK_ID}, {A.k, io, VK_ID},
                 {A.a, io, VK_ID},        {A.b, io, VK_ID}, {A.gy, io, VK_ID}};
  VecOut out[2] = {{A.gv, io}, {A.dsa, 1}};
  seq_run<6, 2, BWA_CH, true>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
  // cotangent of the input state; with length == 0 the returned state is s itself
  const size_t base = (((size_t)st.id.b * A.H + st.id.h) * N64 + st.id.line) * N64 + st.id.q * 16;
  const bool pass = st.id.L == 0 && A.gs_out != nullptr && !st.id.q2drop;
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    float g = st.G[c];
    if (pass) g += ld_state(A.gs_out, A.st_f32, base + c);
    st_state(A.gs, A.st_f32, base + c, g);
  }
}

// ------------------------------------------------------------------ backward sweep B: S by columns (forward)
// thread owns column j = line, rows i = 16q..16q+15
// inputs: 0 d, 1 r, 2 k, 3 v, 4 a, 5 b, 6 gy, 7 sa, 8 dsa ; outputs: 0 gr, 1 ga, 2 e2, 3 e3
constexpr int BWB_CH = 16;
struct BwdBStep {
  float S[16];
  SeqIds id;
  const Wkv7Args* A;

  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[BWB_CH][N64], float (*sout)[BWB_CH][N64],
                                       const uint8_t* sns) {
    float v[16], sa[16], dsa[16], dy[16];
    const int r0 = id.q * 16, j = id.line;
    lds16(&sin[8][tl][r0], dsa);
    lds16(&sin[3][tl][r0], v);
    lds16(&sin[7][tl][r0], sa);
    lds16(&sin[6][tl][r0], dy);
    const float dj = sin[0][tl][j], rj = sin[1][tl][j], kj = sin[2][tl][j], aj = sin[4][tl][j], bj = sin[5][tl][j];
    if (sns[tl]) {
#pragma unroll
      for (int c = 0; c < 16; ++c) S[c] = 0.f;
    }
    const bool dropy = id.compat && sns[tl + 1];
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      p0 = fmaf(S[c], dsa[c], p0);                       // da_j = sum_i S'[i][j] dsa_i
      S[c] = fmaf(S[c], dj, fmaf(sa[c], bj, v[c] * kj));
      p1 = fmaf(S[c], dy[c], p1);                        // dr_j = sum_i S[i][j] dy_i
    }
    const float da = quad_sum(p0);
    float dr = quad_sum(p1);
    if (dropy) dr = 0.f;
    float inj = 0.f;
    if (t == id.L - 1 && A->gs_out != nullptr && !id.q2drop) {
      const size_t base = ((size_t)id.b * A->H + id.h) * N64 * N64;
      float p = 0.f;
#pragma unroll
      for (int c = 0; c < 16; ++c) p = fmaf(ld_state(A->gs_out, A->st_f32, base + (size_t)(r0 + c) * N64 + j), S[c], p);
      inj = quad_sum(p);
    }
    if (id.q == 0) {
      sout[0][tl][j] = dr;
      sout[1][tl][j] = da;
      sout[2][tl][j] = aj * da;
      sout[3][tl][j] = rj * dr + inj;
    }
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv7_seq_bwd_b_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) float smem[];
  BwdBStep st;
  st.id = seq_ids(A);
  st.A = &A;
  const size_t base = ((size_t)st.id.b * A.H + st.id.h) * N64 * N64;
#pragma unroll
  for (int c = 0; c < 16; ++c) st.S[c] = ld_state(A.s, A.st_f32, base + (size_t)(st.id.q * 16 + c) * N64 + st.id.line);
  const int io = A.io_f32;
  VecIn in[9] = {{A.w, io, VK_EXPNEGEXP}, {A.r, io, VK_ID}, {A.k, io, VK_ID}, {A.v, io, VK_ID}, {A.a, io, VK_ID},
                 {A.b, io, VK_ID},        {A.gy, io, VK_ID}, {A.sa_in, io ? 1 : 2, VK_ID}, {A.dsa, 1, VK_ID}};
  VecOut out[4] = {{A.gr, io}, {A.ga, io}, {A.e2, 1}, {A.e3, 1}};
  seq_run<9, 4, BWB_CH, false>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
}

// ------------------------------------------------------------------ backward sweep C: G by columns (reverse)
// inputs: 0 d, 1 -exp(w), 2 r, 3 k, 4 v, 5 a, 6 b, 7 gy, 8 sa, 9 dsa, 10 e2, 11 e3 ; outputs: 0 gk, 1 gb, 2 gw
constexpr int BWC_CH = 16;
struct BwdCStep {
  float G[16];
  float carry;  // (new_starts[t+1] ? 0 : dl_{t+1} + a.da_{t+1}), meaningful in the q == 0 lane copy too
  SeqIds id;
  const Wkv7Args* A;

  __device__ __forceinline__ void step(int tl, int64_t t, float (*sin)[BWC_CH][N64], float (*sout)[BWC_CH][N64],
                                       const uint8_t* sns) {
    float v[16], sa[16], dsa[16], dy[16];
    const int r0 = id.q * 16, j = id.line;
    lds16(&sin[7][tl][r0], dy);
    lds16(&sin[4][tl][r0], v);
    lds16(&sin[8][tl][r0], sa);
    lds16(&sin[9][tl][r0], dsa);
    const float dj = sin[0][tl][j], nej = sin[1][tl][j], rj = sin[2][tl][j], kj = sin[3][tl][j];
    const float aj = sin[5][tl][j], bj = sin[6][tl][j], e2 = sin[10][tl][j], e3 = sin[11][tl][j];
    const bool dropy = id.compat && sns[tl + 1];
    const float rje = dropy ? 0.f : rj;
    if (t == id.L - 1 && A->gs_out != nullptr && !id.q2drop) {
      const size_t base = ((size_t)id.b * A->H + id.h) * N64 * N64;
#pragma unroll
      for (int c = 0; c < 16; ++c) G[c] += ld_state(A->gs_out, A->st_f32, base + (size_t)(r0 + c) * N64 + j);
    }
    float p0 = 0.f, p1 = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      G[c] = fmaf(dy[c], rje, G[c]);
      p0 = fmaf(G[c], v[c], p0);    // dk_j = sum_i G[i][j] v_i
      p1 = fmaf(G[c], sa[c], p1);   // db_j = sum_i G[i][j] sa_i
    }
    const float dk = quad_sum(p0);
    const float db = quad_sum(p1);
    const bool reset = sns[tl] != 0;
#pragma unroll
    for (int c = 0; c < 16; ++c) G[c] = reset ? 0.f : fmaf(G[c], dj, dsa[c] * aj);
    const float D = carry + e3;
    // a reset step has S' = 0, hence no decay gradient and nothing carried further back
    const float dl = reset ? 0.f : D - kj * dk - bj * db;
    carry = reset ? 0.f : dl + e2;
    if (id.q == 0) {
      sout[0][tl][j] = dk;
      sout[1][tl][j] = db;
      sout[2][tl][j] = dl * nej;
    }
  }
  __device__ __forceinline__ void post(int, int, int64_t, float (&)[8], const uint8_t*) {}
};

__global__ __launch_bounds__(SEQ_THREADS) void wkv7_seq_bwd_c_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) float smem[];
  BwdCStep st;
  st.id = seq_ids(A);
  st.A = &A;
  st.carry = 0.f;
#pragma unroll
  for (int c = 0; c < 16; ++c) st.G[c] = 0.f;
  const int io = A.io_f32;
  VecIn in[12] = {{A.w, io, VK_EXPNEGEXP}, {A.w, io, VK_NEGEXP}, {A.r, io, VK_ID},    {A.k, io, VK_ID},
                  {A.v, io, VK_ID},        {A.a, io, VK_ID},     {A.b, io, VK_ID},    {A.gy, io, VK_ID},
                  {A.sa_in, io ? 1 : 2, VK_ID},     {A.dsa, 1, VK_ID},    {A.e2, 1, VK_ID},    {A.e3, 1, VK_ID}};
  VecOut out[3] = {{A.gk, io}, {A.gb, io}, {A.gw, io}};
  seq_run<12, 3, BWC_CH, true>(st, in, out, st.id.b, st.id.h, A.T, A.H, A.ns ? A.ns + st.id.b * A.T : nullptr, smem);
}

// ------------------------------------------------------------------ host launchers
hipError_t launch_wkv7_seq_fwd(const Wkv7Args& A, hipStream_t stream) {
  constexpr size_t smem = seq_smem_bytes<6, 2, FWD_CH>();
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_seq_fwd_kernel), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv7_seq_fwd_kernel, dim3((unsigned)(A.B * A.H)), dim3(SEQ_THREADS), smem, stream, A);
  return hipGetLastError();
}

// The three backward sweeps, in the order they must run (A, B, C).
hipError_t launch_wkv7_seq_bwd_a(const Wkv7Args& A, hipStream_t stream) {
  constexpr size_t smem = seq_smem_bytes<6, 2, BWA_CH>();
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_seq_bwd_a_kernel), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv7_seq_bwd_a_kernel, dim3((unsigned)(A.B * A.H)), dim3(SEQ_THREADS), smem, stream, A);
  return hipGetLastError();
}

hipError_t launch_wkv7_seq_bwd_b(const Wkv7Args& A, hipStream_t stream) {
  constexpr size_t smem = seq_smem_bytes<9, 4, BWB_CH>();
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_seq_bwd_b_kernel), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv7_seq_bwd_b_kernel, dim3((unsigned)(A.B * A.H)), dim3(SEQ_THREADS), smem, stream, A);
  return hipGetLastError();
}

hipError_t launch_wkv7_seq_bwd_c(const Wkv7Args& A, hipStream_t stream) {
  constexpr size_t smem = seq_smem_bytes<12, 3, BWC_CH>();
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_seq_bwd_c_kernel), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv7_seq_bwd_c_kernel, dim3((unsigned)(A.B * A.H)), dim3(SEQ_THREADS), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
