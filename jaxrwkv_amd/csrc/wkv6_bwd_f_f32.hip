// WKV6 backward for fp32 I/O on gfx950, forward sweep F on the matrix cores with fp32 operands
// (v_mfma_f32_16x16x4_f32): gr, gu and the workspaces er = r.(S' dy) and eI = rowsum(dS_out * S_{length-1}) that the
// decay-gradient recursion of the reverse sweep consumes.
//
// State recurrence (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191), S[i][j] = key row i, value col j:
//     S' = new_starts[t] ? 0 : S ;  S = diag(dec_t) S' + k_t v_t^T ,  dec_t = exp(w_t)
//     dr_t[i] = u_i k_i c_t + sum_j S'_t[i][j] dy_j ,  c_t = v_t.dy_t ;   du[i] = sum_t r_i k_i c_t
// A chunk of 16 tokens entering with S0: E_t = prod_{s<=t} dec_s, Ee_t = E_{t-1}, kh_s = k_s/E_s,
//     S' dy_t = Ee_t . ( S0 dy_t + sum_{s<t} (v_s.dy_t) kh_s )        S_C = diag(E_C) (S0 + Kh^T V)
// The Gram tile N[s][t] = v_s.dy_t contracts over the values; its diagonal is c_t.  This is the algebra of the bf16
// sweep (wkv6_chunk_bwd_f.hip) with every product on the fp32 matrix instruction; operand layouts as in
// wkv6_fwd_f32.hip.  One consumer and one producer wave per SIMD: consumer q holds the state rows of keys 16q..16q+15
// (36 matrix instructions per chunk), producer p prepares chunks p, p+4, ... (16 matrix instructions) and owns the
// terms that need no state: u k c_t (handed over as an add-on) and du (summed per producer, combined at the end).
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight (a slot is 27 KB)
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

struct __attribute__((aligned(16))) Slot {
  float DY[CK][RF];            // dy rows [token][value]; rows the entering state does not reach are zero
  float KH[CK][RF];            // k_s/E_s rows [token][key]
  float V[CK][RF];             // v rows, tokens masked for the chunk-end state
  float Ee[CK][RF];            // decay from the chunk start to just before token t, per key
  float UKC[CK][RF];           // u k_t c_t per key
  float R[CK][RF];             // r rows as loaded
  f32x4_t N[64];               // Gram tile v_s.dy_t (s < t), accumulator layout [row s][column t], lane-indexed
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to token length-1
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {
  float V[CK][RF];             // v rows with the tokens masked for the state at token length-1
  float gamma[64];
};
struct __attribute__((aligned(16))) Tail {
  float du[NPROD][64];         // per-producer partial sums of du
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and, of every 64-vector, the elements 16j + 4g + i (j, i = 0..3).
struct Raw {
  float4 r[4], k[4], v[4], w[4], dy[4];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;   // always a valid token; mask_raw zeroes the lanes beyond
  const size_t off = (((size_t)b * A.T + tok) * A.H + h) * 64 + 4 * g;
  auto ld = [&](const void* p, size_t o, float4 (&d)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + o + 16 * j);
  };
  ld(A.r, off, x.r); ld(A.k, off, x.k); ld(A.v, off, x.v); ld(A.gy, off, x.dy);
  // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
  ld(A.w, (A.flags & FLAG_W_PER_HEAD) ? (size_t)h * 64 + 4 * g : off, x.w);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) x.r[j] = x.k[j] = x.v[j] = x.w[j] = x.dy[j] = z;
    }
  }
}
__device__ __forceinline__ void unpack2(const float4 p, const float4 q, float (&o)[8]) {
  o[0] = p.x; o[1] = p.y; o[2] = p.z; o[3] = p.w;
  o[4] = q.x; o[5] = q.y; o[6] = q.z; o[7] = q.w;
}
__device__ __forceinline__ void put2(float* row, int hf, int g, const float (&f)[8], bool keep) {
  const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
  *reinterpret_cast<float4*>(row + 32 * hf + 4 * g) = keep ? make_float4(f[0], f[1], f[2], f[3]) : z;
  *reinterpret_cast<float4*>(row + 32 * hf + 16 + 4 * g) = keep ? make_float4(f[4], f[5], f[6], f[7]) : z;
}

struct Producer {
  int lane;
  float4 u[4];         // bonus of this lane's keys
  float du[16];        // running sum over this producer's tokens of r k c_t, for this lane's token and keys
};

__device__ __forceinline__ void produce(Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint32_t resets = F.ns & 0xffffu;
  const bool slow = resets != 0;                  // a reset inside this chunk
  int lastseg = 0, seg_src = 0;
  bool s0_reaches = true, restart = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(resets, 15);
    s0_reaches = seg_of(resets, t) == 0;                            // the entering state reaches this token
    keep_upd = 0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u);   // tokens from the last reset on
    const uint32_t upto = resets & ((2u << t) - 1u);
    const int pr = upto ? 31 - __builtin_clz(upto) : 0;             // last reset at or before this token
    restart = pr > 0;
    seg_src = (lane & 48) | (pr > 0 ? pr - 1 : 0);
    if (F.snap >= 0) {
      const uint32_t us = resets & keep_snap;
      if (us) keep_snap &= ~((1u << (31 - __builtin_clz(us))) - 1u);
    }
  }

  f32x4_t N = zero4;   // [row s][column t] = v_s . dy_t
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ================= keys of this half: decay scan, k/E rows, Ee rows, r rows
    {
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain: every step is split into a part on a
    //      2^-16 grid, whose running sums are exact, and a remainder below 2^-17, summed separately
    float E[8], El[8];
    {
      float fw[8];
      unpack2(x.w[2 * hf], x.w[2 * hf + 1], fw);
#pragma unroll
      for (int e = 0; e < 8; ++e) fw[e] = fmaxf(fw[e] * LOG2E, MIN_STEP_L2);
      if (F.nvalid != CK) {
        rare_path();
#pragma unroll
        for (int e = 0; e < 8; ++e) fw[e] = valid ? fw[e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float hi = (fw[e] + GRID_MAGIC) - GRID_MAGIC;
        E[e] = row_scan(hi);
        El[e] = row_scan(fw[e] - hi);
      }
      // near the decay floor the split no longer matters: fold it before the floor is applied
      const float lo = fminf(fminf(fminf(E[0], E[1]), fminf(E[2], E[3])), fminf(fminf(E[4], E[5]), fminf(E[6], E[7])));
      if (__ballot(lo < MIN_CUM_L2 + 1.f) != 0ull) {
        rare_path();
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          E[e] += El[e];
          El[e] = 0.f;
        }
        cap_chunk_decay(E, lane, events);
      }
    }
    if (slow) {
      rare_path();
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
        const float basel = __shfl(El[e], seg_src, 64);
        if (restart) {
          E[e] -= base;
          El[e] -= basel;
        }
      }
    }
      float fkh[8], Ee[8];
      {
        float fk[8];
        unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
          const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
          E[e] = exp2_fast(l2) * fl;
          fkh[e] = fk[e] * (exp2_fast(-l2) * (2.f - fl));
          // value of the previous token; 1 for the first token.  At a reset token it belongs to the previous
          // segment, but it then multiplies an exact zero (no state reaches that token).
          Ee[e] = row_prev(E[e], 1.0f);
        }
      }
      put2(slot->Ee[t], hf, g, Ee, true);
      if (t == 15) {
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      if (F.snap >= 0 && t == F.snap) {
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      put2(slot->KH[t], hf, g, fkh, true);
      float fr[8];
      unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
      put2(slot->R[t], hf, g, fr, true);
    }
    // ================= values of this half: v and dy rows, partial Gram sum
    {
      float fv[8], fdy[8];
      unpack2(x.v[2 * hf], x.v[2 * hf + 1], fv);
      unpack2(x.dy[2 * hf], x.dy[2 * hf + 1], fdy);
      put2(slot->DY[t], hf, g, fdy, s0_reaches);
      put2(slot->V[t], hf, g, fv, (keep_upd >> t) & 1u);
      if (F.snap >= 0) {
        rare_path();
        put2(snap->V[t], hf, g, fv, (keep_snap >> t) & 1u);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) N = mfma_f(fv[e], fdy[e], N);
    }
  }
  // ---- c_t = v_t.dy_t is the diagonal of N: held by lane group t/4, register t%4; hand it to all four groups
  const int n = t;
  float c_t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) c_t = (4 * g + i == n) ? N[i] : c_t;
  c_t += __shfl_xor(c_t, 16, 64);
  c_t += __shfl_xor(c_t, 32, 64);
  // ---- u k c_t for the consumers, r k c_t for du
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    float fr[8], fk[8], fu[8], o[8];
    unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
    unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
    unpack2(P.u[2 * hf], P.u[2 * hf + 1], fu);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float kc = fk[e] * c_t;
      o[e] = fu[e] * kc;
      P.du[8 * hf + e] = fmaf(fr[e], kc, P.du[8 * hf + e]);
    }
    put2(slot->UKC[t], hf, g, o, true);
  }
  // ---- strictly lower triangle within a segment
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool lt = m < n;
    if (slow) lt = lt && seg_of(resets, m) == seg_of(resets, n);
    N[i] = lt ? N[i] : 0.f;
  }
  slot->N[lane] = N;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state rows of keys 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16, g = lane/16),
// S[vt][i] = S[key 16q + n][value 16*vt + 4g + i]: register i of a tile is the B operand of the instruction that
// contracts over the values 16*vt + 4g' + i (g' = 0..3).
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

struct OutCursor {
  float* gr;           // output at (b, c0, h, 0)
  float* er;           // fp32 workspace at the same place
  size_t tok;          // elements between consecutive tokens
  uint32_t voff;       // lane part of the address: (4g * H) * 64 + key
};

__device__ __forceinline__ size_t state_el(const Wkv6Args& A, int64_t b, int64_t h, int key, int value) {
  return (((size_t)b * A.H + h) * 64 + key) * 64 + value;
}
__device__ __forceinline__ f32x4_t load_state4(const void* p, int f32, size_t off) {
  f32x4_t r;
  if (f32) {
    const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + off);
    r[0] = x.x; r[1] = x.y; r[2] = x.z; r[3] = x.w;
  } else {
    const uint2 x = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p) + off);
    r[0] = __uint_as_float(x.x << 16); r[1] = __uint_as_float(x.x & 0xffff0000u);
    r[2] = __uint_as_float(x.y << 16); r[3] = __uint_as_float(x.y & 0xffff0000u);
  }
  return r;
}

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, OutCursor& oc) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // B operand of the token contractions: k/E of tokens 4g..4g+3 at this wave's keys
  float tk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) tk[i] = slot->KH[4 * g + i][16 * q + n];
  const bool keep_end = slot->keep_end != 0;
  f32x4_t P = zero4, P2 = zero4;   // [token 4g+i][key n], two accumulation chains joined at the end
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const float4 d4 = *reinterpret_cast<const float4*>(&slot->DY[n][16 * vt + 4 * g]);
    const float dy[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (vt & 1) P2 = mfma_f(dy[i], C.S[vt][i], P2);
      else P = mfma_f(dy[i], C.S[vt][i], P);
    }
  }
  {
    const f32x4_t nt = slot->N[lane];
#pragma unroll
    for (int i = 0; i < 4; ++i) P2 = mfma_f(nt[i], tk[i], P2);
  }
  // A operands of the state update: v of tokens 4g..4g+3 at value 16*vt + n
  float vv[4][4];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt)
#pragma unroll
    for (int i = 0; i < 4; ++i) vv[vt][i] = slot->V[4 * g + i][16 * vt + n];
  // rowsum(dS_out * S_{length-1}) per key (one chunk per sequence)
  if (is_snap) {
    rare_path();
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
    float p = 0.f;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      f32x4_t acc = keep ? C.S[vt] : zero4;
#pragma unroll
      for (int i = 0; i < 4; ++i) acc = mfma_f(snapslot->V[4 * g + i][16 * vt + n], tk[i], acc);
      const f32x4_t gs = load_state4(A.gs_out, A.st_f32, state_el(A, b, h, 16 * q + n, 16 * vt + 4 * g));
#pragma unroll
      for (int i = 0; i < 4; ++i) p = fmaf(gs[i], acc[i] * sg, p);
    }
    p += __shfl_xor(p, 16, 64);
    p += __shfl_xor(p, 32, 64);
    if (g == 0) A.eI[((size_t)b * A.H + h) * 64 + 16 * q + n] = p;
  }
  // state update: S <- diag(gamma) (S + Kh^T V), gamma per key = per lane; the four value tiles take turns
  if (!keep_end) {
    rare_path();
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = zero4;   // a reset inside the chunk cuts the entering state off
  }
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = mfma_f(vv[vt][i], tk[i], C.S[vt]);
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) { C.S[vt][0] *= gm; C.S[vt][1] *= gm; C.S[vt][2] *= gm; C.S[vt][3] *= gm; }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive keys
  float ogr[4], oer[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    const float sdy = (P[i] + P2[i]) * slot->Ee[tok][16 * q + n];
    ogr[i] = slot->UKC[tok][16 * q + n] + sdy;
    oer[i] = slot->R[tok][16 * q + n] * sdy;
  }
  float* const gl = oc.gr + oc.voff;
  float* const el = oc.er + oc.voff;
  if (nvalid == CK) {      // every chunk but a partial last one: no per-lane predicates
#pragma unroll
    for (int i = 0; i < 4; ++i) gl[i * oc.tok] = ogr[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) el[i * oc.tok] = oer[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        gl[i * oc.tok] = ogr[i];
        el[i * oc.tok] = oer[i];
      }
    }
  }
  oc.gr += CK * oc.tok;
  oc.er += CK * oc.tok;
}

}  // namespace

__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv6_bwd_f_f32_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Tail* tail = reinterpret_cast<Tail*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Tail));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int nch = (int)((A.T + CK - 1) / CK);
  const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
  const bool inject = A.gs_out != nullptr && !q2drop;   // a cotangent of the returned state exists
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  if (wave < NCONS) {                 // waves 0..3: one consumer per SIMD; waves 4..7: one producer per SIMD
    __builtin_amdgcn_s_setprio(3);    // the chunk-to-chunk dependency runs through the consumers
    Consumer C;
    C.q = wave;
    C.lane = lane;
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = load_state4(A.s, A.st_f32, state_el(A, b, h, 16 * wave + n, 16 * vt + 4 * g));
    OutCursor oc;
    oc.tok = (size_t)A.H * 64;
    const size_t el0 = (((size_t)b * A.T) * A.H + h) * 64;
    oc.gr = reinterpret_cast<float*>(A.gr) + el0;
    oc.er = A.er + el0;
    oc.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    for (int c = 0; c < nch; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING;
      if (!wait_ready(sy, si, c + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, oc);
      // every LDS read of slot si has returned: its data went into the matrix instructions and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    {
      const float* up = reinterpret_cast<const float*>(A.u) + (size_t)h * 64 + 4 * (lane >> 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) P.u[j] = *reinterpret_cast<const float4*>(up + 16 * j);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) P.du[e] = 0.f;
    Raw raw;
    uint32_t ns_mine = 0u;      // this lane's new_starts byte of the chunk loaded next: fetched a step ahead, like the operands
    if (p < nch) {
      ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)p * CK, lane);
      load_raw(raw, A, b, h, (int64_t)p * CK, lane);
    }
    for (int c = p; c < nch; c += NPROD) {
      const int64_t c0 = (int64_t)c * CK;
      ChunkFlags F = chunk_flags_of(A.ns, ns_mine, A.flags, A.T, c0, L);
      if (!inject) F.snap = -1;
      const int si = c % RING;
      if (c >= RING && !wait_consumed_lazy(sy, si, c - RING + 1, lane)) break;
      mask_raw(raw, F.nvalid, lane);
      produce(P, raw, F, &slots[si], snapslot, events_word(A.status));
      if (c + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, c0 + (int64_t)NPROD * CK, lane);
        load_raw(raw, A, b, h, c0 + (int64_t)NPROD * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && c + 1 == nch) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
    // du of this producer's tokens: sum over the 16 token lanes of a row, one writer per key (element e of the half hf
    // is key 32 hf + 4g + e for e < 4 and 32 hf + 16 + 4g + e - 4 otherwise)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float s = row_scan(P.du[e]);                 // lane 15 of each row holds the row total
      const int key = 32 * (e >> 3) + 16 * ((e >> 2) & 1) + 4 * (lane >> 4) + (e & 3);
      if ((lane & 15) == 15) tail->du[p][key] = s;
    }
  }
  __syncthreads();   // every wave gets here: all loops above are bounded
  if (threadIdx.x < 64) {
    float s = 0.f;
#pragma unroll
    for (int p = 0; p < NPROD; ++p) s += tail->du[p][threadIdx.x];
    A.gu[((size_t)b * A.H + h) * 64 + threadIdx.x] = s;
  }
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gr, 4, b, h, A.T, A.H);
    poison_token_rows(A.er, 4, b, h, A.T, A.H);
    if (threadIdx.x < 64) A.gu[((size_t)b * A.H + h) * 64 + threadIdx.x] = __uint_as_float(0x7fc00000u);
  }
}

hipError_t launch_wkv6_chunk_bwd_f_f32(const Wkv6Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Tail) + sizeof(Sync);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Tail) + sizeof(Sync) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_bwd_f_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_bwd_f_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
