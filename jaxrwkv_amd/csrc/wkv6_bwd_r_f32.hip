// WKV6 backward for fp32 I/O on gfx950, reverse sweep R on the matrix cores with fp32 operands
// (v_mfma_f32_16x16x4_f32): gk, gv, gw, gs.
//
// With G_t the cotangent of the state after token t (reference recurrence: /root/reference/src/jaxrwkv/rwkv6.py:175-191;
// S[i][j] = key row i, value col j; dec_t = exp(w_t)), carried from the last token down:
//     G_t = dec_{t+1} G_{t+1} + r_{t+1} dy_{t+1}^T (+ dS_out at t = length-1),  cut at new_starts
//     dk_t = r_t u c_t + G_t v_t ,  c_t = v_t.dy_t          dv_t = dy_t (r_t.(u k_t)) + G_t^T k_t
//     dw_t = carry_t - er_t ,  carry_t = reset_t ? 0 : carry_{t+1} + er_t (+ eI at t = length-1) - k_t.(G_t v_t)
// (er, eI from the forward sweep).  A chunk of 16 tokens leaving with G_C: E_t = prod_{s<=t} dec_s, Ee_t = E_{t-1},
// rq_s = r_s.Ee_s, kh_t = k_t/E_t, Gh = diag(E_C) G_C:
//     G_t v_t   = (1/E_t) . ( Gh v_t + sum_{s>t} (dy_s.v_t) rq_s )          contracts over values
//     G_t^T k_t = Gh^T kh_t + sum_{s>t} (rq_s.kh_t) dy_s                     contracts over keys
//     G_prev = Gh + sum_s rq_s dy_s^T
// This is the algebra of the bf16 sweep (wkv6_chunk_bwd_r.hip) with every product on the fp32 matrix instruction;
// operand layouts as in wkv6_fwd_f32.hip.  The two contractions run over different axes of G, so every consumer wave
// keeps two copies of its share: the rows of its 16 keys (all values, for G v) and the columns of its 16 values (all
// keys, for G^T k); both get the same rank-16 update (72 matrix instructions per consumer and chunk, 32 per producer).
// One consumer and one producer wave per SIMD; the producers also own the state-free terms r u c_t and dy (r.(u k)),
// handed over as add-ons.  Chunks are handled from the last one down.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns steps p, p + NPROD, ...
constexpr int RING = 4;           // slots in flight (a slot is 33 KB)
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

struct __attribute__((aligned(16))) Slot {
  float V[CK][RF];             // v rows [token][value]; zero where the cotangent of later chunks does not reach
  float KH[CK][RF];            // k_t/E_t rows [token][key], masked likewise
  float RQ[CK][RF];            // r_s.Ee_s rows [token][key]
  float DY[CK][RF];            // dy rows [token][value]
  float Einv[CK][RF];          // 1/E_t per key
  float RUC[CK][RF];           // r_t u c_t per key
  float DYR[CK][RF];           // dy_t (r_t.(u k_t)) per value
  f32x4_t N1[64];              // dy_s.v_t (s > t), accumulator layout [row s][column t], lane-indexed
  f32x4_t N2[64];              // rq_s.kh_t (s > t)
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the cotangent of later chunks reaches the chunk start (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int resets;                  // bit t: new_starts of in-chunk token t
};
struct __attribute__((aligned(16))) SnapSlot {   // row operands masked to the tokens the cotangent entering at length-1 reaches
  float V[CK][RF];
  float KH[CK][RF];
  float gamma[64];
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
};

__device__ __forceinline__ void produce(const Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint32_t resets = F.ns & 0xffffu;
  const bool slow = resets != 0;                  // a reset inside this chunk
  int lastseg = 0, seg_src = 0;
  bool row_keep = true, restart = false;
  uint32_t keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(resets, 15);
    row_keep = seg_of(resets, t) == lastseg;                        // the cotangent of later chunks reaches this token
    const uint32_t upto = resets & ((2u << t) - 1u);
    const int pr = upto ? 31 - __builtin_clz(upto) : 0;             // last reset at or before this token
    restart = pr > 0;
    seg_src = (lane & 48) | (pr > 0 ? pr - 1 : 0);
    if (F.snap >= 0) {
      const uint32_t us = resets & keep_snap;
      if (us) keep_snap &= ~((1u << (31 - __builtin_clz(us))) - 1u);   // tokens of length-1's segment up to it
    }
  }
  const bool snap_keep = (keep_snap >> t) & 1u;

  f32x4_t N1 = zero4, N2 = zero4;   // [row s][column t]: dy_s.v_t and rq_s.kh_t
  float ruk = 0.f;                  // partial r.(u k) over this lane's keys
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ================= keys of this half: decay scan, r.Ee, k/E and 1/E rows
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
      float frq[8], fkh[8], Einv[8];
      {
        float fr[8], fk[8], fu[8];
        unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
        unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
        unpack2(P.u[2 * hf], P.u[2 * hf + 1], fu);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
          const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
          E[e] = exp2_fast(l2) * fl;
          Einv[e] = exp2_fast(-l2) * (2.f - fl);
          // r times the decay up to the previous token (1 for the first token).  At a reset token that value belongs to
          // the previous segment, but every product rq enters for that token is masked out.
          frq[e] = fr[e] * row_prev(E[e], 1.0f);
          fkh[e] = fk[e] * Einv[e];
          ruk = fmaf(fr[e] * fu[e], fk[e], ruk);
        }
      }
      put2(slot->Einv[t], hf, g, Einv, true);
      if (t == 15) {
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      if (F.snap >= 0 && t == F.snap) {
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      put2(slot->KH[t], hf, g, fkh, row_keep);
      put2(slot->RQ[t], hf, g, frq, true);
      if (F.snap >= 0) {
        rare_path();
        put2(snap->KH[t], hf, g, fkh, snap_keep);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) N2 = mfma_f(frq[e], fkh[e], N2);     // [s][t] = rq_s . kh_t
    }
    // ================= values of this half: v and dy rows, partial Gram sum
    {
      float fv[8], fdy[8];
      unpack2(x.v[2 * hf], x.v[2 * hf + 1], fv);
      unpack2(x.dy[2 * hf], x.dy[2 * hf + 1], fdy);
      put2(slot->V[t], hf, g, fv, row_keep);
      put2(slot->DY[t], hf, g, fdy, true);
      if (F.snap >= 0) {
        rare_path();
        put2(snap->V[t], hf, g, fv, snap_keep);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) N1 = mfma_f(fdy[e], fv[e], N1);      // [s][t] = dy_s . v_t
    }
  }
  // ---- c_t = v_t.dy_t is the diagonal of N1 (lane group t/4, register t%4); r.(u k) summed over the key groups
  const int n = t;
  float c_t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) c_t = (4 * g + i == n) ? N1[i] : c_t;
  c_t += __shfl_xor(c_t, 16, 64);
  c_t += __shfl_xor(c_t, 32, 64);
  ruk += __shfl_xor(ruk, 16, 64);
  ruk += __shfl_xor(ruk, 32, 64);
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    float fr[8], fu[8], fd[8], o1[8], o2[8];
    unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
    unpack2(P.u[2 * hf], P.u[2 * hf + 1], fu);
    unpack2(x.dy[2 * hf], x.dy[2 * hf + 1], fd);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      o1[e] = fr[e] * fu[e] * c_t;
      o2[e] = fd[e] * ruk;
    }
    put2(slot->RUC[t], hf, g, o1, true);
    put2(slot->DYR[t], hf, g, o2, true);
  }
  // ---- strictly upper part (s > t) within a segment
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool gt = m > n;
    if (slow) gt = gt && seg_of(resets, m) == seg_of(resets, n);
    N1[i] = gt ? N1[i] : 0.f;
    N2[i] = gt ? N2[i] : 0.f;
  }
  slot->N1[lane] = N1;
  slot->N2[lane] = N2;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
    slot->resets = (int)resets;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q keeps two copies of its share of G as 16x16 accumulator tiles, lane (n = lane%16, g = lane/16):
//   G1[vt][i] = G[key 16q + n][value 16*vt + 4g + i]   rows of its keys: B operand of contractions over values
//               (gk, gw and the cotangent of the input state)
//   G2[kt][i] = G[key 16*kt + 4g + i][value 16q + n]   columns of its values: B operand of contractions over keys (gv)
struct Consumer {
  f32x4_t G1[4], G2[4];
  float carry;         // running sum of the decay-gradient recursion, per key (same in a key's four lanes)
  float er[4], kk[4];  // er and k at this lane's four (token, key) pairs of the chunk handled next, fetched a chunk ahead
  int q, lane;
};

struct Cursor {
  float *gk, *gv, *gw;         // outputs at (b, c0, h, 0)
  size_t tok;                  // elements between consecutive tokens
  uint32_t voff;               // lane part of the address: (4g * H) * 64 + 16q + n
};

// er and k at (tokens c0 + 4g .. + 3, key 16q + n); tokens beyond the sequence read the last one (their results are
// never stored, and their share of the running sum is masked)
__device__ __forceinline__ void fetch_scalars(Consumer& C, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0) {
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t tok = c0 + 4 * g + i;
    tok = tok < A.T ? tok : A.T - 1;
    const size_t el = (((size_t)b * A.T + tok) * A.H + h) * 64 + 16 * C.q + n;
    C.er[i] = A.er[el];
    C.kk[i] = reinterpret_cast<const float*>(A.k)[el];
  }
}

__device__ __forceinline__ size_t state_el(const Wkv6Args& A, int64_t b, int64_t h, int key, int value) {
  return (((size_t)b * A.H + h) * 64 + key) * 64 + value;
}
__device__ __forceinline__ float ld_state_el(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
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
                                        const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool last,
                                        int64_t next_c0, Cursor& cu) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // this chunk's per-token scalars were requested a chunk ago; request the next ones
  float er[4] = {C.er[0], C.er[1], C.er[2], C.er[3]};
  const float kk[4] = {C.kk[0], C.kk[1], C.kk[2], C.kk[3]};
  if (!last) fetch_scalars(C, A, b, h, next_c0);
  // B operands of the token contractions: rq at this wave's keys, dy at this wave's values, tokens 4g..4g+3
  float rq1[4], dyq[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    rq1[i] = slot->RQ[4 * g + i][16 * q + n];
    dyq[i] = slot->DY[4 * g + i][16 * q + n];
  }
  const bool keep_end = slot->keep_end != 0;
  const uint32_t resets = (uint32_t)slot->resets;
  // the cotangent of the chunk-end state, decayed over the chunk: per key = per lane in G1, per register in G2
  {
    const float gm = slot->gamma[16 * q + n];
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) { C.G1[vt][0] *= gm; C.G1[vt][1] *= gm; C.G1[vt][2] *= gm; C.G1[vt][3] *= gm; }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const float4 g4 = *reinterpret_cast<const float4*>(&slot->gamma[16 * kt + 4 * g]);
      C.G2[kt][0] *= g4.x; C.G2[kt][1] *= g4.y; C.G2[kt][2] *= g4.z; C.G2[kt][3] *= g4.w;
    }
  }
  f32x4_t PK = zero4, PV = zero4;   // E_t (G_t v_t) at [token 4g+i][key 16q+n]; G_t^T k_t at [token 4g+i][value 16q+n]
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const float4 v4 = *reinterpret_cast<const float4*>(&slot->V[n][16 * x + 4 * g]);
    const float4 k4 = *reinterpret_cast<const float4*>(&slot->KH[n][16 * x + 4 * g]);
    const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, kh[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      PK = mfma_f(vv[i], C.G1[x][i], PK);
      PV = mfma_f(kh[i], C.G2[x][i], PV);
    }
  }
  {
    const f32x4_t n1 = slot->N1[lane], n2 = slot->N2[lane];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      PK = mfma_f(n1[i], rq1[i], PK);
      PV = mfma_f(n2[i], dyq[i], PV);
    }
  }
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
    rare_path();
#pragma unroll
    for (int x = 0; x < 4; ++x) C.G1[x] = C.G2[x] = zero4;
  }
  // the cotangent of the returned state enters at token length-1 (one chunk per sequence)
  float eI = 0.f;
  int snap_tok = -1;
  if (is_snap) {
    rare_path();
    snap_tok = slot->snap;
    eI = A.eI[((size_t)b * A.H + h) * 64 + 16 * q + n];
    const bool keep = slot->keep_snap != 0;
    const float sg1 = snapslot->gamma[16 * q + n];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const f32x4_t T1 = load_state4(A.gs_out, A.st_f32, state_el(A, b, h, 16 * q + n, 16 * x + 4 * g)) * sg1;
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * x + 4 * g]);
      const float s4[4] = {sg.x, sg.y, sg.z, sg.w};
      f32x4_t T2;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        T2[i] = ld_state_el(A.gs_out, A.st_f32, state_el(A, b, h, 16 * x + 4 * g + i, 16 * q + n)) * s4[i];
      if (keep) {
        C.G1[x] += T1;
        C.G2[x] += T2;
      }
      const float4 v4 = *reinterpret_cast<const float4*>(&snapslot->V[n][16 * x + 4 * g]);
      const float4 k4 = *reinterpret_cast<const float4*>(&snapslot->KH[n][16 * x + 4 * g]);
      const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, kh[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        PK = mfma_f(vv[i], T1[i], PK);
        PV = mfma_f(kh[i], T2[i], PV);
      }
    }
  }
  // cotangent update: G <- Gh + sum_s rq_s dy_s^T over the tokens before the first reset
  {
    float keepf[4] = {1.f, 1.f, 1.f, 1.f};
    if (resets != 0) {
      rare_path();
      const uint32_t keep_upd = (1u << __builtin_ctz(resets)) - 1u;
#pragma unroll
      for (int i = 0; i < 4; ++i) keepf[i] = ((keep_upd >> (4 * g + i)) & 1u) ? 1.f : 0.f;
    }
    float dyu[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) dyu[i] = dyq[i] * keepf[i];
    float da[4][4], ra[4][4];
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        da[x][i] = slot->DY[4 * g + i][16 * x + n] * keepf[i];     // rows = values of tile x
        ra[x][i] = slot->RQ[4 * g + i][16 * x + n];                // rows = keys of tile x
      }
    // the tiles take turns, so that no instruction accumulates on the result of the one before it
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int x = 0; x < 4; ++x) C.G1[x] = mfma_f(da[x][i], rq1[i], C.G1[x]);
#pragma unroll
      for (int x = 0; x < 4; ++x) C.G2[x] = mfma_f(ra[x][i], dyu[i], C.G2[x]);
    }
  }
  // per-token results: register i is token 4g+i, lanes n = 16 consecutive keys (gk, gw) or values (gv)
  float gvk[4], z[4], cy[4];
  if (nvalid != CK) {         // entries of tokens beyond the sequence hold nothing meaningful
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) er[i] = (4 * g + i < nvalid) ? er[i] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    gvk[i] = PK[i] * slot->Einv[tok][16 * q + n];                     // (G_t v_t)[key]
    z[i] = er[i] + (tok == snap_tok ? eI : 0.f) - kk[i] * gvk[i];
  }
  // carry_t = reset_t ? 0 : carry_{t+1} + z_t, from token 15 down
  if (resets == 0) {
    const float s3 = z[3], s2 = z[2] + s3, s1 = z[1] + s2, s0 = z[0] + s1;
    const float t1 = __shfl_down(s0, 16, 64), t2 = __shfl_down(s0, 32, 64), t3 = __shfl_down(s0, 48, 64);
    const float after = C.carry + (g < 3 ? t1 : 0.f) + (g < 2 ? t2 : 0.f) + (g < 1 ? t3 : 0.f);
    cy[3] = s3 + after; cy[2] = s2 + after; cy[1] = s1 + after; cy[0] = s0 + after;
    C.carry = __shfl(cy[0], n, 64);
  } else {
    rare_path();
    float cin = C.carry;
#pragma unroll
    for (int tok = 15; tok >= 0; --tok) {
      const float zv = __shfl(z[tok & 3], n + 16 * (tok >> 2), 64);
      cin = ((resets >> tok) & 1u) ? 0.f : cin + zv;
      if (g == (tok >> 2)) cy[tok & 3] = cin;
    }
    C.carry = cin;
  }
  float ok[4], ow[4], ov[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    ok[i] = slot->RUC[tok][16 * q + n] + gvk[i];
    ow[i] = ((resets >> tok) & 1u) ? 0.f : cy[i] - er[i];
    ov[i] = slot->DYR[tok][16 * q + n] + PV[i];
  }
  float* const kl = cu.gk + cu.voff;
  float* const wl = cu.gw + cu.voff;
  float* const vl = cu.gv + cu.voff;
  if (nvalid == CK) {      // every chunk but a partial last one: no per-lane predicates
#pragma unroll
    for (int i = 0; i < 4; ++i) kl[i * cu.tok] = ok[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) wl[i * cu.tok] = ow[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) vl[i * cu.tok] = ov[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        kl[i * cu.tok] = ok[i];
        wl[i * cu.tok] = ow[i];
        vl[i * cu.tok] = ov[i];
      }
    }
  }
  const size_t d = CK * cu.tok;
  cu.gk -= d; cu.gv -= d; cu.gw -= d;
}

}  // namespace

// Step j handles chunk nch-1-j in slot j % RING.  Producer p fills the slot once every consumer has released step
// j - RING, then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier
// step, so the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv6_bwd_r_f32_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
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
    C.carry = 0.f;
    const int n = lane & 15, g = lane >> 4;
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 4; ++x) C.G1[x] = C.G2[x] = zero4;
#pragma unroll
    for (int i = 0; i < 4; ++i) C.er[i] = C.kk[i] = 0.f;
    Cursor cu;
    cu.tok = (size_t)A.H * 64;
    const size_t el0 = (((size_t)b * A.T + (size_t)(nch - 1) * CK) * A.H + h) * 64;
    cu.gk = reinterpret_cast<float*>(A.gk) + el0;
    cu.gv = reinterpret_cast<float*>(A.gv) + el0;
    cu.gw = reinterpret_cast<float*>(A.gw) + el0;
    cu.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    const int tail = (A.T % CK == 0) ? CK : (int)(A.T % CK);
    if (nch > 0) fetch_scalars(C, A, b, h, (int64_t)(nch - 1) * CK);
    for (int j = 0; j < nch; ++j) {
      const int c = nch - 1 - j;
      const int nvalid = (j == 0) ? tail : CK;
      const int si = j % RING;
      if (!wait_ready(sy, si, j + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, j + 1 == nch, (int64_t)(c - 1) * CK, cu);
      // every LDS read of slot si has returned: its data went into the matrix instructions and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // cotangent of the input state; with length == 0 the returned state is the input state itself
    const bool pass = L == 0 && inject;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      const size_t off = state_el(A, b, h, 16 * wave + n, 16 * vt + 4 * g);
      f32x4_t gsv = C.G1[vt];
      if (pass) gsv += load_state4(A.gs_out, A.st_f32, off);
      if (A.st_f32) *reinterpret_cast<float4*>(reinterpret_cast<float*>(A.gs) + off) = make_float4(gsv[0], gsv[1], gsv[2], gsv[3]);
      else *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(A.gs) + off) = make_uint2(pack_rn(gsv[0], gsv[1]), pack_rn(gsv[2], gsv[3]));
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
    Raw raw;
    uint32_t ns_mine = 0u;      // this lane's new_starts byte of the chunk loaded next: fetched a step ahead, like the operands
    if (p < nch) {
      ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)(nch - 1 - p) * CK, lane);
      load_raw(raw, A, b, h, (int64_t)(nch - 1 - p) * CK, lane);
    }
    for (int j = p; j < nch; j += NPROD) {
      const int c = nch - 1 - j;
      const int64_t c0 = (int64_t)c * CK;
      ChunkFlags F = chunk_flags_of(A.ns, ns_mine, A.flags, A.T, c0, L);
      if (!inject) F.snap = -1;
      const int si = j % RING;
      if (j >= RING && !wait_consumed_lazy(sy, si, j - RING + 1, lane)) break;
      mask_raw(raw, F.nvalid, lane);
      produce(P, raw, F, &slots[si], snapslot, events_word(A.status));
      if (j + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)(c - NPROD) * CK, lane);
        load_raw(raw, A, b, h, (int64_t)(c - NPROD) * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && j + 1 == nch) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gk, 4, b, h, A.T, A.H);
    poison_token_rows(A.gv, 4, b, h, A.T, A.H);
    poison_token_rows(A.gw, 4, b, h, A.T, A.H);
    poison_state(A.gs, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv6_chunk_bwd_r_f32(const Wkv6Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_bwd_r_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_bwd_r_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
