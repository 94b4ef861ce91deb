// WKV7 backward for fp32 I/O on gfx950, forward sweep B on the matrix cores with fp32 operands
// (v_mfma_f32_16x16x4_f32): gr, ga and the per-token workspace f_t = e3_t + e2_{t+1} (e2 = a.da, dropped when token
// t+1 starts a sequence; e3 = r.dr + <dS_out, S> at token length-1) that the decay-gradient recursion of sweep C
// consumes.
//
// With sa_t known from the forward pass the state obeys a linear recurrence (S[i][j] = value row i, key col j;
// reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220):
//     S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;   dr_t = S_t^T dy_t ;   da_t = S_{t-1}^T dsa_t
// A chunk of 16 tokens entering with S0: E_t = prod_{s<=t} d_s, bh_s = b_s/E_s, kh_s = k_s/E_s,
//     dr_t = E_t     . ( S0^T dy_t  + sum_{s<=t} (sa_s.dy_t)  bh_s + (v_s.dy_t)  kh_s )
//     da_t = E_{t-1} . ( S0^T dsa_t + sum_{s<t}  (sa_s.dsa_t) bh_s + (v_s.dsa_t) kh_s )
//     S_C  = (S0 + SA^T Bh + V^T Kh) diag(E_C)
// The 16x16 Gram tiles contract over the 64 values.  This is the algebra of the bf16 sweep (wkv7_chunk_bwd_b.hip) with
// every product on the fp32 matrix instruction, so that no operand is rounded below fp32.  D = A B with A: lane
// (m = lane%16, g = lane/16) holds A[m][k = g], B: lane (n, g) holds B[k = g][n], D: lane (n, g) holds rows 4g..4g+3 of
// column n; an accumulator register i of a tile X is X as a B operand (k-slot g = row 4g+i) and X^T as an A operand.
//
// Work split: one workgroup of eight waves per (sequence, head), one consumer and one producer per SIMD.  Consumer q
// keeps the state columns of keys 16q..16q+15 (all 64 values) in accumulator registers and runs the state-dependent
// part of every chunk (80 matrix instructions); producer p prepares chunks p, p+4, ... (decay scan, scaled operands,
// Gram tiles: 64 matrix instructions) into a ring of LDS slots.  Synchronisation, resets, `length` and the decay floor
// are those of the other chunked kernels (chunk_common.h); the running log-decay is split into a part on a 2^-16 grid
// and a remainder as in wkv7_fwd_f32.hip.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 4;           // slots in flight (a slot is 35 KB); with three, one of the four producers always idles: +10 %
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

struct __attribute__((aligned(16))) Slot {
  float DY[CK][RF];            // dy rows [token][value]; zero where the entering state does not reach or y is a constant
  float DSA[CK][RF];           // dsa rows, zero where the entering state does not reach
  float SA[CK][RF];            // sa rows, tokens masked for the chunk-end state
  float V[CK][RF];             // v rows, masked likewise
  float BH[CK][RF];            // b_s/E_s rows [token][key]
  float KH[CK][RF];            // k_s/E_s rows
  float E[CK + 1][RF];         // row t+1 = E_t per key, row 0 = 1
  f32x4_t Nys[64], Nyv[64];    // sa_s.dy_t, v_s.dy_t (s <= t), accumulator layout [row s][column t], lane-indexed
  f32x4_t Nss[64], Nsv[64];    // sa_s.dsa_t, v_s.dsa_t (s < t)
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to token length-1
  int ns;                      // bit t: new_starts of in-chunk token t; bit 16: of the first token of the next chunk
};
struct __attribute__((aligned(16))) SnapSlot {   // update operands with the tokens masked for the state at token length-1
  float SA[CK][RF];
  float V[CK][RF];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and, of every 64-vector, the elements 16j + 4g + i (j, i = 0..3): one
// 16-byte load per j, and element (j, i) is this lane's k-slot of the Gram instruction (j, i) both as A and as B operand.
struct Raw {
  float4 w[4], k[4], b[4], v[4], dy[4], sa[4], dsa[4];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;   // always a valid token; mask_raw zeroes the lanes beyond
  const size_t off = (((size_t)b * A.T + tok) * A.H + h) * 64 + 4 * g;
  auto ld = [&](const void* p, float4 (&o)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + off + 16 * j);
  };
  ld(A.w, x.w); ld(A.k, x.k); ld(A.b, x.b);
  ld(A.v, x.v); ld(A.gy, x.dy); ld(A.sa_in, x.sa); ld(A.dsa, x.dsa);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) x.w[j] = x.k[j] = x.b[j] = x.v[j] = x.dy[j] = x.sa[j] = x.dsa[j] = z;
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

// Everything of one chunk that does not depend on the carried state.  The two halves (j = 0,1 and j = 2,3) of the keys
// and of the values go through the same pipeline one after the other, which keeps the live register set small.
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  int lastseg = 0, seg_src = 0;
  bool s0_reaches = true, restart = false, drop_dy = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(F.ns, 15);
    s0_reaches = seg_of(F.ns, t) == 0;                              // the entering state reaches this token
    drop_dy = F.compat && ((F.ns >> (t + 1)) & 1u);                 // y[t] is a constant there: dr_t = 0
    if (resets) keep_upd = 0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u);   // tokens from the last reset on
    const uint32_t upto = resets & ((2u << t) - 1u);
    const int pr = upto ? 31 - __builtin_clz(upto) : 0;             // last reset at or before this token
    restart = pr > 0;
    seg_src = (lane & 48) | (pr > 0 ? pr - 1 : 0);
    if (F.snap >= 0) {
      const uint32_t us = resets & keep_snap;
      if (us) keep_snap &= ~((1u << (31 - __builtin_clz(us))) - 1u);   // tokens of length-1's segment up to it
    }
  }

  // Gram tiles over the values, accumulator layout [row m = s][column n = t]
  f32x4_t Nys = zero4, Nyv = zero4, Nss = zero4, Nsv = zero4;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ================= keys of this half: decay scan, b/E, k/E, E rows
    {
      // Decay scan over the 16 tokens (lanes of one DPP row), log2 domain: every step is split into a part on a 2^-16
      // grid, whose running sums are exact, and a remainder below 2^-17, summed separately.
      float E[8], El[8];
      {
        float fw[8];
        unpack2(x.w[2 * hf], x.w[2 * hf + 1], fw);
#pragma unroll
        for (int e = 0; e < 8; ++e) fw[e] = fmaxf(-exp2_fast(fw[e] * LOG2E) * LOG2E, MIN_STEP_L2);
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
      float fkh[8], fbh[8];
      {
        float fk[8], fb[8];
        unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
        unpack2(x.b[2 * hf], x.b[2 * hf + 1], fb);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
          const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
          E[e] = exp2_fast(l2) * fl;
          const float einv = exp2_fast(-l2) * (2.f - fl);
          fkh[e] = fk[e] * einv;
          fbh[e] = fb[e] * einv;
        }
      }
      put2(slot->E[t + 1], hf, g, E, true);
      if (t == 0) {
        const float one[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
        put2(slot->E[0], hf, g, one, true);
      }
      if (t == 15) {
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      if (F.snap >= 0 && t == F.snap) {
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
      put2(slot->BH[t], hf, g, fbh, true);
      put2(slot->KH[t], hf, g, fkh, true);
    }
    // ================= values of this half: sa, v, dy and dsa rows, partial Gram sums
    {
      float fv[8], fdy[8], fsa[8], fds[8];
      unpack2(x.v[2 * hf], x.v[2 * hf + 1], fv);
      unpack2(x.dy[2 * hf], x.dy[2 * hf + 1], fdy);
      unpack2(x.sa[2 * hf], x.sa[2 * hf + 1], fsa);
      unpack2(x.dsa[2 * hf], x.dsa[2 * hf + 1], fds);
      if (slow) {
        rare_path();
        if (drop_dy) {
#pragma unroll
          for (int e = 0; e < 8; ++e) fdy[e] = 0.f;
        }
      }
      put2(slot->DY[t], hf, g, fdy, s0_reaches);
      put2(slot->DSA[t], hf, g, fds, s0_reaches);
      {
        const bool ku = (keep_upd >> t) & 1u;     // tokens before the last reset do not reach the chunk end
        put2(slot->SA[t], hf, g, fsa, ku);
        put2(slot->V[t], hf, g, fv, ku);
      }
      if (F.snap >= 0) {                          // the same masked for the state at token length-1
        rare_path();
        const bool sk = (keep_snap >> t) & 1u;
        put2(snap->SA[t], hf, g, fsa, sk);
        put2(snap->V[t], hf, g, fv, sk);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        Nys = mfma_f(fsa[e], fdy[e], Nys);      // [s][t] = sa_s . dy_t
        Nyv = mfma_f(fv[e], fdy[e], Nyv);       // [s][t] = v_s . dy_t
        Nss = mfma_f(fsa[e], fds[e], Nss);      // [s][t] = sa_s . dsa_t
        Nsv = mfma_f(fv[e], fds[e], Nsv);       // [s][t] = v_s . dsa_t
      }
    }
  }
  // ---- triangular masks (rows s, column t = this lane's token)
  const int n = t;
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      Nys[i] = m <= n ? Nys[i] : 0.f;
      Nyv[i] = m <= n ? Nyv[i] : 0.f;
      Nss[i] = m < n ? Nss[i] : 0.f;
      Nsv[i] = m < n ? Nsv[i] : 0.f;
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      Nys[i] = (m <= n && same) ? Nys[i] : 0.f;
      Nyv[i] = (m <= n && same) ? Nyv[i] : 0.f;
      Nss[i] = (m < n && same) ? Nss[i] : 0.f;
      Nsv[i] = (m < n && same) ? Nsv[i] : 0.f;
    }
  }
  slot->Nys[lane] = Nys;
  slot->Nyv[lane] = Nyv;
  slot->Nss[lane] = Nss;
  slot->Nsv[lane] = Nsv;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
    slot->ns = (int)F.ns;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state columns of keys 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), S[vt][i] = S[value 16*vt + 4g + i][key 16q + n]: register i of a tile is the B operand of the
// instruction that contracts over the values 16*vt + 4g' + i (g' = 0..3).
struct Consumer {
  f32x4_t S[4];
  float pend;          // lanes g = 3: r.dr of the previous chunk's last token, whose workspace entry is still open
  // r and a of this lane's four (token, key) pairs of the chunk handled next: fetched from memory by the consumer
  // itself, one chunk ahead, instead of passing through the LDS slot (8.5 KB per slot: the difference between a ring of
  // three and one of four)
  float rr[4], aa[4];
  int q, lane;
};

// r and a at (tokens c0 + 4g .. + 3, key 16q + n); tokens beyond the sequence read the last one (their results are
// never stored)
__device__ __forceinline__ void fetch_ra(Consumer& C, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0) {
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t tok = c0 + 4 * g + i;
    tok = tok < A.T ? tok : A.T - 1;
    const size_t el = (((size_t)b * A.T + tok) * A.H + h) * 64 + 16 * C.q + n;
    C.rr[i] = reinterpret_cast<const float*>(A.r)[el];
    C.aa[i] = reinterpret_cast<const float*>(A.a)[el];
  }
}

struct OutCursor {
  float *gr, *ga;      // outputs at (b, c0, h, 0)
  float* ef;           // this wave's record of the chunk in the fp32 workspace (f_record)
  size_t tok;          // elements between consecutive tokens
  uint32_t voff;       // lane part of the address: (4g * H) * 64 + key
};

__device__ __forceinline__ size_t state_el(const Wkv7Args& A, int64_t b, int64_t h, int value, int key) {
  return (((size_t)b * A.H + h) * 64 + value) * 64 + key;
}
__device__ __forceinline__ float ld_state_el(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool first,
                                        int64_t next_c0, OutCursor& oc) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const float rr[4] = {C.rr[0], C.rr[1], C.rr[2], C.rr[3]}, aa[4] = {C.aa[0], C.aa[1], C.aa[2], C.aa[3]};
  if (next_c0 >= 0) fetch_ra(C, A, b, h, next_c0);
  // B operands of the token contractions: (b/E, k/E) of tokens 4g..4g+3 at this wave's keys
  float tb[4], tk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    tb[i] = slot->BH[4 * g + i][16 * q + n];
    tk[i] = slot->KH[4 * g + i][16 * q + n];
  }
  const bool keep_end = slot->keep_end != 0;
  f32x4_t DR = zero4, DA = zero4;   // [token 4g+i][key n], two interleaved accumulation chains
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const float4 dy4 = *reinterpret_cast<const float4*>(&slot->DY[n][16 * vt + 4 * g]);
    const float4 ds4 = *reinterpret_cast<const float4*>(&slot->DSA[n][16 * vt + 4 * g]);
    const float dy[4] = {dy4.x, dy4.y, dy4.z, dy4.w}, ds[4] = {ds4.x, ds4.y, ds4.z, ds4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      DR = mfma_f(dy[i], C.S[vt][i], DR);       // S0^T dy_t
      DA = mfma_f(ds[i], C.S[vt][i], DA);       // S0^T dsa_t
    }
  }
  {
    const f32x4_t nys = slot->Nys[lane], nyv = slot->Nyv[lane], nss = slot->Nss[lane], nsv = slot->Nsv[lane];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      DR = mfma_f(nys[i], tb[i], DR); DA = mfma_f(nss[i], tb[i], DA);
      DR = mfma_f(nyv[i], tk[i], DR); DA = mfma_f(nsv[i], tk[i], DA);
    }
  }
  // <dS_out, S_{length-1}> per key (one chunk per sequence)
  float inj = 0.f;
  int snap_tok = -1;
  if (is_snap) {
    rare_path();
    snap_tok = slot->snap;
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
    float p = 0.f;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      f32x4_t acc = keep ? C.S[vt] : zero4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc = mfma_f(snapslot->SA[4 * g + i][16 * vt + n], tb[i], acc);
        acc = mfma_f(snapslot->V[4 * g + i][16 * vt + n], tk[i], acc);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        p = fmaf(ld_state_el(A.gs_out, A.st_f32, state_el(A, b, h, 16 * vt + 4 * g + i, 16 * q + n)), acc[i] * sg, p);
    }
    p += __shfl_xor(p, 16, 64);
    p += __shfl_xor(p, 32, 64);
    inj = p;
  }
  // state update: S <- (S + SA^T Bh + V^T Kh) . gamma (per key = per lane)
  if (!keep_end) {
    rare_path();
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = zero4;   // a reset inside the chunk cuts the entering state off
  }
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    float sa[4], vv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sa[i] = slot->SA[4 * g + i][16 * vt + n];
      vv[i] = slot->V[4 * g + i][16 * vt + n];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      C.S[vt] = mfma_f(sa[i], tb[i], C.S[vt]);
      C.S[vt] = mfma_f(vv[i], tk[i], C.S[vt]);
    }
  }
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) { C.S[vt][0] *= gm; C.S[vt][1] *= gm; C.S[vt][2] *= gm; C.S[vt][3] *= gm; }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive keys
  float e[5];
#pragma unroll
  for (int i = 0; i < 5; ++i) e[i] = slot->E[4 * g + i][16 * q + n];
  const bool full = nvalid == CK;      // every chunk but a partial last one: no per-lane predicates
  float e2[4], e3[4], odr[4], oda[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    odr[i] = DR[i] * e[i + 1];
    oda[i] = DA[i] * e[i];
    e2[i] = aa[i] * oda[i];
    e3[i] = fmaf(rr[i], odr[i], tok == snap_tok ? inj : 0.f);
  }
  if (!full) {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (4 * g + i >= nvalid) e2[i] = 0.f;          // nothing follows the last token of the sequence
  }
  // What the decay-gradient recursion of sweep C adds at token t is e3_t + e2_{t+1}, without e2_{t+1} when token
  // t+1 starts a sequence.  e2 of the next token lives in this lane, in the lane 16 further on (token 4g+4), or in
  // the next chunk: the entry of token 15 stays open until then.
  const uint32_t nsm = (uint32_t)slot->ns;
  auto follows = [&](int tok) { return ((nsm >> tok) & 1u) == 0; };   // token `tok` continues the sequence of tok-1
  const float up = __shfl_down(e2[0], 16, 64);
  float f[4];
#pragma unroll
  for (int i = 0; i < 3; ++i) f[i] = e3[i] + (follows(4 * g + i + 1) ? e2[i + 1] : 0.f);
  f[3] = e3[3] + ((g < 3 && follows(4 * g + 4)) ? up : 0.f);
  const float open_prev = __shfl(C.pend, n + 48, 64);   // the previous chunk's token 15, handed to the lanes of token 0
  C.pend = e3[3];
  float* const rl = oc.gr + oc.voff;
  float* const al = oc.ga + oc.voff;
  if (full) {
#pragma unroll
    for (int i = 0; i < 4; ++i) rl[i * oc.tok] = odr[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) al[i * oc.tok] = oda[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        rl[i * oc.tok] = odr[i];
        al[i * oc.tok] = oda[i];
      }
    }
  }
  // The whole record entry at once.  Token 15 of a chunk that is not the last one is still open: its entry (lanes
  // g = 3, element 3) is a placeholder until the next chunk overwrites it below; both stores come from this wave, to
  // the same address, in program order.  Entries of tokens beyond the sequence are never used.
  *reinterpret_cast<float4*>(oc.ef + 4 * lane) = make_float4(f[0], f[1], f[2], f[3]);
  if (!first && g == 0) (oc.ef - NCONS * F_REC)[4 * (48 + n) + 3] = open_prev + (follows(0) ? e2[0] : 0.f);
  oc.gr += CK * oc.tok; oc.ga += CK * oc.tok;
  oc.ef += NCONS * F_REC;
}

}  // namespace

// Slot c % RING holds chunk c.  Producer p fills it once every consumer has released chunk c - RING, then
// publishes ready = c + 1; consumers take chunks in order.  Every wait is for a strictly earlier chunk, so the
// hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_bwd_b_f32_kernel(Wkv7Args A) {
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
    C.pend = 0.f;
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        C.S[vt][i] = ld_state_el(A.s, A.st_f32, state_el(A, b, h, 16 * vt + 4 * g + i, 16 * wave + n));
    OutCursor oc;
    oc.tok = (size_t)A.H * 64;
    const size_t el0 = (((size_t)b * A.T) * A.H + h) * 64;
    oc.gr = reinterpret_cast<float*>(A.gr) + el0;
    oc.ga = reinterpret_cast<float*>(A.ga) + el0;
    oc.ef = A.e2 + f_record(b, h, A.H, nch, 0, wave);
    oc.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    if (nch > 0) fetch_ra(C, A, b, h, 0);
    for (int c = 0; c < nch; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING;
      if (!wait_ready(sy, si, c + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, c == 0, c + 1 < nch ? (int64_t)(c + 1) * CK : -1, oc);
      // every LDS read of slot si has returned: its data went into the matrix instructions and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
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
      produce(lane, raw, F, &slots[si], snapslot, events_word(A.status));
      if (c + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, c0 + (int64_t)NPROD * CK, lane);
        load_raw(raw, A, b, h, c0 + (int64_t)NPROD * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && c + 1 == nch) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gr, 4, b, h, A.T, A.H);
    poison_token_rows(A.ga, 4, b, h, A.T, A.H);
    for (size_t i = threadIdx.x; i < (size_t)nch * NCONS * F_REC; i += blockDim.x)
      A.e2[f_record(b, h, A.H, nch, 0, 0) + i] = __uint_as_float(0x7fc00000u);
  }
}

hipError_t launch_wkv7_chunk_bwd_b_f32(const Wkv7Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_bwd_b_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_bwd_b_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
