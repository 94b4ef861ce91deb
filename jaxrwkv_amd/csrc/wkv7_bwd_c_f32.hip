// WKV7 backward for fp32 I/O on gfx950, reverse sweep C on the matrix cores with fp32 operands
// (v_mfma_f32_16x16x4_f32): gk, gb and the decay gradient gw.
//
// With dsa_t known from sweep A the cotangent G = dL/dS obeys a linear recurrence, carried from the last token
// down (G~_t the cotangent of S_t; S[i][j] = value row i, key col j; reference:
// /root/reference/src/jaxrwkv/rwkv7.py:200-220):
//     G~_t = dy_t r_t^T + G~_{t+1} diag(d_{t+1}) + dsa_{t+1} a_{t+1}^T ;   dk_t = G~_t^T v_t ;   db_t = G~_t^T sa_t
// A chunk of 16 tokens leaving with G_C: E_t = prod_{s<=t} d_s, qt_s = r_s.E_s, at_s = a_s.E_{s-1}, Gh = G_C diag(E_C):
//     dk_t = (1/E_t) . ( Gh^T v_t  + sum_{s>t} (dsa_s.v_t)  at_s + sum_{s>=t} (dy_s.v_t)  qt_s )
//     db_t = (1/E_t) . ( Gh^T sa_t + sum_{s>t} (dsa_s.sa_t) at_s + sum_{s>=t} (dy_s.sa_t) qt_s )
//     G_prev = Gh + DSA^T At + DY^T Qt
// and the decay gradient from the running sum c_t = reset_t ? 0 : c_{t+1} + f_t - k_t.dk_t - b_t.db_t,
// dw_t = c_t * (-exp(w_t)), with the vector f_t that sweep B leaves (wkv7_chunk_bwd_c.hip derives it).  This is the
// algebra of that bf16 sweep with every product on the fp32 matrix instruction; layouts and work split are those of
// wkv7_bwd_b_f32.hip (consumer q holds the cotangent columns of keys 16q..16q+15; 80 matrix instructions per consumer
// and chunk, 64 per producer).  Chunks are handled from the last one down.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns steps p, p + NPROD, ...
constexpr int RING = 4;           // slots in flight (a slot is 35 KB); with three, one of the four producers always idles
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float row_prev0(float x) {     // previous lane of the row, 0 in lane 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true));
}

struct __attribute__((aligned(16))) Slot {
  float V[CK][RF];             // v rows [token][value]; zero where the cotangent of later chunks does not reach
  float SA[CK][RF];            // sa rows, masked likewise
  float DSA[CK][RF];           // dsa rows, tokens masked for the chunk-start cotangent
  float DY[CK][RF];            // dy rows (zero where y is a constant), masked likewise
  float AT[CK][RF];            // a_s.E_{s-1} rows [token][key]
  float QT[CK][RF];            // r_s.E_s rows
  float Einv[CK][RF];          // 1/E_t per key
  f32x4_t Nsv[64], Nyv[64];    // dsa_s.v_t (s > t), dy_s.v_t (s >= t), accumulator layout [row s][column t], lane-indexed
  f32x4_t Nss[64], Nys[64];    // dsa_s.sa_t (s > t), dy_s.sa_t (s >= t)
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the cotangent of later chunks reaches the chunk start (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int resets;                  // bit t: new_starts of in-chunk token t
};
struct __attribute__((aligned(16))) SnapSlot {   // row operands masked to the tokens the cotangent entering at length-1 reaches
  float V[CK][RF];
  float SA[CK][RF];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and, of every 64-vector, the elements 16j + 4g + i (j, i = 0..3): one
// 16-byte load per j, and element (j, i) is this lane's k-slot of the Gram instruction (j, i) both as A and as B operand.
struct Raw {
  float4 w[4], r[4], a[4], v[4], dy[4], sa[4], dsa[4];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;   // always a valid token; mask_raw zeroes the lanes beyond
  const size_t off = (((size_t)b * A.T + tok) * A.H + h) * 64 + 4 * g;
  auto ld = [&](const void* p, float4 (&o)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + off + 16 * j);
  };
  ld(A.w, x.w); ld(A.r, x.r); ld(A.a, x.a);
  ld(A.v, x.v); ld(A.gy, x.dy); ld(A.sa_in, x.sa); ld(A.dsa, x.dsa);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) x.w[j] = x.r[j] = x.a[j] = x.v[j] = x.dy[j] = x.sa[j] = x.dsa[j] = z;
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

// Everything of one chunk that does not depend on the carried cotangent.  The two halves (j = 0,1 and j = 2,3) of the
// keys and of the values go through the same pipeline one after the other, which keeps the live register set small.
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  int lastseg = 0, seg_src = 0;
  bool row_keep = true, restart = false, drop_dy = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(F.ns, 15);
    row_keep = seg_of(F.ns, t) == lastseg;                          // the cotangent of later chunks reaches this token
    drop_dy = F.compat && ((F.ns >> (t + 1)) & 1u);                 // y[t] is a constant there
    if (resets) keep_upd = (1u << __builtin_ctz(resets)) - 1u;      // tokens before the first reset
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
  f32x4_t Nsv = zero4, Nyv = zero4, Nss = zero4, Nys = zero4;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ================= keys of this half: decay scan, a.E_{t-1}, r.E_t, 1/E rows
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
      float fat[8], fqt[8], Einv[8];
      {
        float fr[8], fa[8];
        unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
        unpack2(x.a[2 * hf], x.a[2 * hf + 1], fa);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
          const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
          E[e] = exp2_fast(l2) * fl;
          Einv[e] = exp2_fast(-l2) * (2.f - fl);
          // The decay up to the previous token is 1 for the chunk's first token.  At a reset token the value belongs to
          // the previous segment, but every product it enters is masked out.
          const float fa0 = (t == 0) ? fa[e] : 0.f;
          fat[e] = fmaf(fa[e], row_prev0(E[e]), fa0);
          fqt[e] = fr[e] * E[e];
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
      put2(slot->AT[t], hf, g, fat, true);
      put2(slot->QT[t], hf, g, fqt, true);
    }
    // ================= values of this half: v, sa, dy and dsa rows, partial Gram sums
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
      put2(slot->V[t], hf, g, fv, row_keep);
      put2(slot->SA[t], hf, g, fsa, row_keep);
      if (F.snap >= 0) {                          // the same masked for the cotangent entering at token length-1
        rare_path();
        const bool sk = (keep_snap >> t) & 1u;
        put2(snap->V[t], hf, g, fv, sk);
        put2(snap->SA[t], hf, g, fsa, sk);
      }
      {
        const bool ku = (keep_upd >> t) & 1u;     // tokens from the first reset on do not reach the chunk start
        put2(slot->DSA[t], hf, g, fds, ku);
        put2(slot->DY[t], hf, g, fdy, ku);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        Nsv = mfma_f(fds[e], fv[e], Nsv);       // [s][t] = dsa_s . v_t
        Nyv = mfma_f(fdy[e], fv[e], Nyv);       // [s][t] = dy_s . v_t
        Nss = mfma_f(fds[e], fsa[e], Nss);      // [s][t] = dsa_s . sa_t
        Nys = mfma_f(fdy[e], fsa[e], Nys);      // [s][t] = dy_s . sa_t
      }
    }
  }
  // ---- triangular masks (rows s, column t = this lane's token)
  const int n = t;
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      Nsv[i] = m > n ? Nsv[i] : 0.f;
      Nss[i] = m > n ? Nss[i] : 0.f;
      Nyv[i] = m >= n ? Nyv[i] : 0.f;
      Nys[i] = m >= n ? Nys[i] : 0.f;
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      Nsv[i] = (m > n && same) ? Nsv[i] : 0.f;
      Nss[i] = (m > n && same) ? Nss[i] : 0.f;
      Nyv[i] = (m >= n && same) ? Nyv[i] : 0.f;
      Nys[i] = (m >= n && same) ? Nys[i] : 0.f;
    }
  }
  slot->Nsv[lane] = Nsv;
  slot->Nyv[lane] = Nyv;
  slot->Nss[lane] = Nss;
  slot->Nys[lane] = Nys;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
    slot->resets = (int)resets;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the cotangent columns of keys 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), G[vt][i] = G[value 16*vt + 4g + i][key 16q + n].
struct Consumer {
  f32x4_t G[4];
  float carry;         // running sum of the decay-gradient recursion, per key (same in the four lanes of a key)
  float4 f;            // this wave's record entry of the chunk handled next (requested one chunk ahead)
  // k, b and w of this lane's four (token, key) pairs of the chunk handled next: fetched from memory by the consumer
  // itself, one chunk ahead, instead of passing through the LDS slot (13 KB per slot: the difference between a ring of
  // three and one of four)
  float kk[4], bb[4], ww[4];
  int q, lane;
};

// k, b, w at (tokens c0 + 4g .. + 3, key 16q + n); tokens beyond the sequence read the last one (their results are
// never stored)
__device__ __forceinline__ void fetch_kbw(Consumer& C, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0) {
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t tok = c0 + 4 * g + i;
    tok = tok < A.T ? tok : A.T - 1;
    const size_t el = (((size_t)b * A.T + tok) * A.H + h) * 64 + 16 * C.q + n;
    C.kk[i] = reinterpret_cast<const float*>(A.k)[el];
    C.bb[i] = reinterpret_cast<const float*>(A.b)[el];
    C.ww[i] = reinterpret_cast<const float*>(A.w)[el];
  }
}

struct Cursor {
  float *gk, *gb, *gw;         // outputs at (b, c0, h, 0)
  const float4* rec;           // this lane's entry of this wave's record of the chunk handled next
  size_t tok;                  // elements between consecutive tokens
  uint32_t voff;               // lane part of the address: (4g * H) * 64 + key
};

__device__ __forceinline__ size_t state_el(const Wkv7Args& A, int64_t b, int64_t h, int value, int key) {
  return (((size_t)b * A.H + h) * 64 + value) * 64 + key;
}
__device__ __forceinline__ float ld_state_el(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool last,
                                        int64_t next_c0, Cursor& cu) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // this chunk's record entry and per-token scalars were requested a chunk ago; request the next ones
  const float4 fr = C.f;
  const float kk[4] = {C.kk[0], C.kk[1], C.kk[2], C.kk[3]}, bb[4] = {C.bb[0], C.bb[1], C.bb[2], C.bb[3]};
  const float ww[4] = {C.ww[0], C.ww[1], C.ww[2], C.ww[3]};
  if (!last) {
    cu.rec -= NCONS * (F_REC / 4);
    C.f = *cu.rec;
    fetch_kbw(C, A, b, h, next_c0);
  }
  // B operands of the token contractions: (a.E_{s-1}, r.E_s) of tokens 4g..4g+3 at this wave's keys
  float ta[4], tq[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ta[i] = slot->AT[4 * g + i][16 * q + n];
    tq[i] = slot->QT[4 * g + i][16 * q + n];
  }
  const bool keep_end = slot->keep_end != 0;
  const uint32_t resets = (uint32_t)slot->resets;
  // the cotangent of the chunk-end state, decayed over the chunk (per key = per lane)
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) { C.G[vt][0] *= gm; C.G[vt][1] *= gm; C.G[vt][2] *= gm; C.G[vt][3] *= gm; }
  f32x4_t DK = zero4, DB = zero4;   // [token 4g+i][key n], two interleaved accumulation chains
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const float4 v4 = *reinterpret_cast<const float4*>(&slot->V[n][16 * vt + 4 * g]);
    const float4 s4 = *reinterpret_cast<const float4*>(&slot->SA[n][16 * vt + 4 * g]);
    const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      DK = mfma_f(vv[i], C.G[vt][i], DK);       // Gh^T v_t
      DB = mfma_f(ss[i], C.G[vt][i], DB);       // Gh^T sa_t
    }
  }
  {
    const f32x4_t nsv = slot->Nsv[lane], nyv = slot->Nyv[lane], nss = slot->Nss[lane], nys = slot->Nys[lane];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      DK = mfma_f(nsv[i], ta[i], DK); DB = mfma_f(nss[i], ta[i], DB);
      DK = mfma_f(nyv[i], tq[i], DK); DB = mfma_f(nys[i], tq[i], DB);
    }
  }
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
    rare_path();
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.G[vt] = zero4;
  }
  // the cotangent of the returned state enters at token length-1 (one chunk per sequence)
  if (is_snap) {
    rare_path();
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      f32x4_t gs;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        gs[i] = ld_state_el(A.gs_out, A.st_f32, state_el(A, b, h, 16 * vt + 4 * g + i, 16 * q + n)) * sg;
      if (keep) C.G[vt] += gs;
      const float4 v4 = *reinterpret_cast<const float4*>(&snapslot->V[n][16 * vt + 4 * g]);
      const float4 s4 = *reinterpret_cast<const float4*>(&snapslot->SA[n][16 * vt + 4 * g]);
      const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        DK = mfma_f(vv[i], gs[i], DK);
        DB = mfma_f(ss[i], gs[i], DB);
      }
    }
  }
  // cotangent update: G <- Gh + DSA^T At + DY^T Qt
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    float ds[4], dd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ds[i] = slot->DSA[4 * g + i][16 * vt + n];
      dd[i] = slot->DY[4 * g + i][16 * vt + n];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      C.G[vt] = mfma_f(ds[i], ta[i], C.G[vt]);
      C.G[vt] = mfma_f(dd[i], tq[i], C.G[vt]);
    }
  }
  // per-token results: register i is token 4g+i, lanes n = 16 consecutive keys
  float dk[4], db[4], z[4], cy[4], nej[4];
  float fv[4] = {fr.x, fr.y, fr.z, fr.w};
  if (nvalid != CK) {         // entries of tokens beyond the sequence hold nothing meaningful
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) fv[i] = (4 * g + i < nvalid) ? fv[i] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float ei = slot->Einv[4 * g + i][16 * q + n];
    dk[i] = DK[i] * ei;
    db[i] = DB[i] * ei;
    z[i] = fv[i] - kk[i] * dk[i] - bb[i] * db[i];
    nej[i] = -exp2_fast(ww[i] * LOG2E);      // -exp(w): the factor between the log-decay gradient and gw
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
  float* const kl = cu.gk + cu.voff;
  float* const bl = cu.gb + cu.voff;
  float* const wl = cu.gw + cu.voff;
  if (nvalid == CK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) kl[i * cu.tok] = dk[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) bl[i * cu.tok] = db[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) wl[i * cu.tok] = cy[i] * nej[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        kl[i * cu.tok] = dk[i];
        bl[i * cu.tok] = db[i];
        wl[i * cu.tok] = cy[i] * nej[i];
      }
    }
  }
  const size_t d = CK * cu.tok;
  cu.gk -= d; cu.gb -= d; cu.gw -= d;
}

}  // namespace

// Step j handles chunk nch-1-j in slot j % RING.  Producer p fills the slot once every consumer has released step
// j - RING, then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier
// step, so the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_bwd_c_f32_kernel(Wkv7Args A) {
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
    for (int vt = 0; vt < 4; ++vt) C.G[vt] = zero4;
    Cursor cu;
    cu.tok = (size_t)A.H * 64;
    const size_t el0 = (((size_t)b * A.T + (size_t)(nch - 1) * CK) * A.H + h) * 64;
    cu.gk = reinterpret_cast<float*>(A.gk) + el0;
    cu.gb = reinterpret_cast<float*>(A.gb) + el0;
    cu.gw = reinterpret_cast<float*>(A.gw) + el0;
    cu.rec = reinterpret_cast<const float4*>(A.e2 + f_record(b, h, A.H, nch, nch - 1, wave)) + lane;
    cu.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    C.f = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nch > 0) {
      C.f = *cu.rec;
      fetch_kbw(C, A, b, h, (int64_t)(nch - 1) * CK);
    }
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    const int tail = (A.T % CK == 0) ? CK : (int)(A.T % CK);
    for (int j = 0; j < nch; ++j) {
      const int c = nch - 1 - j;
      const int nvalid = (j == 0) ? tail : CK;
      const int si = j % RING;
      if (!wait_ready(sy, si, j + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, j + 1 == nch, (int64_t)(c - 1) * CK, cu);
      // every LDS read of slot si has returned: its data went into the matrix instructions and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
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
      produce(lane, raw, F, &slots[si], snapslot, events_word(A.status));
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
    poison_token_rows(A.gb, 4, b, h, A.T, A.H);
    poison_token_rows(A.gw, 4, b, h, A.T, A.H);
  }
}

hipError_t launch_wkv7_chunk_bwd_c_f32(const Wkv7Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_bwd_c_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_bwd_c_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
