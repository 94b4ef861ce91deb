// WKV6 backward, reverse sweep R on the matrix cores (bf16 I/O, gfx950): gk, gv, gw, gs.
//
// With G_t the cotangent of the state after token t (reference recurrence: /root/reference/src/jaxrwkv/rwkv6.py:175-191;
// S[i][j] = key row i, value col j; dec_t = exp(w_t)), carried from the last token down:
//     G_t = dec_{t+1} G_{t+1} + r_{t+1} dy_{t+1}^T (+ dS_out at t = length-1),  cut at new_starts
//     dk_t = r_t u c_t + G_t v_t ,  c_t = v_t.dy_t          dv_t = dy_t (r_t.(u k_t)) + G_t^T k_t
//     dw_t = carry_t - er_t ,  carry_t = reset_t ? 0 : carry_{t+1} + er_t (+ eI at t = length-1) - k_t.(G_t v_t)
// (er, eI from the forward sweep).  A chunk of C = 16 tokens leaving with G_C: E_t = prod_{s<=t} dec_s, Ee_t = E_{t-1},
// rq_s = r_s.Ee_s, kh_t = k_t/E_t, Gh = diag(E_C) G_C:
//     diag(E_t) G_t = Gh + sum_{s>t} rq_s dy_s^T
//     G_t v_t   = (1/E_t) . ( Gh v_t + sum_{s>t} (dy_s.v_t) rq_s )          contracts over values
//     G_t^T k_t = Gh^T kh_t + sum_{s>t} (rq_s.kh_t) dy_s                     contracts over keys
//     G_prev = Gh + sum_s rq_s dy_s^T
// The two contractions run over different axes of G, so there are two kinds of consumer wave, four of each: a key wave
// keeps the rows of its 16 keys (all values, for G v), a value wave the columns of its 16 values (all keys, for
// G^T k); both get the same rank-16 update.  (One wave holding both copies has twice the dependent work per chunk and
// paces the sweep; two kinds of wave halve it, and twelve waves at 160 registers still fit three to a SIMD.)  Products with fp32 quantities run as hi.hi + hi.lo + lo.hi on v_mfma_f32_16x16x32_bf16.
// Work split, LDS ring and hand-shake as in the other chunked kernels; the producers also own the state-free terms
// r u c_t and dy (r.(u k)), handed over as fp32 add-ons.  Range: a chunk's total log decay per channel is capped at -80.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns steps p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight (a slot is 30 KB)
constexpr int ES = 68;            // row stride (floats) of the fp32 [token][.] arrays: conflict-free column reads
constexpr int NCONS_R = 8;        // consumer waves: 0-3 hold G1 (gk, gw, gs), 4-7 hold G2 (gv)

using Sync8 = SyncN<NCONS_R>;     // the hand-shake words for eight consumers

// "lane-indexed" arrays hold, for every lane of the producer, the bytes the same lane of a consumer loads:
// accumulator-layout registers (column lane%16, rows 4*(lane/16)..+3) packed to bf16, hi pair then lo pair.
struct __attribute__((aligned(16))) Slot {
  // v rows (permuted value order) and k/E rows (hi, lo; permuted key order), [token][RS]: the 16-byte vector (j, g)
  // at element 32j + 8g holds elements 32j+4g..+3 followed by 32j+16+4g..+3, the order of the consumers' tiles.
  // Rows that the cotangent of later chunks does not reach are zero.
  uint16_t V[CK][RS];
  uint16_t KH[2][CK][RS];
  uint4 RQ[4][64];             // (r_s.Ee_s)^T per key tile: hi,lo, lane-indexed
  uint2 DYt[4][64];            // dy^T per value tile, lane-indexed
  uint2 DYtU[4][64];           // the same with the tokens masked for the chunk-start cotangent
  uint4 N1[64];                // dy_s.v_t (s > t): hi pair, lo pair, lane-indexed (A operand row t, k-slots s)
  uint4 N2[64];                // rq_s.kh_t (s > t)
  float Einv[CK][ES];          // 1/E_t per key
  float RUC[CK][ES];           // r_t u c_t per key
  float DYR[CK][ES];           // dy_t (r_t.(u k_t)) per value
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the cotangent of later chunks reaches the chunk start (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int resets;                  // bit t: new_starts of in-chunk token t
};
struct __attribute__((aligned(16))) SnapSlot {
  uint16_t V[CK][RS];          // row operands masked to the tokens that the cotangent entering at length-1 reaches
  uint16_t KH[2][CK][RS];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
struct Raw {
  uint4 r[2], k[2], v[2], w[2], dy[2];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  if (c0 + t < A.T) {
    const size_t off = ((((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g) * 2;  // bytes
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off + 64);
    };
    ld(A.r, x.r); ld(A.k, x.k); ld(A.v, x.v); ld(A.gy, x.dy);
    // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
    const size_t woff = (A.flags & FLAG_W_PER_HEAD) ? ((size_t)h * 64 + 8 * g) * 2 : off;
    x.w[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff);
    x.w[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff + 64);
  } else {
    const uint4 z = make_uint4(0, 0, 0, 0);
    x.r[0] = x.r[1] = x.k[0] = x.k[1] = x.v[0] = x.v[1] = x.w[0] = x.w[1] = x.dy[0] = x.dy[1] = z;
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // MFMA-as-transposer selection operands
  uint4 u[2];         // bonus of this lane's keys (bf16)
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
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    lastseg = seg_of(resets, 15);
    row_keep = seg_of(resets, t) == lastseg;                        // the cotangent of later chunks reaches this token
    keep_upd = (1u << __builtin_ctz(resets)) - 1u;                  // tokens before the first reset
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
  auto masked_pack = [&](const f32x4_t d, uint32_t keep) {
    const uint32_t bits = keep >> (4 * g);
    const float d0 = (bits & 1u) ? d[0] : 0.f, d1 = (bits & 2u) ? d[1] : 0.f;
    const float d2 = (bits & 4u) ? d[2] : 0.f, d3 = (bits & 8u) ? d[3] : 0.f;
    return make_uint2(pack_exact(d0, d1), pack_exact(d2, d3));
  };
  auto plain_pack = [&](const f32x4_t d) { return make_uint2(pack_exact(d[0], d[1]), pack_exact(d[2], d[3])); };

  f32x4_t N1 = zero4, N2 = zero4;   // [row s][column t]: dy_s.v_t and rq_s.kh_t
  float ruk = 0.f;                  // partial r.(u k) over this lane's keys
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // first 8-byte piece of this lane in a permuted row
    auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
      *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
      *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
    };
    // ================= keys of this half: decay scan, (r.Ee)^T, k/E rows, 1/E rows
    {
      float E[8];
      {
        float fw[8];
        unpack8(x.w[hf], fw);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float l2 = fmaxf(fw[e] * LOG2E, MIN_STEP_L2);
          if (F.nvalid != CK) l2 = valid ? l2 : 0.f;
          E[e] = row_scan(l2);
        }
        cap_chunk_decay(E, lane, events);
      }
      if (slow) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
          if (restart) E[e] -= base;
        }
      }
      u32x4_t rq_h, rq_l, kh_h, kh_l;
      float Einv[8];
      {
        float fr[8], fk[8], fu[8], Ee[8];
        unpack8(x.r[hf], fr); unpack8(x.k[hf], fk); unpack8(P.u[hf], fu);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = fmaxf(E[e], MIN_CUM_L2);
          E[e] = exp2_fast(l2);
          Einv[e] = exp2_fast(-l2);
          // value of the previous token; 1 for the first token.  At a reset token it belongs to the previous
          // segment, but every product rq enters for that token is masked out.
          Ee[e] = row_prev(E[e], 1.0f);
          ruk = fmaf(fr[e] * fu[e], fk[e], ruk);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = 2 * j;
          uint32_t hi, lo;
          split2(fr[e] * Ee[e], fr[e + 1] * Ee[e + 1], hi, lo); rq_h[j] = hi; rq_l[j] = lo;
          split2(fk[e] * Einv[e], fk[e + 1] * Einv[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
        }
      }
      {
        float* er = &slot->Einv[t][32 * hf + 8 * g];
        *reinterpret_cast<float4*>(er) = make_float4(Einv[0], Einv[1], Einv[2], Einv[3]);
        *reinterpret_cast<float4*>(er + 4) = make_float4(Einv[4], Einv[5], Einv[6], Einv[7]);
      }
      if (t == 15) {
        float* gp = &slot->gamma[8 * g + 32 * hf];
        *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
      }
      if (t == F.snap) {
        float* gp = &snap->gamma[8 * g + 32 * hf];
        *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
      }
      put(slot->KH[0][t], kh_h, row_keep);
      put(slot->KH[1][t], kh_l, row_keep);
      if (F.snap >= 0) {
        put(snap->KH[0][t], kh_h, snap_keep);
        put(snap->KH[1][t], kh_l, snap_keep);
      }
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const u32x4_t sel = P.sel[x2];
        const uint2 dh = plain_pack(mfma(rq_h, sel, zero4)), dl = plain_pack(mfma(rq_l, sel, zero4));
        slot->RQ[2 * hf + x2][lane] = make_uint4(dh.x, dh.y, dl.x, dl.y);
      }
      N2 = mfma(rq_h, kh_h, N2); N2 = mfma(rq_h, kh_l, N2); N2 = mfma(rq_l, kh_h, N2);   // [s][t] = rq_s . kh_t
    }
    // ================= values of this half: dy^T, v rows, partial Gram sum
    {
      const uint4 vr = x.v[hf], dr = x.dy[hf];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w}, dyop = {dr.x, dr.y, dr.z, dr.w};
      put(slot->V[t], vop, row_keep);
      if (F.snap >= 0) put(snap->V[t], vop, snap_keep);
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const f32x4_t dd = mfma(dyop, P.sel[x2], zero4);
        slot->DYt[tile][lane] = plain_pack(dd);
        slot->DYtU[tile][lane] = keep_upd == 0xffffu ? plain_pack(dd) : masked_pack(dd, keep_upd);
      }
      N1 = mfma(dyop, vop, N1);                                       // [s][t] = dy_s . v_t
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
    float fr[8], fu[8], fd[8];
    unpack8(x.r[hf], fr); unpack8(P.u[hf], fu); unpack8(x.dy[hf], fd);
    float* up = &slot->RUC[t][32 * hf + 8 * g];
    *reinterpret_cast<float4*>(up) = make_float4(fr[0] * fu[0] * c_t, fr[1] * fu[1] * c_t, fr[2] * fu[2] * c_t, fr[3] * fu[3] * c_t);
    *reinterpret_cast<float4*>(up + 4) = make_float4(fr[4] * fu[4] * c_t, fr[5] * fu[5] * c_t, fr[6] * fu[6] * c_t, fr[7] * fu[7] * c_t);
    float* dp = &slot->DYR[t][32 * hf + 8 * g];
    *reinterpret_cast<float4*>(dp) = make_float4(fd[0] * ruk, fd[1] * ruk, fd[2] * ruk, fd[3] * ruk);
    *reinterpret_cast<float4*>(dp + 4) = make_float4(fd[4] * ruk, fd[5] * ruk, fd[6] * ruk, fd[7] * ruk);
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
  {
    uint32_t hi0, lo0, hi1, lo1;
    split2(N1[0], N1[1], hi0, lo0); split2(N1[2], N1[3], hi1, lo1);
    slot->N1[lane] = make_uint4(hi0, hi1, lo0, lo1);
    split2(N2[0], N2[1], hi0, lo0); split2(N2[2], N2[3], hi1, lo1);
    slot->N2[lane] = make_uint4(hi0, hi1, lo0, lo1);
  }
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
    slot->resets = (int)resets;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Two kinds of consumer wave, each with its share of G as 16x16 accumulator tiles, lane (n = lane%16, g = lane/16):
//   key wave q:   G[vt][i] = G[key 16q + n][value 16*vt + 4g + i]   (rows of its keys; B operand of contractions
//                 over values): gk, gw and the cotangent of the input state
//   value wave q: G[kt][i] = G[key 16*kt + 4g + i][value 16q + n]   (columns of its values; B operand of contractions
//                 over keys): gv
struct Consumer {
  f32x4_t G[4];
  float carry;         // key waves: running sum of the decay-gradient recursion, per key (same in a key's four lanes)
  int q, lane;
};

struct Pre {           // per-token scalars at (token 4g+i, key 16q+n), fetched one chunk ahead
  float er[4];
  uint16_t k[4];   // bf16 bits, widened where they are used: nothing waits for the loads before that
};

struct Cursor {
  const char *er, *k;          // fp32 workspace and bf16 input at (b, c0, h, 0)
  char *gk, *gv, *gw;          // bf16 outputs
  size_t tok_bytes;            // bytes between consecutive tokens in the bf16 arrays (twice that in the fp32 one)
  uint32_t voff;               // lane part of the address, in elements: (4g * H) * 64 + 16q + n
};

__device__ __forceinline__ void prefetch(Pre& p, const Cursor& cu, int nvalid, int g) {
  const size_t lo = (size_t)cu.voff;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float er = 0.f;
    uint16_t k = 0;
    if (nvalid == CK || 4 * g + i < nvalid) {      // the first test is uniform: no lane predicate but in a partial chunk
      er = *reinterpret_cast<const float*>(cu.er + lo * 4 + 2 * i * cu.tok_bytes);
      k = *reinterpret_cast<const uint16_t*>(cu.k + lo * 2 + i * cu.tok_bytes);
    }
    p.er[i] = er;
    p.k[i] = k;
  }
}

__device__ __forceinline__ void step_back(Cursor& cu) {
  const size_t d = CK * cu.tok_bytes;
  cu.er -= 2 * d; cu.k -= d;
  cu.gk -= d; cu.gv -= d; cu.gw -= d;
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

__device__ __forceinline__ void split_tiles(const f32x4_t (&G)[4], u32x4_t (&Gh)[2], u32x4_t (&Gl)[2]) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2_keep(G[2 * j][0], G[2 * j][1], hi, lo); Gh[j][0] = hi; Gl[j][0] = lo;
    split2_keep(G[2 * j][2], G[2 * j][3], hi, lo); Gh[j][1] = hi; Gl[j][1] = lo;
    split2_keep(G[2 * j + 1][0], G[2 * j + 1][1], hi, lo); Gh[j][2] = hi; Gl[j][2] = lo;
    split2_keep(G[2 * j + 1][2], G[2 * j + 1][3], hi, lo); Gh[j][3] = hi; Gl[j][3] = lo;
  }
}

// ---- key wave: E_t (G_t v_t) per (token, key), the decay-gradient recursion, gk and gw
__device__ __forceinline__ void consume_keys(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                             const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap,
                                             const Pre& pre, Pre& pre_next, const Cursor& cu, const Cursor& cu_next,
                                             bool has_next) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const u32x4_t rq = *reinterpret_cast<const u32x4_t*>(&slot->RQ[q][lane]);   // B operand: rq of tokens 4g.., hi | lo
  const bool keep_end = slot->keep_end != 0;
  const uint32_t resets = (uint32_t)slot->resets;
  {  // the cotangent of the chunk-end state, decayed over the chunk: per key = per lane
    const float gm = slot->gamma[16 * q + n];
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) { C.G[vt][0] *= gm; C.G[vt][1] *= gm; C.G[vt][2] *= gm; C.G[vt][3] *= gm; }
  }
  u32x4_t Gh[2], Gl[2];
  split_tiles(C.G, Gh, Gl);
  f32x4_t PK = zero4, PK2 = zero4;   // [token 4g+i][key 16q+n]: E_t . (G_t v_t)
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t vv = *reinterpret_cast<const u32x4_t*>(&slot->V[n][32 * j + 8 * g]);
    PK = mfma(vv, Gh[j], PK);
    PK2 = mfma(vv, Gl[j], PK2);
  }
  {
    const u32x4_t n1 = *reinterpret_cast<const u32x4_t*>(&slot->N1[lane]);
    const u32x4_t n1hh = {n1[0], n1[1], n1[0], n1[1]}, n1l0 = {n1[2], n1[3], 0u, 0u}, rq0 = {rq[0], rq[1], 0u, 0u};
    PK = mfma(n1hh, rq, PK);                         // N1_hi (rq_hi + rq_lo)
    PK2 = mfma(n1l0, rq0, PK2);                      // N1_lo rq_hi
  }
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
#pragma unroll
    for (int x = 0; x < 4; ++x) C.G[x] = zero4;
  }
  // the cotangent of the returned state enters at token length-1 (one chunk per sequence)
  float eI = 0.f;
  int snap_tok = -1;
  if (is_snap) {
    snap_tok = slot->snap;
    eI = A.eI[((size_t)b * A.H + h) * 64 + 16 * q + n];
    const bool keep = slot->keep_snap != 0;
    const float sg1 = snapslot->gamma[16 * q + n];
    f32x4_t T1[4];
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      T1[vt] = load_state4(A.gs_out, A.st_f32, state_el(A, b, h, 16 * q + n, 16 * vt + 4 * g)) * sg1;
      if (keep) C.G[vt] += T1[vt];
    }
    u32x4_t T1h[2], T1l[2];
    split_tiles(T1, T1h, T1l);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const u32x4_t vv = *reinterpret_cast<const u32x4_t*>(&snapslot->V[n][32 * j + 8 * g]);
      PK = mfma(vv, T1h[j], PK);
      PK2 = mfma(vv, T1l[j], PK2);
    }
  }
  // cotangent update: G <- Gh + sum_s rq_s dy_s^T over the tokens before the first reset
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const uint2 dd = slot->DYtU[vt][lane];
    const u32x4_t A1 = {dd.x, dd.y, dd.x, dd.y};               // rows = values of tile vt, k-slots = dy of tokens, twice
    C.G[vt] = mfma(A1, rq, C.G[vt]);
  }
  // per-token results: register i is token 4g+i, lanes n = 16 consecutive keys
  float gvk[4], z[4], cy[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    gvk[i] = (PK[i] + PK2[i]) * slot->Einv[tok][16 * q + n];          // (G_t v_t)[key]
    z[i] = pre.er[i] + (tok == snap_tok ? eI : 0.f) - bf16_to_f32(pre.k[i]) * gvk[i];
  }
  // carry_t = reset_t ? 0 : carry_{t+1} + z_t, from token 15 down
  if (resets == 0) {
    const float s3 = z[3], s2 = z[2] + s3, s1 = z[1] + s2, s0 = z[0] + s1;
    const float t1 = __shfl_down(s0, 16, 64), t2 = __shfl_down(s0, 32, 64), t3 = __shfl_down(s0, 48, 64);
    const float after = C.carry + (g < 3 ? t1 : 0.f) + (g < 2 ? t2 : 0.f) + (g < 1 ? t3 : 0.f);
    cy[3] = s3 + after; cy[2] = s2 + after; cy[1] = s1 + after; cy[0] = s0 + after;
    C.carry = __shfl(cy[0], n, 64);
  } else {
    float cin = C.carry;
#pragma unroll
    for (int tok = 15; tok >= 0; --tok) {
      const float zv = __shfl(z[tok & 3], n + 16 * (tok >> 2), 64);
      cin = ((resets >> tok) & 1u) ? 0.f : cin + zv;
      if (g == (tok >> 2)) cy[tok & 3] = cin;
    }
    C.carry = cin;
  }
  uint16_t ok[4], ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    ok[i] = f32_to_bf16(slot->RUC[tok][16 * q + n] + gvk[i]);
    ow[i] = f32_to_bf16(((resets >> tok) & 1u) ? 0.f : cy[i] - pre.er[i]);
  }
  // The next chunk's per-token scalars are requested after the last read of this chunk's (into a second set of
  // registers: the caller alternates two sets, so nothing is copied) and before this chunk's stores.  Loads and
  // stores share one in-order counter, a wait for a load also waits for every older store, and the compiler drains
  // the counter completely whenever both kinds are in flight: in this order everything in flight at the next wait
  // is a whole chunk old.  The barriers keep the scheduler from moving the loads up or the stores above them.
  __builtin_amdgcn_sched_barrier(0);
  if (has_next) prefetch(pre_next, cu_next, CK, g);
  __builtin_amdgcn_sched_barrier(0);
  const size_t lo = (size_t)cu.voff;
  auto put = [&](int i, bool full) {
    if (full || 4 * g + i < nvalid) {
      *reinterpret_cast<uint16_t*>(cu.gk + lo * 2 + i * cu.tok_bytes) = ok[i];
      *reinterpret_cast<uint16_t*>(cu.gw + lo * 2 + i * cu.tok_bytes) = ow[i];
    }
  };
  if (nvalid == CK) {      // every chunk but a partial last one: no per-lane predicates
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, true);
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, false);
  }
}

// ---- value wave: G_t^T k_t per (token, value) and gv
__device__ __forceinline__ void consume_values(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                               const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap,
                                               const Cursor& cu) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint2 dq = slot->DYt[q][lane];
  const u32x4_t dyq = {dq.x, dq.y, dq.x, dq.y};                                // B operand: dy of tokens 4g.., twice
  const bool keep_end = slot->keep_end != 0;
#pragma unroll
  for (int kt = 0; kt < 4; ++kt) {   // the cotangent of the chunk-end state, decayed over the chunk: per key = per register
    const float4 g4 = *reinterpret_cast<const float4*>(&slot->gamma[16 * kt + 4 * g]);
    C.G[kt][0] *= g4.x; C.G[kt][1] *= g4.y; C.G[kt][2] *= g4.z; C.G[kt][3] *= g4.w;
  }
  u32x4_t Gh[2], Gl[2];
  split_tiles(C.G, Gh, Gl);
  f32x4_t PV = zero4, PV2 = zero4;   // [token 4g+i][value 16q+n]: G_t^T k_t
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t kh = *reinterpret_cast<const u32x4_t*>(&slot->KH[0][n][32 * j + 8 * g]);
    const u32x4_t kl = *reinterpret_cast<const u32x4_t*>(&slot->KH[1][n][32 * j + 8 * g]);
    PV = mfma(kh, Gh[j], PV);
    PV2 = mfma(kh, Gl[j], PV2);
    PV = mfma(kl, Gh[j], PV);
  }
  {
    const u32x4_t n2 = *reinterpret_cast<const u32x4_t*>(&slot->N2[lane]);
    PV2 = mfma(n2, dyq, PV2);                        // (N2_hi + N2_lo) dy
  }
  if (!keep_end) {
#pragma unroll
    for (int x = 0; x < 4; ++x) C.G[x] = zero4;
  }
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
    f32x4_t T2[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * kt + 4 * g]);
      const float s4[4] = {sg.x, sg.y, sg.z, sg.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
        T2[kt][i] = ld_state_el(A.gs_out, A.st_f32, state_el(A, b, h, 16 * kt + 4 * g + i, 16 * q + n)) * s4[i];
      if (keep) C.G[kt] += T2[kt];
    }
    u32x4_t T2h[2], T2l[2];
    split_tiles(T2, T2h, T2l);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const u32x4_t kh = *reinterpret_cast<const u32x4_t*>(&snapslot->KH[0][n][32 * j + 8 * g]);
      const u32x4_t kl = *reinterpret_cast<const u32x4_t*>(&snapslot->KH[1][n][32 * j + 8 * g]);
      PV = mfma(kh, T2h[j], PV);
      PV2 = mfma(kh, T2l[j], PV2);
      PV = mfma(kl, T2h[j], PV);
    }
  }
  {
    const uint2 du = slot->DYtU[q][lane];
    const u32x4_t dyu = {du.x, du.y, du.x, du.y};
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const u32x4_t ra = *reinterpret_cast<const u32x4_t*>(&slot->RQ[kt][lane]);   // rows = keys of tile kt, hi | lo
      C.G[kt] = mfma(ra, dyu, C.G[kt]);
    }
  }
  uint16_t ov[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) ov[i] = f32_to_bf16(slot->DYR[4 * g + i][16 * q + n] + PV[i] + PV2[i]);
  const size_t lo = (size_t)cu.voff;
  auto put = [&](int i, bool full) {
    if (full || 4 * g + i < nvalid) *reinterpret_cast<uint16_t*>(cu.gv + lo * 2 + i * cu.tok_bytes) = ov[i];
  };
  if (nvalid == CK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, true);
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, false);
  }
}

}  // namespace

// Step j handles chunk nch-1-j in slot j % RING; hand-shake as in the forward kernels.  Waves 0-3 are the key waves,
// 4-7 the value waves, the rest producers: every SIMD runs one wave of each kind.
__global__ __launch_bounds__(64 * (NCONS_R + NPROD)) void wkv6_chunk_bwd_r_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Sync8* sy = reinterpret_cast<Sync8*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int nch = (int)((A.T + CK - 1) / CK);
  const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
  const bool inject = A.gs_out != nullptr && !q2drop;   // a cotangent of the returned state exists
  if (threadIdx.x < sizeof(Sync8) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  if (wave < NCONS_R) {
    __builtin_amdgcn_s_setprio(3);
    const bool keys = wave < 4;
    Consumer C;
    C.q = wave & 3;
    C.lane = lane;
    C.carry = 0.f;
    const int n = lane & 15, g = lane >> 4;
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 4; ++x) C.G[x] = zero4;
    Cursor cu;
    cu.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T + (size_t)(nch - 1) * CK) * A.H + h) * 64;
    cu.er = reinterpret_cast<const char*>(A.er) + el0 * 4;
    cu.k = reinterpret_cast<const char*>(A.k) + el0 * 2;
    cu.gk = reinterpret_cast<char*>(A.gk) + el0 * 2;
    cu.gv = reinterpret_cast<char*>(A.gv) + el0 * 2;
    cu.gw = reinterpret_cast<char*>(A.gw) + el0 * 2;
    cu.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * C.q + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    const int tail = (A.T % CK == 0) ? CK : (int)(A.T % CK);
    if (keys) {
      Pre pre_a, pre_b;
      if (nch > 0) prefetch(pre_a, cu, tail, g);
      auto step = [&](int j, const Pre& pre, Pre& pre_next) -> bool {
        const int c = nch - 1 - j;
        const int nvalid = (j == 0) ? tail : CK;
        const int si = j % RING;
        Cursor nxt = cu;
        step_back(nxt);
        if (!wait_ready(sy, si, j + 1)) return false;
        consume_keys(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, pre, pre_next, cu, nxt, j + 1 < nch);
        cu = nxt;
        if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        return true;
      };
      for (int j = 0; j < nch; j += 2) {      // two steps per turn: the prefetch registers alternate
        if (!step(j, pre_a, pre_b)) break;
        if (j + 1 < nch && !step(j + 1, pre_b, pre_a)) break;
      }
      // cotangent of the input state; with length == 0 the returned state is the input state itself
      const bool pass = L == 0 && inject;
#pragma unroll
      for (int vt = 0; vt < 4; ++vt) {
        const size_t off = state_el(A, b, h, 16 * C.q + n, 16 * vt + 4 * g);
        f32x4_t gsv = C.G[vt];
        if (pass) gsv += load_state4(A.gs_out, A.st_f32, off);
        if (A.st_f32) *reinterpret_cast<float4*>(reinterpret_cast<float*>(A.gs) + off) = make_float4(gsv[0], gsv[1], gsv[2], gsv[3]);
        else *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(A.gs) + off) = make_uint2(pack_rn(gsv[0], gsv[1]), pack_rn(gsv[2], gsv[3]));
      }
    } else {
      for (int j = 0; j < nch; ++j) {
        const int c = nch - 1 - j;
        const int nvalid = (j == 0) ? tail : CK;
        const int si = j % RING;
        if (!wait_ready(sy, si, j + 1)) break;
        consume_values(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, cu);
        step_back(cu);
        if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  } else {
    const int p = wave - NCONS_R;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
    {
      const char* up = reinterpret_cast<const char*>(A.u) + ((size_t)h * 64 + 8 * (lane >> 4)) * 2;
      P.u[0] = *reinterpret_cast<const uint4*>(up);
      P.u[1] = *reinterpret_cast<const uint4*>(up + 64);
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
      Slot* slot = &slots[si];
      if (j >= RING && !wait_consumed(sy, si, j - RING + 1, lane)) break;
      produce(P, raw, F, slot, snapslot, events_word(A.status));
      if (j + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)(c - NPROD) * CK, lane);
        load_raw(raw, A, b, h, (int64_t)(c - NPROD) * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && j + 1 == nch) break;
      if (lane == 0) __hip_atomic_store(&sy->ready[si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gk, 2, b, h, A.T, A.H);
    poison_token_rows(A.gv, 2, b, h, A.T, A.H);
    poison_token_rows(A.gw, 2, b, h, A.T, A.H);
    poison_state(A.gs, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv6_chunk_bwd_r(const Wkv6Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync8);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_chunk_bwd_r_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_chunk_bwd_r_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS_R + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
