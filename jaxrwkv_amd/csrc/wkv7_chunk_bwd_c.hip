// WKV7 backward, reverse sweep C on the matrix cores (bf16 I/O, gfx950): gk, gb and the decay gradient gw.
//
// With dsa_t known from sweep A the cotangent G = dL/dS obeys a linear recurrence, carried from the last token
// down (G~_t the cotangent of S_t; S[i][j] = value row i, key col j):
//     G~_t = dy_t r_t^T + G~_{t+1} diag(d_{t+1}) + dsa_{t+1} a_{t+1}^T ;   dk_t = G~_t^T v_t ;   db_t = G~_t^T sa_t
// A chunk of C = 16 tokens leaving with G_C: E_t = prod_{s<=t} d_s, Ee_t = E_{t-1}, qt_s = r_s.E_s, at_s = a_s.Ee_s,
// Gh = G_C diag(E_C):
//     G~_t diag(E_t) = Gh + sum_{s>=t} dy_s qt_s^T + sum_{s>t} dsa_s at_s^T
//     dk_t = (1/E_t) . ( Gh^T v_t  + sum_{s>t} (dsa_s.v_t)  at_s + sum_{s>=t} (dy_s.v_t)  qt_s )
//     db_t = (1/E_t) . ( Gh^T sa_t + sum_{s>t} (dsa_s.sa_t) at_s + sum_{s>=t} (dy_s.sa_t) qt_s )
//     G_prev = Gh + DSA^T At + DY^T Qt
// i.e. the computation of sweep B run backwards with the operands exchanged (dy <-> v, dsa <-> sa, Bh <-> At,
// Kh <-> Qt) and the decay applied before the update.  The decay gradient needs <G_t, S'_t> per key; as in the
// sequential sweep it comes from the running sum
//     carry_t = reset_t ? 0 : carry_{t+1} + e3_t + e2_t - k_t.dk_t - b_t.db_t ;   dw_t = (carry_t - e2_t) * (-exp(w_t))
// with e2 = a.da and e3 = r.dr (+ <dS_out, S> at token length-1).  In terms of c_t = carry_t - e2_t (c_t = 0 at a
// reset) this is c_t = reset_t ? 0 : c_{t+1} + f_t - k_t.dk_t - b_t.db_t, dw_t = c_t * (-exp(w_t)), with the one
// vector f_t = e3_t + (reset_{t+1} ? 0 : e2_{t+1}) per token that sweep B leaves.
//
// Work split as in sweep B: 4 consumer waves hold G split by key columns (value x key accumulator tiles reused
// as B operands), 4 producer waves prepare the state-independent operands into a ring of LDS slots; bounded-poll
// hand-shake.  new_starts inside a chunk restart the cumulative decay and mask the tiles; the chunk holding token
// length-1 adds the cotangent of the returned state through a second, masked set of row operands.
// Range: as in the forward kernel, a chunk's total log decay per channel is capped at -80.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns steps p, p + NPROD, ...
constexpr int RING = 3;           // slots in flight (a slot is 40 KB)
constexpr int ES = 68;            // row stride (floats) of the fp32 [token][key] array: conflict-free column reads

// "lane-indexed" arrays hold, for every lane of the producer, the bytes the same lane of a consumer loads:
// accumulator-layout registers (column lane%16, rows 4*(lane/16)..+3) packed to bf16, hi pair then lo pair.
struct __attribute__((aligned(16))) Slot {
  // v rows and sa rows (hi, lo), [token][RS]: within a row, the 16-byte vector (j, g) at element 32j + 8g holds
  // values 32j+4g..+3 followed by values 32j+16+4g..+3, the value order of the consumers' tiles.  Rows that the
  // cotangent of later chunks does not reach are zero.
  uint16_t V[CK][RS];
  uint16_t SA[2][CK][RS];
  uint4 BT[2][4][64];          // [at|qt][key tile]: (a_s.Ee_s)^T, (r_s.E_s)^T hi,lo, lane-indexed
  uint4 DSAt[4][64];           // dsa^T per value tile: hi,lo, lane-indexed; tokens masked for the chunk-start cotangent
  uint2 DYt[4][64];            // dy^T per value tile, lane-indexed; masked likewise
  uint4 Nk[2][64];             // [hi|lo] of {dsa_s.v_t (s > t), dy_s.v_t (s >= t)}, lane-indexed: A operand row t, k-slots s
  uint4 Nb[2][64];             // [hi|lo] of {dsa_s.sa_t (s > t), dy_s.sa_t (s >= t)}
  float Einv[CK][ES];          // 1/E_t per key
  // What the decay-gradient recursion reads per token and key, brought in by the producers with the chunk's other
  // operands: the k, b and w rows as they are in memory (bf16, natural key order) and the chunk's four records of
  // the fp32 workspace that the forward sweep left (f_record), one per consumer wave.  Fetched by the consumers
  // themselves, one chunk ahead, these values arrived late (behind the producers' deep queues a load takes several
  // chunk times), and where the compiler put the waits depended on details of the source.  The slot grows to 40 KB
  // and the ring shrinks from five slots to three; measured on MI355X the sweep takes the same time when the
  // outputs sit at their own address phases and 8 % less when every array starts on a 2 MiB boundary.
  uint16_t KBW[3][CK][RS];
  float4 F[NCONS][64];
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the cotangent of later chunks reaches the chunk start (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int resets;                  // bit t: new_starts of in-chunk token t
};
struct __attribute__((aligned(16))) SnapSlot {
  uint16_t V[CK][RS];          // row operands masked to the tokens that the cotangent entering at length-1 reaches
  uint16_t SA[2][CK][RS];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and, of every 64-vector, the elements {8g..8g+7} u {32+8g..32+8g+7}.
struct Raw {
  uint4 w[2], r[2], a[2], v[2], dy[2];
  uint4 sa[2];             // the forward residual, fp16
  uint4 dsa[2];            // sweep A's workspace: 16-bit fixed point, scaled per chunk and value tile (chunk_common.h)
  int4 dsk;                // k of the chunk's four value tiles
  uint4 k[2], b[2];        // passed on to the consumers as they are
  float4 f[NCONS];         // lane l: entry l of each consumer wave's record of this chunk
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  {
    const int nch = (int)((A.T + CK - 1) / CK);
    const float4* rec = reinterpret_cast<const float4*>(A.e2 + f_record(b, h, A.H, nch, (int)(c0 / CK), 0));
#pragma unroll
    for (int q = 0; q < NCONS; ++q) x.f[q] = rec[64 * q + lane];
  }
  x.dsk = *reinterpret_cast<const int4*>(dsa_scales(A.e3, b, h, A.H, (int)((A.T + CK - 1) / CK), (int)(c0 / CK)));
  if (c0 + t < A.T) {
    const size_t el = (((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g;
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + el * 2);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + el * 2 + 64);
    };
    ld(A.w, x.w); ld(A.r, x.r); ld(A.a, x.a); ld(A.v, x.v); ld(A.gy, x.dy);
    ld(A.sa_in, x.sa); ld(A.dsa, x.dsa);
    ld(A.k, x.k); ld(A.b, x.b);
  } else {
    const uint4 z = make_uint4(0, 0, 0, 0);
    x.w[0] = x.w[1] = x.r[0] = x.r[1] = x.a[0] = x.a[1] = x.v[0] = x.v[1] = x.dy[0] = x.dy[1] = z;
    x.sa[0] = x.sa[1] = x.k[0] = x.k[1] = x.b[0] = x.b[1] = z;
    x.dsa[0] = x.dsa[1] = z;
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // MFMA-as-transposer selection operands
};

__device__ __forceinline__ void split8(const float4 lo4, const float4 hi4, u32x4_t& h, u32x4_t& l) {
  uint32_t a, b;
  split2(lo4.x, lo4.y, a, b); h[0] = a; l[0] = b;
  split2(lo4.z, lo4.w, a, b); h[1] = a; l[1] = b;
  split2(hi4.x, hi4.y, a, b); h[2] = a; l[2] = b;
  split2(hi4.z, hi4.w, a, b); h[3] = a; l[3] = b;
}

// the same for eight fp16 values (11 significant bits: the pair is exact)
__device__ __forceinline__ void split8h(const uint4 raw, u32x4_t& h, u32x4_t& l) {
  typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
  const h8_t x = __builtin_bit_cast(h8_t, raw);
  uint32_t a, b;
  split2((float)x[0], (float)x[1], a, b); h[0] = a; l[0] = b;
  split2((float)x[2], (float)x[3], a, b); h[1] = a; l[1] = b;
  split2((float)x[4], (float)x[5], a, b); h[2] = a; l[2] = b;
  split2((float)x[6], (float)x[7], a, b); h[3] = a; l[3] = b;
}

__device__ __forceinline__ void produce(const Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  int lastseg = 0, seg_src = 0;
  bool row_keep = true, restart = false, drop_dy = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
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
  auto masked_pack = [&](const f32x4_t d, uint32_t keep) {
    const uint32_t bits = keep >> (4 * g);
    const float d0 = (bits & 1u) ? d[0] : 0.f, d1 = (bits & 2u) ? d[1] : 0.f;
    const float d2 = (bits & 4u) ? d[2] : 0.f, d3 = (bits & 8u) ? d[3] : 0.f;
    return make_uint2(pack_exact(d0, d1), pack_exact(d2, d3));
  };
  auto plain_pack = [&](const f32x4_t d) { return make_uint2(pack_exact(d[0], d[1]), pack_exact(d[2], d[3])); };
  auto join = [&](const uint2 hi, const uint2 lo) { return make_uint4(hi.x, hi.y, lo.x, lo.y); };

  // the consumers' per-token scalars, as loaded (rows beyond the sequence are zero)
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    *reinterpret_cast<uint4*>(&slot->KBW[0][t][32 * hf + 8 * g]) = x.k[hf];
    *reinterpret_cast<uint4*>(&slot->KBW[1][t][32 * hf + 8 * g]) = x.b[hf];
    *reinterpret_cast<uint4*>(&slot->KBW[2][t][32 * hf + 8 * g]) = x.w[hf];
  }
#pragma unroll
  for (int q = 0; q < NCONS; ++q) slot->F[q][lane] = x.f[q];
  // Gram tiles over the values, accumulator layout [row m = s][column n = t]
  f32x4_t Nsv = zero4, Nyv = zero4, Nss = zero4, Nys = zero4;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // first 8-byte piece of this lane in a permuted row
    auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
      *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
      *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
    };
    // ================= keys of this half: decay scan, (a.Ee)^T, (r.E)^T, 1/E rows
    {
      float E[8];
      {
        float fw[8];
        unpack8(x.w[hf], fw);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float l2 = fmaxf(-exp2_fast(fw[e] * LOG2E) * LOG2E, MIN_STEP_L2);
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
      u32x4_t at_h, at_l, qt_h, qt_l;
      float Einv[8];
      {
        float fr[8], fa[8], Ee[8];
        unpack8(x.r[hf], fr); unpack8(x.a[hf], fa);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = fmaxf(E[e], MIN_CUM_L2);
          E[e] = exp2_fast(l2);
          Einv[e] = exp2_fast(-l2);
          // exclusive: value of the previous token; 1 for the first token of the chunk.  At a reset token the
          // value belongs to the previous segment, but every product it enters is masked out.
          Ee[e] = row_prev(E[e], 1.0f);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = 2 * j;
          uint32_t hi, lo;
          split2(fa[e] * Ee[e], fa[e + 1] * Ee[e + 1], hi, lo); at_h[j] = hi; at_l[j] = lo;
          split2(fr[e] * E[e], fr[e + 1] * E[e + 1], hi, lo); qt_h[j] = hi; qt_l[j] = lo;
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
      // transposes by MFMA: D (lane = key, registers = 4 consecutive tokens) is the B-operand layout of the update
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const u32x4_t sel = P.sel[x2];
        const f32x4_t dah = mfma(at_h, sel, zero4), dal = mfma(at_l, sel, zero4);
        const f32x4_t dqh = mfma(qt_h, sel, zero4), dql = mfma(qt_l, sel, zero4);
        slot->BT[0][tile][lane] = join(plain_pack(dah), plain_pack(dal));
        slot->BT[1][tile][lane] = join(plain_pack(dqh), plain_pack(dql));
      }
    }
    // ================= values of this half: dy^T, dsa^T, v and sa rows, partial Gram sums
    {
      const uint4 vr = x.v[hf];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w};
      uint4 dr = x.dy[hf];
      if (drop_dy) dr = make_uint4(0, 0, 0, 0);
      const u32x4_t dyop = {dr.x, dr.y, dr.z, dr.w};
      u32x4_t sa_h, sa_l, ds_h, ds_l;
      split8h(x.sa[hf], sa_h, sa_l);
      {
        float4 d_lo, d_hi;
        const int kq = hf == 0 ? ((g >> 1) ? x.dsk.y : x.dsk.x) : ((g >> 1) ? x.dsk.w : x.dsk.z);
        unpack_dsa8(x.dsa[hf], kq, d_lo, d_hi);
        split8(d_lo, d_hi, ds_h, ds_l);
      }
      put(slot->V[t], vop, row_keep);
      put(slot->SA[0][t], sa_h, row_keep);
      put(slot->SA[1][t], sa_l, row_keep);
      if (F.snap >= 0) {
        const bool sk = (keep_snap >> t) & 1u;
        put(snap->V[t], vop, sk);
        put(snap->SA[0][t], sa_h, sk);
        put(snap->SA[1][t], sa_l, sk);
      }
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const u32x4_t sel = P.sel[x2];
        const f32x4_t dd = mfma(dyop, sel, zero4), dsh = mfma(ds_h, sel, zero4), dsl = mfma(ds_l, sel, zero4);
        if (keep_upd == 0xffffu) {
          slot->DYt[tile][lane] = plain_pack(dd);
          slot->DSAt[tile][lane] = join(plain_pack(dsh), plain_pack(dsl));
        } else {
          slot->DYt[tile][lane] = masked_pack(dd, keep_upd);
          slot->DSAt[tile][lane] = join(masked_pack(dsh, keep_upd), masked_pack(dsl, keep_upd));
        }
      }
      Nsv = mfma(ds_h, vop, Nsv); Nsv = mfma(ds_l, vop, Nsv);         // [s][t] = dsa_s . v_t
      Nyv = mfma(dyop, vop, Nyv);                                     // [s][t] = dy_s . v_t
      Nss = mfma(ds_h, sa_h, Nss); Nss = mfma(ds_h, sa_l, Nss); Nss = mfma(ds_l, sa_h, Nss);   // dsa_s . sa_t
      Nys = mfma(dyop, sa_h, Nys); Nys = mfma(dyop, sa_l, Nys);       // dy_s . sa_t
    }
  }
  // ---- triangular masks (rows s, column t = this lane's token)
  const int n = t;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool gt = m > n, ge = m >= n;
    if (slow) {
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      gt = gt && same; ge = ge && same;
    }
    Nsv[i] = gt ? Nsv[i] : 0.f;
    Nss[i] = gt ? Nss[i] : 0.f;
    Nyv[i] = ge ? Nyv[i] : 0.f;
    Nys[i] = ge ? Nys[i] : 0.f;
  }
  {
    uint32_t a0, b0, a1, b1, c0, d0, c1, d1;
    split2(Nsv[0], Nsv[1], a0, b0); split2(Nsv[2], Nsv[3], a1, b1);
    split2(Nyv[0], Nyv[1], c0, d0); split2(Nyv[2], Nyv[3], c1, d1);
    slot->Nk[0][lane] = make_uint4(a0, a1, c0, c1);
    slot->Nk[1][lane] = make_uint4(b0, b1, d0, d1);
    split2(Nss[0], Nss[1], a0, b0); split2(Nss[2], Nss[3], a1, b1);
    split2(Nys[0], Nys[1], c0, d0); split2(Nys[2], Nys[3], c1, d1);
    slot->Nb[0][lane] = make_uint4(a0, a1, c0, c1);
    slot->Nb[1][lane] = make_uint4(b0, b1, d0, d1);
  }
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
  int q, lane;
};

struct Cursor {
  char *gk, *gb, *gw;          // bf16 outputs at (b, c0, h, 0)
  size_t tok_bytes;            // bytes between consecutive tokens in the bf16 arrays (twice that in the fp32 ones)
  uint32_t voff;               // lane part of the address, in elements: (4g * H) * 64 + key
};

__device__ __forceinline__ void step_back(Cursor& cu) {
  const size_t d = CK * cu.tok_bytes;
  cu.gk -= d; cu.gb -= d; cu.gw -= d;
}

__device__ __forceinline__ size_t state_el(const Wkv7Args& A, int64_t b, int64_t h, int value, int key) {
  return (((size_t)b * A.H + h) * 64 + value) * 64 + key;
}
__device__ __forceinline__ float ld_state_el(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap,
                                        const Cursor& cu) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // B operands of the token contractions: (a.Ee, r.E) of tokens 4g..4g+3 at this wave's keys
  const u32x4_t ta = *reinterpret_cast<const u32x4_t*>(&slot->BT[0][q][lane]);
  const u32x4_t tq = *reinterpret_cast<const u32x4_t*>(&slot->BT[1][q][lane]);
  const u32x4_t Bh = {ta[0], ta[1], tq[0], tq[1]}, Bl = {ta[2], ta[3], tq[2], tq[3]};
  const bool keep_end = slot->keep_end != 0;
  const uint32_t resets = (uint32_t)slot->resets;
  // the cotangent of the chunk-end state, decayed over the chunk (per key = per lane)
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) { C.G[vt][0] *= gm; C.G[vt][1] *= gm; C.G[vt][2] *= gm; C.G[vt][3] *= gm; }
  // B operands from the cotangent: MFMA j contracts over the values of tiles 2j and 2j+1
  u32x4_t Gh[2], Gl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2_keep(C.G[2 * j][0], C.G[2 * j][1], hi, lo); Gh[j][0] = hi; Gl[j][0] = lo;
    split2_keep(C.G[2 * j][2], C.G[2 * j][3], hi, lo); Gh[j][1] = hi; Gl[j][1] = lo;
    split2_keep(C.G[2 * j + 1][0], C.G[2 * j + 1][1], hi, lo); Gh[j][2] = hi; Gl[j][2] = lo;
    split2_keep(C.G[2 * j + 1][2], C.G[2 * j + 1][3], hi, lo); Gh[j][3] = hi; Gl[j][3] = lo;
  }
  f32x4_t DK = zero4, DB = zero4;   // [token 4g+i][key n]
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t vv = *reinterpret_cast<const u32x4_t*>(&slot->V[n][32 * j + 8 * g]);
    const u32x4_t sh = *reinterpret_cast<const u32x4_t*>(&slot->SA[0][n][32 * j + 8 * g]);
    const u32x4_t sl = *reinterpret_cast<const u32x4_t*>(&slot->SA[1][n][32 * j + 8 * g]);
    DK = mfma(vv, Gh[j], DK); DB = mfma(sh, Gh[j], DB);
    DK = mfma(vv, Gl[j], DK); DB = mfma(sh, Gl[j], DB);
    DB = mfma(sl, Gh[j], DB);
  }
  {
    const u32x4_t nkh = *reinterpret_cast<const u32x4_t*>(&slot->Nk[0][lane]);
    const u32x4_t nkl = *reinterpret_cast<const u32x4_t*>(&slot->Nk[1][lane]);
    const u32x4_t nbh = *reinterpret_cast<const u32x4_t*>(&slot->Nb[0][lane]);
    const u32x4_t nbl = *reinterpret_cast<const u32x4_t*>(&slot->Nb[1][lane]);
    DK = mfma(nkh, Bh, DK); DB = mfma(nbh, Bh, DB);
    DK = mfma(nkh, Bl, DK); DB = mfma(nbh, Bl, DB);
    DK = mfma(nkl, Bh, DK); DB = mfma(nbl, Bh, DB);
  }
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.G[vt] = zero4;
  }
  // the cotangent of the returned state enters at token length-1 (one chunk per sequence)
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t gh, gl;
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int vt = 2 * j + x2;
        f32x4_t gs;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          gs[i] = ld_state_el(A.gs_out, A.st_f32, state_el(A, b, h, 16 * vt + 4 * g + i, 16 * q + n)) * sg;
        if (keep) C.G[vt] += gs;
        uint32_t hi, lo;
        split2(gs[0], gs[1], hi, lo); gh[2 * x2] = hi; gl[2 * x2] = lo;
        split2(gs[2], gs[3], hi, lo); gh[2 * x2 + 1] = hi; gl[2 * x2 + 1] = lo;
      }
      const u32x4_t vv = *reinterpret_cast<const u32x4_t*>(&snapslot->V[n][32 * j + 8 * g]);
      const u32x4_t sh = *reinterpret_cast<const u32x4_t*>(&snapslot->SA[0][n][32 * j + 8 * g]);
      const u32x4_t sl = *reinterpret_cast<const u32x4_t*>(&snapslot->SA[1][n][32 * j + 8 * g]);
      DK = mfma(vv, gh, DK); DB = mfma(sh, gh, DB);
      DK = mfma(vv, gl, DK); DB = mfma(sh, gl, DB);
      DB = mfma(sl, gh, DB);
    }
  }
  // cotangent update: G <- Gh + DSA^T At + DY^T Qt
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const uint4 st = slot->DSAt[vt][lane];
    const uint2 dd = slot->DYt[vt][lane];
    const u32x4_t A1 = {st.x, st.y, dd.x, dd.y}, A3 = {st.z, st.w, 0u, 0u};
    f32x4_t acc = C.G[vt];
    acc = mfma(A1, Bh, acc);
    acc = mfma(A1, Bl, acc);
    acc = mfma(A3, Bh, acc);
    C.G[vt] = acc;
  }
  // per-token results: register i is token 4g+i, lanes n = 16 consecutive keys
  float dk[4], db[4], z[4], cy[4], nej[4];
  const float4 fr = slot->F[q][lane];
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
    const float kk = bf16_to_f32(slot->KBW[0][4 * g + i][16 * q + n]), bb = bf16_to_f32(slot->KBW[1][4 * g + i][16 * q + n]);
    z[i] = fv[i] - kk * dk[i] - bb * db[i];
    nej[i] = -__expf(bf16_to_f32(slot->KBW[2][4 * g + i][16 * q + n]));
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
  uint16_t ok[4], ob[4], ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ok[i] = f32_to_bf16(dk[i]); ob[i] = f32_to_bf16(db[i]); ow[i] = f32_to_bf16(cy[i] * nej[i]);
  }
  const rsrc_t rgk = make_rsrc(cu.gk), rgb = make_rsrc(cu.gb), rgw = make_rsrc(cu.gw);
  const int o2 = (int)(cu.voff * 2u), tokb = (int)cu.tok_bytes;
  auto put = [&](int i, bool full) {
    if (full || 4 * g + i < nvalid) {
      __builtin_amdgcn_raw_buffer_store_b16(ok[i], rgk, o2, i * tokb, 0);
      __builtin_amdgcn_raw_buffer_store_b16(ob[i], rgb, o2, i * tokb, 0);
      __builtin_amdgcn_raw_buffer_store_b16(ow[i], rgw, o2, i * tokb, 0);
    }
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

// Step j handles chunk nch-1-j in slot j % RING.  Producer p fills the slot once every consumer has released step
// j - RING, then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier
// step, so the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_chunk_bwd_c_kernel(Wkv7Args A) {
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

  if (wave < NCONS) {
    __builtin_amdgcn_s_setprio(3);
    Consumer C;
    C.q = wave;
    C.lane = lane;
    C.carry = 0.f;
    const int n = lane & 15, g = lane >> 4;
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.G[vt] = zero4;
    Cursor cu;
    cu.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T + (size_t)(nch - 1) * CK) * A.H + h) * 64;
    cu.gk = reinterpret_cast<char*>(A.gk) + el0 * 2;
    cu.gb = reinterpret_cast<char*>(A.gb) + el0 * 2;
    cu.gw = reinterpret_cast<char*>(A.gw) + el0 * 2;
    cu.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    const int tail = (A.T % CK == 0) ? CK : (int)(A.T % CK);
    for (int j = 0; j < nch; ++j) {
      const int c = nch - 1 - j;
      const int nvalid = (j == 0) ? tail : CK;
      const int si = j % RING;
      if (!wait_ready(sy, si, j + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, cu);
      step_back(cu);
      // every LDS read of slot si has returned: its data went into the MFMAs and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
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
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gk, 2, b, h, A.T, A.H);
    poison_token_rows(A.gb, 2, b, h, A.T, A.H);
    poison_token_rows(A.gw, 2, b, h, A.T, A.H);
  }
}

hipError_t launch_wkv7_chunk_bwd_c(const Wkv7Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_chunk_bwd_c_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_chunk_bwd_c_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
