// WKV7 backward, forward sweep B on the matrix cores (bf16 I/O, gfx950): gr, ga and the per-token workspace
// f_t = e3_t + e2_{t+1} (e2 = a.da, dropped when token t+1 starts a sequence; e3 = r.dr + <dS_out, S> at token
// length-1) that the decay-gradient recursion of sweep C consumes.
//
// With sa_t known from the forward pass the state obeys a linear recurrence (S[i][j] = value row i, key col j):
//     S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;   dr_t = S_t^T dy_t ;   da_t = S_{t-1}^T dsa_t
// A chunk of C = 16 tokens entering with S0: E_t = prod_{s<=t} d_s, Ee_t = E_{t-1}, bh_s = b_s/E_s, kh_s = k_s/E_s,
//     S_t = (S0 + sum_{s<=t} sa_s bh_s^T + v_s kh_s^T) diag(E_t)
//     dr_t = E_t  . ( S0^T dy_t  + sum_{s<=t} (sa_s.dy_t)  bh_s + (v_s.dy_t)  kh_s )
//     da_t = Ee_t . ( S0^T dsa_t + sum_{s<t}  (sa_s.dsa_t) bh_s + (v_s.dsa_t) kh_s )
//     S_C  = (S0 + SA^T Bh + V^T Kh) diag(E_C)
// The 16x16 Gram tiles contract over the 64 values.  All products run on v_mfma_f32_16x16x32_bf16 with fp32
// quantities split into a truncated-bf16 "hi" and a bf16 "lo" part (hi.hi + hi.lo + lo.hi); v and dy are bf16
// already.  The K = 32 slots of one MFMA hold two 16-token products side by side (the sa and the v term).
//
// Work split as in the chunked forward kernel: 4 consumer waves keep the state in accumulator registers, here
// split by key columns (wave q owns keys 16q..16q+15 for all 64 values, value x key tiles that are reused
// directly as B operands); 4 producer waves prepare everything that does not depend on the state (decay scan,
// scaled operands, transposes, Gram tiles) into a ring of LDS slots; bounded-poll hand-shake.
// new_starts inside a chunk restart the cumulative decay and mask the tiles; the chunk holding token length-1
// also evaluates <dS_out, S_{length-1}> with a second, masked set of update operands.
// Range: as in the forward kernel, a chunk's total log decay per channel is capped at -80.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 4;           // slots in flight (a slot is 34 KB)
constexpr int ES = 68;            // row stride (floats) of the fp32 [token][key] array: conflict-free column reads

// "lane-indexed" arrays hold, for every lane of the producer, the bytes the same lane of a consumer loads:
// accumulator-layout registers (column lane%16, rows 4*(lane/16)..+3) packed to bf16, hi pair then lo pair.
struct __attribute__((aligned(16))) Slot {
  // dy rows and dsa rows (hi, lo), [token][RS]: within a row, the 16-byte vector (j, g) at element 32j + 8g holds
  // values 32j+4g..+3 followed by values 32j+16+4g..+3, the value order of the consumers' state tiles.  Rows the
  // entering state does not reach are zero; dy rows whose y is a constant are zero.
  uint16_t DY[CK][RS];
  uint16_t DSA[2][CK][RS];
  uint4 BT[2][4][64];          // [bh|kh][key tile]: (b_s/E_s)^T hi,lo, lane-indexed
  uint4 SAt[4][64];            // sa^T per value tile: hi,lo, lane-indexed; tokens masked for the chunk-end state
  uint2 Vt[4][64];             // v^T per value tile, lane-indexed; masked likewise
  uint4 Ny[2][64];             // [hi|lo] of {sa_s.dy_t, v_s.dy_t} (s <= t), lane-indexed: A operand row t, k-slots s
  uint4 Ns[2][64];             // [hi|lo] of {sa_s.dsa_t, v_s.dsa_t} (s < t)
  float E[CK + 1][ES];         // row t+1 = E_t per key, row 0 = 1
  uint16_t RA[2][CK][RS];      // r and a rows (bf16, natural key order)
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to token length-1
  int ns;                      // bit t: new_starts of in-chunk token t; bit 16: of the first token of the next chunk
};
struct __attribute__((aligned(16))) SnapSlot {
  uint4 SAt[4][64];            // update operands with the tokens masked for the state at token length-1
  uint2 Vt[4][64];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and, of every 64-vector, the elements {8g..8g+7} u {32+8g..32+8g+7}.
struct Raw {
  uint4 w[2], k[2], b[2], r[2], a[2], v[2], dy[2];
  uint4 sa[2];             // the forward residual, fp16
  uint4 dsa[2];            // sweep A's workspace: 16-bit fixed point, scaled per chunk and value tile (chunk_common.h)
  int4 dsk;                // k of the chunk's four value tiles
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  x.dsk = *reinterpret_cast<const int4*>(dsa_scales(A.e3, b, h, A.H, (int)((A.T + CK - 1) / CK), (int)(c0 / CK)));
  if (c0 + t < A.T) {
    const size_t el = (((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g;
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + el * 2);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + el * 2 + 64);
    };
    ld(A.w, x.w); ld(A.k, x.k); ld(A.b, x.b); ld(A.r, x.r); ld(A.a, x.a); ld(A.v, x.v); ld(A.gy, x.dy);
    ld(A.sa_in, x.sa); ld(A.dsa, x.dsa);
  } else {
    const uint4 z = make_uint4(0, 0, 0, 0);
    x.w[0] = x.w[1] = x.k[0] = x.k[1] = x.b[0] = x.b[1] = x.r[0] = x.r[1] = z;
    x.a[0] = x.a[1] = x.v[0] = x.v[1] = x.dy[0] = x.dy[1] = z;
    x.sa[0] = x.sa[1] = z;
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
  bool s0_reaches = true, restart = false, drop_dy = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
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
      if (us) keep_snap &= ~((1u << (31 - __builtin_clz(us))) - 1u);
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

  // Gram tiles over the values, accumulator layout [row m = s][column n = t]
  f32x4_t Nys = zero4, Nyv = zero4, Nss = zero4, Nsv = zero4;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // first 8-byte piece of this lane in a permuted row
    auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
      *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
      *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
    };
    // ================= keys of this half: decay scan, (b/E)^T, (k/E)^T, E rows, r and a rows
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
      u32x4_t kh_h, kh_l, bh_h, bh_l;
      {
        float fk[8], fb[8], Einv[8];
        unpack8(x.k[hf], fk); unpack8(x.b[hf], fb);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = fmaxf(E[e], MIN_CUM_L2);
          E[e] = exp2_fast(l2);
          Einv[e] = exp2_fast(-l2);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = 2 * j;
          uint32_t hi, lo;
          split2(fk[e] * Einv[e], fk[e + 1] * Einv[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
          split2(fb[e] * Einv[e], fb[e + 1] * Einv[e + 1], hi, lo); bh_h[j] = hi; bh_l[j] = lo;
        }
      }
      {
        float* er = &slot->E[t + 1][32 * hf + 8 * g];
        *reinterpret_cast<float4*>(er) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(er + 4) = make_float4(E[4], E[5], E[6], E[7]);
        if (t == 0) {
          float* e1 = &slot->E[0][32 * hf + 8 * g];
          *reinterpret_cast<float4*>(e1) = make_float4(1.f, 1.f, 1.f, 1.f);
          *reinterpret_cast<float4*>(e1 + 4) = make_float4(1.f, 1.f, 1.f, 1.f);
        }
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
      *reinterpret_cast<uint4*>(&slot->RA[0][t][32 * hf + 8 * g]) = x.r[hf];
      *reinterpret_cast<uint4*>(&slot->RA[1][t][32 * hf + 8 * g]) = x.a[hf];
      // transposes by MFMA: D (lane = key, registers = 4 consecutive tokens) is the B-operand layout of the update
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const u32x4_t sel = P.sel[x2];
        const f32x4_t dbh = mfma(bh_h, sel, zero4), dbl = mfma(bh_l, sel, zero4);
        const f32x4_t dkh = mfma(kh_h, sel, zero4), dkl = mfma(kh_l, sel, zero4);
        slot->BT[0][tile][lane] = join(plain_pack(dbh), plain_pack(dbl));
        slot->BT[1][tile][lane] = join(plain_pack(dkh), plain_pack(dkl));
      }
    }
    // ================= values of this half: v^T, sa^T, dy and dsa rows, partial Gram sums
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
      put(slot->DY[t], dyop, s0_reaches);
      put(slot->DSA[0][t], ds_h, s0_reaches);
      put(slot->DSA[1][t], ds_l, s0_reaches);
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const u32x4_t sel = P.sel[x2];
        const f32x4_t dv = mfma(vop, sel, zero4), dsh = mfma(sa_h, sel, zero4), dsl = mfma(sa_l, sel, zero4);
        if (keep_upd == 0xffffu) {
          slot->Vt[tile][lane] = plain_pack(dv);
          slot->SAt[tile][lane] = join(plain_pack(dsh), plain_pack(dsl));
        } else {
          slot->Vt[tile][lane] = masked_pack(dv, keep_upd);
          slot->SAt[tile][lane] = join(masked_pack(dsh, keep_upd), masked_pack(dsl, keep_upd));
        }
        if (F.snap >= 0) {
          snap->Vt[tile][lane] = masked_pack(dv, keep_snap);
          snap->SAt[tile][lane] = join(masked_pack(dsh, keep_snap), masked_pack(dsl, keep_snap));
        }
      }
      Nys = mfma(sa_h, dyop, Nys); Nys = mfma(sa_l, dyop, Nys);       // [s][t] = sa_s . dy_t
      Nyv = mfma(vop, dyop, Nyv);                                     // [s][t] = v_s . dy_t
      Nss = mfma(sa_h, ds_h, Nss); Nss = mfma(sa_h, ds_l, Nss); Nss = mfma(sa_l, ds_h, Nss);   // sa_s . dsa_t
      Nsv = mfma(vop, ds_h, Nsv); Nsv = mfma(vop, ds_l, Nsv);         // v_s . dsa_t
    }
  }
  // ---- triangular masks (rows s, column t = this lane's token)
  const int n = t;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool lt = m < n, le = m <= n;
    if (slow) {
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      lt = lt && same; le = le && same;
    }
    Nys[i] = le ? Nys[i] : 0.f;
    Nyv[i] = le ? Nyv[i] : 0.f;
    Nss[i] = lt ? Nss[i] : 0.f;
    Nsv[i] = lt ? Nsv[i] : 0.f;
  }
  {
    uint32_t a0, b0, a1, b1, c0, d0, c1, d1;
    split2(Nys[0], Nys[1], a0, b0); split2(Nys[2], Nys[3], a1, b1);
    split2(Nyv[0], Nyv[1], c0, d0); split2(Nyv[2], Nyv[3], c1, d1);
    slot->Ny[0][lane] = make_uint4(a0, a1, c0, c1);
    slot->Ny[1][lane] = make_uint4(b0, b1, d0, d1);
    split2(Nss[0], Nss[1], a0, b0); split2(Nss[2], Nss[3], a1, b1);
    split2(Nsv[0], Nsv[1], c0, d0); split2(Nsv[2], Nsv[3], c1, d1);
    slot->Ns[0][lane] = make_uint4(a0, a1, c0, c1);
    slot->Ns[1][lane] = make_uint4(b0, b1, d0, d1);
  }
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
    slot->ns = (int)F.ns;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state columns of keys 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), S[vt][i] = S[value 16*vt + 4g + i][key 16q + n].
struct Consumer {
  f32x4_t S[4];
  float pend;          // lanes g = 3: r.dr of the previous chunk's last token, whose workspace entry is still open
  int q, lane;
};

struct OutCursor {
  char *gr, *ga;       // bf16 outputs at (b, c0, h, 0)
  float* ef;           // this wave's record of the chunk in the fp32 workspace (f_record)
  size_t tok_bytes;    // bytes between consecutive tokens in the bf16 arrays (twice that in the fp32 ones)
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + key
};

__device__ __forceinline__ size_t state_el(const Wkv7Args& A, int64_t b, int64_t h, int value, int key) {
  return (((size_t)b * A.H + h) * 64 + value) * 64 + key;
}
__device__ __forceinline__ float ld_state_el(const void* p, int f32, size_t off) {
  return f32 ? reinterpret_cast<const float*>(p)[off] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p)[off]);
}

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool first,
                                        bool last, OutCursor& oc) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // B operands of the token contractions: (b/E, k/E) of tokens 4g..4g+3 at this wave's keys
  const u32x4_t tb = *reinterpret_cast<const u32x4_t*>(&slot->BT[0][q][lane]);
  const u32x4_t tk = *reinterpret_cast<const u32x4_t*>(&slot->BT[1][q][lane]);
  const u32x4_t Bh = {tb[0], tb[1], tk[0], tk[1]}, Bl = {tb[2], tb[3], tk[2], tk[3]};
  const bool keep_end = slot->keep_end != 0;
  // B operands from the state: MFMA j contracts over the values of tiles 2j and 2j+1
  u32x4_t Sh[2], Sl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2_keep(C.S[2 * j][0], C.S[2 * j][1], hi, lo); Sh[j][0] = hi; Sl[j][0] = lo;
    split2_keep(C.S[2 * j][2], C.S[2 * j][3], hi, lo); Sh[j][1] = hi; Sl[j][1] = lo;
    split2_keep(C.S[2 * j + 1][0], C.S[2 * j + 1][1], hi, lo); Sh[j][2] = hi; Sl[j][2] = lo;
    split2_keep(C.S[2 * j + 1][2], C.S[2 * j + 1][3], hi, lo); Sh[j][3] = hi; Sl[j][3] = lo;
  }
  f32x4_t DR = zero4, DA = zero4;   // [token 4g+i][key n]
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t dy = *reinterpret_cast<const u32x4_t*>(&slot->DY[n][32 * j + 8 * g]);
    const u32x4_t dh = *reinterpret_cast<const u32x4_t*>(&slot->DSA[0][n][32 * j + 8 * g]);
    const u32x4_t dl = *reinterpret_cast<const u32x4_t*>(&slot->DSA[1][n][32 * j + 8 * g]);
    DR = mfma(dy, Sh[j], DR); DA = mfma(dh, Sh[j], DA);
    DR = mfma(dy, Sl[j], DR); DA = mfma(dh, Sl[j], DA);
    DA = mfma(dl, Sh[j], DA);
  }
  {
    const u32x4_t nyh = *reinterpret_cast<const u32x4_t*>(&slot->Ny[0][lane]);
    const u32x4_t nyl = *reinterpret_cast<const u32x4_t*>(&slot->Ny[1][lane]);
    const u32x4_t nsh = *reinterpret_cast<const u32x4_t*>(&slot->Ns[0][lane]);
    const u32x4_t nsl = *reinterpret_cast<const u32x4_t*>(&slot->Ns[1][lane]);
    DR = mfma(nyh, Bh, DR); DA = mfma(nsh, Bh, DA);
    DR = mfma(nyh, Bl, DR); DA = mfma(nsh, Bl, DA);
    DR = mfma(nyl, Bh, DR); DA = mfma(nsl, Bh, DA);
  }
  // A operands of the state update: rows = values of tile vt, k-slots = (sa | v) of tokens 4g..4g+3
  u32x4_t A1[4], A3[4];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const uint4 st = slot->SAt[vt][lane];
    const uint2 vv = slot->Vt[vt][lane];
    A1[vt] = u32x4_t{st.x, st.y, vv.x, vv.y};
    A3[vt] = u32x4_t{st.z, st.w, 0u, 0u};
  }
  // <dS_out, S_{length-1}> per key (one chunk per sequence)
  float inj = 0.f;
  int snap_tok = -1;
  if (is_snap) {
    snap_tok = slot->snap;
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
    float p = 0.f;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      const uint4 st = snapslot->SAt[vt][lane];
      const uint2 vv = snapslot->Vt[vt][lane];
      const u32x4_t S1 = {st.x, st.y, vv.x, vv.y}, S3 = {st.z, st.w, 0u, 0u};
      f32x4_t acc = keep ? C.S[vt] : zero4;
      acc = mfma(S1, Bh, acc);
      acc = mfma(S1, Bl, acc);
      acc = mfma(S3, Bh, acc);
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
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = zero4;   // a reset inside the chunk cuts the entering state off
  }
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    f32x4_t acc = C.S[vt];
    acc = mfma(A1[vt], Bh, acc);
    acc = mfma(A1[vt], Bl, acc);
    acc = mfma(A3[vt], Bh, acc);
    acc[0] *= gm; acc[1] *= gm; acc[2] *= gm; acc[3] *= gm;
    C.S[vt] = acc;
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive keys
  float e[5];
#pragma unroll
  for (int i = 0; i < 5; ++i) e[i] = slot->E[4 * g + i][16 * q + n];
  const size_t lo = (size_t)oc.voff;
  const bool full = nvalid == CK;      // every chunk but a partial last one: no per-lane predicates
  float e2[4], e3[4];
  uint16_t odr[4], oda[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = 4 * g + i;
    const float rr = bf16_to_f32(slot->RA[0][tok][16 * q + n]);
    const float aa = bf16_to_f32(slot->RA[1][tok][16 * q + n]);
    const float dr = DR[i] * e[i + 1];
    const float da = DA[i] * e[i];
    odr[i] = f32_to_bf16(dr); oda[i] = f32_to_bf16(da);
    e2[i] = aa * da;
    e3[i] = fmaf(rr, dr, tok == snap_tok ? inj : 0.f);
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
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (full || 4 * g + i < nvalid) {
      *reinterpret_cast<uint16_t*>(oc.gr + lo * 2 + i * oc.tok_bytes) = odr[i];
      *reinterpret_cast<uint16_t*>(oc.ga + lo * 2 + i * oc.tok_bytes) = oda[i];
    }
  }
  // The whole record entry at once.  Token 15 of a chunk that is not the last one is still open: its entry (lanes
  // g = 3, element 3) is a placeholder until the next chunk overwrites it below; both stores come from this wave, to
  // the same address, in program order.  Entries of tokens beyond the sequence are never used.
  *reinterpret_cast<float4*>(oc.ef + 4 * lane) = make_float4(f[0], f[1], f[2], f[3]);
  if (!first && g == 0) (oc.ef - NCONS * F_REC)[4 * (48 + n) + 3] = open_prev + (follows(0) ? e2[0] : 0.f);
  oc.gr += CK * oc.tok_bytes; oc.ga += CK * oc.tok_bytes;
  oc.ef += NCONS * F_REC;
}

}  // namespace

// Slot c % RING holds chunk c.  Producer p fills it once every consumer has released chunk c - RING, then
// publishes ready = c + 1; consumers take chunks in order.  Every wait is for a strictly earlier chunk, so the
// hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_chunk_bwd_b_kernel(Wkv7Args A) {
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
    C.pend = 0.f;
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        C.S[vt][i] = ld_state_el(A.s, A.st_f32, state_el(A, b, h, 16 * vt + 4 * g + i, 16 * wave + n));
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T) * A.H + h) * 64;
    oc.gr = reinterpret_cast<char*>(A.gr) + el0 * 2;
    oc.ga = reinterpret_cast<char*>(A.ga) + el0 * 2;
    oc.ef = A.e2 + f_record(b, h, A.H, nch, 0, wave);
    oc.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    for (int c = 0; c < nch; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING;
      if (!wait_ready(sy, si, c + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, c == 0, c + 1 == nch, oc);
      // every LDS read of slot si has returned: its data went into the MFMAs and stores above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
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
      Slot* slot = &slots[si];
      if (c >= RING && !wait_consumed(sy, si, c - RING + 1, lane)) break;
      produce(P, raw, F, slot, snapslot, events_word(A.status));
      if (c + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, c0 + NPROD * CK, lane);
        load_raw(raw, A, b, h, c0 + NPROD * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && c + 1 == nch) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // (no retire_loads here: measured, this sweep is 5 % slower with it -- its producers are the bottleneck, and
    // keeping their operand registers alive to the end of the loop costs them more than the consumers gain)
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gr, 2, b, h, A.T, A.H);
    poison_token_rows(A.ga, 2, b, h, A.T, A.H);
    for (size_t i = threadIdx.x; i < (size_t)nch * NCONS * F_REC; i += blockDim.x)
      A.e2[f_record(b, h, A.H, nch, 0, 0) + i] = __uint_as_float(0x7fc00000u);
  }
}

hipError_t launch_wkv7_chunk_bwd_b(const Wkv7Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_chunk_bwd_b_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_chunk_bwd_b_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
