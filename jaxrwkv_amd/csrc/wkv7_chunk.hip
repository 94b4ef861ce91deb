// WKV7 forward, chunked MFMA kernel for bf16 I/O on gfx950.
//
// Recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220), S[i][j] = value row i, key col j:
//     sa_t = S_{t-1} a_t ;  S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;  y_t = S_t r_t ;  d_t = exp(-exp(w_t))
// A chunk of C = 16 tokens entering with state S0 is evaluated in closed form.  With l_t = log d_t,
// Lc_t = sum_{s<=t} l_s, E_t = exp(Lc_t), Ee_t = exp(Lc_{t-1}) and the scaled operands
//     at_t = a_t.Ee_t   qt_t = r_t.E_t   kh_s = k_s/E_s   bh_s = b_s/E_s          (. and / elementwise over keys)
//     Mba[s][t] = bh_s.at_t (s<t)   Mka[s][t] = kh_s.at_t (s<t)   Mbr[s][t] = bh_s.qt_t (s<=t)   Mkr likewise
//     W  = S0 At^T + V^T Mka          (value x token)
//     SA = W (I - Mba)^{-1}            sa_t for the 16 tokens; the inverse of a unit triangular 16x16
//     Y  = S0 Qt^T + SA Mbr + V^T Mkr
//     S_C = (S0 + SA Bh + V^T Kh) diag(E_C)
// (I - M)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M) because M^16 = 0.  Every product runs on
// v_mfma_f32_16x16x32_bf16.  fp32 operands are fed as a truncated-bf16 "hi" plus a bf16 "lo" part and the three
// significant partial products are accumulated (hi.hi + hi.lo + lo.hi), which keeps ~16 mantissa bits; the
// doubling chain of the inverse alone runs in single bf16 (its result is split again).  The K = 32 slots of one
// MFMA hold two 16-token products side by side.  The state stays in fp32 accumulator registers for the whole
// sequence, transposed (key x value tiles), so that accumulator registers are reused directly as B operands.
//
// Work split: one workgroup of 8 waves per (sequence, head).  Waves 0-3 are consumers: wave q owns value rows
// 16q..16q+15 of the state and runs the S0-dependent part of every chunk.  Waves 4-7 are producers: producer p
// prepares chunks p, p+4, p+8, ... (everything that does not depend on S0: decay scan, scaled operands, Gram
// tiles, triangular inverse, operand transposes) into a ring of LDS slots, four chunk periods ahead of the
// consumers.  Synchronisation is a pair of LDS sequence numbers per slot: `ready` (set by the producer when a
// chunk is complete) and `consumed` (one per consumer wave, set when it has read the slot for the last time).
// Waiting is a bounded poll, so that a broken hand-shake ends the kernel (with wrong results) instead of
// hanging the GPU.
// new_starts inside a chunk restart the cumulative decay and mask the Gram tiles (rare, uniform branch).
// `length` snapshots use a second, masked set of update operands for the one chunk that holds token length-1.
//
// Range: the cumulative log decay inside a chunk is clamped at -80 so that 1/E_s stays finite in fp32.  A key
// channel whose decay over at most 16 tokens falls below e^-80 (RWKV-7 models keep d >= 0.54 per token, i.e.
// e^-10 per chunk) is finite but no longer exact; the sequential kernel has no such limit.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight

// One chunk's operands as the consumers read them.  "lane-indexed" arrays hold, for every lane of the producer,
// the 16 bytes that the same lane of a consumer loads: accumulator-layout registers (column lane%16, rows
// 4*(lane/16)..+3) packed to bf16, hi pair then lo pair, which is exactly an A operand (row lane%16, k-slots
// 4*(lane/16)..+3 of the hi part followed by the same slots of the lo part).
struct __attribute__((aligned(16))) Slot {
  // At = a_t.Ee_t and Qt = r_t.E_t, [hi|lo][At|Qt][token][RS]: within a row, the 16-byte vector (j, g) at element
  // 32j + 8g holds keys 32j+4g..+3 followed by keys 32j+16+4g..+3, the key order of the consumers' state tiles.
  // Rows the entering state does not reach are zero; Qt rows whose y is defined as zero are zero.
  uint16_t AQ[2][2][CK][RS];
  uint4 BT[2][4][64];          // [bh|kh][key tile]: (b_s/E_s)^T hi,lo, lane-indexed; masked for the chunk-end state
  uint2 VT[4][64];             // v^T per value tile, lane-indexed
  uint4 Mt[4][64];             // T, Mka, Mbr, Mkr: hi,lo, lane-indexed
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
// Update operands masked for the snapshot token; only one chunk per sequence needs them.
struct __attribute__((aligned(16))) SnapSlot {
  uint4 BT[2][4][64];
  float gamma[64];
};
// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys {8g..8g+7} u {32+8g..32+8g+7}: exactly the A/B
// operand layout of the Gram MFMAs (row/column = token, k-slots = keys), and one 16-byte global load per half.
struct Raw {
  uint4 r[2], w[2], k[2], v[2], a[2], b[2];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const uint4 z = make_uint4(0, 0, 0, 0);
  if (c0 + t < A.T) {
    const size_t off = ((((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g) * 2;  // bytes
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off + 64);
    };
    ld(A.r, x.r); ld(A.w, x.w); ld(A.k, x.k); ld(A.v, x.v); ld(A.a, x.a); ld(A.b, x.b);
  } else {
    x.r[0] = x.r[1] = x.w[0] = x.w[1] = x.k[0] = x.k[1] = z;
    x.v[0] = x.v[1] = x.a[0] = x.a[1] = x.b[0] = x.b[1] = z;
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // B operands that pick keys 16*(tile%2)..+15 out of a 32-key half: MFMA as a transposer
};

// Everything of one chunk that does not depend on the entering state.  The two 32-key halves go through the
// same pipeline one after the other (scan, scaling, hi/lo split, LDS parking, transposes, partial Gram sums),
// which keeps the live register set small enough for three waves per SIMD.
__device__ __forceinline__ void produce(const Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const u32x4_t z4 = {0u, 0u, 0u, 0u};
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  // reset bookkeeping (uniform values unless they depend on t)
  int lastseg = 0, seg_src = 0;
  bool s0_reaches = true, q_keep = true, restart = false, at_reset = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    lastseg = seg_of(F.ns, 15);
    s0_reaches = seg_of(F.ns, t) == 0;                              // the entering state reaches this token
    q_keep = s0_reaches && !(F.compat && ((F.ns >> (t + 1)) & 1u)); // y[t] is defined as zero before a reset
    if (resets) keep_upd = 0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u);   // tokens from the last reset on
    const uint32_t upto = resets & ((2u << t) - 1u);
    const int pr = upto ? 31 - __builtin_clz(upto) : 0;             // last reset at or before this token
    restart = pr > 0;
    seg_src = (lane & 48) | (pr > 0 ? pr - 1 : 0);
    at_reset = (resets >> t) & 1u;
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

  f32x4_t Mba = zero4, MbaT = zero4, Mka = zero4, Mbr = zero4, Mkr = zero4;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ---- v^T of value tiles 2hf, 2hf+1: D[token][value] = sum_k V[token][k] sel[k][value]
    {
      const uint4 vr = x.v[hf];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w};
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) slot->VT[2 * hf + x2][lane] = plain_pack(mfma(vop, P.sel[x2], zero4));
    }
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain
    float E[8], fa[8];
    {
      float fw[8];
      unpack8(x.w[hf], fw);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float l2 = fmaxf(-exp2_fast(fw[e] * LOG2E) * LOG2E, MIN_STEP_L2);
        if (F.nvalid != CK) l2 = valid ? l2 : 0.f;
        l2 += dpp0<0x111>(l2);
        l2 += dpp0<0x112>(l2);
        l2 += dpp0<0x114>(l2);
        l2 += dpp0<0x118>(l2);
        E[e] = l2;
      }
    }
    unpack8(x.a[hf], fa);
    if (slow) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
        if (restart) E[e] -= base;
        if (at_reset) fa[e] = 0.f;                      // the state entering a reset token is zero: sa = 0
      }
    }
    // ---- scaled operands and their hi/lo split
    u32x4_t at_h, at_l, qt_h, qt_l, kh_h, kh_l, bh_h, bh_l;
    {
      float fr[8], fk[8], fb[8], Einv[8], Ee[8];
      unpack8(x.r[hf], fr); unpack8(x.k[hf], fk); unpack8(x.b[hf], fb);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = fmaxf(E[e], MIN_CUM_L2);
        E[e] = exp2_fast(l2);
        Einv[e] = exp2_fast(-l2);
        // exclusive: value of the previous token; 1 for the first token of the chunk (a is zero at reset tokens)
        Ee[e] = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(1.0f), __float_as_int(E[e]), 0x111, 0xf, 0xf, false));
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = 2 * j;
        uint32_t hi, lo;
        split2(fa[e] * Ee[e], fa[e + 1] * Ee[e + 1], hi, lo); at_h[j] = hi; at_l[j] = lo;
        split2(fr[e] * E[e], fr[e + 1] * E[e + 1], hi, lo); qt_h[j] = hi; qt_l[j] = lo;
        split2(fk[e] * Einv[e], fk[e + 1] * Einv[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
        split2(fb[e] * Einv[e], fb[e + 1] * Einv[e + 1], hi, lo); bh_h[j] = hi; bh_l[j] = lo;
      }
    }
    // ---- decay to the chunk end / to the snapshot token
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
    // ---- At, Qt rows for the consumers, in their key order: this lane's keys 8g..8g+3 and 8g+4..8g+7 of the half
    //      are the (g>>1)-th 8-byte piece of the vectors 2(g&1) and 2(g&1)+1 of block j = hf
    {
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // element offset of the first piece
      auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
        *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
        *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
      };
      if (!slow) {
        put(slot->AQ[0][0][t], at_h, true); put(slot->AQ[1][0][t], at_l, true);
        put(slot->AQ[0][1][t], qt_h, true); put(slot->AQ[1][1][t], qt_l, true);
      } else {
        put(slot->AQ[0][0][t], at_h, s0_reaches); put(slot->AQ[1][0][t], at_l, s0_reaches);
        put(slot->AQ[0][1][t], qt_h, q_keep); put(slot->AQ[1][1][t], qt_l, q_keep);
      }
    }
    // ---- (b/E)^T, (k/E)^T of key tiles 2hf, 2hf+1 by MFMA: the accumulator layout of D (lane = key, registers =
    //      4 consecutive tokens) is the A-operand layout of the state update
#pragma unroll
    for (int x2 = 0; x2 < 2; ++x2) {
      const int tile = 2 * hf + x2;
      const u32x4_t sel = P.sel[x2];
      const f32x4_t dbh = mfma(bh_h, sel, zero4), dbl = mfma(bh_l, sel, zero4);
      const f32x4_t dkh = mfma(kh_h, sel, zero4), dkl = mfma(kh_l, sel, zero4);
      if (keep_upd == 0xffffu) {
        slot->BT[0][tile][lane] = join(plain_pack(dbh), plain_pack(dbl));
        slot->BT[1][tile][lane] = join(plain_pack(dkh), plain_pack(dkl));
      } else {
        slot->BT[0][tile][lane] = join(masked_pack(dbh, keep_upd), masked_pack(dbl, keep_upd));
        slot->BT[1][tile][lane] = join(masked_pack(dkh, keep_upd), masked_pack(dkl, keep_upd));
      }
      if (F.snap >= 0) {
        snap->BT[0][tile][lane] = join(masked_pack(dbh, keep_snap), masked_pack(dbl, keep_snap));
        snap->BT[1][tile][lane] = join(masked_pack(dkh, keep_snap), masked_pack(dkl, keep_snap));
      }
    }
    // ---- partial Gram sums over this half's keys (accumulator layout: column n = lane%16, rows 4g..4g+3)
#pragma unroll
    for (int part = 0; part < 3; ++part) {
      const u32x4_t bA = part == 2 ? bh_l : bh_h, kA = part == 2 ? kh_l : kh_h, aA = part == 2 ? at_l : at_h;
      const u32x4_t aB = part == 1 ? at_l : at_h, qB = part == 1 ? qt_l : qt_h, bB = part == 1 ? bh_l : bh_h;
      Mba = mfma(bA, aB, Mba);     // [s][t] = bh_s . at_t
      MbaT = mfma(aA, bB, MbaT);   // [t][s]
      Mka = mfma(kA, aB, Mka);     // [s][t] = kh_s . at_t
      Mbr = mfma(bA, qB, Mbr);     // [s][t] = bh_s . qt_t
      Mkr = mfma(kA, qB, Mkr);     // [s][t] = kh_s . qt_t
    }
  }
  // ---- triangular masks
  const int n = t;
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      Mba[i] = (m < n) ? Mba[i] : 0.f;
      Mka[i] = (m < n) ? Mka[i] : 0.f;
      Mbr[i] = (m <= n) ? Mbr[i] : 0.f;
      Mkr[i] = (m <= n) ? Mkr[i] : 0.f;
      MbaT[i] = (m > n) ? MbaT[i] : 0.f;   // [t = m][s = n], s < t
    }
  } else {
    const bool dropy = F.compat && ((F.ns >> (n + 1)) & 1u);   // y[n] is defined as zero
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      const bool lt = (m < n) && same, le = (m <= n) && same, gt = (m > n) && same;
      Mba[i] = lt ? Mba[i] : 0.f;
      Mka[i] = lt ? Mka[i] : 0.f;
      Mbr[i] = (le && !dropy) ? Mbr[i] : 0.f;
      Mkr[i] = (le && !dropy) ? Mkr[i] : 0.f;
      MbaT[i] = gt ? MbaT[i] : 0.f;
    }
  }
  // ---- T = (I + M^8)(I + M^4)(I + M^2)(I + M), single-bf16 operands
  auto single = [&](const f32x4_t d) {
    u32x4_t o = {pack_rn(d[0], d[1]), pack_rn(d[2], d[3]), 0u, 0u};
    return o;
  };
  f32x4_t Pm = Mba;
#pragma unroll
  for (int i = 0; i < 4; ++i) Pm[i] += (4 * g + i == n) ? 1.f : 0.f;
  f32x4_t Mp = Mba, MpT = MbaT;
#pragma unroll
  for (int lvl = 0; lvl < 3; ++lvl) {
    const u32x4_t om = single(Mp), omt = single(MpT);
    const f32x4_t M2T = mfma(om, omt, zero4);      // (M^2)^T[t][s]
    if (lvl < 2) Mp = mfma(omt, om, zero4);        // (M^2)[s][t]: A rows from the transpose, B columns from M
    MpT = M2T;
    Pm = mfma(single(MpT), single(Pm), Pm);        // P += M^(2^(lvl+1)) P
  }
  uint32_t hi0, lo0, hi1, lo1;
  auto park = [&](int which, const f32x4_t d) {
    split2(d[0], d[1], hi0, lo0);
    split2(d[2], d[3], hi1, lo1);
    slot->Mt[which][lane] = make_uint4(hi0, hi1, lo0, lo1);
  };
  park(0, Pm); park(1, Mka); park(2, Mbr); park(3, Mkr);
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds S^T for value rows 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16, g = lane/16),
// S[tile][i] = S[value 16q+n][key 16*tile + 4g + i].
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

// Operands a consumer carries from one chunk to the next.  Each group is reloaded for the next chunk right
// after its last use in the current one, so the LDS latency hides behind the rest of the chunk and no second set
// of registers is needed.
struct Ops {
  u32x4_t aq[2][2][2];     // [hi|lo][At|Qt][j]: rows in the key order of the state tiles
  u32x4_t T, Ka, Br, Kr;   // T, Mka, Mbr, Mkr: hi pair, lo pair
  u32x4_t vv;              // v^T of this wave's value tile, twice (for a hi and a lo A part side by side)
  int keep_end;
};

__device__ __forceinline__ void load_aq(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int pl = 0; pl < 2; ++pl)
#pragma unroll
    for (int ar = 0; ar < 2; ++ar)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        o.aq[pl][ar][j] = *reinterpret_cast<const u32x4_t*>(&slot->AQ[pl][ar][n][32 * j + 8 * g]);
  o.Ka = *reinterpret_cast<const u32x4_t*>(&slot->Mt[1][lane]);
  o.Kr = *reinterpret_cast<const u32x4_t*>(&slot->Mt[3][lane]);
  const uint2 v0 = slot->VT[q][lane];
  o.vv = u32x4_t{v0.x, v0.y, v0.x, v0.y};
  o.keep_end = slot->keep_end;
}
__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  load_aq(o, slot, q, lane);
  o.T = *reinterpret_cast<const u32x4_t*>(&slot->Mt[0][lane]);
  o.Br = *reinterpret_cast<const u32x4_t*>(&slot->Mt[2][lane]);
}

// Uniform output cursors of a consumer, advanced by one chunk per call.
struct OutCursor {
  char* y;             // A.out at (b, c0, h, 0)
  char* sa;            // A.sa at the same place, or null
  size_t tok_bytes;    // bytes between consecutive tokens in y (twice that in sa)
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + value
};

// The S0-dependent part of one chunk.  `next` is the slot of the following chunk (null after the last one);
// `next_ready` waits until its producer has published it.
template <class WaitNext>
__device__ __forceinline__ void consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
                                        const Slot* __restrict__ next, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool q2drop,
                                        OutCursor& oc, WaitNext&& next_ready) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // update operands of this chunk: needed last, so their latency hides behind the W / SA chain
  u32x4_t bt[2][4];
  float4 gm[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    bt[0][tile] = *reinterpret_cast<const u32x4_t*>(&slot->BT[0][tile][lane]);
    bt[1][tile] = *reinterpret_cast<const u32x4_t*>(&slot->BT[1][tile][lane]);
    gm[tile] = *reinterpret_cast<const float4*>(&slot->gamma[16 * tile + 4 * g]);
  }
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
  // B operands from the state: MFMA j contracts over the keys of tiles 2j and 2j+1
  u32x4_t Sh[2], Sl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2(C.S[2 * j][0], C.S[2 * j][1], hi, lo); Sh[j][0] = hi; Sl[j][0] = lo;
    split2(C.S[2 * j][2], C.S[2 * j][3], hi, lo); Sh[j][1] = hi; Sl[j][1] = lo;
    split2(C.S[2 * j + 1][0], C.S[2 * j + 1][1], hi, lo); Sh[j][2] = hi; Sl[j][2] = lo;
    split2(C.S[2 * j + 1][2], C.S[2 * j + 1][3], hi, lo); Sh[j][3] = hi; Sl[j][3] = lo;
  }
  f32x4_t W = zero4, Y = zero4;   // [token 4g+i][value n], two interleaved accumulation chains
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    W = mfma(o.aq[0][0][j], Sh[j], W); Y = mfma(o.aq[0][1][j], Sh[j], Y);
    W = mfma(o.aq[0][0][j], Sl[j], W); Y = mfma(o.aq[0][1][j], Sl[j], Y);
    W = mfma(o.aq[1][0][j], Sh[j], W); Y = mfma(o.aq[1][1][j], Sh[j], Y);
  }
  W = mfma(o.Ka, o.vv, W);                    // W += Mka^T V^T (hi and lo parts side by side)
  Y = mfma(o.Kr, o.vv, Y);                    // Y += Mkr^T V^T
  const u32x4_t vv = o.vv;
  // At, Qt, Mka, Mkr, v^T are dead now: fetch the next chunk's into the same registers
  if (next != nullptr) {
    next_ready();
    load_aq(o, next, C.q, lane);
  }
  uint32_t h0, l0, h1, l1;
  split2(W[0], W[1], h0, l0);
  split2(W[2], W[3], h1, l1);
  f32x4_t SA;
  {
    // an A operand holds the hi pair in k-slots 0..3 and the lo pair in 4..7: against (x_hi, x_hi) it gives
    // (A_hi + A_lo) x_hi, against (x_lo, 0) it gives A_hi x_lo
    const u32x4_t bhh = {h0, h1, h0, h1}, bl0 = {l0, l1, 0u, 0u};
    SA = mfma(o.T, bhh, zero4);               // (T_hi + T_lo)^T W_hi
    SA = mfma(o.T, bl0, SA);                  // T_hi^T W_lo
  }
  if (next != nullptr) o.T = *reinterpret_cast<const u32x4_t*>(&next->Mt[0][lane]);
  split2(SA[0], SA[1], h0, l0);
  split2(SA[2], SA[3], h1, l1);
  const u32x4_t sHH = {h0, h1, h0, h1}, sL0 = {l0, l1, 0u, 0u};
  Y = mfma(o.Br, sHH, Y);
  Y = mfma(o.Br, sL0, Y);                     // Y^T += Mbr^T SA^T
  if (next != nullptr) o.Br = *reinterpret_cast<const u32x4_t*>(&next->Mt[2][lane]);
  // state snapshot for `length` (one chunk per sequence)
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const u32x4_t sb = *reinterpret_cast<const u32x4_t*>(&snapslot->BT[0][tile][lane]);
      const u32x4_t sk = *reinterpret_cast<const u32x4_t*>(&snapslot->BT[1][tile][lane]);
      f32x4_t acc = keep ? C.S[tile] : zero4;
      acc = mfma(sb, sHH, acc);
      acc = mfma(sk, vv, acc);
      acc = mfma(sb, sL0, acc);
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      acc[0] *= sg.x; acc[1] *= sg.y; acc[2] *= sg.z; acc[3] *= sg.w;
      const size_t off = (((size_t)b * A.H + h) * 64 + 16 * C.q + n) * 64 + 16 * tile + 4 * g;
      if (A.st_f32) {
        float4 ov = q2drop ? make_float4(0.f, 0.f, 0.f, 0.f) : make_float4(acc[0], acc[1], acc[2], acc[3]);
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(A.new_s) + off) = ov;
      } else {
        uint2 ov = q2drop ? make_uint2(0u, 0u) : make_uint2(pack_rn(acc[0], acc[1]), pack_rn(acc[2], acc[3]));
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(A.new_s) + off) = ov;
      }
    }
  }
  // state update, tile by tile: rows = keys.  S <- (S + Bh^T SA^T + Kh^T V^T) . gamma
  if (!keep_end) {
    asm volatile("" ::: "memory");   // keep this a (rare, uniform) branch instead of 16 selects on the hot path
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;   // a reset inside the chunk cuts the entering state off
  }
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    f32x4_t acc = C.S[tile];
    acc = mfma(bt[0][tile], sHH, acc);
    acc = mfma(bt[1][tile], vv, acc);
    acc = mfma(bt[0][tile], sL0, acc);
    acc[0] *= gm[tile].x; acc[1] *= gm[tile].y; acc[2] *= gm[tile].z; acc[3] *= gm[tile].w;
    C.S[tile] = acc;
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  const uint32_t y01 = pack_rn(Y[0], Y[1]), y23 = pack_rn(Y[2], Y[3]);
  char* const yl = oc.y + (size_t)oc.voff * 2;
  if (nvalid == CK) {
    *reinterpret_cast<uint16_t*>(yl) = (uint16_t)(y01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + oc.tok_bytes) = (uint16_t)(y01 >> 16);
    *reinterpret_cast<uint16_t*>(yl + 2 * oc.tok_bytes) = (uint16_t)(y23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + 3 * oc.tok_bytes) = (uint16_t)(y23 >> 16);
    if (oc.sa != nullptr) {
      char* const sl = oc.sa + (size_t)oc.voff * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<float*>(sl + 2 * i * oc.tok_bytes) = SA[i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        const uint32_t yv = (i & 2) ? y23 : y01;
        *reinterpret_cast<uint16_t*>(yl + i * oc.tok_bytes) = (uint16_t)((i & 1) ? (yv >> 16) : (yv & 0xffffu));
        if (oc.sa != nullptr) *reinterpret_cast<float*>(oc.sa + (size_t)oc.voff * 4 + 2 * i * oc.tok_bytes) = SA[i];
      }
    }
  }
  oc.y += CK * oc.tok_bytes;
  if (oc.sa != nullptr) oc.sa += 2 * CK * oc.tok_bytes;
}

__device__ __forceinline__ void load_state(Consumer& C, const Wkv7Args& A, int64_t b, int64_t h) {
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const size_t off = (((size_t)b * A.H + h) * 64 + 16 * C.q + n) * 64 + 16 * tile + 4 * g;
    if (A.st_f32) {
      const float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(A.s) + off);
      C.S[tile][0] = x.x; C.S[tile][1] = x.y; C.S[tile][2] = x.z; C.S[tile][3] = x.w;
    } else {
      const uint2 x = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(A.s) + off);
      C.S[tile][0] = __uint_as_float(x.x << 16); C.S[tile][1] = __uint_as_float(x.x & 0xffff0000u);
      C.S[tile][2] = __uint_as_float(x.y << 16); C.S[tile][3] = __uint_as_float(x.y & 0xffff0000u);
    }
  }
}

__device__ __forceinline__ void store_state0(const Consumer& C, const Wkv7Args& A, int64_t b, int64_t h, bool zero) {
  // length == 0: the returned state is the input state (rwkv7.py:203), or the reset state under the associative rule
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const size_t off = (((size_t)b * A.H + h) * 64 + 16 * C.q + n) * 64 + 16 * tile + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float x = zero ? 0.f : C.S[tile][i];
      if (A.st_f32) reinterpret_cast<float*>(A.new_s)[off + i] = x;
      else reinterpret_cast<uint16_t*>(A.new_s)[off + i] = f32_to_bf16(x);
    }
  }
}

}  // namespace

// Slot c % RING holds chunk c.  Producer p fills it once every consumer has released chunk c - RING, then
// publishes ready = c + 1; consumers take chunks in order.  Every wait is for a strictly earlier chunk, so the
// hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_chunk_fwd_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int64_t nchunks = (A.T + CK - 1) / CK;
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  if (wave < NCONS) {
    // the chunk-to-chunk dependency runs through the consumers: let them issue ahead of the producers
    __builtin_amdgcn_s_setprio(3);
    const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
    Consumer C;
    C.q = wave;
    C.lane = lane;
    load_state(C, A, b, h);
    if (L == 0) store_state0(C, A, b, h, q2drop);
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    oc.y = reinterpret_cast<char*>(A.out) + (((size_t)b * A.T) * A.H + h) * 64 * 2;
    oc.sa = A.sa ? reinterpret_cast<char*>(A.sa) + (((size_t)b * A.T) * A.H + h) * 64 * 4 : nullptr;
    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * wave + (lane & 15));
    const int csnap = L >= 1 ? (int)((L - 1) / CK) : -1;
    const int nch = (int)nchunks;
    Ops ops;
    if (nch > 0) {
      wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], wave, lane);
    }
    for (int c = 0; c < nch; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING, sn = (c + 1) % RING;
      const Slot* next = (c + 1 < nch) ? &slots[sn] : nullptr;
      consume(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, c == csnap, q2drop, oc,
              [&]() { wait_ready(sy, sn, c + 2); });
      // every LDS read of slot si has returned: its data went into the MFMAs above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
    Raw raw;
    if (p < nchunks) load_raw(raw, A, b, h, (int64_t)p * CK, lane);
    for (int64_t c = p; c < nchunks; c += NPROD) {
      const int64_t c0 = c * CK;
      const ChunkFlags F = chunk_flags(A.ns, A.flags, A.T, b, c0, L, lane);
      const int si = (int)(c % RING);
      Slot* slot = &slots[si];
      if (c >= RING) wait_consumed(sy, si, (int)(c - RING) + 1, lane);
      produce(P, raw, F, slot, snapslot);
      if (c + NPROD < nchunks) load_raw(raw, A, b, h, c0 + NPROD * CK, lane);
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], (int)c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
}

hipError_t launch_wkv7_chunk_fwd(const Wkv7Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(wkv7_chunk_fwd_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(wkv7_chunk_fwd_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
