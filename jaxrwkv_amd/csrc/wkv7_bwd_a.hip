// WKV7 backward for bf16 I/O on gfx950, first (reverse) sweep: gv, the workspace dsa and gs, 16 tokens at a time on
// the matrix cores.
//
// Forward recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220), S[i][j] = value row i, key
// col j:  sa_t = S_{t-1} a_t ;  S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;  y_t = S_t r_t ;  d_t = exp(-exp(w_t)).
// With G = dL/dS carried from the last token down (G~_t the cotangent of S_t):
//     G~_t = dy_t r_t^T + G~_{t+1} diag(d_{t+1}) + dsa_{t+1} a_{t+1}^T ;  dsa_t = G~_t b_t ;  dv_t = G~_t k_t
// With l_t = log d_t, Lc_t = sum_{s<=t} l_s, E_t = exp(Lc_t), Ee_t = exp(Lc_{t-1}) and the scaled operands
//     at_t = a_t.Ee_t   qt_t = r_t.E_t   kh_s = k_s/E_s   bh_s = b_s/E_s          (. and / elementwise over keys)
//     Mba[s][t] = bh_s.at_t (s<t)   Mka[s][t] = kh_s.at_t (s<t)   Mbr[s][t] = bh_s.qt_t (s<=t)   Mkr likewise
// a chunk leaving with G_C (cotangent of the chunk-end state from later chunks), Gh = G_C diag(E_C), gives
//     G~_t diag(E_t) = Gh + sum_{s>=t} dy_s qt_s^T + sum_{s>t} dsa_s at_s^T
//     U   = Gh Bh^T + DY^T Mbr^T         DSA = U (I - Mba^T)^{-1}         DV = Gh Kh^T + DSA Mka^T + DY^T Mkr^T
//     G_prev = Gh + DSA At + DY^T Qt      (cotangent of the state entering the chunk)
// which is the forward chunk computation with the operands exchanged (Bh <-> At, Kh <-> Qt, V <-> DY, every Gram
// tile transposed) and the decay applied before instead of after the update.
// (I - M)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M) because M^16 = 0.  Every product runs on
// v_mfma_f32_16x16x32_bf16.  fp32 operands are fed as a truncated-bf16 "hi" plus a bf16 "lo" part and the three
// significant partial products are accumulated (hi.hi + hi.lo + lo.hi), which keeps ~16 mantissa bits; the
// doubling chain of the inverse alone runs in single bf16 (its result is split again).  Cotangents have no bounded
// range, so the fp16 operands of the forward kernel (wkv7_fwd.hip) are not used here.  The K = 32 slots of one MFMA
// hold two 16-token products side by side.  G stays in fp32 accumulator registers for the whole sequence,
// transposed (key x value tiles), so that accumulator registers are reused directly as B operands.
//
// Work split: one workgroup of 8 waves per (sequence, head).  Waves 0-3 are consumers: wave q owns value rows
// 16q..16q+15 of G and runs the G-dependent part of every chunk.  Waves 4-7 are producers: producer p prepares
// chunks p, p+4, p+8, ... counted from the end (everything that does not depend on G: decay scan, scaled operands,
// Gram tiles, triangular inverse, operand transposes) into a ring of LDS slots, four chunk periods ahead of the
// consumers.  Synchronisation is a pair of LDS sequence numbers per slot with bounded waits (chunk_common.h).
// new_starts inside a chunk restart the cumulative decay and mask the Gram tiles (rare, uniform branch).
// The one chunk that holds token length-1 uses a second, masked set of row operands through which the cotangent of
// the returned state enters.
//
// Range: a key channel whose total log decay over a 16-token chunk is below -80 gets its steps of that chunk scaled
// to a total of -80, so that 1/E_s stays finite in fp32 (cap_chunk_decay), as in the forward kernel.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

// Eight producers around six slots: each producer's loads are requested eight chunks ahead, which hides more of their
// latency than four producers do (422 -> 397 us at the headline shape) although twelve waves leave 168 registers and ten
// of the producer's spill.
constexpr int NPROD = 8;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 6;           // slots in flight (a slot is 23 KB)

// One chunk's operands as the consumers read them.  "lane-indexed" arrays hold, for every lane of the producer,
// the 16 bytes that the same lane of a consumer loads: accumulator-layout registers (column lane%16, rows
// 4*(lane/16)..+3) packed to bf16, hi pair then lo pair, which is exactly an A operand (row lane%16, k-slots
// 4*(lane/16)..+3 of the hi part followed by the same slots of the lo part).
// Names are those of the forward chunk computation; this sweep stores (Bh, Kh) rows in AQ, (at, qt)^T in BT, dy^T in
// VT and the transposed Gram tiles (inverse, Mbr^T, Mka^T, Mkr^T) in Mt.
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
  int keep_end;                // the carried state passes through the whole chunk (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int pad;
};
// Row operands masked for token length-1, through which the cotangent of the returned state enters; only one chunk
// per sequence needs them.
struct __attribute__((aligned(16))) SnapSlot {
  uint16_t AQ[2][2][CK][RS];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys {8g..8g+7} u {32+8g..32+8g+7}: exactly the A/B
// operand layout of the Gram MFMAs (row/column = token, k-slots = keys), and one 16-byte global load per half.
struct Raw {
  uint4 r[2], w[2], k[2], v[2], a[2], b[2];   // v holds dy
};

// Loads always touch a valid token (the last one of the sequence for lanes beyond it); mask_raw zeroes those lanes.
__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;
  const size_t off = ((((size_t)b * A.T + tok) * A.H + h) * 64 + 8 * g) * 2;  // bytes
  auto ld = [&](const void* p, uint4 (&o)[2]) {
    o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off);
    o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off + 64);
  };
  ld(A.r, x.r); ld(A.w, x.w); ld(A.k, x.k); ld(A.gy, x.v); ld(A.a, x.a); ld(A.b, x.b);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const uint4 z = make_uint4(0, 0, 0, 0);
      x.r[0] = x.r[1] = x.w[0] = x.w[1] = x.k[0] = x.k[1] = z;
      x.v[0] = x.v[1] = x.a[0] = x.a[1] = x.b[0] = x.b[1] = z;
    }
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // B operands that pick keys 16*(tile%2)..+15 out of a 32-key half: MFMA as a transposer
};

// Everything of one chunk that does not depend on the carried state.  The two 32-key halves go through the
// same pipeline one after the other (scan, scaling, hi/lo split, LDS parking, transposes, partial Gram sums),
// which keeps the live register set small.
__device__ __forceinline__ void produce(const Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  // reset bookkeeping (uniform values unless they depend on t)
  int lastseg = 0, seg_src = 0;
  bool row0_keep = true, row1_keep = true, restart = false, at_reset = false, drop_dy = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(F.ns, 15);
    const int myseg = seg_of(F.ns, t);
    row0_keep = row1_keep = myseg == lastseg;                        // the cotangent from later chunks reaches this token
    if (resets) keep_upd = (1u << __builtin_ctz(resets)) - 1u;       // tokens before the first reset
    drop_dy = F.compat && ((F.ns >> (t + 1)) & 1u);                  // y[t] is a constant there

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

  // Gram tiles in accumulator layout [row m = A-operand token][column n = B-operand token]
  f32x4_t Gab = zero4, GabT = zero4;   // bh_m.at_n and at_m.bh_n
  f32x4_t G1 = zero4, G2 = zero4, G3 = zero4;   // qt_m.bh_n, at_m.kh_n, qt_m.kh_n
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // issue priority rises with the wave's progress through the chunk (see wkv7_fwd.hip)
    if (hf == 0) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(2);
    // ---- v^T (dy^T) of value tiles 2hf, 2hf+1: D[token][value] = sum_k V[token][k] sel[k][value]
    {
      uint4 vr = x.v[hf];
      if (slow) {
        rare_path();
        if (drop_dy) vr = make_uint4(0, 0, 0, 0);
      }
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
      for (int e = 0; e < 8; ++e) fw[e] = fmaxf(-exp2_fast(fw[e] * LOG2E) * LOG2E, MIN_STEP_L2);
      if (F.nvalid != CK) {
        rare_path();
#pragma unroll
        for (int e = 0; e < 8; ++e) fw[e] = valid ? fw[e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) E[e] = row_scan(fw[e]);
      cap_chunk_decay(E, lane, events);
    }
    unpack8(x.a[hf], fa);
    if (slow) {
      rare_path();
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
        if (restart) E[e] -= base;
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
        // exclusive: value of the previous token; 1 for the first token of the chunk.  At a reset token the value
        // belongs to the previous segment, but every product it enters is masked out or multiplies a zero.
        Ee[e] = row_prev(E[e], 1.0f);
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
    // ---- decay to the chunk end / to token length-1
    if (t == 15) {
      float* gp = &slot->gamma[8 * g + 32 * hf];
      *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
    }
    if (F.snap >= 0 && t == F.snap) {
      float* gp = &snap->gamma[8 * g + 32 * hf];
      *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
    }
    // ---- row operands for the consumers (Bh, Kh), in their key order: this lane's keys
    //      8g..8g+3 and 8g+4..8g+7 of the half are the (g>>1)-th 8-byte piece of the vectors 2(g&1) and 2(g&1)+1
    //      of block j = hf
    {
      const u32x4_t &r0h = bh_h, &r0l = bh_l;
      const u32x4_t &r1h = kh_h, &r1l = kh_l;
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // element offset of the first piece
      auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
        *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
        *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
      };
      if (!slow) {
        put(slot->AQ[0][0][t], r0h, true); put(slot->AQ[1][0][t], r0l, true);
        put(slot->AQ[0][1][t], r1h, true); put(slot->AQ[1][1][t], r1l, true);
      } else {
        rare_path();
        put(slot->AQ[0][0][t], r0h, row0_keep); put(slot->AQ[1][0][t], r0l, row0_keep);
        put(slot->AQ[0][1][t], r1h, row1_keep); put(slot->AQ[1][1][t], r1l, row1_keep);
      }
      if (F.snap >= 0) {
        rare_path();
        const bool sk = (keep_snap >> t) & 1u;
        put(snap->AQ[0][0][t], r0h, sk); put(snap->AQ[1][0][t], r0l, sk);
        put(snap->AQ[0][1][t], r1h, sk); put(snap->AQ[1][1][t], r1l, sk);
      }
    }
    // ---- transposed update operands of key tiles 2hf, 2hf+1 by MFMA (at^T,
    //      qt^T): the accumulator layout of D (lane = key, registers = 4 consecutive tokens) is the A-operand
    //      layout of the state update
    {
      const u32x4_t &t0h = at_h, &t0l = at_l;
      const u32x4_t &t1h = qt_h, &t1l = qt_l;
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const u32x4_t sel = P.sel[x2];
        const f32x4_t d0h = mfma(t0h, sel, zero4), d0l = mfma(t0l, sel, zero4);
        const f32x4_t d1h = mfma(t1h, sel, zero4), d1l = mfma(t1l, sel, zero4);
        if (keep_upd == 0xffffu) {
          slot->BT[0][tile][lane] = join(plain_pack(d0h), plain_pack(d0l));
          slot->BT[1][tile][lane] = join(plain_pack(d1h), plain_pack(d1l));
        } else {
          rare_path();
          slot->BT[0][tile][lane] = join(masked_pack(d0h, keep_upd), masked_pack(d0l, keep_upd));
          slot->BT[1][tile][lane] = join(masked_pack(d1h, keep_upd), masked_pack(d1l, keep_upd));
        }
      }
    }
    // ---- partial Gram sums over this half's keys (accumulator layout: column n = lane%16, rows 4g..4g+3)
#pragma unroll
    for (int part = 0; part < 3; ++part) {
      const u32x4_t bA = part == 2 ? bh_l : bh_h, kA = part == 2 ? kh_l : kh_h;
      const u32x4_t aA = part == 2 ? at_l : at_h, qA = part == 2 ? qt_l : qt_h;
      const u32x4_t aB = part == 1 ? at_l : at_h, qB = part == 1 ? qt_l : qt_h;
      const u32x4_t bB = part == 1 ? bh_l : bh_h, kB = part == 1 ? kh_l : kh_h;
      Gab = mfma(bA, aB, Gab);      // [m][n] = bh_m . at_n
      GabT = mfma(aA, bB, GabT);    // [m][n] = at_m . bh_n
      G1 = mfma(qA, bB, G1);      // Mbr^T[m][n] = qt_m . bh_n
      G2 = mfma(aA, kB, G2);      // Mka^T[m][n] = at_m . kh_n
      G3 = mfma(qA, kB, G3);      // Mkr^T[m][n] = qt_m . kh_n
    }
  }
  __builtin_amdgcn_s_setprio(3);
  // ---- triangular masks: later rows m for column n
  const int n = t;
  auto mask_tiles = [&](int i, bool lt, bool le, bool gt, bool ge) {
    Gab[i] = lt ? Gab[i] : 0.f;
    GabT[i] = gt ? GabT[i] : 0.f;
    G1[i] = ge ? G1[i] : 0.f;
    G2[i] = gt ? G2[i] : 0.f;
    G3[i] = ge ? G3[i] : 0.f;
  };
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      mask_tiles(i, m < n, m <= n, m > n, m >= n);
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      mask_tiles(i, (m < n) && same, (m <= n) && same, (m > n) && same, (m >= n) && same);
    }
  }
  // ---- (I - M)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M) in single bf16, M = Mba^T
  auto single = [&](const f32x4_t d) {
    u32x4_t o = {pack_rn(d[0], d[1]), pack_rn(d[2], d[3]), 0u, 0u};
    return o;
  };
  f32x4_t Mp = GabT, MpT = Gab;
  f32x4_t Pm = Mp;
#pragma unroll
  for (int i = 0; i < 4; ++i) Pm[i] += (4 * g + i == n) ? 1.f : 0.f;
#pragma unroll
  for (int lvl = 0; lvl < 3; ++lvl) {
    const u32x4_t om = single(Mp), omt = single(MpT);
    const f32x4_t M2T = mfma(om, omt, zero4);      // (M^2)^T
    if (lvl < 2) Mp = mfma(omt, om, zero4);        // M^2: A rows from the transpose, B columns from M
    MpT = M2T;
    Pm = mfma(single(MpT), single(Pm), Pm);        // P += M^(2^(lvl+1)) P
  }
  uint32_t hi0, lo0, hi1, lo1;
  auto park = [&](int which, const f32x4_t d) {
    split2(d[0], d[1], hi0, lo0);
    split2(d[2], d[3], hi1, lo1);
    slot->Mt[which][lane] = make_uint4(hi0, hi1, lo0, lo1);
  };
  park(0, Pm); park(1, G1); park(2, G2); park(3, G3);
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
  }
  __builtin_amdgcn_s_setprio(0);
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds S^T (G^T in the reverse sweep) for value rows 16q..16q+15 as four 16x16 accumulator tiles: lane
// (n = lane%16, g = lane/16), S[tile][i] = S[value 16q+n][key 16*tile + 4g + i].
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

// Uniform output cursors of a consumer, moved by one chunk per call.
struct OutCursor {
  char* y;             // A.gv at (b, c0, h, 0)
  char* sa;            // A.dsa at the same place (16-bit fixed point scaled per chunk and wave: chunk_common.h)
  int* scale;          // this wave's scale exponent of the chunk
  size_t tok_bytes;    // bytes between consecutive tokens in y and in sa
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + value
};

// element offset of this lane's four consecutive keys of a state tile
__device__ __forceinline__ size_t state_off(const Wkv7Args& A, int64_t b, int64_t h, int q, int lane, int tile) {
  return (((size_t)b * A.H + h) * 64 + 16 * q + (lane & 15)) * 64 + 16 * tile + 4 * (lane >> 4);
}
__device__ __forceinline__ f32x4_t load_state_tile(const void* p, int f32, size_t off) {
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
__device__ __forceinline__ void store_state_tile(void* p, int f32, size_t off, const f32x4_t v) {
  if (f32) *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + off) = make_float4(v[0], v[1], v[2], v[3]);
  else *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p) + off) = make_uint2(pack_rn(v[0], v[1]), pack_rn(v[2], v[3]));
}

// The state-dependent part of one chunk.  `next` is the slot of the chunk handled after this one (null after the
// last one); `next_ready` waits until its producer has published it.
template <class WaitNext>
__device__ __forceinline__ bool consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
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
  // the cotangent of the chunk-end state, decayed over the chunk
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    C.S[tile][0] *= gm[tile].x; C.S[tile][1] *= gm[tile].y; C.S[tile][2] *= gm[tile].z; C.S[tile][3] *= gm[tile].w;
  }

  // B operands from the state: MFMA j contracts over the keys of tiles 2j and 2j+1
  u32x4_t Sh[2], Sl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2_keep(C.S[2 * j][0], C.S[2 * j][1], hi, lo); Sh[j][0] = hi; Sl[j][0] = lo;
    split2_keep(C.S[2 * j][2], C.S[2 * j][3], hi, lo); Sh[j][1] = hi; Sl[j][1] = lo;
    split2_keep(C.S[2 * j + 1][0], C.S[2 * j + 1][1], hi, lo); Sh[j][2] = hi; Sl[j][2] = lo;
    split2_keep(C.S[2 * j + 1][2], C.S[2 * j + 1][3], hi, lo); Sh[j][3] = hi; Sl[j][3] = lo;
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
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
    asm volatile("" ::: "memory");
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;
  }
  // the cotangent of the returned state enters at token length-1 (one chunk per sequence)
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4_t gh, gl;
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * j + x2;
        f32x4_t gs = load_state_tile(A.gs_out, A.st_f32, state_off(A, b, h, C.q, lane, tile));
        const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
        gs[0] *= sg.x; gs[1] *= sg.y; gs[2] *= sg.z; gs[3] *= sg.w;
        if (keep) C.S[tile] += gs;
        uint32_t hi, lo;
        split2(gs[0], gs[1], hi, lo); gh[2 * x2] = hi; gl[2 * x2] = lo;
        split2(gs[2], gs[3], hi, lo); gh[2 * x2 + 1] = hi; gl[2 * x2 + 1] = lo;
      }
      const u32x4_t a0h = *reinterpret_cast<const u32x4_t*>(&snapslot->AQ[0][0][n][32 * j + 8 * g]);
      const u32x4_t a0l = *reinterpret_cast<const u32x4_t*>(&snapslot->AQ[1][0][n][32 * j + 8 * g]);
      const u32x4_t a1h = *reinterpret_cast<const u32x4_t*>(&snapslot->AQ[0][1][n][32 * j + 8 * g]);
      const u32x4_t a1l = *reinterpret_cast<const u32x4_t*>(&snapslot->AQ[1][1][n][32 * j + 8 * g]);
      W = mfma(a0h, gh, W); Y = mfma(a1h, gh, Y);
      W = mfma(a0h, gl, W); Y = mfma(a1h, gl, Y);
      W = mfma(a0l, gh, W); Y = mfma(a1l, gh, Y);
    }
  }

  // At, Qt, Mka, Mkr, v^T are dead now: fetch the next chunk's into the same registers
  bool ok = true;
  if (next != nullptr) {
    ok = next_ready();
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
  // update, tile by tile: rows = keys.  G <- Gh + At^T DSA^T + Qt^T DY^T
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    f32x4_t acc = C.S[tile];
    acc = mfma(bt[0][tile], sHH, acc);
    acc = mfma(bt[1][tile], vv, acc);
    acc = mfma(bt[0][tile], sL0, acc);
    C.S[tile] = acc;
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  const uint32_t y01 = pack_rn(Y[0], Y[1]), y23 = pack_rn(Y[2], Y[3]);
  char* const yl = oc.y + (size_t)oc.voff * 2;
  // dsa leaves as 16-bit fixed point with one power-of-two scale per chunk and wave (chunk_common.h), at half the
  // bytes of fp32; the exponent goes to a side array.
  const int kexp = dsa_scale_exponent(SA);
  const uint32_t d01 = pack_dsa2(SA[0], SA[1], kexp), d23 = pack_dsa2(SA[2], SA[3], kexp);
  if (lane == 0) *oc.scale = kexp;
  char* const sl = oc.sa + (size_t)oc.voff * 2;
  if (nvalid == CK) {
    *reinterpret_cast<uint16_t*>(yl) = (uint16_t)(y01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + oc.tok_bytes) = (uint16_t)(y01 >> 16);
    *reinterpret_cast<uint16_t*>(yl + 2 * oc.tok_bytes) = (uint16_t)(y23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + 3 * oc.tok_bytes) = (uint16_t)(y23 >> 16);
    *reinterpret_cast<uint16_t*>(sl) = (uint16_t)(d01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(sl + oc.tok_bytes) = (uint16_t)(d01 >> 16);
    *reinterpret_cast<uint16_t*>(sl + 2 * oc.tok_bytes) = (uint16_t)(d23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(sl + 3 * oc.tok_bytes) = (uint16_t)(d23 >> 16);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        const uint32_t yv = (i & 2) ? y23 : y01, dv = (i & 2) ? d23 : d01;
        *reinterpret_cast<uint16_t*>(yl + i * oc.tok_bytes) = (uint16_t)((i & 1) ? (yv >> 16) : (yv & 0xffffu));
        *reinterpret_cast<uint16_t*>(sl + i * oc.tok_bytes) = (uint16_t)((i & 1) ? (dv >> 16) : (dv & 0xffffu));
      }
    }
  }
  oc.y -= CK * oc.tok_bytes;
  oc.sa -= CK * oc.tok_bytes;
  oc.scale -= 4;

  return ok;
}

}  // namespace

// Chunks are handled from the last one down; step j
// handles chunk c(j) = nch - 1 - j in slot j % RING.  Producer p fills the slot once every consumer has released step j - RING,
// then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier step, so
// the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_bwd_a_kernel(Wkv7Args A) {
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
  // the returned state is the reset state there (associative-scan rule), a constant
  const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
  // reverse sweep: does a cotangent of the returned state enter at token length-1?
  const bool inject = A.gs_out != nullptr && !q2drop;
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  if (wave < NCONS) {
    // the chunk-to-chunk dependency runs through the consumers: let them issue ahead of the producers
    __builtin_amdgcn_s_setprio(3);
    Consumer C;
    C.q = wave;
    C.lane = lane;
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;

    const int64_t first_tok = (int64_t)(nch - 1) * CK;
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T + first_tok) * A.H + h) * 64;
    oc.y = reinterpret_cast<char*>(A.gv) + el0 * 2;
    oc.sa = reinterpret_cast<char*>(A.dsa) + el0 * 2;
    oc.scale = dsa_scales(A.e3, b, h, A.H, nch, nch - 1) + wave;

    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * wave + (lane & 15));
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    Ops ops;
    bool ok = true;
    if (nch > 0) {
      ok = wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], wave, lane);
    }
    for (int j = 0; j < nch && ok; ++j) {
      const int c = nch - 1 - j;
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = j % RING, sn = (j + 1) % RING;
      const Slot* next = (j + 1 < nch) ? &slots[sn] : nullptr;
      ok = consume(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, c == csnap, q2drop, oc,
                        [&]() { return wait_ready(sy, sn, j + 2); });
      // every LDS read of slot si has returned: its data went into the MFMAs above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // cotangent of the input state; with length == 0 the returned state is the input state itself
    const bool pass = L == 0 && inject;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const size_t off = state_off(A, b, h, wave, lane, tile);
      f32x4_t gsv = C.S[tile];
      if (pass) gsv += load_state_tile(A.gs_out, A.st_f32, off);
      store_state_tile(A.gs, A.st_f32, off, gsv);
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
      mask_raw(raw, F.nvalid, lane);
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
    poison_token_rows(A.gv, 2, b, h, A.T, A.H);
    // the workspace of this (sequence, head) reads as NaN for the next two sweeps: every tile gets the reserved exponent
    for (int i = threadIdx.x; i < nch * NCONS; i += blockDim.x) dsa_scales(A.e3, b, h, A.H, nch, 0)[i] = DSA_BAD;
    poison_state(A.gs, A.st_f32, b, h, A.H);
  }
}

// Reverse sweep of the backward pass: gv, the workspace dsa (cotangent of sa per token) and gs.
hipError_t launch_wkv7_chunk_bwd_a(const Wkv7Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_bwd_a_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_bwd_a_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
