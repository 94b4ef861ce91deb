// WKV7 chunked forward for bf16 I/O on gfx950: 16 tokens at a time on the matrix cores, fp16 operands.
//
// Recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220), S[i][j] = value row i, key col j:
//     sa_t = S_{t-1} a_t ;  S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;  y_t = S_t r_t ;  d_t = exp(-exp(w_t))
// A chunk of 16 tokens entering with state S0 is evaluated in closed form.  With l_t = log d_t, Lc_t = sum_{s<=t} l_s:
//     at_t = a_t exp(Lc_{t-1})   qt_t = r_t exp(Lc_t)   kh_s = k_s exp(-Lc_s)   bh_s = b_s exp(-Lc_s)
//     ke_s = k_s exp(Lc_15 - Lc_s)   be_s = b_s exp(Lc_15 - Lc_s)           (update operands, referenced to the chunk end)
//     Mba[s][t] = bh_s.at_t (s<t)   Mka[s][t] = kh_s.at_t (s<t)   Mbr[s][t] = bh_s.qt_t (s<=t)   Mkr likewise
//     P  = (I - Mba)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M)                    (M^16 = 0)
//     W  = S0 At^T + V^T Mka      SA = W P      Y = S0 Qt^T + SA Mbr + V^T Mkr      S_C = S0 diag(E_15) + SA^T.. Be + V^T.. Ke
//
// Operand formats.  at, qt, ke, be, v, the state, W, SA, P and the three M tiles are bounded by the inputs' magnitudes:
// they go to the matrix cores as single fp16 numbers (11 significant bits; the values must stay inside the fp16
// range, |x| < 65504) -- but for Mkr, which multiplies v straight into y (its diagonal is the token's own k.r) and is
// fed as an fp16 pair hi + lo: one more K = 16 instruction per consumer and chunk for a y error 3.5 times smaller
// where the decay is fast.  kh and bh carry exp(-Lc) and need the fp32 exponent range: the four Gram tiles are formed from
// bf16 hi + lo pairs of kh, bh, at, qt (three partial products).  The state itself stays in fp32 accumulator
// registers for the whole sequence, stored transposed (key x value tiles).
//
// Work split: one workgroup of twelve waves per (sequence, head).  Four are consumers: consumer q owns value rows
// 16q..16q+15 of the state and runs the state-dependent part of every chunk (12 MFMAs).  Eight are producers: producer p
// prepares chunks p, p+8, ... (decay scan, scaled operands, Gram tiles, triangular inverse) into a ring of LDS slots.  Operands
// that the consumers need transposed (be, ke, v: token-contiguous per key or value) are written row-major and read
// with the LDS transpose load (ds_read_b64_tr_b16).  Synchronisation is a pair of LDS sequence numbers per slot
// with a bounded wait (chunk_common.h).
// new_starts inside a chunk restart the cumulative decay and mask the Gram tiles (rare, uniform branch).  The one
// chunk that holds token length-1 gets a second set of update operands, referenced to that token, for the state
// snapshot.
//
// Range: a key channel whose total log decay over a chunk is below -80 gets its steps of that chunk scaled to a total
// of -80 (cap_chunk_decay), so that exp(-Lc) stays finite in fp32.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 8;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 10;          // slots in flight

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// round to nearest fp16 pair: one v_cvt_pk_f16_f32
__device__ __forceinline__ uint32_t pack_h(float x0, float x1) {
  const f16x2_t p = {(_Float16)x0, (_Float16)x1};
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ u32x2_t pack_h4(const f32x4_t d) { return u32x2_t{pack_h(d[0], d[1]), pack_h(d[2], d[3])}; }

// D[m][n] += sum_k A[m][k] B[k][n]; lane (x = lane % 16, g = lane / 16) holds row m = x of A, column n = x of B and
// k-slots 8g..8g+7 (K = 32) or 4g..4g+3 (K = 16); D: lane (n, g) holds rows 4g..4g+3 of column n.
__device__ __forceinline__ f32x4_t mfma_h(const u32x4_t a, const u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma_h16(const u32x2_t a, const u32x2_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
}

// LDS transpose load.  Within each group of 16 lanes, lane i = 4r + j points at 4 consecutive 16-bit elements
// (row r of 4, columns 4j..4j+3 of 16) and receives column i of the 4 x 16 block: rows 0..3 of column i.
__device__ __forceinline__ u32x2_t lds_tr4(const uint16_t* p) {
  typedef __attribute__((address_space(3))) s16x4_t* lds_ptr;
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  return __builtin_bit_cast(u32x2_t, v);
}

// value of lane 15 of the row in every lane of the row (row_newbcast:15)
__device__ __forceinline__ float row_last(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x15F, 0xf, 0xf, true));
}
// value of the previous lane of the row, 0 in lane 0 of the row
__device__ __forceinline__ float row_prev0(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true));
}

// One chunk's operands as the consumers read them.
struct __attribute__((aligned(16))) Slot {
  // fp16 rows [token][RS].  AQ: at, qt; within a row the 16-byte vector (j, g) at element 32j + 8g holds keys
  // 32j+4g..+3 followed by keys 32j+16+4g..+3, the key order of the consumers' state tiles.  Rows the entering state
  // does not reach are zero; qt rows whose y is defined as zero are zero.
  uint16_t AQ[2][CK][RS];
  uint16_t BK[2][CK][RS];      // be, ke in natural key order (tokens outside the last segment are zero)
  uint16_t V[CK][RS];          // v in fp16
  u32x2_t P[64], Ka[64];       // lane-indexed fp16: column t = lane%16, rows 4g..4g+3 (g = lane/16) of P and Mka
  u32x4_t BrKr[64];            // the same of Mbr followed by Mkr
  u32x2_t KrLo[64];            // Mkr minus its fp16 value, in fp16: Mkr multiplies v straight into y
  float gamma[64];             // exp(Lc_15)
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the carried state passes through the whole chunk (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
// Update operands referenced to token length-1; only one chunk per sequence needs them.
struct __attribute__((aligned(16))) SnapSlot {
  uint16_t BK[2][CK][RS];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys {8g..8g+7} u {32+8g..32+8g+7}: exactly the A/B
// operand layout of the Gram MFMAs (row/column = token, k-slots = keys), and one 16-byte global load per half.
struct Raw {
  uint4 r[2], w[2], k[2], v[2], a[2], b[2];
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
  ld(A.r, x.r); ld(A.w, x.w); ld(A.k, x.k); ld(A.v, x.v); ld(A.a, x.a); ld(A.b, x.b);
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

__device__ __forceinline__ uint4 pack_h8(const float (&f)[8]) {
  return make_uint4(pack_h(f[0], f[1]), pack_h(f[2], f[3]), pack_h(f[4], f[5]), pack_h(f[6], f[7]));
}

// Everything of one chunk that does not depend on the carried state.  The two 32-key halves go through the same
// pipeline one after the other, which keeps the live register set small.
//
// Issue priorities: at equal priority a SIMD serves its oldest wave first, and time stamps show the youngest of the
// three producers of a SIMD taking 10 000 cycles for a chunk where the oldest takes 6 000.  Raising a producer's
// priority as it advances through its chunk evens that out and makes an isolated launch 4 % faster, but launches
// issued back to back (the GPU at its power limit) 2.8 % slower, so this kernel's producers stay at the default
// priority; the WKV6 forward, where the same steps gain 3.5 % back to back, has them.
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
  const int t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint4 zero16 = make_uint4(0u, 0u, 0u, 0u);
  const bool slow = F.ns != 0;                    // a reset in this chunk or at the first token of the next
  const uint32_t resets = F.ns & 0xffffu;
  // reset bookkeeping (uniform values unless they depend on t)
  int lastseg = 0, seg_src = 0;
  bool row0_keep = true, row1_keep = true, restart = false, at_reset = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
    lastseg = seg_of(F.ns, 15);
    const int myseg = seg_of(F.ns, t);
    row0_keep = myseg == 0;                                          // the entering state reaches this token
    row1_keep = row0_keep && !(F.compat && ((F.ns >> (t + 1)) & 1u)); // y[t] is defined as zero before a reset
    if (resets) keep_upd = 0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u);   // tokens from the last reset on
    at_reset = (resets >> t) & 1u;
    const uint32_t upto = resets & ((2u << t) - 1u);
    const int pr = upto ? 31 - __builtin_clz(upto) : 0;             // last reset at or before this token
    restart = pr > 0;
    seg_src = (lane & 48) | (pr > 0 ? pr - 1 : 0);
    if (F.snap >= 0) {
      const uint32_t us = resets & keep_snap;
      if (us) keep_snap &= ~((1u << (31 - __builtin_clz(us))) - 1u);   // tokens of length-1's segment up to it
    }
  }

  // Gram tiles in accumulator layout [row m = A-operand token][column n = B-operand token]
  f32x4_t Gab = zero4, GabT = zero4;   // bh_m.at_n and at_m.bh_n
  f32x4_t G1 = zero4, G2 = zero4, G3 = zero4;   // Mka, Mbr, Mkr
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ---- v in fp16, row-major (the consumers read it transposed)
    {
      float fv[8];
      unpack8(x.v[hf], fv);
      *reinterpret_cast<uint4*>(&slot->V[t][32 * hf + 8 * g]) = pack_h8(fv);
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
        if (at_reset) fa[e] = 0.f;                      // the state entering a reset token is zero: sa = 0
      }
    }
    // ---- scaled operands
    float fat[8], fqt[8], fkh[8], fbh[8], fke[8], fbe[8];
    {
      float fr[8], fk[8], fb[8];
      unpack8(x.r[hf], fr); unpack8(x.k[hf], fk); unpack8(x.b[hf], fb);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // cap_chunk_decay keeps the running sums at or above MIN_CUM_L2: exp2(-l2) is finite
        const float l2 = E[e];
        E[e] = exp2_fast(l2);
        const float einv = exp2_fast(-l2);
        // a_t times the decay up to the previous token (1 for the first token of the chunk: fa0 carries that lane).
        // At a reset token the value belongs to the previous segment, but every product it enters is masked out or
        // multiplies a zero.
        const float fa0 = (t == 0) ? fa[e] : 0.f;
        fat[e] = fmaf(fa[e], row_prev0(E[e]), fa0);
        fqt[e] = fr[e] * E[e];
        fkh[e] = fk[e] * einv;
        fbh[e] = fb[e] * einv;
        // times the decay from the (last) segment start to the chunk end
        const float gam = row_last(E[e]);
        fke[e] = fkh[e] * gam;
        fbe[e] = fbh[e] * gam;
      }
    }
    // ---- decay to the chunk end
    if (t == 15) {
      float* gp = &slot->gamma[8 * g + 32 * hf];
      *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
    }
    // ---- update operands for the consumers, row-major in natural key order
    {
      uint4 be = pack_h8(fbe), ke = pack_h8(fke);
      if (keep_upd != 0xffffu) {
        rare_path();
        if (!((keep_upd >> t) & 1u)) be = ke = zero16;     // tokens before the last reset do not reach the chunk end
      }
      *reinterpret_cast<uint4*>(&slot->BK[0][t][32 * hf + 8 * g]) = be;
      *reinterpret_cast<uint4*>(&slot->BK[1][t][32 * hf + 8 * g]) = ke;
    }
    // ---- the same referenced to token length-1 (one chunk per sequence)
    if (F.snap >= 0) {
      rare_path();
      const bool sk = (keep_snap >> t) & 1u;
      float sbe[8], ske[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gs = __shfl(E[e], (lane & 48) | F.snap, 64);
        sbe[e] = fbh[e] * gs;
        ske[e] = fkh[e] * gs;
      }
      *reinterpret_cast<uint4*>(&snap->BK[0][t][32 * hf + 8 * g]) = sk ? pack_h8(sbe) : zero16;
      *reinterpret_cast<uint4*>(&snap->BK[1][t][32 * hf + 8 * g]) = sk ? pack_h8(ske) : zero16;
      if (t == F.snap) {
        float* gp = &snap->gamma[8 * g + 32 * hf];
        *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
      }
    }
    // ---- row operands for the consumers (at, qt) in their key order: this lane's keys 8g..8g+3 and 8g+4..8g+7 of
    //      the half are the (g>>1)-th 8-byte piece of the vectors 2(g&1) and 2(g&1)+1 of block j = hf
    {
      uint4 ah = pack_h8(fat), qh = pack_h8(fqt);
      if (slow) {
        rare_path();
        if (!row0_keep) ah = zero16;
        if (!row1_keep) qh = zero16;
      }
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // element offset of the first piece
      auto put = [&](uint16_t* row, const uint4 v) {
        *reinterpret_cast<uint2*>(row + e0) = make_uint2(v.x, v.y);
        *reinterpret_cast<uint2*>(row + e0 + 8) = make_uint2(v.z, v.w);
      };
      put(slot->AQ[0][t], ah);
      put(slot->AQ[1][t], qh);
    }
    // ---- bf16 hi/lo pairs of the Gram operands and the partial Gram sums over this half's keys
    u32x4_t at_h, at_l, qt_h, qt_l, kh_h, kh_l, bh_h, bh_l;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 2 * j;
      uint32_t hi, lo;
      split2(fat[e], fat[e + 1], hi, lo); at_h[j] = hi; at_l[j] = lo;
      split2(fqt[e], fqt[e + 1], hi, lo); qt_h[j] = hi; qt_l[j] = lo;
      split2(fkh[e], fkh[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
      split2(fbh[e], fbh[e + 1], hi, lo); bh_h[j] = hi; bh_l[j] = lo;
    }
#pragma unroll
    for (int part = 0; part < 3; ++part) {
      const u32x4_t bA = part == 2 ? bh_l : bh_h, kA = part == 2 ? kh_l : kh_h;
      const u32x4_t aA = part == 2 ? at_l : at_h;
      const u32x4_t aB = part == 1 ? at_l : at_h, qB = part == 1 ? qt_l : qt_h;
      const u32x4_t bB = part == 1 ? bh_l : bh_h;
      Gab = mfma(bA, aB, Gab);      // [m][n] = bh_m . at_n
      GabT = mfma(aA, bB, GabT);    // [m][n] = at_m . bh_n
      G1 = mfma(kA, aB, G1);        // Mka[m][n] = kh_m . at_n
      G2 = mfma(bA, qB, G2);        // Mbr[m][n] = bh_m . qt_n
      G3 = mfma(kA, qB, G3);        // Mkr[m][n] = kh_m . qt_n
    }
  }
  // ---- triangular masks: earlier rows m for column n
  const int n = t;
  auto mask_tiles = [&](int i, bool lt, bool le, bool gt) {
    Gab[i] = lt ? Gab[i] : 0.f;
    GabT[i] = gt ? GabT[i] : 0.f;
    G1[i] = lt ? G1[i] : 0.f;
    G2[i] = le ? G2[i] : 0.f;
    G3[i] = le ? G3[i] : 0.f;
  };
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      mask_tiles(i, m < n, m <= n, m > n);
    }
  } else {
    rare_path();
    const bool keepy = !(F.compat && ((F.ns >> (n + 1)) & 1u));   // y[n] may be defined as zero
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      mask_tiles(i, (m < n) && same, (m <= n) && same && keepy, (m > n) && same);
    }
  }
  // ---- P = (I - M)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M), M = Mba, fp16 operands.  Packed accumulator registers
  //      of X are X^T as an A operand and X as a B operand, so mfma_h16(pk(X), pk(Z)) = X^T Z.
  f32x4_t Mp = Gab, MpT = GabT;
  f32x4_t Pm = Mp;
#pragma unroll
  for (int i = 0; i < 4; ++i) Pm[i] += (4 * g + i == n) ? 1.f : 0.f;
#pragma unroll
  for (int lvl = 0; lvl < 3; ++lvl) {
    const u32x2_t om = pack_h4(Mp), omt = pack_h4(MpT);
    const f32x4_t M2T = mfma_h16(om, omt, zero4);        // (M^2)^T
    if (lvl < 2) Mp = mfma_h16(omt, om, zero4);          // M^2
    MpT = M2T;
    Pm = mfma_h16(pack_h4(MpT), pack_h4(Pm), Pm);        // P += M^(2^(lvl+1)) P
  }
  slot->P[lane] = pack_h4(Pm);
  slot->Ka[lane] = pack_h4(G1);
  {
    const u32x2_t br = pack_h4(G2), kr = pack_h4(G3);
    slot->BrKr[lane] = u32x4_t{br[0], br[1], kr[0], kr[1]};
    const f16x4_t krh = __builtin_bit_cast(f16x4_t, kr);
    f32x4_t rest;
#pragma unroll
    for (int i = 0; i < 4; ++i) rest[i] = G3[i] - (float)krh[i];
    slot->KrLo[lane] = pack_h4(rest);
  }
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds S^T for value rows 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16, g = lane/16),
// S[tile][i] = S[value 16q+n][key 16*tile + 4g + i].
// Byte offsets of this lane's operands inside a slot, computed once (the asm statement keeps the compiler from
// recomputing them from the lane index in every chunk).
struct LaneOffs {
  uint32_t aq, l8, l16, vv, upd, gm, ypark;
};
__device__ __forceinline__ LaneOffs lane_offs(int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
  LaneOffs o;
  o.aq = (uint32_t)(offsetof(Slot, AQ) + (n * RS + 8 * g) * 2);
  o.l8 = (uint32_t)(offsetof(Slot, P) + lane * 8);
  o.l16 = (uint32_t)(offsetof(Slot, BrKr) + lane * 16);
  o.vv = (uint32_t)(offsetof(Slot, V) + ((4 * g + (n >> 2)) * RS + 16 * q + 4 * (n & 3)) * 2);
  o.upd = (uint32_t)(offsetof(Slot, BK) + ((4 * g + (n >> 2)) * RS + 4 * (n & 3)) * 2);
  o.gm = (uint32_t)(offsetof(Slot, gamma) + 16 * g);
  o.ypark = (uint32_t)(offsetof(Slot, V) + ((4 * g) * RS + 16 * q + n) * 2);
  asm volatile("" : "+v"(o.aq), "+v"(o.l8), "+v"(o.l16), "+v"(o.vv), "+v"(o.upd), "+v"(o.gm), "+v"(o.ypark));
  return o;
}
struct Consumer {
  f32x4_t S[4];
  int q, lane;
  LaneOffs off;
};

// Operands a consumer fetches a chunk ahead: everything the W / SA / Y chain reads.
struct Ops {
  u32x4_t aq[2][2];        // [at|qt][j]: rows in the key order of the state tiles
  u32x2_t P, Ka;
  u32x4_t BrKr;
  u32x2_t KrLo;
  u32x2_t vv;              // v^T of this wave's value tile: tokens 4g..4g+3 of value n
  int keep_end;
};

__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, const LaneOffs& f) {
  const char* const sb = reinterpret_cast<const char*>(slot);
#pragma unroll
  for (int ar = 0; ar < 2; ++ar)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      o.aq[ar][j] = *reinterpret_cast<const u32x4_t*>(sb + f.aq + ar * (CK * RS * 2) + j * 64);
  o.P = *reinterpret_cast<const u32x2_t*>(sb + f.l8);
  o.Ka = *reinterpret_cast<const u32x2_t*>(sb + f.l8 + (offsetof(Slot, Ka) - offsetof(Slot, P)));
  o.BrKr = *reinterpret_cast<const u32x4_t*>(sb + f.l16);
  o.KrLo = *reinterpret_cast<const u32x2_t*>(sb + f.l8 + (offsetof(Slot, KrLo) - offsetof(Slot, P)));
  o.vv = lds_tr4(reinterpret_cast<const uint16_t*>(sb + f.vv));
  o.keep_end = slot->keep_end;
}

// A operands of the state update of one key tile: be^T then ke^T, tokens 4g..4g+3 of key 16*tile + n
__device__ __forceinline__ u32x4_t load_upd(const uint16_t (*bk)[CK][RS], int tile, int lane) {
  const int n = lane & 15, g = lane >> 4;
  const int row = 4 * g + (n >> 2), col = 16 * tile + 4 * (n & 3);
  const u32x2_t be = lds_tr4(&bk[0][row][col]), ke = lds_tr4(&bk[1][row][col]);
  return u32x4_t{be[0], be[1], ke[0], ke[1]};
}

// Uniform output cursors of a consumer, moved by one chunk per call.
struct OutCursor {
  char* y;             // A.out at (b, c0, h, 0)
  char* sa;            // A.sa (or null) at the same place
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
// last one); `next_ready` waits until its producer has published it.  Returns false when that wait ran out.
template <bool PARK, class PeekNext, class WaitNext>
__device__ __forceinline__ bool consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
                                        const Slot* __restrict__ next, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool q2drop,
                                        OutCursor& oc, PeekNext&& peek_next, WaitNext&& next_ready) {
  const int lane = C.lane, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // the next chunk's sequence number, requested now and looked at after the W / SA / Y chain
  const int peeked = next != nullptr ? peek_next() : 0;
  // update operands of this chunk: needed last, so their latency hides behind the W / SA chain
  u32x4_t up[4];
  float4 gm[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const char* const sb = reinterpret_cast<const char*>(slot);
    const u32x2_t be = lds_tr4(reinterpret_cast<const uint16_t*>(sb + C.off.upd + 32 * tile));
    const u32x2_t ke = lds_tr4(reinterpret_cast<const uint16_t*>(sb + C.off.upd + CK * RS * 2 + 32 * tile));
    up[tile] = u32x4_t{be[0], be[1], ke[0], ke[1]};
    gm[tile] = *reinterpret_cast<const float4*>(sb + C.off.gm + 64 * tile);
  }
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
  // B operands from the state: MFMA j contracts over the keys of tiles 2j and 2j+1
  u32x4_t Sh[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    Sh[j] = u32x4_t{pack_h(C.S[2 * j][0], C.S[2 * j][1]), pack_h(C.S[2 * j][2], C.S[2 * j][3]),
                    pack_h(C.S[2 * j + 1][0], C.S[2 * j + 1][1]), pack_h(C.S[2 * j + 1][2], C.S[2 * j + 1][3])};
  f32x4_t W = zero4;              // [token 4g+i][value n], two interleaved accumulation chains
  f32x4_t Y = mfma_h16(o.KrLo, o.vv, zero4);    // the low part of Mkr^T V^T: no state in it, off the critical path
  mfma_shape_fence(Y);                          // a K = 16 result enters a K = 32 chain
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    W = mfma_h(o.aq[0][j], Sh[j], W);
    Y = mfma_h(o.aq[1][j], Sh[j], Y);
  }
  mfma_shape_fence(W);                          // a K = 32 result enters a K = 16 instruction: the pairing that fails
  W = mfma_h16(o.Ka, o.vv, W);                  // W += Mka^T V^T
  const f32x4_t SA = mfma_h16(o.P, pack_h4(W), zero4);
  const u32x2_t sp = pack_h4(SA);
  const u32x4_t sv = {sp[0], sp[1], o.vv[0], o.vv[1]};   // SA^T (tokens 4g..4g+3) then v^T: B operand of Y and the update
  Y = mfma_h(o.BrKr, sv, Y);                    // Y += Mbr^T SA^T + Mkr^T V^T
  // everything fetched a chunk ahead is dead now: fetch the next chunk's into the same registers
  bool ok = true;
  if (next != nullptr) {
    ok = next_ready(peeked);
    load_ops(o, next, C.off);
  }
  // state snapshot for `length` (one chunk per sequence)
  if (is_snap) {
    rare_path();
    const bool keep = slot->keep_snap != 0;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const u32x4_t su = load_upd(snapslot->BK, tile, lane);
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      f32x4_t acc = zero4;
      if (keep) {
        acc[0] = C.S[tile][0] * sg.x; acc[1] = C.S[tile][1] * sg.y;
        acc[2] = C.S[tile][2] * sg.z; acc[3] = C.S[tile][3] * sg.w;
      }
      acc = mfma_h(su, sv, acc);
      store_state_tile(A.new_s, A.st_f32, state_off(A, b, h, C.q, lane, tile), q2drop ? zero4 : acc);
    }
  }
  // state update, tile by tile: rows = keys.  S <- S diag(gamma) + Be^T SA^T + Ke^T V^T; a reset inside the chunk
  // cuts the entering state off
  if (keep_end) {
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      f32x4_t acc = C.S[tile];
      acc[0] *= gm[tile].x; acc[1] *= gm[tile].y; acc[2] *= gm[tile].z; acc[3] *= gm[tile].w;
      C.S[tile] = mfma_h(up[tile], sv, acc);
    }
  } else {
    rare_path();
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = mfma_h(up[tile], sv, zero4);
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  const uint32_t y01 = pack_rn(Y[0], Y[1]), y23 = pack_rn(Y[2], Y[3]);
  if (PARK) {
    // The launch that also writes `sa`: y is parked in the value columns of V that only this wave reads (it fetched
    // them a chunk ahead), and the producer that takes the slot next writes the chunk's y to memory as whole rows.
    // Eight narrow stores per chunk hold the consumers up; four do not (measured: 4.5 % off this launch, while the
    // launch without `sa` is 5 % slower this way and keeps its direct stores).
    char* const yp = reinterpret_cast<char*>(const_cast<Slot*>(slot)) + C.off.ypark;
    *reinterpret_cast<uint16_t*>(yp) = (uint16_t)(y01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yp + RS * 2) = (uint16_t)(y01 >> 16);
    *reinterpret_cast<uint16_t*>(yp + 2 * RS * 2) = (uint16_t)(y23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yp + 3 * RS * 2) = (uint16_t)(y23 >> 16);
  }
  char* const yl = oc.y + (size_t)oc.voff * 2;
  if (nvalid == CK) {
    if (!PARK) {
      *reinterpret_cast<uint16_t*>(yl) = (uint16_t)(y01 & 0xffffu);
      *reinterpret_cast<uint16_t*>(yl + oc.tok_bytes) = (uint16_t)(y01 >> 16);
      *reinterpret_cast<uint16_t*>(yl + 2 * oc.tok_bytes) = (uint16_t)(y23 & 0xffffu);
      *reinterpret_cast<uint16_t*>(yl + 3 * oc.tok_bytes) = (uint16_t)(y23 >> 16);
    }
    if (oc.sa != nullptr) {      // the residual for the backward pass, in fp16 like the operand it was used as
      char* const sl = oc.sa + (size_t)oc.voff * 2;
      *reinterpret_cast<uint16_t*>(sl) = (uint16_t)(sp[0] & 0xffffu);
      *reinterpret_cast<uint16_t*>(sl + oc.tok_bytes) = (uint16_t)(sp[0] >> 16);
      *reinterpret_cast<uint16_t*>(sl + 2 * oc.tok_bytes) = (uint16_t)(sp[1] & 0xffffu);
      *reinterpret_cast<uint16_t*>(sl + 3 * oc.tok_bytes) = (uint16_t)(sp[1] >> 16);
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        const uint32_t yv = (i & 2) ? y23 : y01;
        if (!PARK) *reinterpret_cast<uint16_t*>(yl + i * oc.tok_bytes) = (uint16_t)((i & 1) ? (yv >> 16) : (yv & 0xffffu));
        if (oc.sa != nullptr) {
          const uint32_t sv2 = sp[i >> 1];
          *reinterpret_cast<uint16_t*>(oc.sa + (size_t)oc.voff * 2 + i * oc.tok_bytes) =
              (uint16_t)((i & 1) ? (sv2 >> 16) : (sv2 & 0xffffu));
        }
      }
    }
  }
  oc.y += CK * oc.tok_bytes;
  if (oc.sa != nullptr) oc.sa += CK * oc.tok_bytes;
  return ok;
}

// y of chunk jj, parked in the slot by the consumers, to memory: lane l stores 16 bytes of rows l/8 and l/8 + 8
__device__ __forceinline__ void flush_y(const Slot* __restrict__ slot, const Wkv7Args& A, int64_t b, int64_t h, int jj,
                                        int nch, int lane) {
  const int nvalid = (jj + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
  const int r = lane >> 3, piece = lane & 7;
  char* const y0 = reinterpret_cast<char*>(A.out) +
                   ((((size_t)b * A.T + (size_t)jj * CK + r) * A.H + h) * 64 + 8 * piece) * 2;
  const uint4 lo = *reinterpret_cast<const uint4*>(&slot->V[r][8 * piece]);
  const uint4 hi = *reinterpret_cast<const uint4*>(&slot->V[r + 8][8 * piece]);
  if (r < nvalid) *reinterpret_cast<uint4*>(y0) = lo;
  if (r + 8 < nvalid) *reinterpret_cast<uint4*>(y0 + (size_t)8 * A.H * 128) = hi;
}

}  // namespace

// Step j handles chunk j in slot j % RING.  Producer p fills the slot once every consumer has released step j - RING,
// then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier step, so
// the hand-shake cannot cycle.
// PARK: the consumers leave y in the slot and the producers write it out (see `consume`); steps nch .. nch + RING - 1
// of the producers then produce nothing and only write out the y of the last RING chunks.
template <bool PARK>
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_fwd_kernel(Wkv7Args A) {
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
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  // Waves go to the four SIMDs round-robin.  Consumers are waves 0, 1, 4, 5: two of them (two independent dependency
  // chains) and one producer share each of SIMDs 0 and 1, three producers each of SIMDs 2 and 3.  Measured 3.5 %
  // faster than one consumer and two producers on every SIMD: a producer's vector instructions delay the consumer
  // that shares its SIMD, and this way each consumer has one such neighbour instead of two.
  static_assert(NPROD == 8, "the wave-to-role map below is written for 4 consumers and 8 producers");
  const bool is_cons = (wave & 2) == 0 && wave < 8;
  const int cq = (wave & 1) | ((wave >> 1) & 2);                                 // waves 0,1,4,5 -> 0..3
  const int pp = wave >= 8 ? wave - 4 : ((wave & 1) | ((wave >> 1) & 2));        // waves 2,3,6,7 -> 0..3, 8..11 -> 4..7
  if (is_cons) {
    // the chunk-to-chunk dependency runs through the consumers: let them issue ahead of the producers
    __builtin_amdgcn_s_setprio(3);
    Consumer C;
    C.q = cq;
    C.lane = lane;
    C.off = lane_offs(cq, lane);
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = load_state_tile(A.s, A.st_f32, state_off(A, b, h, cq, lane, tile));
    // length == 0: the returned state is the input state (rwkv7.py:203), or the reset state under the associative rule
    if (L == 0) {
#pragma unroll
      for (int tile = 0; tile < 4; ++tile)
        store_state_tile(A.new_s, A.st_f32, state_off(A, b, h, cq, lane, tile), q2drop ? zero4 : C.S[tile]);
    }
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T) * A.H + h) * 64;
    oc.y = reinterpret_cast<char*>(A.out) + el0 * 2;
    oc.sa = A.sa ? reinterpret_cast<char*>(A.sa) + el0 * 2 : nullptr;
    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * cq + (lane & 15));
    const int csnap = L >= 1 ? (int)((L - 1) / CK) : -1;
    Ops ops;
    bool ok = true;
    if (nch > 0) {
      ok = wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], C.off);
    }
    int si = 0;                       // j % RING, kept by counting
    for (int j = 0; j < nch && ok; ++j) {
      const int nvalid = (j + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int sn = (si + 1 == RING) ? 0 : si + 1;
      const Slot* next = (j + 1 < nch) ? &slots[sn] : nullptr;
      ok = consume<PARK>(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, j == csnap, q2drop, oc,
                   [&]() { return peek_ready(sy, sn); },
                   [&](int peeked) {
                     return wait_ready_peeked(sy, sn, j + 2, peeked);
                   });
      // every LDS read of slot si has returned: its data went into the MFMAs above
      if (lane == 0) __hip_atomic_store(&sy->consumed[cq][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      si = sn;
    }
    // an operand beyond the fp16 range leaves inf or NaN in the carried state (until a reset discards it): count it
    count_nonfinite(C.S, lane, events_word(A.status));
  } else {
    const int p = pp;
    Raw raw;
    // this lane's new_starts byte of the chunk loaded next: fetched a step ahead, behind the operands (measured: 1.6 %
    // faster here than in front of them, where the other sweeps have it)
    uint32_t ns_mine = 0u;
    if (p < nch) {
      load_raw(raw, A, b, h, (int64_t)p * CK, lane);
      ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)p * CK, lane);
    }
    for (int j = p; j < nch + (PARK ? RING : 0); j += NPROD) {
      const int64_t c0 = (int64_t)j * CK;
      const int si = j % RING;
      Slot* slot = &slots[si];
      if (PARK) {
        // Retire the operand loads requested a step ago before anything else: loads and stores share the memory
        // counter, and a wait for a load inside `produce` would otherwise also wait for the y stores issued below.
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
      }
      if (j >= RING) {
        if (!wait_consumed_lazy(sy, si, j - RING + 1, lane)) break;
        if (PARK) flush_y(slot, A, b, h, j - RING, nch, lane);
      }
      if (PARK && j >= nch) continue;
      const ChunkFlags F = chunk_flags_of(A.ns, ns_mine, A.flags, A.T, c0, L);
      mask_raw(raw, F.nvalid, lane);
      produce(lane, raw, F, slot, snapslot, events_word(A.status));
      if (j + NPROD < nch) {
        load_raw(raw, A, b, h, c0 + (int64_t)NPROD * CK, lane);
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, c0 + (int64_t)NPROD * CK, lane);
      }
      if ((A.flags & FLAG_DROP_PUBLISH) && j + 1 == nch) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.out, 2, b, h, A.T, A.H);
    poison_token_rows(A.sa, 2, b, h, A.T, A.H);
    poison_state(A.new_s, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv7_chunk_fwd(const Wkv7Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync);
  const dim3 grid((unsigned)(A.B * A.H)), block(64 * (NCONS + NPROD));
  if (A.sa != nullptr) {
    static LdsAttrOnce once;
    const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_fwd_kernel<true>), smem);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(wkv7_fwd_kernel<true>, grid, block, smem, stream, A);
  } else {
    static LdsAttrOnce once;
    const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_fwd_kernel<false>), smem);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(wkv7_fwd_kernel<false>, grid, block, smem, stream, A);
  }
  return hipGetLastError();
}

}  // namespace hiprwkv
