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
#include "common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int CK = 16;            // tokens per chunk
constexpr int RS = 72;            // row stride (bf16 elements) of the [token][64] LDS arrays: 144 B (16-byte aligned rows)
constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int NCONS = 4;          // consumer waves, one per 16 value rows
constexpr int RING = 6;           // slots in flight
constexpr int SPIN_LIMIT = 1 << 16;   // polls before a waiter gives up (milliseconds; a healthy wait is microseconds)
constexpr float LOG2E = 1.44269504088896340736f;
constexpr float MIN_STEP_L2 = -1.0e4f;          // keeps the running sum finite
constexpr float MIN_CUM_L2 = -80.0f * LOG2E;    // 2^MIN_CUM_L2 = e^-80

// One chunk's operands as the consumers read them.  "lane-indexed" arrays hold, for every lane of the producer,
// the 8 bytes that the same lane of a consumer loads: accumulator-layout registers (column lane%16, rows
// 4*(lane/16)..+3) packed to bf16, which is exactly the A-operand layout (row lane%16, k-slots 4*(lane/16)..+3).
struct __attribute__((aligned(16))) Slot {
  uint16_t At[2][CK][RS];      // hi/lo of a_t.Ee_t; rows the entering state does not reach are zero
  uint16_t Qt[2][CK][RS];      // hi/lo of r_t.E_t; same masking, plus rows whose y is defined as zero
  uint2 BT[2][2][4][64];       // [bh|kh][hi|lo][key tile]: (b_s/E_s)^T, lane-indexed; masked for the chunk-end state
  uint2 VT[4][64];             // v^T per value tile, lane-indexed
  uint2 Mt[4][2][64];          // T, Mka, Mbr, Mkr: hi/lo, lane-indexed
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
// Update operands masked for the snapshot token; only one chunk per sequence needs them.
struct __attribute__((aligned(16))) SnapSlot {
  uint2 BT[2][2][4][64];
  float gamma[64];
};
// Hand-shake words.  ready[s] = c + 1 once chunk c is complete in slot s; consumed[q][s] = c + 1 once consumer
// q no longer reads chunk c in slot s.
struct __attribute__((aligned(16))) Sync {
  int ready[8];
  int consumed[NCONS][8];
};

__device__ __forceinline__ void wait_ready(const Sync* sy, int slot, int want) {
  for (int spin = 0; spin < SPIN_LIMIT; ++spin) {
    if (__hip_atomic_load(&sy->ready[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == want) return;
    __builtin_amdgcn_s_sleep(1);
  }
}
__device__ __forceinline__ void wait_consumed(const Sync* sy, int slot, int want, int lane) {
  for (int spin = 0; spin < SPIN_LIMIT; ++spin) {
    int seen = want;
    if (lane < NCONS) seen = __hip_atomic_load(&sy->consumed[lane][slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (__ballot(seen < want) == 0ull) return;
    __builtin_amdgcn_s_sleep(1);
  }
}

__device__ __forceinline__ f32x4_t mfma(const u32x4_t a, const u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t pack_rn(float x0, float x1) {
  bf16x2_t p = {(__bf16)x0, (__bf16)x1};
  return __builtin_bit_cast(uint32_t, p);
}
// both values are exactly representable in bf16: keep the high halves
__device__ __forceinline__ uint32_t pack_exact(float x0, float x1) {
  return __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);
}

// (x0, x1) -> packed truncated-bf16 hi parts and packed bf16 lo parts (x = hi + lo up to 2^-17 relative)
__device__ __forceinline__ void split2(float x0, float x1, uint32_t& hi, uint32_t& lo) {
  const uint32_t u0 = __float_as_uint(x0), u1 = __float_as_uint(x1);
  hi = __builtin_amdgcn_perm(u1, u0, 0x07060302u);
  lo = pack_rn(x0 - __uint_as_float(u0 & 0xffff0000u), x1 - __uint_as_float(u1 & 0xffff0000u));
}

template <int CTRL>
__device__ __forceinline__ float dpp0(float x) {  // lanes without a source read 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// Per-chunk facts, identical in every lane.
struct ChunkFlags {
  uint32_t ns;      // bit t: new_starts[c0+t], bit 16: new_starts[c0+16] (0 beyond T)
  int nvalid;       // tokens of this chunk that exist
  int snap;         // in-chunk index of token length-1, or -1
  bool compat;
};

__device__ __forceinline__ int seg_of(uint32_t ns, int t) { return __builtin_popcount(ns & ((2u << t) - 1u)); }

__device__ __forceinline__ ChunkFlags chunk_flags(const Wkv7Args& A, int64_t b, int64_t c0, int64_t L, int lane) {
  ChunkFlags F;
  F.compat = (A.flags & 1u) != 0;
  F.nvalid = (int)((A.T - c0 < CK) ? (A.T - c0) : CK);
  F.snap = (L >= 1 && L - 1 >= c0 && L - 1 < c0 + CK) ? (int)(L - 1 - c0) : -1;
  // lanes 0..16 fetch one flag each; the ballot makes the 17-bit mask uniform
  bool mine = false;
  if (A.ns != nullptr && lane <= CK && c0 + lane < A.T) mine = A.ns[(size_t)b * A.T + c0 + lane] != 0;
  F.ns = (uint32_t)(__ballot(mine) & 0x1ffffull);
  return F;
}

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

__device__ __forceinline__ void unpack16(const uint4 (&p)[2], float (&o)[16]) {
  const uint32_t w[8] = {p[0].x, p[0].y, p[0].z, p[0].w, p[1].x, p[1].y, p[1].z, p[1].w};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// element e of a lane's 16 keys -> key index
__device__ __forceinline__ int key_of(int g, int e) { return (e < 8) ? 8 * g + e : 32 + 8 * g + (e - 8); }

// Producer state carried from one period to the next (registers).
struct Producer {
  int lane;
  u32x4_t sel[2];     // B operands that pick keys 16*(tile%2)..+15 out of a 32-key half: MFMA as a transposer
  // stage 0 -> 1
  float pa[16], pq[16], pk[16], pb[16];   // a.Ee, r.E, k/E, b/E
  // stage 1 -> 2,3
  u32x4_t at_h[2], at_l[2], qt_h[2], qt_l[2], kh_h[2], kh_l[2], bh_h[2], bh_l[2];
  f32x4_t Mba, MbaT, Mka, Mbr, Mkr;
};

// stage 0: decay scan and scaled operands (fp32); v^T and the chunk-end decay go straight to the slot
__device__ __forceinline__ void prod_stage0(Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                            SnapSlot* __restrict__ snap) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  float fr[16], fk[16], fa[16], fb[16], E[16];
  unpack16(x.r, fr); unpack16(x.k, fk); unpack16(x.a, fa); unpack16(x.b, fb);
  {
    // transpose by MFMA: D[token][value of tile] = sum_k V[token][k] sel[k][value]; the accumulator layout of D
    // (lane = value, registers = 4 consecutive tokens) is the B-operand layout the consumers need
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const uint4 vr = x.v[tile >> 1];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w};
      const f32x4_t dv = mfma(vop, P.sel[tile & 1], zero4);
      slot->VT[tile][lane] = make_uint2(pack_exact(dv[0], dv[1]), pack_exact(dv[2], dv[3]));
    }
  }
  {
    float fw[16];
    unpack16(x.w, fw);
    // log2 of the decay, cumulative over the 16 tokens of the chunk (lanes of one DPP row)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float l2 = valid ? fmaxf(-exp2_fast(fw[e] * LOG2E) * LOG2E, MIN_STEP_L2) : 0.f;
      l2 += dpp0<0x111>(l2);
      l2 += dpp0<0x112>(l2);
      l2 += dpp0<0x114>(l2);
      l2 += dpp0<0x118>(l2);
      E[e] = l2;
    }
  }
  const bool slow = (F.ns & 0xffffu) != 0;
  if (slow) {
    // restart the cumulative decay at the last reset at or before this token
    const uint32_t upto = F.ns & ((2u << t) - 1u) & 0xffffu;
    const int p = upto ? 31 - __builtin_clz(upto) : 0;   // position of that reset
    const int src = (lane & 48) | (p > 0 ? p - 1 : 0);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float base = __shfl(E[e], src, 64);
      if (p > 0) E[e] -= base;
    }
    if ((F.ns >> t) & 1u) {
#pragma unroll
      for (int e = 0; e < 16; ++e) fa[e] = 0.f;   // the state entering a reset token is zero: sa = 0
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const float l2 = fmaxf(E[e], MIN_CUM_L2);
    const float Ev = exp2_fast(l2), Einv = exp2_fast(-l2);
    // exclusive: value of the previous token; 1 for the first token of the chunk
    const float Ee = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(1.0f), __float_as_int(Ev), 0x111, 0xf, 0xf, false));
    P.pa[e] = fa[e] * Ee;      // at a reset token a is zero, whatever Ee holds
    P.pq[e] = fr[e] * Ev;
    P.pk[e] = fk[e] * Einv;
    P.pb[e] = fb[e] * Einv;
    E[e] = Ev;
  }
  if (t == 15) {
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      float* gp = &slot->gamma[8 * g + 32 * hf];
      *reinterpret_cast<float4*>(gp) = make_float4(E[8 * hf], E[8 * hf + 1], E[8 * hf + 2], E[8 * hf + 3]);
      *reinterpret_cast<float4*>(gp + 4) = make_float4(E[8 * hf + 4], E[8 * hf + 5], E[8 * hf + 6], E[8 * hf + 7]);
    }
  }
  if (t == F.snap) {
#pragma unroll
    for (int e = 0; e < 16; ++e) snap->gamma[key_of(g, e)] = E[e];
  }
}

// stage 1: hi/lo split and the five Gram tiles
__device__ __forceinline__ void prod_stage1(Producer& P) {
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 8 * hf + 2 * j;
      uint32_t hi, lo;
      split2(P.pa[e], P.pa[e + 1], hi, lo); P.at_h[hf][j] = hi; P.at_l[hf][j] = lo;
      split2(P.pq[e], P.pq[e + 1], hi, lo); P.qt_h[hf][j] = hi; P.qt_l[hf][j] = lo;
      split2(P.pk[e], P.pk[e + 1], hi, lo); P.kh_h[hf][j] = hi; P.kh_l[hf][j] = lo;
      split2(P.pb[e], P.pb[e + 1], hi, lo); P.bh_h[hf][j] = hi; P.bh_l[hf][j] = lo;
    }
  }
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t Mba = zero4, MbaT = zero4, Mka = zero4, Mbr = zero4, Mkr = zero4;
  // accumulator layout: lane holds column n = lane%16, rows m = 4g..4g+3.  Five independent chains, interleaved.
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
    for (int part = 0; part < 3; ++part) {
      const u32x4_t bA = part == 2 ? P.bh_l[hf] : P.bh_h[hf], kA = part == 2 ? P.kh_l[hf] : P.kh_h[hf];
      const u32x4_t aA = part == 2 ? P.at_l[hf] : P.at_h[hf];
      const u32x4_t aB = part == 1 ? P.at_l[hf] : P.at_h[hf], qB = part == 1 ? P.qt_l[hf] : P.qt_h[hf];
      const u32x4_t bB = part == 1 ? P.bh_l[hf] : P.bh_h[hf];
      Mba = mfma(bA, aB, Mba);     // [s][t] = bh_s . at_t
      MbaT = mfma(aA, bB, MbaT);   // [t][s]
      Mka = mfma(kA, aB, Mka);     // [s][t] = kh_s . at_t
      Mbr = mfma(bA, qB, Mbr);     // [s][t] = bh_s . qt_t
      Mkr = mfma(kA, qB, Mkr);     // [s][t] = kh_s . qt_t
    }
  }
  P.Mba = Mba; P.MbaT = MbaT; P.Mka = Mka; P.Mbr = Mbr; P.Mkr = Mkr;
}

// stage 2: triangular masks, T = (I - Mba)^{-1}, park T / Mka / Mbr / Mkr
__device__ __forceinline__ void prod_stage2(Producer& P, const ChunkFlags& F, Slot* __restrict__ slot) {
  const int lane = P.lane, n = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t Mba = P.Mba, MbaT = P.MbaT, Mka = P.Mka, Mbr = P.Mbr, Mkr = P.Mkr;
  const bool slow = F.ns != 0;
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
  // T = (I + M^8)(I + M^4)(I + M^2)(I + M), single-bf16 operands
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
    slot->Mt[which][0][lane] = make_uint2(hi0, hi1);
    slot->Mt[which][1][lane] = make_uint2(lo0, lo1);
  };
  park(0, Pm); park(1, Mka); park(2, Mbr); park(3, Mkr);
}

// stage 3: operands the consumers read through LDS: At, Qt (row-major), transposed bh / kh, flags
__device__ __forceinline__ void prod_stage3(Producer& P, const ChunkFlags& F, Slot* __restrict__ slot,
                                            SnapSlot* __restrict__ snap) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool slow = F.ns != 0;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const u32x4_t z4 = {0u, 0u, 0u, 0u};
  int lastseg = 0;
  bool s0_reaches = true, q_keep = true;
  uint32_t keep_upd = 0xffffu;       // tokens that still contribute to the chunk-end state
  if (slow) {
    lastseg = seg_of(F.ns, 15);
    s0_reaches = seg_of(F.ns, t) == 0;                             // the entering state reaches this token
    q_keep = s0_reaches && !(F.compat && ((F.ns >> (t + 1)) & 1u));
    const uint32_t resets = F.ns & 0xffffu;
    // tokens from the last reset on
    keep_upd = resets ? (0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u)) : 0xffffu;
  }
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int col = 8 * g + 32 * hf;
    *reinterpret_cast<u32x4_t*>(&slot->At[0][t][col]) = s0_reaches ? P.at_h[hf] : z4;
    *reinterpret_cast<u32x4_t*>(&slot->At[1][t][col]) = s0_reaches ? P.at_l[hf] : z4;
    *reinterpret_cast<u32x4_t*>(&slot->Qt[0][t][col]) = q_keep ? P.qt_h[hf] : z4;
    *reinterpret_cast<u32x4_t*>(&slot->Qt[1][t][col]) = q_keep ? P.qt_l[hf] : z4;
  }
  // transposes by MFMA: D[token][key of tile] = sum_k X[token][k] sel[k][key]; the accumulator layout of D
  // (lane = key, registers = 4 consecutive tokens) is the A-operand layout of the state update
  uint32_t keep_snap = 0;
  if (F.snap >= 0) {
    keep_snap = (2u << F.snap) - 1u;
    if (slow) {
      const uint32_t upto = F.ns & keep_snap & 0xffffu;
      if (upto) keep_snap &= ~((1u << (31 - __builtin_clz(upto))) - 1u);
    }
  }
  auto masked_pack = [&](const f32x4_t d, uint32_t keep) {
    const uint32_t bits = keep >> (4 * g);
    const float d0 = (bits & 1u) ? d[0] : 0.f, d1 = (bits & 2u) ? d[1] : 0.f;
    const float d2 = (bits & 4u) ? d[2] : 0.f, d3 = (bits & 8u) ? d[3] : 0.f;
    return make_uint2(pack_exact(d0, d1), pack_exact(d2, d3));
  };
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const int hf = tile >> 1;
    const u32x4_t sel = P.sel[tile & 1];
    const f32x4_t dbh = mfma(P.bh_h[hf], sel, zero4), dbl = mfma(P.bh_l[hf], sel, zero4);
    const f32x4_t dkh = mfma(P.kh_h[hf], sel, zero4), dkl = mfma(P.kh_l[hf], sel, zero4);
    if (keep_upd == 0xffffu) {
      slot->BT[0][0][tile][lane] = make_uint2(pack_exact(dbh[0], dbh[1]), pack_exact(dbh[2], dbh[3]));
      slot->BT[0][1][tile][lane] = make_uint2(pack_exact(dbl[0], dbl[1]), pack_exact(dbl[2], dbl[3]));
      slot->BT[1][0][tile][lane] = make_uint2(pack_exact(dkh[0], dkh[1]), pack_exact(dkh[2], dkh[3]));
      slot->BT[1][1][tile][lane] = make_uint2(pack_exact(dkl[0], dkl[1]), pack_exact(dkl[2], dkl[3]));
    } else {
      slot->BT[0][0][tile][lane] = masked_pack(dbh, keep_upd);
      slot->BT[0][1][tile][lane] = masked_pack(dbl, keep_upd);
      slot->BT[1][0][tile][lane] = masked_pack(dkh, keep_upd);
      slot->BT[1][1][tile][lane] = masked_pack(dkl, keep_upd);
    }
    if (F.snap >= 0) {
      snap->BT[0][0][tile][lane] = masked_pack(dbh, keep_snap);
      snap->BT[0][1][tile][lane] = masked_pack(dbl, keep_snap);
      snap->BT[1][0][tile][lane] = masked_pack(dkh, keep_snap);
      snap->BT[1][1][tile][lane] = masked_pack(dkl, keep_snap);
    }
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
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

__device__ __forceinline__ uint2 lds8(const uint16_t* p) { return *reinterpret_cast<const uint2*>(p); }

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int nvalid, bool q2drop) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
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
  // A operands: rows = tokens (lane%16), same key order as the B operands above
  auto rows = [&](const uint16_t (*arr)[RS], int j) {
    const uint2 p0 = lds8(&arr[n][32 * j + 4 * g]);
    const uint2 p1 = lds8(&arr[n][32 * j + 16 + 4 * g]);
    u32x4_t o = {p0.x, p0.y, p1.x, p1.y};
    return o;
  };
  f32x4_t W = zero4, Y = zero4;   // [token 4g+i][value n]
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t ah = rows(slot->At[0], j), al = rows(slot->At[1], j);
    const u32x4_t qh = rows(slot->Qt[0], j), ql = rows(slot->Qt[1], j);
    W = mfma(ah, Sh[j], W);
    Y = mfma(qh, Sh[j], Y);
    W = mfma(ah, Sl[j], W);
    Y = mfma(qh, Sl[j], Y);
    W = mfma(al, Sh[j], W);
    Y = mfma(ql, Sh[j], Y);
  }
  // v of the four tokens 4g..4g+3 for this lane's value column
  const int val = 16 * C.q + n;
  const uint2 vt = slot->VT[C.q][lane];
  const uint32_t v01 = vt.x, v23 = vt.y;
  const uint2 Th = slot->Mt[0][0][lane], Tl = slot->Mt[0][1][lane];
  const uint2 Kah = slot->Mt[1][0][lane], Kal = slot->Mt[1][1][lane];
  const uint2 Brh = slot->Mt[2][0][lane], Brl = slot->Mt[2][1][lane];
  const uint2 Krh = slot->Mt[3][0][lane], Krl = slot->Mt[3][1][lane];
  {
    const u32x4_t a = {Kah.x, Kah.y, Kal.x, Kal.y}, bb = {v01, v23, v01, v23};
    W = mfma(a, bb, W);                       // W += Mka^T V^T
  }
  uint32_t Wh0, Wl0, Wh1, Wl1;
  split2(W[0], W[1], Wh0, Wl0);
  split2(W[2], W[3], Wh1, Wl1);
  f32x4_t SA;
  {
    const u32x4_t a1 = {Th.x, Th.y, Tl.x, Tl.y}, b1 = {Wh0, Wh1, Wh0, Wh1};
    const u32x4_t a2 = {Th.x, Th.y, 0u, 0u}, b2 = {Wl0, Wl1, 0u, 0u};
    SA = mfma(a1, b1, zero4);
    SA = mfma(a2, b2, SA);                    // SA^T = T^T W^T
  }
  uint32_t Ah0, Al0, Ah1, Al1;
  split2(SA[0], SA[1], Ah0, Al0);
  split2(SA[2], SA[3], Ah1, Al1);
  const u32x4_t bSS = {Ah0, Ah1, Ah0, Ah1}, bLV = {Al0, Al1, v01, v23}, bV0 = {v01, v23, 0u, 0u};
  {
    const u32x4_t a1 = {Brh.x, Brh.y, Brl.x, Brl.y}, a2 = {Brh.x, Brh.y, Krh.x, Krh.y}, a3 = {Krl.x, Krl.y, 0u, 0u};
    Y = mfma(a1, bSS, Y);
    Y = mfma(a2, bLV, Y);
    Y = mfma(a3, bV0, Y);                     // Y^T += Mbr^T SA^T + Mkr^T V^T
  }
  // state update (and the snapshot for `length`), tile by tile: rows = keys
  auto update = [&](const uint2 (*bt)[2][4][64], const float* gam, bool keep, f32x4_t (&out)[4]) {
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const uint2 bh = bt[0][0][tile][lane], bl = bt[0][1][tile][lane];
      const uint2 kh = bt[1][0][tile][lane], kl = bt[1][1][tile][lane];
      const u32x4_t a1 = {bh.x, bh.y, bl.x, bl.y}, a2 = {bh.x, bh.y, kh.x, kh.y}, a3 = {kl.x, kl.y, 0u, 0u};
      f32x4_t acc = keep ? C.S[tile] : zero4;
      acc = mfma(a1, bSS, acc);
      acc = mfma(a2, bLV, acc);
      acc = mfma(a3, bV0, acc);
      const float4 gm = *reinterpret_cast<const float4*>(&gam[16 * tile + 4 * g]);
      acc[0] *= gm.x; acc[1] *= gm.y; acc[2] *= gm.z; acc[3] *= gm.w;
      out[tile] = acc;
    }
  };
  if (slot->snap >= 0) {
    f32x4_t snap[4];
    update(snapslot->BT, snapslot->gamma, slot->keep_snap != 0, snap);
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const size_t off = (((size_t)b * A.H + h) * 64 + val) * 64 + 16 * tile + 4 * g;
      if (A.st_f32) {
        float4 o = q2drop ? make_float4(0.f, 0.f, 0.f, 0.f) : make_float4(snap[tile][0], snap[tile][1], snap[tile][2], snap[tile][3]);
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(A.new_s) + off) = o;
      } else {
        uint2 o = q2drop ? make_uint2(0u, 0u) : make_uint2(pack_rn(snap[tile][0], snap[tile][1]), pack_rn(snap[tile][2], snap[tile][3]));
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(A.new_s) + off) = o;
      }
    }
  }
  update(slot->BT, slot->gamma, slot->keep_end != 0, C.S);
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tt = 4 * g + i;
    if (tt < nvalid) {
      const size_t off = (((size_t)b * A.T + c0 + tt) * A.H + h) * 64 + val;
      reinterpret_cast<uint16_t*>(A.out)[off] = f32_to_bf16(Y[i]);
      if (A.sa != nullptr) A.sa[off] = SA[i];
    }
  }
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
    const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
    Consumer C;
    C.q = wave;
    C.lane = lane;
    load_state(C, A, b, h);
    if (L == 0) store_state0(C, A, b, h, q2drop);
    for (int64_t c = 0; c < nchunks; ++c) {
      const int64_t c0 = c * CK;
      const int nvalid = (int)((A.T - c0 < CK) ? (A.T - c0) : CK);
      const int si = (int)(c % RING);
      wait_ready(sy, si, (int)c + 1);
      consume(C, &slots[si], snapslot, A, b, h, c0, nvalid, q2drop);
      // every LDS read of the slot has returned (its data was used above)
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], (int)c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    {
      // sel[x]: k-slot (g, jj) of a 32-key half stands for key 8g + jj; column n of tile x is key 16x + n
      const int n = lane & 15, g = lane >> 4;
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const int jj = 16 * x + n - 8 * g;
        u32x4_t sl = {0u, 0u, 0u, 0u};
        if (jj >= 0 && jj < 8) sl[jj >> 1] = (jj & 1) ? 0x3f800000u : 0x00003f80u;
        P.sel[x] = sl;
      }
    }
    Raw raw;
    if (p < nchunks) load_raw(raw, A, b, h, (int64_t)p * CK, lane);
    for (int64_t c = p; c < nchunks; c += NPROD) {
      const int64_t c0 = c * CK;
      const ChunkFlags F = chunk_flags(A, b, c0, L, lane);
      const int si = (int)(c % RING);
      Slot* slot = &slots[si];
      if (c >= RING) wait_consumed(sy, si, (int)(c - RING) + 1, lane);
      prod_stage0(P, raw, F, slot, snapslot);
      if (c + NPROD < nchunks) load_raw(raw, A, b, h, c0 + NPROD * CK, lane);
      prod_stage1(P);
      prod_stage2(P, F, slot);
      prod_stage3(P, F, slot, snapslot);
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
