// WKV7 backward for fp32 I/O on gfx950, first (reverse) sweep: gv, the workspace dsa and gs, 16 tokens at a time on
// the matrix cores with fp32 operands (v_mfma_f32_16x16x4_f32), for callers that need cotangents to fp32 accuracy.
//
// Forward recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv7.py:200-220), S[i][j] = value row i, key
// col j:  sa_t = S_{t-1} a_t ;  S_t = S_{t-1} diag(d_t) + sa_t b_t^T + v_t k_t^T ;  y_t = S_t r_t ;  d_t = exp(-exp(w_t)).
// With G~_t the cotangent of S_t, carried from the last token down:
//     G~_t = dy_t r_t^T + G~_{t+1} diag(d_{t+1}) + dsa_{t+1} a_{t+1}^T ;  dsa_t = G~_t b_t ;  dv_t = G~_t k_t
// The chunk algebra is the one of the bf16 sweep (wkv7_bwd_a.hip): with E_t = prod_{s<=t} d_s, at_t = a_t.E_{t-1},
// qt_t = r_t.E_t, kh_s = k_s/E_s, bh_s = b_s/E_s and Gh = G_C diag(E_C) for a chunk leaving with G_C,
//     U   = Gh Bh^T + DY^T Mbr^T         DSA = U (I - Mba^T)^{-1}         DV = Gh Kh^T + DSA Mka^T + DY^T Mkr^T
//     G_prev = Gh + DSA At + DY^T Qt
// i.e. the forward chunk computation (wkv7_fwd_f32.hip) with the operands exchanged (Bh <-> At, Kh <-> Qt, V <-> DY,
// every Gram tile transposed) and the decay applied before instead of after the update; the instruction layouts, the
// split of the running log-decay into an exact grid part and a remainder, and the work split (one consumer and one
// producer wave per SIMD, ring of LDS slots) are those of that kernel.  Chunks are handled from the last one down.
// new_starts inside a chunk restart the cumulative decay and mask the Gram tiles; the chunk that holds token length-1
// uses a second, masked set of row operands through which the cotangent of the returned state enters.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
// X^T Z for two 16x16 tiles in accumulator layout, added to c
__device__ __forceinline__ f32x4_t mfma_tt(const f32x4_t x, const f32x4_t z, f32x4_t c) {
#pragma unroll
  for (int i = 0; i < 4; ++i) c = mfma_f(x[i], z[i], c);
  return c;
}

__device__ __forceinline__ float row_prev0(float x) {     // previous lane of the row, 0 in lane 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true));
}

struct __attribute__((aligned(16))) Slot {
  float AQ[2][CK][RF];         // bh, kh rows [token][key]; rows that the cotangent of later chunks does not reach are zero
  float BK[2][CK][RF];         // at, qt rows (tokens from the first reset on are zero: they do not reach the chunk start)
  float V[CK][RF];             // dy rows (zero where y is a constant)
  f32x4_t P[64], Ka[64], Br[64], Kr[64];   // lane-indexed accumulator tiles: column t = lane%16, rows 4g..4g+3
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the carried cotangent passes through the whole chunk (no reset in the chunk)
  int keep_snap;               // the cotangent entering at token length-1 reaches the chunk start
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {   // row operands masked for token length-1 (one chunk per sequence)
  float AQ[2][CK][RF];
  float gamma[64];             // E at token length-1
};
struct __attribute__((aligned(16))) TrTile {     // a producer's private 16x16 transposer
  float x[CK][CK + 1];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys 16j + 4g + i (j, i = 0..3): one 16-byte load per j, and
// element (j, i) is this lane's k-slot of the Gram instruction (j, i) both as A and as B operand.
struct Raw {
  float4 r[4], w[4], k[4], v[4], a[4], b[4];   // v holds dy
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv7Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;   // always a valid token; mask_raw zeroes the lanes beyond
  const size_t off = (((size_t)b * A.T + tok) * A.H + h) * 64 + 4 * g;
  auto ld = [&](const void* p, float4 (&o)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + off + 16 * j);
  };
  ld(A.r, x.r); ld(A.w, x.w); ld(A.k, x.k); ld(A.gy, x.v); ld(A.a, x.a); ld(A.b, x.b);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) x.r[j] = x.w[j] = x.k[j] = x.v[j] = x.a[j] = x.b[j] = z;
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

// Everything of one chunk that does not depend on the carried state.  The two 32-key halves (j = 0,1 and j = 2,3) go
// through the same pipeline one after the other, which keeps the live register set small.
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, TrTile* __restrict__ tr, unsigned* events) {
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
    row_keep = seg_of(F.ns, t) == lastseg;                           // the cotangent from later chunks reaches this token
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

  // Gram tiles in accumulator layout [row m = A-operand token][column n = B-operand token]
  f32x4_t GabT = zero4, G1 = zero4, G2 = zero4, G3 = zero4;   // at_m.bh_n, qt_m.bh_n, at_m.kh_n, qt_m.kh_n
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    {
      float fv[8];
      unpack2(x.v[2 * hf], x.v[2 * hf + 1], fv);
      bool keep_dy = true;
      if (slow) {
        rare_path();
        keep_dy = !drop_dy;
      }
      put2(slot->V[t], hf, g, fv, keep_dy);
    }
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain.  A running sum of magnitude 16-32 has an
    //      fp32 spacing of 2e-6, which would be the largest error of the whole kernel: every step is split into a part
    //      on a 2^-16 grid, whose running sums are exact, and a remainder below 2^-17, summed separately.
    float E[8], El[8], fa[8];
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
    unpack2(x.a[2 * hf], x.a[2 * hf + 1], fa);
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
    // ---- scaled operands
    float fat[8], fqt[8], fkh[8], fbh[8];
    {
      float fr[8], fk[8], fb[8];
      unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
      unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
      unpack2(x.b[2 * hf], x.b[2 * hf + 1], fb);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
        const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
        E[e] = exp2_fast(l2) * fl;
        const float einv = exp2_fast(-l2) * (2.f - fl);
        // The decay up to the previous token is 1 for the chunk's first token.  At a reset token the value belongs to
        // the previous segment, but every product it enters is masked out or multiplies a zero.
        const float fa0 = (t == 0) ? fa[e] : 0.f;
        fat[e] = fmaf(fa[e], row_prev0(E[e]), fa0);
        fqt[e] = fr[e] * E[e];
        fkh[e] = fk[e] * einv;
        fbh[e] = fb[e] * einv;
      }
    }
    if (t == 15) {
      *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
    }
    if (F.snap >= 0 && t == F.snap) {
      *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
    }
    {
      const bool ku = (keep_upd >> t) & 1u;       // tokens from the first reset on do not reach the chunk start
      put2(slot->BK[0][t], hf, g, fat, ku);
      put2(slot->BK[1][t], hf, g, fqt, ku);
    }
    put2(slot->AQ[0][t], hf, g, fbh, row_keep);
    put2(slot->AQ[1][t], hf, g, fkh, row_keep);
    if (F.snap >= 0) {                            // the same rows masked for the cotangent entering at token length-1
      rare_path();
      const bool sk = (keep_snap >> t) & 1u;
      put2(snap->AQ[0][t], hf, g, fbh, sk);
      put2(snap->AQ[1][t], hf, g, fkh, sk);
    }
    // ---- partial Gram sums over this half's keys
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      GabT = mfma_f(fat[e], fbh[e], GabT);  // Mba^T[m][n] = at_m . bh_n
      G1 = mfma_f(fqt[e], fbh[e], G1);      // Mbr^T[m][n] = qt_m . bh_n
      G2 = mfma_f(fat[e], fkh[e], G2);      // Mka^T[m][n] = at_m . kh_n
      G3 = mfma_f(fqt[e], fkh[e], G3);      // Mkr^T[m][n] = qt_m . kh_n
    }
  }
  // ---- triangular masks: later rows m for column n
  const int n = t;
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      GabT[i] = m > n ? GabT[i] : 0.f;
      G1[i] = m >= n ? G1[i] : 0.f;
      G2[i] = m > n ? G2[i] : 0.f;
      G3[i] = m >= n ? G3[i] : 0.f;
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool same = seg_of(F.ns, m) == seg_of(F.ns, n);
      GabT[i] = (m > n && same) ? GabT[i] : 0.f;
      G1[i] = (m >= n && same) ? G1[i] : 0.f;
      G2[i] = (m > n && same) ? G2[i] : 0.f;
      G3[i] = (m >= n && same) ? G3[i] : 0.f;
    }
  }
  // ---- M^T through the private LDS tile: tr[n][4g+i] = M[4g+i][n], read back as rows
  f32x4_t MpT;
  {
#pragma unroll
    for (int i = 0; i < 4; ++i) tr->x[n][4 * g + i] = GabT[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < 4; ++i) MpT[i] = tr->x[4 * g + i][n];
  }
  // ---- P = (I - M)^{-1} = (I + M^8)(I + M^4)(I + M^2)(I + M), M = Mba^T
  f32x4_t Mp = GabT;
  f32x4_t Pm = Mp;
#pragma unroll
  for (int i = 0; i < 4; ++i) Pm[i] += (4 * g + i == n) ? 1.f : 0.f;
#pragma unroll
  for (int lvl = 0; lvl < 3; ++lvl) {
    const f32x4_t M2T = mfma_tt(Mp, MpT, zero4);         // M^T M^T = (M^2)^T
    if (lvl < 2) Mp = mfma_tt(MpT, Mp, zero4);           // M M
    MpT = M2T;
    Pm = mfma_tt(MpT, Pm, Pm);                           // P += M^(2^(lvl+1)) P
  }
  slot->P[lane] = Pm;
  slot->Ka[lane] = G1;
  slot->Br[lane] = G2;
  slot->Kr[lane] = G3;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(F.ns, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds G^T for value rows 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16, g = lane/16),
// S[tile][i] = G[value 16q+n][key 16*tile + 4g + i]: register i of a tile is the B operand of the instruction that
// contracts over the keys 16*tile + 4g' + i (g' = 0..3).
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

struct Ops {               // fetched a chunk ahead: everything the U / DSA / DV chain reads
  float4 bh[4], kh[4];     // rows of token n: keys 16*tile + 4g .. +3
  float4 gm[4];            // E at the chunk end, keys 16*tile + 4g .. +3
  f32x4_t P, Ka, Br, Kr;   // (I - Mba^T)^{-1}, Mbr^T, Mka^T, Mkr^T
  f32x4_t vv;              // dy of tokens 4g..4g+3, value 16q + n
  int keep_end;
};

__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    o.bh[tile] = *reinterpret_cast<const float4*>(&slot->AQ[0][n][16 * tile + 4 * g]);
    o.kh[tile] = *reinterpret_cast<const float4*>(&slot->AQ[1][n][16 * tile + 4 * g]);
    o.gm[tile] = *reinterpret_cast<const float4*>(&slot->gamma[16 * tile + 4 * g]);
  }
  o.P = slot->P[lane];
  o.Ka = slot->Ka[lane];
  o.Br = slot->Br[lane];
  o.Kr = slot->Kr[lane];
#pragma unroll
  for (int i = 0; i < 4; ++i) o.vv[i] = slot->V[4 * g + i][16 * q + n];
  o.keep_end = slot->keep_end;
}

// A operands of the cotangent update of one key tile: at then qt of tokens 4g..4g+3, key 16*tile + n
__device__ __forceinline__ void load_upd(f32x4_t& ua, f32x4_t& uq, const float (*bk)[CK][RF], int tile, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ua[i] = bk[0][4 * g + i][16 * tile + n];
    uq[i] = bk[1][4 * g + i][16 * tile + n];
  }
}

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

struct OutCursor {
  float* y;            // A.gv at (b, c0, h, 0)
  float* sa;           // A.dsa at the same place
  size_t tok;          // elements between consecutive tokens
  uint32_t voff;       // lane part of the address: (4g * H) * 64 + value
};

// The cotangent-dependent part of one chunk.  SNAP: this chunk holds token length-1 and a cotangent of the returned
// state exists (one chunk per sequence; a separate instantiation keeps the common path free of its branch).
template <bool SNAP, class PeekNext, class WaitNext>
__device__ __forceinline__ bool consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
                                        const Slot* __restrict__ next, const SnapSlot* __restrict__ snapslot,
                                        const Wkv7Args& A, int64_t b, int64_t h, int nvalid,
                                        OutCursor& oc, PeekNext&& peek_next, WaitNext&& next_ready) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const int peeked = next != nullptr ? peek_next() : 0;
  // update operands of this chunk: needed last, so their latency hides behind the U / DSA chain
  f32x4_t uat[4], uqt[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) load_upd(uat[tile], uqt[tile], slot->BK, tile, lane);
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
  // the cotangent of the chunk-end state, decayed over the chunk: Gh = G_C diag(E_C)
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    C.S[tile][0] *= o.gm[tile].x; C.S[tile][1] *= o.gm[tile].y; C.S[tile][2] *= o.gm[tile].z; C.S[tile][3] *= o.gm[tile].w;
  }
  f32x4_t W = zero4, Y = zero4;   // U and DV, [token 4g+i][value n], two interleaved accumulation chains
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const float bh[4] = {o.bh[tile].x, o.bh[tile].y, o.bh[tile].z, o.bh[tile].w};
    const float kh[4] = {o.kh[tile].x, o.kh[tile].y, o.kh[tile].z, o.kh[tile].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      W = mfma_f(bh[i], C.S[tile][i], W);
      Y = mfma_f(kh[i], C.S[tile][i], Y);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    W = mfma_f(o.Ka[i], o.vv[i], W);            // U += Mbr DY
    Y = mfma_f(o.Kr[i], o.vv[i], Y);            // DV += Mkr DY
  }
  const f32x4_t vv = o.vv;
  // a reset inside the chunk cuts the cotangent of later chunks off from the chunk start
  if (!keep_end) {
    rare_path();
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;
  }
  // the cotangent of the returned state enters at token length-1
  if (SNAP) {
    const bool keep = slot->keep_snap != 0;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      f32x4_t gs = load_state_tile(A.gs_out, A.st_f32, state_off(A, b, h, C.q, lane, tile));
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      gs[0] *= sg.x; gs[1] *= sg.y; gs[2] *= sg.z; gs[3] *= sg.w;
      if (keep) C.S[tile] += gs;
      const float4 sb = *reinterpret_cast<const float4*>(&snapslot->AQ[0][n][16 * tile + 4 * g]);
      const float4 sk = *reinterpret_cast<const float4*>(&snapslot->AQ[1][n][16 * tile + 4 * g]);
      const float bh[4] = {sb.x, sb.y, sb.z, sb.w}, kh[4] = {sk.x, sk.y, sk.z, sk.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        W = mfma_f(bh[i], gs[i], W);
        Y = mfma_f(kh[i], gs[i], Y);
      }
    }
  }
  // G <- Gh + At^T DSA + Qt^T DY, rows = keys.  The Qt^T DY half, which depends on nothing computed here, runs between
  // U -> DSA and DSA -> its readers, so that no matrix instruction waits for an operand.
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    C.S[0] = mfma_f(uqt[0][i], vv[i], C.S[0]);
    C.S[1] = mfma_f(uqt[1][i], vv[i], C.S[1]);
  }
  f32x4_t SA = zero4;
#pragma unroll
  for (int i = 0; i < 4; ++i) SA = mfma_f(o.P[i], W[i], SA);      // DSA = P^T U
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    C.S[2] = mfma_f(uqt[2][i], vv[i], C.S[2]);
    C.S[3] = mfma_f(uqt[3][i], vv[i], C.S[3]);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    Y = mfma_f(o.Br[i], SA[i], Y);                                // DV += Mka DSA
    C.S[0] = mfma_f(uat[0][i], SA[i], C.S[0]);
    C.S[1] = mfma_f(uat[1][i], SA[i], C.S[1]);
    C.S[2] = mfma_f(uat[2][i], SA[i], C.S[2]);
    C.S[3] = mfma_f(uat[3][i], SA[i], C.S[3]);
  }
  // everything fetched a chunk ahead is dead now: fetch the next chunk's into the same registers
  bool ok = true;
  if (next != nullptr) {
    ok = next_ready(peeked);
    load_ops(o, next, C.q, lane);
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  float* const yl = oc.y + oc.voff;
  float* const sl = oc.sa + oc.voff;
  if (nvalid == CK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) yl[i * oc.tok] = Y[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) sl[i * oc.tok] = SA[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        yl[i * oc.tok] = Y[i];
        sl[i * oc.tok] = SA[i];
      }
    }
  }
  oc.y -= CK * oc.tok;
  oc.sa -= CK * oc.tok;
  return ok;
}

}  // namespace

// Chunks are handled from the last one down: step j handles chunk nch - 1 - j in slot j % RING.  Producer p fills the
// slot once every consumer has released step j - RING, then publishes ready = j + 1; consumers take the steps in
// order.  Every wait is for a strictly earlier step, so the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv7_bwd_a_f32_kernel(Wkv7Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  TrTile* trs = reinterpret_cast<TrTile*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot) + NPROD * sizeof(TrTile));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int nch = (int)((A.T + CK - 1) / CK);
  // the returned state is the reset state there (associative-scan rule), a constant
  const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
  // does a cotangent of the returned state enter at token length-1?
  const bool inject = A.gs_out != nullptr && !q2drop;
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  __syncthreads();

  if (wave < NCONS) {                 // waves 0..3: one consumer per SIMD; waves 4..7: one producer per SIMD
    __builtin_amdgcn_s_setprio(3);    // the chunk-to-chunk dependency runs through the consumers
    const int cq = wave;
    Consumer C;
    C.q = cq;
    C.lane = lane;
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;
    OutCursor oc;
    oc.tok = (size_t)A.H * 64;
    const size_t el0 = (((size_t)b * A.T + (size_t)(nch - 1) * CK) * A.H + h) * 64;
    oc.y = reinterpret_cast<float*>(A.gv) + el0;
    oc.sa = A.dsa + el0;
    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * cq + (lane & 15));
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    Ops ops;
    bool ok = true;
    if (nch > 0) {
      ok = wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], cq, lane);
    }
    for (int j = 0; j < nch && ok; ++j) {
      const int c = nch - 1 - j;
      const int nvalid = (j > 0 || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = j % RING, sn = (j + 1) % RING;
      const Slot* next = (j + 1 < nch) ? &slots[sn] : nullptr;
      auto peek = [&]() { return peek_ready(sy, sn); };
      auto wait = [&](int peeked) { return wait_ready_peeked(sy, sn, j + 2, peeked); };
      if (c == csnap) {
        rare_path();
        ok = consume<true>(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, oc, peek, wait);
      } else {
        ok = consume<false>(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, oc, peek, wait);
      }
      // every LDS read of slot si has returned: its data went into the matrix instructions above
      if (lane == 0) __hip_atomic_store(&sy->consumed[cq][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // cotangent of the input state; with length == 0 the returned state is the input state itself
    const bool pass = L == 0 && inject;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const size_t off = state_off(A, b, h, cq, lane, tile);
      f32x4_t gsv = C.S[tile];
      if (pass) gsv += load_state_tile(A.gs_out, A.st_f32, off);
      store_state_tile(A.gs, A.st_f32, off, gsv);
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
      produce(lane, raw, F, &slots[si], snapslot, &trs[p], events_word(A.status));
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
    poison_token_rows(A.gv, 4, b, h, A.T, A.H);
    poison_token_rows(A.dsa, 4, b, h, A.T, A.H);
    poison_state(A.gs, A.st_f32, b, h, A.H);
  }
}

// Reverse sweep of the backward pass with fp32 I/O: gv, the workspace dsa (cotangent of sa per token) and gs.
hipError_t launch_wkv7_chunk_bwd_a_f32(const Wkv7Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + NPROD * sizeof(TrTile) + sizeof(Sync);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + NPROD * sizeof(TrTile) + sizeof(Sync) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv7_bwd_a_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv7_bwd_a_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
