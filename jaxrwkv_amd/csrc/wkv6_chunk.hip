// WKV6 forward, chunked MFMA kernel for bf16 I/O on gfx950.
//
// Recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191), S[i][j] = key row i, value col j,
// dec_t = exp(w_t) with w the log decay:
//     S' = new_starts[t] ? 0 : S ;  y_t = r_t^T (diag(u) k_t v_t^T + S') ;  S = diag(dec_t) S' + k_t v_t^T
// A chunk of C = 16 tokens entering with state S0 is evaluated in closed form.  With Lc_t = sum_{s<=t} w_s,
// E_t = exp(Lc_t), Ee_t = exp(Lc_{t-1}) and the scaled operands qt_t = r_t.Ee_t, kh_s = k_s/E_s:
//     M[s][t] = kh_s.qt_t (s < t),  M[t][t] = sum_i r_t[i] u[i] k_t[i]
//     Y   = Qt S0 + M^T V                      (token x value)
//     S_C = diag(E_C) (S0 + Kh^T V)
// The products run on v_mfma_f32_16x16x32_bf16 with fp32 operands fed as a truncated-bf16 "hi" plus a bf16 "lo"
// part (hi.hi + hi.lo + lo.hi); v is bf16 on input and needs no split.
//
// Work split, LDS ring and hand-shake are those of the WKV7 chunked kernel: one workgroup of 8 waves per
// (sequence, head); consumer wave q keeps the state columns of values 16q..16q+15 in accumulator registers for
// the whole sequence (key x value tiles, reused directly as B operands); producer p prepares chunks p, p+4, ...
// (decay scan, scaled operands, Gram tile, operand transposes).  A slot is 12 KB, so two workgroups share a CU.
// new_starts inside a chunk restart the cumulative decay and mask the Gram tile (rare, uniform branch); `length`
// snapshots use a second, masked set of update operands for the one chunk that holds token length-1.
//
// Range: a key channel whose total log decay over a 16-token chunk is below -80 gets its steps of that chunk scaled
// to a total of -80, so that 1/E_s stays finite in fp32: finite and well ordered, but no longer exact for that channel
// (a decay of e^-5 per token sustained over a whole chunk; RWKV-7 keeps d >= 0.54 per token, i.e. e^-10 per chunk).
// The sequential kernels have no such limit.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight

// One chunk's operands as the consumers read them.  "lane-indexed" arrays hold, for every lane of the producer,
// the bytes the same lane of a consumer loads: accumulator-layout registers (column lane%16, rows 4*(lane/16)..+3)
// packed to bf16, hi pair then lo pair, which is an A operand (row lane%16, k-slots 4*(lane/16)..+3 of the hi
// part followed by the same slots of the lo part).
struct __attribute__((aligned(16))) Slot {
  // Qt = r_t.Ee_t, [hi|lo][token][RS]: within a row, the 16-byte vector (j, g) at element 32j + 8g holds keys
  // 32j+4g..+3 followed by keys 32j+16+4g..+3, the key order of the consumers' state tiles.  Rows the entering
  // state does not reach are zero.
  uint16_t Q[2][CK][RS];
  uint4 KT[4][64];             // (k_s/E_s)^T per key tile: hi,lo, lane-indexed; masked for the chunk-end state
  uint2 VT[4][64];             // v^T per value tile, lane-indexed
  uint4 M[64];                 // Gram tile with the bonus diagonal: hi,lo, lane-indexed
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {
  uint4 KT[4][64];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys {8g..8g+7} u {32+8g..32+8g+7}: the A/B operand
// layout of the Gram MFMAs (row/column = token, k-slots = keys), and one 16-byte global load per half.
struct Raw {
  uint4 r[2], k[2], v[2], w[2];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const uint4 z = make_uint4(0, 0, 0, 0);
  if (c0 + t < A.T) {
    const size_t off = ((((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g) * 2;  // bytes
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off + 64);
    };
    ld(A.r, x.r); ld(A.k, x.k); ld(A.v, x.v);
    // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
    const size_t woff = (A.flags & FLAG_W_PER_HEAD) ? ((size_t)h * 64 + 8 * g) * 2 : off;
    x.w[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff);
    x.w[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff + 64);
  } else {
    x.r[0] = x.r[1] = x.k[0] = x.k[1] = x.v[0] = x.v[1] = x.w[0] = x.w[1] = z;
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // MFMA-as-transposer selection operands
  const char* u;      // the bonus of this lane's keys (bf16, staged in LDS): 16 bytes here and 16 bytes 64 bytes on
};

__device__ __forceinline__ void produce(const Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap) {
  const int lane = P.lane, t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint32_t resets = F.ns & 0xffffu;
  const bool slow = resets != 0;                  // a reset inside this chunk
  int lastseg = 0, seg_src = 0;
  bool s0_reaches = true, restart = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    lastseg = seg_of(resets, 15);
    s0_reaches = seg_of(resets, t) == 0;                            // the entering state reaches this token
    keep_upd = 0xffffu & ~((1u << (31 - __builtin_clz(resets))) - 1u);   // tokens from the last reset on
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

  f32x4_t M = zero4;
  float bonus = 0.f;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ---- v^T of value tiles 2hf, 2hf+1
    {
      const uint4 vr = x.v[hf];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w};
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) slot->VT[2 * hf + x2][lane] = plain_pack(mfma(vop, P.sel[x2], zero4));
    }
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain
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
      cap_chunk_decay(E, lane);
    }
    if (slow) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
        if (restart) E[e] -= base;
      }
    }
    // ---- scaled operands and their hi/lo split
    u32x4_t qt_h, qt_l, kh_h, kh_l;
    {
      float fr[8], fk[8], fu[8], Einv[8], Ee[8];
      unpack8(x.r[hf], fr); unpack8(x.k[hf], fk);
      unpack8(*reinterpret_cast<const uint4*>(P.u + 64 * hf), fu);   // re-read per chunk from LDS: frees registers
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = fmaxf(E[e], MIN_CUM_L2);
        E[e] = exp2_fast(l2);
        Einv[e] = exp2_fast(-l2);
        // exclusive: value of the previous token; 1 for the first token of the chunk.  At a reset token the value
        // belongs to the previous segment, but every product it enters is masked out.
        Ee[e] = row_prev(E[e], 1.0f);
        bonus = fmaf(fr[e] * fu[e], fk[e], bonus);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = 2 * j;
        uint32_t hi, lo;
        split2(fr[e] * Ee[e], fr[e + 1] * Ee[e + 1], hi, lo); qt_h[j] = hi; qt_l[j] = lo;
        split2(fk[e] * Einv[e], fk[e + 1] * Einv[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
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
    // ---- Qt rows for the consumers, in their key order: this lane's keys 8g..8g+3 and 8g+4..8g+7 of the half are
    //      the (g>>1)-th 8-byte piece of the vectors 2(g&1) and 2(g&1)+1 of block j = hf
    {
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // element offset of the first piece
      auto put = [&](uint16_t* row, const u32x4_t v, bool keep) {
        *reinterpret_cast<uint2*>(row + e0) = keep ? make_uint2(v[0], v[1]) : make_uint2(0u, 0u);
        *reinterpret_cast<uint2*>(row + e0 + 8) = keep ? make_uint2(v[2], v[3]) : make_uint2(0u, 0u);
      };
      put(slot->Q[0][t], qt_h, s0_reaches);
      put(slot->Q[1][t], qt_l, s0_reaches);
    }
    // ---- (k/E)^T of key tiles 2hf, 2hf+1 by MFMA: the accumulator layout of D (lane = key, registers = 4
    //      consecutive tokens) is the A-operand layout of the state update
#pragma unroll
    for (int x2 = 0; x2 < 2; ++x2) {
      const int tile = 2 * hf + x2;
      const u32x4_t sel = P.sel[x2];
      const f32x4_t dkh = mfma(kh_h, sel, zero4), dkl = mfma(kh_l, sel, zero4);
      if (keep_upd == 0xffffu) slot->KT[tile][lane] = join(plain_pack(dkh), plain_pack(dkl));
      else slot->KT[tile][lane] = join(masked_pack(dkh, keep_upd), masked_pack(dkl, keep_upd));
      if (F.snap >= 0) snap->KT[tile][lane] = join(masked_pack(dkh, keep_snap), masked_pack(dkl, keep_snap));
    }
    // ---- partial Gram sums over this half's keys: [s][t] = kh_s . qt_t (column n = lane%16 = t, rows 4g..4g+3 = s)
    M = mfma(kh_h, qt_h, M);
    M = mfma(kh_h, qt_l, M);
    M = mfma(kh_l, qt_h, M);
  }
  // ---- bonus of token t summed over the four key groups
  bonus += __shfl_xor(bonus, 16, 64);
  bonus += __shfl_xor(bonus, 32, 64);
  // ---- strictly lower triangle within a segment, bonus on the diagonal
  const int n = t;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool lt = m < n;
    if (slow) lt = lt && seg_of(resets, m) == seg_of(resets, n);
    M[i] = lt ? M[i] : (m == n ? bonus : 0.f);
  }
  uint32_t hi0, lo0, hi1, lo1;
  split2(M[0], M[1], hi0, lo0);
  split2(M[2], M[3], hi1, lo1);
  slot->M[lane] = make_uint4(hi0, hi1, lo0, lo1);
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state columns of values 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), S[tile][i] = S[key 16*tile + 4g + i][value 16q + n].
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

// Operands carried from one chunk to the next; reloaded for the next chunk right after their last use.
struct Ops {
  u32x4_t qt[2][2];        // [hi|lo][j]: Qt rows in the key order of the state tiles
  u32x4_t M;               // Gram tile: hi pair, lo pair
  u32x4_t vv;              // v^T of this wave's value tile, twice (for a hi and a lo A part side by side)
  int keep_end;
};

__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int pl = 0; pl < 2; ++pl)
#pragma unroll
    for (int j = 0; j < 2; ++j) o.qt[pl][j] = *reinterpret_cast<const u32x4_t*>(&slot->Q[pl][n][32 * j + 8 * g]);
  o.M = *reinterpret_cast<const u32x4_t*>(&slot->M[lane]);
  const uint2 v0 = slot->VT[q][lane];
  o.vv = u32x4_t{v0.x, v0.y, v0.x, v0.y};
  o.keep_end = slot->keep_end;
}

struct OutCursor {
  char* y;             // A.out at (b, c0, h, 0)
  size_t tok_bytes;    // bytes between consecutive tokens in y
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + value
};

__device__ __forceinline__ size_t state_off(const Wkv6Args& A, int64_t b, int64_t h, int key, int value) {
  return (((size_t)b * A.H + h) * 64 + key) * 64 + value;
}

template <class WaitNext>
__device__ __forceinline__ bool consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
                                        const Slot* __restrict__ next, const SnapSlot* __restrict__ snapslot,
                                        const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool q2drop,
                                        OutCursor& oc, WaitNext&& next_ready) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  u32x4_t kt[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) kt[tile] = *reinterpret_cast<const u32x4_t*>(&slot->KT[tile][lane]);
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
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
  f32x4_t Y = mfma(o.M, o.vv, zero4), Y2 = zero4;   // [token 4g+i][value n]; two accumulation chains
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    Y = mfma(o.qt[0][j], Sh[j], Y);
    Y2 = mfma(o.qt[0][j], Sl[j], Y2);
    Y = mfma(o.qt[1][j], Sh[j], Y);
  }
  const u32x4_t vv = o.vv;
  // Qt and the Gram tile are dead now: fetch the next chunk's into the same registers, and this chunk's decay
  asm volatile("" ::: "memory");   // keeps these loads below the products above (register pressure)
  float4 gm[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) gm[tile] = *reinterpret_cast<const float4*>(&slot->gamma[16 * tile + 4 * g]);
  bool ok = true;
  if (next != nullptr) {
    ok = next_ready();
    load_ops(o, next, C.q, lane);
  }
  // state snapshot for `length` (one chunk per sequence)
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
    // lane part of the state address, formed here so that it does not stay live across the chunk loop
    uint32_t lane_el = (uint32_t)(4 * g * 64 + 16 * C.q + n);
    asm volatile("" : "+v"(lane_el));
    char* const base = reinterpret_cast<char*>(A.new_s) + state_off(A, b, h, 0, 0) * (A.st_f32 ? 4 : 2);
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const u32x4_t sk = *reinterpret_cast<const u32x4_t*>(&snapslot->KT[tile][lane]);
      f32x4_t acc = mfma(sk, vv, keep ? C.S[tile] : zero4);
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      acc[0] *= sg.x; acc[1] *= sg.y; acc[2] *= sg.z; acc[3] *= sg.w;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t el = lane_el + (uint32_t)((16 * tile + i) * 64);
        const float x = q2drop ? 0.f : acc[i];
        if (A.st_f32) *reinterpret_cast<float*>(base + (size_t)el * 4) = x;
        else *reinterpret_cast<uint16_t*>(base + (size_t)el * 2) = f32_to_bf16(x);
      }
    }
  }
  // state update, tile by tile: S <- diag(gamma) (S + Kh^T V)
  if (!keep_end) {
    asm volatile("" ::: "memory");   // keep this a (rare, uniform) branch instead of 16 selects on the hot path
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;   // a reset inside the chunk cuts the entering state off
  }
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    f32x4_t acc = mfma(kt[tile], vv, C.S[tile]);
    acc[0] *= gm[tile].x; acc[1] *= gm[tile].y; acc[2] *= gm[tile].z; acc[3] *= gm[tile].w;
    C.S[tile] = acc;
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  const uint32_t y01 = pack_rn(Y[0] + Y2[0], Y[1] + Y2[1]), y23 = pack_rn(Y[2] + Y2[2], Y[3] + Y2[3]);
  char* const yl = oc.y + (size_t)oc.voff * 2;
  if (nvalid == CK) {
    *reinterpret_cast<uint16_t*>(yl) = (uint16_t)(y01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + oc.tok_bytes) = (uint16_t)(y01 >> 16);
    *reinterpret_cast<uint16_t*>(yl + 2 * oc.tok_bytes) = (uint16_t)(y23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + 3 * oc.tok_bytes) = (uint16_t)(y23 >> 16);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (4 * g + i < nvalid) {
        const uint32_t yv = (i & 2) ? y23 : y01;
        *reinterpret_cast<uint16_t*>(yl + i * oc.tok_bytes) = (uint16_t)((i & 1) ? (yv >> 16) : (yv & 0xffffu));
      }
    }
  }
  oc.y += CK * oc.tok_bytes;
  return ok;
}

__device__ __forceinline__ void load_state(Consumer& C, const Wkv6Args& A, int64_t b, int64_t h) {
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const size_t off = state_off(A, b, h, 16 * tile + 4 * g + i, 16 * C.q + n);
      C.S[tile][i] = A.st_f32 ? reinterpret_cast<const float*>(A.s)[off]
                              : bf16_to_f32(reinterpret_cast<const uint16_t*>(A.s)[off]);
    }
}

__device__ __forceinline__ void store_state0(const Consumer& C, const Wkv6Args& A, int64_t b, int64_t h, bool zero) {
  // length == 0: the returned state is the input state, or the reset state under the associative rule (rwkv6.py:301)
  const int n = C.lane & 15, g = C.lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const size_t off = state_off(A, b, h, 16 * tile + 4 * g + i, 16 * C.q + n);
      const float x = zero ? 0.f : C.S[tile][i];
      if (A.st_f32) reinterpret_cast<float*>(A.new_s)[off] = x;
      else reinterpret_cast<uint16_t*>(A.new_s)[off] = f32_to_bf16(x);
    }
}

}  // namespace

// Slot c % RING holds chunk c.  Producer p fills it once every consumer has released chunk c - RING, then
// publishes ready = c + 1; consumers take chunks in order.  Every wait is for a strictly earlier chunk, so the
// hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD), 4) void wkv6_chunk_fwd_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  uint16_t* ulds = reinterpret_cast<uint16_t*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync));   // u of this head
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int64_t nchunks = (A.T + CK - 1) / CK;
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  if (threadIdx.x < 64) ulds[threadIdx.x] = reinterpret_cast<const uint16_t*>(A.u)[(size_t)(blockIdx.x % A.H) * 64 + threadIdx.x];
  __syncthreads();

  if (wave < NCONS) {
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
    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * wave + (lane & 15));
    const int csnap = L >= 1 ? (int)((L - 1) / CK) : -1;
    const int nch = (int)nchunks;
    Ops ops;
    bool ok = true;
    if (nch > 0) {
      ok = wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], wave, lane);
    }
    for (int c = 0; c < nch && ok; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING, sn = (c + 1) % RING;
      const Slot* next = (c + 1 < nch) ? &slots[sn] : nullptr;
      ok = consume(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, c == csnap, q2drop, oc,
                   [&]() { return wait_ready(sy, sn, c + 2); });
      // every LDS read of slot si has returned: its data went into the MFMAs above
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
    P.u = reinterpret_cast<const char*>(ulds) + 8 * (lane >> 4) * 2;
    Raw raw;
    if (p < nchunks) load_raw(raw, A, b, h, (int64_t)p * CK, lane);
    for (int64_t c = p; c < nchunks; c += NPROD) {
      const int64_t c0 = c * CK;
      const ChunkFlags F = chunk_flags(A.ns, A.flags, A.T, b, c0, L, lane);
      const int si = (int)(c % RING);
      Slot* slot = &slots[si];
      if (c >= RING && !wait_consumed(sy, si, (int)(c - RING) + 1, lane)) break;
      produce(P, raw, F, slot, snapslot);
      if (c + NPROD < nchunks) load_raw(raw, A, b, h, c0 + NPROD * CK, lane);
      if ((A.flags & FLAG_DROP_PUBLISH) && c + 1 == nchunks) break;
      // the release orders this wave's LDS writes before the sequence number
      if (lane == 0) __hip_atomic_store(&sy->ready[si], (int)c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  __syncthreads();
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.out, 2, b, h, A.T, A.H);
    poison_state(A.new_s, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv6_chunk_fwd(const Wkv6Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) + 64 * sizeof(uint16_t);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_chunk_fwd_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_chunk_fwd_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
