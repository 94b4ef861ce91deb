// WKV6 chunked forward for bf16 I/O on gfx950: 16 tokens at a time on the matrix cores, fp16 operands.
//
// Recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191), S[i][j] = key row i, value col j,
// dec_t = exp(w_t) with w the log decay:
//     S' = new_starts[t] ? 0 : S ;  y_t = r_t^T (diag(u) k_t v_t^T + S') ;  S = diag(dec_t) S' + k_t v_t^T
// A chunk of 16 tokens entering with state S0 is evaluated in closed form.  With Lc_t = sum_{s<=t} w_s:
//     qt_t = r_t exp(Lc_{t-1})   kh_s = k_s exp(-Lc_s)   ke_s = k_s exp(Lc_15 - Lc_s)
//     M[s][t] = kh_s.qt_t (s < t),  M[t][t] = sum_i r_t[i] u[i] k_t[i]
//     Y = Qt S0 + M^T V                      S_C = diag(exp(Lc_15)) S0 + Ke^T V
//
// Operand formats.  qt, ke, v, the state and M are bounded by the inputs' magnitudes: they go to the matrix cores as
// fp16 numbers (11 significant bits; the values must stay inside the fp16 range, |x| < 65504) -- single ones but for
// M, whose diagonal and first sub-diagonals carry most of y and which is fed as an fp16 pair hi + lo at no cost (one
// K = 32 instruction instead of a K = 16 one: 8 % of the y elements differed from the exactly rounded ones with a
// single M, 2.6 % with the pair).  kh carries exp(-Lc) and needs the fp32 exponent range: the Gram tile is formed from
// bf16 hi + lo pairs of kh and qt (three partial products).  The state stays in fp32 accumulator registers for the
// whole sequence.
//
// Work split, LDS ring and hand-shake are those of the WKV7 forward kernel (wkv7_fwd.hip): four consumer waves
// (consumer q keeps the state columns of values 16q..16q+15, key x value tiles that are B operands as they are)
// and NPROD producer waves (decay scan, scaled operands, Gram tile) around a ring of LDS slots; ke and v are written
// row-major and read transposed with ds_read_b64_tr_b16.  new_starts inside a chunk restart the cumulative decay and
// mask the Gram tile (rare, uniform branch); the one chunk that holds token length-1 gets a second set of update
// operands, referenced to that token, for the state snapshot.
//
// Range: a key channel whose total log decay over a chunk is below -80 gets its steps of that chunk scaled to a total
// of -80 (cap_chunk_decay), so that exp(-Lc) stays finite in fp32.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 6;          // producer waves; producer p owns chunks p, p + NPROD, ... (4: 20 % slower, 8: +1 %)
constexpr int RING = 10;          // slots in flight

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_h(float x0, float x1) {   // round to nearest fp16 pair
  const f16x2_t p = {(_Float16)x0, (_Float16)x1};
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ u32x2_t pack_h4(const f32x4_t d) { return u32x2_t{pack_h(d[0], d[1]), pack_h(d[2], d[3])}; }
__device__ __forceinline__ uint4 pack_h8(const float (&f)[8]) {
  return make_uint4(pack_h(f[0], f[1]), pack_h(f[2], f[3]), pack_h(f[4], f[5]), pack_h(f[6], f[7]));
}

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

__device__ __forceinline__ float row_last(float x) {      // lane 15 of the row in every lane (row_newbcast:15)
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x15F, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_prev0(float x) {     // previous lane of the row, 0 in lane 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true));
}

// One chunk's operands as the consumers read them.
struct __attribute__((aligned(16))) Slot {
  // qt in fp16, [token][RS]: within a row the 16-byte vector (j, g) at element 32j + 8g holds keys 32j+4g..+3
  // followed by keys 32j+16+4g..+3, the key order of the consumers' state tiles.  Rows the entering state does not
  // reach are zero.
  uint16_t Q[CK][RS];
  uint16_t KE[CK][RS];         // ke in natural key order (tokens outside the last segment are zero)
  uint16_t V[CK][RS];          // v in fp16
  // Gram tile with the bonus diagonal as an fp16 pair hi, lo, lane-indexed: column t = lane%16, rows 4g..4g+3
  u32x4_t M[64];
  float gamma[64];             // exp(Lc_15)
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {   // update operands referenced to token length-1
  uint16_t KE[CK][RS];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys {8g..8g+7} u {32+8g..32+8g+7}: the A/B operand
// layout of the Gram MFMAs (row/column = token, k-slots = keys), and one 16-byte global load per half.
struct Raw {
  uint4 r[2], k[2], v[2], w[2];
};

// Loads always touch a valid token (the last one of the sequence for lanes beyond it); mask_raw zeroes those lanes.
__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;
  const size_t off = ((((size_t)b * A.T + tok) * A.H + h) * 64 + 8 * g) * 2;  // bytes
  auto ld = [&](const void* p, size_t o, uint4 (&d)[2]) {
    d[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + o);
    d[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + o + 64);
  };
  ld(A.r, off, x.r); ld(A.k, off, x.k); ld(A.v, off, x.v);
  // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
  ld(A.w, (A.flags & FLAG_W_PER_HEAD) ? ((size_t)h * 64 + 8 * g) * 2 : off, x.w);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const uint4 z = make_uint4(0, 0, 0, 0);
      x.r[0] = x.r[1] = x.k[0] = x.k[1] = x.v[0] = x.v[1] = x.w[0] = x.w[1] = z;
    }
  }
}

// Everything of one chunk that does not depend on the carried state.  `ulds`: the bonus u of this head in LDS (bf16).
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, const uint16_t* __restrict__ ulds,
                                        Slot* __restrict__ slot, SnapSlot* __restrict__ snap, unsigned* events) {
  const int t = lane & 15, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint4 zero16 = make_uint4(0u, 0u, 0u, 0u);
  const uint32_t resets = F.ns & 0xffffu;
  const bool slow = resets != 0;                  // a reset inside this chunk
  int lastseg = 0, seg_src = 0;
  bool s0_reaches = true, restart = false;
  uint32_t keep_upd = 0xffffu, keep_snap = 0;
  if (F.snap >= 0) keep_snap = (2u << F.snap) - 1u;
  if (slow) {
    rare_path();
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

  f32x4_t M = zero4;           // Gram tile [s = row][t = column]
  float bonus = 0.f;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // issue priority rises with the wave's progress through the chunk (see wkv7_fwd.hip)
    if (hf == 0) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(2);
    {
      float fv[8];
      unpack8(x.v[hf], fv);
      *reinterpret_cast<uint4*>(&slot->V[t][32 * hf + 8 * g]) = pack_h8(fv);
    }
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain
    float E[8];
    {
      float fw[8];
      unpack8(x.w[hf], fw);
#pragma unroll
      for (int e = 0; e < 8; ++e) fw[e] = fmaxf(fw[e] * LOG2E, MIN_STEP_L2);
      if (F.nvalid != CK) {
        rare_path();
#pragma unroll
        for (int e = 0; e < 8; ++e) fw[e] = (t < F.nvalid) ? fw[e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) E[e] = row_scan(fw[e]);
      cap_chunk_decay(E, lane, events);
    }
    if (slow) {
      rare_path();
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
        if (restart) E[e] -= base;
      }
    }
    // ---- scaled operands
    float fqt[8], fkh[8], fke[8];
    {
      float fr[8], fk[8], fu[8];
      unpack8(x.r[hf], fr); unpack8(x.k[hf], fk);
      unpack8(*reinterpret_cast<const uint4*>(ulds + 8 * g + 32 * hf), fu);   // re-read per chunk: frees registers
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = E[e];                    // >= MIN_CUM_L2: exp2(-l2) is finite
        E[e] = exp2_fast(l2);
        const float einv = exp2_fast(-l2);
        // r_t times the decay up to the previous token (1 for the first token of the chunk: fr0 carries that lane).
        // At a reset token the value belongs to the previous segment, but every product it enters is masked out.
        const float fr0 = (t == 0) ? fr[e] : 0.f;
        fqt[e] = fmaf(fr[e], row_prev0(E[e]), fr0);
        fkh[e] = fk[e] * einv;
        fke[e] = fkh[e] * row_last(E[e]);         // times the decay from the (last) segment start to the chunk end
        bonus = fmaf(fr[e] * fu[e], fk[e], bonus);
      }
    }
    if (t == 15) {
      float* gp = &slot->gamma[8 * g + 32 * hf];
      *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
    }
    {
      uint4 ke = pack_h8(fke);
      if (keep_upd != 0xffffu) {
        rare_path();
        if (!((keep_upd >> t) & 1u)) ke = zero16;          // tokens before the last reset do not reach the chunk end
      }
      *reinterpret_cast<uint4*>(&slot->KE[t][32 * hf + 8 * g]) = ke;
    }
    if (F.snap >= 0) {                                     // the same referenced to token length-1
      rare_path();
      const bool sk = (keep_snap >> t) & 1u;
      float ske[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) ske[e] = fkh[e] * __shfl(E[e], (lane & 48) | F.snap, 64);
      *reinterpret_cast<uint4*>(&snap->KE[t][32 * hf + 8 * g]) = sk ? pack_h8(ske) : zero16;
      if (t == F.snap) {
        float* gp = &snap->gamma[8 * g + 32 * hf];
        *reinterpret_cast<float4*>(gp) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(gp + 4) = make_float4(E[4], E[5], E[6], E[7]);
      }
    }
    // ---- qt rows for the consumers in their key order: this lane's keys 8g..8g+3 and 8g+4..8g+7 of the half are
    //      the (g>>1)-th 8-byte piece of the vectors 2(g&1) and 2(g&1)+1 of block j = hf
    {
      uint4 qh = pack_h8(fqt);
      if (slow) {
        rare_path();
        if (!s0_reaches) qh = zero16;
      }
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);
      *reinterpret_cast<uint2*>(&slot->Q[t][e0]) = make_uint2(qh.x, qh.y);
      *reinterpret_cast<uint2*>(&slot->Q[t][e0 + 8]) = make_uint2(qh.z, qh.w);
    }
    // ---- bf16 hi/lo pairs of the Gram operands and the partial Gram sums over this half's keys
    u32x4_t qt_h, qt_l, kh_h, kh_l;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 2 * j;
      uint32_t hi, lo;
      split2(fqt[e], fqt[e + 1], hi, lo); qt_h[j] = hi; qt_l[j] = lo;
      split2(fkh[e], fkh[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
    }
    M = mfma(kh_h, qt_h, M);     // [s][t] = kh_s . qt_t (column n = lane%16 = t, rows 4g..4g+3 = s)
    M = mfma(kh_h, qt_l, M);
    M = mfma(kh_l, qt_h, M);
  }
  __builtin_amdgcn_s_setprio(3);
  // ---- bonus of token t summed over the four key groups
  bonus += __shfl_xor(bonus, 16, 64);
  bonus += __shfl_xor(bonus, 32, 64);
  // ---- strictly lower triangle within a segment, bonus on the diagonal
  const int n = t;
  if (!slow) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      M[i] = m < n ? M[i] : (m == n ? bonus : 0.f);
    }
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * g + i;
      const bool lt = m < n && seg_of(resets, m) == seg_of(resets, n);
      M[i] = lt ? M[i] : (m == n ? bonus : 0.f);
    }
  }
  {
    const u32x2_t hi = pack_h4(M);
    const f16x4_t hf4 = __builtin_bit_cast(f16x4_t, hi);
    f32x4_t rest;
#pragma unroll
    for (int i = 0; i < 4; ++i) rest[i] = M[i] - (float)hf4[i];
    const u32x2_t lo = pack_h4(rest);
    slot->M[lane] = u32x4_t{hi[0], hi[1], lo[0], lo[1]};
  }
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
  }
  __builtin_amdgcn_s_setprio(0);
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state columns of values 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), S[tile][i] = S[key 16*tile + 4g + i][value 16q + n].
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

struct Ops {               // fetched a chunk ahead
  u32x4_t qt[2];           // qt rows in the key order of the state tiles
  u32x4_t M;               // hi part then lo part: the A operand of one K = 32 instruction against (v, v)
  u32x2_t vv;              // v^T of this wave's value tile: tokens 4g..4g+3 of value n
  int keep_end;
};

__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int j = 0; j < 2; ++j) o.qt[j] = *reinterpret_cast<const u32x4_t*>(&slot->Q[n][32 * j + 8 * g]);
  o.M = slot->M[lane];
  o.vv = lds_tr4(&slot->V[4 * g + (n >> 2)][16 * q + 4 * (n & 3)]);
  o.keep_end = slot->keep_end;
}

// A operand of the state update of one key tile: ke^T, tokens 4g..4g+3 of key 16*tile + n
__device__ __forceinline__ u32x2_t load_upd(const uint16_t (*ke)[RS], int tile, int lane) {
  const int n = lane & 15, g = lane >> 4;
  return lds_tr4(&ke[4 * g + (n >> 2)][16 * tile + 4 * (n & 3)]);
}

struct OutCursor {
  char* y;             // A.out at (b, c0, h, 0)
  size_t tok_bytes;    // bytes between consecutive tokens in y
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + value
};

__device__ __forceinline__ size_t state_off(const Wkv6Args& A, int64_t b, int64_t h, int key, int value) {
  return (((size_t)b * A.H + h) * 64 + key) * 64 + value;
}
__device__ __forceinline__ void store_state_tile(const Wkv6Args& A, int64_t b, int64_t h, int q, int lane, int tile,
                                                 const f32x4_t v) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const size_t off = state_off(A, b, h, 16 * tile + 4 * g + i, 16 * q + n);
    if (A.st_f32) reinterpret_cast<float*>(A.new_s)[off] = v[i];
    else reinterpret_cast<uint16_t*>(A.new_s)[off] = f32_to_bf16(v[i]);
  }
}

template <class PeekNext, class WaitNext>
__device__ __forceinline__ bool consume(Consumer& C, Ops& o, const Slot* __restrict__ slot,
                                        const Slot* __restrict__ next, const SnapSlot* __restrict__ snapslot,
                                        const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, bool q2drop,
                                        OutCursor& oc, PeekNext&& peek_next, WaitNext&& next_ready) {
  const int lane = C.lane, g = lane >> 4;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const int peeked = next != nullptr ? peek_next() : 0;
  u32x2_t up[4];
  float4 gm[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    up[tile] = load_upd(slot->KE, tile, lane);
    gm[tile] = *reinterpret_cast<const float4*>(&slot->gamma[16 * tile + 4 * g]);
  }
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
  // B operands from the state: MFMA j contracts over the keys of tiles 2j and 2j+1
  u32x4_t Sh[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    Sh[j] = u32x4_t{pack_h(C.S[2 * j][0], C.S[2 * j][1]), pack_h(C.S[2 * j][2], C.S[2 * j][3]),
                    pack_h(C.S[2 * j + 1][0], C.S[2 * j + 1][1]), pack_h(C.S[2 * j + 1][2], C.S[2 * j + 1][3])};
  f32x4_t Y = mfma_h(o.M, u32x4_t{o.vv[0], o.vv[1], o.vv[0], o.vv[1]}, zero4);   // M^T V: [token 4g+i][value n]
  Y = mfma_h(o.qt[0], Sh[0], Y);
  Y = mfma_h(o.qt[1], Sh[1], Y);
  const u32x2_t vv = o.vv;
  bool ok = true;
  if (next != nullptr) {
    ok = next_ready(peeked);
    load_ops(o, next, C.q, lane);
  }
  // state snapshot for `length` (one chunk per sequence)
  if (is_snap) {
    rare_path();
    const bool keep = slot->keep_snap != 0;
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      const u32x2_t su = load_upd(snapslot->KE, tile, lane);
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      f32x4_t acc = zero4;
      if (keep) {
        acc[0] = C.S[tile][0] * sg.x; acc[1] = C.S[tile][1] * sg.y;
        acc[2] = C.S[tile][2] * sg.z; acc[3] = C.S[tile][3] * sg.w;
      }
      acc = mfma_h16(su, vv, acc);
      store_state_tile(A, b, h, C.q, lane, tile, q2drop ? zero4 : acc);
    }
  }
  // state update, tile by tile: S <- diag(gamma) S + Ke^T V; a reset inside the chunk cuts the entering state off
  if (keep_end) {
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      f32x4_t acc = C.S[tile];
      acc[0] *= gm[tile].x; acc[1] *= gm[tile].y; acc[2] *= gm[tile].z; acc[3] *= gm[tile].w;
      C.S[tile] = mfma_h16(up[tile], vv, acc);
    }
  } else {
    rare_path();
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = mfma_h16(up[tile], vv, zero4);
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  const uint32_t y01 = pack_rn(Y[0], Y[1]), y23 = pack_rn(Y[2], Y[3]);
  char* const yl = oc.y + (size_t)oc.voff * 2;
  if (nvalid == CK) {
    *reinterpret_cast<uint16_t*>(yl) = (uint16_t)(y01 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + oc.tok_bytes) = (uint16_t)(y01 >> 16);
    *reinterpret_cast<uint16_t*>(yl + 2 * oc.tok_bytes) = (uint16_t)(y23 & 0xffffu);
    *reinterpret_cast<uint16_t*>(yl + 3 * oc.tok_bytes) = (uint16_t)(y23 >> 16);
  } else {
    rare_path();
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

}  // namespace

// Step j handles chunk j in slot j % RING.  Producer p fills the slot once every consumer has released step j - RING,
// then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier step, so
// the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv6_fwd_kernel(Wkv6Args A) {
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
  const int nch = (int)((A.T + CK - 1) / CK);
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  if (threadIdx.x < 64) ulds[threadIdx.x] = reinterpret_cast<const uint16_t*>(A.u)[(size_t)h * 64 + threadIdx.x];
  __syncthreads();

  if (wave < NCONS) {
    __builtin_amdgcn_s_setprio(3);    // the chunk-to-chunk dependency runs through the consumers
    const int cq = wave;
    const bool q2drop = (A.flags & 1u) && L < A.T && A.ns != nullptr && A.ns[b * A.T + L] != 0;
    Consumer C;
    C.q = cq;
    C.lane = lane;
    {
      const int n = lane & 15, g = lane >> 4;
#pragma unroll
      for (int tile = 0; tile < 4; ++tile)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const size_t off = state_off(A, b, h, 16 * tile + 4 * g + i, 16 * cq + n);
          C.S[tile][i] = A.st_f32 ? reinterpret_cast<const float*>(A.s)[off]
                                  : bf16_to_f32(reinterpret_cast<const uint16_t*>(A.s)[off]);
        }
    }
    // length == 0: the returned state is the input state, or the reset state under the associative rule (rwkv6.py:301)
    if (L == 0) {
      const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int tile = 0; tile < 4; ++tile) store_state_tile(A, b, h, cq, lane, tile, q2drop ? zero4 : C.S[tile]);
    }
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    oc.y = reinterpret_cast<char*>(A.out) + (((size_t)b * A.T) * A.H + h) * 64 * 2;
    oc.voff = (uint32_t)((4 * (lane >> 4)) * (int)A.H * 64 + 16 * cq + (lane & 15));
    const int csnap = L >= 1 ? (int)((L - 1) / CK) : -1;
    Ops ops;
    bool ok = true;
    if (nch > 0) {
      ok = wait_ready(sy, 0, 1);
      load_ops(ops, &slots[0], cq, lane);
    }
    for (int j = 0; j < nch && ok; ++j) {
      const int nvalid = (j + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = j % RING, sn = (j + 1) % RING;
      const Slot* next = (j + 1 < nch) ? &slots[sn] : nullptr;
      ok = consume(C, ops, &slots[si], next, snapslot, A, b, h, nvalid, j == csnap, q2drop, oc,
                   [&]() { return peek_ready(sy, sn); },
                   [&](int peeked) { return wait_ready_peeked(sy, sn, j + 2, peeked); });
      // every LDS read of slot si has returned: its data went into the MFMAs above
      if (lane == 0) __hip_atomic_store(&sy->consumed[cq][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    // an operand beyond the fp16 range leaves inf or NaN in the carried state (until a reset discards it): count it
    count_nonfinite(C.S, lane, events_word(A.status));
  } else {
    const int p = wave - NCONS;
    Raw raw;
    uint32_t ns_mine = 0u;      // this lane's new_starts byte of the chunk loaded next: fetched a step ahead, like the operands
    if (p < nch) {
      ns_mine = chunk_flag_prefetch(A.ns, A.T, b, (int64_t)p * CK, lane);
      load_raw(raw, A, b, h, (int64_t)p * CK, lane);
    }
    for (int j = p; j < nch; j += NPROD) {
      const int64_t c0 = (int64_t)j * CK;
      const ChunkFlags F = chunk_flags_of(A.ns, ns_mine, A.flags, A.T, c0, L);
      const int si = j % RING;
      if (j >= RING && !wait_consumed_lazy(sy, si, j - RING + 1, lane)) break;
      mask_raw(raw, F.nvalid, lane);
      produce(lane, raw, F, ulds, &slots[si], snapslot, events_word(A.status));
      if (j + NPROD < nch) {
        ns_mine = chunk_flag_prefetch(A.ns, A.T, b, c0 + (int64_t)NPROD * CK, lane);
        load_raw(raw, A, b, h, c0 + (int64_t)NPROD * CK, lane);
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
    poison_state(A.new_s, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv6_chunk_fwd(const Wkv6Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) + 64 * sizeof(uint16_t);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_fwd_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_fwd_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
