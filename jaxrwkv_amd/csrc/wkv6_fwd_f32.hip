// WKV6 chunked forward for fp32 I/O on gfx950: 16 tokens at a time on the matrix cores with fp32 operands
// (v_mfma_f32_16x16x4_f32), for callers that need y and the state to fp32 accuracy.
//
// Recurrence per head (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191), S[i][j] = key row i, value col j,
// dec_t = exp(w_t) with w the log decay:
//     S' = new_starts[t] ? 0 : S ;  y_t = r_t^T (diag(u) k_t v_t^T + S') ;  S = diag(dec_t) S' + k_t v_t^T
// The chunk algebra is the one of the bf16 kernel (wkv6_fwd.hip): with Lc_t = sum_{s<=t} w_s,
//     qt_t = r_t exp(Lc_{t-1})   kh_s = k_s exp(-Lc_s)   ke_s = k_s exp(Lc_15 - Lc_s)
//     M[s][t] = kh_s.qt_t (s < t),  M[t][t] = sum_i r_t[i] u[i] k_t[i]
//     Y = Qt S0 + M^T V                      S_C = diag(exp(Lc_15)) S0 + Ke^T V
// Every product runs on the fp32 matrix instruction, so no operand is rounded below fp32.  D = A B with A: lane
// (m = lane%16, g = lane/16) holds A[m][k = g], B: lane (n, g) holds B[k = g][n], D: lane (n, g) holds rows 4g..4g+3 of
// column n; an accumulator register i of a tile X is X as a B operand (k-slot g = row 4g+i) and X^T as an A operand.
//
// Work split: one workgroup of eight waves per (sequence, head), one consumer and one producer per SIMD.  Consumer q
// keeps the state columns of values 16q..16q+15 in accumulator registers (36 matrix instructions per chunk); producer p
// prepares chunks p, p+4, ... (decay scan, scaled operands, the Gram tile: 16 matrix instructions) into a ring of LDS
// slots.  Synchronisation, resets, `length` and the decay floor are those of the other chunked kernels
// (chunk_common.h); the running log-decay is split into a part on a 2^-16 grid and a remainder as in wkv7_fwd_f32.hip.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 8;           // slots in flight (a slot is 14 KB)
constexpr float LN2 = 0.69314718055994530942f;
constexpr float GRID_MAGIC = 192.f;   // (x + 192) - 192 rounds |x| < 64 to a multiple of 2^-16
constexpr int RF = 68;            // row stride (floats) of the [token][64] LDS arrays: rows 4 apart fall 16 banks apart

__device__ __forceinline__ f32x4_t mfma_f(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float row_last(float x) {      // lane 15 of the row in every lane (row_newbcast:15)
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x15F, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_prev0(float x) {     // previous lane of the row, 0 in lane 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true));
}

struct __attribute__((aligned(16))) Slot {
  float Q[CK][RF];             // qt rows [token][key]; rows the entering state does not reach are zero
  float KE[CK][RF];            // ke rows (tokens outside the last segment are zero)
  float V[CK][RF];
  f32x4_t M[64];               // Gram tile with the bonus diagonal, accumulator layout [row s][column t], lane-indexed
  float gamma[64];             // exp(Lc_15)
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to the snapshot token
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {   // update operands referenced to token length-1 (one chunk per sequence)
  float KE[CK][RF];
  float gamma[64];
};

// ---------------------------------------------------------------------------------------------------- producer
// Lane (t = lane%16, g = lane/16) owns token t and the keys 16j + 4g + i (j, i = 0..3): one 16-byte load per j, and
// element (j, i) is this lane's k-slot of the Gram instruction (j, i) both as A and as B operand.
struct Raw {
  float4 r[4], k[4], v[4], w[4];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  const int64_t tok = (c0 + t < A.T) ? c0 + t : A.T - 1;   // always a valid token; mask_raw zeroes the lanes beyond
  const size_t off = (((size_t)b * A.T + tok) * A.H + h) * 64 + 4 * g;
  auto ld = [&](const void* p, size_t o, float4 (&d)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + o + 16 * j);
  };
  ld(A.r, off, x.r); ld(A.k, off, x.k); ld(A.v, off, x.v);
  // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
  ld(A.w, (A.flags & FLAG_W_PER_HEAD) ? (size_t)h * 64 + 4 * g : off, x.w);
}
__device__ __forceinline__ void mask_raw(Raw& x, int nvalid, int lane) {
  if (nvalid != CK) {
    rare_path();
    if ((lane & 15) >= nvalid) {
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) x.r[j] = x.k[j] = x.v[j] = x.w[j] = z;
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

// Everything of one chunk that does not depend on the carried state.  `ulds`: the bonus u of this head in LDS (fp32).
__device__ __forceinline__ void produce(int lane, const Raw& x, const ChunkFlags& F, const float* __restrict__ ulds,
                                        Slot* __restrict__ slot, SnapSlot* __restrict__ snap, unsigned* events) {
  const int t = lane & 15, g = lane >> 4;
  const bool valid = t < F.nvalid;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
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
    {
      float fv[8];
      unpack2(x.v[2 * hf], x.v[2 * hf + 1], fv);
      put2(slot->V[t], hf, g, fv, true);
    }
    // ---- decay scan over the 16 tokens (lanes of one DPP row), log2 domain: every step is split into a part on a
    //      2^-16 grid, whose running sums are exact, and a remainder below 2^-17, summed separately
    float E[8], El[8];
    {
      float fw[8];
      unpack2(x.w[2 * hf], x.w[2 * hf + 1], fw);
#pragma unroll
      for (int e = 0; e < 8; ++e) fw[e] = fmaxf(fw[e] * LOG2E, MIN_STEP_L2);
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
    float fqt[8], fkh[8], fke[8];
    {
      float fr[8], fk[8];
      unpack2(x.r[2 * hf], x.r[2 * hf + 1], fr);
      unpack2(x.k[2 * hf], x.k[2 * hf + 1], fk);
      const float4 u0 = *reinterpret_cast<const float4*>(ulds + 32 * hf + 4 * g);        // re-read per chunk: frees registers
      const float4 u1 = *reinterpret_cast<const float4*>(ulds + 32 * hf + 16 + 4 * g);
      const float fu[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = E[e];                    // >= MIN_CUM_L2 - 1: exp2(-l2) is finite
        const float fl = fmaf(LN2, El[e], 1.f);   // exp2 of the remainder (|El| < 2^-13: second order below 1e-8)
        E[e] = exp2_fast(l2) * fl;
        const float einv = exp2_fast(-l2) * (2.f - fl);
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
      *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
      *reinterpret_cast<float4*>(&slot->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
    }
    put2(slot->KE[t], hf, g, fke, (keep_upd >> t) & 1u);   // tokens before the last reset do not reach the chunk end
    if (F.snap >= 0) {                                     // the same referenced to token length-1
      rare_path();
      float ske[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) ske[e] = fkh[e] * __shfl(E[e], (lane & 48) | F.snap, 64);
      put2(snap->KE[t], hf, g, ske, (keep_snap >> t) & 1u);
      if (t == F.snap) {
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 4 * g]) = make_float4(E[0], E[1], E[2], E[3]);
        *reinterpret_cast<float4*>(&snap->gamma[32 * hf + 16 + 4 * g]) = make_float4(E[4], E[5], E[6], E[7]);
      }
    }
    put2(slot->Q[t], hf, g, fqt, s0_reaches);
    // ---- partial Gram sums over this half's keys
#pragma unroll
    for (int e = 0; e < 8; ++e) M = mfma_f(fkh[e], fqt[e], M);   // [s][t] = kh_s . qt_t
  }
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
  slot->M[lane] = M;
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state columns of values 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16,
// g = lane/16), S[tile][i] = S[key 16*tile + 4g + i][value 16q + n]: register i of a tile is the B operand of the
// instruction that contracts over the keys 16*tile + 4g' + i (g' = 0..3).
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

struct Ops {               // fetched a chunk ahead
  float4 qt[4];            // row of token n: keys 16*tile + 4g .. +3
  f32x4_t M;
  f32x4_t vv;              // v of tokens 4g..4g+3, value 16q + n
  int keep_end;
};

__device__ __forceinline__ void load_ops(Ops& o, const Slot* __restrict__ slot, int q, int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) o.qt[tile] = *reinterpret_cast<const float4*>(&slot->Q[n][16 * tile + 4 * g]);
  o.M = slot->M[lane];
#pragma unroll
  for (int i = 0; i < 4; ++i) o.vv[i] = slot->V[4 * g + i][16 * q + n];
  o.keep_end = slot->keep_end;
}

// A operand of the state update of one key tile: ke of tokens 4g..4g+3, key 16*tile + n
__device__ __forceinline__ f32x4_t load_upd(const float (*ke)[RF], int tile, int lane) {
  const int n = lane & 15, g = lane >> 4;
  f32x4_t r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = ke[4 * g + i][16 * tile + n];
  return r;
}

struct OutCursor {
  float* y;            // A.out at (b, c0, h, 0)
  size_t tok;          // elements between consecutive tokens
  uint32_t voff;       // lane part of the address: (4g * H) * 64 + value
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
  f32x4_t up[4];
  float4 gm[4];
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    up[tile] = load_upd(slot->KE, tile, lane);
    gm[tile] = *reinterpret_cast<const float4*>(&slot->gamma[16 * tile + 4 * g]);
  }
  const bool keep_end = __builtin_amdgcn_readfirstlane(o.keep_end) != 0;
  // Y = Qt S0 + M^T V, [token 4g+i][value n]; two accumulation chains, joined at the end
  f32x4_t Y = zero4, Y2 = zero4;
#pragma unroll
  for (int i = 0; i < 4; ++i) Y2 = mfma_f(o.M[i], o.vv[i], Y2);
#pragma unroll
  for (int tile = 0; tile < 4; ++tile) {
    const float qt[4] = {o.qt[tile].x, o.qt[tile].y, o.qt[tile].z, o.qt[tile].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (tile & 1) Y2 = mfma_f(qt[i], C.S[tile][i], Y2);
      else Y = mfma_f(qt[i], C.S[tile][i], Y);
    }
  }
  const f32x4_t vv = o.vv;
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
      const f32x4_t su = load_upd(snapslot->KE, tile, lane);
      const float4 sg = *reinterpret_cast<const float4*>(&snapslot->gamma[16 * tile + 4 * g]);
      f32x4_t acc = zero4;
      if (keep) {
        acc[0] = C.S[tile][0] * sg.x; acc[1] = C.S[tile][1] * sg.y;
        acc[2] = C.S[tile][2] * sg.z; acc[3] = C.S[tile][3] * sg.w;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) acc = mfma_f(su[i], vv[i], acc);
      store_state_tile(A, b, h, C.q, lane, tile, q2drop ? zero4 : acc);
    }
  }
  // state update: S <- diag(gamma) S + Ke^T V; a reset inside the chunk cuts the entering state off.  The four key
  // tiles take turns, so that no instruction accumulates on the result of the one before it.
  if (keep_end) {
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
      C.S[tile][0] *= gm[tile].x; C.S[tile][1] *= gm[tile].y; C.S[tile][2] *= gm[tile].z; C.S[tile][3] *= gm[tile].w;
    }
  } else {
    rare_path();
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = zero4;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) C.S[tile] = mfma_f(up[tile][i], vv[i], C.S[tile]);
  // outputs: register i is token 4g+i, lanes n = 16 consecutive values
  Y += Y2;
  float* const yl = oc.y + oc.voff;
  if (nvalid == CK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) yl[i * oc.tok] = Y[i];
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (4 * g + i < nvalid) yl[i * oc.tok] = Y[i];
  }
  oc.y += CK * oc.tok;
  return ok;
}

}  // namespace

// Step j handles chunk j in slot j % RING.  Producer p fills the slot once every consumer has released step j - RING,
// then publishes ready = j + 1; consumers take the steps in order.  Every wait is for a strictly earlier step, so
// the hand-shake cannot cycle.
__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv6_fwd_f32_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  float* ulds = reinterpret_cast<float*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync));   // u of this head
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t b = blockIdx.x / A.H, h = blockIdx.x % A.H;
  int64_t L = A.length ? (int64_t)A.length[b] : A.T;
  L = L < A.T ? L : A.T;
  const int nch = (int)((A.T + CK - 1) / CK);
  if (threadIdx.x < sizeof(Sync) / sizeof(int)) reinterpret_cast<int*>(sy)[threadIdx.x] = 0;
  if (threadIdx.x < 64) ulds[threadIdx.x] = reinterpret_cast<const float*>(A.u)[(size_t)h * 64 + threadIdx.x];
  __syncthreads();

  if (wave < NCONS) {                 // waves 0..3: one consumer per SIMD; waves 4..7: one producer per SIMD
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
    oc.tok = (size_t)A.H * 64;
    oc.y = reinterpret_cast<float*>(A.out) + (((size_t)b * A.T) * A.H + h) * 64;
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
      // every LDS read of slot si has returned: its data went into the matrix instructions above
      if (lane == 0) __hip_atomic_store(&sy->consumed[cq][si], j + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
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
    poison_token_rows(A.out, 4, b, h, A.T, A.H);
    poison_state(A.new_s, A.st_f32, b, h, A.H);
  }
}

hipError_t launch_wkv6_chunk_fwd_f32(const Wkv6Args& A, hipStream_t stream) {
  static_assert(RING <= MAX_RING, "the hand-shake words cover MAX_RING slots");
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) + 64 * sizeof(float);
  static_assert(RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Sync) + 64 * sizeof(float) <= 160 * 1024, "LDS of one CU");
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_fwd_f32_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_fwd_f32_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
