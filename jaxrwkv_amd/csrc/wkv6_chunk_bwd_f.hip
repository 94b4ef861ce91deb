// WKV6 backward, forward sweep F on the matrix cores (bf16 I/O, gfx950): gr, gu and the workspaces er = r.(S' dy)
// and eI = rowsum(dS_out * S_{length-1}) that the decay-gradient recursion of the reverse sweep consumes.
//
// State recurrence (reference: /root/reference/src/jaxrwkv/rwkv6.py:175-191), S[i][j] = key row i, value col j:
//     S' = new_starts[t] ? 0 : S ;  S = diag(dec_t) S' + k_t v_t^T ,  dec_t = exp(w_t)
//     dr_t[i] = u_i k_i c_t + sum_j S'_t[i][j] dy_j ,  c_t = v_t.dy_t ;   du[i] = sum_t r_i k_i c_t
// A chunk of C = 16 tokens entering with S0: E_t = prod_{s<=t} dec_s, Ee_t = E_{t-1}, kh_s = k_s/E_s,
//     S'_t = diag(Ee_t) (S0 + sum_{s<t} kh_s v_s^T)
//     S' dy_t = Ee_t . ( S0 dy_t + sum_{s<t} (v_s.dy_t) kh_s )        S_C = diag(E_C) (S0 + Kh^T V)
// The Gram tile N[s][t] = v_s.dy_t (bf16 x bf16, exact products) contracts over the values; its diagonal is c_t.
// Products with fp32 quantities run as hi.hi + hi.lo + lo.hi on v_mfma_f32_16x16x32_bf16.
//
// Work split as in the chunked forward kernels: 4 consumer waves hold the state split by keys (wave q: keys
// 16q..16q+15, all 64 values, value x key accumulator tiles reused as B operands), 4 producer waves prepare the
// state-independent operands into a ring of LDS slots; bounded-poll hand-shake.  The producers also own the terms
// that need no state: u k c_t (handed over as an fp32 add-on) and du (summed per producer, combined at the end).
// Range: as in the forward kernel, a chunk's total log decay per channel is capped at -80.
#include "chunk_common.h"
#include "wkv_args.h"

namespace hiprwkv {

namespace {

using namespace chunk;

constexpr int NPROD = 4;          // producer waves; producer p owns chunks p, p + NPROD, ...
constexpr int RING = 5;           // slots in flight (a slot is 21 KB)
constexpr int ES = 68;            // row stride (floats) of the fp32 [token][key] arrays: conflict-free column reads

// "lane-indexed" arrays hold, for every lane of the producer, the bytes the same lane of a consumer loads:
// accumulator-layout registers (column lane%16, rows 4*(lane/16)..+3) packed to bf16, hi pair then lo pair.
struct __attribute__((aligned(16))) Slot {
  // dy rows, [token][RS]: within a row, the 16-byte vector (j, g) at element 32j + 8g holds values 32j+4g..+3
  // followed by values 32j+16+4g..+3, the value order of the consumers' state tiles.  Rows the entering state does
  // not reach are zero.
  uint16_t DY[CK][RS];
  uint4 KT[4][64];             // (k_s/E_s)^T per key tile: hi,lo, lane-indexed
  uint2 Vt[4][64];             // v^T per value tile, lane-indexed; tokens masked for the chunk-end state
  uint4 Nt[64];                // Gram tile v_s.dy_t (s < t): hi pair, lo pair, lane-indexed (A operand row t, k-slots s)
  float Ee[CK][ES];            // decay from the chunk start to just before token t, per key
  float UKC[CK][ES];           // u k_t c_t per key
  uint16_t R[CK][RS];          // r rows (bf16, natural key order)
  float gamma[64];             // E at the chunk end
  int snap;                    // -1, or the in-chunk index of token length-1
  int keep_end;                // the entering state survives to the chunk end (no reset in the chunk)
  int keep_snap;               // the entering state survives to token length-1
  int pad;
};
struct __attribute__((aligned(16))) SnapSlot {
  uint2 Vt[4][64];             // v^T with the tokens masked for the state at token length-1
  float gamma[64];
};
struct __attribute__((aligned(16))) Tail {
  float du[NPROD][64];         // per-producer partial sums of du
};

// ---------------------------------------------------------------------------------------------------- producer
struct Raw {
  uint4 r[2], k[2], v[2], w[2], dy[2];
};

__device__ __forceinline__ void load_raw(Raw& x, const Wkv6Args& A, int64_t b, int64_t h, int64_t c0, int lane) {
  const int t = lane & 15, g = lane >> 4;
  if (c0 + t < A.T) {
    const size_t off = ((((size_t)b * A.T + c0 + t) * A.H + h) * 64 + 8 * g) * 2;  // bytes
    auto ld = [&](const void* p, uint4 (&o)[2]) {
      o[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off);
      o[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(p) + off + 64);
    };
    ld(A.r, x.r); ld(A.k, x.k); ld(A.v, x.v); ld(A.gy, x.dy);
    // a decay shared by all tokens (RWKV-5) is one (H,64) row per head
    const size_t woff = (A.flags & FLAG_W_PER_HEAD) ? ((size_t)h * 64 + 8 * g) * 2 : off;
    x.w[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff);
    x.w[1] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.w) + woff + 64);
  } else {
    const uint4 z = make_uint4(0, 0, 0, 0);
    x.r[0] = x.r[1] = x.k[0] = x.k[1] = x.v[0] = x.v[1] = x.w[0] = x.w[1] = x.dy[0] = x.dy[1] = z;
  }
}

struct Producer {
  int lane;
  u32x4_t sel[2];     // MFMA-as-transposer selection operands
  uint4 u[2];         // bonus of this lane's keys (bf16)
  float du[16];       // running sum over this producer's tokens of r k c_t, for this lane's token and keys
};

__device__ __forceinline__ void produce(Producer& P, const Raw& x, const ChunkFlags& F, Slot* __restrict__ slot,
                                        SnapSlot* __restrict__ snap, unsigned* events) {
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

  f32x4_t N = zero4;   // [row s][column t] = v_s . dy_t
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    // ================= keys of this half: decay scan, (k/E)^T, Ee rows, r rows
    {
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
        cap_chunk_decay(E, lane, events);
      }
      if (slow) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float base = __shfl(E[e], seg_src, 64);   // restart the cumulative decay at the last reset
          if (restart) E[e] -= base;
        }
      }
      u32x4_t kh_h, kh_l;
      float Ee[8];
      {
        float fk[8], Einv[8];
        unpack8(x.k[hf], fk);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l2 = fmaxf(E[e], MIN_CUM_L2);
          E[e] = exp2_fast(l2);
          Einv[e] = exp2_fast(-l2);
          // value of the previous token; 1 for the first token.  At a reset token it belongs to the previous
          // segment, but it then multiplies an exact zero (no state reaches that token).
          Ee[e] = row_prev(E[e], 1.0f);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = 2 * j;
          uint32_t hi, lo;
          split2(fk[e] * Einv[e], fk[e + 1] * Einv[e + 1], hi, lo); kh_h[j] = hi; kh_l[j] = lo;
        }
      }
      {
        float* er = &slot->Ee[t][32 * hf + 8 * g];
        *reinterpret_cast<float4*>(er) = make_float4(Ee[0], Ee[1], Ee[2], Ee[3]);
        *reinterpret_cast<float4*>(er + 4) = make_float4(Ee[4], Ee[5], Ee[6], Ee[7]);
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
      *reinterpret_cast<uint4*>(&slot->R[t][32 * hf + 8 * g]) = x.r[hf];
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const u32x4_t sel = P.sel[x2];
        const uint2 dh = plain_pack(mfma(kh_h, sel, zero4)), dl = plain_pack(mfma(kh_l, sel, zero4));
        slot->KT[2 * hf + x2][lane] = make_uint4(dh.x, dh.y, dl.x, dl.y);
      }
    }
    // ================= values of this half: v^T, dy rows, partial Gram sum
    {
      const uint4 vr = x.v[hf], dr = x.dy[hf];
      const u32x4_t vop = {vr.x, vr.y, vr.z, vr.w}, dyop = {dr.x, dr.y, dr.z, dr.w};
      const int e0 = 32 * hf + 16 * (g & 1) + 4 * (g >> 1);     // first 8-byte piece of this lane in a permuted row
      uint16_t* row = slot->DY[t];
      *reinterpret_cast<uint2*>(row + e0) = s0_reaches ? make_uint2(dyop[0], dyop[1]) : make_uint2(0u, 0u);
      *reinterpret_cast<uint2*>(row + e0 + 8) = s0_reaches ? make_uint2(dyop[2], dyop[3]) : make_uint2(0u, 0u);
#pragma unroll
      for (int x2 = 0; x2 < 2; ++x2) {
        const int tile = 2 * hf + x2;
        const f32x4_t dv = mfma(vop, P.sel[x2], zero4);
        slot->Vt[tile][lane] = keep_upd == 0xffffu ? plain_pack(dv) : masked_pack(dv, keep_upd);
        if (F.snap >= 0) snap->Vt[tile][lane] = masked_pack(dv, keep_snap);
      }
      N = mfma(vop, dyop, N);
    }
  }
  // ---- c_t = v_t.dy_t is the diagonal of N: held by lane group t/4, register t%4; hand it to all four groups
  const int n = t;
  float c_t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) c_t = (4 * g + i == n) ? N[i] : c_t;
  c_t += __shfl_xor(c_t, 16, 64);
  c_t += __shfl_xor(c_t, 32, 64);
  // ---- u k c_t for the consumers, r k c_t for du
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    float fr[8], fk[8], fu[8], o[8];
    unpack8(x.r[hf], fr); unpack8(x.k[hf], fk); unpack8(P.u[hf], fu);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float kc = fk[e] * c_t;
      o[e] = fu[e] * kc;
      P.du[8 * hf + e] = fmaf(fr[e], kc, P.du[8 * hf + e]);
    }
    float* up = &slot->UKC[t][32 * hf + 8 * g];
    *reinterpret_cast<float4*>(up) = make_float4(o[0], o[1], o[2], o[3]);
    *reinterpret_cast<float4*>(up + 4) = make_float4(o[4], o[5], o[6], o[7]);
  }
  // ---- strictly lower triangle within a segment
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = 4 * g + i;
    bool lt = m < n;
    if (slow) lt = lt && seg_of(resets, m) == seg_of(resets, n);
    N[i] = lt ? N[i] : 0.f;
  }
  uint32_t hi0, lo0, hi1, lo1;
  split2(N[0], N[1], hi0, lo0);
  split2(N[2], N[3], hi1, lo1);
  slot->Nt[lane] = make_uint4(hi0, hi1, lo0, lo1);
  if (lane == 0) {
    slot->snap = F.snap;
    slot->keep_end = (lastseg == 0) ? 1 : 0;
    slot->keep_snap = (F.snap >= 0 && (!slow || seg_of(resets, F.snap) == 0)) ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------------------------------- consumer
// Wave q holds the state rows of keys 16q..16q+15 as four 16x16 accumulator tiles: lane (n = lane%16, g = lane/16),
// S[vt][i] = S[key 16q + n][value 16*vt + 4g + i].
struct Consumer {
  f32x4_t S[4];
  int q, lane;
};

struct OutCursor {
  char *gr;            // bf16 output at (b, c0, h, 0)
  char *er;            // fp32 workspace at the same place
  size_t tok_bytes;    // bytes between consecutive tokens in gr (twice that in er)
  uint32_t voff;       // lane part of the address, in elements: (4g * H) * 64 + key
};

__device__ __forceinline__ size_t state_el(const Wkv6Args& A, int64_t b, int64_t h, int key, int value) {
  return (((size_t)b * A.H + h) * 64 + key) * 64 + value;
}
__device__ __forceinline__ f32x4_t load_state4(const void* p, int f32, size_t off) {
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

__device__ __forceinline__ void consume(Consumer& C, const Slot* __restrict__ slot, const SnapSlot* __restrict__ snapslot,
                                        const Wkv6Args& A, int64_t b, int64_t h, int nvalid, bool is_snap, OutCursor& oc) {
  const int lane = C.lane, n = lane & 15, g = lane >> 4, q = C.q;
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  // B operands of the token contractions: k/E of tokens 4g..4g+3 at this wave's keys, hi and lo side by side
  const u32x4_t kt = *reinterpret_cast<const u32x4_t*>(&slot->KT[q][lane]);
  const bool keep_end = slot->keep_end != 0;
  u32x4_t Sh[2], Sl[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    uint32_t hi, lo;
    split2_keep(C.S[2 * j][0], C.S[2 * j][1], hi, lo); Sh[j][0] = hi; Sl[j][0] = lo;
    split2_keep(C.S[2 * j][2], C.S[2 * j][3], hi, lo); Sh[j][1] = hi; Sl[j][1] = lo;
    split2_keep(C.S[2 * j + 1][0], C.S[2 * j + 1][1], hi, lo); Sh[j][2] = hi; Sl[j][2] = lo;
    split2_keep(C.S[2 * j + 1][2], C.S[2 * j + 1][3], hi, lo); Sh[j][3] = hi; Sl[j][3] = lo;
  }
  f32x4_t P = zero4, P2 = zero4;   // [token 4g+i][key n]
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const u32x4_t dy = *reinterpret_cast<const u32x4_t*>(&slot->DY[n][32 * j + 8 * g]);
    P = mfma(dy, Sh[j], P);
    P2 = mfma(dy, Sl[j], P2);
  }
  {
    const u32x4_t nt = *reinterpret_cast<const u32x4_t*>(&slot->Nt[lane]);
    const u32x4_t nhh = {nt[0], nt[1], nt[0], nt[1]}, nl0 = {nt[2], nt[3], 0u, 0u};
    P = mfma(nhh, kt, P);                            // N_hi (kh_hi + kh_lo)
    const u32x4_t kh0 = {kt[0], kt[1], 0u, 0u};
    P2 = mfma(nl0, kh0, P2);                         // N_lo kh_hi
  }
  // A operands of the state update: rows = values of tile vt, k-slots = v of tokens 4g..4g+3, twice
  u32x4_t A1[4];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    const uint2 vv = slot->Vt[vt][lane];
    A1[vt] = u32x4_t{vv.x, vv.y, vv.x, vv.y};
  }
  // rowsum(dS_out * S_{length-1}) per key (one chunk per sequence)
  if (is_snap) {
    const bool keep = slot->keep_snap != 0;
    const float sg = snapslot->gamma[16 * q + n];
    float p = 0.f;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) {
      const uint2 vv = snapslot->Vt[vt][lane];
      const u32x4_t S1 = {vv.x, vv.y, vv.x, vv.y};
      const f32x4_t acc = mfma(S1, kt, keep ? C.S[vt] : zero4);
      const f32x4_t gs = load_state4(A.gs_out, A.st_f32, state_el(A, b, h, 16 * q + n, 16 * vt + 4 * g));
#pragma unroll
      for (int i = 0; i < 4; ++i) p = fmaf(gs[i], acc[i] * sg, p);
    }
    p += __shfl_xor(p, 16, 64);
    p += __shfl_xor(p, 32, 64);
    if (g == 0) A.eI[((size_t)b * A.H + h) * 64 + 16 * q + n] = p;
  }
  // state update: S <- diag(gamma) (S + Kh^T V), gamma per key = per lane
  if (!keep_end) {
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = zero4;   // a reset inside the chunk cuts the entering state off
  }
  const float gm = slot->gamma[16 * q + n];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt) {
    f32x4_t acc = mfma(A1[vt], kt, C.S[vt]);
    acc[0] *= gm; acc[1] *= gm; acc[2] *= gm; acc[3] *= gm;
    C.S[vt] = acc;
  }
  // outputs: register i is token 4g+i, lanes n = 16 consecutive keys
  const size_t lo = (size_t)oc.voff;
  auto put = [&](int i, bool full) {
    const int tok = 4 * g + i;
    const float sdy = (P[i] + P2[i]) * slot->Ee[tok][16 * q + n];
    const float rr = bf16_to_f32(slot->R[tok][16 * q + n]);
    const float ukc = slot->UKC[tok][16 * q + n];
    if (full || tok < nvalid) {
      *reinterpret_cast<uint16_t*>(oc.gr + lo * 2 + i * oc.tok_bytes) = f32_to_bf16(ukc + sdy);
      *reinterpret_cast<float*>(oc.er + lo * 4 + 2 * i * oc.tok_bytes) = rr * sdy;
    }
  };
  if (nvalid == CK) {      // every chunk but a partial last one: no per-lane predicates
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, true);
  } else {
    rare_path();
#pragma unroll
    for (int i = 0; i < 4; ++i) put(i, false);
  }
  oc.gr += CK * oc.tok_bytes;
  oc.er += 2 * CK * oc.tok_bytes;
}

}  // namespace

__global__ __launch_bounds__(64 * (NCONS + NPROD)) void wkv6_chunk_bwd_f_kernel(Wkv6Args A) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Slot* slots = reinterpret_cast<Slot*>(smem_raw);
  SnapSlot* snapslot = reinterpret_cast<SnapSlot*>(smem_raw + RING * sizeof(Slot));
  Tail* tail = reinterpret_cast<Tail*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot));
  Sync* sy = reinterpret_cast<Sync*>(smem_raw + RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Tail));
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
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt) C.S[vt] = load_state4(A.s, A.st_f32, state_el(A, b, h, 16 * wave + n, 16 * vt + 4 * g));
    OutCursor oc;
    oc.tok_bytes = (size_t)A.H * 64 * 2;
    const size_t el0 = (((size_t)b * A.T) * A.H + h) * 64;
    oc.gr = reinterpret_cast<char*>(A.gr) + el0 * 2;
    oc.er = reinterpret_cast<char*>(A.er) + el0 * 4;
    oc.voff = (uint32_t)((4 * g) * (int)A.H * 64 + 16 * wave + n);
    const int csnap = (L >= 1 && inject) ? (int)((L - 1) / CK) : -1;
    for (int c = 0; c < nch; ++c) {
      const int nvalid = (c + 1 < nch || A.T % CK == 0) ? CK : (int)(A.T % CK);
      const int si = c % RING;
      if (!wait_ready(sy, si, c + 1)) break;
      consume(C, &slots[si], snapslot, A, b, h, nvalid, c == csnap, oc);
      if (lane == 0) __hip_atomic_store(&sy->consumed[wave][si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  } else {
    const int p = wave - NCONS;
    Producer P;
    P.lane = lane;
    make_sel(P.sel, lane);
    {
      const char* up = reinterpret_cast<const char*>(A.u) + ((size_t)h * 64 + 8 * (lane >> 4)) * 2;
      P.u[0] = *reinterpret_cast<const uint4*>(up);
      P.u[1] = *reinterpret_cast<const uint4*>(up + 64);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) P.du[e] = 0.f;
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
      if (lane == 0) __hip_atomic_store(&sy->ready[si], c + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    retire_loads(raw, ns_mine);
    // du of this producer's tokens: sum over the 16 token lanes of a row, one writer per key
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float s = row_scan(P.du[e]);                 // lane 15 of each row holds the row total
      if ((lane & 15) == 15) tail->du[p][32 * (e >> 3) + 8 * (lane >> 4) + (e & 7)] = s;
    }
  }
  __syncthreads();   // every wave gets here: all loops above are bounded
  if (threadIdx.x < 64) {
    float s = 0.f;
#pragma unroll
    for (int p = 0; p < NPROD; ++p) s += tail->du[p][threadIdx.x];
    A.gu[((size_t)b * A.H + h) * 64 + threadIdx.x] = s;
  }
  if (head_broken(sy, A.status)) {
    poison_token_rows(A.gr, 2, b, h, A.T, A.H);
    poison_token_rows(A.er, 4, b, h, A.T, A.H);
    if (threadIdx.x < 64) A.gu[((size_t)b * A.H + h) * 64 + threadIdx.x] = __uint_as_float(0x7fc00000u);
  }
}

hipError_t launch_wkv6_chunk_bwd_f(const Wkv6Args& A, hipStream_t stream) {
  const size_t smem = RING * sizeof(Slot) + sizeof(SnapSlot) + sizeof(Tail) + sizeof(Sync);
  static LdsAttrOnce once;
  const hipError_t attr = allow_dynamic_lds(once, reinterpret_cast<const void*>(wkv6_chunk_bwd_f_kernel), smem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(wkv6_chunk_bwd_f_kernel, dim3((unsigned)(A.B * A.H)), dim3(64 * (NCONS + NPROD)), smem, stream, A);
  return hipGetLastError();
}

}  // namespace hiprwkv
