// Skeleton shared by the sequential (one token per step, fp32 VALU) matrix-state kernels.
//
// One workgroup of 256 threads owns one (sequence, head).  The 64x64 state is
// spread as 16 contiguous elements per thread: thread tid owns line `tid>>2`
// (a row or a column of the state, the kernel decides) and the 16-element
// quarter `tid&3` of it, so a dot product along a line is 16 FMAs plus a
// quad reduction.  Token vectors are streamed from HBM in stages of CH steps:
// each thread fetches 8 consecutive elements of every input with one 16-byte
// (bf16) or two 16-byte (fp32) loads, the stage is parked in LDS as fp32
// (decay transforms applied once there), the next stage's loads are issued
// before the CH dependent steps run, and per-token results are collected in
// LDS and written back with the same coalesced 8-element pattern.
#pragma once
#include "common.h"

namespace hiprwkv {

constexpr int N64 = 64;
constexpr int SEQ_THREADS = 256;

enum VecKind : int {
  VK_ID = 0,        // x
  VK_EXPNEGEXP = 1, // exp(-exp(x))   WKV7 decay (rwkv7.py:201)
  VK_EXP = 2,       // exp(x)         WKV6 decay (rwkv6.py:176)
  VK_NEGEXP = 3,    // -exp(x)        d(log decay)/dw of WKV7
};

struct VecIn {
  const void* p;  // (B,T,H,64)
  int f32;        // element type: 1 = float, 0 = bf16, 2 = IEEE half
  int kind;       // VecKind
  int per_head;   // 1: p is (H,64), the same vector for every token and sequence
};
struct VecOut {
  void* p;  // may be null: result discarded
  int f32;
};

__device__ __forceinline__ void ld8_any(const VecIn& v, size_t off, float (&o)[8]) {
  if (v.f32 == 1) ld8(reinterpret_cast<const float*>(v.p) + off, o);
  else if (v.f32 == 2) ld8(reinterpret_cast<const _Float16*>(v.p) + off, o);
  else ld8(reinterpret_cast<const bf16_t*>(v.p) + off, o);
}
__device__ __forceinline__ void st8_any(const VecOut& v, size_t off, const float (&o)[8]) {
  if (v.f32 == 1) st8(reinterpret_cast<float*>(v.p) + off, o);
  else if (v.f32 == 2) st8(reinterpret_cast<_Float16*>(v.p) + off, o);
  else st8(reinterpret_cast<bf16_t*>(v.p) + off, o);
}
__device__ __forceinline__ float vec_transform(int kind, float x) {
  switch (kind) {
    case VK_EXPNEGEXP: return expf(-expf(x));
    case VK_EXP: return expf(x);
    case VK_NEGEXP: return -expf(x);
    default: return x;
  }
}

template <int NIN, int NOUT, int CH>
constexpr size_t seq_smem_bytes() {
  return (size_t)(NIN + NOUT) * CH * N64 * sizeof(float) + 128;
}

// Step must provide:
//   void step(int tl, int64_t t, float (*sin)[CH][64], float (*sout)[CH][64], const uint8_t* sns)
//       sns[x] = new_starts[t0 + x] for x in [0, CH], 0 beyond T
//   void post(int o, int tl, int64_t t, float (&vals)[8], const uint8_t* sns)   (per-output fix-up)
template <int NIN, int NOUT, int CH, bool REV, class Step>
__device__ __forceinline__ void seq_run(Step& st, const VecIn* in, const VecOut* out, int64_t b, int64_t h,
                                        int64_t T, int64_t H, const uint8_t* ns_row, float* smem) {
  static_assert(CH * N64 == SEQ_THREADS * 8 || CH * N64 == SEQ_THREADS * 4, "CH must be 32 or 16");
  constexpr int EPT = CH * N64 / SEQ_THREADS;  // elements per thread per vector: 8 or 4
  constexpr int LPS = N64 / 8;                  // 8-element groups per step
  float(*sin)[CH][N64] = reinterpret_cast<float(*)[CH][N64]>(smem);
  float(*sout)[CH][N64] = reinterpret_cast<float(*)[CH][N64]>(smem + (size_t)NIN * CH * N64);
  // new_starts flags of the stage, double-buffered: the write-back of stage s reads them while
  // stage s+1 is already being parked
  uint8_t* sns_base = reinterpret_cast<uint8_t*>(smem + (size_t)(NIN + NOUT) * CH * N64);
  const int tid = threadIdx.x;
  // with EPT == 4 only the even threads move data (8 elements each)
  const bool mover = (EPT == 8) || ((tid & 1) == 0);
  const int slot = (EPT == 8) ? tid : (tid >> 1);
  const int tt = slot / LPS, col = (slot % LPS) * 8;
  const int64_t nst = (T + CH - 1) / CH;
  float pre[NIN][8];

  auto gload = [&](int64_t stage) {
    const int64_t t = stage * CH + tt;
    if (mover && t < T) {
      const size_t off = (((size_t)b * T + t) * H + h) * N64 + col;
#pragma unroll
      for (int x = 0; x < NIN; ++x) ld8_any(in[x], in[x].per_head ? (size_t)h * N64 + col : off, pre[x]);
    } else {
#pragma unroll
      for (int x = 0; x < NIN; ++x)
#pragma unroll
        for (int e = 0; e < 8; ++e) pre[x][e] = 0.f;
    }
  };

  gload(REV ? nst - 1 : 0);
  for (int64_t s = 0; s < nst; ++s) {
    const int64_t stage = REV ? nst - 1 - s : s;
    const int64_t t0 = stage * CH;
    const int nvalid = (int)((T - t0 < CH) ? (T - t0) : CH);
    uint8_t* sns = sns_base + (s & 1) * 64;
    if (mover) {
#pragma unroll
      for (int x = 0; x < NIN; ++x) {
        float4 lo, hi;
        const int kd = in[x].kind;
        lo.x = vec_transform(kd, pre[x][0]); lo.y = vec_transform(kd, pre[x][1]);
        lo.z = vec_transform(kd, pre[x][2]); lo.w = vec_transform(kd, pre[x][3]);
        hi.x = vec_transform(kd, pre[x][4]); hi.y = vec_transform(kd, pre[x][5]);
        hi.z = vec_transform(kd, pre[x][6]); hi.w = vec_transform(kd, pre[x][7]);
        *reinterpret_cast<float4*>(&sin[x][tt][col]) = lo;
        *reinterpret_cast<float4*>(&sin[x][tt][col + 4]) = hi;
      }
    }
    if (tid <= CH) sns[tid] = (ns_row != nullptr && t0 + tid < T) ? ns_row[t0 + tid] : (uint8_t)0;
    __syncthreads();
    if (s + 1 < nst) gload(REV ? stage - 1 : stage + 1);
    if (REV) {
      for (int tl = nvalid - 1; tl >= 0; --tl) st.step(tl, t0 + tl, sin, sout, sns);
    } else {
      for (int tl = 0; tl < nvalid; ++tl) st.step(tl, t0 + tl, sin, sout, sns);
    }
    __syncthreads();
    if (mover && tt < nvalid) {
      const size_t off = (((size_t)b * T + t0 + tt) * H + h) * N64 + col;
#pragma unroll
      for (int o = 0; o < NOUT; ++o) {
        if (out[o].p == nullptr) continue;
        float vals[8];
        float4 lo = *reinterpret_cast<const float4*>(&sout[o][tt][col]);
        float4 hi = *reinterpret_cast<const float4*>(&sout[o][tt][col + 4]);
        vals[0] = lo.x; vals[1] = lo.y; vals[2] = lo.z; vals[3] = lo.w;
        vals[4] = hi.x; vals[5] = hi.y; vals[6] = hi.z; vals[7] = hi.w;
        st.post(o, tt, t0 + tt, vals, sns);
        st8_any(out[o], off, vals);
      }
    }
  }
}

// 16 consecutive floats of an LDS row into registers (4 x ds_read_b128)
__device__ __forceinline__ void lds16(const float* p, float (&o)[16]) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    float4 x = *reinterpret_cast<const float4*>(p + 4 * g);
    o[4 * g] = x.x; o[4 * g + 1] = x.y; o[4 * g + 2] = x.z; o[4 * g + 3] = x.w;
  }
}

}  // namespace hiprwkv
