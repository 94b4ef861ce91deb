// Building blocks shared by the chunked MFMA kernels (gfx950): bf16 hi/lo operand splitting, the 16x16x32 bf16
// MFMA wrapper, DPP helpers for the in-chunk decay scan, per-chunk reset/length facts, and the LDS hand-shake
// between producer and consumer waves.
#pragma once
#include "common.h"

namespace hiprwkv {
namespace chunk {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int CK = 16;            // tokens per chunk
constexpr int RS = 72;            // row stride (bf16 elements) of the [token][64] LDS arrays: 144 B (16-byte aligned rows)
constexpr int NCONS = 4;          // consumer waves, one per 16 value rows (the WKV6 reverse sweep has eight)
constexpr int SPIN_LIMIT = 1 << 16;   // polls before a waiter gives up (milliseconds; a healthy wait is microseconds)
constexpr float LOG2E = 1.44269504088896340736f;
constexpr float MIN_STEP_L2 = -1.0e4f;          // keeps the running sum finite
constexpr float MIN_CUM_L2 = -80.0f * LOG2E;    // floor of a chunk's total log2 decay: 2^MIN_CUM_L2 = e^-80

// Hand-shake words.  ready[s] = c + 1 once chunk c is complete in slot s; consumed[q][s] = c + 1 once consumer
// q no longer reads chunk c in slot s.  Waiting is a bounded poll, so that a broken hand-shake cannot hang the GPU:
// a waiter that gives up sets `broken` and returns false, its wave leaves its chunk loop, and after the
// workgroup's final barrier every output of that (sequence, head) is overwritten with NaN and the library's
// failure counter is incremented (finish_head below), so no launch returns stale data unnoticed.
constexpr int MAX_RING = 16;      // most slots a ring may have
template <int NC>                 // NC = number of consumer waves
struct __attribute__((aligned(16))) SyncN {
  int ready[MAX_RING];
  int consumed[NC][MAX_RING];
  int broken;
  int pad[3];
};
using Sync = SyncN<NCONS>;

template <int NC>
__device__ __forceinline__ bool wait_ready(SyncN<NC>* sy, int slot, int want) {
  for (int spin = 0; spin < SPIN_LIMIT; ++spin) {
    if (__hip_atomic_load(&sy->ready[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == want) return true;
    __builtin_amdgcn_s_sleep(1);
  }
  __hip_atomic_store(&sy->broken, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  return false;
}
template <int NC>
__device__ __forceinline__ bool wait_consumed(SyncN<NC>* sy, int slot, int want, int lane) {
  for (int spin = 0; spin < SPIN_LIMIT; ++spin) {
    int seen = want;
    if (lane < NC) seen = __hip_atomic_load(&sy->consumed[lane][slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (__ballot(seen < want) == 0ull) return true;
    __builtin_amdgcn_s_sleep(1);
  }
  __hip_atomic_store(&sy->broken, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  return false;
}

// The same two waits for kernels whose producers run far ahead of the consumers.  A producer that finds its slot
// still in use sleeps for hundreds of cycles between polls (every poll costs vector instructions that compete with
// the consumer on the same SIMD); a consumer tests a flag value that it requested earlier in the chunk, so that the
// LDS round trip is off its critical path, and only polls if that value was not the wanted one yet.
template <int NC>
__device__ __forceinline__ bool wait_consumed_lazy(SyncN<NC>* sy, int slot, int want, int lane) {
  for (int spin = 0; spin < SPIN_LIMIT / 8; ++spin) {
    int seen = want;
    if (lane < NC) seen = __hip_atomic_load(&sy->consumed[lane][slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (__ballot(seen < want) == 0ull) return true;
    __builtin_amdgcn_s_sleep(8);
  }
  __hip_atomic_store(&sy->broken, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  return false;
}
template <int NC>
__device__ __forceinline__ int peek_ready(const SyncN<NC>* sy, int slot) {
  return __hip_atomic_load(&sy->ready[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
template <int NC>
__device__ __forceinline__ bool wait_ready_peeked(SyncN<NC>* sy, int slot, int want, int peeked) {
  if (__builtin_amdgcn_readfirstlane(peeked) == want) {
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return true;
  }
  return wait_ready(sy, slot, want);
}

// Buffer addressing for the consumers' per-token scalars (2- and 4-byte accesses at (token 4g+i, element 16q+n)): a
// descriptor on the uniform base of the chunk (scalar registers), the lane's byte offset in one vector register and
// the token's offset as a scalar operand, so that no access costs vector address arithmetic or a register pair.
// Measured on the same box: it takes 2 % off the WKV7 reverse sweep C (16 loads and 12 stores per consumer and chunk)
// and is used there only: with it the sweeps whose consumers just store were no faster (WKV6) or 1.5-2.7 % slower
// (WKV7 sweeps A and B).
using rsrc_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}

// Test hook (HIPRWKV_DEBUG_DROP_PUBLISH): the producer of the last step does not publish it, so that the consumers'
// bounded wait runs out while every wave still ends normally.
constexpr unsigned FLAG_DROP_PUBLISH = 0x100u;

// NaN into this head's rows of a (B,T,H,64) tensor; elem = bytes per element (2: bf16, 4: fp32)
__device__ __forceinline__ void poison_token_rows(void* base, int elem, int64_t b, int64_t h, int64_t T, int64_t H) {
  if (base == nullptr) return;
  const int pieces = 64 * elem / 16;
  const uint32_t nan = elem == 2 ? 0x7fc07fc0u : 0x7fc00000u;
  for (int64_t i = threadIdx.x; i < T * pieces; i += blockDim.x) {
    const int64_t t = i / pieces;
    const int pc = (int)(i % pieces);
    char* p = static_cast<char*>(base) + ((((size_t)b * T + t) * H + h) * 64) * elem + 16 * pc;
    *reinterpret_cast<uint4*>(p) = make_uint4(nan, nan, nan, nan);
  }
}
// NaN into this head's 64x64 block of a (B,H,64,64) state tensor
__device__ __forceinline__ void poison_state(void* base, int f32, int64_t b, int64_t h, int64_t H) {
  if (base == nullptr) return;
  const int elem = f32 ? 4 : 2;
  const uint32_t nan = f32 ? 0x7fc00000u : 0x7fc07fc0u;
  char* p = static_cast<char*>(base) + (((size_t)b * H + h) * 4096) * elem;
  for (int i = threadIdx.x; i < 4096 * elem / 16; i += blockDim.x)
    reinterpret_cast<uint4*>(p)[i] = make_uint4(nan, nan, nan, nan);
}
// After the workgroup's final barrier: did any waiter of this workgroup give up?
template <int NC>
__device__ __forceinline__ bool head_broken(const SyncN<NC>* sy, unsigned* status) {
  const bool broken = __hip_atomic_load(&sy->broken, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0;
  if (broken && threadIdx.x == 0 && status != nullptr) atomicAdd(status, 1u);
  return broken;
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
  hi = __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);
  // x - hi in one v_dot2c_f32_bf16 each: acc += hi.lo * -1 + hi.hi * 0  (resp. 0, -1)
  // The two selectors are kept out of the compiler's sight: written as immediates, (-1, 0) would be encoded as
  // the 16-bit inline constant -1.0, whose bit pattern is the fp16 one.  The asm statements are not volatile, so
  // that the selectors are materialised once per kernel, not once per call.
  const bf16x2_t hp = __builtin_bit_cast(bf16x2_t, hi);
  uint32_t m10 = 0x0000bf80u, m01 = 0xbf800000u;
  asm("" : "+s"(m10));
  asm("" : "+s"(m01));
  const float l0 = __builtin_amdgcn_fdot2_f32_bf16(hp, __builtin_bit_cast(bf16x2_t, m10), x0, false);
  const float l1 = __builtin_amdgcn_fdot2_f32_bf16(hp, __builtin_bit_cast(bf16x2_t, m01), x1, false);
  lo = pack_rn(l0, l1);
}

// The same split for sources that stay live afterwards (accumulator registers): mask and subtract run at the full
// VALU rate and leave the source alone, where v_dot2c_f32_bf16 (half rate) accumulates in place and would need a
// register copy first.
__device__ __forceinline__ void split2_keep(float x0, float x1, uint32_t& hi, uint32_t& lo) {
  const uint32_t u0 = __float_as_uint(x0), u1 = __float_as_uint(x1);
  hi = __builtin_amdgcn_perm(u1, u0, 0x07060302u);
  const float l0 = x0 - __uint_as_float(u0 & 0xffff0000u);
  const float l1 = x1 - __uint_as_float(u1 & 0xffff0000u);
  lo = pack_rn(l0, l1);
}

// Keeps two matrix instructions of DIFFERENT opcodes apart when the second one accumulates on the first one's
// result.  Measured on gfx950 with hipcc 7.2: v_mfma_f32_16x16x32_f16 D followed by v_mfma_f32_16x16x16_f16 D, A, B, D
// reads a stale D in the first quarter of the wave (register 0 of lanes 0-15) when three or four other instructions
// sit between the two, and the right one from five on; the compiler's hazard recogniser adds no wait states there
// (it does for every other pairing the library has: same opcode, or a different destination).  Which distance a
// build gets depends on instruction scheduling, so unrelated source changes switched the error on and off.  The
// eight wait states here are the distance the compiler itself keeps between a matrix instruction and an ordinary
// vector instruction that reads its result.  The asm takes the accumulator as an in/out operand, which pins it
// between the two matrix instructions.  tests/test_mfma_hazard.py checks the distance in the compiled code of every
// kernel.
__device__ __forceinline__ void mfma_shape_fence(f32x4_t& acc) { asm volatile("s_nop 7" : "+v"(acc)); }

// Last statement of the producers' branch of a kernel: "uses" every register that the producers load into from global
// memory.  Both roles live in one function, and after the compiler has arranged the control flow the consumers' code
// is, on paper, reachable from the end of the producers'.  Its pass that places the waits for memory operations then
// believes that the registers of the producers' last loads may still be awaited when the consumers' code runs, and
// guards their first reuse there -- inside the consumers' main loop -- with a full `s_waitcnt vmcnt(0)`, which at run
// time waits for the consumer wave's own recent stores and loads in every step (seen in the reverse sweep C of the
// WKV7 backward pass: a memory round trip per chunk on the critical path).  The empty asm statements make the
// compiler wait for those loads here, where nothing is in flight any more, which clears that state.  (A
// `__builtin_amdgcn_s_waitcnt` at the start of the consumers' branch does not do it: the pass removes it.)
template <class R>
__device__ __forceinline__ void retire_loads(const R& x, uint32_t flag_byte) {
  constexpr int N = sizeof(R) / 4;
  struct Words { uint32_t w[N]; };
  const Words v = __builtin_bit_cast(Words, x);
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" ::"v"(v.w[i]));
  asm volatile("" ::"v"(flag_byte));
}

// First statement of a rarely taken, wave-uniform branch (resets inside a chunk, the partial last chunk, the chunk
// of token length-1): keeps the compiler from turning the branch into selects that every chunk would execute.
__device__ __forceinline__ void rare_path() { asm volatile("" ::: "memory"); }

template <int CTRL>
__device__ __forceinline__ float dpp0(float x) {  // lanes without a source read 0
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// inclusive sum over the 16 lanes of a DPP row
__device__ __forceinline__ float row_scan(float x) {
  x += dpp0<0x111>(x);
  x += dpp0<0x112>(x);
  x += dpp0<0x114>(x);
  x += dpp0<0x118>(x);
  return x;
}
// E: inclusive running sums (log2 decay, <= 0, non-increasing along the row) of 8 channels over the 16 token lanes.
// A channel whose total over the chunk is below MIN_CUM_L2 has all its steps of this chunk scaled by the same
// factor so that the total becomes MIN_CUM_L2: 1/E stays finite in fp32 and the relative weights inside the chunk
// keep their order, at the price of an inexact (weaker) decay for that channel in that chunk.  Every wave that caps
// a channel adds one to the library's numeric-event counter (`events`, may be null), so the inexact result does not
// pass unnoticed.
__device__ __forceinline__ void cap_chunk_decay(float (&E)[8], int lane, unsigned* events) {
  // one comparison of the smallest of the eight sums instead of eight
  const float lo = fminf(fminf(fminf(E[0], E[1]), fminf(E[2], E[3])), fminf(fminf(E[4], E[5]), fminf(E[6], E[7])));
  if (__ballot(lo < MIN_CUM_L2) != 0ull) {
    rare_path();
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float tot = __shfl(E[e], (lane & 48) | 15, 64);
      if (tot < MIN_CUM_L2) E[e] *= MIN_CUM_L2 / tot;
    }
    if (lane == 0 && events != nullptr) atomicAdd(events, 1u);
  }
}
// The numeric-event word sits right behind the hand-shake failure word (api.hip: g_status_words).
__device__ __forceinline__ unsigned* events_word(unsigned* status) { return status != nullptr ? status + 1 : nullptr; }
// Non-finite values in a carried 64x64 state (an fp16 operand overflowed: |state|, |sa|, |v| or a scaled input beyond
// 65504): one numeric event per wave that sees one.  Called once per consumer wave, after the last chunk.
__device__ __forceinline__ void count_nonfinite(const f32x4_t (&S)[4], int lane, unsigned* events) {
  float z = 0.f;
#pragma unroll
  for (int tile = 0; tile < 4; ++tile)
#pragma unroll
    for (int i = 0; i < 4; ++i) z = fmaf(S[tile][i], 0.f, z);      // 0 for finite values, NaN for an inf or a NaN
  if (__ballot(!(z == 0.f)) != 0ull && lane == 0 && events != nullptr) atomicAdd(events, 1u);
}

// value of the previous lane of the row; `first` in lane 0 of the row
__device__ __forceinline__ float row_prev(float x, float first) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(first), __float_as_int(x), 0x111, 0xf, 0xf, false));
}

__device__ __forceinline__ void unpack8(const uint4 p, float (&o)[8]) {
  const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// Per-chunk facts, identical in every lane.
struct ChunkFlags {
  uint32_t ns;      // bit t: new_starts[c0+t], bit 16: new_starts[c0+16] (0 beyond T)
  int nvalid;       // tokens of this chunk that exist
  int snap;         // in-chunk index of token length-1, or -1
  bool compat;
};

// number of resets at or before in-chunk token t: the index of its segment
__device__ __forceinline__ int seg_of(uint32_t ns, int t) { return __builtin_popcount(ns & ((2u << t) - 1u)); }

// Lanes 0..16 fetch one flag each (lanes beyond the chunk or the sequence re-read the last flag they may); the
// ballot in chunk_flags_of drops what does not belong to the chunk and makes the 17-bit mask uniform.  Only called
// with a non-null `ns`.
__device__ __forceinline__ uint32_t chunk_flag_fetch(const uint8_t* ns, int64_t T, int64_t b, int64_t c0, int lane) {
  const int64_t room = T - 1 - c0 < CK ? T - 1 - c0 : CK;          // c0 <= T - 1
  const int off = lane < (int)room ? lane : (int)room;
  return __builtin_amdgcn_raw_buffer_load_b8(
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ns + (size_t)b * T + c0), 0, 0x7fffffff, 0x00020000), off, 0, 0);
}
__device__ __forceinline__ ChunkFlags chunk_flags_of(const uint8_t* ns, uint32_t mine, unsigned flags, int64_t T,
                                                     int64_t c0, int64_t L) {
  ChunkFlags F;
  F.compat = (flags & 1u) != 0;
  F.nvalid = (int)((T - c0 < CK) ? (T - c0) : CK);
  F.snap = (L >= 1 && L - 1 >= c0 && L - 1 < c0 + CK) ? (int)(L - 1 - c0) : -1;
  const int have = (int)(T - c0 < CK + 1 ? T - c0 : CK + 1);       // flags c0 .. c0 + have - 1 exist
  F.ns = ns != nullptr ? (uint32_t)(__ballot(mine != 0) & ((1ull << have) - 1ull)) : 0u;
  return F;
}
// The producers fetch this byte one step ahead, before the operands of the same chunk (in that order: waiting for it
// then leaves the operand loads in flight); fetched at the top of the step it would cost every step a full memory
// round trip.  Without new_starts (a null pointer is legal) nothing is loaded: the branch is uniform, the pointer is a
// kernel argument.
__device__ __forceinline__ uint32_t chunk_flag_prefetch(const uint8_t* ns, int64_t T, int64_t b, int64_t c0, int lane) {
  return ns != nullptr ? chunk_flag_fetch(ns, T, b, c0, lane) : 0u;
}

// The fp32 workspace that the forward sweep of the WKV7 backward pass leaves for the reverse sweep after it (one value
// per token and key) is laid out for the waves that write and read it, not by token: per (sequence, head, chunk,
// consumer wave q) one record of 64 x 4 floats, lane (n, g) owning the four tokens 4g..4g+3 at key 16q + n.  Both
// sweeps hold their per-token results in exactly that register layout, so each lane moves its record entry with one
// 16-byte access (1 KiB contiguous per wave) instead of four scattered 4-byte ones.
constexpr int F_REC = 64 * 4;       // floats per record
__device__ __forceinline__ size_t f_record(int64_t b, int64_t h, int64_t H, int nch, int c, int q) {
  return ((((size_t)b * H + h) * nch + c) * NCONS + q) * F_REC;
}

// The WKV7 backward's workspace dsa (cotangent of sa, one value per token and value index) between the chunked bf16
// sweeps: 16-bit signed fixed point with one power-of-two scale per (sequence, head, chunk, consumer wave of the
// reverse sweep A = 16 tokens x 16 value indices), the scale exponents kept as int32 in a side array.  A tile is scaled
// by 2^k so that its largest magnitude lands in [1/2, 1) and rounded to multiples of 1/32767: an absolute error of at
// most 1.6e-5 of the tile's largest magnitude, against 2^-17 relative for the bf16 pairs the sweeps make of it and
// 2^-12 relative for an IEEE half (which put single elements of ga at twice the tolerance of the tests).  Every use of
// dsa is a sum over the value index, so an error that is absolute within a tile is the right kind.  A tile that holds
// inf or NaN gets the exponent DSA_BAD, which makes every value of it NaN for the reader.
constexpr int DSA_BAD = 0x7fffffff;
__device__ __forceinline__ int* dsa_scales(float* side, int64_t b, int64_t h, int64_t H, int nch, int c) {
  return reinterpret_cast<int*>(side) + (((size_t)b * H + h) * nch + c) * NCONS;
}
// x: this lane's four accumulator registers of the tile (any layout); the result is uniform over the wave.  The
// maximum runs over the magnitudes' bit patterns as unsigned integers, which orders finite < inf < NaN, so one biased
// exponent of 255 at the end stands for "inf or NaN somewhere in the tile".
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t x) {
  const uint32_t y = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, CTRL, ROW_MASK, 0xf, false);
  return x > y ? x : y;
}
__device__ __forceinline__ int dsa_scale_exponent(const f32x4_t x) {
  auto mag = [](float v) { return (uint32_t)__float_as_int(v) & 0x7fffffffu; };
  const uint32_t m01 = mag(x[0]) > mag(x[1]) ? mag(x[0]) : mag(x[1]);
  const uint32_t m23 = mag(x[2]) > mag(x[3]) ? mag(x[2]) : mag(x[3]);
  uint32_t m = m01 > m23 ? m01 : m23;
  m = dpp_umax<0x111, 0xf>(m);      // row_shr:1, 2, 4, 8: lane 15 of every row of 16 holds the row's maximum
  m = dpp_umax<0x112, 0xf>(m);
  m = dpp_umax<0x114, 0xf>(m);
  m = dpp_umax<0x118, 0xf>(m);
  m = dpp_umax<0x142, 0xa>(m);      // row_bcast:15 into rows 1 and 3: lanes 31 and 63 hold the maxima of their row pairs
  m = dpp_umax<0x143, 0xc>(m);      // row_bcast:31 into rows 2 and 3: lane 63 holds the wave's maximum
  const int e = (int)((uint32_t)__builtin_amdgcn_readlane((int)m, 63) >> 23);      // biased exponent of it
  return e == 255 ? DSA_BAD : 126 - e;                  // largest magnitude * 2^k in [1/2, 1)
}
// two values of a tile to fixed point (v_cvt_pknorm_i16_f32: round(x * 32767), clamped)
__device__ __forceinline__ uint32_t pack_dsa2(float x0, float x1, int kexp) {
  typedef short s2_t __attribute__((ext_vector_type(2)));
  const int k = kexp == DSA_BAD ? 0 : kexp;
  const s2_t p = __builtin_amdgcn_cvt_pknorm_i16(__builtin_amdgcn_ldexpf(x0, k), __builtin_amdgcn_ldexpf(x1, k));
  return __builtin_bit_cast(uint32_t, p);
}
// eight such values of one lane back to fp32
__device__ __forceinline__ void unpack_dsa8(const uint4 raw, int kexp, float4& lo4, float4& hi4) {
  const float mult = kexp == DSA_BAD ? __int_as_float(0x7fc00000) : __builtin_amdgcn_ldexpf(1.0f / 32767.0f, -kexp);
  auto lo = [&](uint32_t w) { return (float)((int)(w << 16) >> 16) * mult; };
  auto hi = [&](uint32_t w) { return (float)((int)w >> 16) * mult; };
  lo4 = make_float4(lo(raw.x), hi(raw.x), lo(raw.y), hi(raw.y));
  hi4 = make_float4(lo(raw.z), hi(raw.z), lo(raw.w), hi(raw.w));
}

// Selection operands that turn an MFMA into a transposer: against an A operand whose k-slot (g, jj) stands for key
// 8g + jj of a 32-key half, B = sel[x] yields D[token][n] = value at key 16x + n.
__device__ __forceinline__ void make_sel(u32x4_t (&sel)[2], int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    const int jj = 16 * x + n - 8 * g;
    u32x4_t sl = {0u, 0u, 0u, 0u};
    if (jj >= 0 && jj < 8) sl[jj >> 1] = (jj & 1) ? 0x3f800000u : 0x00003f80u;
    sel[x] = sl;
  }
}

}  // namespace chunk
}  // namespace hiprwkv
