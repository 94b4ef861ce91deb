// Plain argument blocks passed by value to the kernels, and the launcher prototypes the C ABI calls.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace hiprwkv {

struct Wkv7Args {
  int64_t B, T, H;
  const void *w, *r, *k, *v, *a, *b, *s;
  const uint32_t* length;
  const uint8_t* ns;
  void* out;
  void* sa;       // forward residual (may be null): fp32 beside fp32 I/O, IEEE half beside bf16 I/O
  void* new_s;
  int io_f32, st_f32;
  unsigned flags;
  // backward only
  const void* gy;
  const void* sa_in;     // the forward residual, in the forward's type
  const void* gs_out;
  void *gw, *gr, *gk, *gv, *ga, *gb, *gs;
  // workspace, three regions of (B,T,H,64) fp32 each.  The sequential sweeps and the chunked fp32 ones keep dsa in the
  // first as fp32; the chunked bf16 sweeps keep it there as 16-bit fixed point with one scale exponent per chunk and
  // value tile, the exponents in the third region (chunk_common.h dsa_scales).  The chunked sweeps keep e3_t + e2_{t+1}
  // in e2, as records per chunk and wave (chunk_common.h f_record), and do not use e3 otherwise.
  float *dsa, *e2, *e3;
  unsigned* status;      // device word counting workgroups whose hand-shake gave up (may be null)
  // Elements between the states of consecutive sequences in `s` / `new_s`; 0 = dense (H*64*64).  Honoured by the
  // small-T kernel only (states read and written inside a packed model state).
  int64_t s_bstride, new_s_bstride;
};

// Wkv6Args::flags bit: w is (H,64), shared by every token and sequence (HIPRWKV_W_PER_HEAD)
constexpr unsigned FLAG_W_PER_HEAD = 0x10u;

struct Wkv6Args {
  int64_t B, T, H;
  const void *r, *k, *v, *w, *u, *s;
  const uint32_t* length;
  const uint8_t* ns;
  void* out;
  void* new_s;
  int io_f32, st_f32;
  unsigned flags;
  // backward only
  const void* gy;
  const void* gs_out;
  void *gr, *gk, *gv, *gw, *gs;
  float* gu;   // (B,H,64)
  float* er;   // workspace (B,T,H,64): r . (S' dy)
  float* eI;   // workspace (B,H,64): rowsum(dS_out * S_{length-1})
  unsigned* status;   // device word counting workgroups whose hand-shake gave up (may be null)
  // Elements between the states of consecutive sequences in `s` / `new_s`; 0 = dense (H*64*64).  Honoured by the
  // small-T kernel only (states read and written inside a packed model state).
  int64_t s_bstride, new_s_bstride;
};

// Wkv4Args::flags bit: the workspace already holds the checkpoints (HIPRWKV_CKPT_READY)
constexpr unsigned FLAG_CKPT_READY = 0x20u;

struct Wkv4Args {
  int64_t B, T, C;
  const void *w, *u, *k, *v, *s;
  const uint32_t* length;
  const uint8_t* ns;
  void* new_s;
  void* out;
  int io_f32;
  unsigned flags;
  // backward only
  const void* gy;
  const void* gs_new;
  void *gk, *gv, *gs;
  float *gw, *gu;   // (B,C) each
  float* ckpt;      // workspace: (B, ceil(T/16), 3, C) states entering every 16th step (forward: optional output)
};

// Raises a kernel's dynamic-LDS limit once per kernel and device instead of at every enqueue (the attribute call
// goes to the driver; hipGetDevice does not).
struct LdsAttrOnce {
  std::atomic<uint64_t> done{0};   // bit d: set on device d
};
inline hipError_t allow_dynamic_lds(LdsAttrOnce& once, const void* kernel, size_t bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (once.done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) once.done.fetch_or(bit, std::memory_order_release);
  return e;
}

hipError_t launch_wkv7_seq_fwd(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_fwd(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_fwd_f32(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_a_f32(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_b_f32(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_c_f32(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_small_t_fwd(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv6_small_t_fwd(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_a(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_b(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_chunk_bwd_c(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_seq_bwd_a(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_seq_bwd_b(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv7_seq_bwd_c(const Wkv7Args& A, hipStream_t stream);
hipError_t launch_wkv6_seq_fwd(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_fwd(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_fwd_f32(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_seq_bwd(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_bwd_f(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_bwd_r(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_bwd_f_f32(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv6_chunk_bwd_r_f32(const Wkv6Args& A, hipStream_t stream);
hipError_t launch_wkv4_fwd(const Wkv4Args& A, hipStream_t stream);
hipError_t launch_wkv4_bwd(const Wkv4Args& A, hipStream_t stream);
hipError_t launch_rwkv7_premix(int io_f32, int64_t rows, int64_t H, const void* k, const void* a, const void* k_k,
                               const void* k_a, void* k_out, void* a_out, void* b_out, hipStream_t stream);
hipError_t launch_rwkv7_postmix(int io_f32, int64_t rows, int64_t H, const void* y, const void* r, const void* k,
                                const void* v, const void* g, const void* ln_w, const void* ln_b, const void* r_k,
                                float eps, void* out, hipStream_t stream);
hipError_t launch_rwkv7_decay(int io_f32, int sigmoid, int64_t rows, int64_t C, const void* x, const void* w0, void* w,
                              hipStream_t stream);
hipError_t launch_rwkv7_decay_bwd(int io_f32, int sigmoid, int64_t rows, int64_t C, const void* x, const void* w0,
                                  const void* g, void* dx, float* dw0, hipStream_t stream);
hipError_t launch_rwkv7_relusq(int io_f32, int64_t n, const void* x, const void* g, void* out, hipStream_t stream);
hipError_t launch_rwkv7_vmix(int io_f32, int64_t rows, int64_t C, const void* v, const void* v_first, const void* x,
                             const void* v0, void* out, hipStream_t stream);
hipError_t launch_rwkv7_vmix_bwd(int io_f32, int64_t rows, int64_t C, const void* v, const void* v_first, const void* x,
                                 const void* v0, const void* g, void* dv, void* dv_first, void* dx, float* dv0,
                                 hipStream_t stream);
hipError_t launch_rwkv7_shiftmix(int io_f32, int64_t B, int64_t T, int64_t C, int n_out, const void* x, const void* prev,
                                 int64_t prev_bstride, const uint8_t* ns, const void* const* mix, void* const* out,
                                 hipStream_t stream);
hipError_t launch_rwkv7_shiftmix_bwd(int io_f32, int64_t B, int64_t T, int64_t C, int n_out, const void* x,
                                     const void* prev, int64_t prev_bstride, const uint8_t* ns, const void* const* mix,
                                     const void* const* g, void* dx, void* dprev, int64_t dprev_bstride, float* dmix,
                                     hipStream_t stream);
hipError_t launch_rwkv7_premix_bwd(int io_f32, int64_t rows, int64_t H, const void* k, const void* a, const void* k_k,
                                   const void* k_a, const void* gko, const void* gao, const void* gbo, void* gk,
                                   void* ga, float* gk_k, float* gk_a, hipStream_t stream);
hipError_t launch_rwkv7_postmix_bwd(int io_f32, int64_t rows, int64_t H, const void* y, const void* r, const void* k,
                                    const void* v, const void* g, const void* ln_w, const void* ln_b, const void* r_k,
                                    float eps, const void* go, void* gy, void* gr, void* gk, void* gv, void* gg,
                                    float* gln_w, float* gln_b, float* gr_k, hipStream_t stream);

}  // namespace hiprwkv
