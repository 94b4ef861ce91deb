// C ABI of libhiprwkv: argument checks, workspace carving, kernel selection.  Declarations: include/hiprwkv.h
#include "../../include/hiprwkv.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <initializer_list>
#include <mutex>

#include "wkv_args.h"

using namespace hiprwkv;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool dtype_ok(int d) { return d == HIPRWKV_F32 || d == HIPRWKV_BF16; }

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Rows of different (B,T,H,N) arrays at the same (token, head) are accessed together; arrays whose base addresses are
// congruent modulo 1 KiB then compete for the same part of the memory system (measured on MI355X: the backward sweeps
// that read and write the workspace arrays lose 5-10 % when everything starts on a 2 MiB boundary, and offsets that
// are multiples of 1 KiB change nothing).  The workspace arrays therefore start at their own 128-byte step past the
// phase of the first operand.
constexpr size_t PHASE_BYTES = 128, PHASE_SPAN = 1024;
char* at_phase(char* p, const void* like, unsigned steps) {
  const uintptr_t want = (reinterpret_cast<uintptr_t>(like) + steps * PHASE_BYTES) % PHASE_SPAN / PHASE_BYTES * PHASE_BYTES;
  const uintptr_t at = reinterpret_cast<uintptr_t>(p);
  const uintptr_t up = (at + 15) & ~(uintptr_t)15;
  return reinterpret_cast<char*>(up + (want + PHASE_SPAN - up % PHASE_SPAN) % PHASE_SPAN);
}

int check_matrix_shape(const char* op, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N) {
  if (!dtype_ok(io_dtype) || !dtype_ok(state_dtype)) return fail(HIPRWKV_EINVAL, "%s: dtype must be HIPRWKV_F32 or HIPRWKV_BF16", op);
  if (N != 64) return fail(HIPRWKV_EINVAL, "%s: head size N=%lld not supported (kernels are built for N=64)", op, (long long)N);
  if (B <= 0 || T <= 0 || H <= 0) return fail(HIPRWKV_EINVAL, "%s: B,T,H must be positive (got %lld,%lld,%lld)", op, (long long)B, (long long)T, (long long)H);
  if (B * H > 0x7fffffffLL) return fail(HIPRWKV_EINVAL, "%s: B*H exceeds the grid limit", op);
  return HIPRWKV_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Word 0 counts the workgroups of the chunked kernels whose bounded hand-shake wait ran out (they overwrite their
// outputs with NaN and add one here).  Word 1 counts numeric events of the chunked kernels: waves that had to cap a
// channel's decay over a chunk, and waves that found inf or NaN in a carried state (an fp16 operand overflowed).
// Every GPU holds its own copy of the words; their address is looked up once per device.
__device__ unsigned int g_status_words[2] = {0u, 0u};

constexpr int MAX_DEVICES = 64;
std::mutex g_sym_mu;
unsigned* g_status_ptr[MAX_DEVICES] = {};

// Workspace of hiprwkv_wkv4_bwd_noalloc: the checkpoint array of the WKV4 backward pass, (B, ceil(T/16), 3, C) fp32,
// for callers that cannot allocate.  Every GPU the library runs on holds its own 16 MiB copy until the process
// ends.  Host code never uses the array's name as an address: the device address is looked up once per device
// (scratch_base) and passed to the kernels like a caller's workspace.
constexpr size_t SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[SCRATCH_BYTES];
void* g_scratch_ptr[MAX_DEVICES] = {};

// Device address of the current device's scratch array; null (with the error text set) when the lookup fails.
void* scratch_base() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    fail(HIPRWKV_ELAUNCH, "wkv4_bwd_noalloc: no usable current device (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_sym_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      fail(HIPRWKV_ELAUNCH, "wkv4_bwd_noalloc: hipGetSymbolAddress failed (%s)", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}

// Public flag bits are accepted everywhere; the test hook HIPRWKV_DEBUG_DROP_PUBLISH only in a process that sets the
// environment variable HIPRWKV_ENABLE_DEBUG_FLAGS=1, so that a stray bit cannot turn a production call's outputs
// into NaN.  Unknown bits are refused.
int check_flags(const char* op, unsigned flags) {
  if (flags & ~(HIPRWKV_PUBLIC_FLAGS | HIPRWKV_DEBUG_DROP_PUBLISH))
    return fail(HIPRWKV_EINVAL, "%s: unknown flag bits 0x%x", op, flags & ~(HIPRWKV_PUBLIC_FLAGS | HIPRWKV_DEBUG_DROP_PUBLISH));
  if (flags & HIPRWKV_DEBUG_DROP_PUBLISH) {
    static const bool enabled = [] { const char* e = getenv("HIPRWKV_ENABLE_DEBUG_FLAGS"); return e != nullptr && e[0] == '1'; }();
    if (!enabled)
      return fail(HIPRWKV_EINVAL, "%s: HIPRWKV_DEBUG_DROP_PUBLISH needs HIPRWKV_ENABLE_DEBUG_FLAGS=1 in the environment", op);
  }
  return HIPRWKV_OK;
}

// Address of the current device's failure counter, or null when it cannot be obtained (the kernels then skip the
// count; the NaN poisoning does not depend on it).
unsigned* status_word() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(g_sym_mu);
  if (g_status_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_status_words)) != hipSuccess) return nullptr;
    g_status_ptr[dev] = static_cast<unsigned*>(p);
  }
  return g_status_ptr[dev];
}

}  // namespace

extern "C" {

const char* hiprwkv_last_error(void) { return g_err; }
int hiprwkv_version(void) { return 107; }

int hiprwkv_handshake_failures(hiprwkv_stream stream, unsigned* count) {
  if (count == nullptr) return fail(HIPRWKV_EINVAL, "handshake_failures: null count pointer");
  unsigned* word = status_word();
  if (word == nullptr) return fail(HIPRWKV_ELAUNCH, "handshake_failures: the device counter is not reachable");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(count, word, sizeof(unsigned), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "handshake_failures: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_numeric_events(hiprwkv_stream stream, unsigned* count) {
  if (count == nullptr) return fail(HIPRWKV_EINVAL, "numeric_events: null count pointer");
  unsigned* word = status_word();
  if (word == nullptr) return fail(HIPRWKV_ELAUNCH, "numeric_events: the device counter is not reachable");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(count, word + 1, sizeof(unsigned), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "numeric_events: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_wkv7_fwd(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* w, const void* r, const void* k, const void* v, const void* a, const void* b,
                     const void* s, const uint32_t* length, const uint8_t* new_starts, void* out, void* sa,
                     void* new_s, unsigned flags) {
  int rc = check_matrix_shape("wkv7_fwd", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv7_fwd", flags)) != HIPRWKV_OK) return rc;
  const void* req[] = {w, r, k, v, a, b, s, out, new_s};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv7_fwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv7_fwd: tensor pointers must be 16-byte aligned");
  }
  if (sa && !aligned16(sa)) return fail(HIPRWKV_EINVAL, "wkv7_fwd: sa must be 16-byte aligned");
  Wkv7Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.w = w; A.r = r; A.k = k; A.v = v; A.a = a; A.b = b; A.s = s;
  A.length = length; A.ns = new_starts;
  A.out = out; A.sa = sa; A.new_s = new_s;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.status = status_word();
  // T <= 8 (decode) runs on the small-T kernel; otherwise the chunked matrix-core kernels (fp16 operands for bf16
  // I/O, fp32 operands for fp32 I/O); HIPRWKV_FORCE_SEQ selects the sequential kernel
  const bool small_t = T <= HIPRWKV_SMALL_T && !(flags & HIPRWKV_NO_SMALL_T);
  const bool chunked = !(flags & HIPRWKV_FORCE_SEQ);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = small_t ? launch_wkv7_small_t_fwd(A, st)
               : !chunked ? launch_wkv7_seq_fwd(A, st)
               : A.io_f32 ? launch_wkv7_chunk_fwd_f32(A, st) : launch_wkv7_chunk_fwd(A, st);
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv7_fwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_wkv7_step(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                      const void* w, const void* r, const void* k, const void* v, const void* a, const void* b,
                      const void* s, int64_t s_batch_stride, const uint32_t* length, const uint8_t* new_starts,
                      void* out, void* new_s, int64_t new_s_batch_stride, unsigned flags) {
  int rc = check_matrix_shape("wkv7_step", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv7_step", flags)) != HIPRWKV_OK) return rc;
  if (T > HIPRWKV_SMALL_T) return fail(HIPRWKV_EINVAL, "wkv7_step: T=%lld, at most %d tokens per call", (long long)T, HIPRWKV_SMALL_T);
  const void* req[] = {w, r, k, v, a, b, s, out, new_s};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv7_step: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv7_step: tensor pointers must be 16-byte aligned");
  }
  const int64_t dense = H * N * N;
  const int64_t elem = state_dtype == HIPRWKV_F32 ? 4 : 2;
  for (int64_t stride : {s_batch_stride, new_s_batch_stride}) {
    if (stride < dense) return fail(HIPRWKV_EINVAL, "wkv7_step: state batch stride %lld is less than H*N*N = %lld", (long long)stride, (long long)dense);
    if ((stride * elem) % 16 != 0) return fail(HIPRWKV_EINVAL, "wkv7_step: state batch stride must be a multiple of 16 bytes");
  }
  Wkv7Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.w = w; A.r = r; A.k = k; A.v = v; A.a = a; A.b = b; A.s = s;
  A.length = length; A.ns = new_starts;
  A.out = out; A.new_s = new_s;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.s_bstride = s_batch_stride; A.new_s_bstride = new_s_batch_stride;
  const hipError_t e = launch_wkv7_small_t_fwd(A, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv7_step: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

size_t hiprwkv_wkv7_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t N) {
  // three fp32 arrays with one value per token and key; the second one is kept per chunk of 16 tokens (f_record)
  const size_t tokens = (size_t)((T + 15) / 16) * 16;
  return 3 * (align256((size_t)B * tokens * H * N * sizeof(float)) + PHASE_SPAN);
}

int hiprwkv_wkv7_bwd(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* w, const void* r, const void* k, const void* v, const void* a, const void* b,
                     const void* s, const uint32_t* length, const uint8_t* new_starts, const void* gy, const void* sa,
                     const void* gs_out, void* gw, void* gr, void* gk, void* gv, void* ga, void* gb, void* gs,
                     void* workspace, size_t workspace_bytes, unsigned flags) {
  int rc = check_matrix_shape("wkv7_bwd", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv7_bwd", flags)) != HIPRWKV_OK) return rc;
  const void* req[] = {w, r, k, v, a, b, s, gy, sa, gw, gr, gk, gv, ga, gb, gs, workspace};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv7_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv7_bwd: tensor pointers must be 16-byte aligned");
  }
  const size_t need = hiprwkv_wkv7_bwd_workspace_bytes(B, T, H, N);
  if (workspace_bytes < need)
    return fail(HIPRWKV_ENOSPACE, "wkv7_bwd: workspace has %zu bytes, %zu needed", workspace_bytes, need);
  Wkv7Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.w = w; A.r = r; A.k = k; A.v = v; A.a = a; A.b = b; A.s = s;
  A.length = length; A.ns = new_starts;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.status = status_word();
  A.gy = gy; A.sa_in = sa; A.gs_out = gs_out;
  A.gw = gw; A.gr = gr; A.gk = gk; A.gv = gv; A.ga = ga; A.gb = gb; A.gs = gs;
  const size_t one = need / 3 - PHASE_SPAN;
  char* ws = static_cast<char*>(workspace);
  A.dsa = reinterpret_cast<float*>(at_phase(ws, r, 3));
  A.e2 = reinterpret_cast<float*>(at_phase(reinterpret_cast<char*>(A.dsa) + one, r, 5));
  A.e3 = reinterpret_cast<float*>(at_phase(reinterpret_cast<char*>(A.e2) + one, r, 7));
  // Three sweeps: A (reverse) -> gv, dsa, gs; B (forward) -> gr, ga, e2, e3 (the chunked B: their sum shifted by a
  // token, in e2); C (reverse) -> gk, gb, gw.
  // All three run on the chunked matrix-core kernels (bf16 pairs for bf16 I/O, fp32 operands for fp32 I/O);
  // HIPRWKV_FORCE_SEQ selects the sequential kernels.
  const bool chunked = !(flags & HIPRWKV_FORCE_SEQ);
  const bool f32 = A.io_f32 != 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = !chunked ? launch_wkv7_seq_bwd_a(A, st) : f32 ? launch_wkv7_chunk_bwd_a_f32(A, st) : launch_wkv7_chunk_bwd_a(A, st);
  if (e == hipSuccess)
    e = !chunked ? launch_wkv7_seq_bwd_b(A, st) : f32 ? launch_wkv7_chunk_bwd_b_f32(A, st) : launch_wkv7_chunk_bwd_b(A, st);
  if (e == hipSuccess)
    e = !chunked ? launch_wkv7_seq_bwd_c(A, st) : f32 ? launch_wkv7_chunk_bwd_c_f32(A, st) : launch_wkv7_chunk_bwd_c(A, st);
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv7_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_wkv6_fwd(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* r, const void* k, const void* v, const void* w, const void* u, const void* s,
                     const uint32_t* length, const uint8_t* new_starts, void* out, void* new_s, unsigned flags) {
  int rc = check_matrix_shape("wkv6_fwd", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv6_fwd", flags)) != HIPRWKV_OK) return rc;
  const void* req[] = {r, k, v, w, u, s, out, new_s};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv6_fwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv6_fwd: tensor pointers must be 16-byte aligned");
  }
  Wkv6Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.r = r; A.k = k; A.v = v; A.w = w; A.u = u; A.s = s;
  A.length = length; A.ns = new_starts;
  A.out = out; A.new_s = new_s;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.status = status_word();
  // chunked matrix-core kernels (fp16 operands for bf16 I/O, fp32 operands for fp32 I/O) unless HIPRWKV_FORCE_SEQ
  const bool chunked = !(flags & HIPRWKV_FORCE_SEQ);
  const bool small_t = T <= HIPRWKV_SMALL_T && !(flags & HIPRWKV_NO_SMALL_T);
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = small_t ? launch_wkv6_small_t_fwd(A, st)
               : !chunked ? launch_wkv6_seq_fwd(A, st)
               : A.io_f32 ? launch_wkv6_chunk_fwd_f32(A, st) : launch_wkv6_chunk_fwd(A, st);
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv6_fwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_wkv6_step(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                      const void* r, const void* k, const void* v, const void* w, const void* u, const void* s,
                      int64_t s_batch_stride, const uint32_t* length, const uint8_t* new_starts, void* out, void* new_s,
                      int64_t new_s_batch_stride, unsigned flags) {
  int rc = check_matrix_shape("wkv6_step", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv6_step", flags)) != HIPRWKV_OK) return rc;
  if (T > HIPRWKV_SMALL_T) return fail(HIPRWKV_EINVAL, "wkv6_step: T=%lld, at most %d tokens per call", (long long)T, HIPRWKV_SMALL_T);
  const void* req[] = {r, k, v, w, u, s, out, new_s};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv6_step: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv6_step: tensor pointers must be 16-byte aligned");
  }
  const int64_t dense = H * N * N;
  const int64_t elem = state_dtype == HIPRWKV_F32 ? 4 : 2;
  for (int64_t stride : {s_batch_stride, new_s_batch_stride}) {
    if (stride < dense) return fail(HIPRWKV_EINVAL, "wkv6_step: state batch stride %lld is less than H*N*N = %lld", (long long)stride, (long long)dense);
    if ((stride * elem) % 16 != 0) return fail(HIPRWKV_EINVAL, "wkv6_step: state batch stride must be a multiple of 16 bytes");
  }
  Wkv6Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.r = r; A.k = k; A.v = v; A.w = w; A.u = u; A.s = s;
  A.length = length; A.ns = new_starts;
  A.out = out; A.new_s = new_s;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.s_bstride = s_batch_stride; A.new_s_bstride = new_s_batch_stride;
  const hipError_t e = launch_wkv6_small_t_fwd(A, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv6_step: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

size_t hiprwkv_wkv6_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t N) {
  return align256((size_t)B * T * H * N * sizeof(float)) + PHASE_SPAN + align256((size_t)B * H * N * sizeof(float));
}

int hiprwkv_wkv6_bwd(hiprwkv_stream stream, int io_dtype, int state_dtype, int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* r, const void* k, const void* v, const void* w, const void* u, const void* s,
                     const uint32_t* length, const uint8_t* new_starts, const void* gy, const void* gs_out, void* gr,
                     void* gk, void* gv, void* gw, float* gu, void* gs, void* workspace, size_t workspace_bytes,
                     unsigned flags) {
  int rc = check_matrix_shape("wkv6_bwd", io_dtype, state_dtype, B, T, H, N);
  if (rc) return rc;
  if ((rc = check_flags("wkv6_bwd", flags)) != HIPRWKV_OK) return rc;
  const void* req[] = {r, k, v, w, u, s, gy, gr, gk, gv, gw, gu, gs, workspace};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv6_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv6_bwd: tensor pointers must be 16-byte aligned");
  }
  const size_t need = hiprwkv_wkv6_bwd_workspace_bytes(B, T, H, N);
  if (workspace_bytes < need)
    return fail(HIPRWKV_ENOSPACE, "wkv6_bwd: workspace has %zu bytes, %zu needed", workspace_bytes, need);
  Wkv6Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.H = H;
  A.r = r; A.k = k; A.v = v; A.w = w; A.u = u; A.s = s;
  A.length = length; A.ns = new_starts;
  A.io_f32 = io_dtype == HIPRWKV_F32; A.st_f32 = state_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.status = status_word();
  A.gy = gy; A.gs_out = gs_out;
  A.gr = gr; A.gk = gk; A.gv = gv; A.gw = gw; A.gu = gu; A.gs = gs;
  char* ws = static_cast<char*>(workspace);
  A.er = reinterpret_cast<float*>(at_phase(ws, r, 5));
  A.eI = reinterpret_cast<float*>(reinterpret_cast<char*>(A.er) + align256((size_t)B * T * H * N * sizeof(float)));
  // Two sweeps: F (forward) -> gr, gu, er, eI; R (reverse) -> gk, gv, gw, gs, on the chunked matrix-core kernels
  // (bf16 pairs for bf16 I/O, fp32 operands for fp32 I/O); HIPRWKV_FORCE_SEQ selects the sequential kernel.
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e;
  if (flags & HIPRWKV_FORCE_SEQ) {
    e = launch_wkv6_seq_bwd(A, st);
  } else if (A.io_f32) {
    e = launch_wkv6_chunk_bwd_f_f32(A, st);
    if (e == hipSuccess) e = launch_wkv6_chunk_bwd_r_f32(A, st);
  } else {
    e = launch_wkv6_chunk_bwd_f(A, st);
    if (e == hipSuccess) e = launch_wkv6_chunk_bwd_r(A, st);
  }
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv6_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

static int wkv4_fwd_impl(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                         const void* u, const void* k, const void* v, const void* s, const uint32_t* length,
                         const uint8_t* new_starts, void* new_s, void* out, float* ckpt, unsigned flags);

int hiprwkv_wkv4_fwd(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                     const void* u, const void* k, const void* v, const void* s, const uint32_t* length,
                     const uint8_t* new_starts, void* new_s, void* out, unsigned flags) {
  return wkv4_fwd_impl(stream, io_dtype, B, T, C, w, u, k, v, s, length, new_starts, new_s, out, nullptr, flags);
}

int hiprwkv_wkv4_fwd_ckpt(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                          const void* u, const void* k, const void* v, const void* s, const uint32_t* length,
                          const uint8_t* new_starts, void* new_s, void* out, void* workspace, size_t workspace_bytes,
                          unsigned flags) {
  if (workspace == nullptr || !aligned16(workspace))
    return fail(HIPRWKV_EINVAL, "wkv4_fwd_ckpt: workspace must be a 16-byte aligned device pointer");
  if (B <= 0 || T <= 0 || C <= 0) return fail(HIPRWKV_EINVAL, "wkv4_fwd_ckpt: B,T,C must be positive");
  const size_t need = hiprwkv_wkv4_bwd_workspace_bytes(B, T, C);
  if (workspace_bytes < need)
    return fail(HIPRWKV_ENOSPACE, "wkv4_fwd_ckpt: workspace has %zu bytes, %zu needed", workspace_bytes, need);
  return wkv4_fwd_impl(stream, io_dtype, B, T, C, w, u, k, v, s, length, new_starts, new_s, out,
                       static_cast<float*>(workspace), flags);
}

static int wkv4_fwd_impl(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                         const void* u, const void* k, const void* v, const void* s, const uint32_t* length,
                         const uint8_t* new_starts, void* new_s, void* out, float* ckpt, unsigned flags) {
  if (int rc = check_flags("wkv4_fwd", flags)) return rc;
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "wkv4_fwd: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (B <= 0 || T <= 0 || C <= 0) return fail(HIPRWKV_EINVAL, "wkv4_fwd: B,T,C must be positive");
  if (B * ((C + 63) / 64) > 0x7fffffffLL) return fail(HIPRWKV_EINVAL, "wkv4_fwd: B*C exceeds the grid limit");
  // the forward kernel addresses a block of 32 tokens with 32-bit byte offsets from the block's first token
  if (C > (1LL << 23)) return fail(HIPRWKV_EINVAL, "wkv4_fwd: C exceeds 2^23 channels");
  const void* req[] = {w, u, k, v, s, new_s, out};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv4_fwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv4_fwd: tensor pointers must be 16-byte aligned");
  }
  Wkv4Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.C = C;
  A.w = w; A.u = u; A.k = k; A.v = v; A.s = s;
  A.length = length; A.ns = new_starts;
  A.new_s = new_s; A.out = out;
  A.ckpt = ckpt;
  A.io_f32 = io_dtype == HIPRWKV_F32;
  A.flags = flags;
  hipError_t e = launch_wkv4_fwd(A, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv4_fwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

size_t hiprwkv_wkv4_bwd_workspace_bytes(int64_t B, int64_t T, int64_t C) {
  return align256((size_t)B * ((T + 15) / 16) * 3 * C * sizeof(float));
}

int hiprwkv_wkv4_bwd(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                     const void* u, const void* k, const void* v, const void* gy, const void* s,
                     const uint32_t* length, const uint8_t* new_starts, const void* gs_new, float* gw, float* gu,
                     void* gk, void* gv, void* gs, void* workspace, size_t workspace_bytes, unsigned flags) {
  if (int rc = check_flags("wkv4_bwd", flags)) return rc;
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "wkv4_bwd: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (B <= 0 || T <= 0 || C <= 0) return fail(HIPRWKV_EINVAL, "wkv4_bwd: B,T,C must be positive");
  if (B * ((C + 63) / 64) > 0x7fffffffLL) return fail(HIPRWKV_EINVAL, "wkv4_bwd: B*C exceeds the grid limit");
  if (C > (1LL << 23)) return fail(HIPRWKV_EINVAL, "wkv4_bwd: C exceeds 2^23 channels");
  const void* req[] = {w, u, k, v, gy, s, gw, gu, gk, gv, gs, workspace};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "wkv4_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "wkv4_bwd: tensor pointers must be 16-byte aligned");
  }
  if (gs_new && !aligned16(gs_new)) return fail(HIPRWKV_EINVAL, "wkv4_bwd: tensor pointers must be 16-byte aligned");
  const size_t need = hiprwkv_wkv4_bwd_workspace_bytes(B, T, C);
  if (workspace_bytes < need)
    return fail(HIPRWKV_ENOSPACE, "wkv4_bwd: workspace has %zu bytes, %zu needed", workspace_bytes, need);
  Wkv4Args A;
  memset(&A, 0, sizeof(A));
  A.B = B; A.T = T; A.C = C;
  A.w = w; A.u = u; A.k = k; A.v = v; A.s = s;
  A.length = length; A.ns = new_starts;
  A.io_f32 = io_dtype == HIPRWKV_F32;
  A.flags = flags;
  A.gy = gy; A.gs_new = gs_new;
  A.gk = gk; A.gv = gv; A.gs = gs; A.gw = gw; A.gu = gu;
  A.ckpt = static_cast<float*>(workspace);
  hipError_t e = launch_wkv4_bwd(A, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "wkv4_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

size_t hiprwkv_wkv4_bwd_noalloc_max_bytes(void) { return SCRATCH_BYTES; }

int hiprwkv_wkv4_bwd_noalloc(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, const void* w,
                             const void* u, const void* k, const void* v, const void* gy, const void* s,
                             const uint32_t* length, const uint8_t* new_starts, const void* gs_new, float* gw,
                             float* gu, void* gk, void* gv, void* gs, unsigned flags) {
  if (B <= 0 || T <= 0 || C <= 0) return fail(HIPRWKV_EINVAL, "wkv4_bwd_noalloc: B,T,C must be positive");
  // the shared scratch array holds whatever the last call left: this entry point always writes its own checkpoints
  if (flags & HIPRWKV_CKPT_READY)
    return fail(HIPRWKV_EINVAL, "wkv4_bwd_noalloc: HIPRWKV_CKPT_READY is not accepted (the built-in scratch is shared between calls)");
  const size_t need = hiprwkv_wkv4_bwd_workspace_bytes(B, T, C);
  if (need > SCRATCH_BYTES)
    return fail(HIPRWKV_ENOSPACE,
                "wkv4_bwd_noalloc: B*ceil(T/16)*3*C*4 = %zu bytes of checkpoints exceed the built-in %zu-byte "
                "scratch; use hiprwkv_wkv4_bwd with a caller-provided workspace", need, SCRATCH_BYTES);
  void* ws = scratch_base();
  if (ws == nullptr) return HIPRWKV_ELAUNCH;
  return hiprwkv_wkv4_bwd(stream, io_dtype, B, T, C, w, u, k, v, gy, s, length, new_starts, gs_new, gw, gu, gk, gv,
                          gs, ws, SCRATCH_BYTES, flags);
}

namespace {
int check_shiftmix(const char* op, int io_dtype, int64_t B, int64_t T, int64_t C, int n_out, const void* x,
                   const void* prev, int64_t prev_bstride, const void* const* mix, const void* const* per_out) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "%s: dtype must be HIPRWKV_F32 or HIPRWKV_BF16", op);
  if (B <= 0 || T <= 0 || C <= 0 || C % 8 != 0) return fail(HIPRWKV_EINVAL, "%s: B, T must be positive and C a positive multiple of 8", op);
  if (B * T * (C / 8) > 0x7fffffffLL * 256) return fail(HIPRWKV_EINVAL, "%s: too many elements for one launch", op);
  if (n_out != 1 && n_out != 6) return fail(HIPRWKV_EINVAL, "%s: n_out must be 1 (channel mixing) or 6 (time mixing)", op);
  if (mix == nullptr || per_out == nullptr) return fail(HIPRWKV_EINVAL, "%s: null pointer array", op);
  const int64_t elem = io_dtype == HIPRWKV_F32 ? 4 : 2;
  if (prev_bstride < C || (prev_bstride * elem) % 16 != 0)
    return fail(HIPRWKV_EINVAL, "%s: the batch stride of the shift row must be at least C and a multiple of 16 bytes", op);
  const void* req[] = {x, prev};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "%s: null tensor pointer", op);
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "%s: tensor pointers must be 16-byte aligned", op);
  }
  for (int i = 0; i < n_out; ++i) {
    if (mix[i] == nullptr || per_out[i] == nullptr) return fail(HIPRWKV_EINVAL, "%s: null tensor pointer", op);
    if (!aligned16(mix[i]) || !aligned16(per_out[i])) return fail(HIPRWKV_EINVAL, "%s: tensor pointers must be 16-byte aligned", op);
  }
  return HIPRWKV_OK;
}
}  // namespace

int hiprwkv_rwkv7_shiftmix(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, int n_out, const void* x,
                           const void* prev, int64_t prev_batch_stride, const uint8_t* new_starts,
                           const void* const* mix, void* const* out) {
  int rc = check_shiftmix("rwkv7_shiftmix", io_dtype, B, T, C, n_out, x, prev, prev_batch_stride, mix,
                          const_cast<const void* const*>(out));
  if (rc) return rc;
  hipError_t e = launch_rwkv7_shiftmix(io_dtype == HIPRWKV_F32, B, T, C, n_out, x, prev, prev_batch_stride, new_starts,
                                       mix, out, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_shiftmix: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_rwkv7_shiftmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, int n_out,
                               const void* x, const void* prev, int64_t prev_batch_stride, const uint8_t* new_starts,
                               const void* const* mix, const void* const* g, void* dx, void* dprev,
                               int64_t dprev_batch_stride, float* dmix) {
  int rc = check_shiftmix("rwkv7_shiftmix_bwd", io_dtype, B, T, C, n_out, x, prev, prev_batch_stride, mix, g);
  if (rc) return rc;
  const void* req[] = {dx, dprev, dmix};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "rwkv7_shiftmix_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "rwkv7_shiftmix_bwd: tensor pointers must be 16-byte aligned");
  }
  const int64_t elem = io_dtype == HIPRWKV_F32 ? 4 : 2;
  if (dprev_batch_stride < C || (dprev_batch_stride * elem) % 16 != 0)
    return fail(HIPRWKV_EINVAL, "rwkv7_shiftmix_bwd: the batch stride of dprev must be at least C and a multiple of 16 bytes");
  hipError_t e = launch_rwkv7_shiftmix_bwd(io_dtype == HIPRWKV_F32, B, T, C, n_out, x, prev, prev_batch_stride, new_starts,
                                           mix, g, dx, dprev, dprev_batch_stride, dmix, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_shiftmix_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

namespace {
int check_gate(const char* op, int io_dtype, int64_t rows, int64_t C, std::initializer_list<const void*> ptrs) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "%s: dtype must be HIPRWKV_F32 or HIPRWKV_BF16", op);
  if (rows <= 0 || C <= 0 || C % 8 != 0) return fail(HIPRWKV_EINVAL, "%s: rows must be positive and C a positive multiple of 8", op);
  if (rows * (C / 8) > 0x7fffffffLL * 256) return fail(HIPRWKV_EINVAL, "%s: too many elements for one launch", op);
  for (const void* p : ptrs) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "%s: null tensor pointer", op);
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "%s: tensor pointers must be 16-byte aligned", op);
  }
  return HIPRWKV_OK;
}
int gate_done(const char* op, hipError_t e) {
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "%s: %s", op, hipGetErrorString(e));
  return HIPRWKV_OK;
}
}  // namespace

int hiprwkv_rwkv7_decay(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* w0, void* w) {
  if (int rc = check_gate("rwkv7_decay", io_dtype, rows, C, {x, w0, w})) return rc;
  return gate_done("rwkv7_decay", launch_rwkv7_decay(io_dtype == HIPRWKV_F32, 0, rows, C, x, w0, w, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_decay_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* w0,
                            const void* g, void* dx, float* dw0) {
  if (int rc = check_gate("rwkv7_decay_bwd", io_dtype, rows, C, {x, w0, g, dx, dw0})) return rc;
  return gate_done("rwkv7_decay_bwd", launch_rwkv7_decay_bwd(io_dtype == HIPRWKV_F32, 0, rows, C, x, w0, g, dx, dw0, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_agate(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* a0, void* a) {
  if (int rc = check_gate("rwkv7_agate", io_dtype, rows, C, {x, a0, a})) return rc;
  return gate_done("rwkv7_agate", launch_rwkv7_decay(io_dtype == HIPRWKV_F32, 1, rows, C, x, a0, a, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_agate_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* a0,
                            const void* g, void* dx, float* da0) {
  if (int rc = check_gate("rwkv7_agate_bwd", io_dtype, rows, C, {x, a0, g, dx, da0})) return rc;
  return gate_done("rwkv7_agate_bwd", launch_rwkv7_decay_bwd(io_dtype == HIPRWKV_F32, 1, rows, C, x, a0, g, dx, da0, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_relusq(hiprwkv_stream stream, int io_dtype, int64_t n, const void* x, void* out) {
  if (int rc = check_gate("rwkv7_relusq", io_dtype, 1, n, {x, out})) return rc;
  return gate_done("rwkv7_relusq", launch_rwkv7_relusq(io_dtype == HIPRWKV_F32, n, x, nullptr, out, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_relusq_bwd(hiprwkv_stream stream, int io_dtype, int64_t n, const void* x, const void* g, void* dx) {
  if (int rc = check_gate("rwkv7_relusq_bwd", io_dtype, 1, n, {x, g, dx})) return rc;
  return gate_done("rwkv7_relusq_bwd", launch_rwkv7_relusq(io_dtype == HIPRWKV_F32, n, x, g, dx, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_vmix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* v, const void* v_first,
                       const void* x, const void* v0, void* out) {
  if (int rc = check_gate("rwkv7_vmix", io_dtype, rows, C, {v, v_first, x, v0, out})) return rc;
  return gate_done("rwkv7_vmix", launch_rwkv7_vmix(io_dtype == HIPRWKV_F32, rows, C, v, v_first, x, v0, out, static_cast<hipStream_t>(stream)));
}
int hiprwkv_rwkv7_vmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* v, const void* v_first,
                           const void* x, const void* v0, const void* g, void* dv, void* dv_first, void* dx, float* dv0) {
  if (int rc = check_gate("rwkv7_vmix_bwd", io_dtype, rows, C, {v, v_first, x, v0, g, dv, dv_first, dx, dv0})) return rc;
  return gate_done("rwkv7_vmix_bwd", launch_rwkv7_vmix_bwd(io_dtype == HIPRWKV_F32, rows, C, v, v_first, x, v0, g, dv, dv_first, dx, dv0, static_cast<hipStream_t>(stream)));
}

int hiprwkv_rwkv7_premix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N, const void* k,
                         const void* a, const void* k_k, const void* k_a, void* k_out, void* a_out, void* b_out) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "rwkv7_premix: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (N != 64) return fail(HIPRWKV_EINVAL, "rwkv7_premix: head size N=%lld not supported (64 only)", (long long)N);
  if (rows <= 0 || H <= 0 || (rows * H + 3) / 4 > 0x7fffffffLL) return fail(HIPRWKV_EINVAL, "rwkv7_premix: bad rows/H");
  const void* req[] = {k, a, k_k, k_a, k_out, a_out, b_out};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "rwkv7_premix: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "rwkv7_premix: tensor pointers must be 16-byte aligned");
  }
  hipError_t e = launch_rwkv7_premix(io_dtype == HIPRWKV_F32, rows, H, k, a, k_k, k_a, k_out, a_out, b_out,
                                     static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_premix: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_rwkv7_postmix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N, const void* y,
                          const void* r, const void* k, const void* v, const void* g, const void* ln_w,
                          const void* ln_b, const void* r_k, float eps, void* out) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "rwkv7_postmix: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (N != 64) return fail(HIPRWKV_EINVAL, "rwkv7_postmix: head size N=%lld not supported (64 only)", (long long)N);
  if (rows <= 0 || H <= 0 || (rows * H + 3) / 4 > 0x7fffffffLL) return fail(HIPRWKV_EINVAL, "rwkv7_postmix: bad rows/H");
  const void* req[] = {y, r, k, v, g, ln_w, ln_b, r_k, out};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "rwkv7_postmix: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "rwkv7_postmix: tensor pointers must be 16-byte aligned");
  }
  hipError_t e = launch_rwkv7_postmix(io_dtype == HIPRWKV_F32, rows, H, y, r, k, v, g, ln_w, ln_b, r_k, eps, out,
                                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_postmix: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_rwkv7_premix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N, const void* k,
                             const void* a, const void* k_k, const void* k_a, const void* gk_out, const void* ga_out,
                             const void* gb_out, void* gk, void* ga, float* gk_k, float* gk_a) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "rwkv7_premix_bwd: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (N != 64) return fail(HIPRWKV_EINVAL, "rwkv7_premix_bwd: head size N=%lld not supported (64 only)", (long long)N);
  if (rows <= 0 || H <= 0 || H > 65536 || (rows * H + 3) / 4 > 0x7fffffffLL)
    return fail(HIPRWKV_EINVAL, "rwkv7_premix_bwd: bad rows/H");
  const void* req[] = {k, a, k_k, k_a, gk_out, ga_out, gb_out, gk, ga, gk_k, gk_a};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "rwkv7_premix_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "rwkv7_premix_bwd: tensor pointers must be 16-byte aligned");
  }
  hipError_t e = launch_rwkv7_premix_bwd(io_dtype == HIPRWKV_F32, rows, H, k, a, k_k, k_a, gk_out, ga_out, gb_out, gk,
                                         ga, gk_k, gk_a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_premix_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

int hiprwkv_rwkv7_postmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N, const void* y,
                              const void* r, const void* k, const void* v, const void* g, const void* ln_w,
                              const void* ln_b, const void* r_k, float eps, const void* gout, void* gy, void* gr,
                              void* gk, void* gv, void* gg, float* gln_w, float* gln_b, float* gr_k) {
  if (!dtype_ok(io_dtype)) return fail(HIPRWKV_EINVAL, "rwkv7_postmix_bwd: dtype must be HIPRWKV_F32 or HIPRWKV_BF16");
  if (N != 64) return fail(HIPRWKV_EINVAL, "rwkv7_postmix_bwd: head size N=%lld not supported (64 only)", (long long)N);
  if (rows <= 0 || H <= 0 || H > 65536 || (rows * H + 3) / 4 > 0x7fffffffLL)
    return fail(HIPRWKV_EINVAL, "rwkv7_postmix_bwd: bad rows/H");
  const void* req[] = {y, r, k, v, g, ln_w, ln_b, r_k, gout, gy, gr, gk, gv, gg, gln_w, gln_b, gr_k};
  for (const void* p : req) {
    if (p == nullptr) return fail(HIPRWKV_EINVAL, "rwkv7_postmix_bwd: null tensor pointer");
    if (!aligned16(p)) return fail(HIPRWKV_EINVAL, "rwkv7_postmix_bwd: tensor pointers must be 16-byte aligned");
  }
  hipError_t e = launch_rwkv7_postmix_bwd(io_dtype == HIPRWKV_F32, rows, H, y, r, k, v, g, ln_w, ln_b, r_k, eps, gout,
                                          gy, gr, gk, gv, gg, gln_w, gln_b, gr_k, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(HIPRWKV_ELAUNCH, "rwkv7_postmix_bwd: %s", hipGetErrorString(e));
  return HIPRWKV_OK;
}

}  // extern "C"
