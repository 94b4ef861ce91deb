/*
 * hiprwkv -- C ABI of the MI355X (gfx950) WKV recurrence library.
 *
 * Every entry point only enqueues work on the caller's HIP stream: it does not
 * allocate, free or synchronise, so it can be called from an XLA custom-call
 * handler thread.  All pointers are device pointers, 16-byte aligned.  Entry points return
 * HIPRWKV_OK or a negative HIPRWKV_E* code; hiprwkv_last_error() then returns a
 * thread-local message.
 *
 * Operand order follows the reference's jax.ffi targets, whose native
 * implementation (package `jaxrwkvkernel`, CUDA only) is not part of the
 * reference tree; each declaration cites the Python call site it replaces.
 *
 * Shapes: B sequences (the reference's vmap axis), T tokens, H heads, N head size.
 *   WKV7/WKV6 token tensors  (B,T,H,N) row-major, io_dtype
 *   WKV7 state               (B,H,N,N) state_dtype, s[b,h,i,j]: value row i, key column j
 *   WKV6 state               (B,H,N,N) state_dtype, s[b,h,i,j]: key row i, value column j
 *   WKV4 token tensors       (B,T,C), state (B,3,C) = (aa,bb,pp)
 *   length                   (B,) uint32, may be NULL (= T)
 *   new_starts               (B,T) one byte per token (0/1), may be NULL (= none)
 * The recurrence always runs in fp32 whatever the io/state dtypes are.
 *
 * Placement of the token tensors.  The kernels touch the rows of all token tensors of a call at the same
 * (token, head) together.  When the tensors' base addresses are congruent modulo 1 KiB (two large allocations
 * of a caching allocator usually are: both start on 2 MiB boundaries) those rows compete for the same part of
 * the memory system.  Measured on MI355X, WKV7 at B8 T4096 H32 bf16, forward with its residual / forward +
 * backward: 303 / 1619 us with every tensor on a 2 MiB boundary; 284 / 1535 us with only the outputs, the
 * gradients and the workspace arrays moved; 265 / 1469 us with each tensor, the inputs included, at its own
 * multiple of 128 bytes past a 1 KiB boundary (0, 128, ..., 896).  Offsets that are multiples of 1 KiB change
 * nothing.  A caller that owns the placement of its operands should stagger them that way; the library does
 * it for the arrays inside `workspace`, and the Python operators do it for every tensor they allocate.
 */
#ifndef HIPRWKV_H_
#define HIPRWKV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPRWKV_OK 0
#define HIPRWKV_EINVAL (-1)   /* bad argument (shape, dtype, NULL pointer) */
#define HIPRWKV_ELAUNCH (-2)  /* hipLaunchKernel reported an error */
#define HIPRWKV_ENOSPACE (-3) /* workspace too small */

#define HIPRWKV_F32 0
#define HIPRWKV_BF16 1

/* flags */
/* Reproduce AssociativeScanRWKV where it differs from the sequential loop:
 * WKV7 y[t] = 0 when new_starts[t+1] (rwkv7.py:331-333,344); returned state is the
 * one entering position `length` (rwkv7.py:345, rwkv6.py:301, rwkv4.py:300). */
#define HIPRWKV_COMPAT_ASSOC 1u
/* Force the sequential fp32 VALU kernel even where a chunked MFMA kernel exists. */
#define HIPRWKV_FORCE_SEQ 2u
/* hiprwkv_wkv7_fwd and hiprwkv_wkv6_fwd run sequences of at most HIPRWKV_SMALL_T tokens (decode steps) on a kernel
 * that streams the state once and has no per-launch set-up; this flag sends them to the general kernels instead. */
#define HIPRWKV_NO_SMALL_T 4u
#define HIPRWKV_SMALL_T 8
/* hiprwkv_wkv6_fwd / hiprwkv_wkv6_bwd: `w` is (H, N), one log decay per head channel shared by every token and
 * sequence (RWKV-5, rwkv5.py:194 / rwkv5_2.py:198), instead of (B, T, H, N).  The backward still writes the decay
 * cotangent per token, (B, T, H, N); the caller sums it over B and T. */
#define HIPRWKV_W_PER_HEAD 0x10u
/* hiprwkv_wkv4_bwd: the workspace already holds the checkpoints that hiprwkv_wkv4_fwd_ckpt wrote for the same
 * inputs; the backward then skips its own first pass over k and v. */
#define HIPRWKV_CKPT_READY 0x20u
/* Test hook for the chunked kernels' bounded hand-shake: the producer wave of the last chunk does not publish it, the
 * consumer waves' wait runs out (a few milliseconds), every wave still ends normally, the outputs of every
 * (sequence, head) are NaN and hiprwkv_handshake_failures() has advanced by B*H per kernel. */
#define HIPRWKV_DEBUG_DROP_PUBLISH 0x100u
/* Every flag a production caller may pass.  Entry points refuse other bits, and refuse HIPRWKV_DEBUG_DROP_PUBLISH
 * unless the process runs with HIPRWKV_ENABLE_DEBUG_FLAGS=1 in its environment. */
#define HIPRWKV_PUBLIC_FLAGS (HIPRWKV_COMPAT_ASSOC | HIPRWKV_FORCE_SEQ | HIPRWKV_NO_SMALL_T | HIPRWKV_W_PER_HEAD | HIPRWKV_CKPT_READY)

typedef void* hiprwkv_stream; /* a hipStream_t */

const char* hiprwkv_last_error(void);
int hiprwkv_version(void);

/* The chunked kernels pass work between waves of a workgroup through a hand-shake with a bounded wait (a broken
 * hand-shake must not hang the GPU).  A workgroup whose wait runs out overwrites all its outputs for that
 * (sequence, head) with NaN and adds one to a per-device counter; this call copies the counter of the current
 * device to *count (host memory).  Unlike every other entry point it synchronises `stream`.  No counterpart in
 * the reference; for health checks and tests. */
int hiprwkv_handshake_failures(hiprwkv_stream stream, unsigned* count);

/* Numeric events of the chunked matrix-core kernels since the process started, per device, copied to *count (host
 * memory; synchronises `stream`).  Two things are counted, once per wave that meets them:
 *  - a key channel whose log decay summed over a 16-token chunk is below -80 (a decay of e^-5 per token sustained over
 *    the chunk; RWKV-7's own w <= -0.5 keeps it above -10): the chunked kernels, fp32 I/O included, scale that
 *    channel's steps of the chunk to a total of -80, so its result is no longer exact.  Every sweep of a backward
 *    call that meets such a chunk counts it again.  HIPRWKV_FORCE_SEQ has no such floor.
 *  - inf or NaN in the carried state of the bf16-I/O forward kernels (WKV7, WKV6) after the last token: their matrix
 *    operands are IEEE half, so |state|, |sa|, |v| or a decay-scaled input beyond 65504 overflow; y and the state
 *    are then inf/NaN from that token on (until a reset starts a new state: an overflow whose state a later reset
 *    discards shows in y alone).
 * Magnitudes far below 1 lose precision silently instead: the half operands have 11 significant bits down to 6e-5
 * and fewer below, so v (and with it the state and sa) scaled by 1e-5 doubles the error of y and 1e-7 brings it to
 * 4 %; the op is linear in (v, s), so a caller with such values scales them by a power of two around the call.
 * No counterpart in the reference; for health checks and tests. */
int hiprwkv_numeric_events(hiprwkv_stream stream, unsigned* count);

/* ---- WKV7 ------------------------------------------------------------------
 * Replaces ffi target "wkv7-fwd-{fp32,bf16}": operands w,r,k,v,a,b,s,length,new_starts
 * -> out, s_restore, sa_restore, new_s  (rwkv7.py:372-375).  `w` is the raw decay
 * argument; the op applies exp(-exp(w)) (rwkv7.py:201).  `sa` (B,T,H,N) is
 * the residual S_{t-1} a_t kept for the backward pass (the reference's sa_restore):
 * fp32 beside fp32 I/O, IEEE half (2 bytes per element) beside bf16 I/O; the caller hands
 * the same buffer to hiprwkv_wkv7_bwd.  Pass NULL for inference.  No state checkpoints
 * (s_restore) are needed. */
int hiprwkv_wkv7_fwd(hiprwkv_stream stream, int io_dtype, int state_dtype,
                     int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* w, const void* r, const void* k, const void* v,
                     const void* a, const void* b, const void* s,
                     const uint32_t* length, const uint8_t* new_starts,
                     void* out, void* sa, void* new_s, unsigned flags);

/* A decode step (T <= HIPRWKV_SMALL_T tokens per sequence) on a state that lives inside the packed model state of the
 * reference: there a sequence's state is (L, 2+N, C) and layer l's rows 2.. are the (H,N,N) WKV state, flat
 * (rwkv7.py:176-180 default_state, :254-260 the slice and reshape around inner_loop), so with a batch axis in front
 * the states of consecutive sequences are H*N*N contiguous elements each, L*(2+N)*C elements apart.  `s` and `new_s`
 * point at the first sequence's state, `*_batch_stride` is that distance in elements (>= H*N*N, a multiple of 16
 * bytes); everything else is as in hiprwkv_wkv7_fwd without `sa`.  Every element of a state is read once, before
 * anything is written, by the thread that writes it: `new_s` may be `s` (same stride) for an update in place. */
int hiprwkv_wkv7_step(hiprwkv_stream stream, int io_dtype, int state_dtype,
                      int64_t B, int64_t T, int64_t H, int64_t N,
                      const void* w, const void* r, const void* k, const void* v,
                      const void* a, const void* b, const void* s, int64_t s_batch_stride,
                      const uint32_t* length, const uint8_t* new_starts,
                      void* out, void* new_s, int64_t new_s_batch_stride, unsigned flags);

/* Bytes of scratch hiprwkv_wkv7_bwd needs for this shape: three fp32 (B,T,H,N) arrays plus 1 KiB each (see "Placement"). */
size_t hiprwkv_wkv7_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t N);

/* Replaces ffi target "wkv7-bwd-{fp32,bf16}": operands w,r,k,v,a,b,s,length,new_starts,
 * gy,s_restore,sa_restore,gs_out -> gw,gr,gk,gv,ga,gb,gs  (rwkv7.py:406-408).
 * Unlike the reference's native op it honours new_starts, takes the cotangent of the
 * returned state (gs_out, may be NULL = 0) and returns the one of the input state.
 * Three sweeps over the sequence on the matrix cores: bf16 hi+lo operand pairs beside bf16
 * I/O (the cotangent of `sa` passes between them as 16-bit fixed point with a power-of-two
 * scale per 16 x 16 tile: 16 bits whatever the size of the cotangents), fp32 operands and an
 * fp32 workspace (no rounding below fp32) beside fp32 I/O; HIPRWKV_FORCE_SEQ runs the
 * sequential fp32 sweeps instead. */
int hiprwkv_wkv7_bwd(hiprwkv_stream stream, int io_dtype, int state_dtype,
                     int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* w, const void* r, const void* k, const void* v,
                     const void* a, const void* b, const void* s,
                     const uint32_t* length, const uint8_t* new_starts,
                     const void* gy, const void* sa, const void* gs_out,
                     void* gw, void* gr, void* gk, void* gv, void* ga, void* gb, void* gs,
                     void* workspace, size_t workspace_bytes, unsigned flags);

/* ---- WKV6 ------------------------------------------------------------------
 * The reference has no native WKV6 op (README.md:93-99); the operand order follows
 * inner_loop(r,k,v,w,time_first,s,length,new_starts) (rwkv6.py:175).  `w` is the log
 * decay -exp(raw) (rwkv6.py:217-218), `u` = time_faaaa (H,N) io_dtype. */
int hiprwkv_wkv6_fwd(hiprwkv_stream stream, int io_dtype, int state_dtype,
                     int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* r, const void* k, const void* v, const void* w,
                     const void* u, const void* s,
                     const uint32_t* length, const uint8_t* new_starts,
                     void* out, void* new_s, unsigned flags);

/* hiprwkv_wkv6_fwd for a decode step (T <= HIPRWKV_SMALL_T) on a state inside the reference's packed model state
 * (rwkv6.py:148-153 default_state: (L, 2+N, C) per sequence; :221-224 the slice state[1:] of the time-mixing part,
 * reshaped to (H,N,N) around inner_loop and written back): `s` and `new_s` point at the first sequence's state, the
 * states of consecutive sequences are `*_batch_stride` elements apart (>= H*N*N, a multiple of 16 bytes); `new_s` may
 * be `s` for an update in place.  Same conventions as hiprwkv_wkv7_step. */
int hiprwkv_wkv6_step(hiprwkv_stream stream, int io_dtype, int state_dtype,
                      int64_t B, int64_t T, int64_t H, int64_t N,
                      const void* r, const void* k, const void* v, const void* w,
                      const void* u, const void* s, int64_t s_batch_stride,
                      const uint32_t* length, const uint8_t* new_starts,
                      void* out, void* new_s, int64_t new_s_batch_stride, unsigned flags);

size_t hiprwkv_wkv6_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t N);

/* Cotangents of wkv6_fwd: gr,gk,gv,gw (B,T,H,N) io_dtype; gu (B,H,N) fp32, to be summed
 * over B by the caller (as the reference does for the WKV4 parameters, rwkv4.py:351);
 * gs (B,H,N,N) state_dtype.  Forward and backward run on the matrix cores for both I/O
 * dtypes (fp32 operands beside fp32 I/O); HIPRWKV_FORCE_SEQ selects the sequential kernels. */
int hiprwkv_wkv6_bwd(hiprwkv_stream stream, int io_dtype, int state_dtype,
                     int64_t B, int64_t T, int64_t H, int64_t N,
                     const void* r, const void* k, const void* v, const void* w,
                     const void* u, const void* s,
                     const uint32_t* length, const uint8_t* new_starts,
                     const void* gy, const void* gs_out,
                     void* gr, void* gk, void* gv, void* gw, float* gu, void* gs,
                     void* workspace, size_t workspace_bytes, unsigned flags);

/* ---- WKV4 ------------------------------------------------------------------
 * Replaces ffi target "wkv4-fwd-{fp32,bf16}": operands w,time_first,k,v,s,length,new_starts
 * -> new_s, out  (rwkv4.py:320-321).  `w` = -exp(time_decay) (rwkv4.py:312) and `u` are (C,)
 * io_dtype; the receptance is applied by the caller (rwkv4.py:406).  C <= 2^23.  The output is
 * num * (1/den) with a 1-ulp reciprocal where the reference divides (difference ~1e-7 relative). */
int hiprwkv_wkv4_fwd(hiprwkv_stream stream, int io_dtype,
                     int64_t B, int64_t T, int64_t C,
                     const void* w, const void* u, const void* k, const void* v, const void* s,
                     const uint32_t* length, const uint8_t* new_starts,
                     void* new_s, void* out, unsigned flags);

size_t hiprwkv_wkv4_bwd_workspace_bytes(int64_t B, int64_t T, int64_t C);

/* hiprwkv_wkv4_fwd for a caller that will run the backward pass (the forward rule of the custom VJP, rwkv4.py:379-383):
 * same results, and the state entering every 16th step goes to `workspace` (hiprwkv_wkv4_bwd_workspace_bytes), which
 * hiprwkv_wkv4_bwd then takes with HIPRWKV_CKPT_READY.  Saves that pass its re-read of k and v. */
int hiprwkv_wkv4_fwd_ckpt(hiprwkv_stream stream, int io_dtype,
                          int64_t B, int64_t T, int64_t C,
                          const void* w, const void* u, const void* k, const void* v, const void* s,
                          const uint32_t* length, const uint8_t* new_starts,
                          void* new_s, void* out, void* workspace, size_t workspace_bytes, unsigned flags);

/* Replaces ffi target "wkv4-bwd-{fp32,bf16}": operands w,u,k,v,gy,s,length,new_starts,gs_new
 * -> gw (B,C), gu (B,C), gk, gv, gs  (rwkv4.py:347-349); gw and gu are per sequence in fp32 and are summed
 * over B by the caller (rwkv4.py:351).  gy is the cotangent of the un-gated output.  Unlike the reference's
 * native op it honours gs_new (may be NULL = 0), returns gs, and cuts the chain at new_starts.  C <= 2^23. */
int hiprwkv_wkv4_bwd(hiprwkv_stream stream, int io_dtype,
                     int64_t B, int64_t T, int64_t C,
                     const void* w, const void* u, const void* k, const void* v, const void* gy, const void* s,
                     const uint32_t* length, const uint8_t* new_starts, const void* gs_new,
                     float* gw, float* gu, void* gk, void* gv, void* gs,
                     void* workspace, size_t workspace_bytes, unsigned flags);

/* hiprwkv_wkv4_bwd for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc): the same kernels, with the checkpoint workspace in a 16 MiB array that is part
 * of the library's device image (one copy per GPU, held until the process ends) instead of a caller's buffer.  It has
 * no counterpart in the reference.  Calls nothing that allocates.  Shapes whose checkpoints
 * (hiprwkv_wkv4_bwd_workspace_bytes) exceed hiprwkv_wkv4_bwd_noalloc_max_bytes() are refused with HIPRWKV_ENOSPACE.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (different streams) race; calls
 * on one stream, or ordered by events, do not.  Nothing in the array needs clearing between calls (each call writes
 * every checkpoint before it reads it). */
size_t hiprwkv_wkv4_bwd_noalloc_max_bytes(void);
int hiprwkv_wkv4_bwd_noalloc(hiprwkv_stream stream, int io_dtype,
                             int64_t B, int64_t T, int64_t C,
                             const void* w, const void* u, const void* k, const void* v, const void* gy, const void* s,
                             const uint32_t* length, const uint8_t* new_starts, const void* gs_new,
                             float* gw, float* gu, void* gk, void* gv, void* gs, unsigned flags);

/* ---- RWKV-7 token shift and interpolation ---------------------------------------------------
 * The head of time_mixing_seq and channel_mixing_seq (rwkv7.py:226-235 and :192-195), which the reference computes in
 * jnp; no counterpart among its ffi targets:
 *     sx_t = (new_starts[t] ? 0 : x_{t-1}) - x_t ,  out_i = x + sx . mix_i ,  i < n_out   (6: x_r x_w x_k x_v x_a x_g; 1: x_k)
 * x and every out_i are (B,T,C) io_dtype; `prev` is the token before t = 0 of every sequence, C elements each,
 * `prev_batch_stride` elements apart (>= C, a multiple of 16 bytes: the layer's shift row inside the packed model
 * state, rwkv7.py:254, :284); `mix` and `out` are host arrays of n_out device pointers, mix[i] a (C,) io_dtype
 * parameter.  C must be a multiple of 8.  new_starts (B,T) bytes or NULL. */
int hiprwkv_rwkv7_shiftmix(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, int n_out,
                           const void* x, const void* prev, int64_t prev_batch_stride, const uint8_t* new_starts,
                           const void* const* mix, void* const* out);
/* Cotangents for cotangents g[i] (B,T,C) of the outputs: dx (B,T,C) and dprev (C elements per sequence,
 * `dprev_batch_stride` apart) in io_dtype, dmix (n_out, C) fp32, summed over sequences and tokens (zeroed by the call). */
int hiprwkv_rwkv7_shiftmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t B, int64_t T, int64_t C, int n_out,
                               const void* x, const void* prev, int64_t prev_batch_stride, const uint8_t* new_starts,
                               const void* const* mix, const void* const* g, void* dx, void* dprev,
                               int64_t dprev_batch_stride, float* dmix);

/* ---- RWKV-7 decay, value mix and gate between the projections and the op -------------------
 * Element-wise steps of time_mixing_seq that the reference computes in jnp (rwkv7.py:237, :241-242, :244); no
 * counterpart among its ffi targets.  Token tensors (rows, C) io_dtype, parameters w0, v0, a0 (C,) io_dtype, C a
 * multiple of 8; the parameter cotangents dw0, dv0, da0 are (C,) fp32 sums over the rows (zeroed by the call).
 *     decay:  w  = -softplus(-(w0 + x)) - 0.5          x = tanh(xw w1) w2
 *     vmix :  v' = v + (v_first - v) sigmoid(v0 + x)   x = (xv v1) v2      (layers after the first)
 *     agate:  a  = sigmoid(a0 + x)                     x = (xa a1) a2 */
int hiprwkv_rwkv7_decay(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* w0, void* w);
int hiprwkv_rwkv7_decay_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* w0,
                            const void* g, void* dx, float* dw0);
int hiprwkv_rwkv7_agate(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* a0, void* a);
int hiprwkv_rwkv7_agate_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* x, const void* a0,
                            const void* g, void* dx, float* da0);
/* Channel mixing's activation, rwkv7.py:196: out = relu(x)^2 over n elements (n a multiple of 8); dx = 2 g relu(x). */
int hiprwkv_rwkv7_relusq(hiprwkv_stream stream, int io_dtype, int64_t n, const void* x, void* out);
int hiprwkv_rwkv7_relusq_bwd(hiprwkv_stream stream, int io_dtype, int64_t n, const void* x, const void* g, void* dx);
int hiprwkv_rwkv7_vmix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* v, const void* v_first,
                       const void* x, const void* v0, void* out);
int hiprwkv_rwkv7_vmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t C, const void* v, const void* v_first,
                           const void* x, const void* v0, const void* g, void* dv, void* dv_first, void* dx, float* dv0);

/* ---- RWKV-7 time-mixing stages around the op ------------------------------------------
 * The element-wise work the reference does in jnp on either side of inner_loop (rwkv7.py:248-252, 257 and :263-265),
 * fused into one pass each; it has no counterpart among the reference's ffi targets.  `rows` = number of tokens
 * (all batch axes flattened), tensors (rows, H, 64) io_dtype, parameters k_k, k_a, ln_w, ln_b, r_k (H, 64) io_dtype.
 *   premix : kk = normalize_head(k . k_k); k_out = k (1 + (a - 1) k_a); a_out = -kk; b_out = kk . a
 *   postmix: out = (group_norm_head(y, eps) . ln_w + ln_b + (sum_j r_j k_j r_k_j) v) . g      (k = premix's k_out) */
int hiprwkv_rwkv7_premix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N,
                         const void* k, const void* a, const void* k_k, const void* k_a,
                         void* k_out, void* a_out, void* b_out);
int hiprwkv_rwkv7_postmix(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N,
                          const void* y, const void* r, const void* k, const void* v, const void* g,
                          const void* ln_w, const void* ln_b, const void* r_k, float eps, void* out);

/* Their backward passes (what jax.grad derives for rwkv7.py:248-252, 257 and :263-265).  The forward quantities are
 * recomputed from the same inputs; nothing is saved.  Cotangents of tensors are io_dtype (rows, H, 64); cotangents of
 * the per-head parameters (sums over all rows) are always fp32 (H, 64) and are overwritten, not accumulated into.
 *   premix_bwd : from the cotangents of k_out, a_out, b_out to those of k, a, k_k, k_a
 *   postmix_bwd: from the cotangent of out to those of y, r, k, v, g, ln_w, ln_b, r_k */
int hiprwkv_rwkv7_premix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N,
                             const void* k, const void* a, const void* k_k, const void* k_a,
                             const void* gk_out, const void* ga_out, const void* gb_out,
                             void* gk, void* ga, float* gk_k, float* gk_a);
int hiprwkv_rwkv7_postmix_bwd(hiprwkv_stream stream, int io_dtype, int64_t rows, int64_t H, int64_t N,
                              const void* y, const void* r, const void* k, const void* v, const void* g,
                              const void* ln_w, const void* ln_b, const void* r_k, float eps, const void* gout,
                              void* gy, void* gr, void* gk, void* gv, void* gg,
                              float* gln_w, float* gln_b, float* gr_k);

#ifdef __cplusplus
}
#endif
#endif /* HIPRWKV_H_ */
