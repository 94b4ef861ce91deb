// XLA FFI handlers over the C ABI of libhiprwkv (include/hiprwkv.h): what `jax.ffi.register_ffi_target` binds on the
// "ROCM" platform.  They replace the symbols the reference loads from its CUDA library
// (`WKV7FwdBF16` ... /root/reference/src/jaxrwkv/rwkv7.py:459-465, `WKV4FwdBF16` ... rwkv4.py:394-400) and add
// WKV6, which the reference has no native op for.
//
// Built only where XLA's FFI headers exist (`python -m jaxrwkv_amd.build --xla-ffi`, include path from
// `jax.ffi.include_dir()`); the rest of the library does not depend on it.
//
// Conventions.  One handler per op, for both dtypes (read from the buffers).  Every leading dimension in front of
// (T, H, N) [WKV4: (T, C)] is one flat batch.  The per-model parameters (WKV6 u (H,N); WKV4 w, u (C,)) must arrive
// at exactly that rank: the C ABI reads one set per call, so a parameter that carries batch dimensions (a vmap that
// broadcast it, or per-example parameters) is refused instead of being read wrongly; the Python binding keeps them
// un-batched with a custom_vmap rule.  Element types are checked against r (k for WKV4): the token operands must
// agree, and the WKV7 residual `sa` is F32 beside F32 I/O and F16 beside BF16 I/O (the reference's sa_restore is F32
// for both, rwkv7.py:364).  XLA owns all buffers: residuals and scratch are results.  A handler only enqueues on the
// stream XLA passes in; it never allocates or synchronises.  Attribute `flags` carries HIPRWKV_COMPAT_ASSOC etc.;
// bits outside HIPRWKV_PUBLIC_FLAGS (the debug hook) are dropped.
#include <cstdint>

#include <hip/hip_runtime.h>

#include "../../include/hiprwkv.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

int dtype_of(ffi::DataType t) { return t == ffi::F32 ? HIPRWKV_F32 : t == ffi::BF16 ? HIPRWKV_BF16 : -1; }

// (batch..., T, H, N) -> B, T, H, N
bool split_thn(ffi::Span<const int64_t> d, int64_t& B, int64_t& T, int64_t& H, int64_t& N) {
  if (d.size() < 3) return false;
  N = d[d.size() - 1]; H = d[d.size() - 2]; T = d[d.size() - 3];
  B = 1;
  for (size_t i = 0; i + 3 < d.size(); ++i) B *= d[i];
  return true;
}

ffi::Error invalid(const char* msg) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, msg); }

unsigned public_flags(int64_t flags) { return static_cast<unsigned>(flags) & HIPRWKV_PUBLIC_FLAGS; }

// every operand has the element type of the first one
template <typename... Bufs>
bool same_type(const ffi::AnyBuffer& first, const Bufs&... rest) {
  return ((rest.element_type() == first.element_type()) && ...);
}

// the WKV7 residual: F32 beside F32 I/O, F16 (IEEE half) beside BF16 I/O
bool sa_type_ok(ffi::DataType io, ffi::DataType sa) {
  return (io == ffi::F32 && sa == ffi::F32) || (io == ffi::BF16 && sa == ffi::F16);
}

ffi::Error status(int rc) {
  return rc == HIPRWKV_OK ? ffi::Error::Success() : ffi::Error(ffi::ErrorCode::kInvalidArgument, hiprwkv_last_error());
}

// ---- WKV7: operands w,r,k,v,a,b,s,length,new_starts -> out, sa, new_s   (rwkv7.py:372-375 without s_restore)
ffi::Error Wkv7Fwd(hipStream_t stream, ffi::AnyBuffer w, ffi::AnyBuffer r, ffi::AnyBuffer k, ffi::AnyBuffer v,
                   ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length,
                   ffi::Buffer<ffi::PRED> new_starts, ffi::Result<ffi::AnyBuffer> out,
                   ffi::Result<ffi::AnyBuffer> sa, ffi::Result<ffi::AnyBuffer> new_s, int64_t flags) {
  int64_t B, T, H, N;
  if (!split_thn(r.dimensions(), B, T, H, N)) return invalid("wkv7: rank < 3");
  if (!same_type(r, w, k, v, a, b)) return invalid("wkv7_fwd: w, r, k, v, a, b must have one element type");
  if (!sa_type_ok(r.element_type(), sa->element_type()))
    return invalid("wkv7_fwd: the residual sa must be F32 beside F32 I/O and F16 beside BF16 I/O");
  return status(hiprwkv_wkv7_fwd(stream, dtype_of(r.element_type()), dtype_of(s.element_type()), B, T, H, N,
                                 w.untyped_data(), r.untyped_data(), k.untyped_data(), v.untyped_data(),
                                 a.untyped_data(), b.untyped_data(), s.untyped_data(), length.typed_data(),
                                 reinterpret_cast<const uint8_t*>(new_starts.typed_data()), out->untyped_data(),
                                 sa->untyped_data(), new_s->untyped_data(), public_flags(flags)));
}

// operands w,r,k,v,a,b,s,length,new_starts,gy,sa,gs_out -> gw,gr,gk,gv,ga,gb,gs,workspace   (rwkv7.py:406-408)
ffi::Error Wkv7Bwd(hipStream_t stream, ffi::AnyBuffer w, ffi::AnyBuffer r, ffi::AnyBuffer k, ffi::AnyBuffer v,
                   ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length,
                   ffi::Buffer<ffi::PRED> new_starts, ffi::AnyBuffer gy, ffi::AnyBuffer sa, ffi::AnyBuffer gs_out,
                   ffi::Result<ffi::AnyBuffer> gw, ffi::Result<ffi::AnyBuffer> gr, ffi::Result<ffi::AnyBuffer> gk,
                   ffi::Result<ffi::AnyBuffer> gv, ffi::Result<ffi::AnyBuffer> ga, ffi::Result<ffi::AnyBuffer> gb,
                   ffi::Result<ffi::AnyBuffer> gs, ffi::Result<ffi::Buffer<ffi::U8>> workspace, int64_t flags) {
  int64_t B, T, H, N;
  if (!split_thn(r.dimensions(), B, T, H, N)) return invalid("wkv7: rank < 3");
  if (!same_type(r, w, k, v, a, b, gy)) return invalid("wkv7_bwd: w, r, k, v, a, b, gy must have one element type");
  if (!sa_type_ok(r.element_type(), sa.element_type()))
    return invalid("wkv7_bwd: the residual sa must be F32 beside F32 I/O and F16 beside BF16 I/O (as wkv7_fwd wrote it)");
  return status(hiprwkv_wkv7_bwd(stream, dtype_of(r.element_type()), dtype_of(s.element_type()), B, T, H, N,
                                 w.untyped_data(), r.untyped_data(), k.untyped_data(), v.untyped_data(),
                                 a.untyped_data(), b.untyped_data(), s.untyped_data(), length.typed_data(),
                                 reinterpret_cast<const uint8_t*>(new_starts.typed_data()), gy.untyped_data(),
                                 sa.untyped_data(), gs_out.untyped_data(), gw->untyped_data(), gr->untyped_data(),
                                 gk->untyped_data(), gv->untyped_data(), ga->untyped_data(), gb->untyped_data(),
                                 gs->untyped_data(), workspace->typed_data(), workspace->element_count(),
                                 public_flags(flags)));
}

// ---- WKV6: operands r,k,v,w,u,s,length,new_starts -> out, new_s   (argument order of rwkv6.py:175)
ffi::Error Wkv6Fwd(hipStream_t stream, ffi::AnyBuffer r, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer w,
                   ffi::AnyBuffer u, ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length, ffi::Buffer<ffi::PRED> new_starts,
                   ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> new_s, int64_t flags) {
  int64_t B, T, H, N;
  if (!split_thn(r.dimensions(), B, T, H, N)) return invalid("wkv6: rank < 3");
  if (!same_type(r, k, v, w, u)) return invalid("wkv6_fwd: r, k, v, w, u must have one element type");
  if (u.dimensions().size() != 2 || u.dimensions()[0] != H || u.dimensions()[1] != N)
    return invalid("wkv6_fwd: u must be (H, N), one parameter set per call (it arrived with batch dimensions)");
  return status(hiprwkv_wkv6_fwd(stream, dtype_of(r.element_type()), dtype_of(s.element_type()), B, T, H, N,
                                 r.untyped_data(), k.untyped_data(), v.untyped_data(), w.untyped_data(),
                                 u.untyped_data(), s.untyped_data(), length.typed_data(),
                                 reinterpret_cast<const uint8_t*>(new_starts.typed_data()), out->untyped_data(),
                                 new_s->untyped_data(), public_flags(flags)));
}

// operands r,k,v,w,u,s,length,new_starts,gy,gs_out -> gr,gk,gv,gw,gu (B,H,N) f32,gs,workspace
ffi::Error Wkv6Bwd(hipStream_t stream, ffi::AnyBuffer r, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer w,
                   ffi::AnyBuffer u, ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length, ffi::Buffer<ffi::PRED> new_starts,
                   ffi::AnyBuffer gy, ffi::AnyBuffer gs_out, ffi::Result<ffi::AnyBuffer> gr,
                   ffi::Result<ffi::AnyBuffer> gk, ffi::Result<ffi::AnyBuffer> gv, ffi::Result<ffi::AnyBuffer> gw,
                   ffi::Result<ffi::Buffer<ffi::F32>> gu, ffi::Result<ffi::AnyBuffer> gs,
                   ffi::Result<ffi::Buffer<ffi::U8>> workspace, int64_t flags) {
  int64_t B, T, H, N;
  if (!split_thn(r.dimensions(), B, T, H, N)) return invalid("wkv6: rank < 3");
  if (!same_type(r, k, v, w, u)) return invalid("wkv6_bwd: r, k, v, w, u must have one element type");
  if (u.dimensions().size() != 2 || u.dimensions()[0] != H || u.dimensions()[1] != N)
    return invalid("wkv6_bwd: u must be (H, N), one parameter set per call (it arrived with batch dimensions)");
  return status(hiprwkv_wkv6_bwd(stream, dtype_of(r.element_type()), dtype_of(s.element_type()), B, T, H, N,
                                 r.untyped_data(), k.untyped_data(), v.untyped_data(), w.untyped_data(),
                                 u.untyped_data(), s.untyped_data(), length.typed_data(),
                                 reinterpret_cast<const uint8_t*>(new_starts.typed_data()), gy.untyped_data(),
                                 gs_out.untyped_data(), gr->untyped_data(), gk->untyped_data(), gv->untyped_data(),
                                 gw->untyped_data(), gu->typed_data(), gs->untyped_data(), workspace->typed_data(),
                                 workspace->element_count(), public_flags(flags)));
}

// ---- WKV4: operands w,u,k,v,s,length,new_starts -> new_s, out   (rwkv4.py:320-321)
ffi::Error Wkv4Fwd(hipStream_t stream, ffi::AnyBuffer w, ffi::AnyBuffer u, ffi::AnyBuffer k, ffi::AnyBuffer v,
                   ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length, ffi::Buffer<ffi::PRED> new_starts,
                   ffi::Result<ffi::AnyBuffer> new_s, ffi::Result<ffi::AnyBuffer> out, int64_t flags) {
  auto d = k.dimensions();
  if (d.size() < 2) return invalid("wkv4: rank < 2");
  const int64_t C = d[d.size() - 1], T = d[d.size() - 2];
  int64_t B = 1;
  for (size_t i = 0; i + 2 < d.size(); ++i) B *= d[i];
  if (!same_type(k, w, u, v)) return invalid("wkv4_fwd: w, u, k, v must have one element type");
  if (w.dimensions().size() != 1 || u.dimensions().size() != 1 || w.dimensions()[0] != C || u.dimensions()[0] != C)
    return invalid("wkv4_fwd: w and u must be (C,), one parameter set per call (they arrived with batch dimensions)");
  return status(hiprwkv_wkv4_fwd(stream, dtype_of(k.element_type()), B, T, C, w.untyped_data(), u.untyped_data(),
                                 k.untyped_data(), v.untyped_data(), s.untyped_data(), length.typed_data(),
                                 reinterpret_cast<const uint8_t*>(new_starts.typed_data()), new_s->untyped_data(),
                                 out->untyped_data(), public_flags(flags)));
}

// operands w,u,k,v,gy,s,length,new_starts,gs_new -> gw (B,C) f32, gu (B,C) f32, gk, gv, gs, workspace (rwkv4.py:347-349)
ffi::Error Wkv4Bwd(hipStream_t stream, ffi::AnyBuffer w, ffi::AnyBuffer u, ffi::AnyBuffer k, ffi::AnyBuffer v,
                   ffi::AnyBuffer gy, ffi::AnyBuffer s, ffi::Buffer<ffi::U32> length, ffi::Buffer<ffi::PRED> new_starts,
                   ffi::AnyBuffer gs_new, ffi::Result<ffi::Buffer<ffi::F32>> gw, ffi::Result<ffi::Buffer<ffi::F32>> gu,
                   ffi::Result<ffi::AnyBuffer> gk, ffi::Result<ffi::AnyBuffer> gv, ffi::Result<ffi::AnyBuffer> gs,
                   ffi::Result<ffi::Buffer<ffi::U8>> workspace, int64_t flags) {
  auto d = k.dimensions();
  if (d.size() < 2) return invalid("wkv4: rank < 2");
  const int64_t C = d[d.size() - 1], T = d[d.size() - 2];
  int64_t B = 1;
  for (size_t i = 0; i + 2 < d.size(); ++i) B *= d[i];
  if (!same_type(k, w, u, v)) return invalid("wkv4_bwd: w, u, k, v must have one element type");
  if (w.dimensions().size() != 1 || u.dimensions().size() != 1 || w.dimensions()[0] != C || u.dimensions()[0] != C)
    return invalid("wkv4_bwd: w and u must be (C,), one parameter set per call (they arrived with batch dimensions)");
  return status(hiprwkv_wkv4_bwd(stream, dtype_of(k.element_type()), B, T, C, w.untyped_data(), u.untyped_data(),
                                 k.untyped_data(), v.untyped_data(), gy.untyped_data(), s.untyped_data(),
                                 length.typed_data(), reinterpret_cast<const uint8_t*>(new_starts.typed_data()),
                                 gs_new.untyped_data(), gw->typed_data(), gu->typed_data(), gk->untyped_data(),
                                 gv->untyped_data(), gs->untyped_data(), workspace->typed_data(),
                                 workspace->element_count(), public_flags(flags)));
}

auto Any() { return ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>(); }

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv7Fwd, Wkv7Fwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Attr<int64_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv7Bwd, Wkv7Bwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::Buffer<ffi::U8>>().Attr<int64_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv6Fwd, Wkv6Fwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Attr<int64_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv6Bwd, Wkv6Bwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
        .Ret<ffi::Buffer<ffi::F32>>().Ret<ffi::AnyBuffer>().Ret<ffi::Buffer<ffi::U8>>().Attr<int64_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv4Fwd, Wkv4Fwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Attr<int64_t>("flags"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(HipWkv4Bwd, Wkv4Bwd,
    Any().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>().Arg<ffi::Buffer<ffi::U32>>().Arg<ffi::Buffer<ffi::PRED>>().Arg<ffi::AnyBuffer>()
        .Ret<ffi::Buffer<ffi::F32>>().Ret<ffi::Buffer<ffi::F32>>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>().Ret<ffi::Buffer<ffi::U8>>().Attr<int64_t>("flags"));
