"""Host-side operators over device tensors: thin, allocation + pointer plumbing around the C ABI.

Tensors are ``torch`` CUDA tensors (torch is used for device memory and streams only).  Every operator takes a
leading batch axis ``B`` -- what the reference gets from ``jax.vmap`` (rwkv7.py:419-431) -- and enqueues on the
current stream.  ``compat=True`` (default) reproduces ``AssociativeScanRWKV``; ``compat=False`` the sequential
``BaseRWKV``/``ScanRWKV`` conventions (they differ only in y[t] when new_starts[t+1], and in the returned state
when new_starts[length]).
"""
import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}
_SA_DT = {torch.float32: torch.float32, torch.bfloat16: torch.float16}   # type of the WKV7 forward residual sa


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _dev(x, dtype=None):
    if not x.is_cuda:
        raise _lib.HipRwkvError("hiprwkv operators need CUDA (ROCm) tensors; there is no CPU path")
    if dtype is not None and x.dtype != dtype:
        x = x.to(dtype)
    return x.contiguous()


# Placement of the (B,T,H,N) arrays one call touches.  Rows of different arrays at the same (token, head) are accessed
# together; when the arrays' base addresses are congruent modulo 1 KiB (any two large allocations of a caching
# allocator are: they start on 2 MiB boundaries) those rows compete for the same part of the memory system, and the
# write streams suffer most.  Measured on MI355X at B8 T4096 H32: the WKV7 forward with its residual 303 us with every
# array on a 2 MiB boundary, 284 us with the two outputs 128 and 256 bytes past one, 265 us with the inputs staggered
# as well; forward + backward 1619 / 1535 / 1469 us.  Offsets that are multiples of 1 KiB change nothing.  The operators
# therefore put every large array they allocate themselves at its own 128-byte step past the phase of the first input.
_PHASE_BYTES, _PHASES, _PHASED_MIN_BYTES = 128, 8, 1 << 20


def _phase(t):
    return (t.data_ptr() // _PHASE_BYTES) % _PHASES


def _empty_phased(shape, dtype, device, phase):
    """An uninitialised contiguous tensor whose address is ``phase`` 128-byte steps past a 1 KiB boundary (a view
    into a buffer 1 KiB larger); small tensors are allocated plainly."""
    n = torch.empty((), dtype=dtype).element_size()
    for d in shape:
        n *= int(d)
    if n < _PHASED_MIN_BYTES:
        return torch.empty(shape, dtype=dtype, device=device)
    buf = torch.empty(n + _PHASE_BYTES * _PHASES, dtype=torch.uint8, device=device)
    off = ((phase % _PHASES) * _PHASE_BYTES - buf.data_ptr()) % (_PHASE_BYTES * _PHASES)
    return buf[off:off + n].view(dtype).view(*shape)


def _empty_like_phased(ref, steps):
    """Like ``torch.empty_like(ref)``, ``steps`` 128-byte phases past ``ref``'s own."""
    return _empty_phased(tuple(ref.shape), ref.dtype, ref.device, _phase(ref) + steps)


def _length_ns(length, new_starts, B, T, device):
    if length is not None:
        length = torch.as_tensor(length, device=device).to(torch.int32).reshape(-1)
        if length.numel() == 1 and B > 1:
            length = length.expand(B)
        length = length.clamp(min=0).contiguous()
        assert length.numel() == B
    if new_starts is not None:
        new_starts = torch.as_tensor(new_starts, device=device).to(torch.bool)
        if new_starts.dim() == 1:
            new_starts = new_starts[None].expand(B, T)
        new_starts = new_starts.contiguous()
        assert new_starts.shape == (B, T)
    return length, new_starts


def _flags(compat, force_seq=False, small_t=True, debug=0):
    return ((_lib.COMPAT_ASSOC if compat else 0) | (_lib.FORCE_SEQ if force_seq else 0)
            | (0 if small_t else _lib.NO_SMALL_T) | int(debug))


def handshake_failures():
    """Workgroups of the chunked kernels whose bounded hand-shake wait ran out since the library was loaded (their
    outputs are NaN).  Synchronises the current stream."""
    lib = _lib.load()
    n = ctypes.c_uint(0)
    _lib.check(lib.hiprwkv_handshake_failures(_stream(), ctypes.byref(n)), "hiprwkv_handshake_failures")
    return int(n.value)


def numeric_events():
    """Numeric events of the chunked kernels since the library was loaded: waves that capped a channel's decay over a
    chunk at e^-80 (its result is then inexact) and waves that found inf or NaN in a carried state of the bf16
    forward kernels (an IEEE-half operand overflowed: |state|, |sa|, |v| beyond 65504).  Synchronises the current
    stream."""
    lib = _lib.load()
    n = ctypes.c_uint(0)
    _lib.check(lib.hiprwkv_numeric_events(_stream(), ctypes.byref(n)), "hiprwkv_numeric_events")
    return int(n.value)


# ----------------------------------------------------------------------------- WKV7
def wkv7_fwd(r, w, k, v, a, b, s, length=None, new_starts=None, compat=True, want_sa=False, force_seq=False,
             small_t=True, debug_flags=0):
    """r,w,k,v,a,b (B,T,H,N) fp32|bf16; s (B,H,N,N) fp32|bf16.  Returns (new_s, y, sa|None); ``sa`` is fp32 for fp32
    inputs and fp16 for bf16 inputs.

    T <= 8 runs on the small-T (decode) kernel unless ``small_t=False``; otherwise on a chunked matrix-core kernel
    (fp16 operands for bf16 I/O, fp32 operands for fp32 I/O); ``force_seq`` selects the sequential fp32 kernel."""
    lib = _lib.load()
    io = r.dtype
    r, w, k, v, a, b = (_dev(x, io) for x in (r, w, k, v, a, b))
    s = _dev(s)
    B, T, H, N = r.shape
    assert s.shape == (B, H, N, N), (s.shape, r.shape)
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    y = _empty_like_phased(r, 1)
    new_s = torch.empty_like(s)
    # the residual for the backward pass: fp32 beside fp32 I/O, fp16 beside bf16 I/O
    sa = _empty_phased((B, T, H, N), _SA_DT[io], r.device, _phase(r) + 2) if want_sa else None
    rc = lib.hiprwkv_wkv7_fwd(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(w), _p(r), _p(k), _p(v), _p(a), _p(b),
                              _p(s), _p(length), _p(new_starts), _p(y), _p(sa), _p(new_s),
                              _flags(compat, force_seq, small_t, debug_flags))
    _lib.check(rc, "hiprwkv_wkv7_fwd")
    return new_s, y, sa


def _packed_state(t, B, H, N):
    """(pointer tensor, batch stride in elements) of a state view whose sequences are H*N*N contiguous elements each."""
    assert t.is_cuda and t.shape[0] == B and t[0].numel() == H * N * N, (t.shape, (B, H, N))
    assert t[0].is_contiguous(), "a sequence's state must be contiguous"
    return t, (t.stride(0) if B > 1 else H * N * N)


def wkv7_step(r, w, k, v, a, b, s, new_s, length=None, new_starts=None, compat=True):
    """A decode step (T <= 8) on states inside a packed model state: ``s`` and ``new_s`` are views with a batch axis in
    front and H*N*N contiguous elements per sequence, e.g. ``state[:, layer, 2:]`` of a ``(B, L, 2+N, C)`` model state
    (rwkv7.py:176-180, 254-260); ``new_s`` is written in place (it may be ``s``).  Returns y.  No autograd."""
    lib = _lib.load()
    io = r.dtype
    r, w, k, v, a, b = (_dev(x, io) for x in (r, w, k, v, a, b))
    B, T, H, N = r.shape
    s, s_stride = _packed_state(s, B, H, N)
    new_s, ns_stride = _packed_state(new_s, B, H, N)
    assert s.dtype == new_s.dtype
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    y = torch.empty_like(r)
    rc = lib.hiprwkv_wkv7_step(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(w), _p(r), _p(k), _p(v), _p(a), _p(b),
                               _p(s), s_stride, _p(length), _p(new_starts), _p(y), _p(new_s), ns_stride,
                               _flags(compat, False, True, 0))
    _lib.check(rc, "hiprwkv_wkv7_step")
    return y


def wkv7_bwd(r, w, k, v, a, b, s, length, new_starts, gy, sa, gs_out=None, compat=True, force_seq=False,
             debug_flags=0):
    """Cotangents (gr, gw, gk, gv, ga, gb, gs) of ``wkv7_fwd`` for cotangents gy of y and gs_out of new_s.

    bf16 inputs use the chunked MFMA kernels where they exist unless ``force_seq`` asks for the sequential ones."""
    lib = _lib.load()
    io = r.dtype
    r, w, k, v, a, b, gy = (_dev(x, io) for x in (r, w, k, v, a, b, gy))
    s = _dev(s)
    sa = _dev(sa, _SA_DT[io])
    gs_out = None if gs_out is None else _dev(gs_out, s.dtype)
    B, T, H, N = r.shape
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    gw, gr, gk, gv, ga, gb = (_empty_like_phased(r, i) for i in range(1, 7))
    gs = torch.empty_like(s)
    nbytes = lib.hiprwkv_wkv7_bwd_workspace_bytes(B, T, H, N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=r.device)
    rc = lib.hiprwkv_wkv7_bwd(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(w), _p(r), _p(k), _p(v), _p(a), _p(b),
                              _p(s), _p(length), _p(new_starts), _p(gy), _p(sa), _p(gs_out),
                              _p(gw), _p(gr), _p(gk), _p(gv), _p(ga), _p(gb), _p(gs), _p(ws), nbytes,
                              _flags(compat, force_seq, debug=debug_flags))
    _lib.check(rc, "hiprwkv_wkv7_bwd")
    return gr, gw, gk, gv, ga, gb, gs


class _Wkv7(torch.autograd.Function):
    """custom VJP, the counterpart of ``wkv7_cuda`` (rwkv7.py:442-446)."""

    @staticmethod
    def forward(ctx, r, w, k, v, a, b, s, length, new_starts, compat, force_seq):
        need = any(x.requires_grad for x in (r, w, k, v, a, b, s))
        new_s, y, sa = wkv7_fwd(r, w, k, v, a, b, s, length, new_starts, compat, want_sa=need, force_seq=force_seq)
        ctx.compat = compat
        ctx.force_seq = force_seq
        ctx.save_for_backward(r, w, k, v, a, b, s, length, new_starts, sa)
        return new_s, y

    @staticmethod
    def backward(ctx, gs_out, gy):
        r, w, k, v, a, b, s, length, new_starts, sa = ctx.saved_tensors
        if gy is None:
            gy = torch.zeros_like(r)
        gr, gw, gk, gv, ga, gb, gs = wkv7_bwd(r, w, k, v, a, b, s, length, new_starts, gy, sa, gs_out, ctx.compat,
                                              ctx.force_seq)
        return gr, gw, gk, gv, ga, gb, gs, None, None, None, None


def wkv7(r, w, k, v, a, b, s, length=None, new_starts=None, compat=True, force_seq=False):
    """Differentiable WKV7: returns (new_s, y).  ``force_seq`` runs the sequential fp32 kernels whatever the dtype."""
    B, T = r.shape[:2]
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    return _Wkv7.apply(r, w, k, v, a, b, s, length, new_starts, compat, force_seq)


# ----------------------------------------------------------------------------- WKV6
def wkv6_fwd(r, k, v, w, u, s, length=None, new_starts=None, compat=True, force_seq=False, small_t=True,
             debug_flags=0):
    """r,k,v (B,T,H,N); w (B,T,H,N), or (H,N) for a log decay shared by all tokens (RWKV-5); u (H,N);
    s (B,H,N,N) [key, value].  Returns (new_s, y).

    T <= 8 runs on the small-T (decode) kernel unless ``small_t=False``; otherwise bf16 inputs run on the chunked
    MFMA kernel unless ``force_seq`` asks for the sequential fp32 one."""
    lib = _lib.load()
    io = r.dtype
    B, T, H, N = r.shape
    r, k, v = (_dev(x, io) for x in (r, k, v))
    per_head = w.numel() == H * N and (B * T != 1 or w.dim() == 2)
    w = _dev(w.reshape(H, N) if per_head else w.reshape(B, T, H, N), io)
    u = _dev(u.reshape(H, N), io)
    s = _dev(s)
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    y = _empty_like_phased(r, 1)
    new_s = torch.empty_like(s)
    rc = lib.hiprwkv_wkv6_fwd(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(r), _p(k), _p(v), _p(w), _p(u), _p(s),
                              _p(length), _p(new_starts), _p(y), _p(new_s),
                              _flags(compat, force_seq, small_t, debug_flags) | (_lib.W_PER_HEAD if per_head else 0))
    _lib.check(rc, "hiprwkv_wkv6_fwd")
    return new_s, y


def wkv6_step(r, k, v, w, u, s, new_s, length=None, new_starts=None, compat=True):
    """A decode step (T <= 8) on states inside a packed model state: ``s`` and ``new_s`` are views with a batch axis in
    front and H*N*N contiguous elements per sequence (rwkv6.py:221-224); ``new_s`` is written in place (it may be
    ``s``).  ``w`` (B,T,H,N) or the shared (H,N) decay.  Returns y.  No autograd."""
    lib = _lib.load()
    io = r.dtype
    B, T, H, N = r.shape
    r, k, v = (_dev(x, io) for x in (r, k, v))
    per_head = w.numel() == H * N and (B * T != 1 or w.dim() == 2)
    w = _dev(w.reshape(H, N) if per_head else w.reshape(B, T, H, N), io)
    u = _dev(u.reshape(H, N), io)
    s, s_stride = _packed_state(s, B, H, N)
    new_s, ns_stride = _packed_state(new_s, B, H, N)
    assert s.dtype == new_s.dtype
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    y = torch.empty_like(r)
    flags = _flags(compat, False, True, 0) | (_lib.W_PER_HEAD if per_head else 0)
    rc = lib.hiprwkv_wkv6_step(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(r), _p(k), _p(v), _p(w), _p(u), _p(s),
                               s_stride, _p(length), _p(new_starts), _p(y), _p(new_s), ns_stride, flags)
    _lib.check(rc, "hiprwkv_wkv6_step")
    return y


def wkv6_bwd(r, k, v, w, u, s, length, new_starts, gy, gs_out=None, compat=True, force_seq=False, debug_flags=0):
    """Cotangents (gr, gk, gv, gw, gu, gs) of ``wkv6_fwd``; gu is summed over the batch here, and so is gw over batch
    and tokens when ``w`` is the shared (H,N) decay.

    bf16 inputs run on the chunked MFMA kernels unless ``force_seq`` asks for the sequential fp32 ones."""
    lib = _lib.load()
    io = r.dtype
    B, T, H, N = r.shape
    r, k, v, gy = (_dev(x, io) for x in (r, k, v, gy))
    per_head = w.numel() == H * N and (B * T != 1 or w.dim() == 2)
    w = _dev(w.reshape(H, N) if per_head else w.reshape(B, T, H, N), io)
    u = _dev(u.reshape(H, N), io)
    s = _dev(s)
    gs_out = None if gs_out is None else _dev(gs_out, s.dtype)
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    gr, gk, gv, gw = (_empty_like_phased(r, i) for i in range(1, 5))
    gu = torch.empty((B, H, N), dtype=torch.float32, device=r.device)
    gs = torch.empty_like(s)
    nbytes = lib.hiprwkv_wkv6_bwd_workspace_bytes(B, T, H, N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=r.device)
    rc = lib.hiprwkv_wkv6_bwd(_stream(), _DT[io], _DT[s.dtype], B, T, H, N, _p(r), _p(k), _p(v), _p(w), _p(u), _p(s),
                              _p(length), _p(new_starts), _p(gy), _p(gs_out), _p(gr), _p(gk), _p(gv), _p(gw), _p(gu),
                              _p(gs), _p(ws), nbytes,
                              _flags(compat, force_seq, debug=debug_flags) | (_lib.W_PER_HEAD if per_head else 0))
    _lib.check(rc, "hiprwkv_wkv6_bwd")
    if per_head:
        gw = gw.float().sum((0, 1)).to(io)
    return gr, gk, gv, gw, gu.sum(0).to(io), gs


class _Wkv6(torch.autograd.Function):
    @staticmethod
    def forward(ctx, r, k, v, w, u, s, length, new_starts, compat, force_seq):
        new_s, y = wkv6_fwd(r, k, v, w, u, s, length, new_starts, compat, force_seq=force_seq)
        ctx.compat = compat
        ctx.force_seq = force_seq
        ctx.shapes = (w.shape, u.shape)
        ctx.save_for_backward(r, k, v, w, u, s, length, new_starts)
        return new_s, y

    @staticmethod
    def backward(ctx, gs_out, gy):
        r, k, v, w, u, s, length, new_starts = ctx.saved_tensors
        if gy is None:
            gy = torch.zeros_like(r)
        gr, gk, gv, gw, gu, gs = wkv6_bwd(r, k, v, w, u, s, length, new_starts, gy, gs_out, ctx.compat, ctx.force_seq)
        return gr, gk, gv, gw.reshape(ctx.shapes[0]), gu.reshape(ctx.shapes[1]), gs, None, None, None, None


def wkv6(r, k, v, w, u, s, length=None, new_starts=None, compat=True, force_seq=False):
    """Differentiable WKV6: returns (new_s, y).  ``force_seq`` runs the sequential fp32 kernels whatever the dtype."""
    B, T = r.shape[:2]
    length, new_starts = _length_ns(length, new_starts, B, T, r.device)
    return _Wkv6.apply(r, k, v, w, u, s, length, new_starts, compat, force_seq)


# ----------------------------------------------------------------------------- WKV4
def wkv4_fwd(w_neg, u, k, v, s, length=None, new_starts=None, compat=True, want_ckpt=False):
    """w_neg = -exp(time_decay), u (C,); k,v (B,T,C); s (B,3,C).  Returns (new_s, wkv) -- receptance not applied.
    ``want_ckpt``: also return the checkpoint workspace that ``wkv4_bwd(..., ckpt=)`` takes (the state entering every
    16th step), so that the backward pass need not recompute it."""
    lib = _lib.load()
    io = k.dtype
    k, v, s, w_neg, u = (_dev(x, io) for x in (k, v, s, w_neg, u))
    B, T, C = k.shape
    assert s.shape == (B, 3, C) and w_neg.shape == (C,) and u.shape == (C,)
    length, new_starts = _length_ns(length, new_starts, B, T, k.device)
    y = torch.empty_like(k)
    new_s = torch.empty_like(s)
    if want_ckpt:
        nbytes = lib.hiprwkv_wkv4_bwd_workspace_bytes(B, T, C)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=k.device)
        rc = lib.hiprwkv_wkv4_fwd_ckpt(_stream(), _DT[io], B, T, C, _p(w_neg), _p(u), _p(k), _p(v), _p(s), _p(length),
                                       _p(new_starts), _p(new_s), _p(y), _p(ws), nbytes, _flags(compat))
        _lib.check(rc, "hiprwkv_wkv4_fwd_ckpt")
        return new_s, y, ws
    rc = lib.hiprwkv_wkv4_fwd(_stream(), _DT[io], B, T, C, _p(w_neg), _p(u), _p(k), _p(v), _p(s), _p(length),
                              _p(new_starts), _p(new_s), _p(y), _flags(compat))
    _lib.check(rc, "hiprwkv_wkv4_fwd")
    return new_s, y


def wkv4_bwd(w_neg, u, k, v, s, length, new_starts, gy, gs_new=None, compat=True, ckpt=None):
    """Cotangents (gw, gu, gk, gv, gs) of ``wkv4_fwd``; gw, gu are summed over the batch here (rwkv4.py:351).
    ``ckpt``: the workspace ``wkv4_fwd(..., want_ckpt=True)`` returned for the same inputs."""
    lib = _lib.load()
    io = k.dtype
    k, v, s, w_neg, u, gy = (_dev(x, io) for x in (k, v, s, w_neg, u, gy))
    gs_new = None if gs_new is None else _dev(gs_new, io)
    B, T, C = k.shape
    length, new_starts = _length_ns(length, new_starts, B, T, k.device)
    gk, gv = torch.empty_like(k), torch.empty_like(v)
    gs = torch.empty_like(s)
    gw = torch.empty((B, C), dtype=torch.float32, device=k.device)
    gu = torch.empty((B, C), dtype=torch.float32, device=k.device)
    nbytes = lib.hiprwkv_wkv4_bwd_workspace_bytes(B, T, C)
    if ckpt is None:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=k.device)
    else:
        ws = ckpt
        assert ws.dtype == torch.uint8 and ws.numel() >= nbytes and ws.is_cuda
    rc = lib.hiprwkv_wkv4_bwd(_stream(), _DT[io], B, T, C, _p(w_neg), _p(u), _p(k), _p(v), _p(gy), _p(s), _p(length),
                              _p(new_starts), _p(gs_new), _p(gw), _p(gu), _p(gk), _p(gv), _p(gs), _p(ws), nbytes,
                              _flags(compat) | (0 if ckpt is None else _lib.CKPT_READY))
    _lib.check(rc, "hiprwkv_wkv4_bwd")
    return gw.sum(0).to(io), gu.sum(0).to(io), gk, gv, gs


class _Wkv4(torch.autograd.Function):
    """custom VJP, the counterpart of ``wkv4_cuda`` (rwkv4.py:379-383)."""

    @staticmethod
    def forward(ctx, w_neg, u, k, v, s, length, new_starts, compat):
        new_s, y, ckpt = wkv4_fwd(w_neg, u, k, v, s, length, new_starts, compat, want_ckpt=True)
        ctx.compat = compat
        ctx.save_for_backward(w_neg, u, k, v, s, length, new_starts, ckpt)
        return new_s, y

    @staticmethod
    def backward(ctx, gs_new, gy):
        w_neg, u, k, v, s, length, new_starts, ckpt = ctx.saved_tensors
        if gy is None:
            gy = torch.zeros_like(k)
        gw, gu, gk, gv, gs = wkv4_bwd(w_neg, u, k, v, s, length, new_starts, gy, gs_new, ctx.compat, ckpt=ckpt)
        return gw, gu, gk, gv, gs, None, None, None


def wkv4(w_neg, u, k, v, s, length=None, new_starts=None, compat=True):
    """Differentiable WKV4 in the op's convention (w_neg = -exp(time_decay), no receptance): returns (new_s, wkv)."""
    B, T = k.shape[:2]
    length, new_starts = _length_ns(length, new_starts, B, T, k.device)
    return _Wkv4.apply(w_neg, u, k, v, s, length, new_starts, compat)


# ----------------------------------------------------------------------------- RWKV-7 time-mixing stages
def _premix_fwd(k, a, k_k, k_a):
    lib = _lib.load()
    io = k.dtype
    H, N = k.shape[-2:]
    rows = k.numel() // (H * N)
    k_out, a_out, b_out = (torch.empty_like(k) for _ in range(3))
    rc = lib.hiprwkv_rwkv7_premix(_stream(), _DT[io], rows, H, N, _p(k), _p(a), _p(k_k), _p(k_a), _p(k_out), _p(a_out),
                                  _p(b_out))
    _lib.check(rc, "hiprwkv_rwkv7_premix")
    return k_out, a_out, b_out


def _postmix_fwd(y, r, k, v, g, ln_w, ln_b, r_k, eps):
    lib = _lib.load()
    io = y.dtype
    H, N = y.shape[-2:]
    rows = y.numel() // (H * N)
    out = torch.empty_like(y)
    rc = lib.hiprwkv_rwkv7_postmix(_stream(), _DT[io], rows, H, N, _p(y), _p(r), _p(k), _p(v), _p(g), _p(ln_w), _p(ln_b),
                                   _p(r_k), float(eps), _p(out))
    _lib.check(rc, "hiprwkv_rwkv7_postmix")
    return out


class _Premix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, k, a, k_k, k_a):
        ctx.save_for_backward(k, a, k_k, k_a)
        return _premix_fwd(k, a, k_k, k_a)

    @staticmethod
    def backward(ctx, gk_out, ga_out, gb_out):
        k, a, k_k, k_a = ctx.saved_tensors
        lib = _lib.load()
        io = k.dtype
        H, N = k.shape[-2:]
        rows = k.numel() // (H * N)
        gk_out, ga_out, gb_out = (_dev(x, io) for x in (gk_out, ga_out, gb_out))
        gk, ga = torch.empty_like(k), torch.empty_like(a)
        gk_k, gk_a = (torch.empty(H, N, dtype=torch.float32, device=k.device) for _ in range(2))
        rc = lib.hiprwkv_rwkv7_premix_bwd(_stream(), _DT[io], rows, H, N, _p(k), _p(a), _p(k_k), _p(k_a), _p(gk_out),
                                          _p(ga_out), _p(gb_out), _p(gk), _p(ga), _p(gk_k), _p(gk_a))
        _lib.check(rc, "hiprwkv_rwkv7_premix_bwd")
        return gk, ga, gk_k.to(io), gk_a.to(io)


class _Postmix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, r, k, v, g, ln_w, ln_b, r_k, eps):
        ctx.save_for_backward(y, r, k, v, g, ln_w, ln_b, r_k)
        ctx.eps = eps
        return _postmix_fwd(y, r, k, v, g, ln_w, ln_b, r_k, eps)

    @staticmethod
    def backward(ctx, gout):
        y, r, k, v, g, ln_w, ln_b, r_k = ctx.saved_tensors
        lib = _lib.load()
        io = y.dtype
        H, N = y.shape[-2:]
        rows = y.numel() // (H * N)
        gout = _dev(gout, io)
        gy, gr, gk, gv, gg = (torch.empty_like(y) for _ in range(5))
        gw, gb, grk = (torch.empty(H, N, dtype=torch.float32, device=y.device) for _ in range(3))
        rc = lib.hiprwkv_rwkv7_postmix_bwd(_stream(), _DT[io], rows, H, N, _p(y), _p(r), _p(k), _p(v), _p(g), _p(ln_w),
                                           _p(ln_b), _p(r_k), float(ctx.eps), _p(gout), _p(gy), _p(gr), _p(gk), _p(gv),
                                           _p(gg), _p(gw), _p(gb), _p(grk))
        _lib.check(rc, "hiprwkv_rwkv7_postmix_bwd")
        return gy, gr, gk, gv, gg, gw.to(io), gb.to(io), grk.to(io), None


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _shift_row(prev, B, C, io):
    """The token before t = 0 of every sequence as (tensor, batch stride in elements): rows of C contiguous elements,
    read where they lie when the stride allows it (a row of the packed model state), else from a dense copy."""
    assert prev.shape == (B, C), (prev.shape, (B, C))
    if not prev.is_cuda:
        raise _lib.HipRwkvError("hiprwkv operators need CUDA (ROCm) tensors; there is no CPU path")
    elem = 4 if io == torch.float32 else 2
    ok = (prev.dtype == io and (C == 1 or prev.stride(1) == 1) and prev.data_ptr() % 16 == 0
          and (B == 1 or (prev.stride(0) >= C and (prev.stride(0) * elem) % 16 == 0)))
    if not ok:
        prev = prev.to(io).contiguous()
    return prev, (prev.stride(0) if B > 1 else C)


def _shiftmix_fwd(x, prev, prev_stride, ns, mix):
    lib = _lib.load()
    io = x.dtype
    B, T, C = x.shape
    outs = [torch.empty_like(x) for _ in mix]
    rc = lib.hiprwkv_rwkv7_shiftmix(_stream(), _DT[io], B, T, C, len(mix), _p(x), _p(prev), prev_stride, _p(ns),
                                    _ptr_array(mix), _ptr_array(outs))
    _lib.check(rc, "hiprwkv_rwkv7_shiftmix")
    return tuple(outs)


class _ShiftMix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, prev, ns, *mix):
        prev_t, stride = _shift_row(prev, x.shape[0], x.shape[2], x.dtype)
        ctx.save_for_backward(x, prev_t, *mix)
        ctx.ns, ctx.stride = ns, stride
        return _shiftmix_fwd(x, prev_t, stride, ns, mix)

    @staticmethod
    def backward(ctx, *gs):
        x, prev, *mix = ctx.saved_tensors
        lib = _lib.load()
        io = x.dtype
        B, T, C = x.shape
        gs = [_dev(g, io) for g in gs]
        dx = torch.empty_like(x)
        dprev = torch.empty((B, C), dtype=io, device=x.device)
        dmix = torch.empty((len(mix), C), dtype=torch.float32, device=x.device)
        rc = lib.hiprwkv_rwkv7_shiftmix_bwd(_stream(), _DT[io], B, T, C, len(mix), _p(x), _p(prev), ctx.stride,
                                            _p(ctx.ns), _ptr_array(mix), _ptr_array(gs), _p(dx), _p(dprev), C, _p(dmix))
        _lib.check(rc, "hiprwkv_rwkv7_shiftmix_bwd")
        return (dx, dprev, None) + tuple(dmix[i].to(io) for i in range(len(mix)))


def rwkv7_shiftmix(x, prev, new_starts, mix):
    """Token shift and interpolation of rwkv7.py:226-235 (six ``mix`` vectors, time mixing) and :192-195 (one, channel
    mixing): x (B,T,C); prev (B,C), the token before t = 0 (a row of the model state; read in place);
    new_starts (B,T) bool or None; mix a list of (C,) parameters.  Returns the tuple of x + sx*mix_i with
    sx = (new_starts ? 0 : previous token) - x.  Differentiable in x, prev and the mix vectors."""
    io = x.dtype
    B, T, C = x.shape
    assert len(mix) in (1, 6) and C % 8 == 0, (len(mix), C)
    x = _dev(x, io)
    mix2 = [_dev(m.reshape(C), io) for m in mix]
    _, ns = _length_ns(None, new_starts, B, T, x.device)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x, prev, *mix)):
        return _ShiftMix.apply(x, prev, ns, *mix2)
    prev_t, stride = _shift_row(prev, B, C, io)
    return _shiftmix_fwd(x, prev_t, stride, ns, mix2)


def _gate_fwd(x, p, kind):
    lib = _lib.load()
    io = x.dtype
    C = x.shape[-1]
    out = torch.empty_like(x)
    fn = (lib.hiprwkv_rwkv7_decay, lib.hiprwkv_rwkv7_agate)[kind]
    _lib.check(fn(_stream(), _DT[io], x.numel() // C, C, _p(x), _p(p), _p(out)), "hiprwkv_rwkv7_" + ("decay", "agate")[kind])
    return out


class _Gate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, p, kind):
        ctx.save_for_backward(x, p)
        ctx.kind = kind
        return _gate_fwd(x, p, kind)

    @staticmethod
    def backward(ctx, g):
        x, p = ctx.saved_tensors
        lib = _lib.load()
        io = x.dtype
        C = x.shape[-1]
        g = _dev(g, io)
        dx = torch.empty_like(x)
        dp = torch.empty(C, dtype=torch.float32, device=x.device)
        fn = (lib.hiprwkv_rwkv7_decay_bwd, lib.hiprwkv_rwkv7_agate_bwd)[ctx.kind]
        _lib.check(fn(_stream(), _DT[io], x.numel() // C, C, _p(x), _p(p), _p(g), _p(dx), _p(dp)),
                   "hiprwkv_rwkv7_" + ("decay", "agate")[ctx.kind] + "_bwd")
        return dx, dp.to(io), None


def _gate(x, p, kind):
    io = x.dtype
    C = x.shape[-1]
    assert C % 8 == 0, C
    x, p2 = _dev(x, io), _dev(p.reshape(C), io)
    if torch.is_grad_enabled() and (x.requires_grad or p.requires_grad):
        return _Gate.apply(x, p2, kind)
    return _gate_fwd(x, p2, kind)


def rwkv7_decay(x, w0):
    """The decay argument of the WKV op, rwkv7.py:237: ``-softplus(-(w0 + x)) - 0.5`` for x (..., C) (the low-rank
    term ``tanh(xw w1) w2``) and the parameter w0 (C,).  Differentiable in both."""
    return _gate(x, w0, 0)


def rwkv7_agate(x, a0):
    """The in-context learning rate, rwkv7.py:244: ``sigmoid(a0 + x)`` for x (..., C) and a0 (C,).  Differentiable."""
    return _gate(x, a0, 1)


def _relusq_fwd(x):
    out = torch.empty_like(x)
    rc = _lib.load().hiprwkv_rwkv7_relusq(_stream(), _DT[x.dtype], x.numel(), _p(x), _p(out))
    _lib.check(rc, "hiprwkv_rwkv7_relusq")
    return out


class _ReluSq(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return _relusq_fwd(x)

    @staticmethod
    def backward(ctx, g):
        x, = ctx.saved_tensors
        g = _dev(g, x.dtype)
        dx = torch.empty_like(x)
        rc = _lib.load().hiprwkv_rwkv7_relusq_bwd(_stream(), _DT[x.dtype], x.numel(), _p(x), _p(g), _p(dx))
        _lib.check(rc, "hiprwkv_rwkv7_relusq_bwd")
        return dx


def rwkv7_relusq(x):
    """Channel mixing's activation, rwkv7.py:196: ``relu(x)**2`` in one pass; differentiable.  numel a multiple of 8."""
    assert x.numel() % 8 == 0, x.shape
    x = _dev(x, x.dtype)
    if torch.is_grad_enabled() and x.requires_grad:
        return _ReluSq.apply(x)
    return _relusq_fwd(x)


def _vmix_fwd(v, vf, x, v0):
    lib = _lib.load()
    io = v.dtype
    C = v.shape[-1]
    out = torch.empty_like(v)
    rc = lib.hiprwkv_rwkv7_vmix(_stream(), _DT[io], v.numel() // C, C, _p(v), _p(vf), _p(x), _p(v0), _p(out))
    _lib.check(rc, "hiprwkv_rwkv7_vmix")
    return out


class _VMix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, v, vf, x, v0):
        ctx.save_for_backward(v, vf, x, v0)
        return _vmix_fwd(v, vf, x, v0)

    @staticmethod
    def backward(ctx, g):
        v, vf, x, v0 = ctx.saved_tensors
        lib = _lib.load()
        io = v.dtype
        C = v.shape[-1]
        g = _dev(g, io)
        dv, dvf, dx = (torch.empty_like(v) for _ in range(3))
        dv0 = torch.empty(C, dtype=torch.float32, device=v.device)
        rc = lib.hiprwkv_rwkv7_vmix_bwd(_stream(), _DT[io], v.numel() // C, C, _p(v), _p(vf), _p(x), _p(v0), _p(g),
                                        _p(dv), _p(dvf), _p(dx), _p(dv0))
        _lib.check(rc, "hiprwkv_rwkv7_vmix_bwd")
        return dv, dvf, dx, dv0.to(io)


def rwkv7_vmix(v, v_first, x, v0):
    """The value residual of the layers after the first, rwkv7.py:241-242: ``v + (v_first - v) sigmoid(v0 + x)`` for
    v, v_first, x (..., C) (x the low-rank term ``(xv v1) v2``) and the parameter v0 (C,).  Differentiable in all four."""
    io = v.dtype
    C = v.shape[-1]
    assert C % 8 == 0, C
    v, vf, x = (_dev(t, io) for t in (v, v_first, x))
    v02 = _dev(v0.reshape(C), io)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (v, v_first, x, v0)):
        return _VMix.apply(v, vf, x, v02)
    return _vmix_fwd(v, vf, x, v02)


def rwkv7_premix(k, a, k_k, k_a):
    """k, a (..., H, N); k_k, k_a (H, N) or (H*N,).  Returns (k', a_i, b_i) of rwkv7.py:248-252, 257:
    kk = normalize_head(k k_k), k' = k (1 + (a - 1) k_a), a_i = -kk, b_i = kk a.  Differentiable in all four inputs
    (the backward kernel recomputes kk; parameter cotangents are summed over the tokens in fp32)."""
    io = k.dtype
    H, N = k.shape[-2:]
    k, a = _dev(k, io), _dev(a, io)
    k_k2, k_a2 = _dev(k_k.reshape(H, N), io), _dev(k_a.reshape(H, N), io)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (k, a, k_k, k_a)):
        return _Premix.apply(k, a, k_k2, k_a2)
    return _premix_fwd(k, a, k_k2, k_a2)


def rwkv7_postmix(y, r, k, v, g, ln_w, ln_b, r_k, eps=64e-5):
    """y, r, k, v, g (..., H, N); ln_w, ln_b, r_k (H, N) or (H*N,).  Returns
    (group_norm_head(y) ln_w + ln_b + (r.k.r_k) v) g of rwkv7.py:263-265.  Differentiable in all eight tensors."""
    io = y.dtype
    H, N = y.shape[-2:]
    y, r, k, v, g = (_dev(x, io) for x in (y, r, k, v, g))
    ln_w2, ln_b2, r_k2 = (_dev(x.reshape(H, N), io) for x in (ln_w, ln_b, r_k))
    if torch.is_grad_enabled() and any(t.requires_grad for t in (y, r, k, v, g, ln_w, ln_b, r_k)):
        return _Postmix.apply(y, r, k, v, g, ln_w2, ln_b2, r_k2, eps)
    return _postmix_fwd(y, r, k, v, g, ln_w2, ln_b2, r_k2, eps)
