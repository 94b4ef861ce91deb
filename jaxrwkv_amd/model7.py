"""RWKV-7 full-model harness around ``HipRWKV.inner_loop``: the caller of the WKV op, restated over torch tensors.

It mirrors the reference's ``RWKV.forward(params, tokens, state, length=, new_starts=)`` and ``default_state``
(/root/reference/src/jaxrwkv/llm.py:71-84, rwkv7.py:176-198, 223-291) with an explicit leading batch axis (the
reference batches with ``jax.vmap``).  Everything except the recurrence is plain torch (projections, LayerNorm,
token shift, LoRA gates, group norm, channel mix): plumbing that stays in the host framework; the recurrence goes
through ``HipRWKV.inner_loop``.  The parameter tree has the reference's names and stacked-per-layer shapes
(rwkv7.py:81-173) so that a converted checkpoint would drop in; ``randomize_weights`` follows the same schedules and
distributions with torch's generator (the reference's threefry streams cannot be reproduced without jax).

Model state per sequence, as in the reference (rwkv7.py:176-180, 254-260, 283-287): ``(L, 2 + N, C)`` in the
parameter dtype; row 0 = channel-mix token-shift state, row 1 = time-mix token-shift state, rows 2.. = the WKV state
of the layer, a flat reinterpretation of ``(H, N, N)`` [value row, key column].
"""
import math

import torch
import torch.nn.functional as F

from . import ops
from .rwkv7 import HipRWKV

HEAD_SIZE = 64


def layer_norm(x, w, eps=1e-5):
    """rwkv7.py:8-12"""
    return F.layer_norm(x.float(), (x.shape[-1],), w["weight"].float(), w["bias"].float(), eps).to(x.dtype)


def _orthogonal(gen, rows, cols, gain, device):
    """rwkv7.py:26-38: QR of a normal matrix with the sign fix, scaled by gain."""
    flat = torch.randn((max(rows, cols), min(rows, cols)), generator=gen, device=device, dtype=torch.float32)
    q, r = torch.linalg.qr(flat)
    q = q * torch.sign(torch.diagonal(r))[None] * gain
    return q if rows >= cols else q.T


def randomize_weights(seed, n_layer, n_embd, vocab_size, dtype=torch.bfloat16, device="cuda", zero_init=True):
    """Schedules and distributions of rwkv7.py:81-173.  ``zero_init=False`` replaces the zero-initialised matrices
    (output, ffn.value, the first LoRA factors) by small random ones, so that the recurrence reaches the logits --
    used by the parity tests; the reference's init makes every block's contribution vanish."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    L, C, N = n_layer, n_embd, HEAD_SIZE
    H = C // N
    f32 = dict(device=device, dtype=torch.float32)
    lay = torch.arange(L, **f32)
    ratio_0_to_1 = lay / max(L - 1, 1)
    ratio_1_to_almost_0 = 1.0 - lay / L
    ddd = torch.arange(C, **f32) / C

    def small(*shape):
        if zero_init:
            return torch.zeros(shape, **f32)
        return 0.02 * torch.randn(shape, generator=gen, **f32)

    def orth_stack(rows, cols, gain):
        return torch.stack([_orthogonal(gen, rows, cols, gain, device) for _ in range(L)])

    att = {}
    for name, p in (("x_r", 0.2), ("x_w", 0.9), ("x_k", 0.7), ("x_v", 0.7), ("x_a", 0.9), ("x_g", 0.2)):
        att[name] = 1 - torch.pow(ddd[None], p * ratio_1_to_almost_0[:, None])
    linear = (torch.arange(C, **f32) / (C - 1) - 0.5)[None].repeat(L, 1)
    zz = ((torch.arange(C, **f32) % N) - (N - 1) / 2) / ((N - 1) / 2)
    zigzag = (zz * zz.abs())[None].repeat(L, 1)
    www = -6 + 6 * torch.pow(torch.arange(C, **f32)[None] / (C - 1), 1 + ratio_0_to_1[:, None] ** 0.3)
    d_decay = max(32, int(round((1.8 * (C ** 0.5)) / 32) * 32))
    d_mv = max(32, int(round((1.3 * (C ** 0.5)) / 32) * 32))
    d_gate = max(32, int(round((0.6 * (C ** 0.8)) / 32) * 32))
    att["w0"] = www + 0.5 + zigzag * 2.5
    att["w1"] = small(L, C, d_decay)
    att["w2"] = orth_stack(d_decay, C, 0.1)
    att["a0"] = -0.19 + zigzag * 0.3 + linear * 0.4
    att["a1"] = small(L, C, d_decay)
    att["a2"] = orth_stack(d_decay, C, 0.1)
    att["v0"] = 0.73 - linear * 0.4
    att["v1"] = small(L, C, d_mv)
    att["v2"] = orth_stack(d_mv, C, 0.1)
    att["g1"] = small(L, C, d_gate)
    att["g2"] = orth_stack(d_gate, C, 0.1)
    att["k_k"] = 0.71 - linear * 0.1
    att["k_a"] = 1.02 + torch.zeros_like(linear)
    att["r_k"] = torch.zeros((L, H, N), **f32) - 0.04
    att["receptance"] = {"weight": orth_stack(C, C, 1.0)}
    att["key"] = {"weight": orth_stack(C, C, 0.1)}
    att["value"] = {"weight": orth_stack(C, C, 1.0)}
    att["output"] = {"weight": small(L, C, C)}
    att["ln_x"] = {"bias": torch.zeros((L, C), **f32),
                   "weight": (((1 + lay) / L)[:, None] ** 0.7).repeat(1, C)}
    ffn = {"x_k": 1 - torch.pow(ddd[None], ratio_1_to_almost_0[:, None] ** 4),
           "key": {"weight": orth_stack(4 * C, C, 1.0)},
           "value": {"weight": small(L, C, 4 * C)}}
    head_scale = 0.5 if vocab_size <= C else 0.5 * math.sqrt(vocab_size / C)
    params = {
        "blocks": {"att": att, "ffn": ffn,
                   "ln1": {"bias": torch.zeros((L, C), **f32), "weight": torch.ones((L, C), **f32)},
                   "ln2": {"bias": torch.zeros((L, C), **f32), "weight": torch.ones((L, C), **f32)}},
        "emb": {"weight": (torch.rand((vocab_size, C), generator=gen, **f32) * 2 - 1) * 1e-4},
        "head": {"weight": _orthogonal(gen, vocab_size, C, head_scale, device)},
        "ln0": {"bias": torch.zeros(C, **f32), "weight": torch.ones(C, **f32)},
        "ln_out": {"bias": torch.zeros(C, **f32), "weight": torch.ones(C, **f32)},
    }
    return tree_map(lambda t: t.to(dtype).contiguous(), params)


def tree_map(fn, tree):
    return {k: tree_map(fn, v) if isinstance(v, dict) else fn(v) for k, v in tree.items()}


def layer_of(tree, i):
    return tree_map(lambda t: t[i], tree)


class RWKV7:
    """``forward`` / ``default_state`` with the reference's argument names; batched over the leading axis."""

    inner = HipRWKV
    #: use the fused kernels beside the recurrence (ops.rwkv7_shiftmix, rwkv7_decay, rwkv7_vmix, rwkv7_agate,
    #: rwkv7_premix, rwkv7_postmix), with or without autograd
    fuse_mix = True

    @classmethod
    def default_state(cls, params, batch):
        """rwkv7.py:176-180 with a batch axis: zeros ``(B, L, 2 + N, C)`` in the parameter dtype."""
        emb = params["emb"]["weight"]
        L, H, N = params["blocks"]["att"]["r_k"].shape
        return torch.zeros((batch, L, 2 + N, emb.shape[1]), dtype=emb.dtype, device=emb.device)

    @classmethod
    def _shift(cls, x, prev, new_starts):
        """Token shift of rwkv7.py:227-229 / 192-194: previous token (state row for t = 0), zero at new_starts."""
        sx = torch.cat([prev[:, None], x[:, :-1]], dim=1)
        sx = torch.where(new_starts[:, :, None], torch.zeros_like(sx), sx)
        return sx - x

    @classmethod
    def channel_mixing_seq(cls, x, state_row, ffn, last_idx, new_starts):
        """rwkv7.py:190-198"""
        if cls.fuse_mix:
            xk, = ops.rwkv7_shiftmix(x, state_row, new_starts, [ffn["x_k"]])
        else:
            xk = x + cls._shift(x, state_row, new_starts) * ffn["x_k"]
        k = xk @ ffn["key"]["weight"].T
        k = ops.rwkv7_relusq(k) if cls.fuse_mix else torch.square(torch.relu(k))
        return k @ ffn["value"]["weight"].T, x[torch.arange(x.shape[0], device=x.device), last_idx]

    @classmethod
    def time_mixing_seq(cls, x, shift_row, wkv_state, v_first, att, length, last_idx, new_starts, layer_id,
                        wkv_out=None):
        """rwkv7.py:223-267.  wkv_state (B, N, C) is the layer's rows 2.. of the model state.  With ``wkv_out`` (the
        same rows of the new model state; decode steps without autograd) the recurrence reads and writes the two views
        in place and the third result is None."""
        B, T, C = x.shape
        H, N = att["r_k"].shape
        mix_names = ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g")
        if cls.fuse_mix:
            xr, xw, xk, xv, xa, xg = ops.rwkv7_shiftmix(x, shift_row, new_starts, [att[n] for n in mix_names])
        else:
            sx = cls._shift(x, shift_row, new_starts)
            xr, xw, xk, xv, xa, xg = (x + sx * att[n] for n in mix_names)
        r = xr @ att["receptance"]["weight"].T
        w_lora = torch.tanh(xw @ att["w1"]) @ att["w2"]
        if cls.fuse_mix:
            w = ops.rwkv7_decay(w_lora, att["w0"])
        else:
            w = -F.softplus(-(att["w0"] + w_lora).float()).to(x.dtype) - 0.5
        k = xk @ att["key"]["weight"].T
        v = xv @ att["value"]["weight"].T
        if layer_id == 0:
            v_first = v
        else:
            v_lora = (xv @ att["v1"]) @ att["v2"]
            if cls.fuse_mix:
                v = ops.rwkv7_vmix(v, v_first, v_lora, att["v0"])
            else:
                v = v + (v_first - v) * torch.sigmoid(att["v0"] + v_lora)
        a_lora = (xa @ att["a1"]) @ att["a2"]
        a = ops.rwkv7_agate(a_lora, att["a0"]) if cls.fuse_mix else torch.sigmoid(att["a0"] + a_lora)
        g = torch.sigmoid(xg @ att["g1"]) @ att["g2"]
        new_shift = x[torch.arange(B, device=x.device), last_idx]
        fused = cls.fuse_mix
        rh, wh, vh = (t.reshape(B, T, H, N) for t in (r, w, v))
        if fused:
            kh, ah, bh = ops.rwkv7_premix(k.reshape(B, T, H, N), a.reshape(B, T, H, N), att["k_k"], att["k_a"])
        else:
            kk = (k * att["k_k"]).reshape(B, T, H, N)
            kk = (kk / torch.clamp(torch.linalg.vector_norm(kk.float(), dim=-1, keepdim=True), min=1e-12).to(kk.dtype))
            kk = kk.reshape(B, T, C)
            k = k * (1 + (a - 1) * att["k_a"])
            kh, ah, bh = (t.reshape(B, T, H, N) for t in (k, -kk, kk * a))
        if wkv_out is not None:
            s_new, out = None, cls.inner.step_packed(rh, wh, kh, vh, ah, bh, wkv_state, wkv_out, length, new_starts)
        else:
            s_new, out = cls.inner.inner_loop(rh, wh, kh, vh, ah, bh, wkv_state.reshape(B, H, N, N), length, new_starts)
            s_new = s_new.reshape(B, N, C)
        if fused:
            y = ops.rwkv7_postmix(out, rh, kh, vh, g.reshape(B, T, H, N), att["ln_x"]["weight"], att["ln_x"]["bias"],
                                  att["r_k"], 64e-5).reshape(B, T, C)
        else:
            y = out.reshape(B * T, H, N).float()
            y = F.group_norm(y.reshape(B * T, C), H, att["ln_x"]["weight"].float(), att["ln_x"]["bias"].float(), 64e-5)
            y = y.to(x.dtype).reshape(B, T, C)
            bonus = ((rh * kh * att["r_k"]).sum(-1, keepdim=True) * vh).reshape(B, T, C)
            y = (y + bonus) * g
        return y @ att["output"]["weight"].T, new_shift, s_new, v_first

    @classmethod
    def forward(cls, params, tokens, state, length=None, new_starts=None):
        """tokens (B,T) int; state (B,L,2+N,C); length (B,) or None (= T); new_starts (B,T) bool or None.
        Returns (logits (B,T,vocab), new state).  llm.py:71-84 + rwkv7.py:269-291."""
        B, T = tokens.shape
        dev = tokens.device
        if length is None:
            length = torch.full((B,), T, dtype=torch.int32, device=dev)
        length = torch.as_tensor(length, device=dev).to(torch.int32).reshape(-1).expand(B)
        if new_starts is None:
            new_starts = torch.zeros((B, T), dtype=torch.bool, device=dev)
        last_idx = (length.long() - 1) % T          # x[length - 1] with the wrap-around of negative indices
        x = params["emb"]["weight"][tokens]
        x = layer_norm(x, params["ln0"])
        L = params["blocks"]["att"]["r_k"].shape[0]
        new_state = torch.empty_like(state)
        # decode steps: the recurrence works on the layers' rows of the two model states directly (no copies of them)
        packed = (T <= 8 and hasattr(cls.inner, "step_packed")
                  and not (torch.is_grad_enabled() and (x.requires_grad or state.requires_grad)))
        v_first = x
        for i in range(L):
            blk = layer_of(params["blocks"], i)
            st = state[:, i]
            dx, shift1, wkv, v_first = cls.time_mixing_seq(layer_norm(x, blk["ln1"]), st[:, 1], st[:, 2:], v_first,
                                                           blk["att"], length, last_idx, new_starts, i,
                                                           new_state[:, i, 2:] if packed else None)
            x = x + dx
            dx, shift0 = cls.channel_mixing_seq(layer_norm(x, blk["ln2"]), st[:, 0], blk["ffn"], last_idx, new_starts)
            x = x + dx
            new_state[:, i, 0] = shift0
            new_state[:, i, 1] = shift1
            if not packed:
                new_state[:, i, 2:] = wkv.to(state.dtype)
        logits = layer_norm(x, params["ln_out"]) @ params["head"]["weight"].T
        return logits, new_state
