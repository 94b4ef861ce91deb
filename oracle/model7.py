"""Float64 NumPy oracle for the RWKV-7 full model around the WKV op (checker only, never shipped).

Restates, without importing it, one stream of the reference's ``RWKV.forward`` with ``AssociativeScanRWKV``:
``forward`` /root/reference/src/jaxrwkv/llm.py:71-84, ``embed``/``outhead`` rwkv7.py:183-188,
``channel_mixing_seq`` :190-198, ``time_mixing_seq`` :223-267, ``forward_seq`` :269-291, ``layer_norm`` /
``group_norm`` :8-24.  The recurrence itself is ``oracle.wkv7.wkv7_base(compat=True)`` (pinned separately against
the associative form).  Parameters are a tree of arrays with the reference's names, stacked per layer.

Pinned by ``tests/test_oracle_model7.py``: split-sequence with carried state equals a single call, a reset equals a
fresh default state, ``length`` equals a truncated run, the time-mix output projection being zero makes the logits
independent of the recurrence (the reference's own initialisation), and norm layers against their definitions.
"""
import numpy as np

from . import wkv7 as o7


def layer_norm(x, w, eps=1e-5):                                           # rwkv7.py:8-12
    mean = x.mean(-1, keepdims=True)
    var = x.var(-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * w["weight"] + w["bias"]


def group_norm_tokens(x, H, weight, bias, eps):                           # rwkv7.py:14-24 on a (T, C) input
    T, C = x.shape
    g = x.reshape(T, H, C // H)
    g = (g - g.mean(-1, keepdims=True)) / np.sqrt(g.var(-1, keepdims=True) + eps)
    return g.reshape(T, C) * weight + bias


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x):
    return np.logaddexp(0.0, x)


def _layer(tree, i):
    return {k: _layer(v, i) if isinstance(v, dict) else v[i] for k, v in tree.items()}


def to_f64(tree):
    return {k: to_f64(v) if isinstance(v, dict) else np.asarray(v, np.float64) for k, v in tree.items()}


def default_state(params):                                                # rwkv7.py:176-180
    C = params["emb"]["weight"].shape[1]
    L, H, N = params["blocks"]["att"]["r_k"].shape
    return np.zeros((L, 2 + N, C))


def channel_mixing_seq(x, state, ffn, length, new_starts):                # rwkv7.py:190-198
    sx = np.concatenate([state, x[:-1]])
    sx = np.where(new_starts[:, None], 0.0, sx)
    sx = sx - x
    xk = x + sx * ffn["x_k"]
    k = np.square(np.maximum(xk @ ffn["key"]["weight"].T, 0.0))
    return k @ ffn["value"]["weight"].T, x[length - 1]


def _bf16(x):
    """Round to the nearest bfloat16 (ties to even), as float64: the op's I/O format in a bf16 model."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def time_mixing_seq(x, state, v_first, att, length, new_starts, H, S, layer_id, op_io=None):   # rwkv7.py:223-267
    T, C = x.shape
    sx = np.concatenate([state[:1], x[:-1]])
    sx = np.where(new_starts[:, None], 0.0, sx)
    sx = sx - x
    xr, xw, xk, xv, xa, xg = (x + sx * att[n] for n in ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g"))
    r = xr @ att["receptance"]["weight"].T
    w = -softplus(-(att["w0"] + np.tanh(xw @ att["w1"]) @ att["w2"])) - 0.5
    k = xk @ att["key"]["weight"].T
    v = xv @ att["value"]["weight"].T
    if layer_id == 0:
        v_first = v
    else:
        v = v + (v_first - v) * sigmoid(att["v0"] + (xv @ att["v1"]) @ att["v2"])
    a = sigmoid(att["a0"] + (xa @ att["a1"]) @ att["a2"])
    g = sigmoid(xg @ att["g1"]) @ att["g2"]
    kk = (k * att["k_k"]).reshape(T, H, -1)
    kk = kk / np.maximum(np.linalg.norm(kk, axis=-1, keepdims=True), 1e-12)
    kk = kk.reshape(T, C)
    k = k * (1 + (a - 1) * att["k_a"])
    state = state.copy()
    state[0] = x[length - 1]
    s = state[1:].reshape(H, S, S)
    r_, w_, k_, v_, a_, b_ = (val.reshape(T, H, S) for val in (r, w, k, v, -kk, kk * a))
    op_in = (r_, w_, k_, v_, a_, b_)
    if op_io == "bf16":      # an op with bf16 I/O: its six inputs and its output are bf16, the state stays wider
        op_in = tuple(_bf16(val) for val in op_in)
    s_new, out = o7.wkv7_base(*(val[None] for val in op_in), s[None], np.array([length]), new_starts[None], compat=True)
    state[1:] = s_new[0].reshape(S, -1)
    if op_io == "bf16":
        out = _bf16(out)
    y = group_norm_tokens(out[0].reshape(T, H * S), H, att["ln_x"]["weight"], att["ln_x"]["bias"], 64e-5)
    y = y + ((r_ * k_ * att["r_k"]).sum(-1, keepdims=True) * v_).reshape(T, C)
    y = y * g
    return y @ att["output"]["weight"].T, state, v_first


def forward(params, tokens, state, length=None, new_starts=None, op_io=None):   # llm.py:71-84, rwkv7.py:269-291
    """One stream: tokens (T,), state (L, 2+N, C).  Returns (logits (T, vocab), new state).  ``op_io="bf16"`` rounds the
    six inputs and the output of every layer's recurrence to bfloat16 and keeps everything else in float64 (the bonus
    term after the op included): what a model computes whose op alone has bf16 I/O."""
    tokens = np.asarray(tokens)
    T = tokens.shape[0]
    if length is None:
        length = T
    if new_starts is None:
        new_starts = np.zeros((T,), bool)
    length = int(length)
    L, H, S = params["blocks"]["att"]["r_k"].shape
    x = layer_norm(params["emb"]["weight"][tokens], params["ln0"])
    state = np.array(state, dtype=np.float64)
    v_first = x
    for i in range(L):
        blk = _layer(params["blocks"], i)
        dx, s, v_first = time_mixing_seq(layer_norm(x, blk["ln1"]), state[i, 1:], v_first, blk["att"], length,
                                         new_starts, H, S, i, op_io)
        state[i, 1:] = s
        x = x + dx
        dx, s0 = channel_mixing_seq(layer_norm(x, blk["ln2"]), state[i, :1], blk["ffn"], length, new_starts)
        state[i, 0] = s0
        x = x + dx
    return layer_norm(x, params["ln_out"]) @ params["head"]["weight"].T, state
