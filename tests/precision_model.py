"""NumPy models of the chunked WKV7 and WKV6 forward kernels with a selectable operand precision for every matrix
product (WKV7 first; the WKV6 model is at the end of the file).

The chunked kernel (jaxrwkv_amd/csrc/wkv7_fwd.hip) evaluates 16 tokens at a time from the entering state S0
(recurrence: /root/reference/src/jaxrwkv/rwkv7.py:200-220).  With l_t = log d_t, Lc_t = sum_{s<=t} l_s:

    at_t = a_t exp(Lc_{t-1})   qt_t = r_t exp(Lc_t)   kh_s = k_s exp(-Lc_s)   bh_s = b_s exp(-Lc_s)
    ke_s = k_s exp(Lc_15 - Lc_s)   be_s = b_s exp(Lc_15 - Lc_s)             (update operands, referenced to the chunk end)
    Mba = [s<t] bh_s.at_t   Mka = [s<t] kh_s.at_t   Mbr = [s<=t] bh_s.qt_t   Mkr = [s<=t] kh_s.qt_t
    T = (I - Mba)^-1 = (I + M^8)(I + M^4)(I + M^2)(I + M)
    W = S0 At^T + V^T Mka      SA = W T      Y = S0 Qt^T + SA Mbr + V^T Mkr      S_C = S0 diag(E_15) + SA^T.. Be + V^T Ke

Every matrix-core operand is a 16-bit number (bf16 or fp16) or a pair hi + lo of them; a product of two pairs keeps
hi.hi + hi.lo + lo.hi.  This module rounds the operands exactly as such a kernel would and accumulates in float64
(the matrix cores accumulate in fp32; that error is four orders of magnitude below the operand rounding).  It is the
tool behind the kernel's choice of formats: ``python -m tests.precision_model`` prints the ablation table, and
tests/test_precision_model.py pins the chosen set against the bf16 bar.

Test infrastructure only: nothing in jaxrwkv_amd imports it.
"""
import numpy as np

from .inputs import bf16_round

CK = 16


def rn(x, fmt):
    """Round to nearest: 'b' bfloat16, 'h' float16 (saturating at the largest finite value), 'f' no rounding."""
    if fmt == "f":
        return np.asarray(x, np.float64)
    if fmt == "b":
        return bf16_round(x).astype(np.float64)
    if fmt == "h":
        return np.clip(np.asarray(x, np.float32), -65504.0, 65504.0).astype(np.float16).astype(np.float64)
    raise ValueError(fmt)


class Q:
    """An operand as the matrix cores see it: hi (+ lo) in one 16-bit format."""

    def __init__(self, x, spec):
        fmt, n = spec[0], int(spec[1])
        self.hi = rn(x, fmt)
        self.lo = rn(np.asarray(x, np.float64) - self.hi, fmt) if n == 2 else None

    @property
    def val(self):
        return self.hi if self.lo is None else self.hi + self.lo


def mm(a, b, sub):
    """einsum of two Q operands keeping hi.hi + hi.lo + lo.hi."""
    out = np.einsum(sub, a.hi, b.hi)
    if a.lo is not None:
        out = out + np.einsum(sub, a.lo, b.hi)
    if b.lo is not None:
        out = out + np.einsum(sub, a.hi, b.lo)
    return out


# operand -> (format, parts).  Keys:
#   s      state in W = S0 At^T and Y = S0 Qt^T          aq    At and Qt in those two products
#   gk     kh, bh in the Gram tiles                      ga    at, qt in the Gram tiles
#   inv    every operand of the doubling chain           m     T, Mka, Mbr, Mkr as the consumers read them
#   mkr    Mkr alone (default: m)
#   w      W in SA = W T                                 sa    SA in Y and in the state update
#   upd    ke, be in the state update
EXACT = dict(s="f1", aq="f1", gk="f1", ga="f1", inv="f1", m="f1", w="f1", sa="f1", upd="f1")
ALL_SPLIT = dict(s="b2", aq="b2", gk="b2", ga="b2", inv="b1", m="b2", w="b2", sa="b2", upd="b2")   # the first kernel
ALL_BF16 = dict(s="b1", aq="b1", gk="b1", ga="b1", inv="b1", m="b1", w="b1", sa="b1", upd="b1")
# the set the kernel uses: fp16 wherever the operand is bounded by the inputs' magnitudes (Mkr, which multiplies v
# straight into y, as an fp16 pair), bf16 pairs for the Gram operands kh, bh (they carry exp(-Lc) and need the fp32
# exponent range) and at, qt
CHOSEN = dict(s="h1", aq="h1", gk="b2", ga="b2", inv="h1", m="h1", mkr="h2", w="h1", sa="h1", upd="h1")


def chunk_forward(r, l, k, v, a, b, S0, p):
    """One chunk for a batch of heads: token arrays (G, 16, 64), l = log decay (<= 0), S0 (G, 64, 64) [value][key].
    Returns y (G,16,64), S_C, sa (G,16,64)."""
    Lc = np.cumsum(l, axis=1)
    Le = np.concatenate([np.zeros_like(Lc[:, :1]), Lc[:, :-1]], axis=1)
    at, qt = a * np.exp(Le), r * np.exp(Lc)
    kh, bh = k * np.exp(-Lc), b * np.exp(-Lc)
    ke, be = k * np.exp(Lc[:, -1:] - Lc), b * np.exp(Lc[:, -1:] - Lc)
    gam = np.exp(Lc[:, -1])                                   # (G, key)
    s_i, t_i = np.arange(CK)[:, None], np.arange(CK)[None, :]
    lt, le = (s_i < t_i), (s_i <= t_i)
    gk_k, gk_b, ga_a, ga_q = Q(kh, p["gk"]), Q(bh, p["gk"]), Q(at, p["ga"]), Q(qt, p["ga"])
    Mba = mm(gk_b, ga_a, "gsj,gtj->gst") * lt
    Mka = mm(gk_k, ga_a, "gsj,gtj->gst") * lt
    Mbr = mm(gk_b, ga_q, "gsj,gtj->gst") * le
    Mkr = mm(gk_k, ga_q, "gsj,gtj->gst") * le
    P = np.eye(CK) + Mba
    Mp = Mba
    for _ in range(3):
        q = Q(Mp, p["inv"])
        Mp = mm(q, q, "gsu,gut->gst")
        P = P + mm(Q(Mp, p["inv"]), Q(P, p["inv"]), "gsu,gut->gst")
    Tq, Kaq, Brq, Krq = Q(P, p["m"]), Q(Mka, p["m"]), Q(Mbr, p["m"]), Q(Mkr, p.get("mkr", p["m"]))
    Sq = Q(S0, p["s"])
    vq = Q(v, "f1")                                           # v is an input: exact in bf16 and (normal range) in fp16
    W = mm(Sq, Q(at, p["aq"]), "gij,gtj->git") + mm(vq, Kaq, "gsi,gst->git")
    SA = mm(Q(W, p["w"]), Tq, "gis,gst->git")
    saq = Q(SA, p["sa"])
    Y = mm(Sq, Q(qt, p["aq"]), "gij,gtj->git") + mm(saq, Brq, "gis,gst->git") + mm(vq, Krq, "gsi,gst->git")
    SC = S0 * gam[:, None, :] + mm(saq, Q(be, p["upd"]), "gis,gsj->gij") + mm(vq, Q(ke, p["upd"]), "gsi,gsj->gij")
    return Y.transpose(0, 2, 1), SC.astype(np.float32).astype(np.float64), SA.transpose(0, 2, 1)


def forward(x, p):
    """Whole sequences without resets: x from tests.inputs.wkv7_inputs (resets=False, lengths=False).
    Returns (S_final, y, sa) with the oracle's shapes."""
    B, T, H, N = x["r"].shape
    assert T % CK == 0
    f = lambda n: x[n].transpose(0, 2, 1, 3).reshape(B * H, T, N)
    r, w, k, v, a, b = (f(n) for n in "rwkvab")
    l = -np.exp(w)
    S = x["s"].reshape(B * H, N, N).astype(np.float64)
    y, sa = np.zeros_like(r), np.zeros_like(r)
    for c0 in range(0, T, CK):
        sl = slice(c0, c0 + CK)
        y[:, sl], S, sa[:, sl] = chunk_forward(r[:, sl], l[:, sl], k[:, sl], v[:, sl], a[:, sl], b[:, sl], S, p)
    g = lambda z: z.reshape(B, H, T, N).transpose(0, 2, 1, 3)
    return S.reshape(B, H, N, N), g(y), g(sa)


def make_inputs(regime, B=2, T=1024, H=4, seed=0):
    """'bench': the benchmark distribution (w ~ N(-0.5, 0.5), state memory of a few tokens).
    'slow': RWKV-7-like decays w ~ U(-8, -0.5) (d between 0.9997 and 0.545: memories of thousands of tokens)."""
    from .inputs import wkv7_inputs
    x = wkv7_inputs(B, T, H, 64, seed=seed, bf16=True, resets=False, lengths=False)
    if regime == "slow":
        g = np.random.default_rng(seed + 1000)
        x["w"] = bf16_round(g.uniform(-8.0, -0.5, size=x["w"].shape)).astype(np.float64)
    return x


def metrics(x, p, ref=None):
    from oracle import wkv7 as o7
    from .gpu_util import tvd_of_projected
    if ref is None:
        ref = o7.wkv7_base(*[x[n] for n in "rwkvab"], x["s"], x["length"], x["new_starts"], return_sa=True)
    ref_s, ref_y, ref_sa = ref
    S, y, sa = forward(x, p)
    rel = lambda got, want: float(np.sqrt(np.mean((got - want) ** 2) / np.mean(want ** 2)))
    yb, rb = bf16_round(y).astype(np.float64), bf16_round(ref_y).astype(np.float64)
    tvd = tvd_of_projected(yb, rb)
    return dict(y=rel(y, ref_y), s=rel(S, ref_s), sa=rel(sa, ref_sa), flips=float(np.mean(yb != rb)),
                tvd_max=float(tvd.max()), tvd_mean=float(tvd.mean())), ref


ABLATION = [
    ("exact operands", EXACT),
    ("bf16 pairs everywhere (inverse chain single)", ALL_SPLIT),
    ("single bf16 everywhere", ALL_BF16),
    ("fp16 everywhere, bf16 pairs in the Gram tiles, Mkr an fp16 pair (chosen)", CHOSEN),
    ("chosen, Mkr single fp16", {**CHOSEN, "mkr": "h1"}),
    ("chosen, Gram operands single bf16", {**CHOSEN, "gk": "b1", "ga": "b1"}),
    ("chosen, Gram kh/bh pairs but at/qt single bf16", {**CHOSEN, "ga": "b1"}),
    ("chosen, state single bf16", {**CHOSEN, "s": "b1", "aq": "b1"}),
    ("chosen, state fp16 pair", {**CHOSEN, "s": "h2"}),
    ("chosen, state and At/Qt fp16 pairs", {**CHOSEN, "s": "h2", "aq": "h2"}),
    ("chosen, inverse chain single bf16", {**CHOSEN, "inv": "b1"}),
    ("chosen, tiles T/Mka/Mbr/Mkr single bf16", {**CHOSEN, "m": "b1", "mkr": "b1"}),
    ("chosen, all four tiles fp16 pairs", {**CHOSEN, "m": "h2"}),
    ("chosen, W single bf16", {**CHOSEN, "w": "b1"}),
    ("chosen, SA single bf16", {**CHOSEN, "sa": "b1"}),
    ("chosen, W and SA fp16 pairs", {**CHOSEN, "w": "h2", "sa": "h2"}),
    ("chosen, update operands single bf16", {**CHOSEN, "upd": "b1"}),
    ("chosen, update operands fp16 pairs", {**CHOSEN, "upd": "h2"}),
]


# ------------------------------------------------------------------------------------------------------ WKV6
# The chunked WKV6 forward (jaxrwkv_amd/csrc/wkv6_fwd.hip; recurrence /root/reference/src/jaxrwkv/rwkv6.py:175-191,
# S[key][value]):  Y = Qt S0 + M^T V,  S_C = diag(E_C) S0 + Ke^T V  with qt_t = r_t exp(Lc_{t-1}), kh_s = k_s exp(-Lc_s),
# ke_s = k_s exp(Lc_15 - Lc_s), M[s][t] = kh_s.qt_t (s < t), M[t][t] = sum r u k.  Operand keys:
#   s  state in Qt S0        q  qt in Qt S0        g  kh, qt in the Gram tile        m  M as the consumers read it
#   upd  ke in the state update
EXACT6 = dict(s="f1", q="f1", g="f1", m="f1", upd="f1")
CHOSEN6 = dict(s="h1", q="h1", g="b2", m="h2", upd="h1")


def chunk_forward6(r, lw, k, v, u, S0, p):
    """One chunk for a batch of heads: token arrays (G, 16, 64), lw = log decay, u (G, 64), S0 (G, 64, 64) [key][value]."""
    Lc = np.cumsum(lw, axis=1)
    Le = np.concatenate([np.zeros_like(Lc[:, :1]), Lc[:, :-1]], axis=1)
    qt, kh = r * np.exp(Le), k * np.exp(-Lc)
    ke = k * np.exp(Lc[:, -1:] - Lc)
    gam = np.exp(Lc[:, -1])
    s_i, t_i = np.arange(CK)[:, None], np.arange(CK)[None, :]
    M = mm(Q(kh, p["g"]), Q(qt, p["g"]), "gsj,gtj->gst") * (s_i < t_i)
    M = M + np.eye(CK) * np.einsum("gtj,gj,gtj->gt", r, u, k)[:, None, :]
    vq = Q(v, "f1")
    Y = mm(Q(qt, p["q"]), Q(S0, p["s"]), "gtj,gji->gti") + mm(Q(M, p["m"]), vq, "gst,gsi->gti")
    SC = S0 * gam[:, :, None] + mm(Q(ke, p["upd"]), vq, "gsj,gsi->gji")
    return Y, SC.astype(np.float32).astype(np.float64)


def forward6(x, p):
    """Whole sequences without resets: x from tests.inputs.wkv6_inputs (resets=False, lengths=False)."""
    B, T, H, N = x["r"].shape
    assert T % CK == 0
    f = lambda n: x[n].transpose(0, 2, 1, 3).reshape(B * H, T, N)
    r, w, k, v = (f(n) for n in "rwkv")
    u = np.broadcast_to(x["u"][None], (B, H, N)).reshape(B * H, N)
    S = x["s"].reshape(B * H, N, N).astype(np.float64)
    y = np.zeros_like(r)
    for c0 in range(0, T, CK):
        sl = slice(c0, c0 + CK)
        y[:, sl], S = chunk_forward6(r[:, sl], w[:, sl], k[:, sl], v[:, sl], u, S, p)
    return S.reshape(B, H, N, N), y.reshape(B, H, T, N).transpose(0, 2, 1, 3)


def metrics6(x, p, ref=None):
    from oracle import wkv6 as o6
    from .gpu_util import tvd_of_projected
    if ref is None:
        ref = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"])
    ref_s, ref_y = ref
    S, y = forward6(x, p)
    rel = lambda got, want: float(np.sqrt(np.mean((got - want) ** 2) / np.mean(want ** 2)))
    yb, rb = bf16_round(y).astype(np.float64), bf16_round(ref_y).astype(np.float64)
    tvd = tvd_of_projected(yb, rb)
    return dict(y=rel(y, ref_y), s=rel(S, ref_s), flips=float(np.mean(yb != rb)), tvd_max=float(tvd.max()),
                tvd_mean=float(tvd.mean())), ref


ABLATION6 = [
    ("exact operands", EXACT6),
    ("single bf16 everywhere", dict(s="b1", q="b1", g="b1", m="b1", upd="b1")),
    ("fp16 everywhere, bf16 pairs in the Gram tile, M an fp16 pair (chosen)", CHOSEN6),
    ("chosen, M single fp16", {**CHOSEN6, "m": "h1"}),
    ("chosen, Gram operands single bf16", {**CHOSEN6, "g": "b1"}),
    ("chosen, state fp16 pair", {**CHOSEN6, "s": "h2"}),
    ("chosen, state and qt fp16 pairs", {**CHOSEN6, "s": "h2", "q": "h2"}),
    ("chosen, update operand single bf16", {**CHOSEN6, "upd": "b1"}),
]


def main():
    for regime in ("bench", "slow"):
        x = make_inputs(regime)
        ref = None
        print(f"\nregime {regime}: B=2 T=1024 H=4, bf16 inputs; errors against the float64 sequential oracle")
        print(f"{'operand formats':66s} {'y relrms':>9s} {'S relrms':>9s} {'sa relrms':>9s} {'y flips':>8s} {'TVD max':>9s} {'TVD mean':>9s}")
        for name, p in ABLATION:
            m, ref = metrics(x, p, ref)
            print(f"{name:66s} {m['y']:9.2e} {m['s']:9.2e} {m['sa']:9.2e} {m['flips']:8.4f} {m['tvd_max']:9.2e} {m['tvd_mean']:9.2e}")
    from .inputs import wkv6_inputs
    x = wkv6_inputs(2, 1024, 4, 64, seed=0, bf16=True, resets=False, lengths=False)
    ref = None
    print("\nWKV6, B=2 T=1024 H=4, bf16 inputs; errors against the float64 sequential oracle")
    print(f"{'operand formats':72s} {'y relrms':>9s} {'S relrms':>9s} {'y flips':>8s} {'TVD max':>9s} {'TVD mean':>9s}")
    for name, p in ABLATION6:
        m, ref = metrics6(x, p, ref)
        print(f"{name:72s} {m['y']:9.2e} {m['s']:9.2e} {m['flips']:8.4f} {m['tvd_max']:9.2e} {m['tvd_mean']:9.2e}")


if __name__ == "__main__":
    main()
