"""Whole-sequence float64 statement of the Fomunex decoder: one function per mechanism, no cache, no state slots, no batching -- a
sequence goes in as a list of token ids and every position's logits come out.  Shares nothing with ssd_amd/ (it reads the
configuration as the plain dict of config.json and the weights as a name -> tensor dict under the checkpoint's names).

Notation: W = width, E = eps of the layer, rms(v) = v / sqrt(mean(v^2) + E) over the last axis, T = tokens of the sequence."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is ONE number for all coordinates."""
    return rms(x, eps) * g.to(F64).reshape(())


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def lin(w, x):
    return x @ w.to(F64).T


# ------------------------------------------------------------------------------------------------------------------
def window_attention(h, w, p, m, eps):
    """Grouped-query attention without rotation: unit-RMS queries and keys, capped scores, a per-head linear distance penalty, a
    sliding window, and a softmax whose denominator also holds exp(sink_h)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(lin(w[p + "q"], h).view(T, H, D), eps)
    k = rms(lin(w[p + "k"], h).view(T, G, D), eps)
    v = lin(w[p + "v"], h).view(T, G, Dv)
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    dist = (i - j).to(F64)
    size = (m.get("mask") or {}).get("size")
    seen = (i - j >= 0) & ((i - j < size) if size else True)
    cap = m.get("softcap")
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s - 2.0 ** (-8.0 * (hh + 1) / H) * dist
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        sink = w[p + "sink"].to(F64)[hh]
        mx = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
        e = torch.exp(s - mx)
        out[:, hh] = (e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - mx))) @ v[:, g]
    return lin(w[p + "o"], out.reshape(T, H * Dv))


def wkv_mixer(h, w, p, m, eps):
    """RWKV-style time mixing: token-shift interpolation per projection, a data-dependent per-channel decay, a bonus for the current
    token, per-head unit-RMS output, gate."""
    T, W = h.shape
    H, D = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, W, dtype=F64), h[:-1]], dim=0)
    mix = lambda s: h + (prev - h) * w[p + "mu." + s].to(F64)
    r = lin(w[p + "r"], mix("r")).view(T, H, D)
    k = lin(w[p + "k"], mix("k")).view(T, H, D)
    v = lin(w[p + "v"], mix("v")).view(T, H, D)
    gate = silu(lin(w[p + "g"], mix("g")))
    dec = torch.exp(-torch.exp(lin(w[p + "w2"], torch.tanh(lin(w[p + "w1"], mix("w")))) + w[p + "w0"].to(F64))).view(T, H, D)
    u = w[p + "u"].to(F64).view(H, D)
    o = torch.zeros(T, H, D, dtype=F64)
    for hh in range(H):
        S = torch.zeros(D, D, dtype=F64)                 # [key channel][value channel]
        for t in range(T):
            kv = torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = (S + u[hh].view(D, 1) * kv).T @ r[t, hh]
            S = dec[t, hh].view(D, 1) * S + kv
    o = rms(o, eps).reshape(T, H * D) * w[p + "norm"].to(F64) * gate
    return lin(w[p + "o"], o)


def mamba2_mixer(h, w, p, m, eps):
    """Selective state space (Mamba-2 form): one scalar decay per head and token, B / C shared by the heads of a group, a short causal
    convolution in front, gate BEFORE the grouped norm."""
    T = h.shape[0]
    H, Dv, N, G, taps, NG = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"]
    inner = H * Dv
    zxbcdt = lin(w[p + "in"], h)
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    cw, cb = w[p + "conv"].to(F64), w[p + "conv.b"].to(F64)
    pad = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F64), xbc], dim=0)
    conv = cb + sum(pad[c:c + T] * cw[:, c] for c in range(taps))          # the last column meets the current token
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, H, Dv)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"].to(F64))
    A = -torch.exp(w[p + "A_log"].to(F64))
    Dskip = w[p + "D"].to(F64)
    y = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, Dv, dtype=F64)
        for t in range(T):
            S = torch.exp(A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(Bm[t, g], x[t, hh])
            y[t, hh] = S.T @ Cm[t, g] + Dskip[hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, NG, inner // NG), eps).reshape(T, inner) * w[p + "norm"].to(F64)
    return lin(w[p + "o"], y)


def polynorm_mlp(h, w, p, eps):
    """W_down act(W_up h), act(z) = a rms(z) + b rms(z^2) + c rms(z^3) + e over a token's ff values."""
    z = lin(w[p + "up"], h)
    a, b, c, e = w[p + "act"].to(F64)
    return lin(w[p + "down"], a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e)


def routed_mlp(h, w, p, ml):
    """Sigmoid router, the `top` largest scores unrenormalised, each multiplying its expert's INPUT; experts are clamped swish-GLUs."""
    T, W = h.shape
    E, top, limit = ml["router"]["experts"], ml["router"]["top"], ml["expert"]["limit"]
    s = torch.sigmoid(lin(w[p + "router"], h))
    out = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            hin = s[t, e] * h[t]
            g = torch.clamp(lin(w[p + f"e{e}.gate"], hin), max=limit)
            u = torch.clamp(lin(w[p + f"e{e}.up"], hin), min=-limit, max=limit)
            out[t] += lin(w[p + f"e{e}.down"], g * torch.sigmoid(1.702 * g) * (u + 1.0))
    return out


# ------------------------------------------------------------------------------------------------------------------
def forward(cfg: dict, w: dict, tokens, taps: list | None = None, round_input=None) -> torch.Tensor:
    """Logits [T][vocab] of one sequence.  taps: receives the residual rows after every layer.  round_input: applied to every
    normalised sublayer input (lets a test model the element type of the GEMM-input rows)."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    T = ids.shape[0]
    x = w["embed"].to(F64)[ids] + w["pos"].to(F64)[:T]
    ri = round_input or (lambda t: t)
    for i, lc in enumerate(cfg["layers"]):
        src = lc.get("weights_of", i)
        p, m, ml = f"l{src}.", lc["mixer"], lc.get("mlp")
        h = ri(scalar_norm(x, w[p + "norm1"], eps))
        if lc["type"] == "attention":
            x = x + window_attention(h, w, p + "mix.", m, eps)
        elif lc["type"] == "wkv":
            x = x + wkv_mixer(h, w, p + "mix.", m, eps)
        elif lc["type"] == "mamba2":
            x = x + mamba2_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(lc["type"])
        if ml is not None:
            h = ri(scalar_norm(x, w[p + "norm2"], eps))
            x = x + (polynorm_mlp(h, w, p + "mlp.", eps) if ml["kind"] == "dense" else routed_mlp(h, w, p + "mlp.", ml))
        if taps is not None:
            taps.append(x.clone())
    logits = lin(w["head"], scalar_norm(x, w["final.norm"], eps)) * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


# ------------------------------------------------------------------------------------------------------------------
# configurations and random weights for tests
# ------------------------------------------------------------------------------------------------------------------
def dense_mlp(ff: int = 40) -> dict:
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts: int = 5, top: int = 2, ff: int = 24, limit: float = 1.25) -> dict:
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.6, softcap=12.0, window=9, mlp=None, weights_of=None) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if window:
        m["mask"] = {"size": window}
    out = {"type": "attention", "mixer": m, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def wkv_layer(heads=3, dim=8, decay_rank=6, mlp=None, weights_of=None) -> dict:
    """decay_rank is not a config.json key (the checkpoint's tensor shapes give it); random_model reads it from here and drops it."""
    out = {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": decay_rank}, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def mamba2_layer(heads=4, vdim=12, state=8, groups=2, conv=4, norm_groups=2, mlp=None, weights_of=None) -> dict:
    out = {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups},
           "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def make_config(layers, vocab=97, width=48, eps=1e-5, max_positions=512, logit_scale=1.5, logit_softcap=25.0) -> dict:
    cfg = {"architecture": "Fomunex", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps}, "layers": layers}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    if logit_softcap:
        cfg["logit_softcap"] = logit_softcap
    return cfg


def random_model(cfg: dict, seed: int = 0, keep_rank: bool = False) -> dict:
    """bf16 weights of the right shapes for `cfg`: matrices N(0, 1 / fan-in), norm numbers around 1, decays that remember hundreds of
    tokens in some channels and a few in others.  Unless keep_rank, the layers' decay_rank entries are removed from cfg afterwards (a
    checkpoint's tensor shapes carry that size)."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}
    bf = torch.bfloat16

    def mat(name, o, i, gain=1.0):
        w[name] = (torch.randn(o, i, generator=gen) * gain / math.sqrt(i)).to(bf)

    def vec(name, n, base=1.0, s=0.1):
        w[name] = (base + s * torch.randn(n, generator=gen)).to(bf)

    def uni(name, n, lo, hi):
        w[name] = (lo + (hi - lo) * torch.rand(n, generator=gen)).to(bf)

    def scalar(name):
        w[name] = torch.tensor(0.8 + 0.5 * torch.rand((), generator=gen).item()).to(bf)

    mat("embed", cfg["vocab"], W, math.sqrt(W))
    w["pos"] = (0.5 * torch.randn(cfg["max_positions"], W, generator=gen)).to(bf)
    for i, lc in enumerate(cfg["layers"]):
        if lc.get("weights_of", i) != i:
            continue
        p, m, ml = f"l{i}.", lc["mixer"], lc.get("mlp")
        scalar(p + "norm1")
        if lc["type"] == "attention":
            mat(p + "mix.q", m["heads"] * m["dim"], W, 2.0)
            mat(p + "mix.k", m["kv_heads"] * m["dim"], W, 2.0)
            mat(p + "mix.v", m["kv_heads"] * m["vdim"], W)
            vec(p + "mix.sink", m["heads"], 0.0, 1.5)
            mat(p + "mix.o", W, m["heads"] * m["vdim"])
        elif lc["type"] == "wkv":
            n, R = m["heads"] * m["dim"], m["decay_rank"]
            for s in "rkvgw":
                uni(p + "mix.mu." + s, W, 0.0, 1.0)
            for s in "rkvg":
                mat(p + "mix." + s, n, W, 1.5)
            mat(p + "mix.w1", R, W)
            mat(p + "mix.w2", n, R)
            uni(p + "mix.w0", n, -6.0, 0.5)
            w[p + "mix.u"] = (0.5 * torch.randn(m["heads"], m["dim"], generator=gen)).to(bf)
            vec(p + "mix.norm", n)
            mat(p + "mix.o", W, n)
        else:
            inner, C = m["heads"] * m["vdim"], m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
            mat(p + "mix.in", 2 * inner + 2 * m["groups"] * m["state"] + m["heads"], W, 1.5)
            w[p + "mix.conv"] = (torch.randn(C, m["conv"], generator=gen) / math.sqrt(m["conv"])).to(bf)
            vec(p + "mix.conv.b", C, 0.0, 0.2)
            uni(p + "mix.dt_bias", m["heads"], -4.0, 0.5)
            uni(p + "mix.A_log", m["heads"], -3.0, 1.0)
            vec(p + "mix.D", m["heads"], 0.5, 0.5)
            vec(p + "mix.norm", inner)
            mat(p + "mix.o", W, inner)
        if ml is None:
            continue
        scalar(p + "norm2")
        if ml["kind"] == "dense":
            mat(p + "mlp.up", ml["ff"], W, 1.5)
            mat(p + "mlp.down", W, ml["ff"])
            w[p + "mlp.act"] = torch.tensor([0.9, 0.4, -0.3, 0.1]).add(0.1 * torch.randn(4, generator=gen)).to(bf)
        else:
            for e in range(ml["router"]["experts"]):
                mat(p + f"mlp.e{e}.gate", ml["expert"]["ff"], W, 2.5)
                mat(p + f"mlp.e{e}.up", ml["expert"]["ff"], W, 2.5)
                mat(p + f"mlp.e{e}.down", W, ml["expert"]["ff"])
            mat(p + "mlp.router", ml["router"]["experts"], W, 2.0)
    scalar("final.norm")
    mat("head", cfg["vocab"], W, 2.0)
    if not keep_rank:
        for lc in cfg["layers"]:
            lc["mixer"].pop("decay_rank", None)
    return w
