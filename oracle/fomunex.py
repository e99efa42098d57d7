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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


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
