"""Whole-sequence float64 statement of the Dosuvik decoder: one function per mechanism, no cache, no state slots, no batching -- a
sequence goes in as a list of token ids and every position's logits come out.  Shares nothing with ssd_amd/ (it reads the
configuration as the plain dict of config.json and the weights as a name -> tensor dict under the checkpoint's names).

Notation: W = width, E = eps of the layer, rms(v) = v / sqrt(mean(v^2) + E) over the last axis, T = tokens of the sequence, positions
0 .. T - 1.  turn(x, p, n, base, layout): the first n entries of the last axis of x are n / 2 pairs (a, b); pair i becomes
(a cos t - b sin t, b cos t + a sin t) with t = p * base^(-2i/n); layout "halves" makes pair i of entries (i, i + n / 2), "interleaved" of
entries (2i, 2i + 1).

    layer i:   x <- x + (1 + w1) rms(mixer(x));  x <- x + (1 + w2) rms(ff(x));  X_(i+1) = x;  x <- sum_(j <= i+1) dwa_i[j] X_j
               (X_0 = the embedding rows; the mixer and the feed-forward read x itself)
    output:    logits = head ((1 + w) rms(x))
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64
SWISH = 1.702


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def lin(w, x):
    return x @ w.to(F64).T


def silu(z):
    return z * torch.sigmoid(z)


def turn(x: torch.Tensor, pos: torch.Tensor, n: int, base: float, layout: str) -> torch.Tensor:
    """x [T, heads, D]; pos [T] (may be negative: turning back)."""
    if n == 0:
        return x
    i = torch.arange(n // 2, dtype=F64)
    t = pos.to(F64).view(-1, 1, 1) * (base ** (-2.0 * i / n)).view(1, 1, -1)
    c, s = torch.cos(t), torch.sin(t)
    ia, ib = (torch.arange(0, n // 2), torch.arange(n // 2, n)) if layout == "halves" else (torch.arange(0, n, 2), torch.arange(1, n, 2))
    a, b = x[..., ia], x[..., ib]
    out = x.clone()
    out[..., ia] = a * c - b * s
    out[..., ib] = b * c + a * s
    return out


# ------------------------------------------------------------------------------------------------------------------
def retention(h, w, p, m, eps):
    """Linear attention with a fixed decay per head: S_t = d_h S_(t-1) + k_t v_t^T from S = 0, o_t = S_t^T q_t; q and k turned ("halves"),
    k times dim^-0.5 after the turn; every head's o divided by its root mean square; silu gate; projection."""
    T = h.shape[0]
    H, D, Dv, r = m["heads"], m["dim"], m["vdim"], m["rot"]
    pos = torch.arange(T)
    q = turn(lin(w[p + "q"], h).view(T, H, D), pos, r["dims"], r["base"], "halves")
    k = turn(lin(w[p + "k"], h).view(T, H, D), pos, r["dims"], r["base"], "halves") * D ** -0.5
    v = lin(w[p + "v"], h).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = float(m["decay"][hh]) * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    o = rms(o, eps).reshape(T, H * Dv) * silu(lin(w[p + "g"], h))
    return lin(w[p + "o"], o)


def latent_attention(h, w, p, m, eps):
    """Keys and values of all heads from one normed latent c (kv_rank wide) plus ONE turned key part shared by the heads; queries from
    h directly, per head [dim plain | rot_dim turned] ("interleaved" pairs); causal softmax (a window if mask.size is given); the
    concatenated heads times sigmoid(W_g h) element by element."""
    T = h.shape[0]
    H, D, R, Dv, C, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["rot"]
    pos = torch.arange(T)
    q = lin(w[p + "q"], h).view(T, H, D + R)
    dkv = lin(w[p + "dkv"], h)
    c = rms(dkv[:, :C], eps) * w[p + "dkv.norm"].to(F64)
    kr = turn(dkv[:, C:].reshape(T, 1, R), pos, r["dims"], r["base"], "interleaved")[:, 0]
    qr = turn(q[..., D:], pos, r["dims"], r["base"], "interleaved")
    ku = lin(w[p + "uk"], c).view(T, H, D)
    v = lin(w[p + "uv"], c).view(T, H, Dv)
    d = pos.view(T, 1) - pos.view(1, T)
    size = (m.get("mask") or {}).get("size")
    seen = (d >= 0) & ((d < size) if size else True)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        s = (q[:, hh, :D] @ ku[:, hh].T + qr[:, hh] @ kr.T) * m["scale"]
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        out[:, hh] = torch.softmax(s, dim=-1) @ v[:, hh]
    return lin(w[p + "o"], out.reshape(T, H * Dv) * torch.sigmoid(lin(w[p + "g"], h)))


def window_attention(h, w, p, m, eps):
    """Grouped-query attention: weighted RMS norm over the WHOLE q and the whole k projection, then heads; q / k turned ("halves") on
    their first rot.dims entries; value j turned by j over all vdim entries, head outputs at i turned back by i; a sliding window; a
    softmax whose denominator also holds exp(sink_h)."""
    T = h.shape[0]
    H, G, D, Dv, r = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["rot"]
    pos = torch.arange(T)
    q = (rms(lin(w[p + "q"], h), eps) * w[p + "q.norm"].to(F64)).view(T, H, D)
    k = (rms(lin(w[p + "k"], h), eps) * w[p + "k.norm"].to(F64)).view(T, G, D)
    q, k = turn(q, pos, r["dims"], r["base"], "halves"), turn(k, pos, r["dims"], r["base"], "halves")
    v = turn(lin(w[p + "v"], h).view(T, G, Dv), pos, Dv, r["base"], "halves")
    d = pos.view(T, 1) - pos.view(1, T)
    size = (m.get("mask") or {}).get("size")
    seen = (d >= 0) & ((d < size) if size else True)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"]
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        sink = w[p + "sink"].to(F64)[hh]
        mx = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
        e = torch.exp(s - mx)
        out[:, hh] = (e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - mx))) @ v[:, g]
    out = turn(out, -pos, Dv, r["base"], "halves")
    return lin(w[p + "o"], out.reshape(T, H * Dv))


def dense_ff(h, w, p, ml):
    lim = ml["limit"]
    g = torch.clamp(lin(w[p + "gate"], h), max=lim)
    u = torch.clamp(lin(w[p + "up"], h), -lim, lim)
    return lin(w[p + "down"], g * torch.sigmoid(SWISH * g) * (u + 1.0))


def route(z, corr, top, groups, keep):
    """z [T, E] router logits -> (chosen experts [T, top], their weights).  s = sigmoid(z); the choice uses s + corr; a group's score is
    the sum of its two largest choice scores; experts outside the best `keep` groups count as -inf; weights = s of the chosen."""
    T, E = z.shape
    s = torch.sigmoid(z)
    ch = s + corr.to(F64)
    per = E // groups
    gs = ch.view(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1)
    kept = torch.zeros(T, groups, dtype=torch.bool)
    kept.scatter_(1, gs.topk(keep, dim=-1).indices, True)
    ch = torch.where(kept.repeat_interleave(per, dim=1), ch, torch.full_like(ch, -math.inf))
    idx = ch.topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def moe_ff(h, w, p, ml, round_input=None):
    r = ml["router"]
    g = r.get("groups") or {}
    idx, wt = route(lin(w[p + "router"], h), w[p + "correction"], r["top"], g.get("count", 1), g.get("keep", g.get("count", 1)))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, e in enumerate(idx[t].tolist()):
            q = p + f"e{e}."
            out[t] += wt[t, j] * lin(w[q + "down"], silu(lin(w[q + "gate"], h[t])) * lin(w[q + "up"], h[t]))
    return out


MIXERS = {"retention": retention, "latent_attention": latent_attention, "attention": window_attention}


def forward(cfg: dict, w: dict, tokens, residuals: list | None = None, round_input=None) -> torch.Tensor:
    """Logits [T, vocab] of every position.  residuals: receives x after every layer (after the depth average).  round_input: applied to
    every sublayer's input (what rounding of the inputs alone does to the statement)."""
    eps = cfg["norm"]["eps"]
    rd = round_input or (lambda t: t)
    one_plus = lambda v, n: rms(v, eps) * (1.0 + w[n].to(F64))
    x = w["embed"].to(F64)[torch.tensor(tokens)]
    X = [x]
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + one_plus(MIXERS[lc["type"]](rd(x), w, p + "mix.", lc["mixer"], eps), p + "norm1")
        ml = lc.get("mlp")
        if ml is not None:
            y = dense_ff(rd(x), w, p + "mlp.", ml) if ml["kind"] == "dense" else moe_ff(rd(x), w, p + "mlp.", ml)
            x = x + one_plus(y, p + "norm2")
        X.append(x)
        c = w[p + "dwa"].to(F64)
        x = sum(c[j] * X[j] for j in range(i + 2))
        if residuals is not None:
            residuals.append(x.clone())
    return lin(w["head"], one_plus(rd(x), "final.norm"))


# ------------------------------------------------------------------------------------------------------------------
# small configurations and random weights for the tests
def retention_layer(heads=2, dim=8, vdim=8, decay=None, rot_dims=None, base=10000.0, mlp=None):
    decay = decay if decay is not None else [1.0 - 2.0 ** -(2 + 6 * h / max(heads - 1, 1)) for h in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                                           "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}, "mlp": mlp}


def latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=12, scale=None, rot_dims=None, base=10000.0, mlp=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                                                  "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
                                                  "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}}, "mlp": mlp}


def attention_layer(heads=4, kv_heads=2, dim=8, vdim=8, scale=None, window=5, rot_dims=None, base=10000.0, mlp=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale if scale is not None else dim ** -0.5, "mask": {"size": window},
                                           "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}, "mlp": mlp}


def dense_mlp(ff=24, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_mlp(experts=4, top=2, ff=8, groups=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def make_config(layers, vocab=64, width=32, eps=1e-5):
    return {"architecture": "Dosuvik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def tensor_shapes(cfg: dict) -> list:
    W = cfg["width"]
    out = [("embed", (cfg["vocab"], W))]
    for i, lc in enumerate(cfg["layers"]):
        p, m, ml = f"l{i}.", lc["mixer"], lc.get("mlp")
        out += [(p + "norm1", (W,))] + ([(p + "norm2", (W,))] if ml is not None else [])
        if lc["type"] == "retention":
            n, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out += [(p + "mix.q", (n, W)), (p + "mix.k", (n, W)), (p + "mix.v", (nv, W)), (p + "mix.g", (nv, W)), (p + "mix.o", (W, nv))]
        elif lc["type"] == "latent_attention":
            nv = m["heads"] * m["vdim"]
            out += [(p + "mix.q", (m["heads"] * (m["dim"] + m["rot_dim"]), W)), (p + "mix.dkv", (m["kv_rank"] + m["rot_dim"], W)),
                    (p + "mix.dkv.norm", (m["kv_rank"],)), (p + "mix.uk", (m["heads"] * m["dim"], m["kv_rank"])),
                    (p + "mix.uv", (nv, m["kv_rank"])), (p + "mix.g", (nv, W)), (p + "mix.o", (W, nv))]
        else:
            nq, nk = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            out += [(p + "mix.q", (nq, W)), (p + "mix.k", (nk, W)), (p + "mix.v", (m["kv_heads"] * m["vdim"], W)), (p + "mix.q.norm", (nq,)),
                    (p + "mix.k.norm", (nk,)), (p + "mix.sink", (m["heads"],)), (p + "mix.o", (W, m["heads"] * m["vdim"]))]
        if ml is not None and ml["kind"] == "dense":
            out += [(p + "mlp.gate", (ml["ff"], W)), (p + "mlp.up", (ml["ff"], W)), (p + "mlp.down", (W, ml["ff"]))]
        elif ml is not None:
            E, ff = ml["router"]["experts"], ml["expert"]["ff"]
            for e in range(E):
                out += [(p + f"mlp.e{e}.gate", (ff, W)), (p + f"mlp.e{e}.up", (ff, W)), (p + f"mlp.e{e}.down", (W, ff))]
            out += [(p + "mlp.router", (E, W)), (p + "mlp.correction", (E,))]
        out.append((p + "dwa", (i + 2,)))
    return out + [("final.norm", (W,)), ("head", (cfg["vocab"], W))]


def random_model(cfg: dict, seed: int = 0) -> dict:
    """bf16 weights: matrices ~ N(0, 1 / fan_in) (attention inputs a little larger so that single keys carry the output), layer norms
    around zero, q / k / latent norms around one, sinks and corrections of the size of the scores they meet, depth weights that keep
    most of the newest result and some of every older one."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    w = {}
    for name, shape in tensor_shapes(cfg):
        if name.endswith((".norm1", ".norm2")) or name == "final.norm":
            t = 0.2 * rn(*shape)
        elif name.endswith(".norm"):
            t = 1.0 + 0.2 * rn(*shape)
        elif name.endswith(".sink"):
            t = 1.5 * rn(*shape)
        elif name.endswith(".correction"):
            t = 0.3 * rn(*shape)
        elif name.endswith(".dwa"):
            t = 0.25 * rn(*shape)
            t[-1] += 1.0
        elif name in ("embed",):
            t = rn(*shape)
        else:
            boost = 2.0 if name.endswith(("mix.q", "mix.k", "mix.dkv", "mlp.router")) else 1.0
            t = boost * rn(*shape) / math.sqrt(shape[-1])
        w[name] = t.to(torch.bfloat16)
    return w
