"""The HIP kernels behind the Fomunex decoder, one mechanism at a time, against plain fp64 torch statements of the same op (the
oracle's functions where one exists): embedding + position rows and the pre-norm tail, PolyNorm rows, the clamped swish-GLU with a
routing weight, the sigmoid router, logit scale + cap, the tanh GEMM epilogue, windowed attention with a sink over scattered pages
(scalar fp32 / bf16 and MFMA forms; prompt portions beside decoded rows; keys just inside and outside the window), token shift +
time-mixing scan and short convolution + state-space scan over state slots in portions (LDS and register forms), the grouped gate norm."""
import math

import pytest
import torch

from oracle import fomunex as F

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64


def H():
    from ssd_amd.hip import ops
    return ops


def rnd(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale)


def elem(f32):
    return torch.float32 if f32 else torch.bfloat16


def tol(f32):
    return dict(rtol=2e-5, atol=2e-5) if f32 else dict(rtol=2e-2, atol=2e-2)


d = lambda t: t.to(DEV).contiguous()


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("W", [40, 328])
def test_embed_position_rows_and_prenorm_tail(f32, W):
    T, V, P, top, eps = 9, 23, 31, 3, 1e-5
    el = elem(f32)
    table, pos, g1, g2 = rnd(V, W, seed=1).to(el), rnd(P, W, seed=2).to(el), torch.full((W,), 1.25).to(el), torch.full((W,), 0.75).to(el)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(4))
    ps = torch.randint(0, P, (T,), generator=torch.Generator().manual_seed(5))
    x = torch.zeros(T, W, device=DEV)
    hn = torch.zeros(T, W, dtype=el, device=DEV)
    H().embed_pos_res32(d(ids), d(ps), d(table), d(pos), x, T, W, f32, norm_weight=d(g1), eps=eps, norm_out=hn)
    ref = table.double()[ids] + pos.double()[ps]
    assert torch.allclose(x.cpu().double(), ref, **tol(True))
    assert torch.allclose(hn.cpu().double(), F.rms(ref, eps) * 1.25, **tol(f32))
    # x += y and the next norm; x += the sum of a token's expert rows (with and without weights), no next norm
    y = rnd(T, W, seed=6)
    H().prenorm_tail(x, eps, T, W, f32, y=d(y), next_weight=d(g2), next_out=hn)
    ref = ref + y.double()
    assert torch.allclose(x.cpu().double(), ref, **tol(True))
    assert torch.allclose(hn.cpu().double(), F.rms(ref, eps) * 0.75, **tol(f32))
    ydn, wt = rnd(T * top, W, seed=8), rnd(T, top, seed=10).abs()
    inv = torch.randperm(T * top, generator=torch.Generator().manual_seed(11)).to(torch.int32)
    H().prenorm_tail(x, eps, T, W, f32, ydn=d(ydn), inv=d(inv), top=top)
    ref = ref + ydn.double()[inv.long()].view(T, top, W).sum(1)
    assert torch.allclose(x.cpu().double(), ref, **tol(True))
    H().prenorm_tail(x, eps, T, W, f32, ydn=d(ydn), inv=d(inv), weights=d(wt), top=top, next_weight=d(g1), next_out=hn)
    ref = ref + (ydn.double()[inv.long()].view(T, top, W) * wt.double().unsqueeze(-1)).sum(1)
    assert torch.allclose(x.cpu().double(), ref, **tol(True))
    assert torch.allclose(hn.cpu().double(), F.rms(ref, eps) * 1.25, **tol(f32))


@pytest.mark.parametrize("f32", [True, False])
def test_polynorm_clamped_glu_router_and_logit_cap(f32):
    T, Fd, eps = 11, 300, 1e-5
    el = elem(f32)
    z = rnd(T, Fd, seed=1, scale=2.0)
    coef = torch.tensor([0.9, 0.4, -0.3, 0.1])
    out = torch.zeros(T, Fd, dtype=el, device=DEV)
    H().polynorm_rows(d(z), d(coef), eps, out, T, Fd, f32)
    zd = z.double()
    ref = 0.9 * F.rms(zd, eps) + 0.4 * F.rms(zd ** 2, eps) - 0.3 * F.rms(zd ** 3, eps) + 0.1
    assert torch.allclose(out.cpu().double(), ref, **tol(f32))
    # clamped GLU: the per-row factor comes through the sort's permutation
    ab, scale = rnd(T, 2 * Fd, seed=2, scale=2.0), rnd(T, seed=3).abs()
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(4)).to(torch.int32)
    limit = 1.25
    H().glu_clamp_rows(d(ab), out, T, Fd, limit, 1.702, f32, row_scale=d(scale), perm=d(perm))
    s = scale.double()[perm.long()].unsqueeze(-1)
    g = torch.clamp(s * ab.double()[:, :Fd], max=limit)
    u = torch.clamp(s * ab.double()[:, Fd:], min=-limit, max=limit)
    assert torch.allclose(out.cpu().double(), g * torch.sigmoid(1.702 * g) * (u + 1), **tol(f32))
    H().glu_clamp_rows(d(ab), out, T, Fd, limit, 1.702, f32)
    g, u = torch.clamp(ab.double()[:, :Fd], max=limit), torch.clamp(ab.double()[:, Fd:], min=-limit, max=limit)
    assert torch.allclose(out.cpu().double(), g * torch.sigmoid(1.702 * g) * (u + 1), **tol(f32))
    if not f32:
        return
    # sigmoid router: the top largest scores as they are, lowest index at a tie; a row stride larger than E
    E, top, ld = 70, 5, 75
    lg = rnd(T, ld, seed=5, scale=2.0)
    lg[3, 7] = lg[3, 60] = 9.0
    idx = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wt = torch.zeros(T, top, device=DEV)
    H().moe_route_sigmoid(d(lg), ld, idx, wt, T, E, top)
    sc = torch.sigmoid(lg[:, :E].double())
    tv, ti = torch.sort(sc, dim=-1, descending=True, stable=True)
    assert torch.equal(idx.cpu().long(), ti[:, :top]) and idx[3, 0] == 7 and idx[3, 1] == 60
    assert torch.allclose(wt.cpu().double(), tv[:, :top], rtol=1e-6, atol=1e-7)
    # logits: scale, then cap; cap 0 = scale only
    V = 3000
    l0 = rnd(T, V, seed=6, scale=20.0)
    l1 = d(l0)
    H().logits_cap_rows(l1, T, V, V, 1.5, 30.0)
    assert torch.allclose(l1.cpu().double(), 30.0 * torch.tanh(1.5 * l0.double() / 30.0), rtol=1e-5, atol=1e-5)
    l1 = d(l0)
    H().logits_cap_rows(l1, T, V, V, 0.5, 0.0)
    assert torch.allclose(l1.cpu().double(), 0.5 * l0.double(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("f32", [True, False])
def test_gemm_with_tanh_epilogue_over_a_column_slice(f32):
    """The decay's first matrix reads one of five interpolations that lie side by side in a row, and its output passes through tanh."""
    T, W, R = 21, 72, 6
    el = elem(f32)
    x, w = rnd(T, 5 * W, seed=1).to(el), rnd(R, W, seed=2, scale=0.2).to(el)
    xd = d(x).view(-1)
    out = torch.zeros(T, R, dtype=el, device=DEV)
    H().gemm_rows_batched(xd[4 * W:], d(w), out, T, R, W, 1, 5 * W, 0, R, 0, f32, H().GR_TANH)
    ref = torch.tanh(x.double()[:, 4 * W:] @ w.double().T)
    assert torch.allclose(out.cpu().double(), ref, **tol(f32))


def attention_reference(q, k, v, sinks, slopes, window, scale, cap, eps):
    """q [n][H][D], k [n][G][D], v [n][G][Dv] of ONE sequence (raw projections) -> [n][H][Dv] in fp64."""
    n, Hh, D = q.shape
    G = k.shape[1]
    q, k = F.rms(q.double(), eps), F.rms(k.double(), eps)
    i, j = torch.arange(n).view(n, 1), torch.arange(n).view(1, n)
    seen = (i >= j) & ((i - j < window) if window else True)
    out = torch.zeros(n, Hh, v.shape[-1], dtype=F64)
    for h in range(Hh):
        g = h // (Hh // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s - slopes[h].double() * (i - j)
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        e = torch.exp(s)
        den = e.sum(-1, keepdim=True) + (torch.exp(sinks[h].double()) if sinks is not None else 0.0)
        out[:, h] = (e / den) @ v.double()[:, g]
    return out


ATT_CASES = [
    # f32, H, G, D, Dv, window, cap, block, use max_q (MFMA where it fits)
    (True, 4, 2, 16, 24, 9, 12.0, 16, False),
    (True, 3, 1, 24, 8, 0, 0.0, 16, False),
    (False, 6, 3, 12, 10, 33, 5.0, 16, True),           # sizes the MFMA form refuses: scalar bf16
    (False, 8, 2, 32, 16, 40, 12.0, 32, True),          # MFMA: 4 rows per token
    (False, 4, 4, 64, 64, 70, 0.0, 64, True),           # MFMA: one row per token, no cap
    (False, 20, 1, 32, 32, 0, 20.0, 32, True),          # MFMA: more rows per token than a wave's tile, no window
    (False, 2, 1, 128, 128, 64, 8.0, 32, True),
    (False, 1, 1, 256, 256, 17, 8.0, 32, True),
]


@pytest.mark.parametrize("case", ATT_CASES)
def test_windowed_attention_with_sink_over_scattered_pages(case):
    """Three sequences in one varlen batch -- a prompt portion that continues an earlier one, a whole short prompt, one decoded row --
    over pages handed out in scattered order; sharp scores, so a key just inside or outside the window or a missing sink shows."""
    f32, Hh, G, D, Dv, window, cap, bs, use_mq = case
    el, eps, scale = elem(f32), 1e-5, 6.0 / math.sqrt(D) * 4
    lens, new = [150, 37, 101], [53, 37, 1]                 # context length after this step, rows this step brings
    nb = sum(-(-n // bs) for n in lens) + 3
    max_blocks = max(-(-n // bs) for n in lens)
    kc = torch.full((nb, G, bs, D), float("nan"), dtype=el, device=DEV)
    vc = torch.full((nb, G, Dv, bs), float("nan"), dtype=el, device=DEV)
    pages = torch.randperm(nb, generator=torch.Generator().manual_seed(1)).tolist()
    bt = torch.zeros(len(lens), max_blocks, dtype=torch.int32)
    sinks, slopes = rnd(Hh, seed=2), torch.tensor([2.0 ** (-8.0 * (h + 1) / Hh) for h in range(Hh)])
    NP = (Hh + G) * D + G * Dv
    refs, rows, pos, slots, cu = [], [], [], [], [0]
    for b, (n, k) in enumerate(zip(lens, new)):
        proj = rnd(n, NP, seed=10 + b)
        mine = [pages.pop() for _ in range(-(-n // bs))]
        bt[b, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        sl = torch.tensor([mine[p // bs] * bs + p % bs for p in range(n)], dtype=torch.int32)
        if n > k:        # earlier portion: stored by a call of its own
            qd = torch.zeros(n - k, Hh * D, dtype=el, device=DEV)
            H().winattn_store(d(proj[:n - k]), NP, eps, d(sl[:n - k]), qd, kc, vc, n - k, Hh, G, D, Dv, bs, f32)
        full = attention_reference(proj[:, :Hh * D].view(n, Hh, D), proj[:, Hh * D:(Hh + G) * D].view(n, G, D),
                                   proj[:, (Hh + G) * D:].view(n, G, Dv), sinks, slopes, window, scale, cap, eps)
        refs.append(full[n - k:])
        rows.append(proj[n - k:])
        pos += list(range(n - k, n))
        slots.append(sl[n - k:])
        cu.append(cu[-1] + k)
    T = cu[-1]
    q = torch.zeros(T, Hh * D, dtype=el, device=DEV)
    out = torch.zeros(T, Hh * Dv, dtype=el, device=DEV)
    H().winattn_store(d(torch.cat(rows)), NP, eps, d(torch.cat(slots)), q, kc, vc, T, Hh, G, D, Dv, bs, f32)
    H().winattn_paged(q, kc, vc, d(slopes), d(sinks), d(bt), max_blocks, d(torch.tensor(pos)), len(lens), T, Hh, G, D, Dv, bs, window, scale,
                      cap, out, f32, cu_q=d(torch.tensor(cu, dtype=torch.int32)), max_q=max(new) if use_mq else 0)
    ref = torch.cat(refs).view(T, Hh * Dv)
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    if f32:
        assert torch.allclose(got, ref, rtol=1e-4, atol=1e-5), float((got - ref).abs().max())
        if window:      # the statement is sharp: one key more or fewer is far away
            other = attention_reference(rnd(lens[0], NP, seed=10)[:, :Hh * D].view(lens[0], Hh, D),
                                        rnd(lens[0], NP, seed=10)[:, Hh * D:(Hh + G) * D].view(lens[0], G, D),
                                        rnd(lens[0], NP, seed=10)[:, (Hh + G) * D:].view(lens[0], G, Dv), sinks, slopes, window + 1, scale, cap, eps)
            assert float((other[lens[0] - new[0]:].reshape(new[0], -1) - ref[:new[0]]).abs().max()) > 1e-2
    else:
        assert float((got - ref).abs().max()) < 0.06 * float(ref.abs().max()), float((got - ref).abs().max())
        assert float((got - ref).pow(2).mean().sqrt()) < 0.01 * float(ref.pow(2).mean().sqrt()) + 1e-3


def wkv_reference(r, k, v, ww, w0, u):
    """One sequence and head: r, k, v, ww [n][D] -> o [n][D] (fp64) and the final state."""
    n, D = r.shape
    S = torch.zeros(D, D, dtype=F64)
    o = torch.zeros(n, D, dtype=F64)
    for t in range(n):
        kv = torch.outer(k[t], v[t])
        o[t] = (S + u.view(D, 1) * kv).T @ r[t]
        S = torch.exp(-torch.exp(ww[t] + w0)).view(D, 1) * S + kv
    return o, S


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("Hh,D", [(3, 12), (2, 32), (1, 64), (2, 128)])
def test_token_shift_and_time_mixing_scan_in_portions_over_slots(f32, Hh, D):
    """Two sequences in slots 2 and 0 of a pool that holds stale numbers; the first arrives in portions of 1, 2, 9 and 30 rows (beside
    the second one's rows), and the rows equal the whole-sequence statement; so do the saved token-shift rows."""
    el, W, N = elem(f32), 40, Hh * D
    nA, nB = 42, 17
    g = torch.Generator().manual_seed(7)
    hnA, hnB = rnd(nA, W, seed=1).to(el), rnd(nB, W, seed=2).to(el)
    mu = torch.rand(5, W, generator=g).to(el)
    projA, projB = rnd(nA, 4 * N, seed=3, scale=0.7), rnd(nB, 4 * N, seed=4, scale=0.7)
    wwA, wwB = rnd(nA, N, seed=5), rnd(nB, N, seed=6)
    w0, u = -6.0 + 6.5 * torch.rand(N, generator=g), rnd(N, seed=8, scale=0.5)
    state = torch.full((3, Hh, D, D), 7.0, device=DEV)
    shift = torch.full((3, W), 7.0, device=DEV)
    outA, outB, mixA = [], [], []
    plan = [(1, 5), (2, 1), (9, 0), (30, 11)]
    a = b = 0
    for ka, kb in plan:
        rowsA, rowsB = slice(a, a + ka), slice(b, b + kb)
        T = ka + kb
        hn = d(torch.cat([hnA[rowsA], hnB[rowsB]]))
        proj, ww = d(torch.cat([projA[rowsA], projB[rowsB]])), d(torch.cat([wwA[rowsA], wwB[rowsB]]))
        pos = d(torch.tensor(list(range(a, a + ka)) + list(range(b, b + kb))))
        seqs = [(2, ka)] + ([(0, kb)] if kb else [])
        cu = d(torch.tensor([0] + list(torch.tensor([k for _, k in seqs]).cumsum(0)), dtype=torch.int32))
        sl = d(torch.tensor([s for s, _ in seqs], dtype=torch.int32))
        mix = torch.zeros(T, 5 * W, dtype=el, device=DEV)
        out = torch.zeros(T, N, device=DEV)
        H().token_shift_mix(hn, d(mu), shift, pos, sl, len(seqs), mix, T, W, 5, f32, cu_q=cu)
        H().wkv_scan(proj, 4 * N, 0, N, 2 * N, ww, N, d(w0), d(u), pos, sl, state, out, hn, shift, W, len(seqs), Hh, D, f32, cu_q=cu)
        outA.append(out[:ka].cpu())
        outB.append(out[ka:].cpu())
        mixA.append(mix[:ka].cpu())
        a, b = a + ka, b + kb
    assert a == nA and b == nB
    for proj, ww, n, got, slot in ((projA, wwA, nA, torch.cat(outA), 2), (projB, wwB, nB, torch.cat(outB), 0)):
        for h in range(Hh):
            c = slice(h * D, (h + 1) * D)
            ref, S = wkv_reference(proj.double()[:, c], proj.double()[:, N + h * D:N + (h + 1) * D], proj.double()[:, 2 * N + h * D:2 * N + (h + 1) * D],
                                   ww.double()[:, c], w0.double()[c], u.double()[c])
            assert torch.allclose(got.double()[:, c], ref, rtol=2e-4, atol=2e-4), float((got.double()[:, c] - ref).abs().max())
            assert torch.allclose(state[slot, h].cpu().double(), S, rtol=2e-4, atol=2e-4)
    assert float(state[1].min()) == 7.0 and float(shift[1].min()) == 7.0          # the slot nobody holds is untouched
    prev = torch.cat([torch.zeros(1, W, dtype=F64), hnA.double()[:-1]])
    ref = torch.stack([hnA.double() + (prev - hnA.double()) * mu.double()[s] for s in range(5)], dim=1).view(nA, 5 * W)
    assert torch.allclose(torch.cat(mixA).double(), ref, **tol(f32))
    assert torch.equal(shift[2].cpu(), hnA[-1].float()) and torch.equal(shift[0].cpu(), hnB[-1].float())


@pytest.mark.parametrize("Hh,G,N,Dv,taps", [(4, 2, 6, 10, 4), (2, 1, 32, 32, 2), (4, 2, 64, 64, 3), (2, 2, 128, 32, 1), (3, 3, 8, 20, 7)])
def test_convolution_and_state_space_scan_in_portions_over_slots(Hh, G, N, Dv, taps):
    """The same two-sequence plan for the state-space mixer: portions shorter than the convolution's reach (1 and 2 rows), the saved
    inputs, the state, stale slots; against the oracle's mixer statement fed with the same projection rows."""
    inner, GN = Hh * Dv, G * N
    C, NP = inner + 2 * GN, 2 * inner + 2 * GN + Hh
    nA, nB = 42, 17
    g = torch.Generator().manual_seed(3)
    projA, projB = rnd(nA, NP, seed=1), rnd(nB, NP, seed=2)
    cw, cb = rnd(C, taps, seed=3, scale=1 / math.sqrt(taps)), rnd(C, seed=4, scale=0.2)
    dtb, alog, skip = -4.0 + 4.5 * torch.rand(Hh, generator=g), -3.0 + 4.0 * torch.rand(Hh, generator=g), rnd(Hh, seed=5)
    state = torch.full((3, Hh, N, Dv), 7.0, device=DEV)
    conv = torch.full((3, max(taps - 1, 1), C), 7.0, device=DEV)
    outA, outB = [], []
    a = b = 0
    for ka, kb in [(1, 5), (2, 1), (9, 0), (30, 11)]:
        T = ka + kb
        proj = d(torch.cat([projA[a:a + ka], projB[b:b + kb]]))
        pos = d(torch.tensor(list(range(a, a + ka)) + list(range(b, b + kb))))
        seqs = [(2, ka)] + ([(0, kb)] if kb else [])
        cu = d(torch.tensor([0] + list(torch.tensor([k for _, k in seqs]).cumsum(0)), dtype=torch.int32))
        sl = d(torch.tensor([s for s, _ in seqs], dtype=torch.int32))
        xbc = torch.zeros(T, C, device=DEV)
        out = torch.zeros(T, inner, device=DEV)
        H().causal_conv_silu(proj, NP, inner, C, d(cw), d(cb), conv, pos, sl, len(seqs), xbc, T, taps, True, cu_q=cu)
        H().ssd_scan(xbc, C, 0, inner, inner + GN, proj, NP, 2 * inner + 2 * GN, d(dtb), d(alog), d(skip), pos, sl, state, out, inner, C, conv,
                     taps, len(seqs), Hh, G, N, Dv, cu_q=cu)
        outA.append(out[:ka].cpu())
        outB.append(out[ka:].cpu())
        a, b = a + ka, b + kb

    def reference(proj):
        n = proj.shape[0]
        p = proj.double()
        pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), p[:, inner:inner + C]])
        xbc = F.silu(cb.double() + sum(pad[c:c + n] * cw.double()[:, c] for c in range(taps)))
        dt = F.softplus(p[:, 2 * inner + 2 * GN:] + dtb.double())
        y = torch.zeros(n, Hh, Dv, dtype=F64)
        for h in range(Hh):
            gi = h // (Hh // G)
            S = torch.zeros(N, Dv, dtype=F64)
            for t in range(n):
                x = xbc[t, h * Dv:(h + 1) * Dv]
                S = torch.exp(-torch.exp(alog.double()[h]) * dt[t, h]) * S + dt[t, h] * torch.outer(xbc[t, inner + gi * N:inner + (gi + 1) * N], x)
                y[t, h] = S.T @ xbc[t, inner + GN + gi * N:inner + GN + (gi + 1) * N] + skip.double()[h] * x
        return y.view(n, inner)

    for proj, got in ((projA, torch.cat(outA)), (projB, torch.cat(outB))):
        ref = reference(proj)
        assert torch.allclose(got.double(), ref, rtol=2e-4, atol=2e-4), float((got.double() - ref).abs().max())
    assert float(state[1].min()) == 7.0 and float(conv[1].min()) == 7.0
    if taps > 1:
        assert torch.equal(conv[2].cpu(), projA[-(taps - 1):, inner:inner + C]) and torch.equal(conv[0].cpu(), projB[-(taps - 1):, inner:inner + C])


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("groups,gate_first", [(1, True), (4, True), (6, False), (24, False)])
def test_grouped_gate_norm(f32, groups, gate_first):
    T, N, ld, eps = 7, 240, 300, 1e-5
    el = elem(f32)
    o, gate, w = rnd(T, N, seed=1, scale=3.0), rnd(T, ld, seed=2), (1 + 0.1 * rnd(N, seed=3)).to(el)
    out = torch.zeros(T, N, dtype=el, device=DEV)
    H().group_gate_norm(d(o), d(gate).view(-1)[40:], ld, d(w), eps, out, T, N, groups, gate_first, f32)
    gs = F.silu(torch.cat([gate.view(-1)[40:], torch.zeros(40)]).view(T, ld)[:, :N].double())
    od = o.double()
    if gate_first:
        ref = F.rms((od * gs).view(T, groups, -1), eps).view(T, N) * w.double()
    else:
        ref = F.rms(od.view(T, groups, -1), eps).view(T, N) * w.double() * gs
    assert torch.allclose(out.cpu().double(), ref, **tol(f32))


@pytest.mark.parametrize("rows_per_token", [1, 3])
@pytest.mark.parametrize("T", [5, 150])
def test_grouped_gemm_with_the_clamped_glu_as_epilogue(T, rows_per_token):
    """bf16: experts' [gate | up] product over rows sorted by expert, the routing weight and the clamps applied to the fp32 accumulators
    (weight rows in (gate, up) pairs) -- few rows (the skinny form) and many (the tile form), against the two-step fp64 statement."""
    E, W, ff, top, limit = 4, 72, 40, rows_per_token, 1.25
    g = torch.Generator().manual_seed(T)
    x = rnd(T, W, seed=1).to(torch.bfloat16)
    gate, up = rnd(E, ff, W, seed=2, scale=0.3).to(torch.bfloat16), rnd(E, ff, W, seed=3, scale=0.3).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wt = torch.rand(T, top, generator=g)
    off = torch.zeros(E + 1, dtype=torch.int32, device=DEV)
    perm = torch.zeros(T * top, dtype=torch.int32, device=DEV)
    inv = torch.zeros(T * top, dtype=torch.int32, device=DEV)
    H().moe_plan(d(idx), T, top, E, off, perm, inv)
    pairs = torch.stack([gate, up], dim=2).reshape(E, 2 * ff, W)
    out = torch.zeros(T * top, ff, dtype=torch.bfloat16, device=DEV)
    H().gemm_rows_grouped_glu_clamp(d(x), d(pairs), out, off, E, T * top, 2 * ff, W, limit, 1.702, row_idx=perm, idx_div=top, row_scale=d(wt))
    got = out.cpu().double()[inv.cpu().long()].view(T, top, ff)
    for t in range(T):
        for j in range(top):
            e, s = int(idx[t, j]), wt[t, j].double()
            gg = torch.clamp(s * (gate[e].double() @ x[t].double()), max=limit)
            uu = torch.clamp(s * (up[e].double() @ x[t].double()), min=-limit, max=limit)
            ref = gg * torch.sigmoid(1.702 * gg) * (uu + 1)
            assert torch.allclose(got[t, j], ref, rtol=2e-2, atol=2e-2), (t, j, float((got[t, j] - ref).abs().max()))
