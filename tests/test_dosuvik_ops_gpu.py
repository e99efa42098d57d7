"""The HIP kernels behind the Dosuvik decoder, one mechanism at a time, against plain fp64 torch statements of the same op (the
oracle's functions where one exists): embedding rows + the output-norm tail with the depth average, the last norm with fp32 weights,
rotary rows in place, gate rows, the grouped sigmoid router with a choice correction, the dense clamped-GLU GEMM epilogue, the raw-input
scan over state slots in portions (LDS and register forms), and the rotary store + windowed attention with rotated values and a sink
over scattered pages (scalar fp32 / bf16 and MFMA forms; prompt portions beside decoded rows; keys just inside and outside the window)."""
import math

import pytest
import torch

from oracle import dosuvik as F

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
# the last case: a row too wide for the registers that keep the routed mix between the statistic and the sum (it is computed twice)
@pytest.mark.parametrize("W,T", [(40, 9), (328, 9), (2304, 5), (4352, 70)])
def test_embedding_rows_output_norm_tail_and_depth_average(f32, W, T):
    V, top, eps, levels, Tmax = 23, 3, 1e-5, 4, T + 7
    el = elem(f32)
    table = rnd(V, W, seed=1).to(el)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(4))
    x = torch.zeros(T, W, device=DEV)
    hist = torch.full((levels, Tmax, W), float("nan"), device=DEV)
    hn = torch.zeros(T, W, dtype=el, device=DEV)
    H().embed_hist(d(ids), d(table), x, T, W, f32, hist0=hist, rows_out=hn)
    X = [table.double()[ids]]
    assert torch.equal(x.cpu().double(), X[0]) and torch.equal(hist[0, :T].cpu().double(), X[0]) and torch.equal(hn.cpu().double(), X[0])
    ref = X[0]
    for lvl in range(1, levels):
        # a mixer's output: x += w * rms(y), no average; then the routed feed-forward's rows and the layer's end
        w1, w2 = 1.0 + rnd(W, seed=10 + lvl, scale=0.2), 1.0 + rnd(W, seed=20 + lvl, scale=0.2)
        y = rnd(T, W, seed=30 + lvl, scale=3.0)
        H().postnorm_tail(x, d(w1), eps, T, W, f32, y=d(y), next_out=hn)
        ref = ref + F.rms(y.double(), eps) * w1.double()
        assert torch.allclose(x.cpu().double(), ref, **tol(True))
        assert torch.allclose(hn.cpu().double(), ref, **tol(f32))
        ydn, wt = rnd(T * top, W, seed=40 + lvl), rnd(T, top, seed=50 + lvl).abs()
        inv = torch.randperm(T * top, generator=torch.Generator().manual_seed(60 + lvl)).to(torch.int32)
        coef = rnd(lvl + 1, seed=70 + lvl)
        H().postnorm_tail(x, d(w2), eps, T, W, f32, ydn=d(ydn), inv=d(inv), weights=d(wt.reshape(-1)), top=top, hist=hist,
                          hist_stride=Tmax * W, hist_levels=lvl + 1, coef=d(coef), next_out=hn)
        mix = (wt.double().unsqueeze(-1) * ydn.double()[inv.long()].view(T, top, W)).sum(1)
        X.append(ref + F.rms(mix, eps) * w2.double())
        assert torch.allclose(hist[lvl, :T].cpu().double(), X[lvl], **tol(True))
        ref = sum(coef.double()[j] * X[j] for j in range(lvl + 1))
        assert torch.allclose(x.cpu().double(), ref, rtol=1e-4, atol=1e-4)
        assert torch.allclose(hn.cpu().double(), ref, **tol(f32))
    # the last norm: fp32 weights, a gather of rows
    wf = 1.0 + rnd(W, seed=90, scale=0.3)
    pick = torch.tensor([T - 1, 0, 2], dtype=torch.int32)
    out = torch.zeros(3, W, dtype=el, device=DEV)
    H().rmsnorm_w32_rows(x, d(wf), eps, out, 3, W, f32, gather=d(pick))
    assert torch.allclose(out.cpu().double(), F.rms(x.cpu().double()[pick.long()], eps) * wf.double(), **tol(f32))


@pytest.mark.parametrize("heads,D,dims", [(3, 8, 8), (2, 24, 10), (1, 64, 0), (5, 6, 2)])
def test_rotary_rows_in_place_on_two_blocks(heads, D, dims):
    T, base, extra = 11, 1000.0, 7
    ld = 2 * heads * D + extra
    rows = rnd(T, ld, seed=1)
    pos = torch.randint(0, 5000, (T,), generator=torch.Generator().manual_seed(2))
    freqs = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)] or [0.0], dtype=F64).float()
    buf = d(rows.clone())
    H().rope_rows(buf, ld, d(pos), d(freqs), dims, heads, D, T, 0, 1.0, heads * D, D ** -0.5)
    got = buf.cpu().double()
    q = F.turn(rows[:, :heads * D].double().view(T, heads, D), pos, dims, base, "halves").reshape(T, -1)
    k = F.turn(rows[:, heads * D:2 * heads * D].double().view(T, heads, D), pos, dims, base, "halves").reshape(T, -1) * D ** -0.5
    # the angle is a float32 product of a position in the thousands: its rounding alone is ~1e-4 rad
    assert torch.allclose(got[:, :heads * D], q, rtol=1e-3, atol=1e-3) and torch.allclose(got[:, heads * D:2 * heads * D], k, rtol=1e-3, atol=1e-3)
    assert torch.equal(got[:, 2 * heads * D:], rows[:, 2 * heads * D:].double())
    small = torch.arange(T)
    buf = d(rows.clone())
    H().rope_rows(buf, ld, d(small), d(freqs), dims, heads, D, T, heads * D)
    assert torch.allclose(buf.cpu().double()[:, heads * D:2 * heads * D],
                          F.turn(rows[:, heads * D:2 * heads * D].double().view(T, heads, D), small, dims, base, "halves").reshape(T, -1), **tol(True))
    assert torch.equal(buf.cpu()[:, :heads * D], rows[:, :heads * D])


@pytest.mark.parametrize("f32", [True, False])
def test_gate_rows(f32):
    T, N = 7, 300
    o, g = rnd(T, N + 5, seed=1), rnd(T, N + 9, seed=2, scale=3.0)
    out = torch.zeros(T, N, dtype=elem(f32), device=DEV)
    H().gate_rows(d(o), N + 5, d(g), N + 9, out, T, N, f32)
    assert torch.allclose(out.cpu().double(), o[:, :N].double() * torch.sigmoid(g[:, :N].double()), **tol(f32))


@pytest.mark.parametrize("E,top,groups,keep", [(10, 4, 2, 1), (12, 3, 4, 2), (6, 2, 1, 1), (8, 8, 2, 2), (9, 2, 9, 3), (5, 1, 5, 1), (64, 6, 8, 3)])
def test_grouped_sigmoid_router_with_choice_correction(E, top, groups, keep):
    """Corrections large enough that the choice differs from the plain scores' order, and negative enough that choice scores of whole
    groups are negative (an excluded expert must count as -inf, not 0)."""
    T = 200
    z = rnd(T, E + 3, seed=E + top, scale=2.0)
    corr = rnd(E, seed=groups, scale=0.6) - 0.8
    idx = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wt = torch.zeros(T, top, device=DEV)
    H().moe_route_sigmoid_grouped(d(z), E + 3, d(corr), idx, wt, T, E, top, groups, keep, 2)
    ri, rw = F.route(z[:, :E].double(), corr, top, groups, keep)
    assert torch.equal(idx.cpu().long(), ri)
    assert torch.allclose(wt.cpu().double(), rw, rtol=1e-6, atol=1e-7)
    plain = torch.sigmoid(z[:, :E].double()).topk(top, dim=-1).indices
    if E > top:
        assert not torch.equal(plain, ri)           # the correction and the groups decide something here


@pytest.mark.parametrize("T", [3, 70])
def test_dense_gemm_with_the_clamped_glu_as_epilogue(T):
    W, ff, limit, alpha = 96, 40, 0.8, 1.702
    x = rnd(T, W, seed=1).to(torch.bfloat16)
    gate, up = rnd(ff, W, seed=2, scale=0.3).to(torch.bfloat16), rnd(ff, W, seed=3, scale=0.3).to(torch.bfloat16)
    gu = torch.stack([gate, up], dim=1).reshape(2 * ff, W)
    out = torch.zeros(T, ff, dtype=torch.bfloat16, device=DEV)
    H().gemm_rows_glu_clamp(d(x), d(gu), out, T, 2 * ff, W, limit, alpha)
    g = torch.clamp(x.double() @ gate.double().T, max=limit)
    u = torch.clamp(x.double() @ up.double().T, -limit, limit)
    ref = g * torch.sigmoid(alpha * g) * (u + 1.0)
    assert (g == limit).any() and (u.abs() == limit).any()
    assert torch.allclose(out.cpu().double(), ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("Hh,D,Dv", [(3, 12, 20), (2, 32, 64), (1, 64, 32)])
def test_raw_input_scan_in_portions_over_slots(Hh, D, Dv):
    """Two sequences over state slots 2 and 0 (filled with NaN: a sequence that starts at position 0 must not read them), the first in
    three portions, the second whole; the rows as they are (no activation), against the recurrence."""
    lens, slots_of = [37, 9], [2, 0]
    decay = torch.tensor([1.0 - 2.0 ** -(2 + h) for h in range(Hh)])
    NP = 2 * Hh * D + Hh * Dv + 5
    state = torch.full((3, Hh, D, Dv), float("nan"), device=DEV)
    projs = [rnd(n, NP, seed=3 + b, scale=0.5) for b, n in enumerate(lens)]

    def reference(p):
        n = p.shape[0]
        q, k, v = p[:, :Hh * D].double().view(n, Hh, D), p[:, Hh * D:2 * Hh * D].double().view(n, Hh, D), p[:, 2 * Hh * D:2 * Hh * D + Hh * Dv].double().view(n, Hh, Dv)
        o = torch.zeros(n, Hh, Dv, dtype=F64)
        for h in range(Hh):
            S = torch.zeros(D, Dv, dtype=F64)
            for t in range(n):
                S = decay.double()[h] * S + torch.outer(k[t, h], v[t, h])
                o[t, h] = S.T @ q[t, h]
        return o.reshape(n, -1)

    refs = [reference(p) for p in projs]
    got = [[], []]
    for step in ([(0, 0, 20), (1, 0, 9)], [(0, 20, 21)], [(0, 21, 37)]):
        rows = torch.cat([projs[b][lo:hi] for b, lo, hi in step])
        pos = torch.cat([torch.arange(lo, hi) for _, lo, hi in step])
        cu = torch.tensor([0] + list(torch.tensor([hi - lo for _, lo, hi in step]).cumsum(0)), dtype=torch.int32)
        out = torch.zeros(rows.shape[0], Hh * Dv, device=DEV)
        H().lightning_scan(d(rows), NP, 0, Hh * D, 2 * Hh * D, d(decay), d(pos), d(torch.tensor([slots_of[b] for b, _, _ in step], dtype=torch.int32)),
                           state, out, len(step), Hh, D, Dv, cu_q=d(cu), act=H().SCAN_RAW)
        at = 0
        for b, lo, hi in step:
            got[b].append(out[at:at + hi - lo].cpu().double())
            at += hi - lo
    for b in range(2):
        assert torch.allclose(torch.cat(got[b]), refs[b], rtol=1e-4, atol=1e-4)
    assert torch.isnan(state[1]).all()


def attention_reference(q, k, v, wq, wk, sinks, window, scale, eps, dims, base):
    """q [n][H][D], k [n][G][D], v [n][G][Dv] of one sequence, as projected -> the heads' outputs [n][H][Dv] (fp64)."""
    n, Hh, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    pos = torch.arange(n)
    q = (F.rms(q.double().reshape(n, -1), eps) * wq.double()).view(n, Hh, D)
    k = (F.rms(k.double().reshape(n, -1), eps) * wk.double()).view(n, G, D)
    q, k = F.turn(q, pos, dims, base, "halves"), F.turn(k, pos, dims, base, "halves")
    v = F.turn(v.double(), pos, Dv, base, "halves")
    dist = pos.view(n, 1) - pos.view(1, n)
    seen = (dist >= 0) & ((dist < window) if window else True)
    out = torch.zeros(n, Hh, Dv, dtype=F64)
    for h in range(Hh):
        g = h // (Hh // G)
        s = torch.where(seen, (q[:, h] @ k[:, g].T) * scale, torch.full((n, n), -math.inf, dtype=F64))
        sink = sinks.double()[h]
        mx = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
        e = torch.exp(s - mx)
        out[:, h] = (e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - mx))) @ v[:, g]
    return F.turn(out, -pos, Dv, base, "halves")


ATT_CASES = [
    # f32, H, G, D, Dv, window, rot dims, block, MFMA form
    (True, 4, 2, 12, 6, 7, 8, 16, False), (True, 3, 1, 24, 10, 33, 24, 16, False), (True, 2, 2, 8, 4, 0, 0, 16, False),
    (False, 4, 2, 12, 6, 7, 8, 16, False), (False, 8, 2, 32, 64, 44, 32, 32, True), (False, 4, 4, 64, 32, 70, 16, 64, True),
    (False, 6, 1, 32, 96, 0, 32, 32, True), (False, 2, 1, 128, 128, 50, 64, 32, True), (False, 2, 2, 32, 32, 1, 32, 32, True),
]


@pytest.mark.parametrize("case", ATT_CASES)
def test_rotary_store_and_windowed_attention_with_rotated_values_over_scattered_pages(case):
    """Three sequences in one varlen batch -- a prompt portion that continues an earlier one, a whole short prompt, one decoded row --
    over pages handed out in scattered order; sharp scores, so a key just inside or outside the window or a missing sink shows."""
    f32, Hh, G, D, Dv, window, dims, bs, use_mq = case
    el, eps, scale, base = elem(f32), 1e-5, 6.0 / math.sqrt(D), 100.0
    lens, new = [150, 37, 101], [53, 37, 1]                 # context length after this step, rows this step brings
    nb = sum(-(-n // bs) for n in lens) + 3
    max_blocks = max(-(-n // bs) for n in lens)
    kc = torch.full((nb, G, bs, D), float("nan"), dtype=el, device=DEV)
    vc = torch.full((nb, G, Dv, bs), float("nan"), dtype=el, device=DEV)
    pages = torch.randperm(nb, generator=torch.Generator().manual_seed(1)).tolist()
    bt = torch.zeros(len(lens), max_blocks, dtype=torch.int32)
    sinks = rnd(Hh, seed=2)
    wq, wk = (1.0 + rnd(Hh * D, seed=3, scale=0.2)).to(el), (1.0 + rnd(G * D, seed=4, scale=0.2)).to(el)
    qf = d(torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)] or [0.0], dtype=F64).float())
    vf = d(torch.tensor([base ** (-2.0 * i / Dv) for i in range(Dv // 2)], dtype=F64).float())
    NP = (Hh + G) * D + G * Dv
    refs, rows, pos, slots, cu = [], [], [], [], [0]
    for b, (n, k) in enumerate(zip(lens, new)):
        proj = rnd(n, NP, seed=10 + b)
        mine = [pages.pop() for _ in range(-(-n // bs))]
        bt[b, :len(mine)] = torch.tensor(mine, dtype=torch.int32)
        sl = torch.tensor([mine[p // bs] * bs + p % bs for p in range(n)], dtype=torch.int32)
        if n > k:        # earlier portion: stored by a call of its own
            qd = torch.zeros(n - k, Hh * D, dtype=el, device=DEV)
            H().winattn_store_rope(d(proj[:n - k]), NP, d(wq), d(wk), eps, d(torch.arange(n - k)), qf, dims, vf, d(sl[:n - k]), qd, kc, vc,
                                   n - k, Hh, G, D, Dv, bs, f32)
        full = attention_reference(proj[:, :Hh * D].view(n, Hh, D), proj[:, Hh * D:(Hh + G) * D].view(n, G, D),
                                   proj[:, (Hh + G) * D:].view(n, G, Dv), wq, wk, sinks, window, scale, eps, dims, base)
        refs.append(full[n - k:])
        rows.append(proj[n - k:])
        pos += list(range(n - k, n))
        slots.append(sl[n - k:])
        cu.append(cu[-1] + k)
    T = cu[-1]
    q = torch.zeros(T, Hh * D, dtype=el, device=DEV)
    out = torch.zeros(T, Hh * Dv, dtype=el, device=DEV)
    H().winattn_store_rope(d(torch.cat(rows)), NP, d(wq), d(wk), eps, d(torch.tensor(pos)), qf, dims, vf, d(torch.cat(slots)), q, kc, vc, T,
                           Hh, G, D, Dv, bs, f32)
    H().winattn_paged(q, kc, vc, None, d(sinks), d(bt), max_blocks, d(torch.tensor(pos)), len(lens), T, Hh, G, D, Dv, bs, window, scale,
                      0.0, out, f32, cu_q=d(torch.tensor(cu, dtype=torch.int32)), max_q=max(new) if use_mq else 0, out_freqs=vf)
    ref = torch.cat(refs).view(T, Hh * Dv)
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    if f32:
        assert torch.allclose(got, ref, rtol=1e-4, atol=2e-5), float((got - ref).abs().max())
        if window:      # the statement is sharp: one key more or fewer is far away
            p0 = rnd(lens[0], NP, seed=10)
            other = attention_reference(p0[:, :Hh * D].view(lens[0], Hh, D), p0[:, Hh * D:(Hh + G) * D].view(lens[0], G, D),
                                        p0[:, (Hh + G) * D:].view(lens[0], G, Dv), wq, wk, sinks, window + 1, scale, eps, dims, base)
            assert float((other[lens[0] - new[0]:].reshape(new[0], -1) - ref[:new[0]]).abs().max()) > 1e-2
    else:
        assert float((got - ref).abs().max()) < 0.06 * float(ref.abs().max()), float((got - ref).abs().max())
        assert float((got - ref).pow(2).mean().sqrt()) < 0.01 * float(ref.pow(2).mean().sqrt()) + 1e-3
