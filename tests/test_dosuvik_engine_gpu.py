"""The Dosuvik decoder through the engine (Config -> ModelRunner -> block manager with state slots -> HIP kernels) against the plain
whole-sequence oracle (oracle/dosuvik.py, float64): small self-made configurations with random weights.  The fp32 element mode is the
sharp one: a dropped or extra key at a window's edge, a wrong page, a lost or stale recurrent state, a forgotten sink, a wrong pair of
a rotation or a missing level of the depth average is orders of magnitude above rounding there.  Attention inputs are scaled so that
single keys carry the output, and the decays so that some heads remember hundreds of tokens."""
import json
import os

import pytest
import torch

from oracle import dosuvik as F

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 6e-2}


def write_model(path, cfg, w):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def row_err(got: torch.Tensor, ref: torch.Tensor) -> torch.Tensor:
    d = got.double().cpu() - ref.double()
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.double().std()


def rel_err(got, ref) -> float:
    return float(row_err(got, ref).max())


def oracle(cfg, w, toks):
    """(logits, per-position rounding floor): the floor is what fp32 rounding of every sublayer's input alone does to the float64
    statement (a retention head whose output is near zero is divided by a root mean square that the eps decides, which amplifies
    rounding); a position's bound is the larger of the fixed one and 50 floors."""
    ref = F.forward(cfg, w, toks)
    low = F.forward(cfg, w, toks, round_input=lambda t: t.float().double())
    return ref, row_err(low, ref)


def floor16(cfg, w, toks, ref) -> torch.Tensor:
    """What bf16 rounding of every sublayer's input alone does to the float64 statement, per position."""
    return row_err(F.forward(cfg, w, toks, round_input=lambda t: t.bfloat16().double()), ref)


def close(got, ref, dtype, floor=None) -> bool:
    """fp32: every position within 1e-4 of the spread (or 50 rounding floors).  bf16: rounding of GEMM inputs, and now and then a router
    decision made the other way at a near-tie -- every sublayer's output is normed to unit size before it joins the residual, so one
    flipped expert moves a position by tens of percent, and every further layer amplifies it: the median within 5 %, nine positions in
    ten within 20 % (or four times what rounding of the sublayer inputs alone does to the statement, when `floor` gives it), all
    finite.  What a schedule, the cache or the state could get wrong is pinned by the fp32 runs."""
    e = row_err(got, ref)
    if dtype == "float32":
        return bool((e < (TOL[dtype] if floor is None else torch.clamp(50 * floor, min=TOL[dtype]))).all())
    med, q90 = (0.05, 0.2) if floor is None else (max(0.05, 4 * float(floor.median())), max(0.2, 4 * float(floor.quantile(0.9))))
    return bool(torch.isfinite(got).all() and e.median() < med and e.quantile(0.9) < q90)


def configs():
    R, L, A, D, M = F.retention_layer, F.latent_layer, F.attention_layer, F.dense_mlp, F.moe_mlp
    return {
        # every mixer and feed-forward; sizes chosen so that nothing the kernels index by coincides; rotations over a part of a head
        "all_kinds": F.make_config([R(heads=3, dim=8, vdim=12, rot_dims=6, mlp=D()),
                                    L(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=20, rot_dims=4, base=500.0, mlp=M(experts=6, top=2, ff=8, groups=3, keep=2)),
                                    A(heads=4, kv_heads=2, dim=12, vdim=6, window=7, rot_dims=8, base=100.0, mlp=M(experts=4, top=2, ff=16)),
                                    R(heads=2, dim=16, vdim=8, mlp=M(experts=8, top=3, ff=8, groups=2, keep=1)),
                                    A(heads=3, kv_heads=1, dim=24, vdim=8, scale=0.9, window=33, mlp=D(40, 0.6)),
                                    L(heads=2, dim=4, rot_dim=8, vdim=6, kv_rank=9, mlp=None)], vocab=101, width=72),
        # its halves: three layers amplify bf16 rounding far less than six
        "kinds_a": F.make_config([R(heads=3, dim=8, vdim=12, rot_dims=6, mlp=D()),
                                  L(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=20, rot_dims=4, base=500.0, mlp=M(experts=6, top=2, ff=8, groups=3, keep=2)),
                                  A(heads=4, kv_heads=2, dim=12, vdim=6, window=7, rot_dims=8, base=100.0, mlp=M(experts=4, top=2, ff=16))],
                                 vocab=101, width=72),
        "kinds_b": F.make_config([R(heads=2, dim=16, vdim=8, mlp=M(experts=8, top=3, ff=8, groups=2, keep=1)),
                                  A(heads=3, kv_heads=1, dim=24, vdim=8, scale=0.9, window=33, mlp=D(40, 0.6)),
                                  L(heads=2, dim=4, rot_dim=8, vdim=6, kv_rank=9, mlp=None)], vocab=101, width=72),
        # values that are 1 or equal: heads, kv heads, window, top, groups, experts per group (a group's "two largest" is one), no rotation
        "ones": F.make_config([A(heads=1, kv_heads=1, dim=8, vdim=8, window=1, mlp=M(experts=3, top=1, ff=8, groups=3, keep=1)),
                               R(heads=1, dim=8, vdim=8, decay=[1.0], rot_dims=0, mlp=D(8)),
                               L(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, rot_dims=0, mlp=M(experts=1, top=1, ff=8)),
                               A(heads=2, kv_heads=2, dim=2, vdim=2, window=2, rot_dims=2, mlp=None)], vocab=33, width=40),
        # no window at all, a window larger than any sequence here, every expert chosen, sizes that are no multiple of 8
        "odd_sizes": F.make_config([A(heads=6, kv_heads=3, dim=12, vdim=10, window=0, rot_dims=4, mlp=M(experts=3, top=3, ff=20)),
                                    R(heads=5, dim=12, vdim=20, rot_dims=10), L(heads=5, dim=6, rot_dim=10, vdim=14, kv_rank=70, mlp=D(52, 3.0)),
                                    A(heads=2, kv_heads=2, dim=20, vdim=36, window=1000)], vocab=77, width=50),
        # sizes the bf16 fast forms take (MFMA attentions: head / latent sizes in multiples of 32, value tiles that fill and that do not
        # fill the register array; register scans: state rows 32 / 64), windows of several 32-key steps
        "fast_forms": F.make_config([A(heads=8, kv_heads=2, dim=32, vdim=64, window=70, mlp=D(48)),
                                     R(heads=2, dim=32, vdim=32, mlp=M(experts=4, top=2, ff=16)),
                                     L(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, mlp=D(48)),
                                     A(heads=4, kv_heads=4, dim=64, vdim=32, window=44, rot_dims=32),
                                     R(heads=1, dim=64, vdim=64, rot_dims=16), L(heads=20, dim=8, rot_dim=32, vdim=8, kv_rank=96, rot_dims=16),
                                     A(heads=20, kv_heads=1, dim=32, vdim=96, window=0, mlp=M(experts=4, top=1, ff=16, groups=2, keep=2))],
                                    vocab=120, width=96),
        # one kind of memory only: no state slots at all / no cache pages at all
        "only_attention": F.make_config([A(window=6, mlp=M(experts=4)), L(mlp=None), A(heads=2, kv_heads=1, window=0, mlp=D())], vocab=40, width=48),
        "only_recurrent": F.make_config([R(mlp=D()), R(heads=2, dim=24, vdim=4, mlp=M(experts=2, top=1))], vocab=40, width=48),
    }


def make(name, seed=0):
    cfg = json.loads(json.dumps(configs()[name]))
    return cfg, F.random_model(cfg, seed)


def engine(tmp_path, cfg, w, dtype, max_tokens=512, block_size=16, **kw):
    from ssd_amd.engine.trace_engine import TraceEngine
    eng = TraceEngine(write_model(tmp_path / "m", cfg, w), dtype=dtype, max_tokens=max_tokens, block_size=block_size, **kw)
    m = eng.runner.model
    for t in m.kv + m.state:                    # a cache row or a state slot that is read before it is written shows as NaN
        for u in ((t,) if isinstance(t, torch.Tensor) else (t or ())):
            u.fill_(float("nan"))
    m.hist.fill_(float("nan"))                  # and so does a level of the depth history
    return eng


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _replay(eng, rid, toks, cuts):
    """Feed toks in portions ending at `cuts`; returns the logits of every position."""
    out, lo = [], 0
    for hi in cuts:
        out.append(eng.step([{"id": rid, "tokens": toks[lo:hi], "want": list(range(hi - lo))}], [rid] if hi == len(toks) else []))
        lo = hi
    return torch.cat(out)


# six sharp layers amplify bf16 rounding beyond any fixed bound: in bf16 "all_kinds" runs as its two halves
@pytest.mark.parametrize("name,dtype", [(n, t) for n in configs() for t in ("float32", "bfloat16") if (n, t) != ("all_kinds", "bfloat16")])
def test_whole_prompt_and_every_layer_match_the_oracle(tmp_path, name, dtype):
    cfg, w = make(name)
    toks = tokens(83, cfg["vocab"], 1)
    res = []
    ref = F.forward(cfg, w, toks, res)
    floor = oracle(cfg, w, toks)[1] if dtype == "float32" else floor16(cfg, w, toks, ref)
    eng = engine(tmp_path, cfg, w, dtype)
    eng.runner.model.tap_residuals = []
    got = eng.step([{"id": "a", "tokens": toks, "want": list(range(len(toks)))}], ["a"])
    taps = eng.runner.model.tap_residuals
    assert len(taps) == len(res) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(taps, res)):
        assert close(a, b, dtype, floor), f"layer {i}: {rel_err(a, b)}"
    assert close(got, ref, dtype, floor), rel_err(got, ref)


@pytest.mark.parametrize("name", list(configs()))
def test_portions_and_token_by_token_decoding_equal_the_whole_prompt(tmp_path, name):
    cfg, w = make(name, seed=2)
    n = 70
    toks = tokens(n, cfg["vocab"], 3)
    ref, floor = oracle(cfg, w, toks)
    eng = engine(tmp_path, cfg, w, "float32", block_size=16)
    whole = _replay(eng, "w", toks, [n])
    assert close(whole, ref, "float32", floor), rel_err(whole, ref)
    schedules = {
        "token by token from the first": list(range(1, n + 1)),
        "prompt then decoding": [41] + list(range(42, n + 1)),
        "portions of two": list(range(2, n + 1, 2)),
        "portions of changing size, cut at and next to page borders": [15, 16, 17, 32, 35, 47, 48, 50, 64, 65, n],
        "three then single tokens over a page border": [3] + list(range(4, 20)) + [n],
    }
    for what, cuts in schedules.items():
        got = _replay(eng, what, toks, cuts)
        # every row is computed from its own inputs, the cache and the state in a fixed order: no dependence on the cut at all
        assert torch.equal(got, whole), what


def test_window_edges_sinks_far_tokens_rotations_and_depth_weights_show(tmp_path):
    """The model is sensitive to what the test is about: against an oracle whose window is one key longer or shorter, whose sink is left
    out, whose slowest decay is a little off, whose values are not rotated, whose correction is left out of the choice or whose depth
    average misses the embedding, the engine is FAR from equal; against the right one it is equal -- in prompts, in portions and in
    decoding, with windows that end inside a page, at its border and several pages back."""
    cfg, w = make("all_kinds", seed=5)
    n = 90
    toks = tokens(n, cfg["vocab"], 6)
    ref, floor = oracle(cfg, w, toks)
    eng = engine(tmp_path, cfg, w, "float32", block_size=16)
    got = _replay(eng, "a", toks, [40] + list(range(41, n + 1)))
    assert close(got, ref, "float32", floor), rel_err(got, ref)
    far = 100 * TOL["float32"]
    for li, delta in ((2, 1), (2, -1), (4, 1), (4, -1)):
        other = json.loads(json.dumps(cfg))
        other["layers"][li]["mixer"]["mask"]["size"] += delta
        wrong = F.forward(other, w, toks)
        first = cfg["layers"][li]["mixer"]["mask"]["size"] + min(delta, 0)      # the first position that sees a different key set
        assert rel_err(got[first:], wrong[first:]) > far, (li, delta)
    other = dict(w)
    other["l2.mix.sink"] = torch.full_like(w["l2.mix.sink"], -60.0)              # as good as no sink
    assert rel_err(got, F.forward(cfg, other, toks)) > far
    other = json.loads(json.dumps(cfg))
    other["layers"][3]["mixer"]["decay"][-1] -= 0.01                             # only the slowest head: far tokens
    assert rel_err(got[60:], F.forward(other, w, toks)[60:]) > far
    other = json.loads(json.dumps(cfg))
    other["layers"][1]["mixer"]["rot"]["dims"] = 6                               # one more pair of the shared key part turns
    assert rel_err(got, F.forward(other, w, toks)) > far
    other = dict(w)
    other["l1.mlp.correction"] = torch.zeros_like(w["l1.mlp.correction"])
    assert rel_err(got, F.forward(cfg, other, toks)) > far
    other = dict(w)
    other["l5.dwa"] = w["l5.dwa"].clone()
    other["l5.dwa"][0] = 0                                                       # the embedding's share of the last average
    assert rel_err(got, F.forward(cfg, other, toks)) > far


def test_one_far_key_at_page_borders_and_window_edges_decides_the_output(tmp_path):
    """A model of one windowless attention layer whose scores are scaled so that the largest one takes the whole softmax: every position
    then copies the value of its best key, wherever it lies -- hundreds of tokens back, at a page's last or first slot.  A second model
    with a window: the best key just inside the window is found, just outside it is not."""
    cfg = F.make_config([F.attention_layer(heads=2, kv_heads=1, dim=16, vdim=8, scale=40.0, window=0, rot_dims=4, mlp=None)], vocab=50, width=32)
    w = F.random_model(cfg, 3)
    n = 300
    toks = tokens(n, 50, 4)
    ref, floor = oracle(cfg, w, toks)
    for dtype in ("float32",):
        eng = engine(tmp_path / dtype, cfg, w, dtype, max_tokens=320, block_size=16)
        got = _replay(eng, "a", toks, [250] + list(range(251, n + 1)))
        assert close(got, ref, dtype, floor), rel_err(got, ref)
    cfg2 = json.loads(json.dumps(cfg))
    cfg2["layers"][0]["mixer"]["mask"]["size"] = 48
    ref2, floor2 = oracle(cfg2, w, toks)
    assert rel_err(ref2, ref) > 0.1                 # the far keys mattered
    eng = engine(tmp_path / "w", cfg2, w, "float32", max_tokens=320, block_size=16)
    got = _replay(eng, "a", toks, [100, 101, 103, 160] + list(range(161, n + 1)))
    assert close(got, ref2, "float32", floor2), rel_err(got, ref2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_of_unequal_requests_with_pages_and_slots_used_again(tmp_path, dtype):
    """Up to three live requests, prompt portions of some beside single tokens of others, in a pool too small for all of them at once:
    pages and state slots of finished requests (filled by them, never cleared) are taken again."""
    cfg, w = make("all_kinds" if dtype == "float32" else "kinds_b", seed=4)
    V = cfg["vocab"]
    reqs = {r: tokens(n, V, 40 + i) for i, (r, n) in enumerate([("a", 61), ("b", 7), ("c", 38), ("d", 1), ("e", 50), ("f", 23)])}
    both = {r: oracle(cfg, w, t) for r, t in reqs.items()}
    refs = {r: v[0] for r, v in both.items()}
    eng = engine(tmp_path, cfg, w, dtype, max_tokens=176, block_size=16, max_live=3)
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    plan = [[("a", 20), ("b", 3)], [("a", 1), ("b", 4), ("c", 2)], [("a", 17), ("c", 1)], [("c", 30), ("a", 1), ("d", 1)],
            [("a", 22), ("c", 5), ("e", 16)], [("e", 1), ("f", 2)], [("e", 33), ("f", 1)], [("f", 20)]]
    for step in plan:
        entries, end = [], []
        for r, k in step:
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + k], "want": list(range(k))})
            at[r] += k
            if at[r] == len(reqs[r]):
                end.append(r)
        out = eng.step(entries, end)
        lo = 0
        for r, k in step:
            got[r].append(out[lo:lo + k])
            lo += k
    assert all(at[r] == len(reqs[r]) for r in reqs)
    assert not eng.live and len(eng.blocks.free_block_ids) == 11 and eng.blocks.free_state_slots == [0, 1, 2]
    if dtype == "float32":
        for r in reqs:
            g = torch.cat(got[r])
            assert close(g, refs[r], dtype, both[r][1]), (r, rel_err(g, refs[r]))
        for r in ("a", "e"):          # each alone gives exactly the same rows
            alone = _replay(eng, r + "x", reqs[r], [len(reqs[r])])
            assert torch.equal(alone, torch.cat(got[r]))
    else:           # the bf16 bound is a statement about many positions: all requests together
        floors = torch.cat([floor16(cfg, w, reqs[r], refs[r]) for r in reqs])
        assert close(torch.cat([torch.cat(got[r]) for r in reqs]), torch.cat([refs[r] for r in reqs]), dtype, floors)


@pytest.mark.parametrize("block_size", [32, 64])
def test_bf16_fast_forms_through_the_engine_portions_decoding_and_mixed_steps(tmp_path, block_size):
    """bf16 with 32 / 64-token pages and sizes that the MFMA attentions and the register scan take: whole prompt, portions cut at and
    next to page borders, decoded tokens (the wave-split / key-slice forms), two requests sharing steps; every position against the
    oracle, the portions against the whole prompt, and the MFMA attentions against the scalar forms on the same inputs."""
    cfg, w = make("fast_forms", seed=9)
    n = 190
    ta, tb = tokens(n, cfg["vocab"], 30), tokens(77, cfg["vocab"], 31)
    ra, rb = F.forward(cfg, w, ta), F.forward(cfg, w, tb)
    fa, fb = floor16(cfg, w, ta, ra), floor16(cfg, w, tb, rb)
    eng = engine(tmp_path, cfg, w, "bfloat16", max_tokens=384, block_size=block_size)
    assert all(eng.runner.model.mfma.values())
    whole = _replay(eng, "w", ta, [n])
    assert close(whole, ra, "bfloat16", fa), rel_err(whole, ra)
    eng.runner.model.scalar_attention = True
    scalar = _replay(eng, "s", ta, [n])
    eng.runner.model.scalar_attention = False
    assert row_err(whole, scalar.double().cpu()).median() < 0.02
    cuts = sorted({block_size - 1, block_size, block_size + 1, 2 * block_size + 2, 150} | set(range(151, n + 1)))
    got = _replay(eng, "c", ta, cuts)
    assert close(got, ra, "bfloat16", fa), rel_err(got, ra)
    assert row_err(got, whole.double().cpu()).median() < 0.02
    ga, gb, ia, ib = [], [], 0, 0
    for ka, kb in [(40, 1), (1, 1), (1, 30), (25, 1), (1, 44)] + [(1, 0)] * 10 + [(n - 78, 0)]:
        entries = []
        if ka:
            entries.append({"id": "a", "tokens": ta[ia:ia + ka], "want": list(range(ka))})
        if kb:
            entries.append({"id": "b", "tokens": tb[ib:ib + kb], "want": list(range(kb))})
        ia, ib = ia + ka, ib + kb
        out = eng.step(entries, [r for r, done in (("a", ia == n), ("b", ib == 77 and kb)) if done])
        ga.append(out[:ka])
        gb.append(out[ka:ka + kb])
    assert ia == n and ib == 77
    assert close(torch.cat(ga), ra, "bfloat16", fa) and close(torch.cat(gb), rb, "bfloat16", fb)


def test_bf16_fast_forms_over_a_long_context_without_windows(tmp_path):
    """Hundreds of keys per row through the MFMA attentions with no window at all (the latent attention's key slices over the grid, the
    grouped-query attention's wave split), a prompt of many pages, then decoding: against the oracle and against the scalar forms."""
    R, L, A, D, M = F.retention_layer, F.latent_layer, F.attention_layer, F.dense_mlp, F.moe_mlp
    cfg = F.make_config([L(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, mlp=D(48)),
                         A(heads=4, kv_heads=2, dim=32, vdim=32, window=0, rot_dims=16, mlp=M(experts=4, top=2, ff=16, groups=2, keep=1)),
                         R(heads=2, dim=32, vdim=32, decay=[0.99, 0.999], mlp=None)], vocab=90, width=64)
    w = F.random_model(cfg, 21)
    n = 700
    toks = tokens(n, cfg["vocab"], 22)
    ref = F.forward(cfg, w, toks)
    fl = floor16(cfg, w, toks, ref)
    cuts = [600] + list(range(601, 641)) + [n]
    eng = engine(tmp_path, cfg, w, "bfloat16", max_tokens=768, block_size=64)
    assert all(eng.runner.model.mfma.values())
    got = _replay(eng, "a", toks, cuts)
    assert close(got, ref, "bfloat16", fl), rel_err(got, ref)
    eng.runner.model.scalar_attention = True
    scalar = _replay(eng, "s", toks, cuts)
    assert row_err(got, scalar.double().cpu()).median() < 0.02
    eng32 = engine(tmp_path / "f", cfg, w, "float32", max_tokens=768, block_size=64)
    got32 = _replay(eng32, "a", toks, cuts)
    assert close(got32, ref, "float32", oracle(cfg, w, toks)[1]), rel_err(got32, ref)


def test_fast_forms_in_fp32_rows_equal_for_any_cut(tmp_path):
    """The register scan also runs in the fp32 element mode; its rows do not depend on the cut either."""
    cfg, w = make("fast_forms", seed=10)
    n = 100
    toks = tokens(n, cfg["vocab"], 12)
    ref, floor = oracle(cfg, w, toks)
    eng = engine(tmp_path, cfg, w, "float32", max_tokens=256, block_size=32)
    whole = _replay(eng, "w", toks, [n])
    assert close(whole, ref, "float32", floor), rel_err(whole, ref)
    got = _replay(eng, "c", toks, [7, 8, 9, 17, 31, 32, 33, 60] + list(range(61, n + 1)))
    assert torch.equal(got, whole)


def test_long_decoding_over_many_pages(tmp_path):
    cfg, w = make("all_kinds", seed=8)
    n = 230
    toks = tokens(n, cfg["vocab"], 9)
    ref, floor = oracle(cfg, w, toks)
    eng = engine(tmp_path, cfg, w, "float32", max_tokens=256, block_size=16)
    got = _replay(eng, "a", toks, [5] + list(range(6, n + 1)))
    assert close(got, ref, "float32", floor), rel_err(got, ref)
    eng16 = engine(tmp_path, cfg, w, "bfloat16", max_tokens=256, block_size=16)
    got16 = _replay(eng16, "a", toks, [5] + list(range(6, n + 1)))
    assert close(got16, ref, "bfloat16", floor16(cfg, w, toks, ref)), rel_err(got16, ref)


def test_pool_and_live_limits_are_enforced(tmp_path):
    cfg, w = make("ones")
    eng = engine(tmp_path, cfg, w, "float32", max_tokens=64, block_size=16, max_live=2)
    eng.step([{"id": "a", "tokens": [1] * 20, "want": []}, {"id": "b", "tokens": [2] * 20, "want": []}])
    with pytest.raises(RuntimeError):
        eng.step([{"id": "c", "tokens": [3], "want": []}])
    eng.step([], ["a"])
    eng.step([{"id": "c", "tokens": [3] * 30, "want": [29]}])
    with pytest.raises(RuntimeError):
        eng.step([{"id": "b", "tokens": [2] * 20, "want": []}])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_llm_generate(tmp_path, dtype):
    """The framework's own entry point and scheduler: batched prefill, batched decode (hipGraph replays), pages and state slots from the
    scheduler's block manager (three slots for four prompts), argmax kernels."""
    from ssd_amd import LLM, SamplingParams
    cfg, w = make("all_kinds", seed=7)
    path = write_model(tmp_path / "m", cfg, w)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (5, 19, 1, 34)]
    new = 24
    llm = LLM(path, dtype=dtype, kvcache_block_size=16, num_kvcache_blocks=32, max_num_seqs=3, max_model_len=128,
              max_num_batched_tokens=128)
    outs, _ = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=new, ignore_eos=True), use_tqdm=False)
    assert len(outs) == len(prompts)
    del llm
    eng = engine(tmp_path / "t", cfg, w, dtype, max_tokens=256)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        gen = o["token_ids"]
        assert len(gen) == new
        # teacher forcing: every generated token is the argmax of its step.  The argmax kernels read the logits rounded to bf16, so a
        # runner-up within that rounding of the top may win.  Against the oracle in fp32; in bf16 (where a router decision flipped by
        # rounding moves these tiny models' logits a lot) against the same arithmetic fed step by step through the trace engine.
        seq = p + gen[:-1]
        if dtype == "float32":
            lg = F.forward(cfg, w, seq)[len(p) - 1:]
        else:
            lg = eng.step([{"id": str(i), "tokens": seq, "want": list(range(len(p) - 1, len(seq)))}], [str(i)]).double().cpu()
        top = lg.max(-1).values
        chosen = lg[torch.arange(new), torch.tensor(gen)]
        assert ((top - chosen) <= 2.0 ** -7 * top.abs() + 1e-3 * lg.std()).all(), (i, (top - chosen).max())


@pytest.mark.parametrize("seed", range(4))
def test_random_configurations_in_both_modes_whole_and_in_portions(tmp_path, seed):
    g = torch.Generator().manual_seed(100 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    layers = []
    for i in range(r(2, 4)):
        kind = r(0, 2)
        mlp = None
        if kind == 1:
            mlp = F.dense_mlp(8 * r(1, 6), 0.5 + 0.5 * r(0, 4))
        elif kind == 2:
            G = r(1, 3)
            per = r(1, 4)
            keep = r(1, G)
            mlp = F.moe_mlp(experts=G * per, top=r(1, per * keep), ff=8 * r(1, 4), groups=G, keep=keep)
        mix = r(0, 2)
        if mix == 0:
            G = r(1, 3)
            d = r(1, 5) * 8
            layers.append(F.attention_layer(heads=G * r(1, 4), kv_heads=G, dim=d, vdim=2 * r(1, 20), scale=0.2 * r(1, 5), window=r(0, 40),
                                            rot_dims=2 * r(0, d // 2), base=10.0 ** r(1, 6), mlp=mlp))
        elif mix == 1:
            d = r(1, 5) * 8
            H = r(1, 4)
            layers.append(F.retention_layer(heads=H, dim=d, vdim=r(1, 5) * 4, decay=[1.0 - 2.0 ** -r(1, 9) for _ in range(H)],
                                            rot_dims=2 * r(0, d // 2), base=10.0 ** r(1, 6), mlp=mlp))
        else:
            R = 2 * r(1, 8)
            layers.append(F.latent_layer(heads=r(1, 5), dim=r(1, 5) * 4, rot_dim=R, vdim=r(1, 20), kv_rank=r(1, 12) * 4, scale=0.1 * r(1, 5),
                                         rot_dims=2 * r(0, R // 2), base=10.0 ** r(1, 6), mlp=mlp))
    cfg = F.make_config(layers, vocab=r(20, 150), width=8 * r(3, 12))
    w = F.random_model(cfg, seed)
    toks = tokens(60, cfg["vocab"], seed)
    ref, floor = oracle(cfg, w, toks)
    for dtype in ("float32", "bfloat16"):
        floor = floor if dtype == "float32" else floor16(cfg, w, toks, ref)
        eng = engine(tmp_path / dtype, cfg, w, dtype, max_tokens=128, block_size=16)
        whole = _replay(eng, "w", toks, [60])
        assert close(whole, ref, dtype, floor), (dtype, rel_err(whole, ref))
        parts = _replay(eng, "p", toks, [7, 9, 31, 32, 33] + list(range(34, 61)))
        assert close(parts, ref, dtype, floor), (dtype, rel_err(parts, ref))


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run as a user runs it: steps on standard input, `done <step>` after each, <step>.f32 for the steps that want logits;
    two requests share steps, one ends and its pages and slot go to a third."""
    import subprocess
    import sys
    import numpy as np
    from tests.conftest import ROOT
    cfg, w = make("all_kinds", seed=11)
    path = write_model(tmp_path / "m", cfg, w)
    V = cfg["vocab"]
    ta, tb, tc = tokens(70, V, 1), tokens(9, V, 2), tokens(40, V, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ta[:50], "want": [0, 49]}, {"id": "b", "tokens": tb[:8], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": tb[8:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ta[50:52], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "c", "tokens": tc, "want": [39]}, {"id": "a", "tokens": ta[52:], "want": [17]}], "end": ["a", "c"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "192", "--max-live", "2"], input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                       capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(4)]
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "3.f32"]
    read = lambda n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V).copy())
    ra, rb, rc = F.forward(cfg, w, ta), F.forward(cfg, w, tb), F.forward(cfg, w, tc)
    assert rel_err(read(0), ra[[0, 49]]) < 1e-3 and rel_err(read(1), rb[[8]]) < 1e-3
    assert rel_err(read(3), torch.stack([rc[39], ra[69]])) < 1e-3
