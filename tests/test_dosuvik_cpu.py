"""CPU-side checks of the Dosuvik integration: the config reader, checkpoint names, synthetic weights, the rotary layout permutation,
state slots through the trace engine (a recording runner, no GPU), the bench option, and the oracle's own mechanisms against hand-made
cases and against restatements (retention as an explicit decayed sum over earlier tokens, latent attention with the per-head matrices
moved to the query and output side, rotated values as a rotation by the distance, the router on a case worked by hand)."""
import json
import math

import pytest
import torch

from oracle import dosuvik as F
from ssd_amd.model_config import DosuvikConfig, Rotary, read_native_config
from ssd_amd.weights import param_shapes, synthetic_state_dict

F64 = torch.float64


def small_config():
    return F.make_config([F.retention_layer(mlp=F.dense_mlp()), F.latent_layer(mlp=F.moe_mlp(experts=6, top=2, groups=3, keep=2)),
                          F.attention_layer(mlp=None), F.retention_layer(heads=3, dim=4, vdim=6, rot_dims=2, mlp=F.moe_mlp())])


def write(path, cfg, w):
    from safetensors.torch import save_file
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(path / "model.safetensors"))


def test_config_reader_names_and_synthetic_weights(tmp_path):
    cfg = small_config()
    w = F.random_model(cfg, 0)
    write(tmp_path, cfg, w)
    c = read_native_config(str(tmp_path))
    assert isinstance(c, DosuvikConfig) and c.family == "dosuvik" and c.recurrent and c.num_layers == 4
    r0, l1, a2 = c.layers[0].mixer, c.layers[1].mixer, c.layers[2].mixer
    assert (r0.kind, r0.heads, r0.dim, r0.vdim, r0.rope.dims, r0.rope.layout) == ("retention", 2, 8, 8, 8, "halves") and len(r0.decay) == 2
    assert (l1.kind, l1.kv_rank, l1.rot_dim, l1.rope.layout, l1.window) == ("latent_attention", 12, 4, "interleaved", 0)
    assert (a2.kind, a2.heads, a2.kv_heads, a2.window, a2.rotate_values, a2.rope.layout) == ("attention", 4, 2, 5, True, "halves")
    m0, m1 = c.layers[0].mlp, c.layers[1].mlp
    assert (m0.kind, m0.ff, m0.limit) == ("dense", 24, 1.5) and (m1.experts, m1.top, m1.groups, m1.keep) == (6, 2, 3, 2)
    assert c.layers[2].mlp is None and c.layers[3].mixer.rope.dims == 2
    assert {n: tuple(s) for n, s in param_shapes(c)} == {n: tuple(t.shape) for n, t in w.items()}
    assert dict(param_shapes(c))["l3.dwa"] == (5,)
    sd = synthetic_state_dict(c, 0, 0.02)
    assert set(sd) == set(w) and all(sd[n].shape == w[n].shape for n in w)
    assert float(sd["l0.norm1"].float().abs().max()) == 0.0 and float(sd["l1.mix.dkv.norm"].float().min()) == 1.0      # 1 + w against plain
    assert abs(float(sd["l2.dwa"][-1]) - 1.0) < 0.2 and float(sd["l2.dwa"][:-1].float().abs().max()) < 0.2
    assert not DosuvikConfig.from_json(F.make_config([F.attention_layer(), F.latent_layer()])).recurrent
    no_groups = json.loads(json.dumps(cfg))
    del no_groups["layers"][1]["mlp"]["router"]["groups"]
    assert (lambda m: (m.groups, m.keep))(DosuvikConfig.from_json(no_groups).layers[1].mlp) == (1, 1)
    for breakit in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][0]["mlp"].update(kind="glu"),
                    lambda d: d["layers"][2]["mixer"].update(kv_heads=3), lambda d: d["layers"][1]["mlp"]["router"].update(top=5),
                    lambda d: d["layers"][0]["mixer"].update(decay=[0.5]), lambda d: d["layers"][1]["mixer"]["rot"].update(dims=6),
                    lambda d: d["layers"][1]["mlp"]["router"]["groups"].update(count=4)):
        bad = json.loads(json.dumps(cfg))
        breakit(bad)
        with pytest.raises(ValueError):
            DosuvikConfig.from_json(bad)


def test_interleaved_pairs_become_halves_by_one_permutation_of_both_sides():
    """Scores are dot products: a rotated part whose entries are reordered alike on the query and the key side gives the same scores,
    and the reordering Rotary.to_halves names turns the (2i, 2i + 1) pairs into (i, i + dims / 2) pairs with the same frequencies."""
    T, H, R = 9, 3, 10
    for dims in (10, 6, 2, 0):
        r = Rotary(dims, 5000.0, "interleaved")
        order = torch.tensor(r.to_halves(R))
        assert sorted(order.tolist()) == list(range(R))
        q, k = torch.randn(T, H, R, dtype=F64), torch.randn(T, 1, R, dtype=F64)
        pos = torch.arange(T) * 37
        a = torch.einsum("thr,jr->htj", F.turn(q, pos, dims, r.base, "interleaved"), F.turn(k, pos, dims, r.base, "interleaved")[:, 0])
        b = torch.einsum("thr,jr->htj", F.turn(q[..., order], pos, dims, r.base, "halves"), F.turn(k[..., order], pos, dims, r.base, "halves")[:, 0])
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)
        assert r.frequencies() == [5000.0 ** (-2.0 * i / dims) for i in range(dims // 2)]
    assert Rotary(8, 10.0).to_halves(12) == list(range(12))


def test_oracle_retention_is_a_decayed_sum_over_earlier_tokens():
    cfg = F.make_config([F.retention_layer(heads=2, dim=6, vdim=4, decay=[0.5, 0.96875], rot_dims=4)], width=16)
    w = F.random_model(cfg, 1)
    m, eps = cfg["layers"][0]["mixer"], 1e-5
    T = 12
    h = torch.randn(T, 16, dtype=F64)
    got = F.retention(h, w, "l0.mix.", m, eps)
    pos = torch.arange(T)
    q = F.turn(F.lin(w["l0.mix.q"], h).view(T, 2, 6), pos, 4, 10000.0, "halves")
    k = F.turn(F.lin(w["l0.mix.k"], h).view(T, 2, 6), pos, 4, 10000.0, "halves") / math.sqrt(6)
    v = F.lin(w["l0.mix.v"], h).view(T, 2, 4)
    o = torch.zeros(T, 2, 4, dtype=F64)
    for hh, dc in enumerate(m["decay"]):
        for i in range(T):
            for j in range(i + 1):
                o[i, hh] += dc ** (i - j) * (q[i, hh] @ k[j, hh]) * v[j, hh]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    ref = F.lin(w["l0.mix.o"], o.reshape(T, 8) * F.silu(F.lin(w["l0.mix.g"], h)))
    assert torch.allclose(got, ref, rtol=1e-10, atol=1e-10)
    # the rotation makes the score a function of the distance: shifting all positions changes nothing (turn both sides by the same angle)
    assert torch.allclose(q[5, 0, :4] @ k[3, 0, :4], F.turn(F.lin(w["l0.mix.q"], h).view(T, 2, 6), pos + 100, 4, 10000.0, "halves")[5, 0, :4]
                          @ (F.turn(F.lin(w["l0.mix.k"], h).view(T, 2, 6), pos + 100, 4, 10000.0, "halves") / math.sqrt(6))[3, 0, :4])


def test_oracle_latent_attention_runs_in_the_latent_space_too():
    """q_plain . (W_uk c_j) = (W_uk^T q_plain) . c_j and sum_j p_j W_uv c_j = W_uv sum_j p_j c_j: only the latent and the turned key part
    have to be kept per token."""
    cfg = F.make_config([F.latent_layer(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=7)], width=16)
    w = F.random_model(cfg, 2)
    m, eps, T = cfg["layers"][0]["mixer"], 1e-5, 10
    h = torch.randn(T, 16, dtype=F64)
    got = F.latent_attention(h, w, "l0.mix.", m, eps)
    pos = torch.arange(T)
    q = F.lin(w["l0.mix.q"], h).view(T, 3, 10)
    dkv = F.lin(w["l0.mix.dkv"], h)
    c = F.rms(dkv[:, :7], eps) * w["l0.mix.dkv.norm"].double()
    kr = F.turn(dkv[:, 7:].reshape(T, 1, 4), pos, 4, 10000.0, "interleaved")[:, 0]
    qr = F.turn(q[..., 6:], pos, 4, 10000.0, "interleaved")
    uk, uv = w["l0.mix.uk"].double().view(3, 6, 7), w["l0.mix.uv"].double().view(3, 5, 7)
    out = torch.zeros(T, 3, 5, dtype=F64)
    for hh in range(3):
        ql = q[:, hh, :6] @ uk[hh]                                  # [T, 7]: the query in the latent space
        s = (ql @ c.T + qr[:, hh] @ kr.T) * m["scale"]
        s = s.masked_fill(pos.view(T, 1) < pos.view(1, T), -math.inf)
        out[:, hh] = (torch.softmax(s, -1) @ c) @ uv[hh].T
    ref = F.lin(w["l0.mix.o"], out.reshape(T, 15) * torch.sigmoid(F.lin(w["l0.mix.g"], h)))
    assert torch.allclose(got, ref, rtol=1e-10, atol=1e-10)


def test_oracle_rotated_values_carry_the_distance_and_the_sink_is_a_key_of_value_zero():
    cfg = F.make_config([F.attention_layer(heads=2, kv_heads=1, dim=4, vdim=6, window=3, rot_dims=2)], width=16)
    w = F.random_model(cfg, 3)
    m, eps, T = cfg["layers"][0]["mixer"], 1e-5, 8
    h = torch.randn(T, 16, dtype=F64)
    got = F.window_attention(h, w, "l0.mix.", m, eps)
    pos = torch.arange(T)
    q = (F.rms(F.lin(w["l0.mix.q"], h), eps) * w["l0.mix.q.norm"].double()).view(T, 2, 4)
    k = (F.rms(F.lin(w["l0.mix.k"], h), eps) * w["l0.mix.k.norm"].double()).view(T, 1, 4)
    q, k = F.turn(q, pos, 2, 10000.0, "halves"), F.turn(k, pos, 2, 10000.0, "halves")
    v = F.lin(w["l0.mix.v"], h).view(T, 1, 6)
    out = torch.zeros(T, 2, 6, dtype=F64)
    for hh in range(2):
        for i in range(T):
            js = [j for j in range(T) if 0 <= i - j < 3]
            s = torch.stack([q[i, hh] @ k[j, 0] * m["scale"] for j in js] + [w["l0.mix.sink"].double()[hh]])
            p = torch.softmax(s, 0)
            for n, j in enumerate(js):          # the value of j, turned by j - i: a function of the distance alone
                out[i, hh] += p[n] * F.turn(v[j].view(1, 1, 6), torch.tensor([j - i]), 6, 10000.0, "halves")[0, 0]
    assert torch.allclose(got, F.lin(w["l0.mix.o"], out.reshape(T, 12)), rtol=1e-10, atol=1e-10)


def test_oracle_router_and_feed_forwards_on_hand_made_cases():
    # 6 experts in 3 groups of 2, keep 2, top 2.  plain scores: sigmoid(z); corrections move expert 4 up and expert 0 down
    z = torch.tensor([[2.0, 1.0, 0.0, 0.5, -1.0, -2.0]], dtype=F64)
    corr = torch.tensor([-1.0, 0.0, 0.0, 0.0, 1.0, 0.0])
    s = torch.sigmoid(z[0])
    ch = s + corr.double()
    groups = [ch[0] + ch[1], ch[2] + ch[3], ch[4] + ch[5]]              # a group's score: its two largest = both
    assert groups[2] > groups[1] > groups[0]                             # group 0 (the largest plain scores) is out
    idx, wt = F.route(z, corr, 2, 3, 2)
    assert idx.tolist() == [[4, 3]] and torch.allclose(wt[0], torch.stack([s[4], s[3]]))        # weights: the plain scores, not renormalised
    # negative choice scores everywhere: an excluded expert counts as -inf, not 0
    idx, _ = F.route(z, torch.full((6,), -3.0), 2, 3, 1)
    assert idx.tolist() == [[0, 1]]
    # one group of one expert: its "two largest" is that one
    assert F.route(torch.tensor([[0.3, -0.2, 0.1]], dtype=F64), torch.zeros(3), 1, 3, 1)[0].tolist() == [[0]]
    # dense: gate clamped from above only, up on both sides
    ml = F.dense_mlp(ff=3, limit=1.0)
    w = {"gate": torch.eye(3), "up": torch.eye(3), "down": torch.eye(3)}
    y = F.dense_ff(torch.tensor([[5.0, -5.0, 0.5]], dtype=F64), w, "", ml)[0]
    g = torch.tensor([1.0, -5.0, 0.5], dtype=F64)
    u = torch.tensor([1.0, -1.0, 0.5], dtype=F64)
    assert torch.allclose(y, g * torch.sigmoid(1.702 * g) * (u + 1.0))


def test_oracle_depth_average_and_output_norms():
    """With one layer whose mixer output is zero (W_o = 0) the layer adds nothing, and the logits are the head of the normed weighted
    average of the embedding with itself."""
    cfg = F.make_config([F.attention_layer(mlp=None)], vocab=10, width=8)
    w = F.random_model(cfg, 4)
    w["l0.mix.o"] = torch.zeros_like(w["l0.mix.o"])
    toks = [1, 2, 3]
    x0 = w["embed"].double()[torch.tensor(toks)]
    c = w["l0.dwa"].double()
    x = (c[0] + c[1]) * x0
    ref = F.lin(w["head"], F.rms(x, 1e-5) * (1.0 + w["final.norm"].double()))
    assert torch.allclose(F.forward(cfg, w, toks), ref, rtol=1e-10, atol=1e-10)


class _Recorder:
    """Stands in for the ModelRunner: records which slots and pages every step's sequences hold."""
    def __init__(self, config):
        self.num_kvcache_blocks = config.num_kvcache_blocks
        self.calls = []

    def run_rows(self, seqs, want):
        self.calls.append([(s.state_slot, list(s.block_table), len(s) - s.num_cached_tokens) for s in seqs])
        return torch.zeros(sum(len(x) for x in want), 4)


def test_trace_engine_hands_out_pages_and_state_slots_and_takes_them_again(tmp_path):
    from ssd_amd.engine.trace_engine import TraceEngine
    cfg = small_config()
    write(tmp_path, cfg, F.random_model(cfg, 0))
    eng = TraceEngine(str(tmp_path), max_tokens=128, block_size=16, max_live=2, runner_factory=_Recorder)
    eng.step([{"id": "a", "tokens": [1] * 20, "want": [19]}, {"id": "b", "tokens": [2] * 3, "want": []}])
    assert [c[0] for c in eng.runner.calls[-1]] == [0, 1] and [c[2] for c in eng.runner.calls[-1]] == [20, 3]
    with pytest.raises(RuntimeError):
        eng.step([{"id": "c", "tokens": [3], "want": []}])
    pages_a = list(eng.live["a"].block_table)
    eng.step([{"id": "b", "tokens": [2], "want": []}], end=["a"])
    eng.step([{"id": "c", "tokens": [3] * 100, "want": []}])
    slot, pages_c, _ = eng.runner.calls[-1][0]
    assert slot == 0 and set(pages_a) <= set(pages_c)                      # a's slot and a's pages are in use again
    eng.step([], end=["b", "c"])
    assert eng.blocks.free_state_slots == [0, 1] and len(eng.blocks.free_block_ids) == 8
    plain = F.make_config([F.attention_layer(), F.latent_layer()])          # no recurrent layer: no slots at all
    write(tmp_path, plain, F.random_model(plain, 0))
    assert TraceEngine(str(tmp_path), max_tokens=64, block_size=16, runner_factory=_Recorder).blocks.free_state_slots is None


def test_bench_option_and_equal_size_pairs():
    """bench.py accepts --workload dosuvik next to its default; every benchmarked size pairs a Dosuvik model with a Zerusun model of the
    same width, layers, vocabulary, experts, top, groups, latent and state sizes and active feed-forward parameters per token."""
    import bench
    from ssd_amd.utils import arch_bench
    assert bench.parse([]).workload == "c4"                                  # the default workload is untouched
    a = bench.parse(["--workload", "dosuvik", "--arch-size", "w2048", "--arch-batch", "1", "--arch-only", "dosuvik"])
    assert a.workload == "dosuvik" and a.arch_size == "w2048" and a.arch_batch == 1 and a.arch_only == "dosuvik"
    for size in arch_bench.SIZES:
        dos, zer = arch_bench.dosuvik_models(size)
        assert dos.hidden_size == zer.hidden_size and dos.vocab_size == zer.vocab_size and dos.num_layers == zer.num_layers
        assert [l.mixer.kind for l in dos.layers] == ["latent_attention", "retention", "attention", "retention"] and dos.recurrent
        md, mz = dos.layers[0].mlp, zer.layers[0].mlp
        assert (md.experts, md.top, md.groups, md.keep) == (mz.experts, mz.top, mz.groups, mz.keep)
        assert md.top * md.ff == mz.top * mz.ff + mz.shared_ff and dos.layers[1].mlp.ff == md.top * md.ff
        ld, lz = dos.layers[0].mixer, zer.layers[0].mixer
        assert (ld.heads, ld.dim, ld.rot_dim, ld.vdim, ld.kv_rank, ld.window) == (lz.heads, lz.dim, lz.rot_dim, lz.vdim, lz.kv_rank, lz.window)
        rd, rz = dos.layers[1].mixer, zer.layers[1].mixer
        assert (rd.heads, rd.dim, rd.vdim) == (rz.heads, rz.dim, rz.vdim)
        assert dict(param_shapes(dos))["l3.dwa"] == (5,)


def test_family_libraries_hold_every_entry_point_their_model_calls():
    """A checkout without a built library compiles only the translation units of the model's family (hip/lib.py FAMILY_SOURCES): every
    wrapper a family's model file (and the base class they share) calls must bind a symbol that one of those units defines -- in
    both element modes, also on branches a quick run does not take."""
    import os
    import re
    from ssd_amd.hip.lib import FAMILY_SOURCES
    from tests.conftest import ROOT
    ops = open(os.path.join(ROOT, "ssd_amd", "hip", "ops.py")).read()
    symbol_of = {}
    for m in re.finditer(r"^def (\w+)\(.*?(?=^def |\Z)", ops, flags=re.M | re.S):
        syms = re.findall(r"\.(ssd_\w+)\(", m.group(0))
        if syms:
            symbol_of[m.group(1)] = syms
    base = open(os.path.join(ROOT, "ssd_amd", "res32.py")).read()
    for family, sources in FAMILY_SOURCES.items():
        defined = set()
        for f in sources:
            defined |= set(re.findall(r'extern "C" int (ssd_\w+)\(', open(os.path.join(ROOT, "ssd_amd", "csrc", f)).read()))
        model = open(os.path.join(ROOT, "ssd_amd", family + ".py")).read()
        used = set(re.findall(r"\bH\.(\w+)\(", model + base))
        assert used, family
        for op in sorted(used):
            for sym in symbol_of[op]:
                assert sym in defined, f"{family}: H.{op} needs {sym}, which none of {sources} defines"
