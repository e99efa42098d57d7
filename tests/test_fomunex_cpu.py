"""CPU-side checks of the Fomunex integration: the config reader (defaults, borrowed weights, sizes that only a tensor's shape gives),
checkpoint names, state slots through the trace engine (a recording runner, no GPU), the bench option, and the oracle's own mechanisms
against hand-made cases and against restatements (attention as an explicit sum with the sink as a key of value zero, the time-mixing
and state-space recurrences as explicit sums over earlier tokens)."""
import json
import math

import pytest
import torch

from oracle import fomunex as F
from ssd_amd.model_config import FomunexConfig, read_native_config
from ssd_amd.weights import param_shapes, synthetic_state_dict

F64 = torch.float64


def small_config():
    return F.make_config([F.attention_layer(mlp=F.dense_mlp()), F.wkv_layer(mlp=F.moe_mlp()), F.mamba2_layer(),
                          F.attention_layer(heads=2, kv_heads=1, window=0, softcap=0, mlp=F.moe_mlp(experts=3, top=1)),
                          F.attention_layer(weights_of=0, mlp=F.dense_mlp()), F.wkv_layer(weights_of=1, mlp=F.moe_mlp())])


def write(path, cfg, w):
    from safetensors.torch import save_file
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(path / "model.safetensors"))


def test_config_reader_defaults_borrowed_weights_and_sizes_from_tensor_shapes(tmp_path):
    cfg = small_config()
    w = F.random_model(cfg, 0)                    # drops decay_rank from cfg: only the checkpoint knows it now
    assert all("decay_rank" not in l["mixer"] for l in cfg["layers"])
    write(tmp_path, cfg, w)
    c = read_native_config(str(tmp_path))
    assert isinstance(c, FomunexConfig) and c.family == "fomunex" and c.recurrent and c.num_layers == 6
    a0, a3 = c.layers[0].mixer, c.layers[3].mixer
    assert (a0.kind, a0.heads, a0.kv_heads, a0.window, a0.softcap) == ("attention", 4, 2, 9, 12.0)
    assert (a3.window, a3.softcap) == (0, 0.0) and c.layers[2].mlp is None
    assert [l.weights_of for l in c.layers] == [0, 1, 2, 3, 0, 1]
    assert c.layers[1].mixer.decay_rank == c.layers[5].mixer.decay_rank == 6          # from l1.mix.w1's shape
    assert a0.slopes() == [2.0 ** (-8.0 * (h + 1) / 4) for h in range(4)]
    assert (c.logit_scale, c.logit_softcap, c.max_position_embeddings) == (1.5, 25.0, 512)
    assert {n: tuple(s) for n, s in param_shapes(c)} == {n: tuple(t.shape) for n, t in w.items()}
    assert not any(n.startswith(("l4.", "l5.")) for n, _ in param_shapes(c))           # borrowed layers own no tensors
    sd = synthetic_state_dict(c, 0, 0.02)
    assert set(sd) == set(w) and all(sd[n].shape == w[n].shape for n in w) and float(sd["l0.norm1"]) == 1.0
    # no max_positions key: the position table's rows; no scale / logit keys: defaults
    bare = json.loads(json.dumps(cfg))
    del bare["max_positions"], bare["logit_scale"], bare["logit_softcap"], bare["layers"][0]["mixer"]["scale"]
    write(tmp_path, bare, w)
    b = read_native_config(str(tmp_path))
    assert b.max_position_embeddings == 512 and (b.logit_scale, b.logit_softcap) == (1.0, 0.0) and b.layers[0].mixer.scale == 16 ** -0.5
    short = json.loads(json.dumps(cfg))                   # a borrowing layer that only names its source: the rest equals the source's
    short["layers"][4] = {"weights_of": 0}
    sc = FomunexConfig.from_json(short)
    assert sc.layers[4].mixer == sc.layers[0].mixer and sc.layers[4].mlp == sc.layers[0].mlp and sc.layers[4].weights_of == 0
    assert not FomunexConfig.from_json(F.make_config([F.attention_layer()])).recurrent
    for breakit in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][0]["mlp"].update(kind="glu"),
                    lambda d: d["layers"][0]["mixer"].update(kv_heads=3), lambda d: d["layers"][1]["mlp"]["router"].update(top=9),
                    lambda d: d["layers"][4].update(weights_of=1), lambda d: d["layers"][5].update(weights_of=4),
                    lambda d: d["layers"][2]["mixer"].update(groups=3)):
        bad = small_config()
        breakit(bad)
        with pytest.raises(ValueError):
            FomunexConfig.from_json(bad)


def test_oracle_attention_is_a_softmax_with_one_more_key_of_value_zero():
    """The sink as an extra key whose score is the sink itself and whose value is zero; the window and the distance penalty by hand."""
    cfg = F.make_config([F.attention_layer(heads=2, kv_heads=1, dim=4, vdim=3, window=3, softcap=2.0, scale=1.5)], width=8)
    w = {n: t.double() for n, t in F.random_model(cfg, 1).items()}
    m, eps = cfg["layers"][0]["mixer"], 1e-5
    T = 7
    h = torch.randn(T, 8, dtype=F64, generator=torch.Generator().manual_seed(2))
    q = F.rms((h @ w["l0.mix.q"].T).view(T, 2, 4), eps)
    k = F.rms((h @ w["l0.mix.k"].T).view(T, 1, 4), eps)
    v = (h @ w["l0.mix.v"].T).view(T, 1, 3)
    out = torch.zeros(T, 2, 3, dtype=F64)
    for hh in range(2):
        slope = 2.0 ** (-8.0 * (hh + 1) / 2)
        for i in range(T):
            js = [j for j in range(T) if 0 <= i - j < 3]
            s = torch.stack([2.0 * torch.tanh(1.5 * (q[i, hh] @ k[j, 0]) / 2.0) - slope * (i - j) for j in js] + [w["l0.mix.sink"][hh]])
            p = torch.softmax(s, 0)
            out[i, hh] = sum(p[n] * v[j, 0] for n, j in enumerate(js))
    ref = out.reshape(T, 6) @ w["l0.mix.o"].T
    assert torch.allclose(F.window_attention(h, w, "l0.mix.", m, eps), ref, rtol=1e-10, atol=1e-10)
    assert len([j for j in range(T) if 0 <= 5 - j < 3]) == 3                      # itself and the two before it


def test_oracle_recurrences_are_explicit_sums_over_earlier_tokens():
    cfg = F.make_config([F.wkv_layer(heads=2, dim=4, decay_rank=3), F.mamba2_layer(heads=2, vdim=3, state=4, groups=1, conv=3, norm_groups=1)], width=8)
    w = {n: t.double() for n, t in F.random_model(cfg, 3).items()}
    eps, T = 1e-5, 9
    h = torch.randn(T, 8, dtype=F64, generator=torch.Generator().manual_seed(4))
    # time mixing: o_t = sum_{j<t} (prod_{j<i<t} w_i) (r_t . k_j) v_j + (r_t . (u k_t)) v_t, per key channel
    p = "l0.mix."
    prev = torch.cat([torch.zeros(1, 8, dtype=F64), h[:-1]])
    mix = lambda s: h + (prev - h) * w[p + "mu." + s]
    r, k, v = ((mix(s) @ w[p + s].T).view(T, 2, 4) for s in "rkv")
    dec = torch.exp(-torch.exp(torch.tanh(mix("w") @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(T, 2, 4)
    o = torch.zeros(T, 2, 4, dtype=F64)
    for t in range(T):
        for hh in range(2):
            o[t, hh] = (r[t, hh] * w[p + "u"][hh] * k[t, hh]).sum() * v[t, hh]
            for j in range(t):
                carry = torch.ones(4, dtype=F64)
                for i in range(j + 1, t):
                    carry = carry * dec[i, hh]
                o[t, hh] += (r[t, hh] * carry * k[j, hh]).sum() * v[j, hh]
    ref = (F.rms(o, eps).reshape(T, 8) * w[p + "norm"] * F.silu(mix("g") @ w[p + "g"].T)) @ w[p + "o"].T
    assert torch.allclose(F.wkv_mixer(h, w, p, cfg["layers"][0]["mixer"], eps), ref, rtol=1e-9, atol=1e-9)
    # state space: y_t = sum_{j<=t} exp(A sum_{j<i<=t} dt_i) dt_j (C_t . B_j) x_j + D x_t
    p, m = "l1.mix.", cfg["layers"][1]["mixer"]
    z = h @ w[p + "in"].T
    inner = 6
    xbc = z[:, inner:2 * inner + 8]
    pad = torch.cat([torch.zeros(2, 14, dtype=F64), xbc])
    xbc = F.silu(w[p + "conv.b"] + sum(pad[c:c + T] * w[p + "conv"][:, c] for c in range(3)))
    x, Bm, Cm = xbc[:, :6].view(T, 2, 3), xbc[:, 6:10], xbc[:, 10:14]
    dt = torch.log1p(torch.exp(z[:, -2:] + w[p + "dt_bias"]))
    A = -torch.exp(w[p + "A_log"])
    y = torch.zeros(T, 2, 3, dtype=F64)
    for t in range(T):
        for hh in range(2):
            y[t, hh] = w[p + "D"][hh] * x[t, hh]
            for j in range(t + 1):
                y[t, hh] += torch.exp(A[hh] * dt[j + 1:t + 1, hh].sum()) * dt[j, hh] * (Cm[t] @ Bm[j]) * x[j, hh]
    ref = (F.rms(y.reshape(T, 6) * F.silu(z[:, :6]), eps) * w[p + "norm"]) @ w[p + "o"].T
    assert torch.allclose(F.mamba2_mixer(h, w, p, m, eps), ref, rtol=1e-9, atol=1e-9)


def test_oracle_feed_forwards_on_hand_made_cases():
    eps = 1e-5
    w = {"up": torch.eye(3, dtype=F64), "down": torch.eye(3, dtype=F64), "act": torch.tensor([2.0, 0.0, 0.0, 0.5], dtype=F64)}
    h = torch.tensor([[3.0, 0.0, -3.0]], dtype=F64)
    assert torch.allclose(F.polynorm_mlp(h, w, "", eps), 2.0 * h / math.sqrt(6.0 + eps) + 0.5)
    w["act"] = torch.tensor([0.0, 1.0, 0.0, 0.0], dtype=F64)
    assert torch.allclose(F.polynorm_mlp(h, w, "", eps), h * h / math.sqrt(54.0 + eps))
    # routed: the weight multiplies the expert's input, so with a clamp it is NOT the weighted output
    ml = F.moe_mlp(experts=2, top=1, ff=1, limit=1.0)
    w = {"router": torch.tensor([[0.0, 0.0], [2.0, 0.0]], dtype=F64), "e0.gate": torch.ones(1, 2, dtype=F64), "e0.up": torch.ones(1, 2, dtype=F64),
         "e0.down": torch.ones(2, 1, dtype=F64), "e1.gate": torch.tensor([[4.0, 0.0]], dtype=F64), "e1.up": torch.tensor([[-8.0, 0.0]], dtype=F64),
         "e1.down": torch.tensor([[1.0], [2.0]], dtype=F64)}
    h = torch.tensor([[1.0, 5.0]], dtype=F64)
    s = 1.0 / (1.0 + math.exp(-2.0))                       # expert 1 wins
    g, u = min(4.0 * s, 1.0), max(-8.0 * s, -1.0)
    val = g / (1.0 + math.exp(-1.702 * g)) * (u + 1.0)
    assert torch.allclose(F.routed_mlp(h, w, "", ml), torch.tensor([[val, 2.0 * val]], dtype=F64))
    h0 = torch.tensor([[0.0, 5.0]], dtype=F64)             # a tie (both scores 0.5): the lower index
    out = F.routed_mlp(h0, w, "", ml)
    g = min(0.5 * 5.0, 1.0)
    assert torch.allclose(out, torch.full((1, 2), g / (1.0 + math.exp(-1.702 * g)) * 2.0, dtype=F64))


class _Recorder:
    """Stands in for the ModelRunner: records what every step would run."""
    def __init__(self, config):
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
    # attention only: no slots at all
    plain = F.make_config([F.attention_layer()])
    write(tmp_path, plain, F.random_model(plain, 0))
    assert TraceEngine(str(tmp_path), max_tokens=64, block_size=16, runner_factory=_Recorder).blocks.free_state_slots is None


def test_bench_option_and_equal_size_pairs():
    """bench.py accepts --workload fomunex next to its default; every benchmarked size pairs a Fomunex model with a Zerusun model of the
    same width, layers, vocabulary, experts, top, window and active feed-forward parameters per token."""
    import bench
    from ssd_amd.utils import arch_bench
    assert bench.parse([]).workload == "c4"                                  # the default workload is untouched
    a = bench.parse(["--workload", "fomunex", "--arch-size", "w2048", "--arch-batch", "1", "--arch-only", "fomunex"])
    assert a.workload == "fomunex" and a.arch_size == "w2048" and a.arch_batch == 1 and a.arch_only == "fomunex"
    for size in arch_bench.SIZES:
        fom, zer = arch_bench.fomunex_models(size)
        assert fom.hidden_size == zer.hidden_size and fom.vocab_size == zer.vocab_size and fom.num_layers == zer.num_layers
        assert [l.mixer.kind for l in fom.layers] == ["attention", "wkv", "attention", "mamba2"] and fom.recurrent
        assert [l.weights_of for l in fom.layers] == list(range(fom.num_layers))
        mf, mz = fom.layers[0].mlp, zer.layers[0].mlp
        assert (mf.experts, mf.top) == (mz.experts, mz.top) and mf.top * mf.ff == mz.top * mz.ff + mz.shared_ff
        assert 2 * fom.layers[1].mlp.ff == 3 * mf.top * mf.ff and fom.layers[0].mixer.window == zer.layers[0].mixer.window
        assert dict(param_shapes(fom))["l1.mix.w1"] == (64, fom.hidden_size)
