"""bench.py --workload fatulix | zerusun: prefill and decode throughput of the Fatulix decoder at layer sizes that resemble real models (random
weights), beside the closest existing family -- a dense grouped-query Llama decoder -- at equal active size: the same width, query /
key / value / output projection sizes (two 64-wide maps per head = one 128-wide head), the same feed-forward parameters per token
(top * 2 * ff + 2 * shared_ff = 3 * intermediate), layers, vocabulary, prompt and batch.  Both run through the same ModelRunner paths
(`run(seqs, is_prefill)`: staging, varlen prefill / hipGraph decode, LM head, argmax).

--workload zerusun: the Zerusun decoder (layers alternate latent attention with a sliding window and linear attention over a recurrent
state; routed three-matrix experts with group-limited choice and a gated shared expert; the stack is one loop of one pass) beside
the closest existing family, Fatulix, at equal size: the same width, layers, vocabulary, experts, top and feed-forward parameters per
token (three-matrix experts of 2/3 the two-matrix experts' ff), mixers of about the same parameter count.

--workload fomunex: the Fomunex decoder (pre-norm layers; windowed attention with a sink / time mixing / windowed attention / state
space; sigmoid-routed clamped-GLU experts and one PolyNorm dense feed-forward) beside the closest existing family, Zerusun (fp32
residual, a windowed attention over a paged cache next to a recurrent mixer over state slots, routed three-matrix experts), at equal
size: the same width, layers, vocabulary, experts, top and active feed-forward parameters per token, the same window, mixers of about
the same parameter count.
--workload dosuvik: the Dosuvik decoder (output-norm layers with a depth average; latent attention / retention / windowed attention with
rotated values and a sink / retention; grouped sigmoid-routed silu-GLU experts and one dense clamped GLU) beside the closest existing
family, Zerusun (the same latent attention and linear-attention scan kernels, a grouped router, silu-GLU experts), at equal size.
"""
from __future__ import annotations

import json
import time

import torch

from ssd_amd.config import Config
from ssd_amd.engine.block_manager import BlockManager
from ssd_amd.engine.sequence import Sequence
from ssd_amd.model_config import (BiasedGroupRoutedMLP, ClampedGluMLP, DosuvikConfig, DosuvikLayer, GatedLatentAttention, RetentionMixer,
                                  Rotary, RotaryWindowAttention)
from ssd_amd.model_config import (DiffAttention, FatulixConfig, FatulixLayer, FomunexConfig, FomunexLayer, GroupRoutedMLP, LatentAttention,
                                  LightningAttention, Mamba2Mixer, ModelConfig, PolyNormMLP, RopeSpec, RoutedMLP, SigmoidRoutedMLP,
                                  WindowAttention, WkvMixer, ZerusunConfig, ZerusunLayer)

VOCAB = 32000
SIZES = {
    # name: (width, layers, heads, kv heads, experts, top, expert ff, shared ff, dense intermediate of the equal Llama)
    "w2048": (2048, 4, 16, 4, 8, 2, 1536, 3072, 4096),
    "w4096": (4096, 4, 32, 8, 16, 2, 3072, 6144, 8192),
}


def models(size: str):
    W, L, Hh, G, E, top, ff, sff, inter = SIZES[size]
    assert top * 2 * ff + 2 * sff == 3 * inter
    layer = FatulixLayer(DiffAttention(Hh, G, 64, 128, 0.25, 64 ** -0.5), RoutedMLP(E, top, ff, sff))
    fat = FatulixConfig(VOCAB, W, 1e-5, [layer] * L)
    llama = ModelConfig("llama", W, L, Hh, G, 128, inter, VOCAB, 1e-5, 5e5, 131072, False)
    return fat, llama


def zerusun_models(size: str):
    """(Zerusun, Fatulix) of equal size."""
    W, L, Hh, G, E, top, ff, sff, inter = SIZES[size]
    fat, _ = models(size)
    rope = RopeSpec(64, 1e6, {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0})
    mlp = GroupRoutedMLP(E, top, ff * 2 // 3, 4, 2, 1.5, sff * 2 // 3)
    lat = ZerusunLayer(LatentAttention(Hh, 128, 64, 128, 3 * W // 8, 512, 192 ** -0.5, 1024, rope), mlp)
    lin = ZerusunLayer(LightningAttention(Hh // 2, 128, 128, [1.0 - 2.0 ** -(3 + 5 * h / (Hh // 2)) for h in range(Hh // 2)]), mlp)
    zer = ZerusunConfig(VOCAB, W, 1e-5, [lat, lin] * (L // 2), 0, L, 1)
    return zer, fat


def fomunex_models(size: str):
    """(Fomunex, Zerusun) of equal size: the experts carry what Zerusun's experts and its shared expert carry per token together."""
    W, L, Hh, G, E, top, ff, sff, inter = SIZES[size]
    zer, _ = zerusun_models(size)
    ffx = (ff + sff // top) * 2 // 3
    moe = SigmoidRoutedMLP(E, top, ffx, 7.0)
    dense = PolyNormMLP(3 * top * ffx // 2)                  # two matrices instead of top * three
    att = WindowAttention(Hh, G, 128, 128, 0.125, 30.0, 1024)
    layers = [FomunexLayer(att, moe, 0), FomunexLayer(WkvMixer(W // 128, 64, 64), dense, 1), FomunexLayer(att, moe, 2),
              FomunexLayer(Mamba2Mixer(W // 64, 64, 128, 1, 4, 1), moe, 3)]
    fom = FomunexConfig(VOCAB, W, 1e-5, (layers * (L // 4 + 1))[:L], 8192, 1.0, 30.0)
    for i, l in enumerate(fom.layers):
        fom.layers[i] = FomunexLayer(l.mixer, l.mlp, i)
    return fom, zer


def dosuvik_models(size: str):
    """(Dosuvik, Zerusun) of equal size: the same width, layers, vocabulary, experts, top, router groups, latent and state sizes; the
    experts carry what Zerusun's experts and its shared expert carry per token together, one layer has the dense feed-forward of the
    same active parameter count."""
    W, L, Hh, G, E, top, ff, sff, inter = SIZES[size]
    zer, _ = zerusun_models(size)
    ffx = (ff + sff // top) * 2 // 3
    moe = BiasedGroupRoutedMLP(E, top, ffx, 4, 2)
    dense = ClampedGluMLP(top * ffx, 7.0)
    lat = GatedLatentAttention(Hh, 128, 64, 128, 512, 192 ** -0.5, Rotary(64, 1e6, "interleaved"), 1024)
    ret = RetentionMixer(Hh // 2, 128, 128, [1.0 - 2.0 ** -(3 + 5 * h / (Hh // 2)) for h in range(Hh // 2)], Rotary(128, 1e6))
    att = RotaryWindowAttention(Hh, G, 128, 128, 128 ** -0.5, 1024, Rotary(64, 1e4))
    layers = [DosuvikLayer(lat, moe), DosuvikLayer(ret, dense), DosuvikLayer(att, moe), DosuvikLayer(ret, moe)]
    return DosuvikConfig(VOCAB, W, 1e-5, (layers * (L // 4 + 1))[:L]), zer


def _runner(cfg, max_len: int, batch: int, dtype: str = "bfloat16"):
    from ssd_amd.engine.model_runner import ModelRunner
    bs = 256
    blocks = batch * (-(-max_len // bs)) + 2
    config = Config("synthetic", hf_config=cfg, dtype=dtype, kvcache_block_size=bs, max_num_seqs=batch, max_model_len=max_len,
                    max_num_batched_tokens=max(max_len, 4096), num_kvcache_blocks=blocks)
    Sequence.block_size = bs
    runner = ModelRunner(config, cfg, is_draft=False, device=torch.device("cuda", 0), weights_seed=0, num_kvcache_blocks=blocks)
    assert runner.num_kvcache_blocks == blocks, "the runner's cache must hold every page the block manager hands out"
    return runner, BlockManager(blocks, bs, max_model_len=max_len, prefix_cache=False,
                                state_slots=batch if getattr(cfg, "recurrent", False) else 0)


def _timed(fn, steps: int, warmup: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def measure(cfg, prompt_len: int, batch: int, steps: int, warmup: int) -> dict:
    """Prefill of ONE prompt_len-token prompt (eager, as the engine prefills) and `batch` sequences decoding from that context."""
    max_len = prompt_len + steps + warmup + 8
    runner, bm = _runner(cfg, max_len, batch)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]

    def prefill_once():
        s = Sequence(prompts[0])
        bm.allocate(s)
        runner.run([s], True)
        bm.deallocate(s)

    t_pf = _timed(prefill_once, max(3, steps // 8), 2)
    seqs = []
    for p in prompts:
        s = Sequence(p)
        bm.allocate(s)
        tok = runner.run([s], True)[0]
        s.append_token(tok)
        s.num_cached_tokens = len(s) - 1
        seqs.append(s)

    def decode_once():
        for s in seqs:
            bm.may_append(s, 1)
        toks = runner.run(seqs, False)
        for s, t in zip(seqs, toks):
            s.append_token(t)
            s.num_cached_tokens = len(s) - 1

    t_dec = _timed(decode_once, steps, warmup)
    out = {"prefill_tok_s": round(prompt_len / t_pf, 1), "prefill_ms": round(t_pf * 1e3, 3), "decode_tok_s": round(batch / t_dec, 1),
           "decode_ms_per_step": round(t_dec * 1e3, 3)}
    m = runner.model
    if hasattr(m, "active_weight_bytes"):
        out["decode_weight_gb"] = round(m.active_weight_bytes(batch) / 1e9, 3)
    else:
        out["decode_weight_gb"] = round(m.weight_bytes() / 1e9, 3)
    out["decode_hbm_roofline_frac"] = round(out["decode_weight_gb"] * 1e9 / t_dec / 8e12, 3)
    runner.exit()
    del runner
    torch.cuda.empty_cache()
    return out


def run_zerusun(args) -> dict:
    steps, warmup = args.steps, args.warmup
    prompt_len = args.input_len if args.input_len != 128 else 2048
    results = {}
    sizes = list(SIZES) if getattr(args, "arch_size", "all") == "all" else [args.arch_size]
    batches = (1, 8) if not getattr(args, "arch_batch", 0) else (args.arch_batch,)
    only = getattr(args, "arch_only", "both")
    for size in sizes:
        zer, fat = zerusun_models(size)
        for batch in batches:
            key = f"{size} prompt={prompt_len} batch={batch}"
            results[key] = {}
            if only in ("both", "zerusun"):
                results[key]["zerusun"] = measure(zer, prompt_len, batch, steps, warmup)
            if only in ("both", "fatulix"):
                results[key]["fatulix_equal_size"] = measure(fat, prompt_len, batch, steps, warmup)
            print(f"[arch_bench] {key}: {json.dumps(results[key])}", flush=True)
    k = f"w4096 prompt={prompt_len} batch=8"
    if k not in results or len(results[k]) < 2:
        return {"metric": "Zerusun / equal-size Fatulix throughput (partial run)", "sizes": results}
    return {"metric": "decode tokens/s, Zerusun w4096 (4 layers: latent attention / linear attention, 16 experts top 2 + shared), batch 8, "
                      "beside an equal-size Fatulix decoder",
            "value": results[k]["zerusun"]["decode_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": results[k]["zerusun"]["decode_ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic (random weights, random tokens)",
            "config": {"model": "zerusun-w4096-synthetic", "global_batch": 8, "seq_len": prompt_len, "parallelism": "single GPU"},
            "closest_model_value": results[k]["fatulix_equal_size"]["decode_tok_s"], "sizes": results}


def run_dosuvik(args) -> dict:
    """bench.py --workload dosuvik: the Dosuvik decoder beside an equal-size Zerusun decoder (the family that shares its latent
    attention, its linear-attention scan, its grouped router and its silu-GLU experts)."""
    sizes = list(SIZES) if args.arch_size == "all" else [args.arch_size]
    batches = [args.arch_batch] if args.arch_batch else [1, 8]
    only = getattr(args, "arch_only", "both")
    prompt_len, steps, warmup = 2048, max(args.steps, 8), max(args.warmup, 2)
    results = {}
    for size in sizes:
        dos, zer = dosuvik_models(size)
        for b in batches:
            key = f"{size}_b{b}"
            results[key] = {}
            if only in ("both", "dosuvik"):
                results[key]["dosuvik"] = measure(dos, prompt_len, b, steps, warmup)
            if only in ("both", "zerusun"):
                results[key]["zerusun_equal_size"] = measure(zer, prompt_len, b, steps, warmup)
            print(f"[arch_bench] {key}: {json.dumps(results[key])}", flush=True)
    k = "w4096_b8"
    if k not in results or len(results[k]) < 2:
        return {"metric": "Dosuvik / equal-size Zerusun throughput (partial run)", "sizes": results}
    return {"metric": "decode tokens/s, Dosuvik w4096 (4 layers: latent attention / retention / windowed attention / retention, 16 "
                      "experts top 2), batch 8, beside an equal-size Zerusun decoder",
            "value": results[k]["dosuvik"]["decode_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": results[k]["dosuvik"]["decode_ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"model": "dosuvik-w4096-synthetic", "global_batch": 8, "seq_len": prompt_len, "parallelism": "single GPU"},
            "closest_model_value": results[k]["zerusun_equal_size"]["decode_tok_s"], "sizes": results}


def run_fomunex(args) -> dict:
    steps, warmup = args.steps, args.warmup
    prompt_len = args.input_len if args.input_len != 128 else 2048
    results = {}
    sizes = list(SIZES) if getattr(args, "arch_size", "all") == "all" else [args.arch_size]
    batches = (1, 8) if not getattr(args, "arch_batch", 0) else (args.arch_batch,)
    only = getattr(args, "arch_only", "both")
    for size in sizes:
        fom, zer = fomunex_models(size)
        for batch in batches:
            key = f"{size} prompt={prompt_len} batch={batch}"
            results[key] = {}
            if only in ("both", "fomunex"):
                results[key]["fomunex"] = measure(fom, prompt_len, batch, steps, warmup)
            if only in ("both", "zerusun"):
                results[key]["zerusun_equal_size"] = measure(zer, prompt_len, batch, steps, warmup)
            print(f"[arch_bench] {key}: {json.dumps(results[key])}", flush=True)
    k = f"w4096 prompt={prompt_len} batch=8"
    if k not in results or len(results[k]) < 2:
        return {"metric": "Fomunex / equal-size Zerusun throughput (partial run)", "sizes": results}
    return {"metric": "decode tokens/s, Fomunex w4096 (4 layers: windowed attention / time mixing / windowed attention / state space, 16 "
                      "experts top 2), batch 8, beside an equal-size Zerusun decoder",
            "value": results[k]["fomunex"]["decode_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": results[k]["fomunex"]["decode_ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic (random weights, random tokens)",
            "config": {"model": "fomunex-w4096-synthetic", "global_batch": 8, "seq_len": prompt_len, "parallelism": "single GPU"},
            "closest_model_value": results[k]["zerusun_equal_size"]["decode_tok_s"], "sizes": results}


def run(args) -> dict:
    steps, warmup = args.steps, args.warmup
    prompt_len = args.input_len if args.input_len != 128 else 2048
    results = {}
    sizes = list(SIZES) if getattr(args, "arch_size", "all") == "all" else [args.arch_size]
    batches = (1, 8) if not getattr(args, "arch_batch", 0) else (args.arch_batch,)
    only = getattr(args, "arch_only", "both")
    for size in sizes:
        fat, llama = models(size)
        for batch in batches:
            key = f"{size} prompt={prompt_len} batch={batch}"
            results[key] = {}
            if only in ("both", "fatulix"):
                results[key]["fatulix"] = measure(fat, prompt_len, batch, steps, warmup)
            if only in ("both", "llama"):
                results[key]["llama_equal_size"] = measure(llama, prompt_len, batch, steps, warmup)
            print(f"[arch_bench] {key}: {json.dumps(results[key])}", flush=True)
    k = f"w4096 prompt={prompt_len} batch=8"
    if k not in results or len(results[k]) < 2:
        return {"metric": "Fatulix / equal-size Llama throughput (partial run)", "sizes": results}
    return {"metric": "decode tokens/s, Fatulix w4096 (4 layers, 16 experts top 2 + shared), batch 8, beside an equal-size Llama decoder",
            "value": results[k]["fatulix"]["decode_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": results[k]["fatulix"]["decode_ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic (random weights, random tokens)",
            "config": {"model": "fatulix-w4096-synthetic", "global_batch": 8, "seq_len": prompt_len, "parallelism": "single GPU"},
            "closest_model_value": results[k]["llama_equal_size"]["decode_tok_s"], "sizes": results}
