"""Replay of a token trace through the engine's own runner and block manager: given token ids are fed step by step -- prompt
portions of any size beside single tokens of other requests, all entries of a step as ONE varlen batch -- and the fp32 logits of the
asked positions come back; nothing is sampled.  The schedule is the caller's (a trace names what runs in which step), everything
else is the generation path's: Config, ModelRunner (weights, paged KV cache, staging, forward, LM head), BlockManager (pages are
taken at admission and as a request grows, and given back when it ends, so pages are used again; a model with recurrent layers
also gets one of `max_live` state slots per request from it) and Sequence.

Prefix caching is off here: a trace asks for logits at given positions, and a position served from another request's pages is
never computed."""
from __future__ import annotations

import os

import torch

from ssd_amd.config import Config
from ssd_amd.engine.block_manager import BlockManager
from ssd_amd.engine.sequence import Sequence, SequenceStatus


class TraceEngine:
    def __init__(self, model: str, dtype: str = "bfloat16", max_tokens: int = 4096, max_live: int = 4, block_size: int = 64,
                 runner_factory=None, **config_kw):
        pool = -(-max_tokens // block_size)
        cap = pool * block_size
        self.config = Config(model, dtype=dtype, kvcache_block_size=block_size, max_num_seqs=max_live, max_model_len=cap,
                             max_num_batched_tokens=cap, num_kvcache_blocks=pool, enforce_eager=True, **config_kw)
        Sequence.block_size = block_size
        self.max_live = max_live
        if runner_factory is None:
            from ssd_amd.engine.model_runner import ModelRunner
            device = torch.device("cuda", 0)
            self.runner = ModelRunner(self.config, self.config.hf_config, is_draft=False, device=device,
                                      model_path=model if os.path.isdir(model) else None, weights_seed=self.config.weights_seed,
                                      num_kvcache_blocks=pool)
        else:
            self.runner = runner_factory(self.config)
        assert getattr(self.runner, "num_kvcache_blocks", pool) == pool, "the runner's cache must hold every page the block manager hands out"
        # a model with recurrent layers: max_live state slots, taken and returned with a request's pages
        recurrent = bool(getattr(self.config.hf_config, "recurrent", False))
        self.blocks = BlockManager(pool, block_size, max_model_len=cap, prefix_cache=False, state_slots=max_live if recurrent else 0)
        self.live: dict[str, Sequence] = {}

    def step(self, entries: list[dict], end: list[str] = ()) -> torch.Tensor | None:
        """entries: [{"id", "tokens", "want"}]; returns the logits of the wanted places (entry order, then want order) or None."""
        seqs, want = [], []
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            assert toks, "an entry brings at least one token"
            seq = self.live.get(e["id"])
            if seq is None:
                if len(self.live) >= self.max_live:
                    raise RuntimeError(f"more than {self.max_live} live requests")
                seq = Sequence(toks)
                if not self.blocks.can_allocate(seq):
                    raise RuntimeError("the KV pool is full")
                self.blocks.allocate(seq)
                seq.status = SequenceStatus.RUNNING
                self.live[e["id"]] = seq
            else:
                seq.token_ids.extend(toks)
                seq.num_tokens += len(toks)
                seq.last_token = toks[-1]
                if not self.blocks.can_append(seq, 0):
                    raise RuntimeError("the KV pool is full")
                self.blocks.may_append(seq, 0)
            seqs.append(seq)
            want.append([int(i) for i in e.get("want", ())])
        logits = None
        if seqs:
            logits = self.runner.run_rows(seqs, want)
            for seq in seqs:
                seq.num_cached_tokens = seq.num_tokens
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                seq.status = SequenceStatus.FINISHED
                self.blocks.deallocate(seq)
        return logits if (logits is not None and logits.shape[0]) else None
