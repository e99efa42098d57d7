"""The Fomunex decoder on MI355X: PRE-NORM layers (x <- x + mixer(g1 rms(x)), x <- x + ff(g2 rms(x)), each norm weight ONE number)
over an fp32 residual that starts as embed[token] + pos[position]; three kinds of mixer -- windowed grouped-query attention with
unit-RMS q / k, capped scores, a per-head distance penalty and a softmax sink over a paged cache; RWKV-style time mixing; a Mamba-2
state space -- the latter two over recurrent fp32 state kept in per-sequence slots; PolyNorm dense or sigmoid-routed (clamped
swish-GLU experts, the routing weight on the expert's input) feed-forwards; a layer may use ANOTHER layer's weights with a cache or
state of its own; logits are scaled and capped.

Launches per layer (T token rows):
    attention      [q | k | v] GEMM -> winattn_store (q / k norms, cache pages) -> winattn_paged -> W_o GEMM
    time mixing    token_shift_mix (5 interpolations) -> batched [r | k | v | g] GEMM -> W_w1 GEMM (tanh epilogue) -> W_w2 GEMM ->
                   wkv_scan (state slot) -> group_gate_norm (per-head norm, gate after) -> W_o GEMM
    state space    W_in GEMM -> causal_conv_silu -> ssd_scan (state slot) -> group_gate_norm (gate first) -> W_o GEMM
    prenorm_tail   x += mixer output, and the feed-forward's norm
    dense ff       W_up GEMM -> polynorm_rows -> W_down GEMM
    routed ff      router GEMM -> moe_route_sigmoid -> moe_plan -> grouped [gate | up] GEMM with the clamped GLU (routing weight, clamps,
                   swish) as epilogue (fp32 mode: + glu_clamp_rows) -> grouped W_down GEMM
    prenorm_tail   x += ff output (the routed sum rides along), and the next layer's first norm
over pre-allocated buffers (nothing is allocated during a forward).  Same interface as ssd_amd.model.HipDecoder towards the ModelRunner.

Arithmetic: residual rows, norms, scores, softmax, router, decays, step sizes, recurrent states, gates of the recurrences and every GEMM
accumulator are fp32 in both modes.  dtype "bfloat16": weights, GEMM-input rows and the KV cache are bf16; "float32": they are fp32 and
products are FMA chains.
"""
from __future__ import annotations

import torch

from ssd_amd.hip import ops as H
from ssd_amd.model import AttnMeta
from ssd_amd.model_config import FomunexConfig
from ssd_amd.res32 import Res32Decoder

BF16 = torch.bfloat16
SWISH_ALPHA = 1.702             # the experts' gate is g * sigmoid(1.702 g)


class HipFomunex(Res32Decoder):
    def __init__(self, cfg: FomunexConfig, *, max_tokens: int, max_seqs: int, max_blocks: int, block_size: int, max_model_len: int,
                 device: torch.device, tp_rank: int = 0, tp_size: int = 1, tp_group=None, max_logit_rows: int | None = None,
                 max_split_tokens: int = 256, force_collectives: bool = False, taps=None, dtype: str = "bfloat16"):
        assert tp_size == 1 and taps is None, "Fomunex models are single-rank and have no activation taps"
        assert dtype in ("bfloat16", "float32")
        self.cfg, self.device = cfg, device
        self.f32 = dtype == "float32"
        self.elem = torch.float32 if self.f32 else BF16
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.use_coll, self.custom_ar, self.acts = False, None, None
        self.h = self.W = cfg.hidden_size
        self.V = cfg.vocab_size
        self.Vp = -(-self.V // 8) * 8
        self.block_size, self.max_blocks = block_size, max_blocks
        self.max_tokens = max_tokens
        self.max_logit_rows = max_logit_rows or max_tokens
        self.state_slots = max_seqs if cfg.recurrent else 0      # one per live sequence; the block manager hands them out
        self.w: dict[str, torch.Tensor] = {}
        self.kv: list = []
        self.state: list = []
        self.scalar_attention = False                 # tests / probes: the scalar form of the attention also where the MFMA form fits
        self.tap_residuals: list | None = None         # tests: receives a copy of the residual rows after every layer (eager only)

        def z(*shape, dtype=torch.float32):
            return torch.zeros(*shape, dtype=dtype, device=device)

        T, W, el = max_tokens, self.W, self.elem
        mixers = [l.mixer for l in cfg.layers]
        att = [m for m in mixers if m.kind == "attention"]
        wkv = [m for m in mixers if m.kind == "wkv"]
        ssm = [m for m in mixers if m.kind == "mamba2"]
        dense = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "dense"]
        moes = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "moe"]
        self.x = z(T, W)
        self.hn = z(T, W, dtype=el)
        self.y = z(T, W)
        self.proj = z(T * max(self._nproj(m) for m in mixers))
        self.att = z(T * max(self._nout(m) for m in mixers), dtype=el)
        if att:
            self.q = z(T * max(m.heads * m.dim for m in att), dtype=el)
        if wkv or ssm:
            self.o = z(T * max(self._nout(m) for m in wkv + ssm))
        if wkv:
            self.mix = z(T * 5 * W, dtype=el)
            self.lora = z(T * max(m.decay_rank for m in wkv), dtype=el)
            self.ww = z(T * max(m.heads * m.dim for m in wkv))
        if ssm:
            self.xbc = z(T * max(m.conv_channels for m in ssm))
        if dense:
            self.zff = z(T * max(m.ff for m in dense))
        if moes:
            top = max(m.top for m in moes)
            E = max(m.experts for m in moes)
            self.r_z = z(T * E)
            self.r_idx = z(T * top, dtype=torch.int32)
            self.r_wt = z(T * top)
            self.r_off = z(E + 1, dtype=torch.int32)
            self.r_perm = z(T * top, dtype=torch.int32)
            self.r_inv = z(T * top, dtype=torch.int32)
            self.ab = z(T * max(2 * m.top * m.ff for m in moes)) if self.f32 else None      # bf16: the GLU is the GEMM's epilogue
            self.ydn = z(T * top * W)
        ffs = [m.ff for m in dense] + [m.top * m.ff for m in moes]
        if ffs:
            self.act = z(T * max(ffs), dtype=el)
        R = self.max_logit_rows
        self.lastn = z(R, W, dtype=el)
        self.logits32 = z(R, self.V)
        self.logits = z(R, self.Vp, dtype=BF16)

    @staticmethod
    def _nproj(m) -> int:
        if m.kind == "attention":
            return (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim
        if m.kind == "wkv":
            return 4 * m.heads * m.dim
        return 2 * m.inner + 2 * m.groups * m.state + m.heads

    @staticmethod
    def _nout(m) -> int:
        return m.heads * m.vdim if m.kind == "attention" else (m.heads * m.dim if m.kind == "wkv" else m.inner)

    # ---------------------------------------------------------------------------------------------
    def load_weights(self, weight_iter) -> None:
        """Consumes (name, tensor) pairs under the checkpoint's names.  A norm's single number becomes a constant vector (the row
        kernels take a weight per coordinate); matrices that read the same rows are stacked ([q | k | v]; [r, k, v, g] for the batched
        product over the five interpolations; per expert [gate | up]); what enters a recurrence or the softmax directly (sink, slopes,
        decay offset, bonus, dt bias, A_log, skip, the activation's coefficients) is kept as fp32."""
        raw = {n: t.to(self.device) for n, t in weight_iter}
        cv = lambda t: t.to(self.elem).contiguous()
        f32 = lambda t: t.float().reshape(-1).contiguous()
        w = self.w = {}
        W = self.W
        scalar_norm = lambda n: cv(raw[n].reshape(1).expand(W))
        w["embed"], w["pos"], w["head"] = cv(raw["embed"]), cv(raw["pos"]), cv(raw["head"])
        w["final.norm"] = scalar_norm("final.norm")
        for i, lc in enumerate(self.cfg.layers):
            if lc.weights_of != i:
                continue
            p, m, ml = f"l{i}.", lc.mixer, lc.mlp
            w[p + "norm1"] = scalar_norm(p + "norm1")
            if m.kind == "attention":
                w[p + "mix.in"] = cv(torch.cat([raw[p + "mix.q"], raw[p + "mix.k"], raw[p + "mix.v"]], dim=0))
                w[p + "mix.sink"] = f32(raw[p + "mix.sink"])
                w[p + "mix.slopes"] = torch.tensor(m.slopes(), dtype=torch.float64).to(torch.float32).to(self.device)
            elif m.kind == "wkv":
                w[p + "mix.mu"] = cv(torch.stack([raw[p + f"mix.mu.{s}"] for s in "rkvgw"]))
                w[p + "mix.in"] = cv(torch.stack([raw[p + f"mix.{s}"] for s in "rkvg"]))
                w[p + "mix.w1"], w[p + "mix.w2"] = cv(raw[p + "mix.w1"]), cv(raw[p + "mix.w2"])
                w[p + "mix.w0"], w[p + "mix.u"] = f32(raw[p + "mix.w0"]), f32(raw[p + "mix.u"])
                w[p + "mix.norm"] = cv(raw[p + "mix.norm"])
            else:
                w[p + "mix.in"] = cv(raw[p + "mix.in"])
                w[p + "mix.conv"], w[p + "mix.conv.b"] = cv(raw[p + "mix.conv"]), cv(raw[p + "mix.conv.b"])
                for n in ("dt_bias", "A_log", "D"):
                    w[p + "mix." + n] = f32(raw[p + "mix." + n])
                w[p + "mix.norm"] = cv(raw[p + "mix.norm"])
            w[p + "mix.o"] = cv(raw[p + "mix.o"])
            if ml is None:
                continue
            w[p + "norm2"] = scalar_norm(p + "norm2")
            if ml.kind == "dense":
                w[p + "mlp.up"], w[p + "mlp.down"] = cv(raw[p + "mlp.up"]), cv(raw[p + "mlp.down"])
                w[p + "mlp.act"] = f32(raw[p + "mlp.act"])
            else:
                # bf16: rows interleaved (gate_0, up_0, gate_1, ...) for the grouped GEMM's paired epilogue; fp32: [gate | up], the
                # clamped GLU is a launch of its own
                pair = (lambda g, u: torch.stack([g, u], dim=1).reshape(-1, g.shape[1])) if not self.f32 else (lambda g, u: torch.cat([g, u], dim=0))
                w[p + "mlp.gu"] = cv(torch.stack([pair(raw[p + f"mlp.e{e}.gate"], raw[p + f"mlp.e{e}.up"]) for e in range(ml.experts)]))
                w[p + "mlp.down"] = cv(torch.stack([raw[p + f"mlp.e{e}.down"] for e in range(ml.experts)]))
                w[p + "mlp.router"] = cv(raw[p + "mlp.router"])
        torch.cuda.synchronize(self.device)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.w.values())

    def active_weight_bytes(self, T: int = 1) -> int:
        """HBM bytes of weights one forward of T tokens must stream at least: every dense matrix once per layer (a layer that borrows
        weights streams them again), of the experts min(E, T * top), the LM head once, one embedding and one position row per token."""
        per = {n: t.numel() * t.element_size() for n, t in self.w.items()}
        total = per["head"] + per["final.norm"]
        for lc in self.cfg.layers:
            p, ml = f"l{lc.weights_of}.", lc.mlp
            total += sum(v for n, v in per.items() if n.startswith(p + "mix.") or n.startswith(p + "norm"))
            if ml is None:
                continue
            if ml.kind == "dense":
                total += per[p + "mlp.up"] + per[p + "mlp.down"]
            else:
                frac = min(ml.experts, T * ml.top) / ml.experts
                total += int((per[p + "mlp.gu"] + per[p + "mlp.down"]) * frac) + per[p + "mlp.router"]
        return total

    def kv_block_bytes(self) -> int:
        es = 4 if self.f32 else 2
        n = sum(l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) * self.block_size * es for l in self.cfg.layers if l.mixer.kind == "attention")
        return max(n, 1)

    def state_bytes(self) -> int:
        """Bytes of recurrent state one live sequence holds (all layers)."""
        n = 0
        for l in self.cfg.layers:
            m = l.mixer
            if m.kind == "wkv":
                n += (m.heads * m.dim * m.dim + self.W) * 4
            elif m.kind == "mamba2":
                n += (m.heads * m.state * m.vdim + (m.conv - 1) * m.conv_channels) * 4
        return n

    def alloc_kv(self, num_blocks: int) -> None:
        """Per LAYER (a layer that borrows weights still has memory of its own): attention -> K pages [blocks][G][block][dim] and V pages
        transposed [blocks][G][vdim][block]; time mixing -> state [slots][H][dim][dim] and the previous token's row [slots][W]; state
        space -> state [slots][H][state][vdim] and the last conv - 1 convolution inputs [slots][conv - 1][channels]; states are fp32.
        A slot is not cleared when it is handed out: a forward whose rows start at position 0 starts from zero by itself."""
        self.num_blocks = num_blocks
        self.kv, self.state = [], []
        dev, bs, S = self.device, self.block_size, self.state_slots
        for l in self.cfg.layers:
            m = l.mixer
            if m.kind == "attention":
                self.kv.append((torch.zeros(num_blocks, m.kv_heads, bs, m.dim, dtype=self.elem, device=dev),
                                torch.zeros(num_blocks, m.kv_heads, m.vdim, bs, dtype=self.elem, device=dev)))
                self.state.append(None)
            elif m.kind == "wkv":
                self.kv.append(None)
                self.state.append((torch.zeros(S, m.heads, m.dim, m.dim, dtype=torch.float32, device=dev),
                                   torch.zeros(S, self.W, dtype=torch.float32, device=dev)))
            else:
                self.kv.append(None)
                self.state.append((torch.zeros(S, m.heads, m.state, m.vdim, dtype=torch.float32, device=dev),
                                   torch.zeros(S, max(m.conv - 1, 1), m.conv_channels, dtype=torch.float32, device=dev)))

    # ---------------------------------------------------------------------------------------------
    def launch_mixer(self, li: int, T: int, positions, meta: AttnMeta) -> None:
        """hn (normalised rows) -> y (fp32 mixer output rows)."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        lc = cfg.layers[li]
        m, p = lc.mixer, f"l{lc.weights_of}.mix."
        NP = self._nproj(m)
        seqs = dict(cu_q=meta.cu_q) if meta.cu_q is not None else dict(q_per_seq=meta.q_per_seq)
        if m.kind == "attention":
            kc, vc = self.kv[li]
            H.gemm_rows(self.hn, w[p + "in"], self.proj, T, NP, W, f)
            H.winattn_store(self.proj, NP, cfg.rms_norm_eps, meta.slot_mapping, self.q, kc, vc, T, m.heads, m.kv_heads, m.dim, m.vdim,
                            self.block_size, f)
            H.winattn_paged(self.q, kc, vc, w[p + "slopes"], w[p + "sink"], meta.block_tables, self.max_blocks, positions, meta.B, T,
                            m.heads, m.kv_heads, m.dim, m.vdim, self.block_size, m.window, m.scale, m.softcap, self.att, f, max_q=0 if self.scalar_attention else meta.max_q, **seqs)
            n_out = m.heads * m.vdim
        elif m.kind == "wkv":
            assert meta.state_slots is not None, "a model with recurrent layers needs the sequences' state slots"
            S, shift = self.state[li]
            N, R = m.heads * m.dim, m.decay_rank
            H.token_shift_mix(self.hn, w[p + "mu"], shift, positions, meta.state_slots, meta.B, self.mix, T, W, 5, f, **seqs)
            H.gemm_rows_batched(self.mix, w[p + "in"], self.proj, T, N, W, 4, 5 * W, W, 4 * N, N, f, H.GR_F32)
            H.gemm_rows_batched(self.mix[4 * W:], w[p + "w1"], self.lora, T, R, W, 1, 5 * W, 0, R, 0, f, H.GR_TANH)
            H.gemm_rows(self.lora, w[p + "w2"], self.ww, T, N, R, f)
            H.wkv_scan(self.proj, NP, 0, N, 2 * N, self.ww, N, w[p + "w0"], w[p + "u"], positions, meta.state_slots, S, self.o, self.hn,
                       shift, W, meta.B, m.heads, m.dim, f, **seqs)
            H.group_gate_norm(self.o, self.proj[3 * N:], NP, w[p + "norm"], cfg.rms_norm_eps, self.att, T, N, m.heads, False, f)
            n_out = N
        else:
            assert meta.state_slots is not None, "a model with recurrent layers needs the sequences' state slots"
            S, conv = self.state[li]
            inner, GN, C = m.inner, m.groups * m.state, m.conv_channels
            H.gemm_rows(self.hn, w[p + "in"], self.proj, T, NP, W, f)
            H.causal_conv_silu(self.proj, NP, inner, C, w[p + "conv"], w[p + "conv.b"], conv, positions, meta.state_slots, meta.B,
                               self.xbc, T, m.conv, f, **seqs)
            H.ssd_scan(self.xbc, C, 0, inner, inner + GN, self.proj, NP, 2 * inner + 2 * GN, w[p + "dt_bias"], w[p + "A_log"], w[p + "D"],
                       positions, meta.state_slots, S, self.o, inner, C, conv, m.conv, meta.B, m.heads, m.groups, m.state, m.vdim, **seqs)
            H.group_gate_norm(self.o, self.proj, NP, w[p + "norm"], cfg.rms_norm_eps, self.att, T, inner, m.norm_groups, True, f)
            n_out = inner
        H.gemm_rows(self.att, w[p + "o"], self.y, T, W, n_out, f)

    def launch_mlp(self, li: int, T: int) -> dict:
        """hn -> the feed-forward's rows; returns the keyword arguments that hand them to prenorm_tail."""
        w, f, W = self.w, self.f32, self.W
        lc = self.cfg.layers[li]
        ml, p = lc.mlp, f"l{lc.weights_of}.mlp."
        if ml.kind == "dense":
            H.gemm_rows(self.hn, w[p + "up"], self.zff, T, ml.ff, W, f)
            H.polynorm_rows(self.zff, w[p + "act"], self.cfg.rms_norm_eps, self.act, T, ml.ff, f)
            H.gemm_rows(self.act, w[p + "down"], self.y, T, W, ml.ff, f)
            return dict(y=self.y)
        E, top = ml.experts, ml.top
        H.gemm_rows(self.hn, w[p + "router"], self.r_z, T, E, W, f)
        H.moe_route_sigmoid(self.r_z, E, self.r_idx, self.r_wt, T, E, top)
        H.moe_plan(self.r_idx, T, top, E, self.r_off, self.r_perm, self.r_inv)
        # the routing weight multiplies the expert's INPUT: both products are linear in it, so it scales their fp32 results
        if f:
            H.gemm_rows_grouped(self.hn, w[p + "gu"], self.ab, self.r_off, E, T * top, 2 * ml.ff, W, f, H.GR_F32, row_idx=self.r_perm, idx_div=top)
            H.glu_clamp_rows(self.ab, self.act, T * top, ml.ff, ml.limit, SWISH_ALPHA, f, row_scale=self.r_wt, perm=self.r_perm)
        else:
            H.gemm_rows_grouped_glu_clamp(self.hn, w[p + "gu"], self.act, self.r_off, E, T * top, 2 * ml.ff, W, ml.limit, SWISH_ALPHA,
                                          row_idx=self.r_perm, idx_div=top, row_scale=self.r_wt)
        H.gemm_rows_grouped(self.act, w[p + "down"], self.ydn, self.r_off, E, T * top, W, ml.ff, f, H.GR_F32)
        return dict(ydn=self.ydn, inv=self.r_inv, top=top)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, T: int, meta: AttnMeta) -> None:
        """Runs every layer over the T token rows; leaves the fp32 residual rows in self.x."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        eps = cfg.rms_norm_eps
        assert T <= self.max_tokens and meta.mode == H.MODE_CAUSAL and (meta.cu_q is not None or meta.q_per_seq > 0)
        src = lambda i: f"l{cfg.layers[i].weights_of}."
        H.embed_pos_res32(input_ids, positions, w["embed"], w["pos"], self.x, T, W, f, norm_weight=w[src(0) + "norm1"], eps=eps,
                          norm_out=self.hn)
        for li, lc in enumerate(cfg.layers):
            self.launch_mixer(li, T, positions, meta)
            nxt = src(li) + "norm2" if lc.mlp is not None else (src(li + 1) + "norm1" if li + 1 < len(cfg.layers) else None)
            norm = dict(next_weight=w[nxt], next_out=self.hn) if nxt else {}
            H.prenorm_tail(self.x, eps, T, W, f, y=self.y, **norm)
            if lc.mlp is not None:
                ff = self.launch_mlp(li, T)
                nxt = src(li + 1) + "norm1" if li + 1 < len(cfg.layers) else None
                norm = dict(next_weight=w[nxt], next_out=self.hn) if nxt else {}
                H.prenorm_tail(self.x, eps, T, W, f, **ff, **norm)
            if self.tap_residuals is not None:
                self.tap_residuals.append(self.x[:T].clone())

    def compute_logits(self, T: int, gather: torch.Tensor | None = None, rows: int | None = None) -> int:
        """Final norm (optionally of the `gather` rows only), LM head, scale and cap: fp32 logits in logits32[:n], their bf16 rounding
        (row stride Vp, padding -inf) in logits[:n] for the sampling kernels.  Returns n."""
        n = T if gather is None else rows
        assert n <= self.max_logit_rows
        cfg = self.cfg
        H.rmsnorm_res32(self.x, self.w["final.norm"], cfg.rms_norm_eps, self.lastn, n, self.W, self.f32, gather=gather)
        H.gemm_rows(self.lastn, self.w["head"], self.logits32, n, self.V, self.W, self.f32)
        if cfg.logit_scale != 1.0 or cfg.logit_softcap > 0.0:
            H.logits_cap_rows(self.logits32, n, self.V, self.V, cfg.logit_scale, cfg.logit_softcap)
        H.rows_f32_to_bf16(self.logits32, self.logits, n, self.V, self.V, self.Vp)
        return n
