"""The Dosuvik decoder on MI355X: layers that normalise a sublayer's OUTPUT only -- x <- x + (1 + w1) rms(mixer(x)), x <- x + (1 + w2)
rms(ff(x)), the sublayers read the fp32 residual row itself -- followed by a learned weighted average over the embedding output and the
results of all layers so far; three kinds of mixer -- retention (linear attention with a fixed decay per head and rotary q / k over a
recurrent fp32 state kept in per-sequence slots), gated latent attention (keys and values from a cached low-rank latent plus one shared
rotated key part) and windowed grouped-query attention with whole-projection q / k norms, rotated values and a softmax sink over a paged
cache; a dense clamped swish-GLU or sigmoid-routed silu-GLU experts (choice correction, group-limited choice) as feed-forward.

Launches per layer (T token rows):
    retention          [q | k | v | g] GEMM -> rope_rows (q, k in place; k scaled) -> lightning_scan (state slot, raw inputs) ->
                       group_gate_norm (per-head unit RMS, silu gate after) -> W_o GEMM
    latent attention   [q | dkv | g] GEMM -> latent_store (latent norm, rope of the shared key part, cache row, q rows) -> per-head
                       W_uk^T GEMM (queries into the latent space) -> latent_attn -> per-head W_uv GEMM -> gate_rows -> W_o GEMM
    attention          [q | k | v] GEMM -> winattn_store_rope (q / k norms, rope, rotated values, cache pages) -> winattn_paged (sink,
                       window, outputs turned back) -> W_o GEMM
    postnorm_tail      x += (1 + w) rms(mixer output); the feed-forward's input rows
    dense ff           [gate | up] GEMM with the clamped GLU as epilogue (fp32 mode: + glu_clamp_rows) -> down GEMM
    routed ff          router GEMM -> moe_route_sigmoid_grouped -> moe_plan -> grouped [gate | up] GEMM (silu GLU epilogue; fp32 mode:
                       + glu_rows) -> grouped down GEMM
    postnorm_tail      x += (1 + w) rms(ff output) (the routed mix rides along), the layer's result into the history, the depth
                       average, the next layer's input rows
over pre-allocated buffers (nothing is allocated during a forward).  Same interface as ssd_amd.model.HipDecoder towards the ModelRunner.

Rotary layouts: the kernels pair entry i with i + dims / 2.  A mixer whose checkpoint pairs 2i with 2i + 1 gets the output rows of its
projections permuted at load (Rotary.to_halves): q and k parts permuted alike leave every score unchanged.

Arithmetic: residual rows and their sums, the history and its average, norms, rope angles, scores, softmax, router, decays, the recurrent
state, gates and every GEMM accumulator are fp32 in both modes.  dtype "bfloat16": weights, GEMM-input rows and the caches are bf16;
"float32": they are fp32 and products are FMA chains.
"""
from __future__ import annotations

import torch

from ssd_amd.hip import ops as H
from ssd_amd.model import AttnMeta
from ssd_amd.model_config import DosuvikConfig
from ssd_amd.res32 import Res32Decoder

BF16 = torch.bfloat16


class HipDosuvik(Res32Decoder):
    def __init__(self, cfg: DosuvikConfig, *, max_tokens: int, max_seqs: int, max_blocks: int, block_size: int, max_model_len: int,
                 device: torch.device, tp_rank: int = 0, tp_size: int = 1, tp_group=None, max_logit_rows: int | None = None,
                 max_split_tokens: int = 256, force_collectives: bool = False, taps=None, dtype: str = "bfloat16"):
        assert tp_size == 1 and taps is None, "Dosuvik models are single-rank and have no activation taps"
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
        self.scalar_attention = False                 # tests / probes: the scalar forms of the attentions also where the MFMA forms fit
        self.tap_residuals: list | None = None         # tests: receives a copy of the residual rows after every layer (eager only)

        def z(*shape, dtype=torch.float32):
            return torch.zeros(*shape, dtype=dtype, device=device)

        T, W, el = max_tokens, self.W, self.elem
        mixers = [l.mixer for l in cfg.layers]
        ret = [m for m in mixers if m.kind == "retention"]
        lat = [m for m in mixers if m.kind == "latent_attention"]
        att = [m for m in mixers if m.kind == "attention"]
        dense = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "dense"]
        moes = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "moe"]
        self.x = z(T, W)
        self.hist = z(len(cfg.layers) + 1, T, W)           # level 0: the embedding output; level i + 1: the result of layer i
        self.hn = z(T, W, dtype=el)
        self.y = z(T, W)
        self.proj = z(T * max(self._nproj(m) for m in mixers))
        self.att = z(T * max(m.heads * m.vdim for m in mixers), dtype=el)
        if ret:
            self.o = z(T * max(m.heads * m.vdim for m in ret))
            self.ones = torch.ones(max(m.heads * m.vdim for m in ret), dtype=el, device=device)
        if lat or att:
            self.q = z(T * max([m.heads * (m.dim + m.rot_dim) for m in lat] + [m.heads * m.dim for m in att]), dtype=el)
        if lat:
            self.q_abs = z(T * max(m.heads * m.kv_rank for m in lat))           # queries in the latent space: fp32, or (its first half)
            self.q_lat = self.q_abs.view(el)                                     # element-type rows where the MFMA attention takes them
            self.mfma = {i: H.latent_attn_mfma_ok(l.mixer.kv_rank, l.mixer.rot_dim, self.f32) for i, l in enumerate(cfg.layers)
                         if l.mixer.kind == "latent_attention"}
            self.olat = z(T * max(m.heads * m.kv_rank for m in lat), dtype=el)
            self.uvo = z(T * max(m.heads * m.vdim for m in lat))
            self.att_ws = z(1024 * (max(m.kv_rank for m in lat) * 16 + 32)) if any(self.mfma.values()) else None
        if moes:
            top = max(m.top for m in moes)
            E = max(m.experts for m in moes)
            self.r_z = z(T * E)
            self.r_idx = z(T * top, dtype=torch.int32)
            self.r_wt = z(T * top)
            self.r_off = z(E + 1, dtype=torch.int32)
            self.r_perm = z(T * top, dtype=torch.int32)
            self.r_inv = z(T * top, dtype=torch.int32)
            self.ydn = z(T * top * W)
        ffs = [m.ff for m in dense] + [m.top * m.ff for m in moes]
        if ffs:
            self.ab = z(T * 2 * max(ffs)) if self.f32 else None       # fp32 [gate | up] rows (bf16: the GEMM epilogue applies the GLU)
            self.act = z(T * max(ffs), dtype=el)
        R = self.max_logit_rows
        self.lastn = z(R, W, dtype=el)
        self.logits32 = z(R, self.V)
        self.logits = z(R, self.Vp, dtype=BF16)

    @staticmethod
    def _nproj(m) -> int:
        if m.kind == "retention":
            return 2 * m.heads * m.dim + 2 * m.heads * m.vdim
        if m.kind == "latent_attention":
            return m.heads * (m.dim + m.rot_dim) + m.kv_rank + m.rot_dim + m.heads * m.vdim
        return (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim

    # ---------------------------------------------------------------------------------------------
    def load_weights(self, weight_iter) -> None:
        """Consumes (name, tensor) pairs under the checkpoint's names.  Matrices that read the same rows are stacked ([q | k | v | g],
        [q | dkv | g], [q | k | v], [gate | up]); the layer norms become fp32 vectors 1 + w (the stored weights lie around zero and their
        sum with one does not fit the element type); W_uk per head transposed; rotated parts stored in the interleaved layout are
        permuted into the halves layout; what enters a softmax, a recurrence or the router's choice directly stays fp32."""
        raw = {n: t.to(self.device) for n, t in weight_iter}
        cv = lambda t: t.to(self.elem).contiguous()
        f32 = lambda t: t.float().reshape(-1).contiguous()
        dev_f32 = lambda vals: torch.tensor(vals, dtype=torch.float64).to(torch.float32).to(self.device)
        one_plus = lambda n: (1.0 + raw[n].float()).contiguous()
        w = self.w = {}

        def pair(gate, up):
            # bf16: rows interleaved (gate_0, up_0, gate_1, ...) for the GEMM's paired epilogue; fp32: [gate | up], a GLU launch follows
            return torch.stack([gate, up], dim=1).reshape(-1, gate.shape[1]) if not self.f32 else torch.cat([gate, up], dim=0)

        w["embed"], w["head"] = cv(raw["embed"]), cv(raw["head"])
        w["final.norm"] = one_plus("final.norm")
        for i, lc in enumerate(self.cfg.layers):
            p, m, ml = f"l{i}.", lc.mixer, lc.mlp
            w[p + "norm1"] = one_plus(p + "norm1")
            w[p + "dwa"] = f32(raw[p + "dwa"])
            if m.kind == "retention":
                assert m.rope.layout == "halves"
                w[p + "mix.in"] = cv(torch.cat([raw[p + "mix.q"], raw[p + "mix.k"], raw[p + "mix.v"], raw[p + "mix.g"]], dim=0))
                w[p + "mix.decay"] = dev_f32(m.decay)
                w[p + "mix.freqs"] = dev_f32(m.rope.frequencies() or [0.0])
            elif m.kind == "latent_attention":
                Hh, D, R, Cr = m.heads, m.dim, m.rot_dim, m.kv_rank
                order = torch.tensor(m.rope.to_halves(R), device=self.device)
                q = raw[p + "mix.q"].view(Hh, D + R, -1)
                q = torch.cat([q[:, :D], q[:, D:][:, order]], dim=1).reshape(Hh * (D + R), -1)
                dkv = torch.cat([raw[p + "mix.dkv"][:Cr], raw[p + "mix.dkv"][Cr:][order]], dim=0)
                w[p + "mix.in"] = cv(torch.cat([q, dkv, raw[p + "mix.g"]], dim=0))
                w[p + "mix.ukt"] = cv(raw[p + "mix.uk"].view(Hh, D, Cr).transpose(1, 2))
                w[p + "mix.dkv.norm"], w[p + "mix.uv"] = cv(raw[p + "mix.dkv.norm"]), cv(raw[p + "mix.uv"])
                w[p + "mix.freqs"] = dev_f32(m.rope.frequencies() or [0.0])
            else:
                assert m.rope.layout == "halves"
                w[p + "mix.in"] = cv(torch.cat([raw[p + "mix.q"], raw[p + "mix.k"], raw[p + "mix.v"]], dim=0))
                w[p + "mix.q.norm"], w[p + "mix.k.norm"] = cv(raw[p + "mix.q.norm"]), cv(raw[p + "mix.k.norm"])
                w[p + "mix.sink"] = f32(raw[p + "mix.sink"])
                w[p + "mix.freqs"] = dev_f32(m.rope.frequencies() or [0.0])
                if m.rotate_values:
                    w[p + "mix.vfreqs"] = dev_f32(m.rope.frequencies(m.vdim))
            w[p + "mix.o"] = cv(raw[p + "mix.o"])
            if ml is None:
                continue
            w[p + "norm2"] = one_plus(p + "norm2")
            if ml.kind == "dense":
                w[p + "mlp.gu"] = cv(pair(raw[p + "mlp.gate"], raw[p + "mlp.up"]))
                w[p + "mlp.down"] = cv(raw[p + "mlp.down"])
            else:
                w[p + "mlp.gu"] = cv(torch.stack([pair(raw[p + f"mlp.e{e}.gate"], raw[p + f"mlp.e{e}.up"]) for e in range(ml.experts)]))
                w[p + "mlp.down"] = cv(torch.stack([raw[p + f"mlp.e{e}.down"] for e in range(ml.experts)]))
                w[p + "mlp.router"] = cv(raw[p + "mlp.router"])
                w[p + "mlp.correction"] = f32(raw[p + "mlp.correction"])
        torch.cuda.synchronize(self.device)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.w.values())

    def active_weight_bytes(self, T: int = 1) -> int:
        """HBM bytes of weights one forward of T tokens must stream at least: every dense matrix once per layer, of the experts
        min(E, T * top), the LM head once, one embedding row per token."""
        per = {n: t.numel() * t.element_size() for n, t in self.w.items()}
        total = per["head"] + per["final.norm"]
        for i, lc in enumerate(self.cfg.layers):
            p, ml = f"l{i}.", lc.mlp
            total += sum(v for n, v in per.items() if n.startswith(p + "mix.") or n.startswith(p + "norm") or n == p + "dwa")
            if ml is None:
                continue
            if ml.kind == "dense":
                total += per[p + "mlp.gu"] + per[p + "mlp.down"]
            else:
                frac = min(ml.experts, T * ml.top) / ml.experts
                total += int((per[p + "mlp.gu"] + per[p + "mlp.down"]) * frac) + per[p + "mlp.router"] + per[p + "mlp.correction"]
        return total

    def kv_block_bytes(self) -> int:
        es = 4 if self.f32 else 2
        n = 0
        for l in self.cfg.layers:
            m = l.mixer
            if m.kind == "attention":
                n += m.kv_heads * (m.dim + m.vdim) * self.block_size * es
            elif m.kind == "latent_attention":
                n += (m.kv_rank + m.rot_dim) * self.block_size * es
        return max(n, 1)

    def state_bytes(self) -> int:
        """Bytes of recurrent state one live sequence holds (all layers)."""
        return sum(l.mixer.heads * l.mixer.dim * l.mixer.vdim * 4 for l in self.cfg.layers if l.mixer.kind == "retention")

    def alloc_kv(self, num_blocks: int) -> None:
        """Per layer: attention -> K pages [blocks][G][block][dim] and V pages transposed [blocks][G][vdim][block] (values rotated by
        their position); latent attention -> cache rows [blocks * block][kv_rank + rot_dim] for all heads together; retention -> state
        [slots][H][dim][vdim] fp32.  A slot is not cleared when it is handed out: a forward whose rows start at position 0 starts from
        zero by itself."""
        self.num_blocks = num_blocks
        self.kv, self.state = [], []
        dev, bs, S = self.device, self.block_size, self.state_slots
        for l in self.cfg.layers:
            m = l.mixer
            if m.kind == "attention":
                self.kv.append((torch.zeros(num_blocks, m.kv_heads, bs, m.dim, dtype=self.elem, device=dev),
                                torch.zeros(num_blocks, m.kv_heads, m.vdim, bs, dtype=self.elem, device=dev)))
                self.state.append(None)
            elif m.kind == "latent_attention":
                self.kv.append(torch.zeros(num_blocks * bs, m.kv_rank + m.rot_dim, dtype=self.elem, device=dev))
                self.state.append(None)
            else:
                self.kv.append(None)
                self.state.append(torch.zeros(S, m.heads, m.dim, m.vdim, dtype=torch.float32, device=dev))

    # ---------------------------------------------------------------------------------------------
    def launch_mixer(self, li: int, T: int, positions, meta: AttnMeta) -> None:
        """hn (the residual rows in the element type) -> y (fp32 mixer output rows)."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        m, p = cfg.layers[li].mixer, f"l{li}.mix."
        NP = self._nproj(m)
        seqs = dict(cu_q=meta.cu_q) if meta.cu_q is not None else dict(q_per_seq=meta.q_per_seq)
        H.gemm_rows(self.hn, w[p + "in"], self.proj, T, NP, W, f)
        if m.kind == "retention":
            assert meta.state_slots is not None, "a model with recurrent layers needs the sequences' state slots"
            Hh, D, Dv = m.heads, m.dim, m.vdim
            H.rope_rows(self.proj, NP, positions, w[p + "freqs"], m.rope.dims, Hh, D, T, 0, 1.0, Hh * D, float(D) ** -0.5)
            H.lightning_scan(self.proj, NP, 0, Hh * D, 2 * Hh * D, w[p + "decay"], positions, meta.state_slots, self.state[li], self.o,
                             meta.B, Hh, D, Dv, act=H.SCAN_RAW, **seqs)
            H.group_gate_norm(self.o, self.proj[2 * Hh * D + Hh * Dv:], NP, self.ones, cfg.rms_norm_eps, self.att, T, Hh * Dv, Hh, False, f)
        elif m.kind == "latent_attention":
            Hh, D, R, Cr, Dv = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
            NQ = Hh * (D + R)
            H.latent_store(self.proj, NP, NQ, Cr, R, Hh, None, w[p + "dkv.norm"], cfg.rms_norm_eps, positions, w[p + "freqs"], 1.0,
                           m.rope.dims, meta.slot_mapping, self.q, self.kv[li], None, T, f)
            mf = self.mfma[li] and not self.scalar_attention
            H.gemm_rows_batched(self.q, w[p + "ukt"], self.q_lat if mf else self.q_abs, T, Cr, D, Hh, NQ, D + R, Hh * Cr, Cr, f,
                                H.GR_ELEM if mf else H.GR_F32)
            H.latent_attn(self.q_lat if mf else self.q_abs, self.q, self.kv[li], None, meta.block_tables, self.max_blocks, positions,
                          meta.B, T, Hh, D, R, Cr, self.block_size, m.window, m.scale, w[p + "freqs"], 1.0, m.rope.dims, self.olat, f,
                          q_abs_elem=mf, workspace=self.att_ws, **seqs)
            H.gemm_rows_batched(self.olat, w[p + "uv"], self.uvo, T, Dv, Cr, Hh, Hh * Cr, Cr, Hh * Dv, Dv, f, H.GR_F32)
            H.gate_rows(self.uvo, Hh * Dv, self.proj[NQ + Cr + R:], NP, self.att, T, Hh * Dv, f)
        else:
            kc, vc = self.kv[li]
            vf = w.get(p + "vfreqs")
            H.winattn_store_rope(self.proj, NP, w[p + "q.norm"], w[p + "k.norm"], cfg.rms_norm_eps, positions, w[p + "freqs"], m.rope.dims,
                                 vf, meta.slot_mapping, self.q, kc, vc, T, m.heads, m.kv_heads, m.dim, m.vdim, self.block_size, f)
            H.winattn_paged(self.q, kc, vc, None, w[p + "sink"], meta.block_tables, self.max_blocks, positions, meta.B, T, m.heads,
                            m.kv_heads, m.dim, m.vdim, self.block_size, m.window, m.scale, 0.0, self.att, f,
                            max_q=0 if self.scalar_attention else meta.max_q, out_freqs=vf, **seqs)
        H.gemm_rows(self.att, w[p + "o"], self.y, T, W, m.heads * m.vdim, f)

    def launch_mlp(self, li: int, T: int) -> dict:
        """hn -> the feed-forward's rows; returns the keyword arguments that hand them to postnorm_tail."""
        w, f, W = self.w, self.f32, self.W
        ml, p = self.cfg.layers[li].mlp, f"l{li}.mlp."
        if ml.kind == "dense":
            if f:
                H.gemm_rows(self.hn, w[p + "gu"], self.ab, T, 2 * ml.ff, W, True)
                H.glu_clamp_rows(self.ab, self.act, T, ml.ff, ml.limit, self.cfg.SWISH_ALPHA, True)
            else:
                H.gemm_rows_glu_clamp(self.hn, w[p + "gu"], self.act, T, 2 * ml.ff, W, ml.limit, self.cfg.SWISH_ALPHA)
            H.gemm_rows(self.act, w[p + "down"], self.y, T, W, ml.ff, f)
            return dict(y=self.y)
        E, top = ml.experts, ml.top
        H.gemm_rows(self.hn, w[p + "router"], self.r_z, T, E, W, f)
        H.moe_route_sigmoid_grouped(self.r_z, E, w[p + "correction"], self.r_idx, self.r_wt, T, E, top, ml.groups, ml.keep, 2)
        H.moe_plan(self.r_idx, T, top, E, self.r_off, self.r_perm, self.r_inv)
        if f:
            H.gemm_rows_grouped(self.hn, w[p + "gu"], self.ab, self.r_off, E, T * top, 2 * ml.ff, W, f, H.GR_F32, row_idx=self.r_perm,
                                idx_div=top)
            H.glu_rows(self.ab, self.act, T * top, ml.ff, H.GLU_SILU, f)
        else:
            H.gemm_rows_grouped(self.hn, w[p + "gu"], self.act, self.r_off, E, T * top, 2 * ml.ff, W, f, H.GR_GLU_SILU, row_idx=self.r_perm,
                                idx_div=top)
        H.gemm_rows_grouped(self.act, w[p + "down"], self.ydn, self.r_off, E, T * top, W, ml.ff, f, H.GR_F32)
        return dict(ydn=self.ydn, inv=self.r_inv, weights=self.r_wt, top=top)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, T: int, meta: AttnMeta) -> None:
        """Runs every layer over the T token rows; leaves the fp32 residual rows (after the last depth average) in self.x."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        eps = cfg.rms_norm_eps
        assert T <= self.max_tokens and meta.mode == H.MODE_CAUSAL and (meta.cu_q is not None or meta.q_per_seq > 0)
        stride = self.hist.shape[1] * W
        H.embed_hist(input_ids, w["embed"], self.x, T, W, f, hist0=self.hist, rows_out=self.hn)
        for li, lc in enumerate(cfg.layers):
            p = f"l{li}."
            depth = dict(hist=self.hist, hist_stride=stride, hist_levels=li + 2, coef=w[p + "dwa"])
            self.launch_mixer(li, T, positions, meta)
            H.postnorm_tail(self.x, w[p + "norm1"], eps, T, W, f, y=self.y, next_out=self.hn, **({} if lc.mlp is not None else depth))
            if lc.mlp is not None:
                ff = self.launch_mlp(li, T)
                H.postnorm_tail(self.x, w[p + "norm2"], eps, T, W, f, next_out=self.hn, **ff, **depth)
            if self.tap_residuals is not None:
                self.tap_residuals.append(self.x[:T].clone())

    def compute_logits(self, T: int, gather: torch.Tensor | None = None, rows: int | None = None) -> int:
        """Final norm (optionally of the `gather` rows only) and the LM head: fp32 logits in logits32[:n], their bf16 rounding (row
        stride Vp, padding -inf) in logits[:n] for the sampling kernels.  Returns n."""
        n = T if gather is None else rows
        assert n <= self.max_logit_rows
        H.rmsnorm_w32_rows(self.x, self.w["final.norm"], self.cfg.rms_norm_eps, self.lastn, n, self.W, self.f32, gather=gather)
        H.gemm_rows(self.lastn, self.w["head"], self.logits32, n, self.V, self.W, self.f32)
        H.rows_f32_to_bf16(self.logits32, self.logits, n, self.V, self.V, self.Vp)
        return n
