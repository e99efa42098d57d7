"""Architecture description shared by the HIP decoder and the test oracle.

The reference reads these fields from a HF ``config.json`` through ``AutoConfig`` (ssd/config.py:56-61) and
consumes them in ``LlamaAttention`` / ``Qwen3Attention`` (ssd/models/llama3.py:15-87, ssd/models/qwen3.py).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict, field


@dataclass
class ModelConfig:
    family: str                 # "llama" | "qwen3" | "eagle3" (the one-layer EAGLE-3 draft, eagle3_draft_llama3.py)
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    qk_norm: bool = False       # Qwen3: per-head RMSNorm on q and k before RoPE (qwen3.py:96-104)
    attention_bias: bool = False
    # EAGLE-3 draft only (ssd/models/eagle3_draft_llama3.py:209-262): the LM head covers draft_vocab_size tokens that d2t maps
    # into the target vocabulary (vocab_size), and fc projects eagle_taps concatenated target activations of width
    # d_model_target each
    draft_vocab_size: int = 0
    d_model_target: int = 0
    eagle_taps: int = 3

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def to_dict(self) -> dict:
        return asdict(self)

    @staticmethod
    def from_hf(hf) -> "ModelConfig":
        """From a transformers config object (or anything with the same attributes)."""
        mt = getattr(hf, "model_type", "llama")
        family = "qwen3" if "qwen" in mt else "llama"
        if getattr(hf, "draft_vocab_size", None) and hf.num_hidden_layers == 1:
            family = "eagle3"       # EAGLE-3 checkpoints: a Llama config.json with one layer + draft_vocab_size
        nh = hf.num_attention_heads
        hd = getattr(hf, "head_dim", None) or hf.hidden_size // nh
        # transformers >= 5 moved rope_theta into rope_parameters; the reference's getattr(config,
        # "rope_theta", default) (llama3.py:163, qwen3.py:173) would silently fall back, so read both.
        theta = getattr(hf, "rope_theta", None)
        if theta is None:
            rp = getattr(hf, "rope_parameters", None) or {}
            theta = rp.get("rope_theta") if isinstance(rp, dict) else None
        if theta is None:
            theta = 1000000.0 if family == "qwen3" else 500000.0
        return ModelConfig(
            family=family,
            hidden_size=hf.hidden_size,
            num_layers=hf.num_hidden_layers,
            num_heads=nh,
            num_kv_heads=getattr(hf, "num_key_value_heads", nh),
            head_dim=hd,
            intermediate_size=hf.intermediate_size,
            vocab_size=hf.vocab_size,
            rms_norm_eps=getattr(hf, "rms_norm_eps", 1e-6),
            rope_theta=float(theta),
            max_position_embeddings=getattr(hf, "max_position_embeddings", 8192),
            tie_word_embeddings=bool(getattr(hf, "tie_word_embeddings", False)),
            qk_norm=(family == "qwen3"),
            attention_bias=bool(getattr(hf, "attention_bias", False)),
            draft_vocab_size=int(getattr(hf, "draft_vocab_size", 0) or 0),
        )


# Public shapes of the models BASELINE.json names (no weights exist offline).
PRESETS = {
    "llama-3.2-1b": ModelConfig("llama", 2048, 16, 32, 8, 64, 8192, 128256, 1e-5, 5e5, 131072, True),
    "llama-3.1-8b": ModelConfig("llama", 4096, 32, 32, 8, 128, 14336, 128256, 1e-5, 5e5, 131072, False),
    "llama-3.1-70b": ModelConfig("llama", 8192, 80, 64, 8, 128, 28672, 128256, 1e-5, 5e5, 131072, False),
    "qwen3-32b": ModelConfig("qwen3", 5120, 64, 64, 8, 128, 25600, 151936, 1e-6, 1e6, 40960, False, True),
    "qwen3-0.6b": ModelConfig("qwen3", 1024, 28, 16, 8, 128, 3072, 151936, 1e-6, 1e6, 40960, True, True),
    # the other sizes the reference's bench.py --size accepts (bench_helpers.py:96-120), public config.json shapes
    "llama-3.2-3b": ModelConfig("llama", 3072, 28, 24, 8, 128, 8192, 128256, 1e-5, 5e5, 131072, True),
    "qwen3-1.7b": ModelConfig("qwen3", 2048, 28, 16, 8, 128, 6144, 151936, 1e-6, 1e6, 40960, True, True),
    "qwen3-4b": ModelConfig("qwen3", 2560, 36, 32, 8, 128, 9728, 151936, 1e-6, 1e6, 40960, True, True),
    "qwen3-8b": ModelConfig("qwen3", 4096, 36, 32, 8, 128, 12288, 151936, 1e-6, 1e6, 40960, False, True),
    "qwen3-14b": ModelConfig("qwen3", 5120, 40, 40, 8, 128, 17408, 151936, 1e-6, 1e6, 40960, False, True),
    # EAGLE-3 drafts the reference's bench.py --eagle selects (bench_helpers.py:50-63, bench_paths.py:33-44); public config.json shapes
    "eagle3-llama-3.1-8b": ModelConfig("eagle3", 4096, 1, 32, 8, 128, 14336, 128256, 1e-5, 5e5, 131072, False,
                                       draft_vocab_size=32000, d_model_target=4096),
    "eagle3-llama-3.3-70b": ModelConfig("eagle3", 6144, 1, 48, 8, 128, 16384, 128256, 1e-5, 5e5, 131072, False,
                                        draft_vocab_size=32000, d_model_target=8192),
}


# --------------------------------------------------------------------------------------------------
# Fatulix: a decoder whose config.json lists its layers one by one (own keys, not a transformers config)
# --------------------------------------------------------------------------------------------------
@dataclass
class RoutedMLP:
    """Mixture-of-experts feed-forward: `top` of `experts` two-matrix experts (relu^2) per token, plus an optional shared expert."""
    experts: int
    top: int
    ff: int
    shared_ff: int = 0          # 0: no shared expert


@dataclass
class DiffAttention:
    """Differential attention: two softmax maps per query head over shared values, per-(head, map) q / k RMS norm, output gate."""
    heads: int
    kv_heads: int
    dim: int                    # query / key size per head and map
    vdim: int                   # value size per head
    diff: float                 # the constant of lambda and of the (1 - diff) output scale
    scale: float                # score scale


@dataclass
class FatulixLayer:
    mixer: DiffAttention
    mlp: RoutedMLP | None


@dataclass
class FatulixConfig:
    """config.json keys: architecture, vocab, width, norm.eps, layers[{type, mixer{heads, kv_heads, dim, vdim, diff, scale},
    mlp{kind, expert{ff}, router{experts, top}, shared{ff} | null} | null}], loop{start, stop, times}."""
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    family: str = "fatulix"
    max_position_embeddings: int = 1 << 20      # no positional limit: positions do not enter the scores
    tie_word_embeddings: bool = False

    def runs(self) -> list[tuple[int, int]]:
        """(layer, pass) of every layer run in execution order.  Layers [loop_start, loop_stop) run loop_times passes with the same
        weights; every run has KV pages of its own."""
        a, b = self.loop_start, self.loop_stop
        span = [(i, ps) for ps in range(self.loop_times) for i in range(a, b)] if b > a else []
        return [(i, 0) for i in range(a)] + span + [(i, 0) for i in range(max(a, b), len(self.layers))]

    @property
    def num_layers(self) -> int:            # KV-cache layers = layer runs
        return len(self.runs())

    def to_dict(self) -> dict:
        return asdict(self)

    @staticmethod
    def from_json(cfg: dict) -> "FatulixConfig":
        layers = []
        for lc in cfg["layers"]:
            if lc["type"] != "attention":
                raise ValueError(f"Fatulix: unknown layer type {lc['type']!r}")
            m = lc["mixer"]
            mixer = DiffAttention(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["diff"]), float(m["scale"]))
            if mixer.heads % mixer.kv_heads:
                raise ValueError("Fatulix: heads must be a multiple of kv_heads")
            ml = lc.get("mlp")
            mlp = None
            if ml is not None:
                if ml.get("kind", "moe") != "moe":
                    raise ValueError(f"Fatulix: unknown feed-forward kind {ml.get('kind')!r}")
                sh = ml.get("shared")
                mlp = RoutedMLP(int(ml["router"]["experts"]), int(ml["router"]["top"]), int(ml["expert"]["ff"]), int(sh["ff"]) if sh else 0)
            layers.append(FatulixLayer(mixer, mlp))
        loop = cfg.get("loop") or {}
        out = FatulixConfig(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, int(loop.get("start", 0)),
                            int(loop.get("stop", 0)), int(loop.get("times", 1)))
        if not (0 <= out.loop_start <= max(out.loop_start, out.loop_stop) <= len(layers)) or out.loop_times < 1:
            raise ValueError("Fatulix: loop out of range")
        return out


# --------------------------------------------------------------------------------------------------
# Zerusun: parallel layers with Dynamic-Tanh norms; mixers are latent attention (sliding window) or linear attention with decay
# --------------------------------------------------------------------------------------------------
@dataclass
class RopeSpec:
    """Rotary positions on the first `dims` entries of a rotated part ("rotate half" pairing: i with i + dims / 2), frequencies
    base^(-2i/dims); scaling (optional) = YaRN: {factor, original, fast, slow}."""
    dims: int
    base: float
    scaling: dict | None = None

    def frequencies(self) -> tuple[list[float], float]:
        """(per-pair angular frequencies, the factor cos and sin carry).  YaRN keeps the pairs that turn more than `fast` times over
        `original` positions, divides the frequency of those that turn fewer than `slow` times by `factor`, and blends linearly
        between the two corner pairs; cos and sin are scaled by 0.1 ln(factor) + 1."""
        import math
        half = self.dims // 2
        f = [self.base ** (-2.0 * i / self.dims) for i in range(half)]
        sc = self.scaling
        if not sc:
            return f, 1.0
        factor, orig = float(sc["factor"]), float(sc["original"])
        corner = lambda turns: self.dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))
        lo = max(math.floor(corner(float(sc["fast"]))), 0)
        hi = min(math.ceil(corner(float(sc["slow"]))), self.dims - 1)
        ramp = [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)]
        return [fi / factor * r + fi * (1.0 - r) for fi, r in zip(f, ramp)], 0.1 * math.log(factor) + 1.0


@dataclass
class LatentAttention:
    """Attention whose queries and keys / values pass through low-rank latents; per head `dim` unrotated + `rot_dim` rotated query / key
    entries (the rotated key part is shared by all heads), value size `vdim`; only the kv latent and the rotated key part are cached.
    window: a token sees itself and the window - 1 tokens before it (0: every earlier token).  Per-head sigmoid output gate."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int
    rope: RopeSpec
    kind: str = "latent_attention"


@dataclass
class LightningAttention:
    """Linear attention with a per-head scalar decay over a recurrent [dim][vdim] state; silu on q, k, v; RMS norm over the concatenated
    heads and an elementwise sigmoid gate before the output projection."""
    heads: int
    dim: int
    vdim: int
    decay: list = field(default_factory=list)
    kind: str = "lightning"


@dataclass
class GluMLP:
    """Dense gated feed-forward W_down(act(W_gate h) * W_up h), act = tanh-form gelu."""
    ff: int
    kind: str = "dense"


@dataclass
class GroupRoutedMLP:
    """Mixture of gated (silu) experts: softmax over all experts, `groups` contiguous groups of which the best `keep` stay eligible,
    the `top` largest scores renormalised and multiplied by `scale`; optional shared expert with a per-token sigmoid gate."""
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    kind: str = "moe"


@dataclass
class ZerusunLayer:
    mixer: object               # LatentAttention | LightningAttention
    mlp: object                 # GluMLP | GroupRoutedMLP | None


@dataclass
class ZerusunConfig:
    """config.json keys: architecture, vocab, width, norm.eps, layers[{type, mixer{...}, mlp{kind, ...} | null}], loop{start, stop, times}.
    Layers [start, stop) run `times` passes with the same weights (each pass with cache pages / state of its own); before the first layer
    of EVERY pass x <- W_in [x; x0] + step[pass], x0 = the embedding output."""
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    family: str = "zerusun"
    max_position_embeddings: int = 1 << 20
    tie_word_embeddings: bool = True

    def runs(self) -> list[tuple[int, int]]:
        """(layer, pass) of every layer run in execution order."""
        a, b = self.loop_start, self.loop_stop
        if b <= a:
            return [(i, 0) for i in range(len(self.layers))]
        span = [(i, ps) for ps in range(self.loop_times) for i in range(a, b)]
        return [(i, 0) for i in range(a)] + span + [(i, 0) for i in range(b, len(self.layers))]

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    @property
    def num_layers(self) -> int:
        return len(self.runs())

    @property
    def recurrent(self) -> bool:
        """True when some layer keeps a per-sequence state that is not a function of cached pages: no prefix caching, and every live
        sequence holds a state slot."""
        return any(l.mixer.kind == "lightning" for l in self.layers)

    def to_dict(self) -> dict:
        return asdict(self)

    @staticmethod
    def from_json(cfg: dict) -> "ZerusunConfig":
        layers = []
        for lc in cfg["layers"]:
            m, kind = lc["mixer"], lc["type"]
            if kind == "latent_attention":
                r = m["rot"]
                rope = RopeSpec(int(r["dims"]), float(r["base"]), dict(r["scaling"]) if r.get("scaling") else None)
                mask = m.get("mask") or {}
                mixer = LatentAttention(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["q_rank"]),
                                        int(m["kv_rank"]), float(m["scale"]), int(mask.get("size") or 0), rope)
                if rope.dims % 2 or rope.dims > mixer.rot_dim:
                    raise ValueError("Zerusun: rot.dims must be even and at most rot_dim")
            elif kind == "lightning":
                mixer = LightningAttention(int(m["heads"]), int(m["dim"]), int(m["vdim"]), [float(d) for d in m["decay"]])
                if len(mixer.decay) != mixer.heads:
                    raise ValueError("Zerusun: one decay per head")
            else:
                raise ValueError(f"Zerusun: unknown layer type {kind!r}")
            ml = lc.get("mlp")
            mlp = None
            if ml is not None:
                if ml["kind"] == "dense":
                    mlp = GluMLP(int(ml["ff"]))
                elif ml["kind"] == "moe":
                    r, g, sh = ml["router"], ml["router"].get("groups") or {}, ml.get("shared")
                    mlp = GroupRoutedMLP(int(r["experts"]), int(r["top"]), int(ml["expert"]["ff"]), int(g.get("count", 1)),
                                         int(g.get("keep", 1)), float(r.get("scale", 1.0)), int(sh["ff"]) if sh else 0)
                    if mlp.experts % mlp.groups or not (1 <= mlp.keep <= mlp.groups) or mlp.top > mlp.experts // mlp.groups * mlp.keep:
                        raise ValueError("Zerusun: router groups do not fit the experts")
                else:
                    raise ValueError(f"Zerusun: unknown feed-forward kind {ml['kind']!r}")
            layers.append(ZerusunLayer(mixer, mlp))
        loop = cfg.get("loop") or {}
        out = ZerusunConfig(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, int(loop.get("start", 0)),
                            int(loop.get("stop", 0)), int(loop.get("times", 1)))
        if not (0 <= out.loop_start and out.loop_stop <= len(layers)) or out.loop_times < 1:
            raise ValueError("Zerusun: loop out of range")
        return out


# --------------------------------------------------------------------------------------------------
# Fomunex: pre-norm layers (one-number RMS norms) over an fp32 residual with a learned position vector; mixers are windowed attention
# with a sink, RWKV-style time mixing, or a Mamba-2 state space; feed-forwards are PolyNorm dense or sigmoid-routed clamped GLUs
# --------------------------------------------------------------------------------------------------
@dataclass
class WindowAttention:
    """Grouped-query attention without rotation: q and k divided by their root mean square per head, scores scale * <q, k> capped by
    softcap * tanh(. / softcap) (0: no cap), minus slope_h * distance with slope_h = 2^(-8 (h + 1) / heads), a sliding window (a token
    sees itself and the window - 1 tokens before it; 0: every earlier token) and a learned per-head sink in the softmax denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    window: int = 0
    kind: str = "attention"

    def slopes(self) -> list[float]:
        return [2.0 ** (-8.0 * (h + 1) / self.heads) for h in range(self.heads)]


@dataclass
class WkvMixer:
    """RWKV-style time mixing: r, k, v, gate and the decay each read their own interpolation between the token's row and the previous
    token's; per head a [dim][dim] fp32 state with a per-channel data-dependent decay exp(-exp(W_w2 tanh(W_w1 mix) + w0)) and a bonus
    for the current token; per-head unit-RMS output, silu gate.  decay_rank: the inner size of the decay's two matrices (a tensor's
    shape, not a config.json key: 0 until a checkpoint's header or the caller gives it)."""
    heads: int
    dim: int
    decay_rank: int = 0
    kind: str = "wkv"


@dataclass
class Mamba2Mixer:
    """Mamba-2 state space: inner = heads * vdim channels, a [state][vdim] fp32 state per head with one decay per head and token,
    B / C shared by the heads of one of `groups` groups, a causal convolution of `conv` taps over [x | B | C], the silu gate applied
    BEFORE an RMS norm in `norm_groups` equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1
    kind: str = "mamba2"

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class PolyNormMLP:
    """Dense feed-forward W_down act(W_up h) with act(z) = a rms(z) + b rms(z^2) + c rms(z^3) + e over a token's ff values."""
    ff: int
    kind: str = "dense"


@dataclass
class SigmoidRoutedMLP:
    """Mixture of experts with a sigmoid router: the `top` largest scores, unrenormalised, each multiplying its expert's INPUT; experts
    g = min(W_gate h, limit), u = clamp(W_up h, +-limit), W_down (g sigmoid(1.702 g) (u + 1))."""
    experts: int
    top: int
    ff: int
    limit: float
    kind: str = "moe"


@dataclass
class FomunexLayer:
    mixer: object               # WindowAttention | WkvMixer | Mamba2Mixer
    mlp: object                 # PolyNormMLP | SigmoidRoutedMLP | None
    weights_of: int             # the layer whose tensors this layer uses (itself unless config.json says otherwise); cache / state are its own


@dataclass
class FomunexConfig:
    """config.json keys: architecture, vocab, width, max_positions, norm.eps, logit_scale, logit_softcap, layers[{type, mixer{...},
    mlp{kind, ...} | null, weights_of?}]."""
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    layers: list = field(default_factory=list)
    max_position_embeddings: int = 2048
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    family: str = "fomunex"
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def recurrent(self) -> bool:
        """True when some layer keeps a per-sequence state that is not a function of cached pages."""
        return any(l.mixer.kind in ("wkv", "mamba2") for l in self.layers)

    def to_dict(self) -> dict:
        return asdict(self)

    def complete_from_checkpoint(self, model_dir: str) -> None:
        """Sizes that only a tensor's shape gives (the decay rank of time-mixing layers): read from the safetensors headers."""
        need = [i for i, l in enumerate(self.layers) if l.mixer.kind == "wkv" and not l.mixer.decay_rank]
        if not need and self.max_position_embeddings > 0:
            return
        import glob
        import struct
        shapes = {}
        for f in sorted(glob.glob(os.path.join(model_dir, "*.safetensors"))):
            with open(f, "rb") as fh:
                n = struct.unpack("<Q", fh.read(8))[0]
                shapes.update({k: v.get("shape") for k, v in json.loads(fh.read(n)).items() if k != "__metadata__"})
        for i in need:
            name = f"l{self.layers[i].weights_of}.mix.w1"
            if name not in shapes:
                raise ValueError(f"Fomunex: {name} not found under {model_dir}")
            self.layers[i].mixer.decay_rank = int(shapes[name][0])
        if self.max_position_embeddings <= 0:          # config.json without max_positions: the position table's rows
            if "pos" not in shapes:
                raise ValueError(f"Fomunex: neither max_positions nor a position table under {model_dir}")
            self.max_position_embeddings = int(shapes["pos"][0])

    @staticmethod
    def from_json(cfg: dict) -> "FomunexConfig":
        layers = []
        for i, lc in enumerate(cfg["layers"]):
            if "weights_of" in lc and 0 <= int(lc["weights_of"]) < len(cfg["layers"]):
                lc = {**cfg["layers"][int(lc["weights_of"])], **lc}          # what a borrowing layer leaves out equals its source's
            m, kind = lc["mixer"], lc["type"]
            if kind == "attention":
                mask = m.get("mask") or {}
                mixer = WindowAttention(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                        float(m["scale"]) if m.get("scale") is not None else int(m["dim"]) ** -0.5,
                                        float(m.get("softcap") or 0.0), int(mask.get("size") or 0))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError("Fomunex: heads must be a multiple of kv_heads")
            elif kind == "wkv":
                mixer = WkvMixer(int(m["heads"]), int(m["dim"]), int(m.get("decay_rank") or 0))
            elif kind == "mamba2":
                mixer = Mamba2Mixer(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)), int(m["conv"]),
                                    int(m.get("norm_groups", 1)))
                if mixer.heads % mixer.groups or mixer.inner % mixer.norm_groups or mixer.conv < 1:
                    raise ValueError("Fomunex: state-space groups do not fit the heads")
            else:
                raise ValueError(f"Fomunex: unknown layer type {kind!r}")
            ml = lc.get("mlp")
            mlp = None
            if ml is not None:
                if ml["kind"] == "dense":
                    mlp = PolyNormMLP(int(ml["ff"]))
                elif ml["kind"] == "moe":
                    mlp = SigmoidRoutedMLP(int(ml["router"]["experts"]), int(ml["router"]["top"]), int(ml["expert"]["ff"]),
                                           float(ml["expert"].get("limit") or 3.0e38))
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError("Fomunex: top does not fit the experts")
                else:
                    raise ValueError(f"Fomunex: unknown feed-forward kind {ml['kind']!r}")
            src = int(lc.get("weights_of", i))
            if not 0 <= src < len(cfg["layers"]) or cfg["layers"][src].get("weights_of", src) != src or cfg["layers"][src]["type"] != kind:
                raise ValueError(f"Fomunex: layer {i} cannot use the weights of layer {src}")
            layers.append(FomunexLayer(mixer, mlp, src))
        for l in layers:        # a layer that borrows weights has its source's sizes, also the one a tensor's shape gives
            if l.mixer.kind == "wkv" and not l.mixer.decay_rank:
                l.mixer.decay_rank = layers[l.weights_of].mixer.decay_rank
        return FomunexConfig(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers, int(cfg.get("max_positions") or 0),
                             float(cfg.get("logit_scale") or 1.0), float(cfg.get("logit_softcap") or 0.0))


# --------------------------------------------------------------------------------------------------
# Dosuvik: layers that normalise a sublayer's OUTPUT only (x <- x + (1 + w) rms(f(x))) over an fp32 residual, followed by a learned
# weighted average over the results of all earlier layers; mixers are retention (linear attention with a fixed decay and rotary
# positions), gated latent attention, or windowed grouped-query attention with rotated values and a sink; feed-forwards are a dense
# clamped swish-GLU or sigmoid-routed silu-GLU experts with a choice correction and group-limited choice
# --------------------------------------------------------------------------------------------------
@dataclass
class Rotary:
    """Rotary positions on the first `dims` entries of a head: pair i turns by position * base^(-2i/dims).  layout "halves" pairs
    entry i with i + dims / 2, "interleaved" pairs entry 2i with 2i + 1."""
    dims: int
    base: float
    layout: str = "halves"

    def frequencies(self, dims: int | None = None) -> list[float]:
        d = self.dims if dims is None else dims
        return [self.base ** (-2.0 * i / d) for i in range(d // 2)]

    def to_halves(self, width: int) -> list[int]:
        """The order of a `width`-wide rotated part that turns this layout into the "halves" layout (the identity for "halves"): a dot
        product of two parts permuted alike is unchanged, so weights whose output rows are permuted so serve kernels that pair i with
        i + dims / 2."""
        if self.layout == "halves":
            return list(range(width))
        return list(range(0, self.dims, 2)) + list(range(1, self.dims, 2)) + list(range(self.dims, width))


@dataclass
class RetentionMixer:
    """Linear attention with one fixed decay per head and no softmax: rotary q and k, k scaled by dim^-0.5 after the rotation, per head
    S <- decay S + k v^T and o = S^T q over a recurrent fp32 [dim][vdim] state; each head's o divided by its root mean square (no
    weight), times silu(W_g h), projected."""
    heads: int
    dim: int
    vdim: int
    decay: list
    rope: Rotary
    kind: str = "retention"


@dataclass
class GatedLatentAttention:
    """Attention whose keys and values come from a cached low-rank latent (kv_rank wide, RMS-normed) plus ONE rotated key part shared by
    all heads; queries straight from the hidden row, per head `dim` unrotated + `rot_dim` rotated entries; ordinary causal softmax
    (window 0 = every earlier token); the concatenated heads times sigmoid(W_g h) element by element."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rope: Rotary
    window: int = 0
    kind: str = "latent_attention"


@dataclass
class RotaryWindowAttention:
    """Grouped-query attention with an RMS norm (plain weights) over the WHOLE q and the whole k projection before the heads are split,
    rotary q / k on the first rope.dims entries, values rotated by their own position over all vdim entries (cached so) and every
    head's output turned back by the query's position, a sliding window (0 = every earlier token) and a learned per-head sink in the
    softmax denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rope: Rotary
    rotate_values: bool = True
    kind: str = "attention"


@dataclass
class ClampedGluMLP:
    """Dense feed-forward W_down(g sigmoid(1.702 g) (u + 1)), g = min(W_gate h, limit), u = clamp(W_up h, +-limit)."""
    ff: int
    limit: float
    kind: str = "dense"


@dataclass
class BiasedGroupRoutedMLP:
    """Mixture of silu-GLU experts behind a sigmoid router: scores s = sigmoid(W_r h); the choice uses s + correction, the weights use
    s as it is; experts in `groups` contiguous groups, a group's score = the sum of its two largest choice scores, only experts of the
    best `keep` groups can be chosen; the `top` largest choice scores win; weights are not renormalised."""
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    kind: str = "moe"


@dataclass
class DosuvikLayer:
    mixer: object               # RetentionMixer | GatedLatentAttention | RotaryWindowAttention
    mlp: object                 # ClampedGluMLP | BiasedGroupRoutedMLP | None


@dataclass
class DosuvikConfig:
    """config.json keys: architecture, vocab, width, norm.eps, layers[{type, mixer{...}, mlp{kind, ...} | null}]."""
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    layers: list = field(default_factory=list)
    family: str = "dosuvik"
    max_position_embeddings: int = 1 << 20
    tie_word_embeddings: bool = False

    SWISH_ALPHA = 1.702         # the dense feed-forward's gate is g * sigmoid(1.702 g)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def recurrent(self) -> bool:
        """True when some layer keeps a per-sequence state that is not a function of cached pages."""
        return any(l.mixer.kind == "retention" for l in self.layers)

    def to_dict(self) -> dict:
        return asdict(self)

    @staticmethod
    def from_json(cfg: dict) -> "DosuvikConfig":
        layers = []
        for lc in cfg["layers"]:
            m, kind = lc["mixer"], lc["type"]
            r = m["rot"]
            if kind == "retention":
                mixer = RetentionMixer(int(m["heads"]), int(m["dim"]), int(m["vdim"]), [float(d) for d in m["decay"]],
                                       Rotary(int(r["dims"]), float(r["base"]), "halves"))
                if len(mixer.decay) != mixer.heads:
                    raise ValueError("Dosuvik: one decay per head")
                width = mixer.dim
            elif kind == "latent_attention":
                mask = m.get("mask") or {}
                mixer = GatedLatentAttention(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                                             float(m["scale"]), Rotary(int(r["dims"]), float(r["base"]), "interleaved"),
                                             int(mask.get("size") or 0))
                width = mixer.rot_dim
            elif kind == "attention":
                mask = m.get("mask") or {}
                mixer = RotaryWindowAttention(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                              int(mask.get("size") or 0), Rotary(int(r["dims"]), float(r["base"]), "halves"))
                if mixer.heads % mixer.kv_heads or mixer.vdim % 2:
                    raise ValueError("Dosuvik: heads must be a multiple of kv_heads and vdim even")
                width = mixer.dim
            else:
                raise ValueError(f"Dosuvik: unknown layer type {kind!r}")
            if mixer.rope.dims % 2 or not 0 <= mixer.rope.dims <= width:
                raise ValueError("Dosuvik: rot.dims must be even and at most the rotated part's size")
            ml = lc.get("mlp")
            mlp = None
            if ml is not None:
                if ml["kind"] == "dense":
                    mlp = ClampedGluMLP(int(ml["ff"]), float(ml["limit"]))
                elif ml["kind"] == "moe":
                    rt = ml["router"]
                    g = rt.get("groups") or {}
                    mlp = BiasedGroupRoutedMLP(int(rt["experts"]), int(rt["top"]), int(ml["expert"]["ff"]), int(g.get("count", 1)),
                                               int(g.get("keep", g.get("count", 1))))
                    if mlp.experts % mlp.groups or not (1 <= mlp.keep <= mlp.groups) or not (1 <= mlp.top <= mlp.experts // mlp.groups * mlp.keep):
                        raise ValueError("Dosuvik: router groups do not fit the experts")
                else:
                    raise ValueError(f"Dosuvik: unknown feed-forward kind {ml['kind']!r}")
            layers.append(DosuvikLayer(mixer, mlp))
        return DosuvikConfig(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), layers)


# config.json "architecture" values that are read by this package's own readers (everything else goes through transformers' AutoConfig)
ARCHITECTURES = {"Fatulix": FatulixConfig.from_json, "Zerusun": ZerusunConfig.from_json, "Fomunex": FomunexConfig.from_json,
                 "Dosuvik": DosuvikConfig.from_json}


def read_native_config(model_dir: str):
    """The model configuration of a directory whose config.json names one of ARCHITECTURES, else None."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        cfg = json.load(f)
    reader = ARCHITECTURES.get(cfg.get("architecture")) if isinstance(cfg, dict) else None
    if not reader:
        return None
    out = reader(cfg)
    if hasattr(out, "complete_from_checkpoint"):      # sizes that only a tensor's shape gives
        out.complete_from_checkpoint(model_dir)
    return out
