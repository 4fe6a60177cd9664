"""Architecture presets for every model the reference names or BASELINE.json configs use
(SURVEY Appendix B).  Dimensions are public model-card facts; weights are random-init
(fixed seed) unless a safetensors checkpoint directory is supplied."""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional


@dataclass
class DecoderConfig:
    name: str
    arch: str                    # "llama" | "opt"
    num_layers: int
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate: int
    vocab_size: int
    max_position: int = 8192
    norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    tie_word_embeddings: bool = False
    bos_token_id: int = 1
    eos_token_ids: tuple = (2,)
    # OPT specifics
    pos_offset: int = 2
    activation: str = "silu"     # silu (SwiGLU) | relu | gelu
    bias: bool = False


@dataclass
class EncoderConfig:
    name: str
    arch: str                    # "bert" | "nomic_bert"
    num_layers: int
    hidden: int
    num_heads: int
    intermediate: int
    vocab_size: int
    max_position: int = 512
    type_vocab_size: int = 2
    norm_eps: float = 1e-12
    pooling: str = "mean"        # mean | cls
    normalize: bool = True
    activation: str = "gelu"     # gelu | swiglu
    rotary: bool = False
    rope_theta: float = 1000.0
    bias: bool = True
    dim: int = field(init=False, default=0)

    def __post_init__(self):
        self.dim = self.hidden

    @property
    def head_dim(self) -> int:
        return self.hidden // self.num_heads


@dataclass
class HybridLayer:
    """One layer of a hybrid decoder: which sequence mixer it has, the mixer's sizes and constants,
    and its feed-forward (None: the layer has none)."""
    type: str                    # "attention" (sigmoid attention) | "mamba2"
    mixer: dict
    mlp: Optional[dict] = None   # {"kind": "dense", "ff": n}


@dataclass
class LebepelConfig:
    """The Lebepel design: parallel blocks (one norm feeds the mixer and the feed-forward, their sum
    scaled by ``residual_mult``) over an f32 residual stream, sigmoid-attention and Mamba-2 mixers
    in any order, a span of layers run ``loop_times`` times with shared weights (the embedding
    output added again before each later pass), learned positions, soft-capped logits.
    Every size and constant comes from the checkpoint's ``config.json`` (:meth:`from_json`)."""
    name: str
    vocab_size: int
    hidden: int
    layers: list                 # [HybridLayer]
    max_position: int = 2048
    norm_eps: float = 1e-5
    residual_mult: float = 1.0
    logit_softcap: float = 0.0   # 0: none
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    arch: str = "lebepel"
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False

    def layer_runs(self) -> list:
        """[(layer index, add the embedding output first)] in execution order: the looped span is
        unrolled; every run has a cache or state of its own."""
        n = len(self.layers)
        a, b, t = self.loop_start, self.loop_stop, self.loop_times
        if not (0 <= a <= b <= n) or t < 1:
            raise ValueError(f"loop [{a}, {b}) x {t} does not fit {n} layers")
        runs = [(i, False) for i in range(a)]
        for k in range(t):
            runs += [(i, k > 0 and i == a) for i in range(a, b)]
        return runs + [(i, False) for i in range(b, n)]

    @property
    def num_layers(self) -> int:
        return len(self.layer_runs())

    @classmethod
    def from_json(cls, d: dict, name: str = "lebepel") -> "LebepelConfig":
        layers = [HybridLayer(l["type"], dict(l["mixer"]), dict(l["mlp"]) if l.get("mlp") else None)
                  for l in d["layers"]]
        for l in layers:
            if l.type not in ("attention", "mamba2"):
                raise ValueError(f"unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {l.mlp.get('kind')!r}")
        loop = d.get("loop") or {}
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=layers,
                   max_position=int(d["max_positions"]), norm_eps=float((d.get("norm") or {}).get("eps", 1e-5)),
                   residual_mult=float(d.get("residual_mult", 1.0)), logit_softcap=float(d.get("logit_softcap") or 0.0),
                   loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                   loop_times=int(loop.get("times", 1)))

    def to_json(self) -> dict:
        d = {"architecture": "Lebepel", "vocab": self.vocab_size, "width": self.hidden,
             "max_positions": self.max_position, "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
             "logit_softcap": self.logit_softcap,
             "layers": [{"type": l.type, "mixer": dict(l.mixer), "mlp": dict(l.mlp) if l.mlp else None}
                        for l in self.layers]}
        if self.loop_times > 1 or self.loop_stop > self.loop_start:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return d


@dataclass
class PemidraConfig:
    """The Pemidra design: post-norm layers over an f32 stream -- ``x <- LN(alpha x + ls * sub(x))`` for the
    mixer and (where present) the gated tanh-GELU feed-forward -- with three kinds of mixer in any order:
    ``retention`` (decayed linear attention), ``general_delta`` (generalized delta rule) and ``parallel``
    (chunk-masked softmax attention with a sink beside a gated delta rule, their RMS-normed results
    averaged).  No learned positions (rotary inside the attention only) and no cap on the logits.
    Every size and constant comes from the checkpoint's ``config.json`` (:meth:`from_json`)."""
    name: str
    vocab_size: int
    hidden: int
    layers: list                 # [HybridLayer]
    norm_eps: float = 1e-6
    postln_alpha: float = 1.0
    max_position: int = 1 << 20  # nothing in the design bounds a sequence; engines pass their own limit
    arch: str = "pemidra"
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False

    MIXERS = ("retention", "general_delta", "parallel")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "pemidra") -> "PemidraConfig":
        layers = [HybridLayer(l["type"], dict(l["mixer"]), dict(l["mlp"]) if l.get("mlp") else None)
                  for l in d["layers"]]
        for l in layers:
            if l.type not in cls.MIXERS:
                raise ValueError(f"unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {l.mlp.get('kind')!r}")
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=layers,
                   norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)), postln_alpha=float(d.get("postln_alpha", 1.0)),
                   max_position=int(d.get("max_positions", 1 << 20)))

    def to_json(self) -> dict:
        return {"architecture": "Pemidra", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
                "postln_alpha": self.postln_alpha,
                "layers": [{"type": l.type, "mixer": dict(l.mixer), "mlp": dict(l.mlp) if l.mlp else None}
                           for l in self.layers]}



@dataclass
class FusasunConfig:
    """The Fusasun design: an f32 residual stream, every sublayer normed before and after
    (``x += rms(gate * sub(rms(x) w_pre)) w_post`` with the gate ``sigmoid(W_rg h + b)`` of the sublayer's
    input), a short causal convolution added to what the mixer reads (``canon_taps`` taps per channel, its
    last inputs part of a sequence's state), two sliding-window mixers in any order -- ``attention``
    (grouped-query, pooled blocks before the window) and ``latent_attention`` -- and a feed-forward of
    experts chosen by the token id from a table.  The embedding is multiplied by ``embed_scale``.
    Every size and constant comes from the checkpoint's ``config.json`` (:meth:`from_json`)."""
    name: str
    vocab_size: int
    hidden: int
    layers: list                 # [HybridLayer]
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    canon_taps: int = 1
    max_position: int = 1 << 20  # nothing in the design bounds a sequence; engines pass their own limit
    arch: str = "fusasun"
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False

    MIXERS = ("attention", "latent_attention")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "fusasun") -> "FusasunConfig":
        layers = [HybridLayer(l["type"], dict(l["mixer"]), dict(l["mlp"]) if l.get("mlp") else None)
                  for l in d["layers"]]
        for l in layers:
            if l.type not in cls.MIXERS:
                raise ValueError(f"unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {l.mlp.get('kind')!r}")
        taps = int((d.get("canon") or {}).get("taps", 1))
        if not 1 <= taps <= 8:
            raise ValueError(f"canon.taps {taps} outside 1..8")
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=layers,
                   norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)),
                   embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)), canon_taps=taps,
                   max_position=int(d.get("max_positions", 1 << 20)))

    def to_json(self) -> dict:
        return {"architecture": "Fusasun", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embed_scale}, "canon": {"taps": self.canon_taps},
                "layers": [{"type": l.type, "mixer": dict(l.mixer), "mlp": dict(l.mlp) if l.mlp else None}
                           for l in self.layers]}


@dataclass
class LumedraConfig:
    """The Lumedra design: an f32 residual stream whose blocks run their mixer and their feed-forward side by
    side on two norms of the same row (``x += mixer(rms(x) w1) + ff(rms(x) w2)``), three mixers in any order --
    ``attention`` (grouped-query, no rotation, capped scores, a sliding window that keeps the first positions,
    values blended with those of the first such layer), ``latent_attention`` (causal, element-wise output gate)
    and ``lightning`` (decayed linear attention) -- and a feed-forward that is either dense (clamped gated
    activation) or a mixture of experts (sigmoid router, group-limited choice, a shared expert).  The LM head is
    the embedding table.  Every size and constant comes from the checkpoint's ``config.json``
    (:meth:`from_json`)."""
    name: str
    vocab_size: int
    hidden: int
    layers: list                 # [HybridLayer]
    norm_eps: float = 1e-6
    max_position: int = 1 << 20  # nothing in the design bounds a sequence; engines pass their own limit
    arch: str = "lumedra"
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = True

    MIXERS = ("attention", "latent_attention", "lightning")
    MLPS = ("dense", "moe")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "lumedra") -> "LumedraConfig":
        layers = [HybridLayer(l["type"], dict(l["mixer"]), dict(l["mlp"]) if l.get("mlp") else None)
                  for l in d["layers"]]
        for l in layers:
            if l.type not in cls.MIXERS:
                raise ValueError(f"unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind") not in cls.MLPS:
                raise ValueError(f"unknown feed-forward kind {l.mlp.get('kind')!r}")
        return cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), layers=layers,
                   norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)), max_position=int(d.get("max_positions", 1 << 20)))

    def to_json(self) -> dict:
        return {"architecture": "Lumedra", "vocab": self.vocab_size, "width": self.hidden, "norm": {"eps": self.norm_eps},
                "layers": [{"type": l.type, "mixer": dict(l.mixer), "mlp": dict(l.mlp) if l.mlp else None}
                           for l in self.layers]}


def lumedra_layers(n: int, heads: int, head_dim: int, ff: int, experts: int = 0, top: int = 2, kv_heads: Optional[int] = None,
                   window: int = 1024, keep_first: int = 4, softcap: float = 30.0, rot_dim: int = 64, q_rank: int = 768,
                   kv_rank: int = 512, groups: int = 4, keep: int = 2, shared_ff: int = 0, router_scale: float = 2.5,
                   pattern=("attention", "latent_attention", "lightning"), dense_first: bool = True) -> list:
    """``n`` layers cycling through ``pattern`` with one set of head sizes (presets and benchmarks).  ``experts``
    0: every feed-forward is dense of size ``ff``; else experts of size ``ff`` (the first layer stays dense, of
    ``top`` experts' size, with ``dense_first``)."""
    kv = kv_heads or heads
    out = []
    for i in range(n):
        t = pattern[i % len(pattern)]
        if t == "attention":
            mixer = {"heads": heads, "kv_heads": kv, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
                     "softcap": softcap, "mask": {"size": window, "keep_first": keep_first}, "v_mix": True}
        elif t == "latent_attention":
            mixer = {"heads": heads, "dim": head_dim, "rot_dim": rot_dim, "vdim": head_dim, "q_rank": q_rank, "kv_rank": kv_rank,
                     "scale": (head_dim + rot_dim) ** -0.5, "rot": {"base": 10000.0, "dims": rot_dim}}
        else:
            mixer = {"heads": heads, "dim": head_dim, "vdim": head_dim,
                     "decay": [1.0 - 2.0 ** (-5.0 - 4.0 * j / max(heads - 1, 1)) for j in range(heads)]}
        if not ff:
            mlp = None
        elif experts and not (dense_first and i == 0):
            mlp = {"kind": "moe", "expert": {"ff": ff},
                   "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}, "scale": router_scale}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff}
        else:
            mlp = {"kind": "dense", "ff": ff * (top if experts else 1), "limit": 7.0}
        out.append(HybridLayer(t, mixer, mlp))
    return out


def fusasun_layers(n: int, heads: int, head_dim: int, ff: int, experts: int, top: int, kv_heads: Optional[int] = None,
                   window: int = 1024, pool: int = 64, rot_dim: int = 64, q_rank: int = 768, kv_rank: int = 256,
                   pattern=("attention", "latent_attention"), original: int = 8192) -> list:
    """``n`` layers cycling through ``pattern`` with one set of head sizes (presets and benchmarks)."""
    kv = kv_heads or heads
    out = []
    for i in range(n):
        t = pattern[i % len(pattern)]
        if t == "attention":
            mixer = {"heads": heads, "kv_heads": kv, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
                     "mask": {"size": window, "pool": pool},
                     "rot": {"base": 500000.0, "dims": head_dim,
                             "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": original}}}
        else:
            mixer = {"heads": heads, "dim": head_dim, "rot_dim": rot_dim, "vdim": head_dim, "q_rank": q_rank, "kv_rank": kv_rank,
                     "scale": (head_dim + rot_dim) ** -0.5, "mask": {"size": window},
                     "rot": {"base": 10000.0, "dims": rot_dim,
                             "scaling": {"factor": 4.0, "original": original, "fast": 32.0, "slow": 1.0}}}
        out.append(HybridLayer(t, mixer, {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
                               if ff else None))
    return out

def pemidra_layers(n: int, heads: int, head_dim: int, ff: int, kv_heads: Optional[int] = None, chunk: int = 256,
                   rot_dims: Optional[int] = None, lora: int = 128, conv: int = 4,
                   pattern=("general_delta", "retention", "parallel")) -> list:
    """``n`` layers cycling through ``pattern`` with one set of head sizes (presets and benchmarks).  Only the
    ``parallel`` layers carry a feed-forward, as the mixers of the other two are cheap by themselves."""
    kv = kv_heads or heads
    out = []
    for i in range(n):
        t = pattern[i % len(pattern)]
        if t == "retention":
            mixer = {"heads": heads, "dim": head_dim, "vdim": head_dim,
                     "decay": [0.9 + 0.0125 * (j % 8) for j in range(heads)]}
        elif t == "general_delta":
            mixer = {"heads": heads, "dim": head_dim, "lora": lora}
        else:
            mixer = {"left": {"heads": heads, "kv_heads": kv, "dim": head_dim, "vdim": head_dim, "scale": head_dim ** -0.5,
                              "mask": {"size": chunk}, "rot": {"dims": rot_dims or head_dim, "base": 10000.0}},
                     "right": {"heads": heads, "kv_heads": kv, "dim": head_dim, "vdim": head_dim, "conv": conv, "lora": lora}}
        out.append(HybridLayer(t, mixer, {"kind": "dense", "ff": ff} if ff and t == "parallel" else None))
    return out


def lebepel_layers(n: int, hidden: int, heads: int, kv_heads: int, head_dim: int, ff: int, ssm_heads: int, ssm_p: int,
                   ssm_state: int, ssm_groups: int = 1, conv: int = 4, norm_groups: int = 1, pattern=("attention", "mamba2"),
                   scale: Optional[float] = None) -> list:
    """``n`` layers cycling through ``pattern`` with one set of mixer sizes (presets and benchmarks)."""
    out = []
    for i in range(n):
        t = pattern[i % len(pattern)]
        if t == "attention":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim,
                     "scale": scale if scale is not None else head_dim ** -0.5}
        else:
            mixer = {"heads": ssm_heads, "vdim": ssm_p, "state": ssm_state, "groups": ssm_groups, "conv": conv,
                     "norm_groups": norm_groups}
        out.append(HybridLayer(t, mixer, {"kind": "dense", "ff": ff} if ff else None))
    return out


LLAMA3_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                  "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

DECODERS = {
    "llama-3-8b": DecoderConfig("llama-3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256,
                                max_position=131072, rope_scaling=LLAMA3_SCALING,
                                bos_token_id=128000, eos_token_ids=(128001, 128008, 128009)),
    "llama-3-70b": DecoderConfig("llama-3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256,
                                 max_position=131072, rope_scaling=LLAMA3_SCALING,
                                 bos_token_id=128000, eos_token_ids=(128001, 128008, 128009)),
    "opt-125m": DecoderConfig("opt-125m", "opt", 12, 768, 12, 12, 64, 3072, 50272,
                              max_position=2048, norm_eps=1e-5, tie_word_embeddings=True,
                              bos_token_id=2, eos_token_ids=(2,), activation="relu", bias=True),
    # small shapes for tests / smoke runs (same code paths, tiny weights)
    # (vocab = the built-in tokenizer's 32768 so text round-trips through the servers)
    "llama-tiny": DecoderConfig("llama-tiny", "llama", 2, 256, 4, 2, 64, 512, 32768,
                                max_position=4096, rope_theta=10000.0),
    "opt-tiny": DecoderConfig("opt-tiny", "opt", 2, 128, 2, 2, 64, 256, 32768, max_position=512,
                              tie_word_embeddings=True, activation="relu", bias=True,
                              bos_token_id=2, eos_token_ids=(2,)),
}

DECODERS.update({
    # hybrid sigmoid-attention / Mamba-2 decoders (random-init presets; checkpoints bring their own config.json)
    "lebepel-tiny": LebepelConfig("lebepel-tiny", 32768, 128, lebepel_layers(3, 128, 4, 2, 32, 256, 4, 16, 16, 2, 4, 2,
                                                                              ("mamba2", "attention", "mamba2")),
                                  max_position=1024, residual_mult=0.7, logit_softcap=20.0, loop_start=1, loop_stop=3,
                                  loop_times=2),
    "lebepel-1b": LebepelConfig("lebepel-1b", 32768, 2048, lebepel_layers(16, 2048, 16, 4, 128, 5632, 64, 64, 128, 8, 4, 8),
                                max_position=8192, residual_mult=1.0, logit_softcap=30.0),
})

DECODERS.update({
    # post-norm linear-state / chunk-attention decoders (random-init presets; checkpoints bring their own config.json)
    "pemidra-tiny": PemidraConfig("pemidra-tiny", 32768, 128, pemidra_layers(3, 4, 32, 256, kv_heads=2, chunk=24, rot_dims=16,
                                                                              lora=8), postln_alpha=1.5),
    "pemidra-1b": PemidraConfig("pemidra-1b", 32768, 2048, pemidra_layers(18, 16, 128, 5632, kv_heads=4), postln_alpha=2.0),
})

DECODERS.update({
    # pooled-window / latent attention decoders with table-routed experts (random-init presets)
    "fusasun-tiny": FusasunConfig("fusasun-tiny", 32768, 128, fusasun_layers(3, 4, 24, 40, 6, 2, kv_heads=2, window=20, pool=6,
                                                                              rot_dim=8, q_rank=48, kv_rank=40, original=64),
                                  embed_scale=2.0, canon_taps=4),
    "fusasun-1b": FusasunConfig("fusasun-1b", 32768, 2048, fusasun_layers(16, 16, 128, 512, 16, 2, kv_heads=4),
                                embed_scale=1.0, canon_taps=4),
})

DECODERS.update({
    # parallel-block decoders of capped-window / latent / lightning attention with routed experts (random-init presets)
    "lumedra-tiny": LumedraConfig("lumedra-tiny", 32768, 128, lumedra_layers(4, 4, 24, 40, 6, 2, kv_heads=2, window=20, keep_first=3,
                                                                              softcap=15.0, rot_dim=8, q_rank=48, kv_rank=40, groups=3,
                                                                              keep=2, shared_ff=48,
                                                                              pattern=("attention", "latent_attention", "lightning", "attention"))),
    "lumedra-1b": LumedraConfig("lumedra-1b", 32768, 2048, lumedra_layers(18, 16, 128, 704, 16, 4, kv_heads=4, shared_ff=1408)),
})

ENCODERS = {
    "bge-base": EncoderConfig("bge-base", "bert", 12, 768, 12, 3072, 30522, pooling="cls"),
    "minilm-l6": EncoderConfig("minilm-l6", "bert", 6, 384, 12, 1536, 30522, pooling="mean"),
    "nomic-embed-text": EncoderConfig("nomic-embed-text", "nomic_bert", 12, 768, 12, 3072, 30528,
                                      max_position=8192, pooling="mean", activation="swiglu",
                                      rotary=True, rope_theta=1000.0, bias=False),
    "bert-tiny": EncoderConfig("bert-tiny", "bert", 2, 128, 2, 256, 32768, max_position=512),
    "nomic-tiny": EncoderConfig("nomic-tiny", "nomic_bert", 2, 128, 2, 256, 32768,
                                max_position=2048, activation="swiglu", rotary=True, bias=False),
}


def decoder_config(name: str, **overrides):
    cfg = dataclasses.replace(DECODERS[name])
    for k, v in overrides.items():
        setattr(cfg, k, v)
    return cfg


def encoder_config(name: str, **overrides) -> EncoderConfig:
    cfg = dataclasses.replace(ENCODERS[name])
    for k, v in overrides.items():
        setattr(cfg, k, v)
    return cfg


def param_count(cfg) -> int:
    if isinstance(cfg, LumedraConfig):
        W, n = cfg.hidden, cfg.vocab_size * cfg.hidden + cfg.hidden
        for l in cfg.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m["heads"] * (m["dim"] + m["vdim"]) + m["kv_heads"] * (m["dim"] + m["vdim"])) + 1
            elif l.type == "latent_attention":
                qd = m["dim"] + m["rot_dim"]
                n += W * (m["q_rank"] + m["kv_rank"] + m["rot_dim"]) + m["q_rank"] * (1 + m["heads"] * qd) \
                    + m["kv_rank"] * (1 + m["heads"] * (m["dim"] + m["vdim"])) + 2 * W * m["heads"] * m["vdim"]
            else:
                n += W * m["heads"] * (2 * m["dim"] + 3 * m["vdim"]) + m["heads"] * m["vdim"]
            n += W
            if l.mlp and l.mlp["kind"] == "dense":
                n += 3 * W * l.mlp["ff"] + W
            elif l.mlp:
                r = l.mlp["router"]
                n += r["experts"] * (3 * W * l.mlp["expert"]["ff"] + W) + W
                n += 3 * W * l.mlp["shared"]["ff"] if l.mlp.get("shared") else 0
        return n
    if isinstance(cfg, FusasunConfig):
        W, n = cfg.hidden, 2 * cfg.vocab_size * cfg.hidden + cfg.hidden
        for l in cfg.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m["heads"] * (m["dim"] + m["vdim"]) + m["kv_heads"] * (m["dim"] + m["vdim"]))
            else:
                qd = m["dim"] + m["rot_dim"]
                n += W * (m["q_rank"] + m["kv_rank"] + m["rot_dim"] + m["heads"]) + m["q_rank"] * (1 + m["heads"] * qd) \
                    + m["kv_rank"] * (1 + m["heads"] * (m["dim"] + m["vdim"])) + W * m["heads"] * m["vdim"]
            n += 2 * W + W * cfg.canon_taps + W * W + W
            if l.mlp:
                n += l.mlp["router"]["experts"] * 3 * W * l.mlp["expert"]["ff"] + 2 * W + W * W + W
        return n
    if isinstance(cfg, PemidraConfig):
        W, n = cfg.hidden, 2 * cfg.vocab_size * cfg.hidden + 2 * cfg.hidden
        for l in cfg.layers:
            m = l.mixer
            if l.type == "retention":
                n += W * m["heads"] * (2 * m["dim"] + 3 * m["vdim"])
            elif l.type == "general_delta":
                hd, r = m["heads"] * m["dim"], m.get("lora", 0)
                n += 6 * W * hd + r * (W + hd) + 3 * hd
            else:
                a, b = m["left"], m["right"]
                n += W * (a["heads"] * (a["dim"] + 2 * a["vdim"] + 1) + a["kv_heads"] * (a["dim"] + a["vdim"]))
                r = b.get("lora", 0)
                n += W * (2 * b["kv_heads"] * b["dim"] + 2 * b["heads"] * b["vdim"] + b["heads"] + 2 * r) \
                    + r * b["heads"] * (b["dim"] + b["vdim"]) + 2 * W
            n += 3 * W + (3 * W * l.mlp["ff"] + 3 * W if l.mlp else 0)
        return n
    if isinstance(cfg, LebepelConfig):
        W, n = cfg.hidden, (cfg.vocab_size * 2 + cfg.max_position + 1) * cfg.hidden
        for l in cfg.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m["heads"] + m["kv_heads"]) * m["dim"] + 2 * W * m["kv_heads"] * m["vdim"] \
                    + W * (m["heads"] - m["kv_heads"]) * m["vdim"]
            else:
                inner = m["heads"] * m["vdim"]
                n += W * (2 * inner + 2 * m["groups"] * m["state"] + m["heads"]) + W * inner
            n += W + (3 * W * l.mlp["ff"] if l.mlp else 0)
        return n
    H, I, L, V = cfg.hidden, cfg.intermediate, cfg.num_layers, cfg.vocab_size
    qkv = H * (cfg.num_heads + 2 * cfg.num_kv_heads) * cfg.head_dim
    o = cfg.num_heads * cfg.head_dim * H
    mlp = (3 if cfg.activation == "silu" else 2) * H * I
    emb = V * H * (1 if cfg.tie_word_embeddings else 2)
    return L * (qkv + o + mlp + 2 * H) + emb + H


def pad_vocab(n: int, tile: int = 256) -> int:
    """Rows of an LM head padded to the MFMA GEMM kernels' 256-column tile."""
    return -(-n // tile) * tile
