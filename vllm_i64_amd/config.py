"""Model configuration of the token-routed-MoE forward (fields of the reference's ComplexityDeepConfig that the
forward path reads: vllm_i64/models/complexity_deep/config.py:15-86)."""
from __future__ import annotations

from dataclasses import dataclass, fields


@dataclass
class ModelConfig:
    name: str = "model"
    vocab_size: int = 32000
    hidden_size: int = 1024
    num_layers: int = 24
    num_heads: int = 16
    num_kv_heads: int = 4
    intermediate_size: int = 3584
    num_experts: int = 8                  # 1 => dense SwiGLU MLP
    shared_intermediate_size: int = 1792  # 0 => no shared expert
    top_k: int = 2
    primary_weight: float = 0.5           # reference default when unset is 0.95 (token_routed_mlp.py:53-54)
    routed_scale: float = 1.0
    shared_scale: float = 1.0
    rms_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_pos: int = 2304
    table_routing: bool = True
    kv_block: int = 16                    # reference hard-codes 16 (engine/i64_engine.py:245)
    use_mu_guidance: bool = False         # MuGuidance (models/complexity_deep/model.py:58-67): a per-token vector handed from layer to layer

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_heads

    @property
    def expert_inter(self) -> int:
        return self.intermediate_size // max(1, self.num_experts)

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 1

    @property
    def route_weights(self):
        if self.top_k <= 1:
            return [1.0]
        w0 = min(1.0, max(0.0, float(self.primary_weight)))
        return [w0] + [(1.0 - w0) / (self.top_k - 1)] * (self.top_k - 1)

    @classmethod
    def from_any(cls, other) -> "ModelConfig":
        """Build from any object / dict exposing the same field names (extra fields ignored)."""
        get = (lambda k: other[k]) if isinstance(other, dict) else (lambda k: getattr(other, k))
        kw = {}
        for f in fields(cls):
            try:
                kw[f.name] = get(f.name)
            except (KeyError, AttributeError):
                pass
        return cls(**kw)


def trhash500m_synth() -> ModelConfig:
    """Synthetic stand-in for tr-hash-moe-500m (its config.json is not available offline): 492.10 M parameters."""
    return ModelConfig(name="trhash500m-synth")


def trmoe306_synth() -> ModelConfig:
    return ModelConfig(name="trmoe306-synth", num_layers=18, intermediate_size=2048, num_experts=4, shared_intermediate_size=2048,
                       top_k=2, primary_weight=0.95, table_routing=False)


def dense306_synth() -> ModelConfig:
    return ModelConfig(name="dense306-synth", num_layers=18, intermediate_size=4096, num_experts=1, shared_intermediate_size=0,
                       top_k=1, primary_weight=1.0, table_routing=False)


# ---------------------------------------------------------------------------------------------------------------------------
# Morilorn: post-norm decoder with gated residuals, grouped RMS norm, depth mixing and latent attention.  Every size and every
# constant comes from the checkpoint's config.json; layers are listed one by one and may differ from each other.
# ---------------------------------------------------------------------------------------------------------------------------
@dataclass
class LatentAttentionConfig:
    heads: int
    dim: int                 # unrotated query / key dimensions per head
    rot_dim: int             # rotated query / key dimensions per head (the key part is shared by all heads)
    vdim: int                # value dimensions per head
    kv_rank: int             # width of the cached latent
    scale: float             # multiplies the scores
    window: int = 0          # a position sees itself and the window - 1 before it; 0: all earlier positions
    rot_base: float = 10000.0
    rot_dims: int = 0        # leading dimensions of the rotated part that are rotated (the rest pass through)
    sink: bool = False       # a learned score per head in the softmax's denominator, without key or value (tensor 'sink')

    @property
    def q_width(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def cache_width(self) -> int:
        return self.kv_rank + self.rot_dim

    @classmethod
    def from_dict(cls, m: dict, sink: bool = False) -> "LatentAttentionConfig":
        rot = m.get("rot") or {}
        rot_dim = int(m.get("rot_dim", 0))
        mask = m.get("mask") or {}
        c = cls(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim, vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                scale=float(m["scale"]), window=int(mask.get("size", 0)), rot_base=float(rot.get("base", 10000.0)),
                rot_dims=int(rot.get("dims", rot_dim)) if rot_dim else 0, sink=bool(sink))
        if c.rot_dims > c.rot_dim or c.rot_dims % 2:
            raise ValueError(f"latent_attention: {c.rot_dims} rotated dimensions do not fit a rotated part of {c.rot_dim}")
        if min(c.heads, c.dim, c.vdim, c.kv_rank) <= 0 or c.window < 0:
            raise ValueError(f"latent_attention: bad sizes {m}")
        return c


@dataclass
class DenseMlpConfig:
    ff: int
    kind: str = "dense"

    @classmethod
    def from_dict(cls, m: dict) -> "DenseMlpConfig":
        if m.get("kind", "dense") != "dense":
            raise ValueError(f"feed-forward kind '{m.get('kind')}' is not built")
        return cls(ff=int(m["ff"]))

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass
class MoeMlpConfig:
    """Mixture of gated feed-forward experts.  The router scores `experts + identity` entries (the last `identity` of them hand their
    input through and have no tensors); its entries form `groups` equal groups of neighbours of which the `keep` best (by their largest
    corrected score) may be chosen from; every token takes `top` entries, weighted by their uncorrected scores, renormalised and
    multiplied by `scale`.  shared_ff > 0: one more expert of that size runs for every token."""
    ff: int
    experts: int
    top: int
    identity: int = 0
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    kind: str = "moe"

    @property
    def entries(self) -> int:
        return self.experts + self.identity

    @classmethod
    def from_dict(cls, m: dict) -> "MoeMlpConfig":
        r = m["router"]
        g = r.get("groups") or {}
        c = cls(ff=int(m["expert"]["ff"]), experts=int(r["experts"]), top=int(r["top"]), identity=int(r.get("identity", 0)), groups=int(g.get("count", 1)),
                keep=int(g.get("keep", g.get("count", 1))), scale=float(r.get("scale", 1.0)), shared_ff=int((m.get("shared") or {}).get("ff", 0)))
        if min(c.ff, c.experts, c.top, c.groups, c.keep) <= 0 or c.identity < 0 or c.shared_ff < 0 or c.top > c.entries or c.entries % c.groups or \
                c.keep > c.groups or c.keep * (c.entries // c.groups) < c.top:
            raise ValueError(f"mixture of experts: bad sizes {m}")
        return c

    def to_dict(self) -> dict:
        d = {"kind": "moe", "expert": {"ff": self.ff},
             "router": {"experts": self.experts, "top": self.top, "identity": self.identity, "scale": self.scale, "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


MLPS = {"dense": DenseMlpConfig, "moe": MoeMlpConfig}


@dataclass
class Mamba2Config:
    """State-space mixer with a scalar decay per head: inner = heads * vdim channels, a (state x vdim) matrix per head and sequence,
    `groups` shared input / output maps, a causal convolution of `conv` taps in front, an RMS norm in `norm_groups` parts behind."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    conv: int = 4
    norm_groups: int = 1

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def in_width(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.state + self.heads

    @classmethod
    def from_dict(cls, m: dict) -> "Mamba2Config":
        c = cls(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]), groups=int(m.get("groups", 1)), conv=int(m.get("conv", 1)),
                norm_groups=int(m.get("norm_groups", 1)))
        if min(c.heads, c.vdim, c.state, c.groups, c.conv, c.norm_groups) <= 0 or c.heads % c.groups or c.inner % c.norm_groups:
            raise ValueError(f"mamba2: bad sizes {m}")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv, "norm_groups": self.norm_groups}


@dataclass
class KeyAttentionConfig:
    """Attention whose values are the projected keys: whole-row query / key norms, a per-head temperature, a learned bias by bucketed
    distance (as many buckets as the table has rows, logarithmic up to bias_max), visibility limited to the query's chunk of `chunk`
    positions (0: all earlier positions), a softmax with one added to the denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0
    bias_max: float = 0.0

    @classmethod
    def from_dict(cls, m: dict) -> "KeyAttentionConfig":
        c = cls(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                scale=float(m["scale"]), chunk=int((m.get("mask") or {}).get("size", 0)), bias_max=float(m.get("bias_max", 0.0)))
        if min(c.heads, c.kv_heads, c.dim) <= 0 or c.heads % c.kv_heads or c.chunk < 0:
            raise ValueError(f"attention: bad sizes {m}")
        if c.vdim != c.dim:
            raise ValueError(f"attention: the values are the keys, so vdim {c.vdim} has to equal dim {c.dim}")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale, "bias_max": self.bias_max}
        if self.chunk:
            d["mask"] = {"size": self.chunk}
        return d


@dataclass
class MinGruConfig:
    width: int

    @classmethod
    def from_dict(cls, m: dict) -> "MinGruConfig":
        if int(m["width"]) <= 0:
            raise ValueError(f"gated recurrence: bad width {m}")
        return cls(width=int(m["width"]))

    def to_dict(self) -> dict:
        return {"width": self.width}


@dataclass
class ParallelMixerConfig:
    """Two mixers that read the same input; the result is the mean of their separately normed outputs."""
    left: KeyAttentionConfig
    right: MinGruConfig

    @classmethod
    def from_dict(cls, m: dict) -> "ParallelMixerConfig":
        return cls(left=KeyAttentionConfig.from_dict(m["left"]), right=MinGruConfig.from_dict(m["right"]))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass
class Hgrn2Config:
    """Gated linear recurrence: per head a (dim x vdim) matrix with a forget gate per key channel, bounded below by a learned value; what
    the gate does not keep is written (the key is one minus the gate).  The head outputs pass an RMS norm over vdim."""
    heads: int
    dim: int
    vdim: int

    @classmethod
    def from_dict(cls, m: dict) -> "Hgrn2Config":
        c = cls(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])))
        if min(c.heads, c.dim, c.vdim) <= 0:
            raise ValueError(f"hgrn2: bad sizes {m}")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}


@dataclass
class BiasedAttentionConfig:
    """Causal attention with grouped key / value heads, separate key and value sizes, no rotation, and a learned bias by bucketed distance
    (as many buckets as the table has rows, logarithmic up to bias_max).  kv_from: the layer whose cached keys and values this layer
    attends over instead of projecting its own."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float = 0.0
    kv_from: "int | None" = None

    @classmethod
    def from_dict(cls, m: dict) -> "BiasedAttentionConfig":
        src = m.get("kv_from")
        c = cls(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                scale=float(m["scale"]), bias_max=float(m.get("bias_max", 0.0)), kv_from=int(src) if src is not None else None)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads:
            raise ValueError(f"attention: bad sizes {m}")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale, "bias_max": self.bias_max}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


MIXERS = {"latent_attention": LatentAttentionConfig, "mamba2": Mamba2Config, "parallel": ParallelMixerConfig, "hgrn2": Hgrn2Config,
          "attention": BiasedAttentionConfig}


@dataclass
class DecoderLayerConfig:
    type: str
    mixer: object
    mlp: "DenseMlpConfig | None"
    weights_of: "int | None" = None      # the layer whose tensors this layer uses (its cache and state stay its own)

    @classmethod
    def from_dict(cls, d: dict, mixers: "dict | None" = None) -> "DecoderLayerConfig":
        """mixers: a design's own table of layer type -> reader of the 'mixer' entry, where its types mean other mixers than MIXERS'."""
        MIXERS = mixers if mixers is not None else globals()["MIXERS"]
        kind = d.get("type")
        if kind not in MIXERS:
            raise ValueError(f"layer type '{kind}' is not built (known: {sorted(MIXERS)})")
        mlp = d.get("mlp")
        share = d.get("weights_of")
        if mlp and mlp.get("kind", "dense") not in MLPS:
            raise ValueError(f"feed-forward kind '{mlp.get('kind')}' is not built (known: {sorted(MLPS)})")
        reader = MIXERS[kind]
        return cls(type=kind, mixer=reader.from_dict(d["mixer"]) if hasattr(reader, "from_dict") else reader(d["mixer"]), mlp=MLPS[mlp.get("kind", "dense")].from_dict(mlp) if mlp else None,
                   weights_of=int(share) if share is not None else None)


@dataclass
class MorilornConfig:
    vocab: int
    width: int
    layers: list
    embedding_scale: float = 1.0
    postln_alpha: float = 1.0
    norm_eps: float = 1e-6
    norm_groups: int = 1
    logit_softcap: float = 0.0     # 0: logits are not capped
    name: str = "Morilorn"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_pos(self) -> int:
        """Positions are computed, not tabulated: a sequence is bounded by the page pool only."""
        return 1 << 30

    @classmethod
    def from_dict(cls, d: dict) -> "MorilornConfig":
        norm = d.get("norm") or {}
        c = cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=[DecoderLayerConfig.from_dict(l) for l in d["layers"]],
                embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), postln_alpha=float(d.get("postln_alpha", 1.0)),
                norm_eps=float(norm.get("eps", 1e-6)), norm_groups=int(norm.get("groups", 1)), logit_softcap=float(d.get("logit_softcap") or 0.0),
                name=str(d.get("architecture", "Morilorn")))
        if c.width % c.norm_groups:
            raise ValueError(f"width {c.width} does not split into {c.norm_groups} norm groups")
        return c

    def to_dict(self) -> dict:
        layers = []
        for l in self.layers:
            m = l.mixer
            mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                     "rot": {"base": m.rot_base, "dims": m.rot_dims}}
            if m.window:
                mixer["mask"] = {"size": m.window}
            layers.append({"type": l.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": l.mlp.ff} if l.mlp else None})
        return {"architecture": "Morilorn", "vocab": self.vocab, "width": self.width, "layers": layers, "embedding": {"scale": self.embedding_scale},
                "postln_alpha": self.postln_alpha, "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "logit_softcap": self.logit_softcap}


# ---------------------------------------------------------------------------------------------------------------------------
# Dogalorn: pre-norm decoder with a multi-stream residual (hyper-connections), single-number RMS norm weights, a hashed bigram
# embedding, layers that may borrow another layer's tensors, and two kinds of mixer: a state-space layer, and an attention over
# chunks of positions side by side with a gated recurrence.  Every size and constant comes from the checkpoint's config.json.
# ---------------------------------------------------------------------------------------------------------------------------
@dataclass
class BigramConfig:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class DogalornConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    streams: int = 0               # 0: the ordinary residual sum
    logit_scale: float = 1.0
    bigram: "BigramConfig | None" = None
    name: str = "Dogalorn"

    LAYER_TYPES = ("mamba2", "parallel")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_pos(self) -> int:
        """Positions are computed, not tabulated: a sequence is bounded by the page pool only."""
        return 1 << 30

    @classmethod
    def from_dict(cls, d: dict) -> "DogalornConfig":
        bg = (d.get("embedding") or {}).get("bigram")
        layers = [DecoderLayerConfig.from_dict(l) for l in d["layers"]]
        c = cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)),
                streams=int(d.get("streams") or 0), logit_scale=float(d.get("logit_scale", 1.0)),
                bigram=BigramConfig(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None,
                name=str(d.get("architecture", "Dogalorn")))
        for i, l in enumerate(layers):
            if l.type not in cls.LAYER_TYPES:
                raise ValueError(f"layer {i}: type '{l.type}' is not part of this design (known: {cls.LAYER_TYPES})")
            if l.weights_of is not None:
                j = l.weights_of
                if not 0 <= j < len(layers) or layers[j].weights_of is not None or (layers[j].type, layers[j].mixer, layers[j].mlp) != (l.type, l.mixer, l.mlp):
                    raise ValueError(f"layer {i}: borrows the tensors of layer {j}, which is no layer of the same shape with tensors of its own")
        if c.bigram is not None and c.bigram.buckets <= 0:
            raise ValueError("bigram embedding: no buckets")
        return c

    def to_dict(self) -> dict:
        layers = []
        for l in self.layers:
            e = {"type": l.type, "mixer": l.mixer.to_dict(), "mlp": {"kind": "dense", "ff": l.mlp.ff} if l.mlp else None}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        d = {"architecture": "Dogalorn", "vocab": self.vocab, "width": self.width, "layers": layers, "norm": {"eps": self.norm_eps},
             "logit_scale": self.logit_scale}
        if self.streams:
            d["streams"] = self.streams
        if self.bigram is not None:
            d["embedding"] = {"bigram": {"buckets": self.bigram.buckets, "mul_prev": self.bigram.mul_prev, "mul_cur": self.bigram.mul_cur}}
        return d


# ---------------------------------------------------------------------------------------------------------------------------
# Zabutar: sandwich-norm decoder (an RMS norm in front of and behind every sublayer, weights stored as distances from one) with
# learned absolute positions, a short causal convolution added to every sublayer's input, and layers that mix either by a gated
# linear recurrence or by attention with a distance bias (some attending over another layer's cached keys and values); dense
# feed-forwards with a two-branch quadratic / exponential activation, or mixtures of gated experts.  Every size and constant comes
# from the checkpoint's config.json.
# ---------------------------------------------------------------------------------------------------------------------------
@dataclass
class ZabutarConfig:
    vocab: int
    width: int
    layers: list
    max_positions: int
    norm_eps: float = 1e-6
    canon_taps: int = 1
    name: str = "Zabutar"

    LAYER_TYPES = ("hgrn2", "attention")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_pos(self) -> int:
        """Positions are rows of a learned table: a sequence ends where the table does."""
        return self.max_positions

    @classmethod
    def from_dict(cls, d: dict) -> "ZabutarConfig":
        layers = [DecoderLayerConfig.from_dict(l) for l in d["layers"]]
        c = cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, max_positions=int(d["max_positions"]),
                norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)), canon_taps=int((d.get("canon") or {}).get("taps", 1)),
                name=str(d.get("architecture", "Zabutar")))
        if min(c.vocab, c.width, c.max_positions, c.canon_taps) <= 0:
            raise ValueError("bad sizes")
        for i, l in enumerate(layers):
            if l.type not in cls.LAYER_TYPES:
                raise ValueError(f"layer {i}: type '{l.type}' is not part of this design (known: {cls.LAYER_TYPES})")
            if l.weights_of is not None:
                raise ValueError(f"layer {i}: this design has no layers that borrow tensors")
            if l.type == "attention" and l.mixer.kv_from is not None:
                j, m = l.mixer.kv_from, l.mixer
                o = layers[j].mixer if 0 <= j < i and layers[j].type == "attention" else None
                if o is None or o.kv_from is not None or (o.kv_heads, o.dim, o.vdim) != (m.kv_heads, m.dim, m.vdim):
                    raise ValueError(f"layer {i}: takes keys and values from layer {j}, which is no earlier attention layer with projections of its own and the same sizes")
        return c

    def to_dict(self) -> dict:
        return {"architecture": "Zabutar", "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
                "canon": {"taps": self.canon_taps},
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": l.mlp.to_dict() if l.mlp else None} for l in self.layers]}


# ---------------------------------------------------------------------------------------------------------------------------
# Fukatar: a decoder whose sublayers read the residual itself and whose results pass a centred norm before they are added; the
# mixer's input is first blended per channel with the row before (token shift); scaled embedding plus a hashed bigram row; per
# layer one of three mixers: softmax attention with rotated queries, keys AND values (whole-row query / key norms, capped scores,
# a sigmoid gate per head), latent attention without positions and with a learned sink, or a capped unit-norm attention side by
# side with a gated delta rule; feed-forwards with a squared relu; capped logits.  Every size and constant comes from config.json.
# ---------------------------------------------------------------------------------------------------------------------------
@dataclass
class RotaryConfig:
    """Rotation of the first `dims` values of a head by position * base^(-2i / dims).  With scaling the frequencies whose period is
    long against `original` positions are divided by `factor`, the short-period ones kept, with a linear ramp over the pair index
    between the two at which `original` positions make `fast` and `slow` turns; sine and cosine then carry 0.1 ln(factor) + 1."""
    base: float
    dims: int
    factor: float = 0.0          # 0: no scaling
    original: float = 0.0
    fast: float = 0.0
    slow: float = 0.0

    @classmethod
    def from_dict(cls, r: dict) -> "RotaryConfig":
        sc = r.get("scaling") or {}
        c = cls(base=float(r["base"]), dims=int(r["dims"]), factor=float(sc.get("factor", 0.0)), original=float(sc.get("original", 0.0)),
                fast=float(sc.get("fast", 0.0)), slow=float(sc.get("slow", 0.0)))
        if c.dims < 0 or c.dims % 2 or c.base <= 1.0 or (c.factor and min(c.factor, c.original, c.fast, c.slow) <= 0):
            raise ValueError(f"rotation: bad constants {r}")
        return c

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.factor:
            d["scaling"] = {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}
        return d

    def frequencies(self):
        """([dims / 2] frequencies evaluated in 64 bits, the factor on sine and cosine)."""
        import math
        half, D, b = self.dims // 2, self.dims, self.base
        f = [b ** (-2.0 * i / D) for i in range(half)]
        if not self.factor:
            return f, 1.0
        where = lambda turns: D * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(b))
        lo, hi = max(math.floor(where(self.fast)), 0), min(math.ceil(where(self.slow)), D - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / self.factor * ramp + f[i] * (1.0 - ramp)
        return f, 0.1 * math.log(self.factor) + 1.0


@dataclass
class RotaryAttentionConfig:
    """Causal softmax attention over grouped key / value heads with separate key and value sizes and rotated positions.  What a design
    fixes comes in as flags: qk_norm 'row' (RMS norm over the whole projection with weights 'q.norm' / 'k.norm', before the rotation),
    'head' (per head, without weights, after it) or None; interleaved pairs (2i, 2i + 1) or halves (i, i + dims / 2); rotated values
    (all vdim dimensions by the value's own position, the head's sum turned back by the query's); a sigmoid gate per head ('g')."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0           # 0: scores are not capped
    rot: "RotaryConfig | None" = None
    qk_norm: "str | None" = None
    interleaved: bool = False
    rotate_values: bool = False
    head_gate: bool = False

    @classmethod
    def from_dict(cls, m: dict, **design) -> "RotaryAttentionConfig":
        c = cls(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                softcap=float(m.get("softcap") or 0.0), rot=RotaryConfig.from_dict(m["rot"]) if m.get("rot") else None, **design)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads or c.softcap < 0 or (c.rot is not None and c.rot.dims > c.dim):
            raise ValueError(f"attention: bad sizes {m}")
        if c.rotate_values and c.rot is not None and c.vdim % 2:
            raise ValueError(f"attention: rotated values of an odd size {c.vdim}")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap:
            d["softcap"] = self.softcap
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass
class GatedDeltaConfig:
    """Gated delta rule: per head a (dim x vdim) matrix that decays by a scalar per head and token, is corrected towards the value along
    the (unit) key with a sigmoid strength, and is read by the (unit, scaled) query after the write; `kv_heads` query / key heads serve
    `heads` value heads; a causal convolution of `conv` taps and silu in front of q, k and v; a gated RMS norm over vdim behind."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int = 1

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @classmethod
    def from_dict(cls, m: dict) -> "GatedDeltaConfig":
        c = cls(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), conv=int(m.get("conv", 1)))
        if min(c.heads, c.kv_heads, c.dim, c.vdim, c.conv) <= 0 or c.heads % c.kv_heads:
            raise ValueError(f"gated delta rule: bad sizes {m}")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


def _fukatar_latent(m: dict) -> LatentAttentionConfig:
    c = LatentAttentionConfig.from_dict(m, sink=True)
    if c.rot_dim or c.window:
        raise ValueError("latent attention of this design has no rotated part and no window")
    return c


def _fukatar_parallel(m: dict) -> ParallelMixerConfig:
    return ParallelMixerConfig(left=RotaryAttentionConfig.from_dict(m["left"], qk_norm="head", interleaved=True),
                               right=GatedDeltaConfig.from_dict(m["right"]))


FUKATAR_MIXERS = {"attention": lambda m: RotaryAttentionConfig.from_dict(m, qk_norm="row", rotate_values=True, head_gate=True),
                  "latent_attention": _fukatar_latent, "parallel": _fukatar_parallel}


@dataclass
class FukatarConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    bigram: "BigramConfig | None" = None
    logit_softcap: float = 0.0     # 0: logits are not capped
    name: str = "Fukatar"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_pos(self) -> int:
        """Positions are computed, not tabulated: a sequence is bounded by the page pool only."""
        return 1 << 30

    @classmethod
    def from_dict(cls, d: dict) -> "FukatarConfig":
        emb = d.get("embedding") or {}
        bg = emb.get("bigram")
        layers = [DecoderLayerConfig.from_dict(l, FUKATAR_MIXERS) for l in d["layers"]]
        c = cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers, norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)),
                embedding_scale=float(emb.get("scale", 1.0)), bigram=BigramConfig(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None,
                logit_softcap=float(d.get("logit_softcap") or 0.0), name=str(d.get("architecture", "Fukatar")))
        if min(c.vocab, c.width) <= 0 or (c.bigram is not None and c.bigram.buckets <= 0):
            raise ValueError("bad sizes")
        for i, l in enumerate(layers):
            if l.weights_of is not None:
                raise ValueError(f"layer {i}: this design has no layers that borrow tensors")
            if l.mlp is not None and l.mlp.kind != "dense":
                raise ValueError(f"layer {i}: feed-forward kind '{l.mlp.kind}' is not part of this design")
        return c

    def to_dict(self) -> dict:
        emb = {"scale": self.embedding_scale}
        if self.bigram is not None:
            emb["bigram"] = {"buckets": self.bigram.buckets, "mul_prev": self.bigram.mul_prev, "mul_cur": self.bigram.mul_cur}
        layers = []
        for l in self.layers:
            m = l.mixer
            if l.type == "latent_attention":
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale}
            else:
                mixer = m.to_dict()
            layers.append({"type": l.type, "mixer": mixer, "mlp": l.mlp.to_dict() if l.mlp else None})
        d = {"architecture": "Fukatar", "vocab": self.vocab, "width": self.width, "embedding": emb, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        return d
