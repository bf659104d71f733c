"""Typed model configuration, read from the architecture's own config.json keys.

Every size and constant of the model comes from here; nothing downstream carries a
number of its own.  Field meanings and the rejected options follow the reference
(atomserve/config.py:15-65).
"""

from dataclasses import dataclass, replace


class ConfigError(ValueError):
    """config.json names something this engine does not compute."""


def _require(raw: dict, keys: list[str]) -> None:
    missing = [k for k in keys if k not in raw]
    if missing:
        raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")


@dataclass(frozen=True)
class Qwen3Config:
    """Shape and numerics of a Qwen3 dense decoder (reference atomserve/config.py:19-29)."""

    vocab_size: int  # rows of the embedding and of the head
    hidden_size: int  # width of the residual stream
    intermediate_size: int  # width inside the gated feed-forward
    num_layers: int  # decoder layers
    num_heads: int  # query heads
    num_kv_heads: int  # key/value heads; fewer than query heads means grouped queries
    head_dim: int  # width of one head; heads * head_dim need not equal hidden_size
    rms_norm_eps: float  # epsilon of every RMSNorm, the per-head q/k norms included
    rope_theta: float  # base of the rotary frequencies
    tie_word_embeddings: bool  # the head is the embedding table
    max_position_embeddings: int  # longest context the model was trained for

    architecture = "Qwen3ForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        """Validate a parsed config.json; anything that would change the math is refused
        rather than ignored (reference atomserve/config.py:31-60)."""
        for key, why in (
            ("attention_bias", "projection biases are not computed"),
            ("rope_scaling", "scaled rotary frequencies are not computed"),
            ("use_sliding_window", "sliding-window attention is not part of this architecture here"),
        ):
            if raw.get(key):
                raise ConfigError(f"{key}={raw[key]!r} is not supported: {why}")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act={raw['hidden_act']!r} is not supported (only 'silu')")
        _require(
            raw,
            ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
             "num_attention_heads", "num_key_value_heads", "rms_norm_eps", "rope_theta",
             "max_position_embeddings"],
        )  # fmt: skip
        heads = int(raw["num_attention_heads"])
        cfg = cls(
            vocab_size=int(raw["vocab_size"]),
            hidden_size=int(raw["hidden_size"]),
            intermediate_size=int(raw["intermediate_size"]),
            num_layers=int(raw["num_hidden_layers"]),
            num_heads=heads,
            num_kv_heads=int(raw["num_key_value_heads"]),
            head_dim=int(raw.get("head_dim") or int(raw["hidden_size"]) // heads),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=float(raw["rope_theta"]),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            max_position_embeddings=int(raw["max_position_embeddings"]),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_layers", "num_heads",
                     "num_kv_heads", "head_dim", "max_position_embeddings"):  # fmt: skip
            if getattr(self, name) < 1:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_heads} is not a multiple of "
                f"num_key_value_heads {self.num_kv_heads}"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs)")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        return {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "attention_bias": False,
            "torch_dtype": "bfloat16",
        }


# ---- Dozusun ------------------------------------------------------------------------------------------


def _need(raw: dict, key: str, where: str):
    if not isinstance(raw, dict) or key not in raw:
        raise ConfigError(f"config.json lacks {where}{key}")
    return raw[key]


@dataclass(frozen=True)
class DozusunDelta:
    """A gated-delta-rule mixer's sizes."""

    heads: int  # value heads
    kv_heads: int  # query/key heads
    dim: int  # width of a query/key head
    vdim: int  # width of a value head
    conv: int  # taps of the short convolutions

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DozusunDelta":
        return cls(*(int(_need(raw, k, where)) for k in ("heads", "kv_heads", "dim", "vdim", "conv")))


@dataclass(frozen=True)
class DozusunSideBySide:
    """An attention (left) and a gated linear recurrence (right) reading the same input."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int  # keys a position sees, itself included; 0: all
    scale: float  # multiplies q.k
    left_scale: float
    width: int  # channels of the recurrence
    blocks: int  # diagonal blocks of its gates
    conv: int
    right_scale: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DozusunSideBySide":
        left, right = _need(raw, "left", where), _need(raw, "right", where)
        mask = left.get("mask") or {}
        return cls(
            heads=int(_need(left, "heads", where + "left.")),
            kv_heads=int(_need(left, "kv_heads", where + "left.")),
            dim=int(_need(left, "dim", where + "left.")),
            vdim=int(_need(left, "vdim", where + "left.")),
            window=int(mask.get("size", 0)),
            scale=float(_need(left, "scale", where + "left.")),
            left_scale=float(_need(raw, "left_scale", where)),
            width=int(_need(right, "width", where + "right.")),
            blocks=int(_need(right, "blocks", where + "right.")),
            conv=int(_need(right, "conv", where + "right.")),
            right_scale=float(_need(raw, "right_scale", where)),
        )


@dataclass(frozen=True)
class DozusunFeedForward:
    kind: str  # "dense" or "moe"
    ff: int  # width inside the feed-forward (of one expert for "moe")
    experts: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DozusunFeedForward":
        kind = _need(raw, "kind", where)
        if kind == "dense":
            return cls("dense", int(_need(raw, "ff", where)))
        if kind == "moe":
            router = _need(raw, "router", where)
            return cls("moe", int(_need(_need(raw, "expert", where), "ff", where + "expert.")),
                       int(_need(router, "experts", where + "router.")), int(_need(router, "top", where + "router.")))  # fmt: skip
        raise ConfigError(f"{where}kind={kind!r} is not supported ('dense' or 'moe')")


@dataclass(frozen=True)
class DozusunLayer:
    type: str  # "delta" or "parallel"
    mixer: object  # DozusunDelta or DozusunSideBySide
    mlp: object  # DozusunFeedForward or None


@dataclass(frozen=True)
class DozusunConfig:
    """A Dozusun decoder: layers of two kinds of mixers with dense or table-routed feed-forwards, both parts of
    a layer reading the same stream; a stretch of layers may run several times in a row."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple  # of DozusunLayer
    loop_start: int = 0  # layers loop_start .. loop_stop - 1 run loop_times times in a row
    loop_stop: int = 0
    loop_times: int = 1

    architecture = "Dozusun"

    @classmethod
    def from_dict(cls, raw: dict) -> "DozusunConfig":
        _require(raw, ["vocab", "width", "layers", "norm"])
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            if kind == "delta":
                mixer = DozusunDelta.from_dict(_need(entry, "mixer", where), where + "mixer.")
            elif kind == "parallel":
                mixer = DozusunSideBySide.from_dict(_need(entry, "mixer", where), where + "mixer.")
            else:
                raise ConfigError(f"{where}type={kind!r} is not supported ('delta' or 'parallel')")
            mlp = entry.get("mlp")
            layers.append(DozusunLayer(kind, mixer, None if mlp is None else DozusunFeedForward.from_dict(mlp, where + "mlp.")))
        loop = raw.get("loop") or {}
        cfg = cls(
            vocab_size=int(raw["vocab"]),
            hidden_size=int(raw["width"]),
            norm_eps=float(_need(raw["norm"], "eps", "norm.")),
            layers=tuple(layers),
            loop_start=int(loop.get("start", 0)),
            loop_stop=int(loop.get("stop", 0)),
            loop_times=int(loop.get("times", 1)),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers) or self.loop_times < 1:
            raise ConfigError(f"loop {self.loop_start}:{self.loop_stop} x {self.loop_times} does not fit {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.kv_heads, m.dim, m.vdim, m.conv) < 1 or m.heads % m.kv_heads:
                raise ConfigError(f"layers[{i}]: head counts and sizes must be positive, heads a multiple of kv_heads")
            if layer.type == "parallel" and (m.width < 1 or m.blocks < 1 or m.width % m.blocks or m.window < 0):
                raise ConfigError(f"layers[{i}]: width must divide into blocks, and a window is not negative")
            f = layer.mlp
            if f is not None and (f.ff < 1 or (f.kind == "moe" and not 1 <= f.top <= f.experts)):
                raise ConfigError(f"layers[{i}].mlp: sizes must be positive and top at most the number of experts")

    def run_order(self) -> list:
        """Indices of the layers in the order they run."""
        n = len(self.layers)
        inside = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + inside * self.loop_times + list(range(self.loop_stop, n))

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "delta":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            else:
                left = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.window:
                    left["mask"] = {"size": m.window}
                mixer = {"left": left, "left_scale": m.left_scale, "right_scale": m.right_scale,
                         "right": {"width": m.width, "blocks": m.blocks, "conv": m.conv}}  # fmt: skip
            f = layer.mlp
            if f is None:
                mlp = None
            elif f.kind == "dense":
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        raw = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "layers": layers}  # fmt: skip
        if self.loop_times > 1 or self.loop_stop > self.loop_start:
            raw["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return raw


# ---- Koravik ------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class KoravikAttention:
    """An attention mixer's sizes and constants."""

    heads: int
    kv_heads: int
    dim: int  # width of a query/key head
    vdim: int  # width of a value head: the keys are the values, so this is `dim`
    scale: float  # multiplies q.k
    rot_dims: int  # coordinates of a head that turn with the position
    rot_base: float
    window: int  # keys a position sees, itself included; 0: all
    keep_first: int  # the sequence's first tokens, which stay visible behind the window

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "KoravikAttention":
        rot, mask = raw.get("rot") or {}, raw.get("mask") or {}  # neither: nothing turns, every earlier key is seen
        return cls(
            heads=int(_need(raw, "heads", where)),
            kv_heads=int(_need(raw, "kv_heads", where)),
            dim=int(_need(raw, "dim", where)),
            vdim=int(raw.get("vdim", raw.get("dim", 0))),
            scale=float(_need(raw, "scale", where)),
            rot_dims=int(rot.get("dims", 0)),
            rot_base=float(_need(rot, "base", where + "rot.")) if rot.get("dims") else 1.0,
            window=int(mask.get("size", 0)),
            keep_first=int(mask.get("keep_first", 0)),
        )

    def to_dict(self) -> dict:
        raw = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
               "rot": {"dims": self.rot_dims, "base": self.rot_base}}  # fmt: skip
        if self.window:
            raw["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return raw


@dataclass(frozen=True)
class KoravikExperts:
    """A feed-forward of routed experts with one shared expert (shared_ff 0: none)."""

    ff: int  # width inside one expert
    experts: int
    top: int
    shared_ff: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "KoravikExperts":
        kind = _need(raw, "kind", where)
        if kind != "moe":
            raise ConfigError(f"{where}kind={kind!r} is not supported (only 'moe')")
        router = _need(raw, "router", where)
        shared = raw.get("shared") or {}
        return cls(
            ff=int(_need(_need(raw, "expert", where), "ff", where + "expert.")),
            experts=int(_need(router, "experts", where + "router.")),
            top=int(_need(router, "top", where + "router.")),
            shared_ff=int(shared.get("ff", 0)),
        )

    def to_dict(self) -> dict:
        raw = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            raw["shared"] = {"ff": self.shared_ff}
        return raw


@dataclass(frozen=True)
class KoravikLayer:
    type: str  # "attention"
    mixer: KoravikAttention
    mlp: object  # KoravikExperts or None


@dataclass(frozen=True)
class KoravikConfig:
    """A Koravik decoder: pre-norm layers of a mixed-heads attention and routed experts whose outputs enter the
    stream through a sigmoid gate and a common factor; the embedding is normed; a stretch of layers may run
    several times in a row, each pass entering through a matrix that also reads the embedding's output; the
    head is the embedding table, its logits scaled."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    logit_scale: float
    layers: tuple  # of KoravikLayer
    loop: bool = False  # whether a stretch is looped (and `loop.in` exists)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    architecture = "Koravik"

    @classmethod
    def from_dict(cls, raw: dict) -> "KoravikConfig":
        _require(raw, ["vocab", "width", "layers", "norm", "residual_mult", "logit_scale"])
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            if kind != "attention":
                raise ConfigError(f"{where}type={kind!r} is not supported (only 'attention')")
            mixer = KoravikAttention.from_dict(_need(entry, "mixer", where), where + "mixer.")
            mlp = entry.get("mlp")
            layers.append(KoravikLayer(kind, mixer, None if mlp is None else KoravikExperts.from_dict(mlp, where + "mlp.")))
        loop = raw.get("loop")
        cfg = cls(
            vocab_size=int(raw["vocab"]),
            hidden_size=int(raw["width"]),
            norm_eps=float(_need(raw["norm"], "eps", "norm.")),
            residual_mult=float(raw["residual_mult"]),
            logit_scale=float(raw["logit_scale"]),
            layers=tuple(layers),
            loop=bool(loop),
            loop_start=int(_need(loop, "start", "loop.")) if loop else 0,
            loop_stop=int(_need(loop, "stop", "loop.")) if loop else 0,
            loop_times=int(_need(loop, "times", "loop.")) if loop else 1,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers) or self.loop_times < 1:
            raise ConfigError(f"loop {self.loop_start}:{self.loop_stop} x {self.loop_times} does not fit {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.kv_heads, m.dim) < 1 or m.heads % m.kv_heads:
                raise ConfigError(f"layers[{i}]: head counts and sizes must be positive, heads a multiple of kv_heads")
            if m.vdim != m.dim:
                raise ConfigError(f"layers[{i}]: the values are the keys, so vdim {m.vdim} must equal dim {m.dim}")
            if m.rot_dims < 0 or m.rot_dims % 2 or m.rot_dims > m.dim or not m.rot_base > 0:
                raise ConfigError(f"layers[{i}]: rot.dims must be even and at most dim, rot.base positive")
            if m.window < 0 or m.keep_first < 0:
                raise ConfigError(f"layers[{i}]: mask.size and mask.keep_first must not be negative")
            f = layer.mlp
            if f is not None and (f.ff < 1 or f.shared_ff < 0 or not 1 <= f.top <= f.experts):
                raise ConfigError(f"layers[{i}].mlp: sizes must be positive and top at most the number of experts")

    def run_order(self) -> list:
        """(layer, whether the stream re-enters before it) in the order the layers run: the looped stretch
        `times` times, every pass entering through the loop's matrix before its first layer."""
        n = len(self.layers)
        order = [(i, False) for i in range(self.loop_start)]
        for _ in range(self.loop_times if self.loop else 0):
            order += [(i, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return order + [(i, False) for i in range(self.loop_stop if self.loop else 0, n)]

    @property
    def reenters(self) -> bool:
        return any(r for _, r in self.run_order())

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        layers = [{"type": layer.type, "mixer": layer.mixer.to_dict(), "mlp": None if layer.mlp is None else layer.mlp.to_dict()}
                  for layer in self.layers]  # fmt: skip
        raw = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "logit_scale": self.logit_scale,
               "layers": layers}  # fmt: skip
        if self.loop:
            raw["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return raw


# ---- Mumizen ------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class MumizenDecay:
    """A linear-attention mixer with a fixed decay per head ("lightning" or "retention")."""

    heads: int
    dim: int  # width of a query/key head
    vdim: int  # width of a value head
    decay: tuple  # per head

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MumizenDecay":
        decay = _need(raw, "decay", where)
        return cls(int(_need(raw, "heads", where)), int(_need(raw, "dim", where)), int(_need(raw, "vdim", where)),
                   tuple(float(d) for d in decay))  # fmt: skip

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class MumizenLatent:
    """An attention through a latent.  kv_from >= 0: the layer has no latent of its own and reads that layer's."""

    heads: int
    dim: int  # coordinates of a query/key head that are not rotated
    rot_dim: int  # and those that are
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    scaling: object  # None, or (factor, original, fast, slow)
    kv_from: int = -1

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MumizenLatent":
        rot = raw.get("rot") or {}
        rot_dim = int(_need(raw, "rot_dim", where))
        if rot_dim and int(_need(rot, "dims", where + "rot.")) != rot_dim:
            raise ConfigError(f"{where}rot.dims must equal rot_dim")
        scaling = rot.get("scaling")
        if scaling:
            scaling = tuple(float(_need(scaling, k, where + "rot.scaling.")) for k in ("factor", "original", "fast", "slow"))
        return cls(
            heads=int(_need(raw, "heads", where)),
            dim=int(_need(raw, "dim", where)),
            rot_dim=rot_dim,
            vdim=int(_need(raw, "vdim", where)),
            q_rank=int(_need(raw, "q_rank", where)),
            kv_rank=int(_need(raw, "kv_rank", where)),
            scale=float(_need(raw, "scale", where)),
            rot_base=float(_need(rot, "base", where + "rot.")) if rot_dim else 1.0,
            scaling=scaling or None,
            kv_from=int(raw["kv_from"]) if raw.get("kv_from") is not None else -1,
        )

    def to_dict(self) -> dict:
        raw = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
               "kv_rank": self.kv_rank, "scale": self.scale}  # fmt: skip
        if self.rot_dim:
            raw["rot"] = {"dims": self.rot_dim, "base": self.rot_base}
            if self.scaling:
                raw["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        if self.kv_from >= 0:
            raw["kv_from"] = self.kv_from
        return raw


@dataclass(frozen=True)
class MumizenFeedForward:
    kind: str  # "dense" or "moe"
    ff: int  # width inside the feed-forward (of one expert for "moe")
    limit: float
    experts: int = 0
    top: int = 0
    shared_ff: int = 0
    shared_limit: float = 0.0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MumizenFeedForward":
        kind = _need(raw, "kind", where)
        if kind == "dense":
            return cls("dense", int(_need(raw, "ff", where)), float(_need(raw, "limit", where)))
        if kind == "moe":
            expert, router = _need(raw, "expert", where), _need(raw, "router", where)
            shared = raw.get("shared") or {}
            return cls("moe", int(_need(expert, "ff", where + "expert.")), float(_need(expert, "limit", where + "expert.")),
                       int(_need(router, "experts", where + "router.")), int(_need(router, "top", where + "router.")),
                       int(shared.get("ff", 0)), float(_need(shared, "limit", where + "shared.")) if shared.get("ff") else 0.0)  # fmt: skip
        raise ConfigError(f"{where}kind={kind!r} is not supported ('dense' or 'moe')")

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        raw = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            raw["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return raw


@dataclass(frozen=True)
class MumizenLayer:
    type: str  # "lightning", "retention" or "latent_attention"
    mixer: object  # MumizenDecay or MumizenLatent
    mlp: object  # MumizenFeedForward or None


@dataclass(frozen=True)
class MumizenConfig:
    """A Mumizen decoder: pre-norm layers with norms in groups, a token shift before every mixer and an average over
    the results of all layers so far after every layer; mixers are linear attentions with fixed decays or attentions
    through a latent (which may read an earlier layer's), feed-forwards dense or routed with a shared expert."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    norm_groups: int
    layers: tuple  # of MumizenLayer

    architecture = "Mumizen"
    MIXERS = ("lightning", "retention", "latent_attention")

    @classmethod
    def from_dict(cls, raw: dict) -> "MumizenConfig":
        _require(raw, ["vocab", "width", "layers", "norm"])
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            if kind in ("lightning", "retention"):
                mixer = MumizenDecay.from_dict(_need(entry, "mixer", where), where + "mixer.")
            elif kind == "latent_attention":
                mixer = MumizenLatent.from_dict(_need(entry, "mixer", where), where + "mixer.")
            else:
                raise ConfigError(f"{where}type={kind!r} is not supported (one of {', '.join(cls.MIXERS)})")
            mlp = entry.get("mlp")
            layers.append(MumizenLayer(kind, mixer, None if mlp is None else MumizenFeedForward.from_dict(mlp, where + "mlp.")))
        cfg = cls(
            vocab_size=int(raw["vocab"]),
            hidden_size=int(raw["width"]),
            norm_eps=float(_need(raw["norm"], "eps", "norm.")),
            norm_groups=int(raw["norm"].get("groups", 1)),
            layers=tuple(layers),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.norm_groups < 1 or self.hidden_size % self.norm_groups:
            raise ConfigError(f"norm.groups {self.norm_groups} does not divide the width {self.hidden_size}")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if layer.type == "latent_attention":
                if min(m.heads, m.dim, m.vdim, m.q_rank, m.kv_rank) < 1 or m.rot_dim < 0 or m.rot_dim % 2:
                    raise ConfigError(f"layers[{i}]: sizes must be positive and rot_dim even")
                if m.rot_dim and not m.rot_base > 1:
                    raise ConfigError(f"layers[{i}]: rot.base must exceed 1")
                if m.kv_from >= 0:
                    src = self.layers[m.kv_from] if m.kv_from < i else None
                    if src is None or src.type != "latent_attention" or src.mixer.kv_from >= 0:
                        raise ConfigError(f"layers[{i}]: kv_from names an earlier latent-attention layer with a latent of its own")
                    s = src.mixer
                    if (s.kv_rank, s.rot_dim, s.rot_base, s.scaling) != (m.kv_rank, m.rot_dim, m.rot_base, m.scaling):
                        raise ConfigError(f"layers[{i}]: kv_rank, rot_dim and rotation must equal those of layer {m.kv_from}")
            else:
                if min(m.heads, m.dim, m.vdim) < 1 or len(m.decay) != m.heads:
                    raise ConfigError(f"layers[{i}]: sizes must be positive, with one decay per head")
                if any(not 0.0 <= d <= 1.0 for d in m.decay):
                    raise ConfigError(f"layers[{i}]: decays lie between 0 and 1")
            f = layer.mlp
            if f is not None and (f.ff < 1 or not f.limit > 0 or (f.kind == "moe" and not 1 <= f.top <= f.experts)
                                  or f.shared_ff < 0 or (f.shared_ff and not f.shared_limit > 0)):  # fmt: skip
                raise ConfigError(f"layers[{i}].mlp: sizes and limits must be positive and top at most the number of experts")

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        layers = [{"type": layer.type, "mixer": layer.mixer.to_dict(), "mlp": None if layer.mlp is None else layer.mlp.to_dict()}
                  for layer in self.layers]  # fmt: skip
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "layers": layers}  # fmt: skip


# ---- Natatar ------------------------------------------------------------------------------------------


def _rotation(raw, where: str):
    """(dims, base, scaling) of a mixer's `rot`, scaling None or (factor, original, fast, slow); None without `rot`."""
    if not raw:
        return None
    scaling = raw.get("scaling")
    if scaling:
        scaling = tuple(float(_need(scaling, k, where + "scaling.")) for k in ("factor", "original", "fast", "slow"))
    return (int(_need(raw, "dims", where)), float(_need(raw, "base", where)), scaling or None)


def _rotation_dict(rot) -> dict:
    raw = {"dims": rot[0], "base": rot[1]}
    if rot[2]:
        raw["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot[2]))
    return raw


@dataclass(frozen=True)
class NatatarAttention:
    """A softmax attention's sizes and options.  As a layer's own mixer ("attention") it has biases, a norm over the
    whole of q and of k and, with v_mix, values mixed with those of the first such layer; as the left half of a
    "parallel" mixer it has a rotation and an output gate instead."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    v_mix: bool = False
    rot: object = None  # None, or (dims, base, scaling)

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "NatatarAttention":
        return cls(*(int(_need(raw, k, where)) for k in ("heads", "kv_heads", "dim", "vdim")),
                   scale=float(_need(raw, "scale", where)), v_mix=bool(raw.get("v_mix", False)),
                   rot=_rotation(raw.get("rot"), where + "rot."))  # fmt: skip

    def to_dict(self) -> dict:
        raw = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.v_mix:
            raw["v_mix"] = True
        if self.rot:
            raw["rot"] = _rotation_dict(self.rot)
        return raw


@dataclass(frozen=True)
class NatatarMemory:
    """A matrix memory with exponential gates (the right half of a "parallel" mixer)."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "NatatarMemory":
        return cls(*(int(_need(raw, k, where)) for k in ("heads", "dim", "vdim")), gate_cap=float(_need(raw, "gate_cap", where)))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class NatatarParallel:
    left: NatatarAttention
    right: NatatarMemory
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "NatatarParallel":
        return cls(NatatarAttention.from_dict(_need(raw, "left", where), where + "left."),
                   NatatarMemory.from_dict(_need(raw, "right", where), where + "right."),
                   float(_need(raw, "left_scale", where)), float(_need(raw, "right_scale", where)))  # fmt: skip

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}  # fmt: skip


@dataclass(frozen=True)
class NatatarChannelDelta:
    """A gated delta rule with a decay per head and key channel.  The ranks of the two-step projections (of the
    decay's step size and of the output gate) are sizes that only the checkpoint's shapes tell: a configuration
    read from a model folder is completed from them, one written by this package names them itself."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int = 0
    gate_rank: int = 0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "NatatarChannelDelta":
        return cls(*(int(_need(raw, k, where)) for k in ("heads", "kv_heads", "dim", "vdim", "conv")),
                   decay_rank=int(raw.get("decay_rank", 0)), gate_rank=int(raw.get("gate_rank", 0)))  # fmt: skip

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
                "decay_rank": self.decay_rank, "gate_rank": self.gate_rank}  # fmt: skip


@dataclass(frozen=True)
class NatatarExperts:
    ff: int
    experts: int
    top: int
    scale: float = 1.0
    groups: int = 1  # equal groups of neighbouring experts
    keep: int = 1  # groups of which experts can be chosen

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "NatatarExperts":
        kind = _need(raw, "kind", where)
        if kind != "moe":
            raise ConfigError(f"{where}kind={kind!r} is not supported ('moe')")
        expert, router = _need(raw, "expert", where), _need(raw, "router", where)
        groups = router.get("groups") or {}
        count = int(groups.get("count", 1))
        return cls(int(_need(expert, "ff", where + "expert.")), int(_need(router, "experts", where + "router.")),
                   int(_need(router, "top", where + "router.")), float(router.get("scale", 1.0)), count,
                   int(groups.get("keep", count)))  # fmt: skip

    def to_dict(self) -> dict:
        router = {"experts": self.experts, "top": self.top, "scale": self.scale}
        if self.groups > 1:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": router}


@dataclass(frozen=True)
class NatatarLayer:
    type: str  # "attention", "parallel" or "channel_delta"
    mixer: object
    mlp: object  # NatatarExperts or None


@dataclass(frozen=True)
class NatatarConfig:
    """A Natatar decoder: pre-norm layers over several residual streams that every sublayer reads as one weighted
    sum and writes back through a mixing matrix; norms whose gains are stored around zero; mixers of three kinds
    (a biased softmax attention that may mix its values with an earlier layer's, a rotary gated attention beside a
    matrix memory, a delta rule with decays per key channel); feed-forwards of experts chosen within the best
    groups; the embedding table, scaled on the way in, is also the head."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple  # of NatatarLayer
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    streams: int = 0  # 0: one stream and plain residual sums

    architecture = "Natatar"
    MIXERS = ("attention", "parallel", "channel_delta")

    @classmethod
    def from_dict(cls, raw: dict) -> "NatatarConfig":
        _require(raw, ["vocab", "width", "layers", "norm"])
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            mixer = _need(entry, "mixer", where)
            if kind == "attention":
                mixer = NatatarAttention.from_dict(mixer, where + "mixer.")
            elif kind == "parallel":
                mixer = NatatarParallel.from_dict(mixer, where + "mixer.")
            elif kind == "channel_delta":
                mixer = NatatarChannelDelta.from_dict(mixer, where + "mixer.")
            else:
                raise ConfigError(f"{where}type={kind!r} is not supported (one of {', '.join(cls.MIXERS)})")
            mlp = entry.get("mlp")
            layers.append(NatatarLayer(kind, mixer, None if mlp is None else NatatarExperts.from_dict(mlp, where + "mlp.")))
        cfg = cls(
            vocab_size=int(raw["vocab"]),
            hidden_size=int(raw["width"]),
            norm_eps=float(_need(raw["norm"], "eps", "norm.")),
            layers=tuple(layers),
            residual_mult=float(raw.get("residual_mult", 1.0)),
            embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
            streams=int(raw.get("streams") or 0),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size < 1 or self.hidden_size < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.streams < 0:
            raise ConfigError("streams is not negative")
        mixed = None
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            for a in ([m] if layer.type == "attention" else [m.left] if layer.type == "parallel" else []):
                if min(a.heads, a.kv_heads, a.dim, a.vdim) < 1 or a.heads % a.kv_heads:
                    raise ConfigError(f"layers[{i}]: head counts and sizes must be positive, heads a multiple of kv_heads")
                if a.rot and (a.rot[0] < 2 or a.rot[0] % 2 or a.rot[0] > a.dim or not a.rot[1] > 1):
                    raise ConfigError(f"layers[{i}]: rot.dims is even and at most dim, rot.base exceeds 1")
            if layer.type == "attention" and m.v_mix:
                if mixed is not None and mixed.kv_heads * mixed.vdim != m.kv_heads * m.vdim:
                    raise ConfigError(f"layers[{i}]: layers that mix values have value projections of one size")
                mixed = mixed or m
            if layer.type == "parallel" and min(m.right.heads, m.right.dim, m.right.vdim) < 1:
                raise ConfigError(f"layers[{i}]: the memory's head count and sizes must be positive")
            if layer.type == "parallel" and not m.right.gate_cap > 0:
                raise ConfigError(f"layers[{i}]: gate_cap must be positive")
            if layer.type == "channel_delta":
                if min(m.heads, m.kv_heads, m.dim, m.vdim, m.conv) < 1 or m.heads % m.kv_heads:
                    raise ConfigError(f"layers[{i}]: head counts and sizes must be positive, heads a multiple of kv_heads")
            f = layer.mlp
            if f is not None:
                if f.ff < 1 or not 1 <= f.top <= f.experts:
                    raise ConfigError(f"layers[{i}].mlp: sizes must be positive and top at most the number of experts")
                if f.groups < 1 or f.experts % f.groups or not 1 <= f.keep <= f.groups or f.keep * (f.experts // f.groups) < f.top:
                    raise ConfigError(f"layers[{i}].mlp: experts divide into equal groups, and the kept groups hold at least top experts")

    def completed(self, shape_of) -> "NatatarConfig":
        """This configuration with the sizes that only tensors tell: shape_of(checkpoint name) -> shape or None."""
        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if layer.type == "channel_delta":
                a1, g1 = shape_of(f"l{i}.mix.a1"), shape_of(f"l{i}.mix.g1")
                m = replace(m, decay_rank=int(a1[0]) if a1 else m.decay_rank, gate_rank=int(g1[0]) if g1 else m.gate_rank)
            layers.append(replace(layer, mixer=m))
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to this object."""
        layers = [{"type": layer.type, "mixer": layer.mixer.to_dict(), "mlp": None if layer.mlp is None else layer.mlp.to_dict()}
                  for layer in self.layers]  # fmt: skip
        raw = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
               "embedding": {"scale": self.embedding_scale}, "layers": layers}  # fmt: skip
        if self.streams:
            raw["streams"] = self.streams
        return raw
