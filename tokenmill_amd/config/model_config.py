"""Typed model configuration read from the architecture's own config.json keys.

Keys, fall-backs and the order in which end-of-sequence ids are collected follow the reference's
ModelConfig.from_pretrained_dir (reference src/infer/config.py:41-69).  Nothing here carries a
model size: a key without a fall-back in the reference is required.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value the engine cannot run."""


def _require(raw: dict, key: str):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json has no '{key}'")
    return raw[key]


def collect_eos_ids(sources: list[dict]) -> tuple[int, ...]:
    """Ordered union of ``eos_token_id`` (int or list) over the given dicts
    (reference src/infer/config.py:45-53: generation_config.json first, then config.json)."""
    eos: list[int] = []
    for source in sources:
        val = source.get("eos_token_id")
        if val is None:
            continue
        for tok in val if isinstance(val, list) else [val]:
            if int(tok) not in eos:
                eos.append(int(tok))
    return tuple(eos)


@dataclass(frozen=True)
class Qwen2Config:
    """The Qwen2 / Qwen2.5 dense decoder (reference src/infer/config.py:13-39)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Qwen2ForCausalLM"

    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "Qwen2Config":
        heads = int(_require(raw, "num_attention_heads"))
        hidden = int(_require(raw, "hidden_size"))
        rope_theta = raw.get("rope_theta")
        if rope_theta is None:          # newer writers nest it (reference src/infer/config.py:54-56)
            rope_theta = (raw.get("rope_parameters") or {}).get("rope_theta", 10000.0)
        head_dim = raw.get("head_dim")
        if head_dim is None:            # derived when absent (reference src/infer/config.py:29-31)
            if hidden % heads:
                raise ConfigError(f"hidden_size {hidden} is not a multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        cfg = cls(
            vocab_size=int(_require(raw, "vocab_size")),
            hidden_size=hidden,
            intermediate_size=int(_require(raw, "intermediate_size")),
            num_hidden_layers=int(_require(raw, "num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            rope_theta=float(rope_theta),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]),
        )
        cfg.validate(raw)
        return cfg

    def validate(self, raw: dict | None = None) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")
        raw = raw or {}
        # The reference's model keeps every key and knows one activation and one rotary table;
        # a checkpoint that asks for something else must not run silently as if it did not.
        if raw.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not supported by the Qwen2 model of this engine")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act '{raw.get('hidden_act')}' is not supported (silu only)")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("rope_scaling is not supported")

    def to_json_dict(self) -> dict:
        """config.json contents that read back to this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


@dataclass(frozen=True)
class ModinexLayer:
    """One entry of a Modinex model's list of layers."""
    type: str                                  # "attention" | "gla"
    mixer: dict                                # the mixer's sizes and constants, as config.json gives them
    ff: int | None                             # width of the dense feed-forward; None: the layer has none


@dataclass(frozen=True)
class ModinexConfig:
    """The Modinex decoder: token embedding plus a learned position table; layers that each name their mixer
    (sigmoid attention in chunks, or gated linear attention) and may have a dense feed-forward; a norm in groups
    before and behind every sublayer. Every size and constant that can differ between two models of the design is
    read here from config.json; sizes it does not give (the width of the narrow projection in front of a gla
    mixer's decays) come from the checkpoint's tensors."""

    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    norm_eps: float
    norm_groups: int
    layers: tuple[ModinexLayer, ...]
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Modinex"
    MIXERS = ("attention", "gla")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "ModinexConfig":
        norm = _require(raw, "norm")
        layers = []
        for i, entry in enumerate(_require(raw, "layers")):
            kind = entry.get("type")
            if kind not in cls.MIXERS:
                raise ConfigError(f"layers[{i}]: type '{kind}' is not one of {list(cls.MIXERS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"layers[{i}] has no 'mixer' sizes")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"layers[{i}]: feed-forward kind '{mlp.get('kind')}' is not supported (dense only)")
                if "ff" not in mlp:
                    raise ConfigError(f"layers[{i}]: the feed-forward has no 'ff' width")
            need = ("heads", "dim", "vdim") + (("scale",) if kind == "attention" else ("tau",))
            for key in need:
                if mixer.get(key) is None:
                    raise ConfigError(f"layers[{i}]: the {kind} mixer has no '{key}'")
            layers.append(ModinexLayer(kind, dict(mixer), int(mlp["ff"]) if mlp is not None else None))
        cfg = cls(vocab_size=int(_require(raw, "vocab")), hidden_size=int(_require(raw, "width")),
                  max_position_embeddings=int(_require(raw, "max_positions")), norm_eps=float(_require(norm, "eps")),
                  norm_groups=int(norm.get("groups", 1)), layers=tuple(layers),
                  eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "max_position_embeddings", "norm_groups"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.hidden_size % self.norm_groups:
            raise ConfigError(f"norm.groups {self.norm_groups} does not divide the width {self.hidden_size}")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            for key in ("heads", "dim", "vdim"):
                if int(m[key]) <= 0:
                    raise ConfigError(f"layers[{i}]: {key} must be positive")
            if layer.type == "attention":
                kv = int(m.get("kv_heads") or m["heads"])
                if kv <= 0 or int(m["heads"]) % kv:
                    raise ConfigError(f"layers[{i}]: {m['heads']} heads do not divide into {kv} kv heads")
                rot = m.get("rot")
                if rot:
                    dims = int(rot.get("dims", 0))
                    if dims < 0 or dims % 2 or dims > int(m["dim"]):
                        raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most dim {m['dim']}")
                    if dims and not float(rot.get("base", 0)) > 0:
                        raise ConfigError(f"layers[{i}]: rot.base must be positive")
                mask = m.get("mask")
                if mask and mask.get("size") is not None and int(mask["size"]) <= 0:
                    raise ConfigError(f"layers[{i}]: mask.size must be positive")
            elif not float(m["tau"]) > 0:
                raise ConfigError(f"layers[{i}]: tau must be positive")
            if layer.ff is not None and layer.ff <= 0:
                raise ConfigError(f"layers[{i}]: ff must be positive")


@dataclass(frozen=True)
class LusolixLayer:
    """One entry of a Lusolix model's list of layers."""
    type: str                                  # "latent_attention"
    mixer: dict                                # the mixer's sizes and constants, as config.json gives them
    mlp: dict | None                           # {"kind": "dense", "ff": F} | {"kind": "moe", "ff": F, "experts": E, "top": k} | None


@dataclass(frozen=True)
class LusolixConfig:
    """The Lusolix decoder: token embedding plus a learned position table; pre-norm layers (layer norm with bias) whose
    sublayers' results are scaled by ``residual_mult`` and gated on their way into the residual stream; a short causal
    convolution of ``canon.taps`` taps in front of every mixer; attention through a shared latent inside a sliding
    window; a dense feed-forward with the PolyNorm activation or experts chosen by a table of the token id; the output
    head is the embedding table. Every size and constant that can differ between two models is read from config.json."""

    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    norm_eps: float
    residual_mult: float
    conv_taps: int
    layers: tuple[LusolixLayer, ...]
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Lusolix"
    MIXERS = ("latent_attention",)
    MLPS = ("dense", "moe")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "LusolixConfig":
        norm = _require(raw, "norm")
        layers = []
        for i, entry in enumerate(_require(raw, "layers")):
            kind = entry.get("type")
            if kind not in cls.MIXERS:
                raise ConfigError(f"layers[{i}]: type '{kind}' is not one of {list(cls.MIXERS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"layers[{i}] has no 'mixer' sizes")
            for key in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale"):
                if mixer.get(key) is None:
                    raise ConfigError(f"layers[{i}]: the {kind} mixer has no '{key}'")
            mlp = entry.get("mlp")
            if mlp is not None:
                how = mlp.get("kind", "dense")
                if how not in cls.MLPS:
                    raise ConfigError(f"layers[{i}]: feed-forward kind '{how}' is not one of {list(cls.MLPS)}")
                if how == "dense":
                    if mlp.get("ff") is None:
                        raise ConfigError(f"layers[{i}]: the feed-forward has no 'ff' width")
                    mlp = {"kind": "dense", "ff": int(mlp["ff"])}
                else:
                    expert, router = mlp.get("expert") or {}, mlp.get("router") or {}
                    for where, key in ((expert, "ff"), (router, "experts"), (router, "top")):
                        if where.get(key) is None:
                            raise ConfigError(f"layers[{i}]: the experts have no '{key}'")
                    mlp = {"kind": "moe", "ff": int(expert["ff"]), "experts": int(router["experts"]), "top": int(router["top"])}
            layers.append(LusolixLayer(kind, dict(mixer), mlp))
        cfg = cls(vocab_size=int(_require(raw, "vocab")), hidden_size=int(_require(raw, "width")),
                  max_position_embeddings=int(_require(raw, "max_positions")), norm_eps=float(_require(norm, "eps")),
                  residual_mult=float(raw.get("residual_mult", 1.0)), conv_taps=int((raw.get("canon") or {}).get("taps", 0)),
                  layers=tuple(layers), eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not 0 <= self.conv_taps <= 16:
            raise ConfigError(f"canon.taps {self.conv_taps}: 0 (none) to 16")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            for key in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
                if int(m[key]) <= 0:
                    raise ConfigError(f"layers[{i}]: {key} must be positive")
            if int(m["rot_dim"]) < 0:
                raise ConfigError(f"layers[{i}]: rot_dim must not be negative")
            rot = m.get("rot")
            if rot:
                dims = int(rot.get("dims", 0))
                if dims < 0 or dims % 2 or dims > int(m["rot_dim"]):
                    raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most rot_dim {m['rot_dim']}")
                if dims and not float(rot.get("base", 0)) > 0:
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")
            mask = m.get("mask")
            if mask and mask.get("size") is not None and int(mask["size"]) <= 0:
                raise ConfigError(f"layers[{i}]: mask.size must be positive")
            mlp = layer.mlp
            if mlp is not None:
                if mlp["ff"] <= 0:
                    raise ConfigError(f"layers[{i}]: ff must be positive")
                if mlp["kind"] == "moe" and not 0 < mlp["top"] <= mlp["experts"]:
                    raise ConfigError(f"layers[{i}]: {mlp['top']} of {mlp['experts']} experts")


@dataclass(frozen=True)
class GaboraxLayer:
    """One entry of a Gaborax model's list of layers."""
    type: str                                  # "attention" | "attention_2"
    mixer: dict                                # the mixer's sizes and constants, as config.json gives them
    mlp: dict | None                           # {"ff", "experts", "identity", "top", "shared_ff"} | None


@dataclass(frozen=True)
class GaboraxConfig:
    """The Gaborax decoder: token embedding; layers whose sublayers read the residual stream itself and whose results pass
    an RMS norm (weight stored around zero) and a per-channel layer scale on their way into it; softmax attention with q and
    k normed over the whole projection, in two kinds (``attention``: rotation of half-apart pairs, a gate per head, possibly
    on another layer's keys and values; ``attention_2``: biases, rotation of neighbouring pairs with scaled frequencies,
    capped scores); a feed-forward of routed experts (relu squared, experts that stand for the input, a gated shared
    expert); the output head is the embedding table. Every size and constant that can differ between two models is read
    from config.json; the model has no position limit of its own (``max_positions`` if the file gives one)."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple[GaboraxLayer, ...]
    max_position_embeddings: int | None = None
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Gaborax"
    MIXERS = ("attention", "attention_2")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "GaboraxConfig":
        norm = _require(raw, "norm")
        layers = []
        for i, entry in enumerate(_require(raw, "layers")):
            kind = entry.get("type")
            if kind not in cls.MIXERS:
                raise ConfigError(f"layers[{i}]: type '{kind}' is not one of {list(cls.MIXERS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"layers[{i}] has no 'mixer' sizes")
            for key in ("heads", "dim", "vdim", "scale"):
                if mixer.get(key) is None:
                    raise ConfigError(f"layers[{i}]: the {kind} mixer has no '{key}'")
            mlp = entry.get("mlp")
            if mlp is not None:
                how = mlp.get("kind", "moe")
                if how != "moe":
                    raise ConfigError(f"layers[{i}]: feed-forward kind '{how}' is not 'moe'")
                expert, router, shared = mlp.get("expert") or {}, mlp.get("router") or {}, mlp.get("shared")
                for where, key in ((router, "experts"), (router, "top")):
                    if where.get(key) is None:
                        raise ConfigError(f"layers[{i}]: the experts have no '{key}'")
                if int(router["experts"]) > 0 and expert.get("ff") is None:
                    raise ConfigError(f"layers[{i}]: the experts have no 'ff' width")
                mlp = {"ff": int(expert.get("ff") or 0), "experts": int(router["experts"]), "identity": int(router.get("identity") or 0),
                       "top": int(router["top"]), "shared_ff": int(shared["ff"]) if shared and shared.get("ff") else None}
            layers.append(GaboraxLayer(kind, dict(mixer), mlp))
        most = raw.get("max_positions")
        cfg = cls(vocab_size=int(_require(raw, "vocab")), hidden_size=int(_require(raw, "width")), norm_eps=float(_require(norm, "eps")),
                  layers=tuple(layers), max_position_embeddings=int(most) if most is not None else None,
                  eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.max_position_embeddings is not None and self.max_position_embeddings <= 0:
            raise ConfigError("max_positions must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            for key in ("heads", "dim", "vdim"):
                if int(m[key]) <= 0:
                    raise ConfigError(f"layers[{i}]: {key} must be positive")
            heads, kv = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
            if kv <= 0 or heads % kv:
                raise ConfigError(f"layers[{i}]: {heads} heads do not divide into {kv} kv_heads")
            rot = m.get("rot")
            if rot:
                dims = int(rot.get("dims", 0))
                if dims < 0 or dims % 2 or dims > int(m["dim"]):
                    raise ConfigError(f"layers[{i}]: rot.dims {dims} must be even and at most dim {m['dim']}")
                if dims and not float(rot.get("base", 0)) > 0:
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")
                sc = rot.get("scaling")
                if sc:
                    for key in ("factor", "original", "fast", "slow"):
                        if sc.get(key) is None or not float(sc[key]) > 0:
                            raise ConfigError(f"layers[{i}]: rot.scaling.{key} must be positive")
            if m.get("softcap") is not None and not float(m["softcap"]) > 0:
                raise ConfigError(f"layers[{i}]: softcap must be positive")
            src = m.get("kv_from")
            if src is not None:
                if layer.type != "attention":
                    raise ConfigError(f"layers[{i}]: only an 'attention' mixer reads another layer's keys and values")
                src = int(src)
                if not 0 <= src < i or self.layers[src].mixer.get("kv_from") is not None:
                    raise ConfigError(f"layers[{i}]: kv_from must name an earlier layer that has keys and values of its own")
                other = self.layers[src].mixer
                same = all(int(other.get(k) or other["heads"]) == int(m.get(k) or m["heads"]) for k in ("kv_heads",)) and \
                    all(int(other[k]) == int(m[k]) for k in ("heads", "dim", "vdim")) and (other.get("rot") or {}) == (m.get("rot") or {})
                if not same:
                    raise ConfigError(f"layers[{i}]: layer {src}'s head counts, sizes and rotation must equal this layer's")
            mlp = layer.mlp
            if mlp is not None:
                if mlp["experts"] < 0 or mlp["identity"] < 0 or not 0 < mlp["top"] <= mlp["experts"] + mlp["identity"]:
                    raise ConfigError(f"layers[{i}]: {mlp['top']} of {mlp['experts']} + {mlp['identity']} experts")
                if mlp["experts"] and mlp["ff"] <= 0:
                    raise ConfigError(f"layers[{i}]: expert.ff must be positive")
                if mlp["shared_ff"] is not None and mlp["shared_ff"] <= 0:
                    raise ConfigError(f"layers[{i}]: shared.ff must be positive")


@dataclass(frozen=True)
class LuzevikLayer:
    type: str                       # "latent_attention" | "parallel"
    mixer: dict                     # the mixer's sizes and constants, as config.json gives them
    mlp: dict | None                # {"kind": "dense", "ff"} | {"kind": "moe", "ff", "experts", "top"} | None


@dataclass
class LuzevikConfig:
    """The Luzevik decoder: token embedding times a constant; layers whose sublayers read the residual stream itself and whose
    results pass an RMS norm (plain weight) on their way into it; a mixer that is either attention through a shared latent
    (queries through a latent of their own, rotation of pairs half the rotated width apart, a sink per head in the softmax,
    possibly on another layer's cached rows) or two mixers side by side, softmax attention over grouped heads (biases,
    per-head norm of q and k, linearly scaled rotation) and a gated delta rule behind short convolutions; a feed-forward
    that is dense with a tanh-GELU gate or a set of routed SwiGLU experts (router with a bias, softmax over the chosen
    logits); the output head is the embedding table. Every size and constant that can differ between two models is read
    from config.json; the model has no position limit of its own (``max_positions`` if the file gives one)."""

    vocab_size: int
    hidden_size: int
    norm_eps: float
    embedding_scale: float
    layers: tuple[LuzevikLayer, ...]
    max_position_embeddings: int | None = None
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Luzevik"
    MIXERS = ("latent_attention", "parallel")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "LuzevikConfig":
        norm = _require(raw, "norm")
        layers = []
        for i, entry in enumerate(_require(raw, "layers")):
            kind = entry.get("type")
            if kind not in cls.MIXERS:
                raise ConfigError(f"layers[{i}]: type '{kind}' is not one of {list(cls.MIXERS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"layers[{i}] has no 'mixer' sizes")
            if kind == "latent_attention":
                wanted = [(mixer, k, "latent attention") for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale")]
            else:
                left, right = mixer.get("left"), mixer.get("right")
                if not isinstance(left, dict) or not isinstance(right, dict):
                    raise ConfigError(f"layers[{i}]: a parallel mixer has 'left' and 'right' sizes")
                wanted = [(left, k, "left mixer") for k in ("heads", "kv_heads", "dim", "vdim", "scale")] + \
                    [(right, k, "right mixer") for k in ("heads", "kv_heads", "dim", "vdim", "conv")]
            for where, key, what in wanted:
                if where.get(key) is None:
                    raise ConfigError(f"layers[{i}]: the {what} has no '{key}'")
            mlp = entry.get("mlp")
            if mlp is not None:
                how = mlp.get("kind")
                if how == "dense":
                    if mlp.get("ff") is None:
                        raise ConfigError(f"layers[{i}]: the dense feed-forward has no 'ff' width")
                    mlp = {"kind": "dense", "ff": int(mlp["ff"])}
                elif how == "moe":
                    expert, router = mlp.get("expert") or {}, mlp.get("router") or {}
                    for where, key in ((expert, "ff"), (router, "experts"), (router, "top")):
                        if where.get(key) is None:
                            raise ConfigError(f"layers[{i}]: the experts have no '{key}'")
                    mlp = {"kind": "moe", "ff": int(expert["ff"]), "experts": int(router["experts"]), "top": int(router["top"])}
                else:
                    raise ConfigError(f"layers[{i}]: feed-forward kind '{how}' is not 'dense' or 'moe'")
            layers.append(LuzevikLayer(kind, dict(mixer), mlp))
        most = raw.get("max_positions")
        cfg = cls(vocab_size=int(_require(raw, "vocab")), hidden_size=int(_require(raw, "width")), norm_eps=float(_require(norm, "eps")),
                  embedding_scale=float(_require(_require(raw, "embedding"), "scale")), layers=tuple(layers),
                  max_position_embeddings=int(most) if most is not None else None,
                  eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]))
        cfg.validate()
        return cfg

    @staticmethod
    def _check_rot(i: int, where: str, rot: dict | None, most: int, scaled: bool) -> None:
        if not rot:
            return
        dims = int(rot.get("dims", 0))
        if dims < 0 or dims % 2 or dims > most:
            raise ConfigError(f"layers[{i}]: {where} rot.dims {dims} must be even and at most {most}")
        if dims and not float(rot.get("base", 0)) > 0:
            raise ConfigError(f"layers[{i}]: {where} rot.base must be positive")
        sc = rot.get("scaling")
        if sc:
            if not scaled:
                raise ConfigError(f"layers[{i}]: {where} rotation has no scaling")
            if sc.get("factor") is None or not float(sc["factor"]) > 0:
                raise ConfigError(f"layers[{i}]: {where} rot.scaling.factor must be positive")

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.max_position_embeddings is not None and self.max_position_embeddings <= 0:
            raise ConfigError("max_positions must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if layer.type == "latent_attention":
                for key in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
                    if int(m[key]) <= 0:
                        raise ConfigError(f"layers[{i}]: {key} must be positive")
                if int(m["rot_dim"]) < 0:
                    raise ConfigError(f"layers[{i}]: rot_dim must not be negative")
                self._check_rot(i, "the", m.get("rot"), int(m["rot_dim"]), scaled=False)
                src = m.get("kv_from")
                if src is not None:
                    src = int(src)
                    if not 0 <= src < i or self.layers[src].type != "latent_attention" or self.layers[src].mixer.get("kv_from") is not None:
                        raise ConfigError(f"layers[{i}]: kv_from must name an earlier latent-attention layer that has a latent of its own")
                    other = self.layers[src].mixer
                    if any(int(other[k]) != int(m[k]) for k in ("kv_rank", "rot_dim")) or (other.get("rot") or {}) != (m.get("rot") or {}):
                        raise ConfigError(f"layers[{i}]: layer {src}'s kv_rank, rot_dim and rotation must equal this layer's")
            else:
                for side in ("left", "right"):
                    part = m[side]
                    for key in ("heads", "kv_heads", "dim", "vdim"):
                        if int(part[key]) <= 0:
                            raise ConfigError(f"layers[{i}]: {side}.{key} must be positive")
                    if int(part["heads"]) % int(part["kv_heads"]):
                        raise ConfigError(f"layers[{i}]: {side}: {part['heads']} heads do not divide into {part['kv_heads']} kv_heads")
                self._check_rot(i, "left", m["left"].get("rot"), int(m["left"]["dim"]), scaled=True)
                if int(m["right"]["conv"]) < 1:
                    raise ConfigError(f"layers[{i}]: right.conv must be at least 1")
            mlp = layer.mlp
            if mlp is not None:
                if mlp["ff"] <= 0:
                    raise ConfigError(f"layers[{i}]: the feed-forward's ff must be positive")
                if mlp["kind"] == "moe" and not 0 < mlp["top"] <= mlp["experts"]:
                    raise ConfigError(f"layers[{i}]: {mlp['top']} of {mlp['experts']} experts")


def read_json(path: Path) -> dict:
    try:
        return json.loads(path.read_text())
    except FileNotFoundError:
        raise ConfigError(f"{path} does not exist") from None
