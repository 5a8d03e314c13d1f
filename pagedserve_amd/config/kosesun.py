"""Typed Kosesun configuration, read from the keys of its ``config.json``.

A Kosesun model lists its layers one by one: each names its mixer (``attention`` or ``gla``)
with the mixer's own sizes and constants, and its feed-forward (or none).  The residual stream
may be kept in several copies (``streams``).  Every size and constant comes from the file; the
rank of the decay's low-rank projection is the one size that only the tensors give, and the
loader reads it from there (``decay_rank`` may name it in the file).
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, require_int

MIXERS = ("attention", "gla")


def _number(raw, key, where, positive=True):
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json {where} '{key}' must be a number, got {value!r}")
    if positive and not value > 0:
        raise ConfigError(f"config.json {where} '{key}' must be positive, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class KosesunAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    v_mix: bool

    def to_dict(self):
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale, "v_mix": self.v_mix}
        if self.rot_dims:
            out["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        return out


@dataclass(frozen=True)
class KosesunGLA:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int] = None     # None: read from the tensor's shape

    def to_dict(self):
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        return out


@dataclass(frozen=True)
class KosesunLayer:
    type: str
    mixer: object
    ff: Optional[int]          # inner width of the dense feed-forward, None: no feed-forward

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class KosesunConfig:
    vocab: int
    width: int
    layers: Tuple[KosesunLayer, ...]
    norm_eps: float
    embedding_scale: float
    logit_softcap: float       # 0: none
    streams: int               # 0: one plain residual stream
    max_positions: int

    architecture = "Kosesun"
    eos_token_id = None        # the configuration names no token that ends a request

    @property
    def vocab_size(self) -> int:
        return self.vocab
    # positions have no bound of their own (rotations).  Where the file names none, requests may
    # grow to this many tokens (block tables of 2,048 pages of 16, the widest that the tiled
    # attention kernel keeps); an engine's pool or its own bound may be smaller.
    DEFAULT_MAX_POSITIONS = 32768

    @classmethod
    def from_dict(cls, raw) -> "KosesunConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json 'layers' must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXERS:
                raise ConfigError(f"config.json {where} 'type' must be one of {', '.join(MIXERS)}, "
                                  f"got {entry.get('type') if isinstance(entry, dict) else entry!r}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"config.json {where} lacks 'mixer'")
            try:
                if entry["type"] == "attention":
                    heads = require_int(mixer, "heads")
                    kv_heads = require_int(mixer, "kv_heads", default=heads)
                    if heads % kv_heads:
                        raise ConfigError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
                    dim = require_int(mixer, "dim")
                    rot = mixer.get("rot") or {}
                    rot_dims = require_int(rot, "dims", default=0, minimum=0)
                    if rot_dims % 2 or rot_dims > dim:
                        raise ConfigError(f"rot.dims ({rot_dims}) must be even and at most dim ({dim})")
                    built = KosesunAttention(
                        heads=heads, kv_heads=kv_heads, dim=dim,
                        vdim=require_int(mixer, "vdim", default=dim),
                        scale=_number(mixer, "scale", where + ".mixer"),
                        rot_dims=rot_dims,
                        rot_base=_number(rot, "base", where + ".mixer.rot") if rot_dims else 10000.0,
                        v_mix=bool(mixer.get("v_mix", False)))
                else:
                    rank = mixer.get("decay_rank")
                    built = KosesunGLA(
                        heads=require_int(mixer, "heads"), dim=require_int(mixer, "dim"),
                        vdim=require_int(mixer, "vdim"), tau=_number(mixer, "tau", where + ".mixer"),
                        decay_rank=None if rank is None else require_int(mixer, "decay_rank"))
            except ConfigError as error:
                raise ConfigError(f"{where}: {error}") from None
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json {where} 'mlp.kind' must be 'dense', got {mlp!r}")
                ff = require_int(mlp, "ff")
            layers.append(KosesunLayer(entry["type"], built, ff))
        sources = [layer.mixer for layer in layers if layer.type == "attention" and layer.mixer.v_mix]
        for mixer in sources[1:]:
            if (mixer.kv_heads, mixer.vdim) != (sources[0].kv_heads, sources[0].vdim):
                raise ConfigError("layers that mix values must agree in kv_heads and vdim")
        norm = raw.get("norm") or {}
        embedding = raw.get("embedding") or {}
        softcap = raw.get("logit_softcap")
        return cls(
            vocab=require_int(raw, "vocab"),
            width=require_int(raw, "width"),
            layers=tuple(layers),
            norm_eps=_number(norm, "eps", "norm"),
            embedding_scale=_number(embedding, "scale", "embedding") if "scale" in embedding else 1.0,
            logit_softcap=0.0 if softcap is None else _number(raw, "logit_softcap", ""),
            streams=require_int(raw, "streams", default=0, minimum=0),
            max_positions=require_int(raw, "max_positions", default=cls.DEFAULT_MAX_POSITIONS),
        )

    def to_dict(self) -> dict:
        out = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "layers": [layer.to_dict() for layer in self.layers],
            "norm": {"eps": self.norm_eps},
            "embedding": {"scale": self.embedding_scale},
        }
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.streams:
            out["streams"] = self.streams
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    def with_decay_ranks(self, rank_of) -> "KosesunConfig":
        """This configuration with every unknown decay rank taken from ``rank_of(layer index)``."""
        layers = []
        for index, layer in enumerate(self.layers):
            if layer.type == "gla" and layer.mixer.decay_rank is None:
                mixer = KosesunGLA(layer.mixer.heads, layer.mixer.dim, layer.mixer.vdim, layer.mixer.tau,
                                   int(rank_of(index)))
                layer = KosesunLayer(layer.type, mixer, layer.ff)
            layers.append(layer)
        return KosesunConfig(self.vocab, self.width, tuple(layers), self.norm_eps, self.embedding_scale,
                             self.logit_softcap, self.streams, self.max_positions)
