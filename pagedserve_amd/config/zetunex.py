"""Typed Zetunex configuration, read from the keys of its ``config.json``.

A Zetunex model lists its layers one by one: each names its mixer (``lightning`` or
``parallel``) with the mixer's own sizes and constants, and its feed-forward (``dense``,
``moe`` or none).  ``loop`` names a run of layers that is passed several times with the same
weights, ``residual_mult`` the factor on what a layer adds to the stream.  Every size and
constant comes from the file.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, require_int

MIXERS = ("lightning", "parallel")


def _number(raw, key, where, positive=True):
    value = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json {where} '{key}' must be a number, got {value!r}")
    if positive and not value > 0:
        raise ConfigError(f"config.json {where} '{key}' must be positive, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class ZetunexLightning:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class ZetunexWindowed:
    """The attention half of a ``parallel`` mixer."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "scale": self.scale, "mask": {"size": self.window}}


@dataclass(frozen=True)
class ZetunexScan:
    """The state-space half of a ``parallel`` mixer."""

    inner: int
    state: int
    dt_rank: int
    conv: int

    def to_dict(self):
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class ZetunexParallel:
    left: ZetunexWindowed
    right: ZetunexScan

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class ZetunexFeedForward:
    kind: str                  # "dense" or "moe"
    ff: int                    # inner width (of every expert)
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    scale: float = 1.0

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "scale": self.scale,
                           "groups": {"count": self.groups, "keep": self.keep}}}


@dataclass(frozen=True)
class ZetunexLayer:
    type: str
    mixer: object
    mlp: Optional[ZetunexFeedForward]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_mixer(kind, mixer, where):
    if kind == "lightning":
        heads = require_int(mixer, "heads")
        decay = mixer.get("decay")
        if (not isinstance(decay, list) or len(decay) != heads
                or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay)):
            raise ConfigError(f"'decay' must list one number per head ({heads}), got {decay!r}")
        return ZetunexLightning(heads=heads, dim=require_int(mixer, "dim"),
                                vdim=require_int(mixer, "vdim"), decay=tuple(float(d) for d in decay))
    left, right = mixer.get("left"), mixer.get("right")
    if not isinstance(left, dict) or not isinstance(right, dict):
        raise ConfigError("a parallel mixer needs 'left' and 'right'")
    heads = require_int(left, "heads")
    kv_heads = require_int(left, "kv_heads", default=heads)
    if heads % kv_heads:
        raise ConfigError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    dim = require_int(left, "dim")
    mask = left.get("mask") or {}
    return ZetunexParallel(
        left=ZetunexWindowed(heads=heads, kv_heads=kv_heads, dim=dim,
                             vdim=require_int(left, "vdim", default=dim),
                             scale=_number(left, "scale", where + ".mixer.left"),
                             window=require_int(mask, "size", default=0, minimum=0)),
        right=ZetunexScan(inner=require_int(right, "inner"), state=require_int(right, "state"),
                          dt_rank=require_int(right, "dt_rank"), conv=require_int(right, "conv")))


def _read_feed_forward(mlp, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind", "dense") not in ("dense", "moe"):
        raise ConfigError(f"config.json {where} 'mlp.kind' must be 'dense' or 'moe', got {mlp!r}")
    if mlp.get("kind", "dense") == "dense":
        return ZetunexFeedForward("dense", require_int(mlp, "ff"))
    router = mlp.get("router")
    expert = mlp.get("expert")
    if not isinstance(router, dict) or not isinstance(expert, dict):
        raise ConfigError(f"config.json {where} 'mlp' of kind moe needs 'router' and 'expert'")
    groups = router.get("groups") or {}
    experts = require_int(router, "experts")
    count = require_int(groups, "count", default=1)
    keep = require_int(groups, "keep", default=count)
    top = require_int(router, "top")
    if experts % count or keep > count or top > (experts // count) * keep:
        raise ConfigError(f"config.json {where}: {experts} experts in {count} groups (keep {keep}) "
                          f"cannot give {top} per token")
    return ZetunexFeedForward(
        "moe", require_int(expert, "ff"), experts=experts, top=top, groups=count, keep=keep,
        scale=_number(router, "scale", where + ".mlp.router") if "scale" in router else 1.0)


@dataclass(frozen=True)
class ZetunexConfig:
    vocab: int
    width: int
    layers: Tuple[ZetunexLayer, ...]
    norm_eps: float
    residual_mult: float
    loop_start: int            # layers loop_start .. loop_stop - 1 run loop_times times in a row
    loop_stop: int
    loop_times: int            # 0: no loop
    max_positions: int

    architecture = "Zetunex"
    eos_token_id = None        # the configuration names no token that ends a request
    # no layer reads positions; where the file names no bound, requests may grow to this many
    # tokens (an engine's pool or its own bound may be smaller)
    DEFAULT_MAX_POSITIONS = 32768

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw) -> "ZetunexConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json 'layers' must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXERS:
                raise ConfigError(f"config.json {where} 'type' must be one of {', '.join(MIXERS)}, "
                                  f"got {entry.get('type') if isinstance(entry, dict) else entry!r}")
            if not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json {where} lacks 'mixer'")
            try:
                mixer = _read_mixer(entry["type"], entry["mixer"], where)
                mlp = _read_feed_forward(entry.get("mlp"), where)
            except ConfigError as error:
                raise ConfigError(f"{where}: {error}") from None
            layers.append(ZetunexLayer(entry["type"], mixer, mlp))
        loop = raw.get("loop")
        start = stop = times = 0
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json 'loop' must be an object")
            start = require_int(loop, "start", minimum=0)
            stop = require_int(loop, "stop")
            times = require_int(loop, "times")
            if not start < stop <= len(layers):
                raise ConfigError(f"config.json 'loop' {start}..{stop} does not lie within the "
                                  f"{len(layers)} layers")
        norm = raw.get("norm") or {}
        return cls(
            vocab=require_int(raw, "vocab"),
            width=require_int(raw, "width"),
            layers=tuple(layers),
            norm_eps=_number(norm, "eps", "norm"),
            residual_mult=_number(raw, "residual_mult", "", positive=False) if "residual_mult" in raw else 1.0,
            loop_start=start, loop_stop=stop, loop_times=times,
            max_positions=require_int(raw, "max_positions", default=cls.DEFAULT_MAX_POSITIONS),
        )

    def to_dict(self) -> dict:
        out = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "layers": [layer.to_dict() for layer in self.layers],
            "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult,
        }
        if self.loop_times:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.max_positions != self.DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    def run_order(self):
        """(layer, number of the pass that this call opens or -1) for every call, in order."""
        count = len(self.layers)
        if not self.loop_times:
            return [(index, -1) for index in range(count)]
        order = [(index, -1) for index in range(self.loop_start)]
        for turn in range(self.loop_times):
            order.extend((index, turn if index == self.loop_start else -1)
                         for index in range(self.loop_start, self.loop_stop))
        order.extend((index, -1) for index in range(self.loop_stop, count))
        return order
