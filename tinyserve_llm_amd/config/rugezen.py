"""Typed configuration of the Rugezen decoder, read from the keys of its config.json: a list of
layers, each with a mixer of its own kind and sizes ("attention" or "mingru") and an optional dense
feed-forward, a stretch of layers that runs several times in a row with the same weights, one RMS
norm eps, and a multiplier on what a layer adds to the residual stream. Every size and constant of
a model stands here and nowhere else."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from tinyserve_llm_amd.config.llama import ConfigError


def _need(raw: Mapping[str, Any], key: str, where: str) -> Any:
    if not isinstance(raw, Mapping) or key not in raw or raw[key] is None:
        raise ConfigError(f"config.json lacks the required key {key!r} in {where}")
    return raw[key]


@dataclass(frozen=True)
class RugezenAttention:
    heads: int
    kv_heads: int
    dim: int                 # size of a query / key head
    vdim: int                # size of a value head
    rot_dims: int            # leading dimensions of a head that turn, in interleaved pairs
    rot_base: float
    scale: float
    softcap: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "RugezenAttention":
        rot = _need(raw, "rot", where)
        c = cls(heads=int(_need(raw, "heads", where)), kv_heads=int(_need(raw, "kv_heads", where)),
                dim=int(_need(raw, "dim", where)), vdim=int(_need(raw, "vdim", where)),
                rot_dims=int(_need(rot, "dims", where + ".rot")), rot_base=float(_need(rot, "base", where + ".rot")),
                scale=float(_need(raw, "scale", where)), softcap=float(_need(raw, "softcap", where)))
        if c.heads <= 0 or c.kv_heads <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}.kv_heads: {c.heads} heads do not divide into {c.kv_heads} key/value heads")
        if c.rot_dims % 2 or not 0 <= c.rot_dims <= c.dim:
            raise ConfigError(f"{where}.rot.dims {c.rot_dims}: an even number up to dim {c.dim}")
        if c.softcap <= 0:
            raise ConfigError(f"{where}.softcap {c.softcap}: a positive number")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "rot": {"base": self.rot_base, "dims": self.rot_dims}, "scale": self.scale, "softcap": self.softcap,
                "vdim": self.vdim}


@dataclass(frozen=True)
class RugezenMinGRU:
    width: int

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "RugezenMinGRU":
        c = cls(width=int(_need(raw, "width", where)))
        if c.width <= 0:
            raise ConfigError(f"{where}.width {c.width}: a positive number")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"width": self.width}


MIXERS = {"attention": RugezenAttention, "mingru": RugezenMinGRU}


@dataclass(frozen=True)
class RugezenLayer:
    type: str                                    # which mixer: a key of MIXERS
    mixer: "RugezenAttention | RugezenMinGRU"
    ff: int | None                               # width of the dense feed-forward; None: the layer has none

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "RugezenLayer":
        kind = _need(raw, "type", where)
        if kind not in MIXERS:
            raise ConfigError(f"{where}.type {kind!r}: one of {sorted(MIXERS)}")
        mixer = MIXERS[kind].from_dict(_need(raw, "mixer", where), where + ".mixer")
        mlp = raw.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ConfigError(f"{where}.mlp.kind {mlp.get('kind')!r}: this decoder has dense feed-forwards")
            ff = int(_need(mlp, "ff", where + ".mlp"))
        return cls(kind, mixer, ff)

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"}}


@dataclass(frozen=True)
class RugezenConfig:
    vocab: int
    width: int
    layers: tuple[RugezenLayer, ...]
    norm_eps: float
    residual_mult: float = 1.0
    # layers loop_start .. loop_stop - 1 run loop_times times in a row; loop_times 1: every layer once
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    architecture: str = "Rugezen"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "RugezenConfig":
        layers = tuple(RugezenLayer.from_dict(l, f"layers[{i}]") for i, l in enumerate(_need(raw, "layers", "config.json")))
        if not layers:
            raise ConfigError("layers: the model has at least one")
        loop = raw.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            start, stop, times = (int(_need(loop, k, "loop")) for k in ("start", "stop", "times"))
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"loop {dict(loop)}: 0 <= start <= stop <= {len(layers)} layers, times >= 1")
        return cls(vocab=int(_need(raw, "vocab", "config.json")), width=int(_need(raw, "width", "config.json")), layers=layers,
                   norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
                   residual_mult=float(_need(raw, "residual_mult", "config.json")), loop_start=start, loop_stop=stop,
                   loop_times=times)

    def to_dict(self) -> dict[str, Any]:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times},
                "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}

    def run_order(self) -> list[int]:
        """Layer indices in the order they run: the looped stretch `loop_times` times in a row."""
        n = len(self.layers)
        stretch = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + stretch * self.loop_times + list(range(self.loop_stop, n))
