"""Typed configuration of the Fanotar decoder, read from the keys of its config.json: a scale on the
embedding, a list of layers, each with an attention mixer of its own sizes and constants and an
optional feed-forward (dense, or a mixture of experts with an optional shared expert), and the eps of
the heads' norms. A layer may name another layer whose keys and values it reads instead of making its
own. Every size and constant of a model stands here and nowhere else."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from tinyserve_llm_amd.config.llama import ConfigError


def _need(raw: Mapping[str, Any], key: str, where: str) -> Any:
    if not isinstance(raw, Mapping) or key not in raw or raw[key] is None:
        raise ConfigError(f"config.json lacks the required key {key!r} in {where}")
    return raw[key]


@dataclass(frozen=True)
class FanotarAttention:
    heads: int
    kv_heads: int
    dim: int                     # size of a query / key head
    vdim: int                    # size of a value head
    conv: int                    # taps of the short convolution on q, k and v (1: a weight per channel, no past)
    window: int                  # keys a position sees, itself included (0: all)
    scale: float
    q_temp_coef: float           # q times 1 + coef ln(floor((p + 1) / every) + 1); coef 0: not
    q_temp_every: int
    kv_from: int | None = None   # the layer whose keys and values this one reads (None: its own)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FanotarAttention":
        mask, temp = raw.get("mask"), raw.get("q_temp")
        kv_from = raw.get("kv_from")
        c = cls(heads=int(_need(raw, "heads", where)), kv_heads=int(_need(raw, "kv_heads", where)),
                dim=int(_need(raw, "dim", where)), vdim=int(_need(raw, "vdim", where)), conv=int(_need(raw, "conv", where)),
                window=int(_need(mask, "size", where + ".mask")) if mask else 0, scale=float(_need(raw, "scale", where)),
                q_temp_coef=float(_need(temp, "coef", where + ".q_temp")) if temp else 0.0,
                q_temp_every=int(_need(temp, "every", where + ".q_temp")) if temp else 1,
                kv_from=None if kv_from is None else int(kv_from))
        if c.heads <= 0 or c.kv_heads <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}.kv_heads: {c.heads} heads do not divide into {c.kv_heads} key/value heads")
        if c.dim <= 0 or c.vdim <= 0:
            raise ConfigError(f"{where}: dim and vdim are positive")
        if c.conv < 1:
            raise ConfigError(f"{where}.conv {c.conv}: at least one tap")
        if c.window < 0 or (mask and c.window < 1):
            raise ConfigError(f"{where}.mask.size {c.window}: a positive number of keys")
        if c.q_temp_every < 1:
            raise ConfigError(f"{where}.q_temp.every {c.q_temp_every}: at least 1")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                               "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        if self.window:
            out["mask"] = {"size": self.window}
        if self.q_temp_coef:
            out["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return out


@dataclass(frozen=True)
class FanotarGatedUnit:
    """A gated feed-forward of width `ff` whose branches are capped at `limit`."""
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FanotarGatedUnit":
        c = cls(ff=int(_need(raw, "ff", where)), limit=float(_need(raw, "limit", where)))
        if c.ff <= 0 or c.limit <= 0:
            raise ConfigError(f"{where}: ff and limit are positive")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class FanotarExperts:
    experts: int
    top: int
    scale: float                 # on the chosen experts' normalised weights
    expert: FanotarGatedUnit
    shared: FanotarGatedUnit | None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FanotarExperts":
        router = _need(raw, "router", where)
        c = cls(experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
                scale=float(_need(router, "scale", where + ".router")),
                expert=FanotarGatedUnit.from_dict(_need(raw, "expert", where), where + ".expert"),
                shared=FanotarGatedUnit.from_dict(raw["shared"], where + ".shared") if raw.get("shared") else None)
        if not 1 <= c.top <= c.experts:
            raise ConfigError(f"{where}.router.top {c.top}: between 1 and the {c.experts} experts")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"expert": self.expert.to_dict(), "kind": "moe",
                "router": {"experts": self.experts, "scale": self.scale, "top": self.top},
                "shared": None if self.shared is None else self.shared.to_dict()}


@dataclass(frozen=True)
class FanotarLayer:
    mixer: FanotarAttention
    mlp: "FanotarGatedUnit | FanotarExperts | None"      # dense, a mixture of experts, or none
    type: str = "attention"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FanotarLayer":
        kind = _need(raw, "type", where)
        if kind != "attention":
            raise ConfigError(f"{where}.type {kind!r}: this decoder's mixer is 'attention'")
        mixer = FanotarAttention.from_dict(_need(raw, "mixer", where), where + ".mixer")
        mlp = raw.get("mlp")
        if mlp is not None:
            which = _need(mlp, "kind", where + ".mlp")
            if which == "dense":
                mlp = FanotarGatedUnit.from_dict(mlp, where + ".mlp")
            elif which == "moe":
                mlp = FanotarExperts.from_dict(mlp, where + ".mlp")
            else:
                raise ConfigError(f"{where}.mlp.kind {which!r}: 'dense' or 'moe'")
        return cls(mixer, mlp, kind)

    def to_dict(self) -> dict[str, Any]:
        mlp = None if self.mlp is None else self.mlp.to_dict()
        if isinstance(self.mlp, FanotarGatedUnit):
            mlp["kind"] = "dense"
        return {"mixer": self.mixer.to_dict(), "mlp": mlp, "type": self.type}


@dataclass(frozen=True)
class FanotarConfig:
    vocab: int
    width: int
    layers: tuple[FanotarLayer, ...]
    norm_eps: float
    embedding_scale: float = 1.0
    architecture: str = "Fanotar"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FanotarConfig":
        layers = tuple(FanotarLayer.from_dict(l, f"layers[{i}]") for i, l in enumerate(_need(raw, "layers", "config.json")))
        if not layers:
            raise ConfigError("layers: the model has at least one")
        for i, layer in enumerate(layers):
            j, m = layer.mixer.kv_from, layer.mixer
            if j is None:
                continue
            if not 0 <= j < i:
                raise ConfigError(f"layers[{i}].mixer.kv_from {j}: a layer before this one")
            o = layers[j].mixer
            if o.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from {j}: that layer has no keys and values of its own")
            if (o.kv_heads, o.dim, o.vdim) != (m.kv_heads, m.dim, m.vdim):
                raise ConfigError(f"layers[{i}].mixer.kv_from {j}: key/value heads and sizes of the two layers differ")
        embedding = raw.get("embedding") or {}
        return cls(vocab=int(_need(raw, "vocab", "config.json")), width=int(_need(raw, "width", "config.json")), layers=layers,
                   norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
                   embedding_scale=float(embedding.get("scale", 1.0)))

    def to_dict(self) -> dict[str, Any]:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                "width": self.width}
