"""Typed configuration of the Tegolix decoder, read from the keys of its config.json: one eps for every norm, the
width of the per-layer token input (`token_side.dim`; absent: none) and a list of layers. A layer names its mixer's
kind ("gla": gated linear attention; "parallel": windowed attention and an RWKV-style recurrence side by side) with the
mixer's sizes and constants, and an optional feed-forward (dense, or a mixture of experts with identity experts and a
shared expert). Every size and constant of a model stands here and nowhere else; the ranks of the low-rank decay
projections are shapes of the checkpoint's tensors and are read from there (`ranks_from`)."""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping

from tinyserve_llm_amd.config.bafarax import Rotation, _need
from tinyserve_llm_amd.config.llama import ConfigError


@dataclass(frozen=True)
class TegolixGLA:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = 32         # inner size of the decays' two projections (the checkpoint's `a1` has that many rows)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "TegolixGLA":
        c = cls(heads=int(_need(raw, "heads", where)), dim=int(_need(raw, "dim", where)), vdim=int(_need(raw, "vdim", where)),
                tau=float(_need(raw, "tau", where)), decay_rank=int(raw.get("decay_rank", 32)))
        if min(c.heads, c.dim, c.vdim, c.decay_rank) <= 0 or not c.tau > 0:
            raise ConfigError(f"{where}: heads, dim, vdim and tau are positive")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"decay_rank": self.decay_rank, "dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}


@dataclass(frozen=True)
class TegolixWindowAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float               # scores are capped as softcap tanh(score / softcap); 0: not
    rot: Rotation                # pairs (i, i + dims/2); its base also turns the values, over all of vdim
    window: int                  # a position sees itself and the window - 1 before it (0: all before it)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "TegolixWindowAttention":
        mask = raw.get("mask") or {}
        c = cls(heads=int(_need(raw, "heads", where)), kv_heads=int(_need(raw, "kv_heads", where)), dim=int(_need(raw, "dim", where)),
                vdim=int(_need(raw, "vdim", where)), scale=float(_need(raw, "scale", where)), softcap=float(raw.get("softcap") or 0.0),
                rot=Rotation.from_dict(_need(raw, "rot", where), where + ".rot"), window=int(mask.get("size", 0)) if mask else 0)
        if c.heads <= 0 or c.kv_heads <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}.kv_heads: {c.heads} heads do not divide into {c.kv_heads} key/value heads")
        if c.dim <= 0 or c.vdim <= 0 or c.vdim % 2 or c.rot.dims > c.dim or c.softcap < 0 or c.window < 0 or (mask and c.window < 1):
            raise ConfigError(f"{where}: dim and an even vdim are positive, rot.dims at most dim, softcap and mask.size not negative")
        if c.rot.base <= 0:
            raise ConfigError(f"{where}.rot.base: positive (it also turns the values)")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "rot": self.rot.to_dict(),
                               "scale": self.scale, "vdim": self.vdim}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.window:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class TegolixRecurrence:
    heads: int
    dim: int
    decay_rank: int = 32         # (the checkpoint's `w1` has that many rows)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "TegolixRecurrence":
        c = cls(heads=int(_need(raw, "heads", where)), dim=int(_need(raw, "dim", where)), decay_rank=int(raw.get("decay_rank", 32)))
        if min(c.heads, c.dim, c.decay_rank) <= 0:
            raise ConfigError(f"{where}: heads and dim are positive")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"decay_rank": self.decay_rank, "dim": self.dim, "heads": self.heads}


@dataclass(frozen=True)
class TegolixParallel:
    left: TegolixWindowAttention
    right: TegolixRecurrence
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "TegolixParallel":
        return cls(TegolixWindowAttention.from_dict(_need(raw, "left", where), where + ".left"),
                   TegolixRecurrence.from_dict(_need(raw, "right", where), where + ".right"),
                   float(_need(raw, "left_scale", where)), float(_need(raw, "right_scale", where)))

    def to_dict(self) -> dict[str, Any]:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(), "right_scale": self.right_scale}


MIXERS = {"gla": TegolixGLA, "parallel": TegolixParallel}


@dataclass(frozen=True)
class TegolixDense:
    ff: int

    def to_dict(self) -> dict[str, Any]:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class TegolixExperts:
    experts: int                 # experts with matrices
    identity: int                # router outputs beyond them, which stand for experts that hand their input through
    top: int
    ff: int                      # width of one expert
    shared_ff: int               # width of the shared expert (0: none)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe",
                               "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _mlp(raw: Mapping[str, Any] | None, where: str) -> "TegolixDense | TegolixExperts | None":
    if raw is None:
        return None
    kind = _need(raw, "kind", where)
    if kind == "dense":
        c = TegolixDense(ff=int(_need(raw, "ff", where)))
        if c.ff <= 0:
            raise ConfigError(f"{where}.ff: positive")
        return c
    if kind == "moe":
        router = _need(raw, "router", where)
        shared = raw.get("shared") or {}
        e = TegolixExperts(experts=int(_need(router, "experts", where + ".router")), identity=int(router.get("identity") or 0),
                           top=int(_need(router, "top", where + ".router")), ff=int(_need(_need(raw, "expert", where), "ff", where + ".expert")),
                           shared_ff=int(_need(shared, "ff", where + ".shared")) if shared else 0)
        if e.experts <= 0 or e.identity < 0 or e.ff <= 0 or e.shared_ff < 0 or not 1 <= e.top <= e.experts + e.identity:
            raise ConfigError(f"{where}: positive experts and expert.ff, identity not negative, router.top between 1 and all of them")
        return e
    raise ConfigError(f"{where}.kind {kind!r}: 'dense' or 'moe'")


@dataclass(frozen=True)
class TegolixLayer:
    type: str
    mixer: "TegolixGLA | TegolixParallel"
    mlp: "TegolixDense | TegolixExperts | None"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "TegolixLayer":
        kind = _need(raw, "type", where)
        if kind not in MIXERS:
            raise ConfigError(f"{where}.type {kind!r}: one of {sorted(MIXERS)}")
        return cls(kind, MIXERS[kind].from_dict(_need(raw, "mixer", where), where + ".mixer"), _mlp(raw.get("mlp"), where + ".mlp"))

    def to_dict(self) -> dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class TegolixConfig:
    vocab: int
    width: int
    layers: tuple[TegolixLayer, ...]
    norm_eps: float
    side_dim: int = 0            # width of a layer's stretch of the second token table (0: no per-layer token input)
    architecture: str = "Tegolix"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "TegolixConfig":
        layers = tuple(TegolixLayer.from_dict(l, f"layers[{i}]") for i, l in enumerate(_need(raw, "layers", "config.json")))
        if not layers:
            raise ConfigError("layers: the model has at least one")
        side = raw.get("token_side") or {}
        c = cls(vocab=int(_need(raw, "vocab", "config.json")), width=int(_need(raw, "width", "config.json")), layers=layers,
                norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
                side_dim=int(_need(side, "dim", "token_side")) if side else 0)
        if c.vocab <= 0 or c.width <= 0 or c.norm_eps < 0 or c.side_dim < 0:
            raise ConfigError("vocab and width are positive, norm.eps and token_side.dim are not negative")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out

    def ranks_from(self, shapes: Mapping[str, "tuple[int, ...]"]) -> "TegolixConfig":
        """The same configuration with the decays' ranks as the checkpoint's tensors have them (`shapes`: tensor name ->
        shape): config.json does not give them, a tensor's shape does."""
        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, TegolixGLA) and f"l{i}.mix.a1" in shapes:
                m = replace(m, decay_rank=int(shapes[f"l{i}.mix.a1"][0]))
            elif isinstance(m, TegolixParallel) and f"l{i}.mix.right.w1" in shapes:
                m = replace(m, right=replace(m.right, decay_rank=int(shapes[f"l{i}.mix.right.w1"][0])))
            layers.append(replace(layer, mixer=m))
        return replace(self, layers=tuple(layers))
