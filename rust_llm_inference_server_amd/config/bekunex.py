"""Typed configuration of the Bekunex decoder, read from its ``config.json``.

The file names the design under ``architecture`` and gives every size and every constant that
may differ between two models of it: vocabulary, width, the norms' epsilon, the multiplier of
the logits, and a list of layers.  A layer's ``type`` names its mixer: ``latent_attention``
(keys and values from a cached latent, a rotated key part shared by the heads, causal),
``latent_attention_2`` (the same without positions: sliding window, a sink in the softmax, a
sigmoid gate on the output; with ``kv_from`` it reads the latents an earlier layer cached) or
``mamba1`` (selective scan).  Its ``mlp`` is null or a mixture of experts.

The parser refuses what the engine would compute wrongly, with the key's name."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .gipotar import _obj, _positive
from .llama import _need, _typed

ARCHITECTURE = "Bekunex"


@dataclass(frozen=True)
class LatentMixer:
    """``latent_attention`` (rot_dim > 0, no window, no sink, no gate) or
    ``latent_attention_2`` (rot_dim 0, window, sink and gate)."""
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_dim: int = 0
    rot_dims: int = 0                 # how many of the rot_dim numbers are rotated
    rot_base: float = 10000.0
    window: Optional[int] = None
    kv_from: Optional[int] = None
    second: bool = False              # the kind without positions

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, second: bool) -> "LatentMixer":
        kw: Dict[str, Any] = dict(
            heads=_positive(_need(d, "heads", int, where), "heads", where),
            dim=_positive(_need(d, "dim", int, where), "dim", where),
            vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
            kv_rank=_positive(_need(d, "kv_rank", int, where), "kv_rank", where),
            scale=_need(d, "scale", float, where), second=second)
        if second:
            mask = _obj(d, "mask", where)
            kw["window"] = _positive(_need(mask, "size", int, where + " mask"), "size",
                                     where + " mask")
            if d.get("kv_from") is not None:
                kw["kv_from"] = _typed(d["kv_from"], "kv_from", int, where)
            if d.get("rot_dim"):
                raise ConfigError(f"{where}: this mixer has no rotated part ('rot_dim')")
        else:
            rot = _obj(d, "rot", where)
            kw["rot_dim"] = _positive(_need(d, "rot_dim", int, where), "rot_dim", where)
            kw["rot_dims"] = _need(rot, "dims", int, where + " rot")
            kw["rot_base"] = _need(rot, "base", float, where + " rot")
            if kw["rot_dims"] <= 0 or kw["rot_dims"] % 2 or kw["rot_dims"] > kw["rot_dim"]:
                raise ConfigError(f"{where} rot: 'dims' {kw['rot_dims']} must be even, positive "
                                  f"and at most 'rot_dim' {kw['rot_dim']}")
            if not kw["rot_base"] > 0:
                raise ConfigError(f"{where} rot: 'base' must be positive")
        return cls(**kw)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank,
                             "scale": self.scale, "vdim": self.vdim}
        if self.second:
            d["mask"] = {"size": self.window}
            if self.kv_from is not None:
                d["kv_from"] = self.kv_from
        else:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            d["rot_dim"] = self.rot_dim
        return d


@dataclass(frozen=True)
class ScanMixer:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "ScanMixer":
        out = cls(*(_positive(_need(d, k, int, where), k, where)
                    for k in ("inner", "state", "dt_rank", "conv")))
        if out.conv > 16:
            raise ConfigError(f"{where}: 'conv' {out.conv} is more taps than the engine takes (16)")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dt_rank": self.dt_rank, "inner": self.inner,
                "state": self.state}


@dataclass(frozen=True)
class MoeMlp:
    expert_ff: int
    experts: int
    top: int
    groups: int
    keep: int
    scale: float
    shared_ff: Optional[int]

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "MoeMlp":
        kind = _need(d, "kind", str, where)
        if kind != "moe":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (known: 'moe')")
        router = _obj(d, "router", where)
        rw = where + " router"
        groups = router.get("groups")
        if groups is not None and not isinstance(groups, dict):
            raise ConfigError(f"{rw}: 'groups' must be an object")
        shared = d.get("shared")
        if shared is not None and not isinstance(shared, dict):
            raise ConfigError(f"{where}: 'shared' must be an object or null")
        out = cls(
            expert_ff=_positive(_need(_obj(d, "expert", where), "ff", int, where + " expert"),
                                "ff", where + " expert"),
            experts=_positive(_need(router, "experts", int, rw), "experts", rw),
            top=_positive(_need(router, "top", int, rw), "top", rw),
            groups=1 if groups is None else _positive(_need(groups, "count", int, rw + " groups"),
                                                      "count", rw + " groups"),
            keep=1 if groups is None else _positive(_need(groups, "keep", int, rw + " groups"),
                                                    "keep", rw + " groups"),
            scale=_need(router, "scale", float, rw),
            shared_ff=None if shared is None else _positive(
                _need(shared, "ff", int, where + " shared"), "ff", where + " shared"))
        if out.experts % out.groups:
            raise ConfigError(f"{rw}: {out.experts} experts do not form {out.groups} equal groups")
        if out.keep > out.groups:
            raise ConfigError(f"{rw} groups: 'keep' {out.keep} exceeds 'count' {out.groups}")
        if out.top > out.keep * (out.experts // out.groups):
            raise ConfigError(f"{rw}: 'top' {out.top} exceeds the experts of the kept groups")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"expert": {"ff": self.expert_ff}, "kind": "moe",
                "router": {"experts": self.experts,
                           "groups": {"count": self.groups, "keep": self.keep},
                           "scale": self.scale, "top": self.top},
                "shared": None if self.shared_ff is None else {"ff": self.shared_ff}}


LAYER_TYPES = ("latent_attention", "latent_attention_2", "mamba1")


@dataclass(frozen=True)
class BekunexLayer:
    type: str
    mixer: Any                         # LatentMixer or ScanMixer
    mlp: Optional[MoeMlp]

    @classmethod
    def from_dict(cls, d: Any, index: int) -> "BekunexLayer":
        where = f"config.json layers[{index}]"
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: must be an object")
        kind = _need(d, "type", str, where)
        mixer = _obj(d, "mixer", where)
        if kind == "mamba1":
            m: Any = ScanMixer.from_dict(mixer, where + " mixer")
        elif kind in ("latent_attention", "latent_attention_2"):
            m = LatentMixer.from_dict(mixer, where + " mixer", kind == "latent_attention_2")
        else:
            raise ConfigError(f"{where}: type '{kind}' is not supported (known: "
                              f"{', '.join(LAYER_TYPES)})")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: 'mlp' must be an object or null")
        return cls(kind, m, None if mlp is None else MoeMlp.from_dict(mlp, where + " mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class BekunexConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: Tuple[BekunexLayer, ...]
    architecture: str = ARCHITECTURE

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "BekunexConfig":
        where = "config.json"
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        out = cls(vocab=_positive(_need(d, "vocab", int), "vocab", where),
                  width=_positive(_need(d, "width", int), "width", where),
                  norm_eps=_need(_obj(d, "norm", where), "eps", float, where + " norm"),
                  logit_scale=_need(d, "logit_scale", float),
                  layers=tuple(BekunexLayer.from_dict(l, i) for i, l in enumerate(layers)))
        if not out.norm_eps > 0:
            raise ConfigError(f"{where} norm: 'eps' must be positive")
        for i, layer in enumerate(out.layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            lw = f"{where} layers[{i}] mixer"
            if not 0 <= src < i:
                raise ConfigError(f"{lw}: 'kv_from' {src} must name an earlier layer")
            other = out.layers[src]
            if other.type != "latent_attention_2" or other.mixer.kv_from is not None:
                raise ConfigError(f"{lw}: 'kv_from' {src} names a layer that caches no latent "
                                  "of this kind of its own")
            if other.mixer.kv_rank != layer.mixer.kv_rank:
                raise ConfigError(f"{lw}: 'kv_rank' {layer.mixer.kv_rank} differs from layer "
                                  f"{src}'s {other.mixer.kv_rank}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture,
                "layers": [l.to_dict() for l in self.layers],
                "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps},
                "vocab": self.vocab, "width": self.width}
