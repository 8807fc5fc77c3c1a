"""Typed configuration of the Gipotar decoder, read from its ``config.json``.

The file names the design under ``architecture`` and gives every size and every constant that
may differ between two models of it: vocabulary, width, the multiplier of the embedding, the
multiplier with which a sublayer's output joins the residual stream, the norm's epsilon, the
cap of the logits, and a list of layers.  A layer is of type ``parallel`` (softmax attention
beside an RWKV-style time mix) or ``delta`` (gated delta rule) and may or may not have a
feed-forward.  What the file leaves to the tensors' shapes (the rank of the time mix's decay
projection) is filled in from the checkpoint (``with_tensor_shapes``); a configuration that is
to get random weights names it as ``rank`` in the layer's ``mixer.right``.

The parser refuses what the engine would compute wrongly, with the key's name."""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from .errors import ConfigError
from .llama import _need, _typed

ARCHITECTURE = "Gipotar"


def _obj(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object")
    return v


def _positive(v: int, key: str, where: str) -> int:
    if v <= 0:
        raise ConfigError(f"{where}: key '{key}' must be positive, got {v}")
    return v


@dataclass(frozen=True)
class AttentionBranch:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int
    rot_base: float
    scale: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "AttentionBranch":
        rot = _obj(d, "rot", where)
        out = cls(heads=_positive(_need(d, "heads", int, where), "heads", where),
                  kv_heads=_positive(_need(d, "kv_heads", int, where), "kv_heads", where),
                  dim=_positive(_need(d, "dim", int, where), "dim", where),
                  vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
                  rot_dims=_need(rot, "dims", int, where + " rot"),
                  rot_base=_need(rot, "base", float, where + " rot"),
                  scale=_need(d, "scale", float, where))
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: 'heads' {out.heads} is not a multiple of 'kv_heads' "
                              f"{out.kv_heads}")
        if out.rot_dims < 0 or out.rot_dims % 2 or out.rot_dims > out.dim:
            raise ConfigError(f"{where} rot: 'dims' {out.rot_dims} must be even and at most "
                              f"'dim' {out.dim}")
        if out.rot_dims and not out.rot_base > 0:
            raise ConfigError(f"{where} rot: 'base' must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim,
                "vdim": self.vdim, "rot": {"dims": self.rot_dims, "base": self.rot_base},
                "scale": self.scale}


@dataclass(frozen=True)
class TimeMixBranch:
    heads: int
    dim: int
    rank: Optional[int] = None      # rows of the decay's first projection; from the tensors

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "TimeMixBranch":
        rank = d.get("rank")
        return cls(heads=_positive(_need(d, "heads", int, where), "heads", where),
                   dim=_positive(_need(d, "dim", int, where), "dim", where),
                   rank=None if rank is None else _positive(_typed(rank, "rank", int, where),
                                                            "rank", where))

    def to_dict(self) -> Dict[str, Any]:
        d = {"heads": self.heads, "dim": self.dim}
        if self.rank is not None:
            d["rank"] = self.rank
        return d


@dataclass(frozen=True)
class ParallelMixer:
    left: AttentionBranch
    right: TimeMixBranch
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "ParallelMixer":
        return cls(left=AttentionBranch.from_dict(_obj(d, "left", where), where + " left"),
                   right=TimeMixBranch.from_dict(_obj(d, "right", where), where + " right"),
                   left_scale=_need(d, "left_scale", float, where),
                   right_scale=_need(d, "right_scale", float, where))

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale,
                "right": self.right.to_dict(), "right_scale": self.right_scale}


@dataclass(frozen=True)
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "DeltaMixer":
        out = cls(heads=_positive(_need(d, "heads", int, where), "heads", where),
                  kv_heads=_positive(_need(d, "kv_heads", int, where), "kv_heads", where),
                  dim=_positive(_need(d, "dim", int, where), "dim", where),
                  vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
                  conv=_positive(_need(d, "conv", int, where), "conv", where))
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: 'heads' {out.heads} is not a multiple of 'kv_heads' "
                              f"{out.kv_heads}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads,
                "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class DenseMlp:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "DenseMlp":
        kind = _need(d, "kind", str, where)
        if kind != "dense":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (known: 'dense')")
        out = cls(ff=_positive(_need(d, "ff", int, where), "ff", where),
                  limit=_need(d, "limit", float, where))
        if not out.limit > 0:
            raise ConfigError(f"{where}: 'limit' must be positive, got {out.limit}")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclass(frozen=True)
class GipotarLayer:
    type: str                          # "parallel" or "delta"
    mixer: Any                         # ParallelMixer or DeltaMixer
    mlp: Optional[DenseMlp]

    @classmethod
    def from_dict(cls, d: Any, index: int) -> "GipotarLayer":
        where = f"config.json layers[{index}]"
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: must be an object")
        kind = _need(d, "type", str, where)
        mixer = _obj(d, "mixer", where)
        if kind == "parallel":
            m: Any = ParallelMixer.from_dict(mixer, where + " mixer")
        elif kind == "delta":
            m = DeltaMixer.from_dict(mixer, where + " mixer")
        else:
            raise ConfigError(f"{where}: type '{kind}' is not supported (known: 'parallel', "
                              "'delta')")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: 'mlp' must be an object or null")
        return cls(kind, m, None if mlp is None else DenseMlp.from_dict(mlp, where + " mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class GipotarConfig:
    vocab: int
    width: int
    embedding_scale: float
    residual_mult: float
    norm_eps: float
    logit_softcap: float
    layers: Tuple[GipotarLayer, ...]
    architecture: str = ARCHITECTURE

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GipotarConfig":
        where = "config.json"
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        out = cls(vocab=_positive(_need(d, "vocab", int), "vocab", where),
                  width=_positive(_need(d, "width", int), "width", where),
                  embedding_scale=_need(_obj(d, "embedding", where), "scale", float,
                                        where + " embedding"),
                  residual_mult=_need(d, "residual_mult", float),
                  norm_eps=_need(_obj(d, "norm", where), "eps", float, where + " norm"),
                  logit_softcap=_need(d, "logit_softcap", float),
                  layers=tuple(GipotarLayer.from_dict(l, i) for i, l in enumerate(layers)))
        if not out.logit_softcap > 0:
            raise ConfigError(f"{where}: 'logit_softcap' must be positive")
        if not out.norm_eps > 0:
            raise ConfigError(f"{where} norm: 'eps' must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [l.to_dict() for l in self.layers],
                "logit_softcap": self.logit_softcap, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}

    def with_tensor_shapes(self, shapes: Mapping[str, Sequence[int]]) -> "GipotarConfig":
        """The configuration with what only the checkpoint's shapes say filled in: the rank of
        every time mix's decay projection (rows of ``l<i>.mix.right.w1``)."""
        layers = []
        for i, layer in enumerate(self.layers):
            if layer.type == "parallel" and layer.mixer.right.rank is None:
                shape = shapes.get(f"l{i}.mix.right.w1")
                if shape is not None and len(shape) == 2:
                    right = replace(layer.mixer.right, rank=int(shape[0]))
                    layer = replace(layer, mixer=replace(layer.mixer, right=right))
            layers.append(layer)
        return replace(self, layers=tuple(layers))
