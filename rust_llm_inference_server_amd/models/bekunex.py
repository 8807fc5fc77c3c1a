"""The Bekunex decoder as a ``ModelSpec``: a token embedding, parallel blocks (one layer norm
whose output both the mixer and the feed-forward read, their outputs joining the residual
stream together), a final layer norm, a head whose logits carry a multiplier.  A block's mixer
is attention over a cached latent (with a rotated key part and a full causal mask, or without
positions under a sliding window with a sink and an output gate, possibly reading the latents
that an earlier layer cached) or a selective scan; its feed-forward, when it has one, is a
mixture of gated units with a shared one.  Every part is one of the package's registered kinds
with this model's sizes and constants as parameters; tensor names are the checkpoint's
(``embed``, ``l<i>.norm1``, ``l<i>.norm1.b``, ``l<i>.mix. ...``, ``l<i>.mlp. ...``,
``final.norm``, ``final.norm.b``, ``head``).

A layer with ``kv_from: j`` runs on the cache of layer j's run (``RunEntry.cache_of``); the
cache of a layer that is read by others keeps the widest window among its readers."""
from __future__ import annotations

from typing import Dict, Optional

from ..config.bekunex import ARCHITECTURE, BekunexConfig, BekunexLayer
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, RunEntry


def _cache_windows(cfg: BekunexConfig) -> Dict[int, Optional[int]]:
    """Per layer that caches latents under a window: the widest window among the layers that
    read its cache (its own included)."""
    out: Dict[int, Optional[int]] = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type != "latent_attention_2":
            continue
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        out[owner] = max(out.get(owner) or 0, layer.mixer.window)
    return out


def _mixer(cfg: BekunexConfig, layer: BekunexLayer, cache_window: Optional[int]) -> PartSpec:
    W, m = cfg.width, layer.mixer
    if layer.type == "mamba1":
        return PartSpec("selective_scan", {"hidden_size": W, "inner": m.inner, "state": m.state,
                                           "dt_rank": m.dt_rank, "conv": m.conv})
    params = {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
              "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps,
              "window": m.window, "cache_window": cache_window, "sink": m.second,
              "gate": m.second, "own_latent": m.kv_from is None}
    if m.rot_dim:
        params["position"] = PartSpec("rope", {"rot_dim": m.rot_dims, "theta": m.rot_base,
                                               "scaling": None, "precise": True})
    return PartSpec("latent_attention", params)


def bekunex_spec(cfg: BekunexConfig) -> ModelSpec:
    W = cfg.width
    norm = PartSpec("layernorm", {"size": W, "eps": cfg.norm_eps, "weight_name": "",
                                  "bias_name": "b"})
    windows = _cache_windows(cfg)
    layers, runs = [], []
    for i, layer in enumerate(cfg.layers):
        ff = None
        if layer.mlp is not None:
            p = layer.mlp
            ff = PartSpec("routed_swiglu", {
                "hidden_size": W, "expert_size": p.expert_ff, "experts": p.experts, "top": p.top,
                "groups": p.groups, "keep": p.keep, "scale": p.scale,
                "shared_size": p.shared_ff})
        src = getattr(layer.mixer, "kv_from", None)
        owner = i if src is None else src
        block = PartSpec("parallel", {
            "mixer": _mixer(cfg, layer, windows.get(owner)), "feed_forward": ff, "norm": norm,
            "names": {"norm": "norm1", "mixer": "mix", "feed_forward": "mlp"}})
        layers.append(LayerSpec(block, f"l{i}"))
        runs.append(RunEntry(i, cache_of=src))
    return ModelSpec(
        hidden_size=W,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W,
                                     "weight_name": ""}),
        embedding_prefix="embed",
        layers=layers,
        run_order=runs,
        final_norm=norm,
        final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": None,
                                 "weight_name": "", "scale": cfg.logit_scale}),
        head_prefix="head",
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    parse_config=BekunexConfig.from_dict,
    build_spec=bekunex_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
))
