"""The Gipotar decoder as a ``ModelSpec``: a token embedding with a multiplier, pre-norm blocks
whose sublayers join the residual stream with a multiplier, a final norm, a head whose logits
pass a tanh cap.  Norm weights are stored around zero (``1 + w`` multiplies).  A block's mixer
is either softmax attention (grouped heads, keys and values of different sizes, rotation of
part of a head) beside an RWKV-style time mix, or the gated delta rule; its feed-forward, when
it has one, is the clamped gated unit.  Every part is one of the package's registered kinds with
this model's sizes and constants as parameters; tensor names are the checkpoint's
(``embed``, ``l<i>.norm1``, ``l<i>.mix. ...``, ``l<i>.mlp. ...``, ``final.norm``, ``head``)."""
from __future__ import annotations

from ..config.errors import ConfigError
from ..config.gipotar import ARCHITECTURE, GipotarConfig, GipotarLayer
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec

GLU_ALPHA = 1.702       # the design fixes the sigmoid's slope in its feed-forward


def _mixer(cfg: GipotarConfig, layer: GipotarLayer, index: int) -> PartSpec:
    W, m = cfg.width, layer.mixer
    if layer.type == "delta":
        return PartSpec("gated_delta", {
            "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
            "head_dim": m.dim, "value_dim": m.vdim, "conv": m.conv, "eps": cfg.norm_eps})
    left, right = m.left, m.right
    if right.rank is None:
        raise ConfigError(f"config.json layers[{index}] mixer right: the rank of the decay "
                          "projection is known neither from a checkpoint nor from 'rank'")
    attention = PartSpec("attention", {
        "hidden_size": W, "num_heads": left.heads, "num_kv_heads": left.kv_heads,
        "head_dim": left.dim, "value_dim": left.vdim, "scale": left.scale, "window": None,
        "position": PartSpec("rope", {"rot_dim": left.rot_dims, "theta": left.rot_base,
                                      "scaling": None}) if left.rot_dims else PartSpec("none"),
        "names": {"q": "q", "k": "k", "v": "v", "o": "o"}})
    time_mix = PartSpec("time_mix", {
        "hidden_size": W, "num_heads": right.heads, "head_dim": right.dim,
        "decay_rank": right.rank, "eps": cfg.norm_eps})
    return PartSpec("parallel", {"branches": [
        {"mixer": attention, "name": "left", "scale": m.left_scale},
        {"mixer": time_mix, "name": "right", "scale": m.right_scale}]})


def gipotar_spec(cfg: GipotarConfig) -> ModelSpec:
    W = cfg.width
    norm = PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "weight_offset": 1.0,
                                "weight_name": ""})
    layers = []
    for i, layer in enumerate(cfg.layers):
        ff = None
        if layer.mlp is not None:
            ff = PartSpec("clamped_glu", {
                "hidden_size": W, "intermediate_size": layer.mlp.ff, "limit": layer.mlp.limit,
                "alpha": GLU_ALPHA, "names": {"gate": "gate", "up": "up", "down": "down"}})
        block = PartSpec("prenorm", {
            "mixer": _mixer(cfg, layer, i), "feed_forward": ff, "mixer_norm": norm,
            "ffn_norm": norm, "residual_scale": cfg.residual_mult,
            "names": {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2",
                      "feed_forward": "mlp"}})
        layers.append(LayerSpec(block, f"l{i}"))
    return ModelSpec(
        hidden_size=W,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W,
                                     "scale": cfg.embedding_scale, "weight_name": ""}),
        embedding_prefix="embed",
        layers=layers,
        final_norm=norm,
        final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": None,
                                 "weight_name": "", "soft_cap": cfg.logit_softcap}),
        head_prefix="head",
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    parse_config=GipotarConfig.from_dict,
    build_spec=gipotar_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
    complete_config=lambda cfg, shapes: cfg.with_tensor_shapes(shapes),
))
