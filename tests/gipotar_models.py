"""Small Gipotar configurations and weights for the tests: sizes that differ from layer to layer
and between the two configurations (head counts and grouping, key and value sizes on either
side of each other, rotated width below and at the head size, taps, a feed-forward present or
not on either kind of layer, either kind first), and weights at scales at which every
mechanism matters (slow decays, so that a state that was lost or came from another request
shows; norm weights spread around zero; blend weights across [0, 1])."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import torch


def _attn(heads, kv, dim, vdim, rot, base, scale):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
            "rot": {"dims": rot, "base": base}, "scale": scale}


def _parallel(left, right_heads, right_dim, rank, ls, rs, mlp):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "left_scale": ls,
                      "right": {"heads": right_heads, "dim": right_dim, "rank": rank},
                      "right_scale": rs}}


def _delta(heads, kv, dim, vdim, conv, mlp):
    return {"type": "delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}}


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


CONFIG_A = {
    "architecture": "Gipotar", "vocab": 97, "width": 48, "embedding": {"scale": 3.0},
    "residual_mult": 0.6, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
    "layers": [
        _delta(4, 2, 16, 24, 3, _mlp(80, 1.5)),
        _parallel(_attn(4, 2, 16, 32, 8, 1000.0, 0.3), 3, 16, 8, 0.7, 1.3, None),
        _parallel(_attn(2, 1, 32, 16, 32, 50000.0, 0.2), 2, 24, 5, 1.1, 0.4, _mlp(56, 3.0)),
    ],
}
CONFIG_B = {
    "architecture": "Gipotar", "vocab": 131, "width": 64, "embedding": {"scale": 1.0},
    "residual_mult": 1.0, "norm": {"eps": 1e-6}, "logit_softcap": 40.0,
    "layers": [
        _parallel(_attn(2, 2, 32, 32, 16, 10000.0, 0.25), 1, 64, 16, 1.0, 1.0, _mlp(96, 2.5)),
        _delta(1, 1, 80, 8, 2, None),
        _delta(2, 2, 32, 32, 5, _mlp(72, 1.0)),
        _parallel(_attn(4, 1, 16, 16, 4, 200.0, 0.4), 4, 16, 4, 0.5, 0.9, None),
    ],
}
# Only the delta rule (no mixer asks for pages), one layer with a single tap (no tail at all)
# and one whose three value heads share one query/key head; and only parallel layers, one with
# no rotation and heads of 24 (no multiple of 16: the generic attention kernel in bfloat16).
CONFIG_C = {
    "architecture": "Gipotar", "vocab": 64, "width": 40, "embedding": {"scale": 2.0},
    "residual_mult": 0.8, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
    "layers": [
        _delta(2, 2, 24, 16, 1, None),
        _delta(3, 1, 16, 24, 4, _mlp(48, 2.0)),
    ],
}
CONFIG_D = {
    "architecture": "Gipotar", "vocab": 80, "width": 48, "embedding": {"scale": 4.0},
    "residual_mult": 0.9, "norm": {"eps": 1e-6}, "logit_softcap": 15.0,
    "layers": [
        _parallel(_attn(2, 2, 24, 24, 0, 10000.0, 0.2), 2, 16, 8, 0.6, 0.8, _mlp(64, 2.0)),
        _parallel(_attn(3, 1, 16, 48, 16, 300.0, 0.25), 1, 32, 3, 1.2, 0.3, None),
    ],
}
CONFIGS = {"a": CONFIG_A, "b": CONFIG_B, "c": CONFIG_C, "d": CONFIG_D}


def spec_of(config: dict):
    from rust_llm_inference_server_amd.registry import architecture_of
    arch = architecture_of(config)
    return arch.build_spec(arch.parse_config(config))


def make_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors by checkpoint name, values chosen by what the tensor is."""
    g = torch.Generator().manual_seed(seed)
    normal = lambda shape, std=1.0: torch.randn(shape, generator=g) * std
    uniform = lambda shape, lo, hi: lo + (hi - lo) * torch.rand(shape, generator=g)
    out = {}
    for t in spec_of(config).tensor_specs():
        name, shape = t.name, tuple(t.shape)
        last = name.split(".")[-1]
        if name == "embed":
            w = normal(shape, 0.5)
        elif last in ("norm1", "norm2") or name == "final.norm":
            w = normal(shape, 0.3)
        elif ".mu." in name:
            w = uniform(shape, 0.0, 1.0)
        elif last == "w0":
            w = uniform(shape, -5.0, -0.5)
        elif last == "u":
            w = normal(shape, 0.5)
        elif last == "norm":
            w = 1.0 + normal(shape, 0.3)
        elif last == "conv":
            w = normal(shape, 0.6)
        elif last == "A_log":
            w = uniform(shape, -3.0, 0.5)
        elif last == "dt_bias":
            w = uniform(shape, -3.0, 1.0)
        elif len(shape) == 2:
            w = normal(shape, shape[1] ** -0.5)
        else:
            raise AssertionError(f"no rule for {name}")
        out[name] = w.contiguous()
    return out


def write_folder(path, config: dict, weights: Dict[str, torch.Tensor], dtype=torch.float32,
                 drop_rank: bool = False) -> str:
    """A model folder; ``drop_rank`` leaves the decay projection's rank to the tensors' shapes."""
    from rust_llm_inference_server_amd.weights.safetensors_io import save_file
    os.makedirs(str(path), exist_ok=True)
    config = copy.deepcopy(config)
    if drop_rank:
        for layer in config["layers"]:
            if layer["type"] == "parallel":
                layer["mixer"]["right"].pop("rank", None)
    with open(os.path.join(str(path), "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()},
              os.path.join(str(path), "model.safetensors"))
    return str(path)


def as_stored(weights: Dict[str, torch.Tensor], dtype) -> Dict[str, torch.Tensor]:
    """The numbers a folder of ``dtype`` holds, in float64 for the plain implementation."""
    return {k: v.to(dtype).to(torch.float64) for k, v in weights.items()}


def prompts(vocab: int, lengths: List[int], seed: int) -> List[List[int]]:
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


def row_error(got: torch.Tensor, want: torch.Tensor) -> float:
    """Root mean square of the difference (mean taken off) over that of the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean()
    w = want.double() - want.double().mean()
    return float(torch.sqrt((d * d).mean()) / torch.sqrt((w * w).mean()))


# What rounding alone does to a row of logits at these sizes and weight scales: float32 rows
# stay below 2e-4; bfloat16 rows (weights stored in bfloat16, the plain implementation run in
# float64 on those numbers) have a median of 0.003 to 0.01 by the configuration and a 98th
# percentile of 0.03, and one in a hundred reaches 0.08.  A token lost from the cache or the
# state moves a row by 0.8 and more.
TOLERANCE = {"float32": 2e-4, "bfloat16": 6e-2}


def judge(errors: List[float], dtype: str) -> None:
    """No row beyond two and a half times the tolerance, and at most one in fifty beyond it."""
    tol = TOLERANCE[dtype]
    over = sum(e > tol for e in errors)
    assert max(errors) < 2.5 * tol, f"worst row error {max(errors):.3g}"
    assert over <= max(1, len(errors) // 50), f"{over} of {len(errors)} rows beyond {tol}"
