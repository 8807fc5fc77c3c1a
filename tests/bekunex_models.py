"""Small Bekunex configurations and weights for the tests: sizes that differ from layer to
layer and between the configurations (head counts down to one, key, value and latent sizes on
either side of each other and off the multiples of 8, windows of 1, of a page and of more than
the cache's writer, a reader of another layer's latents whose window is the wider one, states
of 5 to 70 numbers, one to four taps, experts in one group or several with one or more kept,
one to three experts chosen, with and without a shared unit, layers without a feed-forward,
either kind of layer first), and weights at scales at which every mechanism matters: slow
decays, sinks of the size of the scores, corrections that change the choice of experts, norm
weights and biases spread out."""
from __future__ import annotations

from typing import Dict

import torch

from typing import List

from gipotar_models import (as_stored, prompts, row_error, write_folder,  # noqa: F401
                            TOLERANCE)


def _moe(ff, experts, groups, keep, top, scale, shared):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "groups": {"count": groups, "keep": keep},
                       "scale": scale, "top": top},
            "shared": None if shared is None else {"ff": shared}}


def _latent(heads, dim, rot, base, vdim, rank, scale, mlp):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "rot": {"dims": rot, "base": base},
                      "vdim": vdim, "kv_rank": rank, "scale": scale}}


def _latent2(heads, dim, vdim, rank, window, scale, mlp, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "mask": {"size": window},
         "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention_2", "mlp": mlp, "mixer": m}


def _scan(inner, state, rank, conv, mlp):
    return {"type": "mamba1", "mlp": mlp,
            "mixer": {"inner": inner, "state": state, "dt_rank": rank, "conv": conv}}


CONFIG_A = {
    "architecture": "Bekunex", "vocab": 97, "width": 48, "norm": {"eps": 1e-5},
    "logit_scale": 0.5,
    "layers": [
        _latent2(3, 16, 24, 40, 20, 0.3, _moe(24, 6, 3, 2, 3, 2.0, 40)),
        _scan(64, 8, 5, 3, None),
        _latent(2, 24, 8, 1000.0, 16, 32, 0.2, _moe(32, 4, 1, 1, 1, 1.0, None)),
        _latent2(2, 8, 16, 40, 33, 0.35, _moe(24, 6, 2, 1, 2, 0.7, 16), kv_from=0),
    ],
}
CONFIG_B = {
    "architecture": "Bekunex", "vocab": 131, "width": 64, "norm": {"eps": 1e-6},
    "logit_scale": 3.0,
    "layers": [
        _latent(4, 16, 16, 50000.0, 16, 24, 0.25, _moe(16, 8, 4, 2, 2, 1.5, 48)),
        _latent2(1, 32, 32, 16, 7, 0.2, None),
        _scan(96, 20, 3, 4, _moe(40, 3, 3, 3, 3, 1.0, 24)),
        _scan(32, 70, 8, 1, None),
        _latent2(2, 16, 8, 16, 64, 0.3, _moe(16, 8, 2, 1, 4, 2.5, None)),
    ],
}
# Only scans (no mixer asks for pages), sizes off every multiple of 4.
CONFIG_C = {
    "architecture": "Bekunex", "vocab": 64, "width": 40, "norm": {"eps": 1e-5},
    "logit_scale": 1.0,
    "layers": [
        _scan(56, 5, 7, 2, _moe(12, 5, 1, 1, 2, 1.2, 20)),
        _scan(24, 33, 2, 4, None),
    ],
}
# Only attention (no state slots); head sizes, latent sizes and rotated widths off the multiples
# of 8; windows of one position and of exactly a page; a chain of two readers of one cache.
CONFIG_D = {
    "architecture": "Bekunex", "vocab": 80, "width": 56, "norm": {"eps": 1e-6},
    "logit_scale": 1.7,
    "layers": [
        _latent(3, 12, 6, 300.0, 20, 28, 0.28, _moe(20, 4, 2, 2, 2, 1.0, 12)),
        _latent2(2, 20, 12, 36, 16, 0.22, None),
        _latent2(4, 8, 8, 36, 1, 0.4, _moe(8, 2, 1, 1, 1, 3.0, None), kv_from=1),
        _latent2(1, 24, 40, 36, 50, 0.2, None, kv_from=1),
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
        parts = name.split(".")
        last = parts[-1]
        if name == "embed":
            w = normal(shape, 0.5)
        elif last in ("norm1", "norm") and len(shape) == 1:
            w = 1.0 + normal(shape, 0.3)
        elif last == "b" and parts[-2] in ("norm1", "norm"):
            w = normal(shape, 0.2)
        elif last == "sink":
            w = normal(shape, 1.0)
        elif last == "correction":
            w = normal(shape, 0.3)
        elif last == "router":
            w = normal(shape, 2.0 * shape[1] ** -0.5)
        elif last == "conv":
            w = normal(shape, 0.6)
        elif last == "b" and parts[-2] == "conv":
            w = normal(shape, 0.3)
        elif last == "b" and parts[-2] == "dt":
            w = uniform(shape, -3.0, 0.0)
        elif last == "A_log":
            w = uniform(shape, -3.0, 0.5)
        elif last == "D":
            w = normal(shape, 1.0)
        elif len(shape) == 2:
            w = normal(shape, shape[1] ** -0.5)
        else:
            raise AssertionError(f"no rule for {name}")
        out[name] = w.contiguous()
    return out


def judge(errors: List[float], dtype: str) -> None:
    """float32: no row beyond two and a half times the tolerance and at most one in fifty beyond
    it.  bfloat16: at most one row in twenty-five beyond the tolerance, whatever its size, and
    nine in ten within half of it: where two experts' choice scores lie closer than bfloat16
    resolves the router's input, the engine may take the other one, and that row (seldom a
    later one) is then far from the plain logits; at these sizes, with single experts chosen
    out of four, that happens to two or three rows in a hundred, while a fault of the cache or
    the state moves most rows."""
    tol = TOLERANCE[dtype]
    over = sum(e > tol for e in errors)
    if dtype == "float32":
        assert over <= max(1, len(errors) // 50), f"{over} of {len(errors)} rows beyond {tol}"
        assert max(errors) < 2.5 * tol, f"worst row error {max(errors):.3g}"
    else:
        assert over <= max(1, len(errors) // 25), f"{over} of {len(errors)} rows beyond {tol}"
        ranked = sorted(errors)
        p90 = ranked[min(len(ranked) - 1, int(0.9 * len(ranked)))]
        assert p90 < tol / 2 or len(ranked) < 20, f"90th percentile of the row errors {p90:.3g}"
