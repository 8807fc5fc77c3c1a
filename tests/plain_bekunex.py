"""A plain, slow implementation of the Bekunex decoder, one function per mechanism, in float64
on the CPU.  It takes a whole sequence at a time and keeps nothing between calls; it shares no
code with the package.  ``weights`` maps checkpoint names to tensors, ``config`` is the
config.json dict.

Notation: T tokens, W the width, x the residual stream (T, W), h the normalised input of a
layer's two sublayers."""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional, Tuple

import torch

F = torch.float64


def _w(weights: Dict[str, torch.Tensor], name: str) -> torch.Tensor:
    return weights[name].to(F)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotate(v: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """Rotate the first ``dims`` entries of the last axis of ``v (T, ..., d)`` by position:
    entry i is paired with entry i + dims/2; angle = position * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=F)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(F).reshape(-1, *([1] * (v.dim() - 1))) * freq
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                      window: Optional[int], sink: Optional[torch.Tensor]) -> torch.Tensor:
    """q (T, H, d), k (T, H, d), v (T, H, dv) of one sequence from position 0.  Query i sees
    key j with j <= i and, under a window, i - j < window.  With ``sink`` (H) the softmax's
    denominator also holds exp(sink_h)."""
    T, H, _ = q.shape
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    i = torch.arange(T).reshape(T, 1)
    j = torch.arange(T).reshape(1, T)
    seen = j <= i
    if window is not None:
        seen = seen & (i - j < window)
    s = s.masked_fill(~seen, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.reshape(H, 1, 1))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.reshape(H, 1, 1) - m)
    return torch.einsum("hij,jhd->ihd", e / den, v)


def latent_attention(h: torch.Tensor, weights, prefix: str, m: Dict[str, Any], eps: float,
                     positions: torch.Tensor) -> torch.Tensor:
    """Keys and values come from a normed latent; a rotated part of the key is shared by the
    heads; causal, ordinary softmax."""
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    q = (h @ _w(weights, prefix + ".q").T).reshape(T, H, d + r)
    dkv = h @ _w(weights, prefix + ".dkv").T
    c = rms_norm(dkv[:, :R], _w(weights, prefix + ".dkv.norm"), eps)
    kr = rotate(dkv[:, R:], positions, m["rot"]["dims"], m["rot"]["base"])
    qr = rotate(q[..., d:], positions, m["rot"]["dims"], m["rot"]["base"])
    k = (c @ _w(weights, prefix + ".uk").T).reshape(T, H, d)
    v = (c @ _w(weights, prefix + ".uv").T).reshape(T, H, dv)
    qf = torch.cat([q[..., :d], qr], dim=-1)
    kf = torch.cat([k, kr.reshape(T, 1, r).expand(T, H, r)], dim=-1)
    o = softmax_attention(qf, kf, v, m["scale"], None, None)
    return o.reshape(T, H * dv) @ _w(weights, prefix + ".o").T


def latent_of(h: torch.Tensor, weights, prefix: str, eps: float) -> torch.Tensor:
    return rms_norm(h @ _w(weights, prefix + ".dkv").T, _w(weights, prefix + ".dkv.norm"), eps)


def latent_attention_2(h: torch.Tensor, weights, prefix: str, m: Dict[str, Any], eps: float,
                       latent: torch.Tensor) -> torch.Tensor:
    """No positions; sliding window; a sink in the softmax; a sigmoid gate on the heads'
    outputs.  ``latent`` (T, kv_rank) is this layer's own or another layer's."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ _w(weights, prefix + ".q").T).reshape(T, H, d)
    k = (latent @ _w(weights, prefix + ".uk").T).reshape(T, H, d)
    v = (latent @ _w(weights, prefix + ".uv").T).reshape(T, H, dv)
    o = softmax_attention(q, k, v, m["scale"], m["mask"]["size"], _w(weights, prefix + ".sink"))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ _w(weights, prefix + ".g").T)
    return o @ _w(weights, prefix + ".o").T


def mamba1(h: torch.Tensor, weights, prefix: str, m: Dict[str, Any]) -> torch.Tensor:
    """Selective scan with a short causal convolution in front, one sequence from its start."""
    C, N, rank, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    T = h.shape[0]
    xz = h @ _w(weights, prefix + ".in").T
    x, z = xz[:, :C], xz[:, C:]
    cw, cb = _w(weights, prefix + ".conv"), _w(weights, prefix + ".conv.b")
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F), x], dim=0)
    conv = cb.reshape(1, C).expand(T, C).clone()
    for j in range(taps):
        conv = conv + padded[j:j + T] * cw[:, j]
    x = silu(conv)
    low = x @ _w(weights, prefix + ".x").T
    dt_low, B, Cm = low[:, :rank], low[:, rank:rank + N], low[:, rank + N:]
    dt = torch.nn.functional.softplus(dt_low @ _w(weights, prefix + ".dt").T
                                      + _w(weights, prefix + ".dt.b"), threshold=1e9)
    A = -torch.exp(_w(weights, prefix + ".A_log"))
    D = _w(weights, prefix + ".D")
    S = torch.zeros(C, N, dtype=F)
    ys = []
    for t in range(T):
        S = torch.exp(dt[t].reshape(C, 1) * A) * S + (dt[t] * x[t]).reshape(C, 1) * B[t]
        ys.append(S @ Cm[t] + D * x[t])
    y = torch.stack(ys) * silu(z)
    return y @ _w(weights, prefix + ".o").T


def gated_unit(h: torch.Tensor, weights, prefix: str) -> torch.Tensor:
    g = h @ _w(weights, prefix + ".gate").T
    u = h @ _w(weights, prefix + ".up").T
    return (silu(g) * u) @ _w(weights, prefix + ".down").T


def route(h: torch.Tensor, weights, prefix: str, router: Dict[str, Any]
          ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Chosen experts (T, top) and their weights (T, top)."""
    E, top = router["experts"], router["top"]
    G, keep = router["groups"]["count"], router["groups"]["keep"]
    s = torch.sigmoid(h @ _w(weights, prefix + ".router").T)
    choice = s + _w(weights, prefix + ".correction")
    T = h.shape[0]
    per = E // G
    grouped = choice.reshape(T, G, per)
    gscore = grouped.topk(min(2, per), dim=-1).values.sum(-1)
    kept = gscore.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, G, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = grouped.masked_fill(~allowed.reshape(T, G, 1), -math.inf).reshape(T, E)
    chosen = masked.topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen) * router["scale"]


def moe(h: torch.Tensor, weights, prefix: str, mlp: Dict[str, Any]) -> torch.Tensor:
    chosen, wts = route(h, weights, prefix, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), wts[t]):
            out[t] += w * gated_unit(h[t:t + 1], weights, f"{prefix}.e{e}")[0]
    if mlp.get("shared") is not None:
        out = out + gated_unit(h, weights, prefix + ".shared")
    return out


def forward(weights, config: Dict[str, Any], tokens: List[int], return_layers: bool = False):
    """Logits (T, vocab) of one sequence from its start; with ``return_layers`` also the
    residual stream after every layer."""
    eps = config["norm"]["eps"]
    x = _w(weights, "embed")[torch.tensor(tokens, dtype=torch.long)]
    positions = torch.arange(len(tokens))
    latents: Dict[int, torch.Tensor] = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h = layer_norm(x, _w(weights, p + ".norm1"), _w(weights, p + ".norm1.b"), eps)
        if layer["type"] == "latent_attention":
            y = latent_attention(h, weights, p + ".mix", m, eps, positions)
        elif layer["type"] == "latent_attention_2":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_of(h, weights, p + ".mix", eps)
                src = i
            y = latent_attention_2(h, weights, p + ".mix", m, eps, latents[src])
        elif layer["type"] == "mamba1":
            y = mamba1(h, weights, p + ".mix", m)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + moe(h, weights, p + ".mlp", layer["mlp"])
        x = x + y
        after.append(x)
    h = layer_norm(x, _w(weights, "final.norm"), _w(weights, "final.norm.b"), eps)
    logits = h @ _w(weights, "head").T * config["logit_scale"]
    return (logits, torch.stack(after)) if return_layers else logits


def greedy_generate(weights, config, prompt: List[int], count: int) -> List[int]:
    tokens, out = list(prompt), []
    for _ in range(count):
        nxt = int(forward(weights, config, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out
