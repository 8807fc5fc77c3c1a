"""A plain, slow implementation of the Gipotar decoder, one function per mechanism, written
from the design's equations and sharing nothing with the engine: token by token, in the
precision of the tensors it is given (the tests hand it float64).  It is the oracle that the
engine's kernels, cache and state handling are held against.

Notation.  ``x`` is the residual stream (T, W); a linear weight is (out, in) and applied as
``x @ W.T``; ``rms(x) = x / sqrt(mean(x^2) + eps)``.

    layer:      x += m * mixer(norm1(x));  x += m * ff(norm2(x))   (the second only with a ff)
    norm:       rms(x) * (1 + w)
    parallel:   a_l * attention(h) + a_r * timemix(h)
    delta:      gated delta rule
    ff:         down((g * sigmoid(1.702 g)) * (u + 1)), g = min(gate h, L), u = clamp(up h, -L, L)
    output:     c * tanh(head(norm(x)) / c)
"""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * (1.0 + w)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def rotate(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x: (T, heads, d).  The first ``dims`` of every head turn: dim i pairs with i + dims/2,
    by the angle position * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    ang = positions.to(torch.float64).reshape(-1, 1, 1) * freq.reshape(1, 1, -1)
    c, s = torch.cos(ang).to(x.dtype), torch.sin(ang).to(x.dtype)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: Dict[str, Any]) -> torch.Tensor:
    """Causal softmax attention with grouped heads, keys of size ``dim``, values of ``vdim``."""
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    pos = torch.arange(T)
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    q = rotate(q, pos, p["rot"]["dims"], p["rot"]["base"])
    k = rotate(k, pos, p["rot"]["dims"], p["rot"]["base"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, head]) * p["scale"]
            a = torch.softmax(s, dim=0)
            out[t, head] = a @ v[:t + 1, g]
    return out.reshape(T, H * dv) @ w["o"].T


def time_mix(h: torch.Tensor, w: Dict[str, torch.Tensor], p: Dict[str, Any], eps: float
             ) -> torch.Tensor:
    """Token-shift mixes, a decay per key channel, a matrix state per head with a bonus for the
    current token, unit-rms heads, a gate."""
    T, W = h.shape
    H, d = p["heads"], p["dim"]
    prev = torch.cat([torch.zeros(1, W, dtype=h.dtype), h[:-1]], dim=0)

    def mix(s):
        return h + (prev - h) * w["mu." + s]

    r = (mix("r") @ w["r"].T).reshape(T, H, d)
    k = (mix("k") @ w["k"].T).reshape(T, H, d)
    v = (mix("v") @ w["v"].T).reshape(T, H, d)
    gate = silu(mix("g") @ w["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ w["w1"].T) @ w["w2"].T + w["w0"]))
    decay = decay.reshape(T, H, d)
    out = decayed_state(r, k, v, decay, w["u"].reshape(H, d))
    out = rms(out, eps).reshape(T, H * d) * w["norm"] * gate
    return out @ w["o"].T


def decayed_state(r, k, v, decay, bonus, S=None):
    """Per head a matrix S [key channel][value channel]: the token reads
    ``(S + diag(bonus) k v^T)^T r``, then ``S <- diag(decay) S + k v^T``.
    r, k, v, decay: (T, H, d); bonus (H, d).  ``S`` (H, d, d) is changed in place when given."""
    T, H, d = r.shape
    S = torch.zeros(H, d, d, dtype=r.dtype) if S is None else S
    out = torch.zeros(T, H, d, dtype=r.dtype)
    for t in range(T):
        for head in range(H):
            kv = torch.outer(k[t, head], v[t, head])
            out[t, head] = (S[head] + bonus[head].reshape(-1, 1) * kv).T @ r[t, head]
            S[head] = decay[t, head].reshape(-1, 1) * S[head] + kv
    return out


def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x: (T, C); taps: (C, K), the last column multiplies the current token."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], dim=0)
    out = torch.zeros_like(x)
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j]
    return out


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def gated_delta(h: torch.Tensor, w: Dict[str, torch.Tensor], p: Dict[str, Any], eps: float
                ) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = silu(short_conv(h @ w["q"].T, w["q.conv"])).reshape(T, G, d)
    k = silu(short_conv(h @ w["k"].T, w["k.conv"])).reshape(T, G, d)
    v = silu(short_conv(h @ w["v"].T, w["v.conv"])).reshape(T, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    beta = torch.sigmoid(h @ w["b"].T)                                     # (T, H)
    g = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    out = delta_state(q, k, v, beta, g)
    gate = silu(h @ w["g"].T).reshape(T, H, dv)
    out = rms(out, eps) * w["norm"] * gate
    return out.reshape(T, H * dv) @ w["o"].T


def delta_state(q, k, v, beta, g, S=None):
    """Per head a matrix S [key channel][value channel]: ``S <- g S``, then the token replaces
    what its key reads, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, and reads ``S^T q``.
    q, k: (T, G, d); v: (T, H, dv); beta, g: (T, H); head h uses q/k head ``h // (H / G)``."""
    T, G, d = q.shape
    H, dv = v.shape[1], v.shape[2]
    S = torch.zeros(H, d, dv, dtype=q.dtype) if S is None else S
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        for head in range(H):
            j = head // (H // G)
            S[head] = g[t, head] * S[head]
            u = beta[t, head] * (v[t, head] - S[head].T @ k[t, j])
            S[head] = S[head] + torch.outer(k[t, j], u)
            out[t, head] = S[head].T @ q[t, j]
    return out


def clamped_glu(h: torch.Tensor, w: Dict[str, torch.Tensor], limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    n = len(prefix) + 1
    return {k[n:]: v for k, v in weights.items() if k.startswith(prefix + ".")}


def forward(config: Dict[str, Any], weights: Dict[str, torch.Tensor], tokens: List[int],
            layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits (T, vocab) for one sequence from its first token on.  ``layers_out`` collects the
    residual stream after every layer."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = weights["embed"][torch.tensor(tokens)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        name = f"l{i}"
        h = offset_norm(x, weights[name + ".norm1"], eps)
        mp = layer["mixer"]
        if layer["type"] == "parallel":
            y = mp["left_scale"] * attention(h, sub(weights, name + ".mix.left"), mp["left"]) \
                + mp["right_scale"] * time_mix(h, sub(weights, name + ".mix.right"), mp["right"], eps)
        elif layer["type"] == "delta":
            y = gated_delta(h, sub(weights, name + ".mix"), mp, eps)
        else:
            raise ValueError(layer["type"])
        x = x + m * y
        if layer["mlp"] is not None:
            h = offset_norm(x, weights[name + ".norm2"], eps)
            x = x + m * clamped_glu(h, sub(weights, name + ".mlp"), layer["mlp"]["limit"])
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = offset_norm(x, weights["final.norm"], eps) @ weights["head"].T
    cap = config["logit_softcap"]
    return cap * torch.tanh(logits / cap)


def greedy(config: Dict[str, Any], weights: Dict[str, torch.Tensor], prompt: List[int],
           new_tokens: int):
    """Greedy continuation, each token from a full forward pass; returns the tokens and, per
    pick, the margin between the best and the second logit."""
    tokens, margins = list(prompt), []
    for _ in range(new_tokens):
        last = forward(config, weights, tokens)[-1]
        top = torch.topk(last, 2).values
        margins.append(float(top[0] - top[1]))
        tokens.append(int(torch.argmax(last)))
    return tokens[len(prompt):], margins
