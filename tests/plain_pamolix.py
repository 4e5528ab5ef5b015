"""The Pamolix decoder written out plainly in torch (float64 by default), one function per
mechanism, for tests to hold the engine against.  It shares nothing with the package: it reads
a config.json dictionary and a dictionary of tensors by their checkpoint names, and runs whole
sequences without a cache.

Notation: ``x`` is a sequence of rows ``(n, width)``; positions count from 0.
"""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Every row divided by the root of (its mean square plus eps)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' norm: the stored weight is the distance from one."""
    return rms(x, eps) * (1.0 + w)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0.0) ** 2


def query_temperature(n: int, coef: float, every: int, dtype) -> torch.Tensor:
    """The factor of the queries at positions 0 .. n - 1: 1 + coef ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(n, dtype=torch.int64)
    steps = torch.div(p + 1, every, rounding_mode="floor").to(dtype)
    return 1.0 + coef * torch.log(steps + 1.0)


def rotate_half_pairs(x: torch.Tensor, dims: int, base: float, factor: float) -> torch.Tensor:
    """``x (n, heads, size)``: the first ``dims`` numbers of every head turned by the position's
    angles, number i paired with number i + dims / 2; frequency i is base^(-2 i / dims) / factor."""
    n, half = x.shape[0], dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims) / factor
    angle = torch.arange(n, dtype=x.dtype).reshape(n, 1) * freq.reshape(1, half)
    c, s = torch.cos(angle).unsqueeze(1), torch.sin(angle).unsqueeze(1)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def visible(n: int, size: Optional[int], keep_first: int) -> torch.Tensor:
    """``(n, n)`` booleans: may query i (rows) see key j (columns)?  Causal; with a window of
    ``size`` a key is seen when it is fewer than ``size`` positions back or among the first
    ``keep_first`` of the sequence."""
    i = torch.arange(n).reshape(n, 1)
    j = torch.arange(n).reshape(1, n)
    ok = j <= i
    if size is not None:
        ok = ok & ((i - j < size) | (j < keep_first))
    return ok


def softmax_rows(scores: torch.Tensor, ok: torch.Tensor, sink: Optional[torch.Tensor]
                 ) -> torch.Tensor:
    """``scores (heads, n, n)`` -> weights of the visible keys.  ``sink (heads)``: every row's
    denominator also holds e^sink of its head, which stands for no key."""
    scores = scores.masked_fill(~ok, float("-inf"))
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.reshape(-1, 1, 1))
    e = torch.exp(scores - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink.reshape(-1, 1, 1) - top)
    return e / total


def _heads(x: torch.Tensor, heads: int) -> torch.Tensor:
    return x.reshape(x.shape[0], heads, -1)


def _attend(q, k, v, scale, ok, sink, softcap):
    """q ``(n, H, d)``, k ``(n, G, d)``, v ``(n, G, dv)`` -> ``(n, H * dv)``."""
    H, G = q.shape[1], k.shape[1]
    rep = H // G
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if softcap:
        scores = softcap * torch.tanh(scores / softcap)
    w = softmax_rows(scores, ok, sink)
    return torch.einsum("hij,jhd->ihd", w, vv)


def attention_keys_values(h: torch.Tensor, m: Dict[str, Any], w: Dict[str, torch.Tensor],
                          pre: str, eps: float):
    """Keys (normalised) and values of the first kind of attention, as its cache holds them."""
    G = m["kv_heads"]
    k = _heads(h @ w[pre + "k"].T + w[pre + "k.b"], G)
    v = _heads(h @ w[pre + "v"].T + w[pre + "v.b"], G)
    return rms(k, eps) * w[pre + "k.norm"], v


def attention(h: torch.Tensor, m: Dict[str, Any], w: Dict[str, torch.Tensor], pre: str,
              eps: float, kv=None) -> torch.Tensor:
    """The mixer 'attention': biased projections, a norm over every query and key head, queries
    times a factor that grows with the position, all earlier keys, a sink per head."""
    n, H = h.shape[0], m["heads"]
    q = _heads(h @ w[pre + "q"].T + w[pre + "q.b"], H)
    q = rms(q, eps) * w[pre + "q.norm"]
    if m.get("q_temp"):
        q = q * query_temperature(n, m["q_temp"]["coef"], m["q_temp"]["every"],
                                  h.dtype).reshape(n, 1, 1)
    k, v = kv if kv is not None else attention_keys_values(h, m, w, pre, eps)
    out = _attend(q, k, v, m["scale"], visible(n, None, 0), w[pre + "sink"], None)
    return out.reshape(n, -1) @ w[pre + "o"].T


def _rotated(x: torch.Tensor, m: Dict[str, Any]) -> torch.Tensor:
    rot = m.get("rot")
    if not rot:
        return x
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    return rotate_half_pairs(x, rot["dims"], rot["base"], factor)


def attention_2_keys_values(h: torch.Tensor, m: Dict[str, Any], w: Dict[str, torch.Tensor],
                            pre: str):
    """Keys (rotated) and values of the second kind of attention, as its cache holds them."""
    G = m["kv_heads"]
    return _rotated(_heads(h @ w[pre + "k"].T, G), m), _heads(h @ w[pre + "v"].T, G)


def attention_2(h: torch.Tensor, m: Dict[str, Any], w: Dict[str, torch.Tensor], pre: str,
                kv=None) -> torch.Tensor:
    """The mixer 'attention_2': rotated queries and keys, capped scores, a window that also
    keeps the sequence's first keys, a gate per head on the output; ``kv``: another layer's
    keys and values in place of its own."""
    n, H = h.shape[0], m["heads"]
    q = _rotated(_heads(h @ w[pre + "q"].T, H), m)
    k, v = kv if kv is not None else attention_2_keys_values(h, m, w, pre)
    mask = m.get("mask") or {}
    ok = visible(n, mask.get("size"), mask.get("keep_first", 0))
    out = _attend(q, k, v, m["scale"], ok, None, m.get("softcap"))
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    out = out * gate.unsqueeze(-1)
    return out.reshape(n, -1) @ w[pre + "o"].T


def dense(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    return gelu_erf(h @ w[pre + "up"].T) @ w[pre + "down"].T


def mixture(h: torch.Tensor, mlp: Dict[str, Any], w: Dict[str, torch.Tensor], pre: str
            ) -> torch.Tensor:
    """Every row takes the ``top`` experts with the largest router logits, weighted by the
    softmax over those logits alone."""
    top = mlp["router"]["top"]
    z = h @ w[pre + "router"].T + w[pre + "router.b"]
    best, chosen = torch.topk(z, top, dim=-1)
    share = torch.softmax(best, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for r in range(top):
            e = int(chosen[t, r])
            y = relu_squared(h[t] @ w[f"{pre}e{e}.up"].T) @ w[f"{pre}e{e}.down"].T
            out[t] = out[t] + share[t, r] * y
    return out


def forward(config: Dict[str, Any], weights: Dict[str, torch.Tensor], tokens: List[int],
            dtype=torch.float64, layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits ``(n, vocab)`` of a whole sequence.  ``layer_outputs``: a list that receives the
    sum of the streams behind every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    S = config.get("streams")
    x0 = w["embed"][torch.tensor(tokens)] * config["embedding"]["scale"]
    lanes = [x0.clone() for _ in range(S or 1)]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}."
        m = layer["mixer"]

        def mixer(h):
            if m.get("kv_from") is not None:
                kv = kept[m["kv_from"]]
            elif layer["type"] == "attention":
                kv = attention_keys_values(h, m, w, pre + "mix.", eps)
            else:
                kv = attention_2_keys_values(h, m, w, pre + "mix.")
            kept[i] = kv
            if layer["type"] == "attention":
                return attention(h, m, w, pre + "mix.", eps, kv)
            return attention_2(h, m, w, pre + "mix.", kv)

        def feed(h):
            if layer["mlp"]["kind"] == "dense":
                return dense(h, w, pre + "mlp.")
            return mixture(h, layer["mlp"], w, pre + "mlp.")

        subs = [(1, mixer)] + ([(2, feed)] if layer.get("mlp") else [])
        for q, fn in subs:
            if S:
                a, b, c = (w[f"{pre}hc{q}.{n}"] for n in ("in", "out", "mix"))
                u = sum(a[s] * lanes[s] for s in range(S))
                y = fn(norm_around_zero(u, w[f"{pre}norm{q}"], eps))
                lanes = [sum(c[s, t] * lanes[s] for s in range(S)) + b[t] * y
                         for t in range(S)]
            else:
                lanes = [lanes[0] + fn(norm_around_zero(lanes[0], w[f"{pre}norm{q}"], eps))]
        if layer_outputs is not None:
            layer_outputs.append(sum(lanes))
    x = sum(lanes)
    return norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T
