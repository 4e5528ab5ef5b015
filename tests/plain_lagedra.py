"""The Lagedra decoder in plain, slow torch (float64, one sequence at a time, no cache): what
the engine is held against.  One function per mechanism; nothing here is shared with the
package.  ``config`` is the dict that config.json holds, ``w`` maps tensor names to tensors.

A layer reads one stream x and adds both of its sublayers to it, each behind a norm of its
own: ``y = x + mixer(n1(x)) + ff(n2(x))``; what the next layer reads is a learned mix of the
embedding output and of every layer's y so far.  Mixers: linear attention with a fixed decay per
head (``lightning``), or windowed softmax attention behind short convolutions (``attention``).
"""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def _w(w: Dict[str, torch.Tensor], name: str) -> torch.Tensor:
    return w[name].to(F64)


# ------------------------------------------------------------------------------- pieces
def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose weight is one number for all coordinates."""
    return rms_unit(x, eps) * g.reshape(())


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def embed(w: Dict[str, torch.Tensor], tokens: List[int], start: int = 0) -> torch.Tensor:
    ids = torch.tensor(tokens, dtype=torch.long)
    pos = torch.arange(start, start + len(tokens))
    return _w(w, "embed")[ids] + _w(w, "pos")[pos]


def short_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """y[t, c] = sum_j taps[c, j] * u[t - (K - 1) + j, c], zeros in front of the sequence."""
    T, C = u.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros((K - 1, C), dtype=u.dtype), u], dim=0)
    y = torch.zeros_like(u)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y


def rotary_tables(rot: Dict[str, Any], positions: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos and sin ``(T, dims / 2)`` with the stretched frequencies and their magnitude."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, original = float(sc["factor"]), float(sc["original"])

        def turn_dim(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = positions.to(F64).reshape(-1, 1) * f.reshape(1, -1)
    return torch.cos(ang) * mag, torch.sin(ang) * mag


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, dims: int) -> torch.Tensor:
    """x ``(T, heads, d)``: dim i is paired with dim i + dims / 2; the rest passes."""
    half = dims // 2
    a, b, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)


# ------------------------------------------------------------------------------- mixers
def lightning_mixer(w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], h: torch.Tensor,
                    eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ _w(w, p + ".q").T).reshape(T, H, d)
    k = silu(h @ _w(w, p + ".k").T).reshape(T, H, d)
    v = silu(h @ _w(w, p + ".v").T).reshape(T, H, dv)
    o = torch.zeros((T, H, dv), dtype=F64)
    for hd in range(H):
        lam = float(m["decay"][hd])
        S = torch.zeros((d, dv), dtype=F64)
        for t in range(T):
            S = lam * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms_unit(o.reshape(T, H * dv), eps) * _w(w, p + ".norm")
    y = y * torch.sigmoid(h @ _w(w, p + ".g").T)
    return y @ _w(w, p + ".o").T


def attention_values(w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], h: torch.Tensor
                     ) -> torch.Tensor:
    """The layer's own values behind their convolution, ``(T, kv_heads * vdim)``."""
    return short_conv(h @ _w(w, p + ".v").T, _w(w, p + ".v.conv"))


def attention_mixer(w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], h: torch.Tensor,
                    v_first: Optional[torch.Tensor], start: int = 0) -> torch.Tensor:
    """``v_first``: the values of the first value-mixing layer for the same tokens, or None
    when this layer is that one (or mixes nothing)."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = short_conv(h @ _w(w, p + ".q").T, _w(w, p + ".q.conv")).reshape(T, H, d)
    k = short_conv(h @ _w(w, p + ".k").T, _w(w, p + ".k.conv")).reshape(T, G, d)
    v = attention_values(w, p, m, h)
    if v_first is not None:
        lam = _w(w, p + ".vmix").reshape(())
        v = (1.0 - lam) * v + lam * v_first
    v = v.reshape(T, G, dv)
    pos = torch.arange(start, start + T)
    rot = m["rot"]
    cos, sin = rotary_tables(rot, pos)
    q, k = rotate(q, cos, sin, int(rot["dims"])), rotate(k, cos, sin, int(rot["dims"]))
    temp = _w(w, p + ".temp")
    cap, size = float(m["softcap"]), int(m["mask"]["size"])
    i, j = pos.reshape(-1, 1), pos.reshape(1, -1)
    seen = (i - j >= 0) & (i - j < size)
    out = torch.zeros((T, H, dv), dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"]) * temp[hd]
        s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, -math.inf)
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    return out.reshape(T, H * dv) @ _w(w, p + ".o").T


# ------------------------------------------------------------------------- feed-forwards
def dense_ff(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return gelu_tanh(h @ _w(w, p + ".up").T) @ _w(w, p + ".down").T


def expert(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor, limit: float) -> torch.Tensor:
    g = (h @ _w(w, p + ".gate").T).clamp(max=limit)
    u = (h @ _w(w, p + ".up").T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _w(w, p + ".down").T


def route(z: torch.Tensor, router: Dict[str, Any]) -> Tuple[List[List[int]], torch.Tensor]:
    """Per row of logits: the chosen experts and their weights."""
    E, top = int(router["experts"]), int(router["top"])
    count, keep = int(router["groups"]["count"]), int(router["groups"]["keep"])
    s = torch.softmax(z, dim=-1)
    per = E // count
    chosen, weights = [], []
    for t in range(z.shape[0]):
        best = s[t].reshape(count, per).max(dim=1).values
        kept = sorted(range(count), key=lambda g: (-float(best[g]), g))[:keep]
        allowed = [e for e in range(E) if e // per in kept]
        picks = sorted(allowed, key=lambda e: (-float(s[t, e]), e))[:top]
        sc = torch.stack([s[t, e] for e in picks])
        chosen.append(picks)
        weights.append(sc / (sc.sum() + 1e-20))
    return chosen, torch.stack(weights)


def moe_ff(w: Dict[str, torch.Tensor], p: str, mlp: Dict[str, Any], h: torch.Tensor) -> torch.Tensor:
    z = h @ _w(w, p + ".router").T
    chosen, weights = route(z, mlp["router"])
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for n, e in enumerate(chosen[t]):
            out[t] = out[t] + weights[t, n] * expert(w, f"{p}.e{e}", h[t:t + 1], limit)[0]
    return out


# ------------------------------------------------------------------------------ the model
def forward(config: Dict[str, Any], w: Dict[str, torch.Tensor], tokens: List[int]
            ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Logits ``(T, vocab)`` and the stream after every layer ``(layers, T, width)`` for one
    whole sequence."""
    eps = float(config["norm"]["eps"])
    x = embed(w, tokens)
    history = [x]
    v_first = None
    after = []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h1 = scalar_norm(x, _w(w, p + ".norm1"), eps)
        if layer["type"] == "lightning":
            mixed = lightning_mixer(w, p + ".mix", m, h1, eps)
        elif layer["type"] == "attention":
            if m.get("v_mix"):
                mixed = attention_mixer(w, p + ".mix", m, h1, v_first)
                if v_first is None:
                    v_first = attention_values(w, p + ".mix", m, h1)
            else:
                mixed = attention_mixer(w, p + ".mix", m, h1, None)
        else:
            raise ValueError(layer["type"])
        y = x + mixed
        mlp = layer.get("mlp")
        if mlp is not None:
            h2 = scalar_norm(x, _w(w, p + ".norm2"), eps)
            y = y + (dense_ff(w, p + ".mlp", h2) if mlp["kind"] == "dense"
                     else moe_ff(w, p + ".mlp", mlp, h2))
        history.append(y)
        mix = _w(w, p + ".dwa")
        x = sum(mix[j] * history[j] for j in range(len(history)))
        after.append(x)
    out = scalar_norm(x, _w(w, "final.norm"), eps)
    return out @ _w(w, "head").T, torch.stack(after)
