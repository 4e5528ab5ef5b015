"""The kernels of a routed feed-forward (``csrc/kernels/moe.hip``) as Python functions: the
choice of experts per token, and the chosen gated units of all tokens in one pass.

Nothing here waits for the device: which rows go to which expert is sorted out by a kernel,
and the products walk tiles of rows that have one expert each."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import lib
from .lib import KernelError

_DT = {torch.float32: 0, torch.bfloat16: 1}

# Steps with at most this many (token, expert) pairs, or at most 16 pairs per expert on average,
# take tiles of 16 rows (an expert's weights are then streamed by waves that carry no padding
# rows through their products), larger ones of 64: a row's sums are the same either way.
SMALL_TILE_MAX_PAIRS = 256
SMALL_TILE_MAX_PAIRS_PER_EXPERT = 16
# bfloat16 steps with at least this many pairs per expert on average take tiles of 128 rows that
# are staged through LDS (another matrix instruction: a row's sums agree to rounding).
LARGE_TILE_MIN_PAIRS_PER_EXPERT = 96


def router_logits(resid: torch.Tensor, norm_weight: torch.Tensor, norm_bias: torch.Tensor,
                  eps: float, w_router: torch.Tensor) -> torch.Tensor:
    """``layer_norm(resid) @ w_router.T`` in float32 from the float32 residual rows ``(T, W)``:
    the router's logits on the unrounded normalised input.  Norm weight, bias and the router's
    weight ``(E, W)`` share a dtype (float32 or bfloat16)."""
    if not resid.is_cuda or resid.dtype != torch.float32 or resid.dim() != 2 \
            or not resid.is_contiguous():
        raise KernelError("router_logits: the residual must be contiguous float32 (T, W)")
    T, W = resid.shape
    E = w_router.shape[0]
    for t, shape, what in ((norm_weight, (W,), "norm weight"), (norm_bias, (W,), "norm bias"),
                           (w_router, (E, W), "router weight")):
        if tuple(t.shape) != shape or t.dtype != w_router.dtype or not t.is_contiguous() \
                or t.dtype not in _DT:
            raise KernelError(f"router_logits: the {what} must be contiguous {shape} of the "
                              "router weight's dtype")
    z = torch.empty((T, E), dtype=torch.float32, device=resid.device)
    lib.call("rlis_moe_router_logits", resid.data_ptr(), norm_weight.data_ptr(),
             norm_bias.data_ptr(), float(eps), w_router.data_ptr(), _DT[w_router.dtype],
             z.data_ptr(), T, W, E, lib.stream_ptr())
    return z


def route(logits: torch.Tensor, correction: Optional[torch.Tensor], groups: int, keep: int,
          top: int, scale: float, scores: str = "sigmoid", group_score: str = "top2",
          renormalise: bool = False, bias: Optional[torch.Tensor] = None
          ) -> Tuple[torch.Tensor, torch.Tensor]:
    """From router logits ``(T, E)`` float32: scores ``s = sigmoid(logits)`` (``scores``
    "softmax": their softmax over all experts), choice scores ``s + correction`` (None: no
    correction); experts stand in ``groups`` equal groups of neighbours, a group's score
    is the sum of its two largest choice scores (``group_score`` "max": the largest), and only
    experts of the ``keep`` best groups can be chosen; the ``top`` largest choice scores win.
    Returns the chosen experts ``(T, top)`` int32 and their weights ``(T, top)`` float32:
    ``s * scale``, with ``renormalise`` divided by their sum + 1e-20.  ``bias`` (float32, one per
    expert): added to the logits in front of everything else.  (Softmax scores that are
    renormalised are the softmax over the chosen logits alone.)"""
    if not logits.is_cuda or logits.dtype != torch.float32 or logits.dim() != 2 \
            or (logits.shape[1] > 1 and logits.stride(1) != 1):
        raise KernelError("route: the logits must be float32 (T, E) on the GPU")
    T, E = logits.shape
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != E
                                   or not correction.is_contiguous()):
        raise KernelError(f"route: the correction must be {E} float32 values")
    if scores not in ("sigmoid", "softmax") or group_score not in ("top2", "max"):
        raise KernelError(f"route: unknown scores '{scores}' or group score '{group_score}'")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != E
                             or not bias.is_contiguous() or not bias.is_cuda):
        raise KernelError(f"route: the bias must be {E} float32 values")
    ldz = logits.stride(0) if T > 1 else max(logits.stride(0), E)
    chosen = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    lib.call("rlis_moe_route", logits.data_ptr(), ldz,
             None if correction is None else correction.data_ptr(), T, E, int(groups),
             int(keep), int(top), float(scale), chosen.data_ptr(), weights.data_ptr(),
             int(scores == "softmax"), int(group_score == "max"), int(bool(renormalise)),
             None if bias is None else bias.data_ptr(), lib.stream_ptr())
    return chosen, weights


def routed_units(x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                 chosen: torch.Tensor, weights: torch.Tensor,
                 addend: Optional[torch.Tensor] = None, limit: float = 0.0,
                 alpha: float = 1.0, plain: bool = False) -> torch.Tensor:
    """``out[t] = sum_k weights[t, k] * unit(chosen[t, k], x[t])  (+ addend[t])`` in float32,
    where unit ``e`` is ``Wd[e] (silu(Wg[e] x) * (Wu[e] x))`` with ``w_gate_up (E, 2 F, W)``
    (an expert's gate rows in front of its up rows) and ``w_down (E, W, F)``, both in the dtype
    of ``x (T, W)``.  A token's units are added in the order of its choices.  ``limit`` > 0: the
    units are of the bounded kind, ``Wd[e] (g sigmoid(alpha g) (u + 1))`` with
    ``g = min(Wg[e] x, limit)`` and ``u = clamp(Wu[e] x, -limit, limit)``.  ``plain``: the units
    are not gated, ``Wd[e] relu(Wu[e] x)^2`` with ``w_gate_up (E, F, W)`` the one projection
    ``Wu`` (an even number of rows) and ``w_down (E, W, F)``."""
    if not x.is_cuda or x.dim() != 2 or x.dtype not in _DT or (x.shape[1] > 1 and x.stride(1) != 1):
        raise KernelError("routed_units: x must be (T, W) on the GPU with contiguous rows")
    T, W = x.shape
    E, F2, W2 = w_gate_up.shape
    F = F2 // 2
    inner = F2 if plain else F          # columns of a hidden row
    if W2 != W or F2 % 2 or tuple(w_down.shape) != (E, W, inner) or w_gate_up.dtype != x.dtype \
            or w_down.dtype != x.dtype or not w_gate_up.is_contiguous() \
            or not w_down.is_contiguous():
        raise KernelError("routed_units: the experts' weights do not match x")
    top = chosen.shape[1]
    if chosen.dtype != torch.int32 or tuple(chosen.shape) != (T, top) \
            or not chosen.is_contiguous() or weights.dtype != torch.float32 \
            or tuple(weights.shape) != (T, top) or not weights.is_contiguous():
        raise KernelError("routed_units: chosen (int32) and weights (float32) must be (T, top)")
    out = torch.empty((T, W), dtype=torch.float32, device=x.device)
    if T == 0:
        return out
    P = T * top
    rows = 16 if P <= max(SMALL_TILE_MAX_PAIRS, SMALL_TILE_MAX_PAIRS_PER_EXPERT * E) else 64
    if x.dtype == torch.bfloat16 and P >= LARGE_TILE_MIN_PAIRS_PER_EXPERT * E and W % 8 == 0 \
            and inner % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0:
        rows = 128
    tiles = min(P, -(-(P + E * (rows - 1)) // rows))
    order = torch.empty(tiles * rows, dtype=torch.int32, device=x.device)
    tile_expert = torch.empty(tiles, dtype=torch.int32, device=x.device)
    lib.call("rlis_moe_sort", chosen.data_ptr(), P, E, rows, tiles, order.data_ptr(),
             tile_expert.data_ptr(), lib.stream_ptr())
    hidden = torch.empty((tiles * rows, inner), dtype=x.dtype, device=x.device)
    y = torch.empty((P, W), dtype=torch.float32, device=x.device)
    ldx = x.stride(0) if T > 1 else max(x.stride(0), W)
    lib.call("rlis_moe_experts", x.data_ptr(), _DT[x.dtype], ldx, w_gate_up.data_ptr(),
             w_down.data_ptr(), order.data_ptr(), tile_expert.data_ptr(), weights.data_ptr(),
             rows, tiles, top, F, W, hidden.data_ptr(), y.data_ptr(), float(limit),
             -1.0 if plain else float(alpha), lib.stream_ptr())
    if addend is not None and (tuple(addend.shape) != (T, W) or not addend.is_contiguous()
                               or addend.dtype not in _DT):
        raise KernelError("routed_units: the addend must be a contiguous (T, W) tensor")
    lib.call("rlis_moe_combine", out.data_ptr(), y.data_ptr(),
             None if addend is None else addend.data_ptr(),
             0 if addend is None else _DT[addend.dtype], T, top, W, lib.stream_ptr())
    return out
