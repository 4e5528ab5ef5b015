"""The kernels of mixers with a state of fixed size per request (``csrc/kernels/recurrent.hip``)
as Python functions: token shift, input tails, the short causal convolution, the two scans over
a matrix state per head, and the per-head norm with weight and gate behind them.

A ``state`` argument is a float32 view ``(slots, n)`` of the mixer's area in the runner's state
buffer (rows a whole slot apart); ``cu``, ``slots`` and ``seq_of_token`` are the step's
cumulative token counts, state slots and sequence of each token, int32 on the device.  Every
function checks on the host what its kernel and grid assume."""
from __future__ import annotations

from typing import Optional

import torch

from . import lib
from .lib import KernelError

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype} (float32 and bfloat16 only)") from None


def _state(state: torch.Tensor, need: int, what: str) -> int:
    if not state.is_cuda or state.dtype != torch.float32 or state.dim() != 2:
        raise KernelError(f"{what}: the state must be a float32 (slots, n) view on the GPU")
    if state.shape[1] < need or (state.shape[1] > 1 and state.stride(1) != 1):
        raise KernelError(f"{what}: the state holds {state.shape[1]} floats a slot, {need} needed")
    return state.stride(0) if state.shape[0] > 1 else max(state.stride(0), state.shape[1])


def _meta(t: torch.Tensor, n: int, what: str) -> int:
    if not t.is_cuda or t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < n:
        raise KernelError(f"{what}: needs {n} contiguous int32 entries on the GPU")
    return t.data_ptr()


def _rows(t: torch.Tensor, what: str, dtype=None) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if not t.is_cuda or t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: a 2-D tensor on the GPU with contiguous rows is needed")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{what}: expected {dtype}, got {t.dtype}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _vec(t: torch.Tensor, n: int, what: str) -> int:
    if not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise KernelError(f"{what}: needs {n} contiguous float32 values on the GPU, got "
                          f"{tuple(t.shape)} {t.dtype}")
    return t.data_ptr()


# A step with at least this many tokens per sequence on average takes the scans' tiled kernels
# (known from the host: the number of rows and of sequences).
TILED_SCAN_MIN_MEAN_TOKENS = 4


def _long_runs(T: int, num_seqs: int) -> bool:
    return T >= TILED_SCAN_MIN_MEAN_TOKENS * max(1, num_seqs)


def _scan_form(tiled, T: int, num_seqs: int) -> int:
    """The kernels' form argument: 0 the streaming kernel, 1 the tiled one (two value channels a
    wave where the grid is small, else four), 2 / 3 the tiled one with four / two channels a
    wave (``"wide"`` / ``"narrow"``, for tests)."""
    if tiled is None:
        tiled = _long_runs(T, num_seqs)
    return {False: 0, True: 1, "wide": 2, "narrow": 3}[tiled]


def shift_mix(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, seq_of_token: torch.Tensor,
              cu: torch.Tensor, slots: torch.Tensor, num_seqs: int) -> torch.Tensor:
    """``out[m] = x + (prev - x) * mu[m]`` for every row of ``x (T, W)``, ``prev`` being the row
    of the token before (for a sequence's first token of the step: the row kept in ``state``).
    Returns ``(mixes, T, W)`` in the dtype of ``x``."""
    if not x.is_cuda or x.dim() != 2 or not x.is_contiguous():
        raise KernelError("shift_mix: x must be a contiguous (T, W) tensor on the GPU")
    T, W = x.shape
    mixes = mu.shape[0]
    _vec(mu.reshape(-1), mixes * W, "shift_mix mu")
    stride = _state(state, W, "shift_mix")
    out = torch.empty((mixes, T, W), dtype=x.dtype, device=x.device)
    lib.call("rlis_shift_mix", out.data_ptr(), x.data_ptr(), _dt(x), mu.data_ptr(),
             state.data_ptr(), stride, _meta(seq_of_token, T, "seq_of_token"),
             _meta(cu, num_seqs + 1, "cu"), _meta(slots, num_seqs, "slots"), T, W, mixes,
             lib.stream_ptr())
    return out


def tail_update(state: torch.Tensor, x: torch.Tensor, channels: int, rows: int, cu: torch.Tensor,
                slots: torch.Tensor, num_seqs: int) -> None:
    """Every sequence's tail in ``state`` (``rows`` rows of ``channels`` floats, oldest first)
    becomes the last ``rows`` of (its old tail, then the step's rows of ``x[:, :channels]``)."""
    ldx = _rows(x, "tail_update x")
    if x.shape[1] < channels:
        raise KernelError(f"tail_update: x has {x.shape[1]} columns, {channels} needed")
    stride = _state(state, channels * rows, "tail_update")
    lib.call("rlis_tail_update", state.data_ptr(), stride, x.data_ptr(), _dt(x), ldx, channels,
             rows, _meta(cu, num_seqs + 1, "cu"), _meta(slots, num_seqs, "slots"), num_seqs,
             lib.stream_ptr())


def causal_conv(x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor,
                seq_of_token: torch.Tensor, cu: torch.Tensor, slots: torch.Tensor, num_seqs: int,
                unit_channels: int = 0, unit_group: int = 0, scaled_channels: int = 0,
                scale: float = 1.0, unit_eps: float = 0.0, rest_group: int = 256,
                bias: Optional[torch.Tensor] = None,
                out_dtype: torch.dtype = torch.float32, activation: bool = True,
                blend: Optional[torch.Tensor] = None, blend_from: int = 0,
                blend_weight: float = 0.0) -> torch.Tensor:
    """``silu`` of the causal convolution over time of the first ``C`` columns of ``x`` (float32)
    with ``taps (C, K)`` (the last column multiplies the current row; the ``K - 1`` rows in
    front of the step come from ``state``), plus ``bias (C)`` under the ``silu`` when given;
    without ``activation`` the convolution as it is.  With ``blend`` (rows of the same tokens in
    ``out_dtype``, ``C - blend_from`` columns) the channels from ``blend_from`` on become
    ``(1 - blend_weight) * y + blend_weight * blend``.  Channels below ``unit_channels`` are then made
    unit vectors in groups of ``unit_group``: ``y / sqrt(sum y^2 + unit_eps)``, those below
    ``scaled_channels`` times ``scale``.  Returns ``(T, C)`` in ``out_dtype`` (float32 arithmetic)."""
    ldx = _rows(x, "causal_conv x", torch.float32)
    C, K = taps.shape
    _vec(taps.reshape(-1), C * K, "causal_conv taps")
    if x.shape[1] < C:
        raise KernelError(f"causal_conv: x has {x.shape[1]} columns, the taps {C} channels")
    T = x.shape[0]
    stride = _state(state, C * (K - 1), "causal_conv")
    out = torch.empty((T, C), dtype=out_dtype, device=x.device)
    blend_ptr, ld_blend = None, 0
    if blend is not None:
        ld_blend = _rows(blend, "causal_conv blend", out_dtype)
        if blend.shape[0] != T or blend.shape[1] != C - blend_from or not 0 <= blend_from < C:
            raise KernelError(f"causal_conv: rows to mix in of shape {tuple(blend.shape)} for "
                              f"channels {blend_from} to {C} of {T} tokens")
        blend_ptr = blend.data_ptr()
    lib.call("rlis_causal_conv", out.data_ptr(), _DT[out_dtype], x.data_ptr(), ldx,
             taps.data_ptr(), None if bias is None else _vec(bias, C, "causal_conv bias"), C, K,
             state.data_ptr(), stride, _meta(seq_of_token, T, "seq_of_token"),
             _meta(cu, num_seqs + 1, "cu"), _meta(slots, num_seqs, "slots"), T,
             int(unit_channels), int(unit_group), int(scaled_channels), float(scale),
             float(unit_eps), int(rest_group), int(bool(activation)), blend_ptr, ld_blend,
             int(blend_from), float(blend_weight), lib.stream_ptr())
    return out


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b_raw: torch.Tensor,
               a_raw: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
               state: torch.Tensor, cu: torch.Tensor, slots: torch.Tensor, num_seqs: int,
               heads: int, kv_heads: int, dk: int, dv: int,
               tiled=None) -> torch.Tensor:
    """The gated delta rule over every sequence's tokens of the step.  ``q``, ``k``
    ``(T, kv_heads * dk)`` and ``v (T, heads * dv)`` are float32 column ranges of one matrix
    (one row stride), ``b_raw``, ``a_raw`` ``(T, heads)`` of another; per token and head
    ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` with
    ``g = exp(-exp(a_log) * softplus(a_raw + dt_bias))`` and ``beta = sigmoid(b_raw)``.
    ``state (slots, heads * dv * dk)`` holds S as [head][value channel][key channel] and is
    left as after each sequence's last token.  Returns ``o (T, heads * dv)`` float32.
    ``tiled`` chooses the kernel that stages tiles of tokens through LDS (for steps in which a
    sequence brings many tokens; None: from four tokens per sequence on average); the two
    agree to rounding (the tiled kernel forms a token's four sums over the wave together)."""
    ld = _rows(q, "delta_scan q", torch.float32)
    if _rows(k, "delta_scan k", torch.float32) != ld or _rows(v, "delta_scan v", torch.float32) != ld:
        raise KernelError("delta_scan: q, k and v must share a row stride")
    ldba = _rows(b_raw, "delta_scan b", torch.float32)
    if _rows(a_raw, "delta_scan a", torch.float32) != ldba:
        raise KernelError("delta_scan: a and b must share a row stride")
    T = q.shape[0]
    if q.shape[1] != kv_heads * dk or k.shape != q.shape or v.shape != (T, heads * dv) \
            or b_raw.shape != (T, heads) or a_raw.shape != (T, heads):
        raise KernelError("delta_scan: operand shapes do not match the head counts and sizes")
    stride = _state(state, heads * dv * dk, "delta_scan")
    out = torch.empty((T, heads * dv), dtype=torch.float32, device=q.device)
    lib.call("rlis_delta_scan", out.data_ptr(), heads * dv, q.data_ptr(), k.data_ptr(),
             v.data_ptr(), ld, b_raw.data_ptr(), a_raw.data_ptr(), ldba,
             _vec(a_log, heads, "delta_scan A_log"), _vec(dt_bias, heads, "delta_scan dt_bias"),
             state.data_ptr(), stride, _meta(cu, num_seqs + 1, "cu"),
             _meta(slots, num_seqs, "slots"), num_seqs, heads, kv_heads, dk, dv,
             _scan_form(tiled, T, num_seqs), lib.stream_ptr())
    return out


def decay_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor,
               w0: torch.Tensor, bonus: torch.Tensor, state: torch.Tensor, cu: torch.Tensor,
               slots: torch.Tensor, num_seqs: int, heads: int, d: int,
               tiled=None) -> torch.Tensor:
    """A matrix state per head with a decay per key channel and a bonus for the current token:
    per token ``o = (S + diag(bonus) k v^T)^T r; S <- diag(w) S + k v^T`` with
    ``w = exp(-exp(z + w0))``.  ``r``, ``k``, ``v``, ``z`` are contiguous float32
    ``(T, heads * d)``; ``state (slots, heads * d * d)`` holds S as [head][value channel][key
    channel].  Returns ``o (T, heads * d)`` float32.  ``tiled`` as for ``delta_scan``."""
    T = r.shape[0]
    for name, t in (("r", r), ("k", k), ("v", v), ("z", z)):
        if not t.is_cuda or t.dtype != torch.float32 or t.shape != (T, heads * d) \
                or not t.is_contiguous():
            raise KernelError(f"decay_scan: {name} must be contiguous float32 (T, heads * d)")
    stride = _state(state, heads * d * d, "decay_scan")
    out = torch.empty((T, heads * d), dtype=torch.float32, device=r.device)
    lib.call("rlis_decay_scan", out.data_ptr(), r.data_ptr(), k.data_ptr(), v.data_ptr(),
             z.data_ptr(), heads * d, _vec(w0, heads * d, "decay_scan w0"),
             _vec(bonus.reshape(-1), heads * d, "decay_scan bonus"), state.data_ptr(), stride,
             _meta(cu, num_seqs + 1, "cu"), _meta(slots, num_seqs, "slots"), num_seqs, heads, d,
             _scan_form(tiled, T, num_seqs), lib.stream_ptr())
    return out


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, heads: int, dv: int,
                   eps: float, out_dtype: torch.dtype, sigmoid_gate: bool = False) -> torch.Tensor:
    """``o / sqrt(mean o^2 + eps)`` per head, times ``weight`` (``heads * dv`` values, or ``dv``
    shared by the heads), times ``silu(gate)`` (``sigmoid_gate``: times ``sigmoid(gate)``).  One
    head of all the channels is the norm over the heads together.  ``o`` contiguous float32 ``(T, heads * dv)``,
    ``gate`` of that shape with contiguous rows."""
    T = o.shape[0]
    if not o.is_cuda or o.dtype != torch.float32 or o.shape != (T, heads * dv) \
            or not o.is_contiguous():
        raise KernelError("head_norm_gate: o must be contiguous float32 (T, heads * dv)")
    ldg = _rows(gate, "head_norm_gate gate")
    if gate.shape != o.shape:
        raise KernelError("head_norm_gate: the gate must have the shape of o")
    if weight.numel() == heads * dv and heads > 1:
        wstride = dv
    elif weight.numel() == dv:
        wstride = 0
    else:
        raise KernelError(f"head_norm_gate: weight of {weight.numel()} values for {heads} heads "
                          f"of {dv}")
    _vec(weight.reshape(-1), weight.numel(), "head_norm_gate weight")
    out = torch.empty((T, heads * dv), dtype=out_dtype, device=o.device)
    lib.call("rlis_head_norm_gate", out.data_ptr(), _DT[out_dtype], o.data_ptr(),
             weight.data_ptr(), wstride, gate.data_ptr(), _dt(gate), ldg, T, heads, dv, float(eps),
             int(bool(sigmoid_gate)), lib.stream_ptr())
    return out


# A step of at least DECAY_CHUNKED_MIN_TOKENS tokens whose sequences bring at least
# DECAY_CHUNKED_MIN_MEAN_TOKENS each on average, or any step in which one sequence brings
# DECAY_CHUNKED_MIN_LONGEST (a portion beside decoded tokens: token by token it would take
# 0.8 us a token, however few the others are), takes the chunked form of the
# linear attention (chunks of DECAY_CHUNK_LEN tokens on the matrix cores, float32 products; heads
# of at most DECAY_CHUNKED_MAX_DIM channels); every other step walks token by token.  The two
# agree to rounding.  The rule looks at what the host knows: rows and sequences of the step and
# its longest portion.
DECAY_CHUNKED_MIN_TOKENS = 256
DECAY_CHUNKED_MIN_MEAN_TOKENS = 64
DECAY_CHUNKED_MIN_LONGEST = 64
DECAY_CHUNKED_MAX_DIM = 128
DECAY_CHUNK_LEN = 64


def decay_attention_chunked(T: int, num_seqs: int, dim: int, vdim: int, dtype: torch.dtype,
                            longest: Optional[int] = None) -> bool:
    if dtype != torch.float32 or max(dim, vdim) > DECAY_CHUNKED_MAX_DIM:
        return False
    if longest is not None and longest >= DECAY_CHUNKED_MIN_LONGEST:
        return True
    return (T >= DECAY_CHUNKED_MIN_TOKENS
            and T >= DECAY_CHUNKED_MIN_MEAN_TOKENS * max(1, num_seqs))


def decay_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor,
                    state: torch.Tensor, cu: torch.Tensor, slots: torch.Tensor, num_seqs: int,
                    heads: int, dim: int, vdim: int, activation: bool = True,
                    longest: Optional[int] = None) -> torch.Tensor:
    """Linear attention with a fixed decay per head: ``S <- decay[h] S + k v^T``, ``o = S^T q``
    (the token's own key and value are in what its query reads).  ``q``, ``k`` ``(T, heads *
    dim)`` and ``v`` ``(T, heads * vdim)`` are the raw projections of one dtype, with row
    strides; they pass SiLU in float32 on the way in (``activation``).  ``state``: per slot
    ``heads * vdim * dim`` float32, left as after each sequence's last token.  Returns
    ``(T, heads * vdim)`` float32.  Long portions take the chunked kernels
    (``decay_attention_chunked``; ``longest``: the most tokens a sequence brings, where known)."""
    T = q.shape[0]
    ldq, ldk, ldv = _rows(q, "decay_attention q"), _rows(k, "decay_attention k"), \
        _rows(v, "decay_attention v")
    if q.dtype != k.dtype or q.dtype != v.dtype or k.shape[0] != T or v.shape[0] != T \
            or q.shape[1] != heads * dim or k.shape[1] != heads * dim \
            or v.shape[1] != heads * vdim:
        raise KernelError("decay_attention: q, k (T, heads * dim) and v (T, heads * vdim) of one "
                          "dtype")
    stride = _state(state, heads * vdim * dim, "decay_attention")
    out = torch.empty((T, heads * vdim), dtype=torch.float32, device=q.device)
    if decay_attention_chunked(T, num_seqs, dim, vdim, q.dtype, longest):
        max_chunks = T // DECAY_CHUNK_LEN + num_seqs        # an upper bound, known on the host
        ws = torch.empty((max_chunks, heads * vdim * dim), dtype=torch.float32, device=q.device)
        lib.call("rlis_decay_attention_chunks", out.data_ptr(), q.data_ptr(), ldq, k.data_ptr(),
                 ldk, v.data_ptr(), ldv, _vec(decay, heads, "decay_attention decay"),
                 state.data_ptr(), stride, _meta(cu, num_seqs + 1, "cu"),
                 _meta(slots, num_seqs, "slots"), num_seqs, T, heads, dim, vdim,
                 int(bool(activation)), ws.data_ptr(), max_chunks, lib.stream_ptr())
        return out
    lib.call("rlis_decay_attention_scan", out.data_ptr(), q.data_ptr(), ldq, k.data_ptr(), ldk,
             v.data_ptr(), ldv, _dt(q), _vec(decay, heads, "decay_attention decay"),
             state.data_ptr(), stride, _meta(cu, num_seqs + 1, "cu"),
             _meta(slots, num_seqs, "slots"), num_seqs, T, heads, dim, vdim,
             int(bool(activation)), lib.stream_ptr())
    return out


# A step whose sequences bring at least this many tokens on average, and together at most this
# many channels, spreads a channel's states over sixteen lanes instead of four (known from the
# host: the number of rows and of sequences).
SPREAD_SCAN_MIN_MEAN_TOKENS = 64
SPREAD_SCAN_MAX_CHANNELS = 65536
# A step of at least CHUNKED_SCAN_MIN_TOKENS tokens whose sequences bring at least
# CHUNKED_SCAN_MIN_MEAN_TOKENS each on average walks chunks of CHUNKED_SCAN_LEN tokens side by
# side: every chunk from a zero state, the chunks' states joined in order, every chunk again from
# its true start state (the recurrence is linear in the state).  The result agrees with the
# sequential walk to rounding.
CHUNKED_SCAN_MIN_TOKENS = 512
CHUNKED_SCAN_MIN_MEAN_TOKENS = 128
CHUNKED_SCAN_LEN = 64


def selective_scan(x: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, b: torch.Tensor,
                   c: torch.Tensor, z: torch.Tensor, a_log: torch.Tensor, skip: torch.Tensor,
                   state: torch.Tensor, cu: torch.Tensor, slots: torch.Tensor,
                   num_seqs: int) -> torch.Tensor:
    """A state of ``N`` numbers per channel with an input-dependent step, over every sequence's
    tokens of the step: ``dt = softplus(dt_raw + dt_bias)``,
    ``S[ch][n] <- exp(dt * A[ch][n]) * S[ch][n] + dt * x[ch] * b[n]`` with ``A = -exp(a_log)``,
    ``y[ch] = sum_n S[ch][n] * c[n] + skip[ch] * x[ch]``, result ``y * silu(z)``.

    ``x (T, C)`` is in the activation dtype and so is the result; ``dt_raw`` and ``z`` ``(T, C)``
    and ``b``, ``c`` ``(T, N)`` (column ranges of one matrix) are float32 with contiguous rows;
    ``a_log (C, N)``; ``state (slots, C * N)`` holds S as [channel][n], float32, and is left as
    after each sequence's last token."""
    T, C = x.shape
    N = a_log.shape[1]
    ldx = _rows(x, "selective_scan x")
    lddt = _rows(dt_raw, "selective_scan dt", torch.float32)
    ldz = _rows(z, "selective_scan z", torch.float32)
    ldbc = _rows(b, "selective_scan B", torch.float32)
    if _rows(c, "selective_scan C", torch.float32) != ldbc:
        raise KernelError("selective_scan: B and C must share a row stride")
    if dt_raw.shape != (T, C) or z.shape != (T, C) or b.shape != (T, N) or c.shape != (T, N) \
            or a_log.shape != (C, N):
        raise KernelError("selective_scan: operand shapes do not match the channels and states")
    stride = _state(state, C * N, "selective_scan")
    out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    chunk_len = max_chunks = 0
    chunk_state = chunk_dt = None
    if T >= CHUNKED_SCAN_MIN_TOKENS and T >= CHUNKED_SCAN_MIN_MEAN_TOKENS * max(1, num_seqs):
        chunk_len = int(CHUNKED_SCAN_LEN)
        max_chunks = -(-T // chunk_len) + num_seqs          # an upper bound, known on the host
        chunk_state = torch.empty((max_chunks, C * N), dtype=torch.float32, device=x.device)
        chunk_dt = torch.empty((max_chunks, C), dtype=torch.float32, device=x.device)
    lib.call("rlis_selective_scan", out.data_ptr(), _dt(out), C, x.data_ptr(), ldx,
             dt_raw.data_ptr(), lddt, _vec(dt_bias, C, "selective_scan dt bias"), b.data_ptr(),
             c.data_ptr(), ldbc, z.data_ptr(), ldz, _vec(a_log.reshape(-1), C * N,
                                                         "selective_scan A_log"),
             _vec(skip, C, "selective_scan skip"), state.data_ptr(), stride,
             _meta(cu, num_seqs + 1, "cu"), _meta(slots, num_seqs, "slots"), num_seqs, C, N,
             int(chunk_len == 0 and T >= SPREAD_SCAN_MIN_MEAN_TOKENS * max(1, num_seqs)
                 and num_seqs * C <= SPREAD_SCAN_MAX_CHANNELS), chunk_len, max_chunks,
             None if chunk_state is None else chunk_state.data_ptr(),
             None if chunk_dt is None else chunk_dt.data_ptr(), lib.stream_ptr())
    return out
