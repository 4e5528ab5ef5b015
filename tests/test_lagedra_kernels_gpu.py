"""Each kernel that the Lagedra design added or extended, alone, against the plain formulas of
``plain_lagedra.py`` (float64), at sizes the models of the other tests do not have: heads of more
than 64 and more than 128 key channels, value sizes that are no multiple of a wave's columns,
several sequences per step in state slots that are not in order, the state carried over steps,
long portions through the chunked form and the same portions token by token, scores far on
the flat part of the cap, through the vector-unit and the matrix-core attention kernels."""
import math

import pytest
import torch

import plain_lagedra as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ops():
    from rust_llm_inference_server_amd import ops
    return ops


def _meta(lengths, slots):
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32, device=DEV)
    seq = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths)).to(
        torch.int32).to(DEV)
    return cu, torch.tensor(slots, dtype=torch.int32, device=DEV), seq


def _state(num_slots, used, extra=24):
    """A state buffer whose rows are longer than the mixer's area, filled with garbage that the
    test clears for the slots it uses (as the runner does for a request at position 0)."""
    buf = torch.full((num_slots, used + extra), 7.5, dtype=torch.float32, device=DEV)
    return buf, buf[:, 8:8 + used]


def rel(got, want):
    return float((got.double() - want.double()).norm() / want.double().norm())


def _linear_attention(q, k, v, decay, S):
    """Token by token in float64: ``S <- decay S + k v^T``, ``o = S^T q``; q, k ``(T, H, d)``,
    v ``(T, H, dv)``, S ``(H, d, dv)`` (changed in place)."""
    out = torch.zeros(v.shape, dtype=torch.float64)
    qa, ka, va = plain.silu(q.double()), plain.silu(k.double()), plain.silu(v.double())
    for t in range(q.shape[0]):
        S *= decay.double().reshape(-1, 1, 1)
        S += ka[t].unsqueeze(-1) * va[t].unsqueeze(-2)
        out[t] = torch.einsum("hdv,hd->hv", S, qa[t])
    return out


STEPS = [[5, 1, 9], [1, 1, 2], [3, 1, 1], [70, 2, 33], [1, 1, 1]]
LONG_STEPS = [[130, 200, 64], [1, 3, 1], [257, 65, 191], [2, 1, 1]]
SLOTS = [3, 0, 2]


@pytest.mark.parametrize("form", ["scan", "chunks", "either"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, d, dv", [(3, 16, 16), (2, 96, 40), (1, 160, 33), (2, 50, 130),
                                          (4, 64, 64), (2, 128, 128), (3, 6, 10)])
def test_linear_attention_with_a_decay_per_head(heads, d, dv, dtype, form, monkeypatch):
    """Three sequences over several steps in slots that are not in order, from raw projections
    in either dtype with row strides, the state carried from step to step and left in the slot
    as [head][value channel][key channel]; a head that forgets nothing among them.  ``form``:
    token by token, the chunked form for every step it takes (float32 inputs, heads of up to
    128 channels), or what the steps' shapes choose."""
    ops = _ops()
    from rust_llm_inference_server_amd.ops import recurrent
    steps = STEPS if form == "scan" else LONG_STEPS
    if form == "scan":
        monkeypatch.setattr(recurrent, "DECAY_CHUNKED_MIN_TOKENS", 1 << 30)
        monkeypatch.setattr(recurrent, "DECAY_CHUNKED_MIN_LONGEST", 1 << 30)
    elif form == "chunks":
        if dtype != torch.float32 or max(d, dv) > 128:
            pytest.skip("the chunked form takes float32 rows and heads of up to 128 channels")
        monkeypatch.setattr(recurrent, "DECAY_CHUNKED_MIN_TOKENS", 1)
        monkeypatch.setattr(recurrent, "DECAY_CHUNKED_MIN_MEAN_TOKENS", 0)
    g = torch.Generator().manual_seed(heads * 1000 + d + dv)
    totals = [sum(s[i] for s in steps) for i in range(3)]
    data = [{"q": torch.randn(T, heads * d, generator=g).to(dtype),
             "k": torch.randn(T, heads * d, generator=g).to(dtype),
             "v": torch.randn(T, heads * dv, generator=g).to(dtype)} for T in totals]
    decay = torch.tensor(([1.0, 0.5, 0.97, 0.999] * heads)[:heads], dtype=torch.float32)
    buf, state = _state(4, heads * dv * d)
    state[SLOTS] = 0.0
    want, S = [], []
    for x in data:
        Sx = torch.zeros(heads, d, dv, dtype=torch.float64)
        want.append(_linear_attention(x["q"].reshape(-1, heads, d), x["k"].reshape(-1, heads, d),
                                      x["v"].reshape(-1, heads, dv), decay, Sx))
        S.append(Sx)
    at_seq = [0, 0, 0]
    tol = 2e-5             # in either dtype: the inputs are rounded, not the sums
    for lengths in steps:
        cu, slots, _ = _meta(lengths, SLOTS)
        rows = {n: torch.cat([data[i][n][at_seq[i]:at_seq[i] + lengths[i]] for i in range(3)])
                for n in "qkv"}
        # the three projections as column ranges of one wider row, as the mixer hands them over
        wide = torch.cat([rows["q"], rows["k"], rows["v"]], dim=1).to(DEV)
        q, k, v = wide[:, :heads * d], wide[:, heads * d:2 * heads * d], wide[:, 2 * heads * d:]
        out = ops.decay_attention(q, k, v, decay.to(DEV), state, cu, slots, 3, heads, d, dv).cpu()
        at = 0
        for i, n in enumerate(lengths):
            ref = want[i][at_seq[i]:at_seq[i] + n].reshape(n, heads * dv)
            assert rel(out[at:at + n], ref) < tol, (lengths, i)
            at += n
            at_seq[i] += n
    for i, slot in enumerate(SLOTS):
        got = state[slot].cpu().reshape(heads, dv, d).transpose(1, 2)
        assert rel(got, S[i]) < tol
    assert float(buf[1].min()) == 7.5 and float(buf[:, :8].min()) == 7.5    # nothing else touched


def test_the_chunked_form_is_chosen_by_the_steps_shape():
    from rust_llm_inference_server_amd.ops.recurrent import decay_attention_chunked as chosen
    f32, bf16 = torch.float32, torch.bfloat16
    assert chosen(2048, 1, 64, 64, f32) and chosen(256, 4, 128, 96, f32)
    assert not chosen(255, 1, 64, 64, f32)          # short steps walk token by token
    assert not chosen(2048, 40, 64, 64, f32)        # and so do steps of many short portions
    assert not chosen(2048, 1, 160, 64, f32) and not chosen(2048, 1, 64, 64, bf16)
    # a long portion beside many decoded tokens
    assert chosen(2048 + 200, 201, 64, 64, f32, longest=2048)
    assert chosen(90, 21, 64, 64, f32, longest=70) and not chosen(400, 201, 64, 64, f32, longest=50)


@pytest.mark.parametrize("T, C", [(5, 48), (3, 1000), (1, 7)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_over_all_heads_with_a_sigmoid_gate(T, C, dtype):
    """``o / rms(o) * weight * sigmoid(gate)`` over the concatenated heads (one group of all
    the channels), the gate read from a wider row."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * C)
    o = torch.randn(T, C, generator=g) * 3.0
    w = 1.0 + 0.3 * torch.randn(C, generator=g)
    wide = torch.randn(T, C + 16, generator=g)
    got = ops.head_norm_gate(o.to(DEV), w.to(DEV), wide.to(DEV)[:, 16:], 1, C, 1e-5, dtype,
                             sigmoid_gate=True)
    want = plain.rms_unit(o.double(), 1e-5) * w.double() * torch.sigmoid(wide[:, 16:].double())
    assert got.dtype == dtype and rel(got.cpu(), want) < (1e-5 if dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolution_without_activation_and_values_mixed_in(taps, dtype):
    """The plain convolution (no SiLU) over steps with tails in slots, and behind it
    ``(1 - w) y + w other`` on the last channels only."""
    ops = _ops()
    C, blend_from, weight = 72, 40, 0.3
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(C, taps, generator=g) * 0.6
    totals = [sum(s[i] for s in STEPS) for i in range(3)]
    xs = [torch.randn(T, C, generator=g) for T in totals]
    others = [torch.randn(T, C - blend_from, generator=g).to(dtype) for T in totals]
    want = []
    for x, other in zip(xs, others):
        y = plain.short_conv(x.double(), w.double())
        y[:, blend_from:] = (1.0 - weight) * y[:, blend_from:] + weight * other.double()
        want.append(y)
    buf, state = _state(4, max(1, C * (taps - 1)))
    state[SLOTS] = 0.0
    at_seq = [0, 0, 0]
    for lengths in STEPS:
        cu, slots, seq = _meta(lengths, SLOTS)
        x = torch.cat([xs[i][at_seq[i]:at_seq[i] + lengths[i]] for i in range(3)]).to(DEV)
        other = torch.cat([others[i][at_seq[i]:at_seq[i] + lengths[i]] for i in range(3)]).to(DEV)
        out = ops.causal_conv(x, w.to(DEV), state, seq, cu, slots, 3, out_dtype=dtype,
                              activation=False, blend=other, blend_from=blend_from,
                              blend_weight=weight).cpu()
        if taps > 1:
            ops.tail_update(state, x, C, taps - 1, cu, slots, 3)
        at = 0
        for i, n in enumerate(lengths):
            ref = want[i][at_seq[i]:at_seq[i] + n]
            assert rel(out[at:at + n], ref) < (1e-5 if dtype == torch.float32 else 5e-3)
            at += n
            at_seq[i] += n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_learned_positions_gelu_and_depth_mix(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    V, W, P, T = 50, 72, 40, 9
    table, pos = torch.randn(V, W, generator=g).to(dtype), torch.randn(P, W, generator=g).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    places = torch.randint(0, P, (T,), generator=g).to(torch.int32)
    got = ops.embed(ids.to(DEV), table.to(DEV), 1.0, pos.to(DEV), places.to(DEV))
    want = table.double()[ids.long()] + pos.double()[places.long()]
    assert got.dtype == torch.float32 and rel(got.cpu(), want) < 1e-6
    x = (torch.randn(T, 130, generator=g) * 3.0).to(dtype)
    assert rel(ops.gelu_tanh(x.to(DEV)).cpu(), plain.gelu_tanh(x.double())) < \
        (1e-6 if dtype == torch.float32 else 4e-3)
    # three layers' worth of the mix: the stream becomes the weighted sum of all results so far
    layers = 3
    history = torch.full((layers + 1, T, W), 9.0, dtype=torch.float32, device=DEV)
    x = torch.randn(T, W, generator=g)
    kept, stream = [x.double()], x.to(DEV)
    for i in range(layers):
        delta = torch.randn(T, W, generator=g)
        weights = torch.randn(i + 2, generator=g).to(dtype)
        kept.append(stream.cpu().double() + delta.double())
        ops.depth_mix_(stream, delta.to(DEV), history, i + 2, weights.to(DEV), save_input=i == 0)
        want = sum(weights.double()[j] * kept[j] for j in range(i + 2))
        assert rel(stream.cpu(), want) < 1e-6
        kept[0] = history[0].cpu().double()
        assert rel(history[i + 1].cpu(), kept[i + 1]) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, W", [(1, 40), (9, 256), (70, 100)])
def test_norm_whose_weight_is_one_number(T, W, dtype):
    """The norm part with a weight without axes, on a stream with a delta still to be added:
    the sum is normalised, in float32, and the stream keeps it."""
    from rust_llm_inference_server_amd.parts.base import (BuildContext, PartSpec, ResidualStream,
                                                          create)
    g = torch.Generator().manual_seed(T + W)
    weight = torch.tensor(1.7).to(dtype)
    ctx = BuildContext(device=torch.device(DEV), act_dtype=dtype, weights={"n": weight.to(DEV)},
                       max_positions=16)
    norm = create("norm", PartSpec("rmsnorm", {"size": W, "eps": 1e-5, "scalar": True,
                                               "weight_name": ""}), "n", ctx)
    x, delta = torch.randn(T, W, generator=g) * 2.0, torch.randn(T, W, generator=g)
    stream = ResidualStream(x.to(DEV), dtype)
    stream.add(delta.to(DEV))
    h = norm.forward(stream)
    h = h if isinstance(h, torch.Tensor) else h.tensor()
    want = plain.scalar_norm(x.double() + delta.double(), weight.double(), 1e-5)
    assert rel(h.cpu(), want) < (1e-6 if dtype == torch.float32 else 4e-3)
    assert rel(stream.flush().cpu(), x.double() + delta.double()) < 1e-6


def test_rotation_tables_with_stretched_frequencies():
    """The tables of the rotation part against the plain formulas: ramps that begin at pair 0,
    that end before the last pair, that are one pair wide; the magnitude on both tables."""
    from rust_llm_inference_server_amd.parts.base import BuildContext, PartSpec, create
    ctx = BuildContext(device=torch.device(DEV), act_dtype=torch.float32, weights={},
                       max_positions=700)
    for dims, base, (factor, original, fast, slow) in [
            (80, 40000.0, (3.0, 2048, 16.0, 2.0)), (16, 300.0, (2.0, 32, 4.0, 0.5)),
            (64, 10000.0, (8.0, 4096, 1.0, 1.0)), (8, 1000.0, (16.0, 16, 2.0, 1.0)),
            (32, 1e6, (1.0, 64, 32.0, 1.0))]:
        rot = {"dims": dims, "base": base, "scaling": {"factor": factor, "original": original,
                                                       "fast": fast, "slow": slow}}
        part = create("position", PartSpec("rope", {
            "rot_dim": dims, "theta": base, "precise": False,
            "scaling": {"rope_type": "yarn", **rot["scaling"]}}), "", ctx)
        cos, sin = plain.rotary_tables(rot, torch.arange(700))
        assert float((part.cos.cpu().double() - cos).abs().max()) < 2e-6
        assert float((part.sin.cpu().double() - sin).abs().max()) < 2e-6


def _shaped_reference(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, head_scales, cap, window):
    outs = []
    q_all = qkv.double().cpu()[:, :nh * d]
    for s, (c, n) in enumerate(zip(cached, new)):
        q = q_all[cu[s]:cu[s + 1]].reshape(n, nh, d)
        k, v = ks[s].double(), vs[s].double()
        i = torch.arange(c, c + n).reshape(-1, 1)
        j = torch.arange(c + n).reshape(1, -1)
        seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
        o = torch.zeros(n, nh, d, dtype=torch.float64)
        for h in range(nh):
            kv = h // (nh // nkv)
            sc = (q[:, h] @ k[:, kv].T) * scale * float(head_scales[h])
            sc = cap * torch.tanh(sc / cap)
            sc = sc.masked_fill(~seen, -math.inf)
            o[:, h] = torch.softmax(sc, dim=-1) @ v[:, kv]
        outs.append(o.reshape(n, nh * d))
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,ps", [(6, 2, 32, 8), (5, 5, 48, 16), (32, 8, 64, 16),
                                         (8, 2, 128, 16), (4, 2, 96, 16)])
def test_attention_with_a_number_per_head_and_a_cap(dtype, nh, nkv, d, ps, monkeypatch):
    """Scores times a number per head, then ``cap * tanh(score / cap)``, with and without a
    window: portions beside single tokens, single tokens alone over several decode partitions,
    a long portion over key runs and in tiles of 128 queries, through the kernels that the
    batch takes by itself (bfloat16: the matrix-core kernels' shaped forms; float32: the
    vector-unit kernels), through the vector-unit kernels for bfloat16 too, and through the
    generic kernel.  The queries are large, so that most scores lie on the flat part of the
    cap and both an engine without it and one that caps in front of the head's number are far
    off."""
    from test_kernels_gpu import attention_constants, key_runs, paged_case
    import rust_llm_inference_server_amd.ops as ops
    scale, cap = 1.0 / math.sqrt(d), 4.0
    head_scales = torch.tensor([0.5 + 0.37 * (h % 5) for h in range(nh)], dtype=torch.float32)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for cached, new in (([0, 5, 40, 130, 17], [33, 1, 70, 2, 64]), ([4, 99, 0, 640], [1, 1, 1, 1]),
                        ([1, 1100], [1, 1]), ([1200, 2], [1, 130]), ([20], [300])):
        for window in (None, 50):
            qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype,
                                                           seed=nh + 9, q_scale=3.0)
            want = _shaped_reference(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, head_scales,
                                     cap, window)
            for matrix in (True, False):
                monkeypatch.setattr(ops, "SHAPED_SCORES_MATRIX", matrix)
                with attention_constants(DECODE_PART_KEYS=256, PREFILL_WIDE_MIN_GROUPS=0,
                                         **key_runs(3)):
                    for force in (None, "generic"):
                        got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale,
                                                  window, head_scales=head_scales.to(DEV),
                                                  softcap=cap, force=force)
                        assert rel(got.cpu(), want) < tol, (cached, new, window, matrix, force)
            uncapped = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                           head_scales=head_scales.to(DEV))
            unscaled = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                           softcap=cap)
            assert rel(uncapped.cpu(), want) > 0.05 and rel(unscaled.cpu(), want) > 0.02
            # either shaping alone
            ones = torch.ones(nh)
            assert rel(uncapped.cpu(), _shaped_reference(qkv, ks, vs, cu, cached, new, nh, nkv, d,
                                                         scale, head_scales, 1e9, window)) < tol
            assert rel(unscaled.cpu(), _shaped_reference(qkv, ks, vs, cu, cached, new, nh, nkv, d,
                                                         scale, ones, cap, window)) < tol


@pytest.mark.parametrize("E, G, keep, top", [(16, 4, 3, 4), (6, 3, 2, 2), (8, 1, 1, 3), (5, 5, 2, 1),
                                             (64, 8, 4, 8)])
def test_the_softmax_router_with_groups(E, G, keep, top):
    """Softmax over all experts, a group's score its largest, the best groups kept, the largest
    scores among them chosen and divided by their sum."""
    ops = _ops()
    g = torch.Generator().manual_seed(E * 10 + top)
    z = torch.randn(40, E, generator=g) * 2.0
    chosen, weights = ops.route(z.to(DEV), None, G, keep, top, 1.0, scores="softmax",
                                group_score="max", renormalise=True)
    router = {"experts": E, "top": top, "groups": {"count": G, "keep": keep}}
    want_chosen, want_weights = plain.route(z.double(), router)
    for t in range(z.shape[0]):
        got = dict(zip(chosen[t].tolist(), weights[t].tolist()))
        assert sorted(got) == sorted(want_chosen[t])
        for n, e in enumerate(want_chosen[t]):
            assert abs(got[e] - float(want_weights[t, n])) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, E, top, W, F", [(1, 4, 2, 48, 24), (7, 6, 1, 40, 20), (70, 16, 4, 256, 96),
                                             (300, 8, 3, 128, 72)])
def test_bounded_units_behind_a_router(dtype, T, E, top, W, F):
    """``min(gate, limit) * sigmoid(1.702 min(gate, limit)) * (clamp(up) + 1)`` through the
    routed kernels of every tile size, with inputs large enough that the bounds bind."""
    ops = _ops()
    g = torch.Generator().manual_seed(T + E)
    limit, alpha = 0.8, 1.702
    x = torch.randn(T, W, generator=g).to(dtype)
    w = {}
    for e in range(E):
        w[f"m.e{e}.gate"] = (torch.randn(F, W, generator=g) * W ** -0.5 * 1.5).to(dtype)
        w[f"m.e{e}.up"] = (torch.randn(F, W, generator=g) * W ** -0.5 * 1.5).to(dtype)
        w[f"m.e{e}.down"] = (torch.randn(W, F, generator=g) * F ** -0.5).to(dtype)
    chosen = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    weights = torch.rand(T, top, generator=g)
    gate_up = torch.stack([torch.cat([w[f"m.e{e}.gate"], w[f"m.e{e}.up"]]) for e in range(E)])
    down = torch.stack([w[f"m.e{e}.down"] for e in range(E)])
    got = ops.routed_units(x.to(DEV), gate_up.to(DEV).contiguous(), down.to(DEV).contiguous(),
                           chosen.to(DEV), weights.to(DEV), None, limit=limit, alpha=alpha)
    want = torch.zeros(T, W, dtype=torch.float64)
    for t in range(T):
        for n in range(top):
            e = int(chosen[t, n])
            want[t] += weights[t, n].double() * plain.expert(w, f"m.e{e}", x[t:t + 1].double(),
                                                             limit)[0]
    bound = (plain.expert(w, "m.e0", x.double(), limit) -
             plain.expert(w, "m.e0", x.double(), 100.0)).abs().max()
    assert float(bound) > 0.05                                    # the bounds do bind
    assert rel(got.float().cpu(), want) < (2e-5 if dtype == torch.float32 else 2e-2)
