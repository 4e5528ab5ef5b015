"""Each kernel that the Pamolix design added or extended, alone, against the plain formulas of
``plain_pamolix.py`` (float64), at sizes the models of the other tests do not have: a sink in
the softmax and kept first keys beside a window through the vector-unit kernels, the
matrix-core kernels and the generic kernel (portions beside single tokens, decode partitions,
key runs, tiles of 128 queries); the residual streams' step with one to seven streams, with and
without an update, a read-out, a norm and picked rows; biases, head norms and the queries'
factor on the rows of a fused projection; the gate per head; the erf form of GELU; the biased
router and the units without gates."""
import math

import pytest
import torch

import plain_pamolix as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel(got, want):
    return float((got.double().cpu() - want.double().cpu()).norm() / want.double().cpu().norm())


def _reference(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, sinks, window, keep, cap):
    outs = []
    q_all = qkv.double().cpu()[:, :nh * d]
    for s, (c, n) in enumerate(zip(cached, new)):
        q = q_all[cu[s]:cu[s + 1]].reshape(n, nh, d)
        k, v = ks[s].double(), vs[s].double()
        ok = plain.visible(c + n, window, keep)[c:]
        kk = k.repeat_interleave(nh // nkv, dim=1)
        vv = v.repeat_interleave(nh // nkv, dim=1)
        sc = torch.einsum("ihd,jhd->hij", q, kk) * scale
        if cap:
            sc = cap * torch.tanh(sc / cap)
        w = plain.softmax_rows(sc, ok, None if sinks is None else sinks.double())
        outs.append(torch.einsum("hij,jhd->ihd", w, vv).reshape(n, nh * d))
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,ps", [(6, 2, 32, 8), (5, 5, 48, 16), (32, 8, 64, 16),
                                         (8, 2, 128, 16), (4, 1, 80, 16)])
def test_attention_with_a_sink_and_kept_first_keys(dtype, nh, nkv, d, ps, monkeypatch):
    """A sink per head (from far below the scores to far above them), and windows of 50 and 300
    that keep no first keys, 1, 7, a page and a half of them, 100 and more than the context:
    through the kernels that the batch takes by itself (bfloat16: the matrix-core kernels;
    float32: the vector-unit kernels), through the vector-unit kernels for bfloat16 too, and
    through the generic kernel.  An engine that drops the sink, counts it per key run or
    partition, or is one off in the kept keys is far off."""
    from test_kernels_gpu import attention_constants, key_runs, paged_case
    import rust_llm_inference_server_amd.ops as ops
    scale = 1.0 / math.sqrt(d)
    sinks = torch.tensor([-20.0, 0.0, 1.5, 4.0, 9.0][:nh] + [0.3 * (h % 7) for h in range(max(0, nh - 5))],
                         dtype=torch.float32)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for cached, new in (([0, 5, 40, 130, 17], [33, 1, 70, 2, 64]), ([4, 99, 0, 640], [1, 1, 1, 1]),
                        ([1, 1100], [1, 1]), ([1200, 2], [1, 130]), ([20], [300]), ([700], [90])):
        for window, keep, with_sink, cap in ((None, 0, True, 0.0), (50, 0, False, 0.0),
                                             (50, 1, False, 0.0), (50, 7, True, 3.0),
                                             (50, 24, False, 0.0), (300, 100, False, 2.0),
                                             (50, 5000, True, 0.0), (64, 32, False, 0.0)):
            qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype,
                                                           seed=nh + 3, q_scale=2.0)
            sk = sinks if with_sink else None
            want = _reference(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, sk, window, keep, cap)
            kw = dict(sinks=None if sk is None else sk.to(DEV), keep_first=keep, softcap=cap)
            for vector in (False, True):
                monkeypatch.setattr(ops, "PLAIN_EXTRAS", vector)
                with attention_constants(DECODE_PART_KEYS=256, PREFILL_WIDE_MIN_GROUPS=0,
                                         **key_runs(3)):
                    for force in (None, "generic"):
                        got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale,
                                                  window, force=force, **kw)
                        assert rel(got, want) < tol, (cached, new, window, keep, vector, force)
            monkeypatch.setattr(ops, "PLAIN_EXTRAS", False)
            if with_sink and dtype == torch.float32:
                bare = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                           keep_first=keep, softcap=cap)
                assert rel(bare, want) > 1e-3
            if keep and window and dtype == torch.float32 \
                    and max(c + n for c, n in zip(cached, new)) > window + keep + 40:
                for other in (keep - 1, keep + 1):
                    off = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                              keep_first=other, sinks=kw["sinks"], softcap=cap)
                    assert rel(off, want) > 1e-4


@pytest.mark.parametrize("S", [1, 2, 3, 7])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, H", [(1, 40), (9, 256), (70, 100), (5, 4100), (3, 30), (11, 125)])
def test_the_residual_streams_step(S, y_dtype, T, H):
    """Update, read-out and norm in one pass and each alone; streams that still share one
    tensor; a result that comes as partial sums; picked rows, which leave the streams alone."""
    from rust_llm_inference_server_amd import ops
    g = torch.Generator().manual_seed(S * 100 + T)
    rand = lambda *shape: torch.randn(*shape, generator=g)
    lanes, mix, back, read, w = rand(S, T, H), rand(S, S), rand(S), rand(S), 1.0 + 0.3 * rand(H)
    y = rand(T, H).to(y_dtype)
    eps = 1e-5

    def updated(l):
        l, yy = l.double(), y.double()
        return torch.stack([sum(mix[s, t].double() * l[s] for s in range(S)) + back[t].double() * yy
                            for t in range(S)])

    def read_out(l, coef, norm):
        u = sum((1.0 if coef is None else coef[s].double()) * l[s].double() for s in range(S))
        return plain.rms(u, eps) * w.double() if norm else u

    dev = lambda t: t.to(DEV)
    # update + read + norm
    new, out = ops.lanes_step(dev(lanes), S, update=(dev(y), dev(mix), dev(back)), read=dev(read),
                              norm_weight=dev(w), eps=eps, out_dtype=torch.float32)
    assert rel(new, updated(lanes)) < 2e-6 and rel(out, read_out(updated(lanes), read, True)) < 2e-6
    # the update alone, then the plain sum, unnormalised
    new, out = ops.lanes_step(dev(lanes), S, update=(dev(y), dev(mix), dev(back)), want=False)
    assert out is None and rel(new, updated(lanes)) < 2e-6
    _, total = ops.lanes_step(new, S)
    assert rel(total, read_out(updated(lanes), None, False)) < 2e-6
    # streams that still share one tensor
    one = lanes[0].contiguous()
    shared = torch.stack([one] * S)
    new, out = ops.lanes_step(dev(one), S, read=dev(read), norm_weight=dev(w), eps=eps,
                              out_dtype=torch.bfloat16)
    assert new.dim() == 2 and rel(out, read_out(shared, read, True)) < 6e-3
    new, out = ops.lanes_step(dev(one), S, update=(dev(y), dev(mix), dev(back)), read=dev(read),
                              norm_weight=dev(w), eps=eps, out_dtype=torch.float32)
    assert tuple(new.shape) == (S, T, H) and rel(new, updated(shared)) < 2e-6
    assert rel(out, read_out(updated(shared), read, True)) < 2e-6
    # picked rows: the pending update is applied for the read-out only
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    before = dev(lanes)
    keep = before.clone()
    new, out = ops.lanes_step(before, S, update=(dev(y), dev(mix), dev(back)), norm_weight=dev(w),
                              eps=eps, out_dtype=torch.float32, rows=dev(rows))
    assert torch.equal(before, keep) and new is before
    assert rel(out, read_out(updated(lanes), None, True)[rows.long()]) < 2e-6
    # partial sums, rounded once to bfloat16 before they join
    if y_dtype == torch.float32:
        parts = rand(3, T, H)
        whole = parts[0] + parts[1] + parts[2]
        y = whole.to(torch.bfloat16).to(torch.float32)
        new, _ = ops.lanes_step(dev(lanes), S, update=(dev(parts), dev(mix), dev(back)),
                                round_parts=True, want=False)
        assert rel(new, updated(lanes)) < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh, nkv, D, dim", [(4, 2, 16, 16), (6, 3, 64, 48), (3, 1, 80, 72),
                                             (2, 2, 160, 130), (5, 0, 32, 20)])
def test_bias_head_norm_and_the_queries_factor(dtype, nh, nkv, D, dim):
    """On rows that carry more columns than the heads (gates behind them): every combination of
    bias, norm and factor; padding dims stay zero; values get the bias alone."""
    from rust_llm_inference_server_amd import ops
    g = torch.Generator().manual_seed(nh * 10 + D)
    T, extra = 37, 8
    cols = (nh + 2 * nkv) * D
    x = torch.randn(T, cols + extra, generator=g)
    x[:, :cols] = (x[:, :cols].reshape(T, -1, D) * (torch.arange(D) < dim)).reshape(T, cols)
    x = x.to(dtype)
    bias = torch.randn(nh + 2 * nkv, D, generator=g) * (torch.arange(D) < dim)
    qw, kw = 1.0 + 0.3 * torch.randn(dim, generator=g), 1.0 + 0.3 * torch.randn(dim, generator=g)
    pos = torch.randint(0, 400, (T,), generator=g, dtype=torch.int32)
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    for use_bias, use_norm, temp in ((True, True, (0.5, 16)), (False, True, None),
                                     (True, False, None), (False, False, (1.3, 1)),
                                     (True, True, (0.2, 1000))):
        got = x.to(DEV).clone()
        ops.head_prepare_(got, nh, nkv, D, dim, bias.reshape(-1).to(DEV) if use_bias else None,
                          qw.to(DEV) if use_norm else None,
                          kw.to(DEV) if use_norm and nkv else None, 1e-5,
                          pos.to(DEV), *(temp or (0.0, 0)))
        h = x[:, :cols].double().reshape(T, -1, D)
        if use_bias:
            h = h + bias.double()
        q, k, v = h[:, :nh, :dim], h[:, nh:nh + nkv, :dim], h[:, nh + nkv:, :dim]
        if use_norm:
            q, k = plain.rms(q, 1e-5) * qw.double(), plain.rms(k, 1e-5) * kw.double()
        if temp:
            steps = torch.div(pos.long() + 1, temp[1], rounding_mode="floor").double()
            q = q * (1.0 + temp[0] * torch.log(steps + 1.0)).reshape(T, 1, 1)
        want = torch.zeros(T, nh + 2 * nkv, D, dtype=torch.float64)
        want[:, :, :dim] = torch.cat([q, k, v], dim=1)
        assert rel(got[:, :cols], want.reshape(T, cols)) < tol
        assert torch.equal(got[:, cols:].cpu(), x[:, cols:])           # what rides behind
        pad = got[:, :cols].reshape(T, -1, D)[:, :, dim:]
        assert float(pad.abs().max()) == 0.0 if pad.numel() else True


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_per_head_and_the_erf_form_of_gelu(dtype):
    from rust_llm_inference_server_amd import ops
    g = torch.Generator().manual_seed(4)
    T, nh, D = 29, 5, 24
    x = torch.randn(T, nh * D, generator=g).to(dtype)
    rows = (3.0 * torch.randn(T, 40 + 8, generator=g)).to(dtype)     # gates behind 40 columns
    got = ops.head_gate_(x.to(DEV).clone(), rows.to(DEV)[:, 40:], nh, D)
    want = x.double().reshape(T, nh, D) * torch.sigmoid(rows[:, 40:40 + nh].double()).unsqueeze(-1)
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    assert rel(got, want.reshape(T, -1)) < tol
    z = (2.5 * torch.randn(1000, generator=g)).to(dtype)
    assert rel(ops.gelu_erf(z.to(DEV)), plain.gelu_erf(z.double())) < tol
    # (far from the tanh form)
    assert rel(ops.gelu_tanh(z.to(DEV)), plain.gelu_erf(z.double())) > 1e-5 or dtype != torch.float32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, E, top, W, F", [(1, 4, 2, 48, 24), (7, 6, 1, 40, 20), (70, 16, 4, 256, 96),
                                             (300, 3, 3, 64, 10), (2500, 8, 2, 128, 64)])
def test_the_biased_router_and_units_without_gates(dtype, T, E, top, W, F):
    """The choice by logits plus bias, weights by the softmax over the chosen logits alone, and
    ``down(relu(up x)^2)`` through every tile form, against the plain mixture."""
    from rust_llm_inference_server_amd import ops
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, W, generator=g).to(dtype)
    w = {"router": torch.randn(E, W, generator=g) * W ** -0.5 * 3.0,
         "router.b": torch.randn(E, generator=g)}
    for e in range(E):
        w[f"e{e}.up"] = (torch.randn(F, W, generator=g) * W ** -0.5).to(dtype)
        w[f"e{e}.down"] = (torch.randn(W, F, generator=g) * F ** -0.5).to(dtype)
    logits = (x.double() @ w["router"].double().T).float()
    chosen, weights = ops.route(logits.to(DEV), None, 1, 1, top, 1.0, scores="softmax",
                                group_score="max", renormalise=True, bias=w["router.b"].to(DEV))
    z = logits.double() + w["router.b"].double()
    best, idx = torch.topk(z, top, dim=-1)
    assert torch.equal(chosen.cpu().long(), idx)
    assert rel(weights, torch.softmax(best, dim=-1)) < 1e-5
    up = torch.stack([w[f"e{e}.up"] for e in range(E)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(DEV)
    got = ops.routed_units(x.to(DEV), up, down, chosen, weights, plain=True)
    want = torch.zeros(T, W, dtype=torch.float64)
    for t in range(T):
        for r in range(top):
            e = int(idx[t, r])
            hidden = plain.relu_squared(w[f"e{e}.up"].double() @ x[t].double())
            if dtype == torch.bfloat16:
                hidden = hidden.to(torch.bfloat16).double()
            want[t] += float(weights[t, r]) * (w[f"e{e}.down"].double() @ hidden)
    assert rel(got, want) < (2e-5 if dtype == torch.float32 else 1e-2)
