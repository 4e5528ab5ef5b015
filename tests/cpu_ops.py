"""A test double for the kernel layer: the same functions as ``rust_llm_inference_server_amd.ops``
in slow torch code on the CPU, so that the host logic around the kernels (batch layout, page
tables, cache manager, scheduler, engine loop) can be tested on a machine without a GPU.

It is installed by the ``cpu_ops`` fixture only; the package itself never falls back to it.
It follows the kernels' contracts (page layouts, in-place rotation, transposed values), not
their code.
"""
from __future__ import annotations


import torch


def embed(ids, table, scale=1.0, learned=None, positions=None):
    out = table[ids.long()].to(torch.float32) * scale
    return out if learned is None else out + learned[positions.long()].to(torch.float32)


def gelu_tanh(x):
    z = x.float()
    return (0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))).to(x.dtype)


def gelu_erf(x):
    z = x.float()
    return (0.5 * z * (1.0 + torch.erf(z * 0.7071067811865476))).to(x.dtype)


def lanes_step(lanes, count, update=None, read=None, norm_weight=None, eps=0.0, out_dtype=None,
               rows=None, round_parts=False, want=True):
    S = count
    cur = lanes.unsqueeze(0).expand(S, *lanes.shape) if lanes.dim() == 2 else lanes
    if update is not None:
        y, mix, back = update
        y = (y.sum(0) if y.dim() == 3 else y).float()
        cur = torch.stack([sum(mix[s, t] * cur[s] for s in range(S)) + back[t] * y
                           for t in range(S)])
    out = None
    if want:
        pick = cur if rows is None else cur[:, rows.long()]
        u = sum((1.0 if read is None else read[s]) * pick[s] for s in range(S))
        if norm_weight is not None:
            u = u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * norm_weight.float()
        out = u.to(out_dtype or torch.float32)
    keep = update is not None and rows is None
    return (cur.contiguous() if keep else lanes), out


def head_prepare_(qkv, num_heads, num_kv_heads, head_dim, real_dim, bias=None, q_weight=None,
                  k_weight=None, eps=0.0, positions=None, temp_coef=0.0, temp_every=0):
    T, nh, nkv, D = qkv.shape[0], num_heads, num_kv_heads, head_dim
    cols = (nh + 2 * nkv) * D
    x = qkv[:, :cols].float()
    if bias is not None:
        x = x + bias
    x = x.reshape(T, nh + 2 * nkv, D).clone()
    for lo, hi, w in ((0, nh, q_weight), (nh, nh + nkv, k_weight)):
        if w is not None and hi > lo:
            part = x[:, lo:hi, :real_dim]
            x[:, lo:hi, :real_dim] = part / torch.sqrt((part * part).mean(-1, keepdim=True) + eps) * w
            x[:, lo:hi, real_dim:] = 0.0
    if temp_every > 0:
        steps = torch.div(positions.long() + 1, temp_every, rounding_mode="floor").float()
        x[:, :nh] = x[:, :nh] * (1.0 + temp_coef * torch.log(steps + 1.0)).reshape(T, 1, 1)
    qkv[:, :cols] = x.reshape(T, cols).to(qkv.dtype)
    return qkv


def head_gate_(x, gate, num_heads, head_dim):
    T = x.shape[0]
    g = torch.sigmoid(gate[:, :num_heads].float()).reshape(T, num_heads, 1)
    x.copy_((x.float().reshape(T, num_heads, head_dim) * g).reshape(T, -1).to(x.dtype))
    return x


def depth_mix_(x, delta, history, count, weights, save_input=False):
    if save_input:
        history[0] = x
    history[count - 1] = x + delta
    x.copy_(sum(weights[j].float() * history[j] for j in range(count)))


def decay_attention(q, k, v, decay, state, cu, slots, num_seqs, heads, dim, vdim, activation=True,
                    longest=None):
    T = q.shape[0]
    act = (lambda z: z / (1.0 + torch.exp(-z))) if activation else (lambda z: z)
    qq, kk = act(q.float()).reshape(T, heads, dim), act(k.float()).reshape(T, heads, dim)
    vv = act(v.float()).reshape(T, heads, vdim)
    out = torch.empty((T, heads * vdim), dtype=torch.float32)
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        S = state[slot, :heads * vdim * dim].reshape(heads, vdim, dim).clone()   # [head][value][key]
        for t in range(t0, t1):
            for h in range(heads):
                S[h] = decay[h] * S[h] + torch.outer(vv[t, h], kk[t, h])
                out[t, h * vdim:(h + 1) * vdim] = S[h] @ qq[t, h]
        state[slot, :heads * vdim * dim] = S.reshape(-1)
    return out


def add_residual(resid, delta, round_parts=False, delta_scale=1.0):
    resid += delta_scale * delta.to(torch.float32)


def add_rmsnorm(resid, delta, weight, eps, out_dtype, rows=None, write_resid=True,
                round_parts=False, delta_scale=1.0):
    x = resid if delta is None else resid + delta_scale * delta.to(torch.float32)
    if rows is not None:
        x = x[rows.long()]
    elif delta is not None and write_resid:
        resid.copy_(x)
    ms = (x * x).mean(dim=-1, keepdim=True)
    return (x / torch.sqrt(ms + eps) * weight.to(torch.float32)).to(out_dtype)


def swiglu(gu):
    i = gu.shape[1] // 2
    g, u = gu[:, :i].float(), gu[:, i:].float()
    return (g / (1.0 + torch.exp(-g)) * u).to(gu.dtype)


def clamped_glu(gu, limit, alpha):
    i = gu.shape[1] // 2
    g = gu[:, :i].float().clamp(max=limit)
    u = gu[:, i:].float().clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def weighted_sum(x, a, y, b=0.0, round_parts=False):
    x = x.sum(0) if x.dim() == 3 else x
    out = a * x.float()
    if y is not None:
        out = out + b * (y.sum(0) if y.dim() == 3 else y).float()
    return out


def linear_f32(x, w):
    return linear(x, w, torch.float32)


def soft_cap_(x, cap):
    x.copy_((cap * torch.tanh(x.float() / cap)).to(x.dtype))
    return x


# ---- mixers with a state of fixed size: the kernels' contracts, sequence by sequence --------
def _seqs(cu, slots, num_seqs):
    cu, slots = cu.tolist(), slots.tolist()
    return [(cu[s], cu[s + 1], slots[s]) for s in range(num_seqs)]


def shift_mix(x, mu, state, seq_of_token, cu, slots, num_seqs):
    out = torch.empty((mu.shape[0],) + tuple(x.shape), dtype=x.dtype)
    xf = x.float()
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        if t1 > t0:
            prev = torch.cat([state[slot, :x.shape[1]].reshape(1, -1), xf[t0:t1 - 1]], dim=0)
            cur = xf[t0:t1]
            for m in range(mu.shape[0]):
                out[m, t0:t1] = (cur + (prev - cur) * mu[m]).to(x.dtype)
    return out


def tail_update(state, x, channels, rows, cu, slots, num_seqs):
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        old = state[slot, :channels * rows].reshape(rows, channels).clone()
        both = torch.cat([old, x[t0:t1, :channels].float()], dim=0)
        state[slot, :channels * rows] = both[both.shape[0] - rows:].reshape(-1)


def causal_conv(x, taps, state, seq_of_token, cu, slots, num_seqs, unit_channels=0, unit_group=0,
                scaled_channels=0, scale=1.0, unit_eps=0.0, rest_group=256, bias=None,
                out_dtype=torch.float32, activation=True, blend=None, blend_from=0,
                blend_weight=0.0):
    C, K = taps.shape
    out = torch.empty((x.shape[0], C), dtype=torch.float32)
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        before = state[slot, :C * (K - 1)].reshape(K - 1, C) if K > 1 else x.new_zeros((0, C))
        both = torch.cat([before.float(), x[t0:t1, :C].float()], dim=0)
        acc = torch.zeros(t1 - t0, C) if bias is None else bias.reshape(1, C).repeat(t1 - t0, 1)
        for j in range(K):
            acc += both[j:j + t1 - t0] * taps[:, j]
        out[t0:t1] = acc / (1.0 + torch.exp(-acc)) if activation else acc
    if blend is not None:
        out[:, blend_from:] = (1.0 - blend_weight) * out[:, blend_from:] + blend_weight * blend.float()
    if unit_channels:
        y = out[:, :unit_channels].reshape(x.shape[0], -1, unit_group)
        y = y / torch.sqrt((y * y).sum(-1, keepdim=True) + unit_eps)
        out[:, :unit_channels] = y.reshape(x.shape[0], unit_channels)
        out[:, :scaled_channels] *= scale
    return out.to(out_dtype)


def selective_scan(x, dt_raw, dt_bias, b, c, z, a_log, skip, state, cu, slots, num_seqs):
    T, C = x.shape
    N = a_log.shape[1]
    out = torch.empty((T, C), dtype=torch.float32)
    A = -torch.exp(a_log)
    dt = torch.nn.functional.softplus(dt_raw + dt_bias)
    xf = x.float()
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        S = state[slot, :C * N].reshape(C, N).clone()
        for t in range(t0, t1):
            S = torch.exp(dt[t].reshape(C, 1) * A) * S + (dt[t] * xf[t]).reshape(C, 1) * b[t]
            y = S @ c[t] + skip * xf[t]
            out[t] = y * (z[t] / (1.0 + torch.exp(-z[t])))
        state[slot, :C * N] = S.reshape(-1)
    return out.to(x.dtype)


# ---- attention over a cached latent --------------------------------------------------------
def add_layernorm(resid, delta, weight, bias, eps, out_dtype, rows=None, write_resid=True,
                  round_parts=False, delta_scale=1.0):
    if delta is not None and delta.dim() == 3:
        delta = delta.sum(0)
    x = resid if delta is None else resid + delta_scale * delta.to(torch.float32)
    if rows is not None:
        x = x[rows.long()]
    elif delta is not None and write_resid:
        resid.copy_(x)
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return ((x - mean) / torch.sqrt(var + eps) * weight.float() + bias.float()).to(out_dtype)


def scale_(x, factor):
    x.mul_(factor)
    return x


def head_linear(x, w, x_head, out=None, out_head=None, out_dtype=None):
    H, N, K = w.shape
    T = x.shape[0]
    if out is None:
        out_head, out = N, torch.empty((T, H * N), dtype=out_dtype or x.dtype)
    for h in range(H):
        out[:, h * out_head:h * out_head + N] = \
            (x[:, h * x_head:h * x_head + K].float() @ w[h].float().t()).to(out.dtype)
    return out


def _turned(v, pos, cos, sin, dims):
    half = dims // 2
    c, s = cos[pos.long()], sin[pos.long()]
    while c.dim() < v.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)


def latent_mfma_ok(dtype, rank, row, page_size=16):
    return False


def latent_write(x, weight, eps, rank, rot_width, rot_dims, cos, sin, positions, slots, pages, q,
                 q_head, q_out, heads, pages_t=None):
    D = rank + rot_width
    if x is not None:
        lat = x[:, :rank]
        row = lat / torch.sqrt((lat * lat).mean(-1, keepdim=True) + eps) * weight
        if rot_width:
            kr = x[:, rank:D]
            row = torch.cat([row, _turned(kr, positions, cos, sin, rot_dims) if rot_dims else kr], -1)
        ps = pages.shape[1]
        for t in range(x.shape[0]):
            pages[int(slots[t]) // ps, int(slots[t]) % ps] = row[t].to(pages.dtype)
    if rot_width:
        T = q.shape[0]
        qr = q.float().reshape(T, heads, q_head)[..., q_head - rot_width:]
        if rot_dims:
            qr = _turned(qr, positions, cos, sin, rot_dims)
        q_out.reshape(T, heads, D)[..., rank:] = qr.to(q_out.dtype)


def latent_attention(q, pages, block_tables, seq_of_token, positions, heads, rank, scale,
                     window=None, sink=None, pages_t=None, cu=None, num_seqs=0):
    T = q.shape[0]
    ps, D = pages.shape[1], pages.shape[2]
    qf = q.float().reshape(T, heads, D)
    out = torch.zeros(T, heads, rank)
    for t in range(T):
        table = block_tables[int(seq_of_token[t])].tolist()
        pos = int(positions[t])
        lo = max(0, pos - window + 1) if window else 0
        rows = torch.stack([pages[table[p // ps], p % ps] for p in range(lo, pos + 1)]).float()
        s = (qf[t] @ rows.t()) * scale                                    # (heads, keys)
        if sink is not None:
            s = torch.cat([s, sink.reshape(heads, 1)], dim=1)
        p = torch.softmax(s, dim=1)[:, :rows.shape[0]]
        out[t] = p @ rows[:, :rank]
    return out.reshape(T, heads * rank).to(q.dtype)


def sigmoid_gate_(o, g):
    o.copy_((o.float() * torch.sigmoid(g.float())).to(o.dtype))
    return o


# ---- routed feed-forward -----------------------------------------------------------------
def router_logits(resid, norm_weight, norm_bias, eps, w_router):
    mean = resid.mean(-1, keepdim=True)
    var = ((resid - mean) ** 2).mean(-1, keepdim=True)
    h = (resid - mean) / torch.sqrt(var + eps) * norm_weight.float() + norm_bias.float()
    return h @ w_router.float().t()


def route(logits, correction, groups, keep, top, scale, scores="sigmoid", group_score="top2",
          renormalise=False, bias=None):
    T, E = logits.shape
    if bias is not None:
        logits = logits + bias
    s = torch.sigmoid(logits) if scores == "sigmoid" else torch.softmax(logits, dim=-1)
    choice = (s if correction is None else s + correction).reshape(T, groups, E // groups)
    score = choice.topk(1 if group_score == "max" else min(2, E // groups), dim=-1).values.sum(-1)
    kept = torch.zeros(T, groups, dtype=torch.bool)
    kept.scatter_(1, score.topk(keep, dim=-1).indices, True)
    choice = choice.masked_fill(~kept.unsqueeze(-1), float("-inf")).reshape(T, E)
    chosen = choice.topk(top, dim=-1).indices
    weights = (s.gather(1, chosen) * scale).float()
    if renormalise:
        weights = weights / (weights.sum(-1, keepdim=True) + 1e-20)
    return chosen.to(torch.int32), weights


def routed_units(x, w_gate_up, w_down, chosen, weights, addend=None, limit=0.0, alpha=1.0,
                 plain=False):
    T, W = x.shape
    F = w_gate_up.shape[1] // 2
    out = torch.zeros(T, W)
    for t in range(T):
        for e, wt in zip(chosen[t].tolist(), weights[t].tolist()):
            gu = w_gate_up[e].float() @ x[t].float()
            if plain:
                hidden = (gu.clamp(min=0.0) ** 2).to(x.dtype).float()
            elif limit > 0:
                g, u = gu[:F].clamp(max=limit), gu[F:].clamp(-limit, limit)
                hidden = (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(x.dtype).float()
            else:
                hidden = (gu[:F] / (1.0 + torch.exp(-gu[:F])) * gu[F:]).to(x.dtype).float()
            out[t] += wt * (w_down[e].float() @ hidden)
    return out if addend is None else out + addend.float()


def delta_scan(q, k, v, b_raw, a_raw, a_log, dt_bias, state, cu, slots, num_seqs, heads,
               kv_heads, dk, dv, tiled=None):
    T = q.shape[0]
    out = torch.empty((T, heads * dv), dtype=torch.float32)
    g = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(a_raw + dt_bias))
    beta = torch.sigmoid(b_raw)
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        S = state[slot, :heads * dv * dk].reshape(heads, dv, dk).clone()     # [head][value][key]
        for t in range(t0, t1):
            for h in range(heads):
                j = h // (heads // kv_heads)
                kt, qt = k[t, j * dk:(j + 1) * dk], q[t, j * dk:(j + 1) * dk]
                S[h] = g[t, h] * S[h]
                u = beta[t, h] * (v[t, h * dv:(h + 1) * dv] - S[h] @ kt)
                S[h] = S[h] + torch.outer(u, kt)
                out[t, h * dv:(h + 1) * dv] = S[h] @ qt
        state[slot, :heads * dv * dk] = S.reshape(-1)
    return out


def decay_scan(r, k, v, z, w0, bonus, state, cu, slots, num_seqs, heads, d, tiled=None):
    T = r.shape[0]
    out = torch.empty((T, heads * d), dtype=torch.float32)
    w = torch.exp(-torch.exp(z + w0)).reshape(T, heads, d)
    u = bonus.reshape(heads, d)
    rr, kk, vv = (t.reshape(T, heads, d) for t in (r, k, v))
    for t0, t1, slot in _seqs(cu, slots, num_seqs):
        S = state[slot, :heads * d * d].reshape(heads, d, d).clone()         # [head][value][key]
        for t in range(t0, t1):
            for h in range(heads):
                vk = torch.outer(vv[t, h], kk[t, h])
                out[t, h * d:(h + 1) * d] = (S[h] + vk * u[h]) @ rr[t, h]
                S[h] = S[h] * w[t, h] + vk
        state[slot, :heads * d * d] = S.reshape(-1)
    return out


def head_norm_gate(o, weight, gate, heads, dv, eps, out_dtype, sigmoid_gate=False):
    T = o.shape[0]
    x = o.reshape(T, heads, dv)
    x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    w = weight.reshape(heads, dv) if weight.numel() == heads * dv else weight.reshape(1, dv)
    g = gate.float().reshape(T, heads, dv)
    g = torch.sigmoid(g) if sigmoid_gate else g / (1.0 + torch.exp(-g))
    return (x * w * g).reshape(T, heads * dv).to(out_dtype)


def linear(x, w, out_dtype=None, partials=False):
    return (x.float() @ w.float().t()).to(out_dtype or x.dtype)


def pending_linear(x, w, out_dtype=None):
    return linear(x, w, out_dtype, partials=True)


def linear_swiglu(x, w_gate_up):
    return swiglu(linear(x, w_gate_up, x.dtype))


def can_fuse_norm_linear(resid, w, rows=None):
    return False


def rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, cos, sin, positions, slots, k_pages,
                  v_pages, page_size, write_kv=True, interleaved=False):
    assert not interleaved, "the test double rotates halves only"
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    x = qkv.float()
    q = x[:, :nh * d].reshape(T, nh, d).clone()
    k = x[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d).clone()
    v = x[:, (nh + nkv) * d:(nh + 2 * nkv) * d].reshape(T, nkv, d)
    if cos is not None:
        half = cos.shape[1]
        c = cos[positions.long()].unsqueeze(1)
        s = sin[positions.long()].unsqueeze(1)
        for t in (q, k):
            x1, x2 = t[..., :half].clone(), t[..., half:2 * half].clone()
            t[..., :half] = x1 * c - x2 * s
            t[..., half:2 * half] = x2 * c + x1 * s
    qkv[:, :nh * d] = q.reshape(T, nh * d).to(qkv.dtype)
    if write_kv:
        for t in range(T):
            page, off = int(slots[t]) // page_size, int(slots[t]) % page_size
            k_pages[page, :, off, :] = k[t].to(k_pages.dtype)
            v_pages[page, :, :, off] = v[t].to(v_pages.dtype)


def copy_pages(pages, src, dst):
    for s, d in zip(src.tolist(), dst.tolist()):
        pages[:, d] = pages[:, s]


def attention_planner(num_heads, num_kv_heads, head_dim, dtype, biased=False, shaped=False,
                      plain=False):
    from rust_llm_inference_server_amd.ops.attention_plan import AttentionPlanner
    return AttentionPlanner(num_heads, num_kv_heads, head_dim, matrix=dtype == torch.bfloat16)


def paged_attention(qkv, num_heads, num_kv_heads, head_dim, k_pages, v_pages, page_size,
                    block_tables, step, scale, window=None, force=None, plan=None,
                    bias_slopes=None, counters=None, head_scales=None, softcap=0.0, sinks=None,
                    keep_first=0):
    assert bias_slopes is None, "the test double adds no bias"
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    g = nh // nkv
    q = qkv[:, :nh * d].float().reshape(T, nh, d)
    out = torch.zeros(T, nh * d)
    seq_of = step.seq_of_token.tolist()
    pos = step.positions.tolist()
    for t in range(T):
        table = block_tables[seq_of[t]].tolist()
        lo = max(0, pos[t] - window + 1) if window else 0
        keys = list(range(0, min(keep_first, lo) if window else 0)) + list(range(lo, pos[t] + 1))
        k = torch.stack([k_pages[table[p // page_size], :, p % page_size, :] for p in keys]).float()
        v = torch.stack([v_pages[table[p // page_size], :, :, p % page_size] for p in keys]).float()
        for h in range(nh):
            s = (k[:, h // g, :] @ q[t, h]) * scale
            if head_scales is not None:
                s = s * head_scales[h]
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if sinks is not None:
                p = torch.softmax(torch.cat([s, sinks[h].reshape(1).float()]), dim=0)[:-1]
            else:
                p = torch.softmax(s, dim=0)
            out[t, h * d:(h + 1) * d] = p @ v[:, h // g, :]
    return out.to(qkv.dtype)


def rope_attention(qkv, num_heads, num_kv_heads, head_dim, cos, sin, positions, slots, k_pages,
                   v_pages, page_size, block_tables, step, scale, window=None, write_kv=True,
                   plan=None, interleaved=False, bias_slopes=None, counters=None,
                   head_scales=None, softcap=0.0, sinks=None, keep_first=0):
    own = 0 if qkv.shape[1] == num_heads * head_dim else num_kv_heads     # queries alone?
    rope_kv_write(qkv, num_heads, own, head_dim, cos, sin, positions, slots, k_pages,
                  v_pages, page_size, write_kv=write_kv and own > 0)
    return paged_attention(qkv, num_heads, num_kv_heads, head_dim, k_pages, v_pages, page_size,
                           block_tables, step, scale, window, head_scales=head_scales,
                           softcap=softcap, sinks=sinks, keep_first=keep_first)


def _lowbias32(x):
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def sample_rows(logits, keys, inv_temps):
    import numpy as np
    out = []
    for r in range(logits.shape[0]):
        x = logits[r].numpy().astype(np.float32)
        inv_t = float(inv_temps[r])
        if inv_t > 0:
            key = int(keys[r]) & 0xFFFFFFFF
            s = np.empty_like(x)
            for v in range(x.shape[0]):
                h = _lowbias32(key ^ ((v * 0x9E3779B9) & 0xFFFFFFFF))
                u = np.float32((np.float32(h >> 9) + np.float32(0.5)) * np.float32(1.0 / 8388608.0))
                s[v] = np.float32(x[v] * np.float32(inv_t)) + np.float32(-np.log(-np.log(u)))
            x = s
        out.append(int(np.argmax(x)))
    return torch.tensor(out, dtype=torch.int32)


def install(monkeypatch) -> None:
    """Replace the package's kernel functions with the ones above."""
    import rust_llm_inference_server_amd.ops as ops
    import rust_llm_inference_server_amd.engine.runner as runner
    for name in ("embed", "add_residual", "add_rmsnorm", "swiglu", "linear", "linear_swiglu",
                 "pending_linear", "can_fuse_norm_linear", "rope_kv_write", "rope_attention",
                 "copy_pages", "attention_planner", "paged_attention", "sample_rows",
                 "clamped_glu", "weighted_sum", "linear_f32", "soft_cap_", "shift_mix", "tail_update",
                 "causal_conv", "delta_scan", "decay_scan", "head_norm_gate", "selective_scan",
                 "add_layernorm", "scale_", "head_linear", "latent_write", "latent_attention",
                 "latent_mfma_ok",
                 "sigmoid_gate_", "route", "routed_units", "router_logits", "gelu_tanh",
                 "depth_mix_", "decay_attention", "gelu_erf", "lanes_step", "head_prepare_",
                 "head_gate_"):
        monkeypatch.setattr(ops, name, globals()[name])
    monkeypatch.setattr(runner, "default_device", lambda: torch.device("cpu"))
