"""Stand-ins for the HIP kernels, written with torch on the CPU.

The product has no CPU path.  These functions exist so that tests which run without
a GPU can exercise everything *around* the kernels (batch descriptors, block
tables, page reuse, the scheduler) by patching `cwm_amd.ops`; they follow the same
signatures and the same cache layout as the kernels' wrappers.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from helpers import cache_layout


def embedding(tokens, table, scale=1.0):
    return table[tokens.long()].float() * scale


def add_rmsnorm(h, delta, weight, eps, out_dtype, rows=None):
    if delta is not None and delta.dim() == 3:
        delta = delta.float().sum(0)
    if delta is not None:
        if rows is None:
            h += delta.float()
            x = h
        else:
            x = h + delta.float()
    else:
        x = h
    if rows is not None:
        x = x[rows.long()]
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * weight.float()
    return y.to(out_dtype)


def silu_mul(gate_up, out_dtype=None, grouped=False):
    if gate_up.dim() == 3:
        gate_up = gate_up.sum(0).to(out_dtype or torch.float32)
    f = gate_up.shape[1] // 2
    if grouped:
        pairs = gate_up.reshape(gate_up.shape[0], f // 8, 2, 8)
        g, u = pairs[:, :, 0].reshape(-1, f).float(), pairs[:, :, 1].reshape(-1, f).float()
    else:
        g, u = gate_up[:, :f].float(), gate_up[:, f:].float()
    return (g * torch.sigmoid(g) * u).to(gate_up.dtype)


def gate_up_silu(x, weight, bias, grouped, streamed=None):
    return silu_mul(linear(x, weight, bias), grouped=grouped)


def linear(x, weight, bias=None, out_dtype=None, partials_ok=False, streamed=None):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype or x.dtype)


gemm_f32 = linear
gemm_bf16 = linear


def _rotate(x, positions, inv_freq):
    ang = positions.float()[:, None] * inv_freq[None, :]
    c = torch.cos(ang)[:, None, :]
    s = torch.sin(ang)[:, None, :]
    xf = x.float()
    re, im = xf[..., 0::2], xf[..., 1::2]
    out = torch.empty_like(xf)
    out[..., 0::2] = re * c - im * s
    out[..., 1::2] = im * c + re * s
    return out.to(x.dtype)


def rope_kv_write(q, k, v, positions, inv_freq, cache=None, block_table=None, seq_of_token=None):
    if inv_freq is not None:
        q.copy_(_rotate(q, positions, inv_freq))
        if k is not None:
            k.copy_(_rotate(k, positions, inv_freq))
    if cache is None:
        return
    n_tokens, n_kv, hd = k.shape
    page_size = cache.shape[3] // hd
    for t in range(n_tokens):
        pos = int(positions[t])
        page = int(block_table[int(seq_of_token[t]), pos // page_size])
        assert page >= 0, "write to a page that is not held"
        slot = pos % page_size
        cache_layout.write_kv(cache, page, slot, k[t], v[t], hd)


def qkv_rope_write(x, weight, bias, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, cache, block_table, seq_of_token, streamed=None):
    qkv = linear(x, weight, bias)
    q_out, kv_out = n_q_heads * head_dim, n_kv_heads * head_dim
    q = qkv[:, :q_out].unflatten(1, (n_q_heads, head_dim))
    k = qkv[:, q_out : q_out + kv_out].unflatten(1, (n_kv_heads, head_dim))
    v = qkv[:, q_out + kv_out :].unflatten(1, (n_kv_heads, head_dim))
    rope_kv_write(q, k, v, positions, inv_freq, cache, block_table, seq_of_token)
    return qkv


def paged_attention(q, cache, block_table, batch, window, scale, sink=None, softcap=None, chunk=None):
    n_tokens, n_q, hd = q.shape
    n_kv = cache.shape[2]
    page_size = cache.shape[3] // hd
    group = n_q // n_kv
    out = torch.empty((n_tokens, n_q, hd), dtype=torch.float32)
    for t in range(n_tokens):
        p = int(batch.positions[t])
        b = int(batch.seq_of_token[t])
        lo = 0 if window is None else max(0, p - (window - 1))
        if chunk is not None:
            lo = p - p % chunk
        keys, vals = [], []
        for j in range(lo, p + 1):
            page = int(block_table[b, j // page_size])
            assert page >= 0, f"key {j} of sequence {b} has no page"
            slot = j % page_size
            kk_, vv_ = cache_layout.read_kv(cache, page, slot, hd)
            keys.append(kk_.float())
            vals.append(vv_.float())
        kk = torch.stack(keys, 1)  # [n_kv, n, hd]
        vv = torch.stack(vals, 1)
        for h in range(n_q):
            g = h // group
            s = (kk[g] @ q[t, h].float()) * scale
            if softcap is not None:
                s = softcap * torch.tanh(s / softcap)
            if sink is not None:  # one more term of the denominator, without a key or a value
                w = torch.softmax(torch.cat([s, sink[h].float().reshape(1)]), -1)[:-1]
            else:
                w = torch.softmax(s, -1)
            out[t, h] = w @ vv[g]
    return out.reshape(n_tokens, n_q * hd).to(q.dtype)


def sample(logits, temperature, top_p, uniform):
    n, vocab = logits.shape
    toks = torch.empty(n, dtype=torch.int32)
    lp = torch.empty(n)
    slp = torch.empty(n)
    for r in range(n):
        x = logits[r].float()
        logp = torch.log_softmax(x, -1)
        t = float(temperature[r])
        if not t > 0:
            tok = int(torch.argmax(x))
            toks[r], lp[r], slp[r] = tok, logp[tok], 0.0
            continue
        probs = torch.softmax(x / t, -1)
        tp = float(top_p[r])
        if tp < 1.0:
            sp, order = torch.sort(probs, descending=True)
            cs = torch.cumsum(sp, -1)
            sp[cs - sp > tp] = 0.0
            kept = torch.zeros_like(probs)
            kept[order] = sp
            probs = kept
        c = torch.cumsum(probs.double(), -1)
        target = float(uniform[r]) * float(c[-1])
        tok = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64), right=True))
        tok = min(tok, vocab - 1)
        while probs[tok] <= 0:
            tok -= 1
        toks[r], lp[r], slp[r] = tok, logp[tok], math.log(float(probs[tok] / probs.sum()))
    return toks, lp, slp


def sample_packed(logits, temperature, top_p, uniform):
    toks, lp, slp = sample(logits, temperature, top_p, uniform)
    return torch.stack([toks, lp.float().view(torch.int32), slp.float().view(torch.int32)])


def token_logprobs(logits, rows, targets):
    lp = torch.log_softmax(logits.float()[rows.long()], -1)
    return lp.gather(1, targets.long()[:, None])[:, 0]


# ---- layers with group norms, token shift, a selective state space, a latent attention and routed experts ---- #
def group_rmsnorm(x, weight, groups, eps, out_dtype, rows=None, out=None, accumulate=False, gate=None, copy=None):
    v = x.float().sum(0) if x.dim() == 3 else x.float()
    if gate is not None:
        g = gate.float()
        v = v * (g * torch.sigmoid(g))
    if rows is not None:
        v = v[rows.long()]
    parts = v.reshape(v.shape[0], groups, -1)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    y = parts.reshape(v.shape) * weight.float()
    if out is None:
        return y.to(out_dtype)
    if accumulate:
        out += y.to(out.dtype)
    else:
        out.copy_(y.to(out.dtype))
    if copy is not None:
        copy.copy_(out.to(copy.dtype))
    return out


def cast_rows(h, dtype):
    return h if h.dtype == dtype else h.to(dtype)


def token_shift(h, mu, state, batch, out_dtype, write_state=True):
    out = torch.empty(h.shape, dtype=torch.float32)
    for b in range(batch.n_seqs):
        lo, hi = int(batch.cu_q[b]), int(batch.cu_q[b + 1])
        slot = int(batch.state_slots[b])
        first = torch.zeros_like(h[0]) if int(batch.positions[lo]) == 0 else state[slot].clone()
        prev = torch.cat([first[None], h[lo : hi - 1]], 0)
        out[lo:hi] = h[lo:hi] + (prev - h[lo:hi]) * mu
        if write_state:
            state[slot] = h[hi - 1]
    return out.to(out_dtype)


def sigmoid_mul(a, gate):
    return (a.float() * torch.sigmoid(gate.float())).to(a.dtype)


def causal_conv_silu(x, weight, bias, state, state_offset, batch, weight_by_tap=None):
    taps, channels = weight.shape[1], x.shape[1]
    out = torch.empty(x.shape, dtype=torch.float32)
    for b in range(batch.n_seqs):
        lo, hi = int(batch.cu_q[b]), int(batch.cu_q[b + 1])
        slot = int(batch.state_slots[b])
        kept = state[slot, state_offset : state_offset + (taps - 1) * channels].reshape(taps - 1, channels)
        seq = torch.cat([kept, x[lo:hi].float()], 0)
        acc = bias.expand(hi - lo, -1).clone()
        for k in range(taps):
            acc = acc + seq[k : k + hi - lo] * weight[:, k]
        out[lo:hi] = acc * torch.sigmoid(acc)
        state[slot, state_offset : state_offset + (taps - 1) * channels] = seq[seq.shape[0] - (taps - 1) :].reshape(-1)
    return out.to(x.dtype)


def selective_scan(xbc, dt, dt_bias, a_log, d_skip, state, batch, heads, head_dim, n_state, groups):
    inner = heads * head_dim
    y = torch.empty((xbc.shape[0], inner), dtype=torch.float32)
    per_group = heads // groups
    for b in range(batch.n_seqs):
        lo, hi = int(batch.cu_q[b]), int(batch.cu_q[b + 1])
        slot = int(batch.state_slots[b])
        carry = state[slot, : heads * n_state * head_dim].reshape(heads, n_state, head_dim).clone()
        for t in range(lo, hi):
            row = xbc[t].float()
            x = row[:inner].reshape(heads, head_dim)
            bm = row[inner : inner + groups * n_state].reshape(groups, n_state).repeat_interleave(per_group, 0)
            cm = row[inner + groups * n_state :].reshape(groups, n_state).repeat_interleave(per_group, 0)
            step = torch.nn.functional.softplus(dt[t].float() + dt_bias)
            decay = torch.exp(-torch.exp(a_log) * step)
            carry = decay[:, None, None] * carry + step[:, None, None] * bm[:, :, None] * x[:, None, :]
            y[t] = (torch.einsum("hnp,hn->hp", carry, cm) + d_skip[:, None] * x).reshape(-1)
        state[slot, : heads * n_state * head_dim] = carry.reshape(-1)
    return y


def route_top(logits, top, scores="softmax_chosen", correction=None, scale=1.0, renormalize=False):
    if scores == "softmax_all":
        s = torch.softmax(logits.float(), -1)
        choice = s + correction.float() if correction is not None else s
        chosen = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        w = torch.gather(s, 1, chosen)
        if renormalize:
            w = w / w.sum(-1, keepdim=True)
        return chosen.to(torch.int32), w * scale
    order = torch.sort(logits, dim=-1, descending=True, stable=True)
    values, chosen = order.values[:, :top], order.indices[:, :top]
    return chosen.to(torch.int32), torch.softmax(values, -1)


def group_by_expert(chosen, n_experts):
    return chosen  # the stand-ins keep one row a pair, in the order of the pairs


def grouped_gate_up(x, groups, gate, up, activation=None):
    e = groups.reshape(-1).long()
    rows = x.float().repeat_interleave(groups.shape[1], 0)
    g = torch.einsum("rd,rfd->rf", rows, gate.float()[e])
    u = torch.einsum("rd,rfd->rf", rows, up.float()[e])
    if activation is not None and activation.kind == "clamped_swish":
        g = g.clamp(max=activation.limit)
        u = u.clamp(-activation.limit, activation.limit)
        return (g * torch.sigmoid(activation.alpha * g) * (u + 1)).to(x.dtype)
    return (g * torch.sigmoid(g) * u).to(x.dtype)


def grouped_linear(rows, groups, weight):
    return torch.einsum("rf,rdf->rd", rows.float(), weight.float()[groups.reshape(-1).long()])


def combine_routed(rows, groups, weights):
    n, top = weights.shape
    return (rows.reshape(n, top, -1) * weights[:, :, None]).sum(1)


def absorb_queries(q, lead, weight):
    rest = torch.einsum("thd,hnd->thn", q[:, :, lead:].float(), weight.float())
    return torch.cat([q[:, :, :lead].float(), rest], -1).to(q.dtype).contiguous()


def expand_values(mixed, lead, weight):
    return torch.einsum("thn,hvn->thv", mixed[:, :, lead:].float(), weight.float()).reshape(mixed.shape[0], -1).to(mixed.dtype)


def embedding_streams(tokens, table, streams, scale=1.0):
    return (table[tokens.long()].float() * scale).repeat(1, streams)


def stream_mix_norm(x, streams, y, mix, out_coef, in_coef, weight, eps, out_dtype, rows=None):
    n = x.shape[0]
    xs = x.view(n, streams, -1)
    new = xs
    if y is not None and hasattr(y, "groups"):  # a weighted sum of rows that has not been added up
        y = combine_routed(y.rows, y.groups, y.weights)
    if y is not None:
        if y.dim() == 3:
            y = y.float().sum(0)
        m = mix if mix is not None else torch.eye(streams)
        b = out_coef if out_coef is not None else torch.ones(streams)
        new = torch.einsum("st,nsd->ntd", m.float(), xs) + b.float()[None, :, None] * y.float()[:, None, :]
        if rows is None:
            xs.copy_(new)
    a = in_coef if in_coef is not None else torch.ones(streams)
    u = (a.float()[None, :, None] * new).sum(1)
    if rows is not None:
        u = u[rows.long()]
    return (u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype)


def act_rows(x, kind, out_dtype):
    if x.dim() == 3:
        x = x.sum(0)
    z = x.float()
    if kind == "relu2":
        z = torch.relu(z) ** 2
    elif kind == "relu":
        z = torch.relu(z)
    elif kind == "gelu_tanh":
        z = torch.nn.functional.gelu(z, approximate="tanh")
    else:
        z = z * torch.sigmoid(z)
    return z.to(out_dtype)


def qk_norm_rope_write(qkv, n_q_heads, n_kv_heads, qk_dim, v_dim, head_dim, q_weight, k_weight, eps, positions, inv_freq, out_dtype,
                       cache=None, block_table=None, seq_of_token=None):
    if qkv.dim() == 3:
        qkv = qkv.sum(0)
    qkv = qkv.float()
    n = qkv.shape[0]
    qw, kw = n_q_heads * qk_dim, n_kv_heads * qk_dim
    q, k, v = qkv[:, :qw], qkv[:, qw : qw + kw], qkv[:, qw + kw :]
    if q_weight is not None:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.float()
    if k_weight is not None:
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.float()

    def padded(t, heads, width):
        out = torch.zeros((n, heads, head_dim), dtype=torch.float32)
        out[:, :, :width] = t.reshape(n, heads, width)
        return out

    q, k, v = padded(q, n_q_heads, qk_dim), padded(k, n_kv_heads, qk_dim), padded(v, n_kv_heads, v_dim)
    if inv_freq is not None:
        q, k = _rotate(q, positions, inv_freq), _rotate(k, positions, inv_freq)
    q, k, v = q.to(out_dtype), k.to(out_dtype), v.to(out_dtype)
    if cache is not None:
        rope_kv_write(q.clone(), k, v, positions, None, cache, block_table, seq_of_token)
    return q


def talking_attention(q, cache, block_table, batch, window, scale, sink=None, talk=None):
    n_tokens, n_q, hd = q.shape
    n_kv = cache.shape[2]
    page_size = cache.shape[3] // hd
    group = n_q // n_kv
    out = torch.empty((n_tokens, n_q, hd), dtype=torch.float32)
    for t in range(n_tokens):
        p = int(batch.positions[t])
        b = int(batch.seq_of_token[t])
        lo = 0 if window is None else max(0, p - (window - 1))
        keys, vals = [], []
        for j in range(lo, p + 1):
            page = int(block_table[b, j // page_size])
            assert page >= 0, f"key {j} of sequence {b} has no page"
            kk_, vv_ = cache_layout.read_kv(cache, page, j % page_size, hd)
            keys.append(kk_.float())
            vals.append(vv_.float())
        kk = torch.stack(keys, 1)  # [n_kv, n, hd]
        vv = torch.stack(vals, 1)
        weights = []
        for h in range(n_q):
            s = (kk[h // group] @ q[t, h].float()) * scale
            if sink is not None:
                weights.append(torch.softmax(torch.cat([s, sink[h].float().reshape(1)]), -1)[:-1])
            else:
                weights.append(torch.softmax(s, -1))
        w = torch.stack(weights)  # [n_q, n]
        if talk is not None:
            w = talk.float() @ w
        for h in range(n_q):
            out[t, h] = w[h] @ vv[h // group]
    return out.reshape(n_tokens, n_q * hd).to(q.dtype)


def gated_linear_attention(proj, decay_logits, weight, state, batch, heads, dim, vdim, tau, eps, q_scale=None):
    """The state's layout is the stand-in's own: per head the matrix [dim, vdim]."""
    n = proj.shape[0]
    p = proj.float()
    q = p[:, : heads * dim].reshape(n, heads, dim) * (dim ** -0.5 if q_scale is None else q_scale)
    k = p[:, heads * dim : 2 * heads * dim].reshape(n, heads, dim)
    v = p[:, 2 * heads * dim : 2 * heads * dim + heads * vdim].reshape(n, heads, vdim)
    g = p[:, 2 * heads * dim + heads * vdim : 2 * heads * (dim + vdim)].reshape(n, heads, vdim)
    alpha = torch.exp(torch.nn.functional.logsigmoid(decay_logits.float()) / tau).reshape(n, heads, dim)
    y = torch.zeros((n, heads, vdim))
    for b in range(batch.n_seqs):
        row = state[int(batch.state_slots[b])]
        S = row[: heads * dim * vdim].reshape(heads, dim, vdim).clone()
        for t in range(int(batch.cu_q[b]), int(batch.cu_q[b + 1])):
            S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            y[t] = torch.einsum("hde,hd->he", S, q[t])
        row[: heads * dim * vdim] = S.reshape(-1)
    y = y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps) * weight.float()
    return (y * (g * torch.sigmoid(g))).reshape(n, heads * vdim).to(proj.dtype)


def short_conv(x, weights, state, batch, write_state=True):
    taps, dim = weights[0].shape
    xf = x.float()
    outs = [torch.empty_like(xf) for _ in weights]
    for b in range(batch.n_seqs):
        t0, t1 = int(batch.cu_q[b]), int(batch.cu_q[b + 1])
        if taps > 1:
            row = state[int(batch.state_slots[b])]
            past = row[: (taps - 1) * dim].reshape(taps - 1, dim)
            full = torch.cat([past, xf[t0:t1]])
        else:
            full = xf[t0:t1]
        for w, out in zip(weights, outs):
            for t in range(t1 - t0):
                out[t0 + t] = xf[t0 + t] + (w.float() * full[t : t + taps]).sum(0)
        if taps > 1 and write_state:
            row[: (taps - 1) * dim] = full[full.shape[0] - (taps - 1) :].reshape(-1)
    return tuple(out.to(x.dtype) for out in outs)


def _as(t, dtype):
    return t.to(dtype).float()


def token_side(h, tokens, table, column0, w_gate, w_proj_t, weight, eps, round_inputs, pending=None):
    if pending is not None:
        h += _total(pending)
    side_dim = w_gate.shape[0]
    rd = torch.bfloat16 if round_inputs else torch.float32
    z = _as(_as(h, rd) @ w_gate.float().T, rd)
    gelu = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    g = _as(gelu * table[tokens.long(), column0 : column0 + side_dim].float(), rd)
    y = g @ w_proj_t.float()
    h += y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps) * weight.float()


def gated_act_rows(x, hidden, activation, out_dtype, row_gate_col=None):
    if x.dim() == 3:
        x = x.sum(0)
    x = x.float()
    g, u = x[:, :hidden], x[:, hidden : 2 * hidden]
    if activation.kind == "clamped_swish":
        g = torch.clamp(g, max=activation.limit)
        u = torch.clamp(u, min=-activation.limit, max=activation.limit)
        y = g * torch.sigmoid(activation.alpha * g) * (u + 1.0)
    else:
        y = g * torch.sigmoid(g) * u
    if row_gate_col is not None:
        y = y * torch.sigmoid(x[:, row_gate_col : row_gate_col + 1])
    return y.to(out_dtype)


def _total(delta):
    """A pending update (a tensor, partial sums, or a sum of scaled terms) as one float32 tensor."""
    terms = delta.terms if hasattr(delta, "terms") else [(delta, 1.0)]
    out = None
    for t, c in terms:
        x = (t.float().sum(0) if t.dim() == 3 else t.float()) * c
        out = x if out is None else out + x
    return out


def add_layernorm(h, delta, weight, bias, eps, out_dtype, rows=None, weight2=None, bias2=None):
    x = h
    if delta is not None:
        if rows is None:
            h += _total(delta)
        else:
            x = h + _total(delta)
    if weight is None:
        return None
    if rows is not None:
        x = x[rows.long()]
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    unit = (x - mean) * torch.rsqrt(var + eps)
    first = (unit * weight.float() + bias.float()).to(out_dtype)
    if weight2 is None:
        return first
    return first, (unit * weight2.float() + bias2.float()).to(out_dtype)


def head_norm_rope_write(qkv, n_q_heads, n_kv_heads, qk_dim, v_dim, head_dim, bias, q_weight, k_weight, eps, positions, inv_freq, out_dtype,
                         cache=None, block_table=None, seq_of_token=None, v_other=None, v_mix=None, keep_values=False):
    if qkv.dim() == 3:
        qkv = qkv.sum(0)
    n = qkv.shape[0]
    qw, kw, vw = n_q_heads * qk_dim, n_kv_heads * qk_dim, n_kv_heads * v_dim
    qkv = qkv.float()[:, : qw + kw + vw]
    if bias is not None:
        qkv = qkv + bias.float()
    q, k, v = qkv[:, :qw].reshape(n, n_q_heads, qk_dim), qkv[:, qw : qw + kw].reshape(n, n_kv_heads, qk_dim), qkv[:, qw + kw :]
    if q_weight is not None:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.float()
    if k_weight is not None:
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.float()
    if v_other is not None:
        lam = float(v_mix.reshape(-1)[0])
        v = (1.0 - lam) * v + lam * v_other.float()
    kept = v.to(out_dtype)

    def padded(t, heads, width):
        out = torch.zeros((n, heads, head_dim), dtype=torch.float32)
        out[:, :, :width] = t.reshape(n, heads, width)
        return out

    q, k, v = padded(q, n_q_heads, qk_dim), padded(k, n_kv_heads, qk_dim), padded(v, n_kv_heads, v_dim)
    if inv_freq is not None:
        q, k = _rotate(q, positions, inv_freq), _rotate(k, positions, inv_freq)
    q, k, v = q.to(out_dtype), k.to(out_dtype), v.to(out_dtype)
    if cache is not None:
        rope_kv_write(q.clone(), k, v, positions, None, cache, block_table, seq_of_token)
    return (q, kept) if keep_values else q


def matrix_memory(proj, gates, weight, state, batch, heads, dim, vdim, cap, eps, q_scale=None):
    """The state's layout is the stand-in's own: per head the matrix [dim, vdim], then the normaliser, then the maximum."""
    n = proj.shape[0]
    p = proj.float()
    q = p[:, : heads * dim].reshape(n, heads, dim) * (dim ** -0.5 if q_scale is None else q_scale)
    k = p[:, heads * dim : 2 * heads * dim].reshape(n, heads, dim)
    v = p[:, 2 * heads * dim : 2 * heads * dim + heads * vdim].reshape(n, heads, vdim)
    g = p[:, 2 * heads * dim + heads * vdim :].reshape(n, heads, vdim)
    gi = cap * torch.tanh(gates.float()[:, :heads] / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(gates.float()[:, heads:] / cap))
    y = torch.zeros((n, heads, vdim))
    per = dim * vdim + dim + 1
    for b in range(batch.n_seqs):
        row = state[int(batch.state_slots[b])]
        for h in range(heads):
            st = row[h * per : (h + 1) * per]
            S, nn, m = st[: dim * vdim].reshape(dim, vdim).clone(), st[dim * vdim : dim * vdim + dim].clone(), float(st[-1])
            for t in range(int(batch.cu_q[b]), int(batch.cu_q[b + 1])):
                m_new = max(float(gf[t, h]) + m, float(gi[t, h]))
                keep, take = math.exp(float(gf[t, h]) + m - m_new), math.exp(float(gi[t, h]) - m_new)
                S = keep * S + take * torch.outer(k[t, h], v[t, h])
                nn = keep * nn + take * k[t, h]
                m = m_new
                y[t, h] = (S.T @ q[t, h]) / (max(abs(float(nn @ q[t, h])), math.exp(-m)) + 1e-6)
            st[: dim * vdim], st[dim * vdim : dim * vdim + dim], st[-1] = S.reshape(-1), nn, m
    y = y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps)
    return (y.reshape(n, heads * vdim) * weight.float() * torch.sigmoid(g.reshape(n, heads * vdim))).to(proj.dtype)


STAND_INS = (
    "talking_attention", "gated_linear_attention", "short_conv", "token_side", "gated_act_rows",
    "add_layernorm", "head_norm_rope_write", "matrix_memory",
    "embedding_streams", "stream_mix_norm", "act_rows", "qk_norm_rope_write",
    "embedding", "add_rmsnorm", "silu_mul", "gate_up_silu", "linear", "gemm_f32", "gemm_bf16",
    "rope_kv_write", "qkv_rope_write", "paged_attention", "sample", "sample_packed", "token_logprobs",
    "group_rmsnorm", "cast_rows", "token_shift", "sigmoid_mul", "causal_conv_silu", "selective_scan", "route_top",
    "group_by_expert", "grouped_gate_up", "grouped_linear", "combine_routed", "absorb_queries", "expand_values",
)


def install(monkeypatch) -> None:
    """Patch every kernel entry point of `cwm_amd.ops` with its stand-in."""
    import cwm_amd.ops as ops

    for name in STAND_INS:
        monkeypatch.setattr(ops, name, globals()[name])
