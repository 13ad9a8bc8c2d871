"""The Digasun decoder, written plainly: whole sequences, no cache, float64, one function per mechanism.
Nothing here is imported from the product; the product is compared with this.

Notation: T tokens, D the model's width.  A model is a dictionary `config` (as config.json holds it) and a
dictionary `w` of float64 tensors by the folder's names.

    x_0        = c_e E[token]
    layer i:     h = ln(x);  a = h + conv_1(h);  b = h + conv_2(h)        causal convolutions over time, a channel each
                 x <- x + mixer(a) + ff(b)
                 y = P (gelu_tanh(G x) * E_side[token, i-th part]);  x <- x + y / rms(y) * n      (after the sum above)
    ln(v)      = (v - mean) / sqrt(var + eps) * g + b                     var: mean squared deviation
    attention:   q, k, v = W h + bias;  the first `rot.dims` of a head turned in pairs (i, i + dims/2) by
                 p * base^(-2i/dims);  s = scale q.k over the keys j with 0 <= i - j < mask.size;
                 p_g(i, j) = exp(s) / (sum_j' exp(s) + exp(sink_g));  weights of head h: sum_g T[h, g] p_g, applied to
                 the values of h's own key/value head;  out = W_o heads + bias.  With `kv_from` keys and values are
                 another layer's.
    gla:         q = W_q h / sqrt(d), k = W_k h, v = W_v h;  alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau), a key channel each;
                 S_t = diag(alpha_t) S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t;  out = W_o (rms(o per head) * n * silu(W_g h))
    dense ff:    g = min(W_gate h, l), u = clamp(W_up h, -l, l);  W_down (g sigmoid(1.702 g) (u + 1))
    experts:     z = W_r h + b;  the `top` largest;  weights softmax over those alone;  sum_e w_e W_down,e (silu(W_gate,e h) * W_up,e h)
                 + sigmoid(w_sg . h) * shared(h)
    logits     = W_head ln_final(x)
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

F = torch.float64


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


def layer_norm(x: torch.Tensor, g: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * g + b


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def causal_conv(h: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """h [T, D], weight [D, taps]: out_t = sum over lags 0 .. taps - 1 of weight[:, taps - 1 - lag] * h_(t - lag), h_t = 0 for t < 0."""
    n, taps = h.shape[0], weight.shape[1]
    out = torch.zeros_like(h)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += weight[:, j] * h[s]
    return out


def turn_halves(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, H, d]: element i < dims/2 of every head is paired with element i + dims/2; the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=F)
    freq = base ** (-2.0 * i / dims)
    a = positions.to(F)[:, None] * freq[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sliding_visible(n: int, size: Optional[int]) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & (i - j < size)
    return ok


def sink_softmax(scores: torch.Tensor, visible: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """scores [H, T, T] -> weights [H, T, T] whose rows add up to less than one by the sink's share."""
    s = scores.masked_fill(~visible[None], float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    denom = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None] - m)
    return e / denom


def mix_heads(weights: torch.Tensor, talk: Optional[torch.Tensor]) -> torch.Tensor:
    """weights [H, T, T], talk [H, H]: head h gets sum_g talk[h, g] weights_g."""
    if talk is None:
        return weights
    return torch.einsum("hg,gij->hij", talk, weights)


def project(w: Dict[str, torch.Tensor], name: str, h: torch.Tensor) -> torch.Tensor:
    y = h @ w[name].T
    if name + ".b" in w:
        y = y + w[name + ".b"]
    return y


def attention_keys_values(w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, rounded: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """The rotated keys [T, G, d] and the values [T, G, e] that a layer with projections of its own makes and caches."""
    rd = bf16_round if rounded else (lambda t: t)
    n = h.shape[0]
    k = rd(project(w, p + "k", h)).reshape(n, m["kv_heads"], m["dim"])
    v = rd(project(w, p + "v", h)).reshape(n, m["kv_heads"], m["vdim"])
    rot = m.get("rot")
    if rot is not None and rot.get("dims", 0) > 0:
        k = turn_halves(k, torch.arange(n), rot["dims"], rot["base"])
    return rd(k), v


def attention_mixer(
    w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, rounded: bool = False,
) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    n = h.shape[0]
    heads, groups = m["heads"], m["kv_heads"]
    q = rd(project(w, p + "q", h)).reshape(n, heads, m["dim"])
    rot = m.get("rot")
    if rot is not None and rot.get("dims", 0) > 0:
        q = rd(turn_halves(q, torch.arange(n), rot["dims"], rot["base"]))
    per = heads // groups
    scores = torch.stack([(q[:, hh] @ keys[:, hh // per].T) * m["scale"] for hh in range(heads)])
    size = (m.get("mask") or {}).get("size")
    weights = sink_softmax(scores, sliding_visible(n, size), w.get(p + "sink"))
    weights = mix_heads(weights, w.get(p + "talk"))
    out = torch.cat([weights[hh] @ values[:, hh // per] for hh in range(heads)], dim=-1)
    return project(w, p + "o", rd(out))


def gla_decay(w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    z = rd(h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    return torch.sigmoid(z) ** (1.0 / m["tau"])


def gla_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor, state: Optional[torch.Tensor] = None):
    """q, k, alpha [T, H, d], v [T, H, e]; S [H, d, e].  Returns (o [T, H, e], the last state)."""
    n, heads, d = q.shape
    e = v.shape[-1]
    S = torch.zeros(heads, d, e, dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(n, heads, e, dtype=q.dtype)
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out, S


def gla_mixer(w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, eps: float, rounded: bool = False) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    n = h.shape[0]
    heads, d, e = m["heads"], m["dim"], m["vdim"]
    q = rd(h @ w[p + "q"].T).reshape(n, heads, d) * d ** -0.5
    k = rd(h @ w[p + "k"].T).reshape(n, heads, d)
    v = rd(h @ w[p + "v"].T).reshape(n, heads, e)
    alpha = gla_decay(w, p, m, h, rounded).reshape(n, heads, d)
    o, _ = gla_recurrence(q, k, v, alpha)
    o = unit_rms(o, eps) * w[p + "norm"]
    gate = silu(rd(h @ w[p + "g"].T))
    return rd(o.reshape(n, heads * e) * gate) @ w[p + "o"].T


def dense_ff(w: Dict[str, torch.Tensor], p: str, limit: float, h: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return rd(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def gated_expert(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    return rd(silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(logits: torch.Tensor, top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """logits [T, E] -> (chosen [T, top], weights [T, top]): the largest logits, softmax over those alone."""
    values, chosen = torch.topk(logits, top, dim=-1)
    return chosen, torch.softmax(values, dim=-1)


def router_logits(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return h @ w[p + "router"].T + w[p + "router.b"]


def route_margin(logits: torch.Tensor, top: int) -> torch.Tensor:
    """How far, as a share of the largest logit's size, the last chosen logit lies above the first one left out: a
    change of the logits by less cannot turn the choice (infinite where every expert is chosen)."""
    if top >= logits.shape[-1]:
        return torch.full(logits.shape[:-1], float("inf"), dtype=logits.dtype)
    values = torch.sort(logits, dim=-1, descending=True).values
    return (values[..., top - 1] - values[..., top]) / logits.abs().max(dim=-1).values.clamp_min(1e-30)


def expert_ff(w: Dict[str, torch.Tensor], p: str, mlp: dict, h: torch.Tensor, rounded: bool = False, margins: Optional[list] = None) -> torch.Tensor:
    logits = router_logits(w, p, h)
    if margins is not None:
        margins.append(route_margin(logits, mlp["router"]["top"]))
    chosen, weights = route(logits, mlp["router"]["top"])
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, c in zip(chosen[t].tolist(), weights[t]):
            out[t] += c * gated_expert(w, f"{p}e{e}.", h[t : t + 1], rounded)[0]
    if mlp.get("shared") is not None:
        share = torch.sigmoid(h @ w[p + "shared.sg"].T)  # [T, 1]
        out = out + share * gated_expert(w, p + "shared.", h, rounded)
    return out


def feed_forward(w: Dict[str, torch.Tensor], p: str, mlp: dict, h: torch.Tensor, rounded: bool = False, margins: Optional[list] = None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return dense_ff(w, p, mlp["limit"], h, rounded)
    if mlp["kind"] == "moe":
        return expert_ff(w, p, mlp, h, rounded, margins)
    raise ValueError(mlp["kind"])


def token_side(w: Dict[str, torch.Tensor], p: str, x: torch.Tensor, rows: torch.Tensor, eps: float, rounded: bool = False) -> torch.Tensor:
    """rows [T, dim]: this layer's part of the tokens' side embedding.  Returns what is added to x."""
    rd = bf16_round if rounded else (lambda t: t)
    g = gelu_tanh(rd(x) @ w[p + "gate"].T) * rows
    y = rd(g) @ w[p + "proj"].T
    return unit_rms(y, eps) * w[p + "norm"]


def forward(
    config: dict, w: Dict[str, torch.Tensor], tokens: List[int], rounded: bool = False, layers_out: Optional[list] = None,
    margins: Optional[list] = None,
) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `rounded`: inputs of matrix products are rounded to bfloat16 where
    an engine that stores activations in bfloat16 would.  `layers_out` receives the residual after every layer,
    `margins` every router's margins [T] (see `route_margin`)."""
    rd = bf16_round if rounded else (lambda t: t)
    eps = config["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    x = w["embed"][tok] * config.get("embedding", {}).get("scale", 1.0)
    side = config.get("token_side")
    canon = config.get("canon")
    cached: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = rd(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps))
        a, b = h, h
        if canon is not None:
            a = rd(h + causal_conv(h, w[p + "canon1"]))
            if layer.get("mlp") is not None:
                b = rd(h + causal_conv(h, w[p + "canon2"]))
        m = layer["mixer"]
        kind = layer["type"].split("_")[0]  # a numeric suffix marks another set of sizes of the same mixer
        if kind == "attention":
            if m.get("kv_from") is not None:
                keys, values = cached[m["kv_from"]]
            else:
                keys, values = attention_keys_values(w, p + "mix.", m, a, rounded)
                cached[i] = (keys, values)
            mixed = attention_mixer(w, p + "mix.", m, a, keys, values, rounded)
        elif kind == "gla":
            mixed = gla_mixer(w, p + "mix.", m, a, eps, rounded)
        else:
            raise ValueError(layer["type"])
        ff = feed_forward(w, p + "mlp.", layer["mlp"], b, rounded, margins) if layer.get("mlp") is not None else 0.0
        x = x + (mixed + ff)
        if side is not None:
            dim = side["dim"]
            rows = w["side.embed"][tok][:, i * dim : (i + 1) * dim]
            x = x + token_side(w, p + "side.", x, rows, eps, rounded)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rd(layer_norm(x, w["final.norm"], w["final.norm.b"], eps))
    return x @ w["head"].T
