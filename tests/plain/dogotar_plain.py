"""The Dogotar decoder, written plainly: whole sequences, no cache, float64, one function per mechanism.
Nothing here is imported from the product; the product is compared with this.

Notation: T tokens, D the model's width.  A model is a dictionary `config` (as config.json holds it) and a
dictionary `w` of float64 tensors by the folder's names.

    x_0        = E[token]
    layer:       x <- x + mixer(ln1(x)) + ff(ln2(x))                  both sublayers read the same x
    ln(v)      = (v - mean) / sqrt(var + eps) * g + b                 var: mean squared deviation
    attention:   q, k, v = W h + bias;  q, k <- rms per head * weight;  the first `rot.dims` of a head turned in
                 pairs (i, i + dims/2) by p * base^(-2i/dims) / factor;  s = cap tanh(scale q.k / cap);
                 softmax over the keys j with 0 <= i - j < window;  v <- (1 - lam) v + lam v_first in all v_mix layers
                 but the first;  out = W_o (heads * sigmoid(W_g h))
    parallel:    a_l left(h) + a_r right(h);  left: attention without rotation whose query i reads the keys j <= i
                 of its own block of `mask.size` positions;  right: a matrix memory per head (see `matrix_memory`)
    ff:          W_down gelu_tanh(W_up h)
    logits     = E ln_final(x)
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


def turn_halves(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, factor: float) -> torch.Tensor:
    """x [T, H, d]: element i < dims/2 of every head is paired with element i + dims/2; the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=F)
    freq = base ** (-2.0 * i / dims) / factor
    a = positions.to(F)[:, None] * freq[None, :]  # [T, half]
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


def block_visible(n: int, size: Optional[int]) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if size is not None:
        ok = ok & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))
    return ok


def capped_softmax_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: Optional[float], visible: torch.Tensor
) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H * e]; query head h reads key/value head h // (H / G)."""
    n, heads, _ = q.shape
    per = heads // k.shape[1]
    out = []
    for h in range(heads):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~visible, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, g])
    return torch.cat(out, dim=-1)


def project_heads(w: Dict[str, torch.Tensor], name: str, h: torch.Tensor, heads: int) -> torch.Tensor:
    y = h @ w[name].T
    if name + ".b" in w:
        y = y + w[name + ".b"]
    return y.reshape(h.shape[0], heads, -1)


def softmax_attention_mixer(
    w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, eps: float, visible: torch.Tensor,
    v_first: Optional[torch.Tensor] = None, rounded: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (output [T, D], the values this layer used [T, G, e])."""
    n = h.shape[0]
    rd = bf16_round if rounded else (lambda t: t)
    q = rd(project_heads(w, p + "q", h, m["heads"]))
    k = rd(project_heads(w, p + "k", h, m["kv_heads"]))
    v = rd(project_heads(w, p + "v", h, m["kv_heads"]))
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    rot = m.get("rot")
    if rot is not None and rot.get("dims", 0) > 0:
        factor = (rot.get("scaling") or {}).get("factor", 1.0)
        pos = torch.arange(n)
        q = turn_halves(q, pos, rot["dims"], rot["base"], factor)
        k = turn_halves(k, pos, rot["dims"], rot["base"], factor)
    if m.get("v_mix") and v_first is not None:
        lam = w[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    q, k, v = rd(q), rd(k), rd(v)
    mixed = rd(capped_softmax_attention(q, k, v, m["scale"], m.get("softcap"), visible))
    if p + "g" in w:
        mixed = rd(mixed * torch.sigmoid(rd(h @ w[p + "g"].T)))
    return rd(mixed @ w[p + "o"].T), v


def memory_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gi: torch.Tensor, gf: torch.Tensor) -> torch.Tensor:
    """q (already scaled), k [T, H, d], v [T, H, e], log input and forget gates gi, gf [T, H].  Per head, with S [d, e],
    n [d] and a running maximum r, all zero before the first token:
        r_t = max(f_t + r_(t-1), i_t)
        S_t = exp(f_t + r_(t-1) - r_t) S_(t-1) + exp(i_t - r_t) k_t v_t^T,   n_t likewise with k_t
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-r_t)) + 1e-6)
    Returns o [T, H, e]."""
    T, H, d = k.shape
    e = v.shape[2]
    out = torch.zeros(T, H, e, dtype=F)
    for a in range(H):
        S = torch.zeros(d, e, dtype=F)
        nrm = torch.zeros(d, dtype=F)
        r = 0.0
        for t in range(T):
            r_new = max(float(gf[t, a]) + r, float(gi[t, a]))
            keep = math.exp(float(gf[t, a]) + r - r_new)
            take = math.exp(float(gi[t, a]) - r_new)
            S = keep * S + take * torch.outer(k[t, a], v[t, a])
            nrm = keep * nrm + take * k[t, a]
            r = r_new
            den = max(abs(float(nrm @ q[t, a])), math.exp(-r)) + 1e-6
            out[t, a] = (S.T @ q[t, a]) / den
    return out


def capped_log_gates(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor, c: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """i = c tanh((W_i h + b_i) / c),  f = logsigmoid(c tanh((W_f h + b_f) / c)), [T, H] each."""
    gi = c * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / c)
    gf = torch.nn.functional.logsigmoid(c * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / c))
    return gi, gf


def matrix_memory(
    w: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, eps: float, rounded: bool = False
) -> torch.Tensor:
    """q = W_q h / sqrt(d), k = W_k h, v = W_v h and capped log gates enter `memory_recurrence`; then every head's o
    over its root mean square, all heads times the weight, times sigmoid(W_g h), then W_o."""
    T = h.shape[0]
    H, d, e, c = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    rd = bf16_round if rounded else (lambda t: t)
    q = rd(h @ w[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = rd(h @ w[p + "k"].T).reshape(T, H, d)
    v = rd(h @ w[p + "v"].T).reshape(T, H, e)
    gi, gf = capped_log_gates(w, p, h, c)
    out = memory_recurrence(q, k, v, gi, gf)
    y = unit_rms(out, eps).reshape(T, H * e) * w[p + "norm"]
    y = rd(y * torch.sigmoid(rd(h @ w[p + "g"].T)))
    return rd(y @ w[p + "o"].T)


def dense_ff(w: Dict[str, torch.Tensor], p: str, h: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    rd = bf16_round if rounded else (lambda t: t)
    return rd(rd(gelu_tanh(h @ w[p + "up"].T)) @ w[p + "down"].T)


def forward(config: dict, w: Dict[str, torch.Tensor], tokens: List[int], rounded: bool = False, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `rounded`: round to bfloat16 where an engine that keeps
    activations in bfloat16 stores them (products' results, cached rows, the sublayers' inputs)."""
    eps = config["norm"]["eps"]
    rd = bf16_round if rounded else (lambda t: t)
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)].clone()
    n = x.shape[0]
    v_first = None
    for li, layer in enumerate(config["layers"]):
        p = f"l{li}."
        m = layer["mixer"]
        h1 = rd(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps))
        kind = layer["type"].rsplit("_", 1)[0] if layer["type"].rsplit("_", 1)[-1].isdigit() else layer["type"]  # "_<number>": other sizes
        if kind == "attention":
            size = (m.get("mask") or {}).get("size")
            y, v_used = softmax_attention_mixer(w, p + "mix.", m, h1, eps, sliding_visible(n, size), v_first, rounded)
            if m.get("v_mix") and v_first is None:
                v_first = v_used
        elif kind == "parallel":
            lm = m["left"]
            size = (lm.get("mask") or {}).get("size")
            left, _ = softmax_attention_mixer(w, p + "mix.left.", lm, h1, eps, block_visible(n, size), None, rounded)
            right = matrix_memory(w, p + "mix.right.", m["right"], h1, eps, rounded)
            y = m.get("left_scale", 1.0) * left + m.get("right_scale", 1.0) * right
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            h2 = rd(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps))
            y = y + dense_ff(w, p + "mlp.", h2, rounded)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    xf = rd(layer_norm(x, w["final.norm"], w["final.norm.b"], eps))
    return xf @ w["embed"].T
