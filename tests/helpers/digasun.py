"""Small configurations of the Digasun architecture with weights drawn so that every mechanism matters, the writer of
their model folders, and the plain implementation's logits for them.

Sizes differ wherever two could be equal (query and key/value heads, query/key and value head sizes, the rotated part
of a head, windows, the heads of the two kinds of mixer, taps, experts and how many are chosen), layers come in every
order, with and without a feed-forward, with and without a shared expert, and layers that read another layer's keys
and values do so through a window of their own."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch

from helpers import lapevik  # the same limits: float32 sums in another order; what bfloat16 storage costs
from plain import digasun_plain


def attention(heads, kv_heads, dim, vdim, scale, mask=None, rot=None, kv_from=None, mlp=None, kind="attention") -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if mask is not None:
        mixer["mask"] = {"size": mask}
    if rot is not None:  # (base, dims)
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def gla(heads, dim, vdim, tau, mlp=None, kind="gla") -> dict:
    return {"type": kind, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def dense(ff: int, limit: float) -> dict:
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts: int, top: int, ff: int, shared: Optional[int] = None) -> dict:
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def model_of(layers, width=40, vocab=83, eps=1e-5, scale=None, taps=3, side=4) -> dict:
    config = {"architecture": "Digasun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}
    if scale is not None:
        config["embedding"] = {"scale": scale}
    if taps is not None:
        config["canon"] = {"taps": taps}
    if side is not None:
        config["token_side"] = {"dim": side}
    return config


# heads of 12 and 20 share a cached head of 32; a layer reads the first layer's keys and values with more query heads and
# through a longer window than the layer that made them; all of three experts chosen; a layer without a feed-forward;
# a window of one key; a whole head rotated
TINY_G = model_of(
    [
        attention(4, 2, 12, 20, 0.3, mask=9, rot=(100.0, 8), mlp=dense(56, 1.5)),
        gla(3, 10, 14, 8.0, mlp=moe(5, 2, 24, shared=16)),
        attention(6, 2, 12, 20, 0.25, mask=13, rot=(100.0, 8), kv_from=0, mlp=moe(3, 3, 20)),
        attention(3, 3, 8, 8, 0.4, mask=1, rot=(1000.0, 8)),
        attention(3, 3, 8, 8, 0.4, mask=5, rot=(1000.0, 8), kv_from=3, mlp=dense(24, 0.8), kind="attention_2"),
    ],
    width=48, vocab=131, eps=1e-5, scale=2.5, taps=3, side=6,
)
# sharp: large scales, so that single keys, also those at a window's edge, decide a token; one head a mixer; a state
# that forgets fast and one that forgets slowly; two taps; two side values; one expert of seven; no scale on the embedding
TINY_H = model_of(
    [
        gla(1, 17, 5, 1.0, mlp=moe(7, 1, 12, shared=9)),
        attention(2, 1, 16, 8, 2.0, mask=11, rot=(300.0, 16), mlp=dense(30, 3.0)),
        attention(1, 1, 24, 8, 3.0, mask=16),
        gla(4, 6, 33, 64.0, mlp=dense(20, 1.0), kind="gla_7"),
        attention(4, 2, 10, 6, 1.5, mask=32, rot=(50.0, 2), mlp=moe(4, 2, 12)),
        attention(2, 2, 10, 6, 1.0, mask=7, rot=(50.0, 2), kv_from=4, mlp=moe(2, 1, 8, shared=8)),
    ],
    width=40, vocab=97, eps=1e-6, scale=None, taps=2, side=2,
)
# heads of 80; windows of two pages and more; four taps; a state whose rows are shared by two lanes; every layer but
# the first reads the first layer's keys and values
TINY_I = model_of(
    [
        attention(2, 1, 80, 48, 0.11, mask=50, rot=(10000.0, 40), mlp=dense(96, 2.0)),
        attention(4, 1, 80, 48, 0.11, mask=40, rot=(10000.0, 40), kv_from=0, mlp=moe(6, 3, 32, shared=40)),
        gla(2, 40, 24, 12.0, mlp=moe(6, 4, 16)),
        attention(1, 1, 80, 48, 0.15, mask=64, rot=(10000.0, 40), kv_from=0, mlp=dense(64, 2.5)),
    ],
    width=64, vocab=211, eps=1e-5, scale=0.5, taps=4, side=9,
)
# wider, so that prompts of some hundred tokens take the kernels' shapes for many rows
MEDIUM = model_of(
    [
        attention(8, 2, 64, 64, 0.125, mask=100, rot=(10000.0, 32), mlp=dense(512, 3.0)),
        gla(4, 64, 32, 8.0, mlp=moe(8, 2, 128, shared=128)),
        attention(8, 2, 64, 64, 0.125, mask=257, rot=(10000.0, 32), kv_from=0, mlp=moe(6, 3, 80)),
        attention(4, 4, 128, 64, 0.09, mask=300, rot=(500000.0, 64), mlp=dense(384, 1.5)),
    ],
    width=256, vocab=320, eps=1e-5, scale=1.5, taps=4, side=12,
)

ALL = {"tiny_g": TINY_G, "tiny_h": TINY_H, "tiny_i": TINY_I}


def get(name: str) -> dict:
    return copy.deepcopy(ALL[name])


def layer_kind(layer: dict) -> str:
    return layer["type"].split("_")[0]


def draw_weights(config: dict, seed: int, decay_rank: int = 5) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by name.  Matrices N(0, 1 / fan-in); norm weights around one with biases that are not small;
    sinks of the size of a score; mixing matrices of the heads that are far from the identity; convolutions whose taps
    count as much as the input itself; decays between nearly none and fast; routers whose logits lie well apart."""
    gen = torch.Generator().manual_seed(seed)
    normal = lambda *shape, std=1.0: torch.randn(*shape, generator=gen) * std  # noqa: E731
    uniform = lambda lo, hi, *shape: torch.rand(*shape, generator=gen) * (hi - lo) + lo  # noqa: E731
    matrix = lambda out, inp: normal(out, inp, std=inp ** -0.5)  # noqa: E731
    width, vocab, n_layers = config["width"], config["vocab"], len(config["layers"])
    w = {"embed": normal(vocab, width, std=0.7), "head": matrix(vocab, width) * 2.0, "final.norm": uniform(0.5, 1.5, width), "final.norm.b": normal(width, std=0.2)}
    side = (config.get("token_side") or {}).get("dim")
    if side:
        w["side.embed"] = normal(vocab, n_layers * side)
    taps = (config.get("canon") or {}).get("taps")

    def expert(p: str, ff: int) -> None:
        w[p + "gate"], w[p + "up"], w[p + "down"] = matrix(ff, width) * 1.5, matrix(ff, width) * 1.5, matrix(width, ff)

    for i, layer in enumerate(config["layers"]):
        m, p, mlp = layer["mixer"], f"l{i}.", layer["mlp"]
        w[p + "norm1"], w[p + "norm1.b"] = uniform(0.5, 1.5, width), normal(width, std=0.2)
        if taps:
            w[p + "canon1"] = normal(width, taps, std=0.5)
            if mlp is not None:
                w[p + "canon2"] = normal(width, taps, std=0.5)
        q = p + "mix."
        if layer_kind(layer) == "attention":
            heads = m["heads"]
            q_out, k_out, v_out = heads * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            w[q + "q"], w[q + "q.b"] = matrix(q_out, width), normal(q_out, std=0.3)
            if m.get("kv_from") is None:
                w[q + "k"], w[q + "v"] = matrix(k_out, width), matrix(v_out, width)
                w[q + "k.b"], w[q + "v.b"] = normal(k_out, std=0.3), normal(v_out, std=0.3)
            w[q + "o"], w[q + "o.b"] = matrix(width, heads * m["vdim"]), normal(width, std=0.3)
            w[q + "sink"] = normal(heads, std=1.0)
            w[q + "talk"] = 0.6 * torch.eye(heads) + normal(heads, heads, std=0.4)
        else:
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            w[q + "q"], w[q + "k"], w[q + "v"], w[q + "g"] = matrix(qk, width) * 2.0, matrix(qk, width), matrix(vv, width), matrix(vv, width) * 2.0
            w[q + "o"], w[q + "norm"] = matrix(width, vv), uniform(0.5, 1.5, m["vdim"])
            w[q + "a1"], w[q + "a2"], w[q + "a2.b"] = matrix(decay_rank, width), matrix(qk, decay_rank) * 2.0, uniform(-1.0, 4.0, qk)
        if mlp is not None and mlp["kind"] == "dense":
            expert(p + "mlp.", mlp["ff"])
        elif mlp is not None:
            experts = mlp["router"]["experts"]
            w[p + "mlp.router"], w[p + "mlp.router.b"] = normal(experts, width, std=0.5), normal(experts, std=0.5)
            for e in range(experts):
                expert(p + f"mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared") is not None:
                expert(p + "mlp.shared.", mlp["shared"]["ff"])
                w[p + "mlp.shared.sg"] = matrix(1, width) * 2.0
        if side:
            w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"] = matrix(side, width) * 2.0, matrix(width, side), uniform(0.3, 1.0, width)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def make_folder(root, name: str, seed: int = 1, config: Optional[dict] = None, weights: Optional[Dict[str, torch.Tensor]] = None) -> str:
    from safetensors.torch import save_file

    config = config or get(name)
    folder = os.path.join(str(root), f"{name}_{seed}")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh)
    save_file(weights if weights is not None else draw_weights(config, seed), os.path.join(folder, "model.safetensors"))
    return folder


def read_folder(folder: str):
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    return config, {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# A router's choice between two experts is not compared in bfloat16 where a change of the router's logits by this share
# of their size could turn it: what reaches a router in bfloat16 differs from the exact input by about a hundredth
# after a few layers, and whichever of the two experts an implementation then takes is right.  Such tokens are left
# out of the bfloat16 comparison, and in a model with a recurrent layer every token after them, since the state carries the
# other expert's result along; the float32 comparison leaves none out.
CLOSE_CALL = 0.05
MOST_CLOSE_CALLS = 0.5
LOOSE_FACTOR = 50.0  # float32 sums in another order, as a multiple of a change of the weights by 1e-7 of themselves


class Expected(lapevik.Expected):
    """Exact logits, what bfloat16 storage alone costs, the tokens whose routers made no close call, and, for float32
    runs that ask for it, how far every position's logits move when all weights change in their last float32 bits."""

    def __init__(self, exact: np.ndarray, rounded: Optional[np.ndarray], margins: np.ndarray, loose: Optional[np.ndarray] = None, carried: bool = False) -> None:
        self.clear = margins >= CLOSE_CALL
        self.carried = carried
        if carried:
            # a state that is carried from token to token takes a turned choice along: what comes after a close call
            # is not compared either
            self.clear = np.logical_and.accumulate(self.clear)
        if self.clear.any():
            super().__init__(exact[self.clear], rounded[self.clear] if rounded is not None else None)
        self.exact = exact
        self.loose = loose


def expected(folder: str, requests: Dict[str, List[int]], dtype: str, conditioning: bool = False, drop_after_close_calls: bool = False) -> Dict[str, Expected]:
    """`drop_after_close_calls`: in a model with a recurrent layer, also leave out of the bfloat16 comparison every token
    after a router's close call (for configurations that are drawn, whose routers nobody has looked at)."""
    config, weights = read_folder(folder)
    gen = torch.Generator().manual_seed(1)
    out = {}
    for rid, toks in requests.items():
        margins: list = []
        exact64 = digasun_plain.forward(config, weights, toks, margins=margins)
        least = torch.stack(margins).min(0).values.numpy() if margins else np.full(len(toks), np.inf)
        exact = exact64.to(torch.float32).numpy()
        rounded = loose = None
        if dtype == "bfloat16":
            rounded = digasun_plain.forward(config, weights, toks, rounded=True).to(torch.float32).numpy()
        elif conditioning:
            shaken = [{k: v * (1.0 + 1e-7 * torch.randn(v.shape, generator=gen, dtype=torch.float64)) for k, v in weights.items()} for _ in range(2)]
            loose = np.maximum(*[(digasun_plain.forward(config, s, toks) - exact64).abs().max(dim=1).values.numpy() for s in shaken])
        carried = drop_after_close_calls and any(layer_kind(layer) == "gla" for layer in config["layers"]) and bool(margins)
        out[rid] = Expected(exact, rounded, least, loose, carried=carried)
    return out


def check(got: np.ndarray, want: Expected, dtype: str, what: str) -> None:
    assert got.shape == want.exact.shape, f"{what}: logits {got.shape}, expected {want.exact.shape}"
    assert not np.isnan(got).any(), f"{what}: missing or NaN logits"
    if dtype == "float32":
        err = np.abs(got.astype(np.float64) - want.exact.astype(np.float64)).max(axis=1)
        limit = lapevik.FLOAT32_LIMIT * float(np.abs(want.exact).max()) + (LOOSE_FACTOR * want.loose if want.loose is not None else 0.0) + 0.0 * err
        over = err - limit
        assert over.max() <= 0, f"{what}: first position over its limit {int(np.argmax(over > 0))}, error {err[np.argmax(over)]:.3e} vs {limit[np.argmax(over)]:.3e}"
        return
    if not want.carried:
        assert (~want.clear).sum() <= max(2, MOST_CLOSE_CALLS * want.clear.size), f"{what}: too many close calls for a comparison in bfloat16"
    if not want.clear.any():
        return
    clear = lapevik.Expected.__new__(lapevik.Expected)
    clear.exact, clear.rms, clear.max = want.exact[want.clear], want.rms, want.max
    lapevik.check(got[want.clear], clear, dtype, what + " (tokens without a close call of a router)")


def check_together(got: Dict[str, np.ndarray], want: Dict[str, Expected], dtype: str, what: str) -> None:
    """Every request on its own in float32; in bfloat16 all requests of a model as one, since what bfloat16 storage costs
    is itself a draw, and a request of a few tokens is a small sample of it."""
    if dtype != "bfloat16":
        for rid in want:
            check(got[rid], want[rid], dtype, f"{what} {rid}")
        return
    rids = [r for r in want if want[r].clear.any()]
    if not rids:
        return
    sizes = np.array([want[r].exact[want[r].clear].size for r in rids], dtype=np.float64)
    pooled = lapevik.Expected.__new__(lapevik.Expected)
    pooled.exact = np.concatenate([want[r].exact[want[r].clear] for r in rids])
    pooled.rms = float(np.sqrt((sizes * np.array([want[r].rms for r in rids]) ** 2).sum() / sizes.sum()))
    pooled.max = max(want[r].max for r in rids)
    lapevik.check(np.concatenate([got[r][want[r].clear] for r in rids]), pooled, dtype, what)


def plain_greedy(folder: str, prompt: List[int], n_new: int) -> List[int]:
    config, weights = read_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n_new):
        out.append(int(torch.argmax(digasun_plain.forward(config, weights, toks)[-1])))
        toks.append(out[-1])
    return out
