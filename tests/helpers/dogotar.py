"""Small configurations of the Dogotar architecture with weights drawn so that every mechanism matters, the writer of
their model folders, and the plain implementation's logits for them.

Sizes differ wherever two could be equal (query and key/value heads, query/key and value head sizes, the rotated part
of a head, windows and blocks, the two mixers of a parallel layer), layers come in every order, with and without a
feed-forward, with and without rotation, cap, mask and blended values."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch

from helpers import lapevik  # the same limits: float32 sums in another order; what bfloat16 storage costs
from plain import dogotar_plain


def attn_sizes(heads, kv_heads, dim, vdim, scale, softcap=None, mask=None, rot=None, v_mix=None) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        mixer["softcap"] = softcap
    if mask is not None:
        mixer["mask"] = {"size": mask}
    if rot is not None:  # (base, dims) or (base, dims, factor)
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
        if len(rot) > 2:
            mixer["rot"]["scaling"] = {"factor": rot[2]}
    if v_mix is not None:
        mixer["v_mix"] = v_mix
    return mixer


def attention(*args, mlp=None, kind="attention", **kwargs) -> dict:
    return {"type": kind, "mixer": attn_sizes(*args, **kwargs), "mlp": mlp}


def parallel(left: dict, heads, dim, vdim, gate_cap, left_scale=None, right_scale=None, mlp=None, kind="parallel") -> dict:
    mixer = {"left": left, "right": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}}
    if left_scale is not None:
        mixer["left_scale"] = left_scale
    if right_scale is not None:
        mixer["right_scale"] = right_scale
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def dense(ff: int) -> dict:
    return {"kind": "dense", "ff": ff}


# a parallel layer first; values blended over three later attention layers whose query heads and windows differ;
# heads of 12 and 20 share a cached head of 32; a layer without a feed-forward; a layer with no rotation, mask or cap
TINY_D = {
    "architecture": "Dogotar", "vocab": 131, "width": 48, "norm": {"eps": 1e-5},
    "layers": [
        parallel(attn_sizes(4, 2, 12, 20, 0.3, softcap=5.0, mask=7), 3, 10, 14, 4.0, 0.7, 1.3, mlp=dense(56)),
        attention(6, 2, 16, 8, 0.25, softcap=8.0, mask=9, rot=(100.0, 8, 2.0), v_mix=True),
        attention(2, 2, 20, 8, 0.2, mask=33, rot=(1000.0, 20), v_mix=True, mlp=dense(40)),
        attention(3, 3, 8, 24, 0.4, softcap=3.0, v_mix=False, mlp=dense(24), kind="attention_2"),
        attention(6, 2, 16, 8, 0.25, softcap=8.0, mask=9, rot=(100.0, 8, 2.0), v_mix=True, mlp=dense(30)),
    ],
}
# sharp: large scales and wide caps, so that single keys, also those at a window's or a block's edge, decide a token,
# and a memory that forgets slowly; one head a mixer; a block of a page, a block of one position, a window of one key
TINY_E = {
    "architecture": "Dogotar", "vocab": 97, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        attention(2, 1, 16, 8, 2.0, softcap=30.0, mask=11, rot=(300.0, 16, 1.5), v_mix=True, mlp=dense(30)),
        parallel(attn_sizes(1, 1, 24, 8, 3.0, softcap=40.0, mask=16), 1, 17, 5, 9.0, mlp=None),
        parallel(attn_sizes(5, 5, 8, 8, 1.5, mask=1), 2, 6, 33, 2.0, 1.0, 0.5, mlp=dense(20), kind="parallel_7"),
        attention(4, 2, 10, 6, 1.0, softcap=25.0, mask=1, mlp=dense(12)),
        parallel(attn_sizes(2, 2, 16, 16, 2.5, softcap=50.0), 4, 20, 12, 30.0, 1.5, 1.0, mlp=dense(36)),
    ],
}
# heads of 80; blocks and windows of two pages and more; only parallel layers but the last
TINY_F = {
    "architecture": "Dogotar", "vocab": 211, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        parallel(attn_sizes(2, 1, 80, 48, 0.11, softcap=12.0, mask=50), 2, 32, 32, 8.0, 1.1, 0.9, mlp=dense(96)),
        parallel(attn_sizes(8, 2, 16, 32, 0.25, mask=32), 5, 12, 20, 6.0, mlp=dense(64)),
        attention(4, 4, 32, 16, 0.18, softcap=15.0, mask=40, rot=(10000.0, 16, 8.0), v_mix=True, mlp=dense(72)),
    ],
}
# wider, so that prompts of some hundred tokens take the kernels' shapes for many rows
MEDIUM = {
    "architecture": "Dogotar", "vocab": 320, "width": 256, "norm": {"eps": 1e-6},
    "layers": [
        attention(8, 2, 64, 64, 0.125, softcap=20.0, mask=100, rot=(10000.0, 32, 4.0), v_mix=True, mlp=dense(512)),
        parallel(attn_sizes(4, 4, 32, 64, 0.18, softcap=10.0, mask=128), 4, 64, 32, 10.0, 1.2, 0.8, mlp=dense(384)),
        attention(4, 2, 128, 64, 0.09, softcap=20.0, mask=257, rot=(500000.0, 64), v_mix=True, mlp=dense(256)),
    ],
}

ALL = {"tiny_d": TINY_D, "tiny_e": TINY_E, "tiny_f": TINY_F}


def get(name: str) -> dict:
    return copy.deepcopy(ALL[name])


def layer_kind(layer: dict) -> str:
    return layer["type"].split("_")[0]


def draw_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by name.  Matrices N(0, 1 / fan-in); norm weights around one with biases that are not small;
    query and key norms large enough for scores to reach their cap; blending weights well inside (0, 1); gates whose
    projections reach a small cap, input gates around zero and forget gates that keep most of the state."""
    gen = torch.Generator().manual_seed(seed)
    normal = lambda *shape, std=1.0: torch.randn(*shape, generator=gen) * std  # noqa: E731
    uniform = lambda lo, hi, *shape: torch.rand(*shape, generator=gen) * (hi - lo) + lo  # noqa: E731
    matrix = lambda out, inp: normal(out, inp, std=inp ** -0.5)  # noqa: E731
    width, vocab = config["width"], config["vocab"]
    w = {"embed": normal(vocab, width, std=0.7), "final.norm": uniform(0.5, 1.5, width), "final.norm.b": normal(width, std=0.2)}

    def attention_tensors(p: str, m: dict, gate: bool) -> None:
        q_out, k_out, v_out = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
        w[p + "q"], w[p + "k"], w[p + "v"] = matrix(q_out, width), matrix(k_out, width), matrix(v_out, width)
        w[p + "q.b"], w[p + "k.b"], w[p + "v.b"] = normal(q_out, std=0.3), normal(k_out, std=0.3), normal(v_out, std=0.3)
        w[p + "q.norm"], w[p + "k.norm"] = uniform(1.0, 2.5, m["dim"]), uniform(1.0, 2.5, m["dim"])
        w[p + "o"] = matrix(width, m["heads"] * m["vdim"])
        if gate:
            w[p + "g"] = matrix(m["heads"] * m["vdim"], width) * 2.0
        if m.get("v_mix"):
            w[p + "vmix"] = uniform(0.25, 0.75, 1).reshape(())

    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        for q in [1] + ([2] if layer["mlp"] is not None else []):
            w[p + f"norm{q}"] = uniform(0.5, 1.5, width)
            w[p + f"norm{q}.b"] = normal(width, std=0.2)
        if layer_kind(layer) == "attention":
            attention_tensors(p + "mix.", m, gate=True)
        else:
            attention_tensors(p + "mix.left.", m["left"], gate=False)
            r, q = m["right"], p + "mix.right."
            qk, vv = r["heads"] * r["dim"], r["heads"] * r["vdim"]
            w[q + "q"], w[q + "k"], w[q + "v"], w[q + "g"] = matrix(qk, width) * 2.0, matrix(qk, width), matrix(vv, width), matrix(vv, width) * 2.0
            w[q + "o"], w[q + "norm"] = matrix(width, vv), uniform(0.5, 1.5, vv)
            reach = min(0.35 * r["gate_cap"], 2.5)  # small caps are reached; no token outweighs the rest by more than float32 resolves
            w[q + "i"], w[q + "f"] = matrix(r["heads"], width) * reach, matrix(r["heads"], width) * reach
            w[q + "i.b"], w[q + "f.b"] = normal(r["heads"], std=1.0), uniform(1.0, 4.0, r["heads"])
        if layer["mlp"] is not None:
            w[p + "mlp.up"] = matrix(layer["mlp"]["ff"], width) * 1.5
            w[p + "mlp.down"] = matrix(width, layer["mlp"]["ff"])
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


class Expected(lapevik.Expected):
    """Also, for float32 runs that ask for it, how far every position's logits move when all weights change in their last
    float32 bits (`loose`, one value a position): where a normaliser nearly cancels, or a unit norm divides by next
    to nothing, any order of float32 sums moves the result by a multiple of that."""

    def __init__(self, exact: np.ndarray, rounded: Optional[np.ndarray], loose: Optional[np.ndarray] = None) -> None:
        super().__init__(exact, rounded)
        self.loose = loose


def expected(folder: str, requests: Dict[str, List[int]], dtype: str, conditioning: bool = False) -> Dict[str, Expected]:
    config, weights = read_folder(folder)
    gen = torch.Generator().manual_seed(1)
    shaken = [{k: v * (1.0 + 1e-7 * torch.randn(v.shape, generator=gen, dtype=torch.float64)) for k, v in weights.items()} for _ in range(2)]
    out = {}
    for rid, toks in requests.items():
        exact64 = dogotar_plain.forward(config, weights, toks)
        exact = exact64.to(torch.float32).numpy()
        rounded = loose = None
        if dtype == "bfloat16":
            rounded = dogotar_plain.forward(config, weights, toks, rounded=True).to(torch.float32).numpy()
        elif conditioning:
            loose = np.maximum(*[(dogotar_plain.forward(config, w, toks) - exact64).abs().max(dim=1).values.numpy() for w in shaken])
        out[rid] = Expected(exact, rounded, loose)
    return out


LOOSE_FACTOR = 50.0  # float32 sums in another order, as a multiple of a change of the weights by 1e-7 of themselves


def check(got: np.ndarray, want: Expected, dtype: str, what: str) -> None:
    if dtype == "float32" and getattr(want, "loose", None) is not None:
        assert got.shape == want.exact.shape, f"{what}: logits {got.shape}, expected {want.exact.shape}"
        assert not np.isnan(got).any(), f"{what}: missing or NaN logits"
        err = np.abs(got.astype(np.float64) - want.exact.astype(np.float64)).max(axis=1)
        limit = lapevik.FLOAT32_LIMIT * float(np.abs(want.exact).max()) + LOOSE_FACTOR * want.loose
        over = err - limit
        assert over.max() <= 0, f"{what}: first position over its limit {int(np.argmax(over > 0))}, error {err[np.argmax(over)]:.3e} vs {limit[np.argmax(over)]:.3e}"
        assert np.median(limit) < 1e-3 * float(np.abs(want.exact).max()), f"{what}: the case itself hangs on the last bits"
        return
    lapevik.check(got, want, dtype, what)


def check_together(got: Dict[str, np.ndarray], want: Dict[str, Expected], dtype: str, what: str) -> None:
    """Every request on its own in float32; in bfloat16 all requests of a model as one, since what bfloat16 storage costs
    is itself a draw, and a request of a few tokens is a small sample of it."""
    if dtype != "bfloat16":
        for rid in want:
            check(got[rid], want[rid], dtype, f"{what} {rid}")
        return
    rids = list(want)
    sizes = np.array([want[r].exact.size for r in rids], dtype=np.float64)
    pooled = Expected(np.concatenate([want[r].exact for r in rids]), None)
    pooled.rms = float(np.sqrt((sizes * np.array([want[r].rms for r in rids]) ** 2).sum() / sizes.sum()))
    pooled.max = max(want[r].max for r in rids)
    lapevik.check(np.concatenate([got[r] for r in rids]), pooled, dtype, what)


def plain_greedy(folder: str, prompt: List[int], n_new: int) -> List[int]:
    config, weights = read_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n_new):
        out.append(int(torch.argmax(dogotar_plain.forward(config, weights, toks)[-1])))
        toks.append(out[-1])
    return out
