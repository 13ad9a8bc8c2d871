"""Digasun without a GPU: the plain implementation's mechanisms against library routines, invariants and formulas
unrolled by hand; that a mechanism left out or a window one key off would show; the strict configuration and the plan
(tensor names, run order, which caches are shared and which are not, what a shared cache keeps); and everything
around the kernels (descriptor, tables, pages and slots that are used again) with torch in the kernels' place."""

import math

import numpy as np
import pytest
import torch

from helpers import cpu_ops, digasun, traces
from plain import digasun_plain as gp

F = torch.float64


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=F) * scale


# ---- the plain implementation's mechanisms ---------------------------------------------------------------------- #
def test_layer_norm_is_the_library_s():
    x, g, b = rnd((5, 24), 1, 3.0) + 2.0, rnd((24,), 2), rnd((24,), 3)
    torch.testing.assert_close(gp.layer_norm(x, g, b, 1e-5), torch.nn.functional.layer_norm(x, (24,), g, b, 1e-5))


def test_gelu_and_silu_are_the_library_s():
    z = torch.linspace(-6, 6, 101, dtype=F)
    torch.testing.assert_close(gp.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    torch.testing.assert_close(gp.silu(z), torch.nn.functional.silu(z))


def test_convolution_is_the_library_s_with_zeros_before_the_start():
    h, w = rnd((11, 6), 1), rnd((6, 4), 2)
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), w[:, None, :], groups=6)[0].T
    torch.testing.assert_close(gp.causal_conv(h, w), lib)
    # the last tap is the current token's own
    only_last = torch.zeros(6, 4, dtype=F)
    only_last[:, 3] = 2.0
    torch.testing.assert_close(gp.causal_conv(h, only_last), 2.0 * h)


def test_rotation_pairs_halves_of_the_turned_part():
    x = rnd((3, 2, 10), 1)
    pos = torch.tensor([0, 5, 117])
    y = gp.turn_halves(x, pos, 6, 100.0)
    torch.testing.assert_close(y[0], x[0])  # position 0 turns nothing
    torch.testing.assert_close(y[..., 6:], x[..., 6:])  # what lies beyond the turned part passes
    for i in range(3):  # element i with element i + 3, by p * 100^(-2i/6)
        a = 117 * 100.0 ** (-2 * i / 6)
        u, v = x[2, :, i], x[2, :, i + 3]
        torch.testing.assert_close(y[2, :, i], u * math.cos(a) - v * math.sin(a))
        torch.testing.assert_close(y[2, :, i + 3], v * math.cos(a) + u * math.sin(a))
    # a score depends on the distance only
    q, k = rnd((1, 1, 6), 2), rnd((1, 1, 6), 3)
    s = lambda p, r: (gp.turn_halves(q, torch.tensor([p]), 6, 100.0) * gp.turn_halves(k, torch.tensor([r]), 6, 100.0)).sum()  # noqa: E731
    torch.testing.assert_close(s(40, 33), s(1007, 1000))


def test_the_sink_takes_its_share_and_the_heads_mix_afterwards():
    scores = rnd((3, 6, 6), 1)
    visible = gp.sliding_visible(6, 4)
    sink = torch.tensor([0.3, -2.0, 5.0], dtype=F)
    w = gp.sink_softmax(scores, visible, sink)
    assert (w[:, 0, 1:] == 0).all() and (w[:, 5, :2] == 0).all() and (w[:, 5, 2:] > 0).all()
    for h in range(3):
        for i in range(6):
            lo = max(0, i - 3)
            e = torch.exp(scores[h, i, lo : i + 1])
            torch.testing.assert_close(w[h, i, lo : i + 1], e / (e.sum() + math.exp(float(sink[h]))))
    talk = rnd((3, 3), 2)
    mixed = gp.mix_heads(w, talk)
    torch.testing.assert_close(mixed[1], talk[1, 0] * w[0] + talk[1, 1] * w[1] + talk[1, 2] * w[2])
    # rows add up to the mixed shares of what the sinks left
    torch.testing.assert_close(mixed.sum(-1), talk @ w.sum(-1))


def _attention_tensors(width, m, seed=0, own=True):
    w = {"q": rnd((m["heads"] * m["dim"], width), seed + 1, 0.3), "q.b": rnd((m["heads"] * m["dim"],), seed + 2, 0.3),
         "o": rnd((width, m["heads"] * m["vdim"]), seed + 3, 0.3), "o.b": rnd((width,), seed + 4, 0.3),
         "sink": rnd((m["heads"],), seed + 5), "talk": rnd((m["heads"], m["heads"]), seed + 6, 0.5)}
    if own:
        w.update({"k": rnd((m["kv_heads"] * m["dim"], width), seed + 7, 0.3), "k.b": rnd((m["kv_heads"] * m["dim"],), seed + 8, 0.3),
                  "v": rnd((m["kv_heads"] * m["vdim"], width), seed + 9, 0.3), "v.b": rnd((m["kv_heads"] * m["vdim"],), seed + 10, 0.3)})
    return w


def test_attention_is_the_unrolled_formula_for_one_query():
    width = 16
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.37, "mask": {"size": 3}, "rot": {"base": 50.0, "dims": 4}}
    w = _attention_tensors(width, m)
    h = rnd((7, width), 20)
    keys, values = gp.attention_keys_values(w, "", m, h)
    out = gp.attention_mixer(w, "", m, h, keys, values)
    i = 6
    q = gp.turn_halves((h[i : i + 1] @ w["q"].T + w["q.b"]).reshape(1, 4, 6), torch.tensor([i]), 4, 50.0)[0]
    shares = []
    for g in range(4):
        s = torch.stack([(q[g] * keys[j, g // 2]).sum() * 0.37 for j in (4, 5, 6)])
        e = torch.exp(s)
        shares.append(e / (e.sum() + torch.exp(w["sink"][g])))
    heads = []
    for hh in range(4):
        mixed = sum(w["talk"][hh, g] * shares[g] for g in range(4))
        heads.append(sum(mixed[n] * values[j, hh // 2] for n, j in enumerate((4, 5, 6))))
    torch.testing.assert_close(out[i], torch.cat(heads) @ w["o"].T + w["o.b"])


def test_linear_attention_is_its_unrolled_sum():
    n, heads, d, e = 9, 2, 3, 4
    q, k, v = rnd((n, heads, d), 1), rnd((n, heads, d), 2), rnd((n, heads, e), 3)
    alpha = torch.sigmoid(rnd((n, heads, d), 4))
    o, state = gp.gla_recurrence(q, k, v, alpha)
    t = 8
    want = torch.zeros(heads, e, dtype=F)
    for s in range(t + 1):
        decay = torch.prod(alpha[s + 1 : t + 1], dim=0)  # [heads, d]: the decays after s, a key channel each
        want += torch.einsum("hd,hd,he->he", q[t], decay * k[s], v[s])
    torch.testing.assert_close(o[t], want)
    # a portion goes on from the state the one before left
    o1, s1 = gp.gla_recurrence(q[:4], k[:4], v[:4], alpha[:4])
    o2, s2 = gp.gla_recurrence(q[4:], k[4:], v[4:], alpha[4:], state=s1)
    torch.testing.assert_close(torch.cat([o1, o2]), o)
    torch.testing.assert_close(s2, state)


def test_decays_are_a_root_of_the_sigmoid():
    w = {"a1": rnd((3, 8), 1), "a2": rnd((6, 3), 2), "a2.b": rnd((6,), 3)}
    h = rnd((4, 8), 4)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    torch.testing.assert_close(gp.gla_decay(w, "", {"tau": 12.0}, h) ** 12, torch.sigmoid(z))


def test_dense_feed_forward_clamps_before_the_gate():
    w = {"gate": rnd((5, 4), 1, 2.0), "up": rnd((5, 4), 2, 2.0), "down": torch.eye(5, dtype=F)}
    h = rnd((6, 4), 3, 2.0)
    g, u = h @ w["gate"].T, h @ w["up"].T
    assert (g > 1.5).any() and (u.abs() > 1.5).any()
    g, u = g.clamp(max=1.5), u.clamp(-1.5, 1.5)
    torch.testing.assert_close(gp.dense_ff(w, "", 1.5, h), g * torch.sigmoid(1.702 * g) * (u + 1))


def test_router_weights_are_a_softmax_over_the_chosen_and_the_shared_expert_is_gated():
    logits = torch.tensor([[0.1, 2.0, -1.0, 1.5], [3.0, 3.5, 0.0, -2.0]], dtype=F)
    chosen, weights = gp.route(logits, 2)
    assert chosen.tolist() == [[1, 3], [1, 0]]
    torch.testing.assert_close(weights[0], torch.softmax(torch.tensor([2.0, 1.5], dtype=F), 0))
    torch.testing.assert_close(gp.route_margin(logits, 2), torch.tensor([1.4 / 2.0, 3.0 / 3.5], dtype=F))
    width, mlp = 6, {"kind": "moe", "router": {"experts": 3, "top": 1}, "expert": {"ff": 4}, "shared": {"ff": 5}}
    w = {"router": rnd((3, width), 1), "router.b": torch.tensor([0.0, 50.0, 0.0], dtype=F), "shared.sg": rnd((1, width), 2)}
    for name, ff in [("e0.", 4), ("e1.", 4), ("e2.", 4), ("shared.", 5)]:
        w.update({name + "gate": rnd((ff, width), 3), name + "up": rnd((ff, width), 4), name + "down": rnd((width, ff), 5)})
    h = rnd((3, width), 9)
    want = gp.gated_expert(w, "e1.", h) + torch.sigmoid(h @ w["shared.sg"].T) * gp.gated_expert(w, "shared.", h)
    torch.testing.assert_close(gp.expert_ff(w, "", mlp, h), want)  # the bias decides: every token goes to expert 1, weight 1


def test_a_window_one_key_off_a_sink_mixing_a_tap_or_a_lost_state_would_show():
    config = digasun.get("tiny_h")
    w = {k: v.to(F) for k, v in digasun.draw_weights(config, 3).items()}
    toks = traces.random_tokens(5, 60, config["vocab"])
    base = gp.forward(config, w, toks)
    size = float(base.abs().max())

    def moved(change_config=None, change_weights=None):
        c, ww = digasun.get("tiny_h"), dict(w)
        if change_config:
            change_config(c)
        if change_weights:
            change_weights(ww)
        return float((gp.forward(c, ww, toks) - base).abs().max()) / size

    assert moved(lambda c: c["layers"][1]["mixer"]["mask"].update(size=12)) > 1e-2
    assert moved(lambda c: c["layers"][1]["mixer"]["mask"].update(size=10)) > 1e-2
    assert moved(change_weights=lambda ww: ww.update({"l1.mix.sink": ww["l1.mix.sink"] - 30.0})) > 1e-2
    assert moved(change_weights=lambda ww: ww.update({"l1.mix.talk": torch.eye(2, dtype=F)})) > 1e-2
    assert moved(change_weights=lambda ww: ww.update({"l2.canon1": ww["l2.canon1"] * torch.tensor([0.0, 1.0], dtype=F)})) > 1e-2
    assert moved(lambda c: c["layers"][3]["mixer"].update(tau=1.0)) > 1e-2
    assert moved(lambda c: c.pop("token_side")) > 1e-2
    assert moved(lambda c: c["layers"][5]["mixer"].pop("kv_from"), lambda ww: ww.update({"l5.mix.k": ww["l4.mix.k"][:20], "l5.mix.k.b": ww["l4.mix.k.b"][:20], "l5.mix.v": ww["l4.mix.v"], "l5.mix.v.b": ww["l4.mix.v.b"]})) > 1e-3


# ---- configuration and plan --------------------------------------------------------------------------------------- #
def test_config_is_strict_and_the_plan_names_the_folder_s_tensors():
    from cwm_amd.config import ConfigError, parse_config
    from cwm_amd.models.model import Model
    from cwm_amd.parts.base import PagedKVSpec, StateSpec

    for name in digasun.ALL:
        config = digasun.get(name)
        arch, typed = parse_config(config)
        model = Model(arch.build_plan(typed))
        drawn = digasun.draw_weights(config, 1, decay_rank=7)
        specs = model.tensor_specs()
        assert set(n for n, s in specs.items() if not s.optional) == set(drawn)
        for n, t in drawn.items():
            assert specs[n].fits(tuple(t.shape)), n
    bad = digasun.get("tiny_g")
    bad["layers"][0]["mixer"]["softcap"] = 3.0
    with pytest.raises(ConfigError, match="softcap"):
        parse_config(bad)
    for change in (
        lambda c: c["layers"][2]["mixer"].update(kv_from=1),  # not an attention layer
        lambda c: c["layers"][2]["mixer"].update(kv_from=2),  # not an earlier layer
        lambda c: c["layers"][4]["mixer"].update(kv_from=2),  # a layer without keys and values of its own
        lambda c: c["layers"][2]["mixer"].update(dim=16),  # other sizes than the layer it reads
        lambda c: c["layers"][0]["mlp"].pop("limit"),
        lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
        lambda c: c["layers"][1].update(type="mamba"),
    ):
        bad = digasun.get("tiny_g")
        change(bad)
        with pytest.raises(ConfigError):
            parse_config(bad)

    arch, typed = parse_config(digasun.get("tiny_g"))
    model = Model(arch.build_plan(typed))
    # every layer: the convolutions' state, then the mixer's cache; layer 2 reads layer 0's keys and values, layer 4 layer 3's
    assert model.cache_slots == [(0, 1), (2, 3), (4, 1), (5, 6), (7, 6)]
    assert model.writes_cache == [True, True, (True, False), True, (True, False)]
    kv0, kv3 = model.cache_specs[1], model.cache_specs[6]
    assert isinstance(kv0, PagedKVSpec) and kv0.window == 13 and kv0.head_dim == 32  # the reader's longer window is kept
    assert kv3.window == 5 and kv3.n_kv_heads == 3
    assert all(isinstance(model.cache_specs[i], StateSpec) for i in (0, 2, 3, 4, 5, 7))
    assert model.cache_specs[0].shape == (2 * 48,)  # taps - 1 rows of the width

    # a reader without a window keeps every key of the layer it reads
    from cwm_amd.models.digasun import cache_windows

    wide = digasun.model_of([digasun.attention(2, 2, 8, 8, 0.3, mask=6), digasun.attention(4, 2, 8, 8, 0.3, kv_from=0)])
    assert cache_windows(parse_config(wide)[1]) == {0: None}


def test_configurations_without_the_optional_keys_have_neither_part():
    from cwm_amd.config import parse_config
    from cwm_amd.models.model import Model

    config = digasun.model_of([digasun.attention(2, 1, 8, 8, 0.3, mask=4)], taps=None, side=None)
    arch, typed = parse_config(config)
    model = Model(arch.build_plan(typed))
    assert not any("canon" in n or "side" in n for n in model.tensor_specs())
    assert len(model.cache_specs) == 1


# ---- everything around the kernels --------------------------------------------------------------------------------- #
LENGTHS = {"tiny_g": [1, 6, 21, 40], "tiny_h": [9, 33, 2, 17, 26], "tiny_i": [70, 12, 45]}


@pytest.mark.parametrize("name", list(digasun.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_regimes_against_plain(tmp_path, monkeypatch, name, regime):
    """Pages that are freed (also by the windows, the shared caches among them) and used again, state slots that are
    used again, portions down to two tokens, unequal requests side by side: with torch in the kernels' place every
    difference is a fault of the descriptor, the tables, the slots or the plan."""
    from cwm_amd.replay import Replayer

    cpu_ops.install(monkeypatch)
    folder = digasun.make_folder(tmp_path, name, seed=3)
    vocab = digasun.get(name)["vocab"]
    requests = {f"r{i}": traces.random_tokens(11 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}
    steps = {"whole": traces.whole, "tail": lambda r: traces.tail_one_by_one(r, tail=8), "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=2, decode_tail=5)}[regime](requests)
    rep = Replayer(folder, "float32", traces.max_live_tokens(steps), device="cpu", page_size=4 if regime == "mixed" else 16,
                   max_requests=2 if regime == "mixed" else 4, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = digasun.expected(folder, requests, "float32")
    for rid in requests:
        assert not np.isnan(got[rid]).any(), f"{rid}: missing or NaN logits"
        np.testing.assert_allclose(got[rid], want[rid].exact, rtol=2e-3, atol=2e-4 * float(np.abs(want[rid].exact).max()), err_msg=f"{name} {regime} {rid}")
    assert rep.manager.live_requests() == []
    assert all(f == g.pool.num_pages for f, g in zip(rep.manager.free_pages(), rep.manager.groups))
