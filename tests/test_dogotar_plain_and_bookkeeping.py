"""Without a GPU: the plain implementation's mechanisms against library routines, invariants and hand-unrolled
formulas, the configuration and the plan of the Dogotar architecture, the cache need of blocks of positions, the
attention work lists with such blocks, and everything around the kernels (pages, windows, blocks, state slots,
portions, mixed steps) with the kernels replaced by torch stand-ins."""

import math

import numpy as np
import pytest
import torch

from helpers import cpu_ops, dogotar, traces
from plain import dogotar_plain as dp

F64 = torch.float64


# ---- the plain implementation itself -------------------------------------------------------------------------- #
def test_layer_norm_is_the_library_s():
    x = torch.randn(5, 24, dtype=F64) * 3 + 1
    g, b = torch.randn(24, dtype=F64), torch.randn(24, dtype=F64)
    assert torch.allclose(dp.layer_norm(x, g, b, 1e-5), torch.nn.functional.layer_norm(x, (24,), g, b, 1e-5))
    tiny = torch.tensor([[1e-4, -1e-4]], dtype=F64)  # eps inside the root
    assert torch.allclose(dp.layer_norm(tiny, torch.ones(2, dtype=F64), torch.zeros(2, dtype=F64), 1e-6), tiny / math.sqrt(1e-8 + 1e-6))


def test_gelu_is_the_tanh_form():
    z = torch.linspace(-4, 4, 41, dtype=F64)
    assert torch.allclose(dp.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))


def test_rotation_pairs_halves_of_the_turned_part_and_stretches_positions():
    q, k = torch.randn(1, 1, 10, dtype=F64), torch.randn(1, 1, 10, dtype=F64)
    at = lambda x, p: dp.turn_halves(x, torch.tensor([p]), 6, 100.0, 4.0)  # noqa: E731
    assert torch.allclose((at(q, 9) * at(k, 4)).sum(), (at(q, 25) * at(k, 20)).sum())  # the distance only
    assert torch.equal(at(q, 7)[..., 6:], q[..., 6:])  # the rest passes
    assert torch.allclose(at(q, 0), q)
    # element 0 is paired with element 3 (= dims / 2) and turns by position / factor: base^0 = 1
    x = torch.zeros(1, 1, 8, dtype=F64)
    x[0, 0, 0] = 1.0
    y = dp.turn_halves(x, torch.tensor([2]), 6, 50.0, 4.0)[0, 0]
    assert torch.allclose(y[[0, 3]], torch.tensor([math.cos(0.5), math.sin(0.5)], dtype=F64)) and y[[1, 2, 4, 5]].abs().max() == 0
    # element 2 with element 5, by position * base^(-4/6) / factor
    x = torch.zeros(1, 1, 8, dtype=F64)
    x[0, 0, 5] = 1.0
    a = 3 * 50.0 ** (-4 / 6) / 4.0
    y = dp.turn_halves(x, torch.tensor([3]), 6, 50.0, 4.0)[0, 0]
    assert torch.allclose(y[[2, 5]], torch.tensor([-math.sin(a), math.cos(a)], dtype=F64))


def test_masks():
    w = dp.sliding_visible(8, 3)
    assert [int(w[5, j]) for j in range(8)] == [0, 0, 0, 1, 1, 1, 0, 0]
    c = dp.block_visible(8, 3)
    assert [int(c[5, j]) for j in range(8)] == [0, 0, 0, 1, 1, 1, 0, 0]
    assert [int(c[6, j]) for j in range(8)] == [0, 0, 0, 0, 0, 0, 1, 0]  # the first position of the third block sees itself only
    assert [int(c[4, j]) for j in range(8)] == [0, 0, 0, 1, 1, 0, 0, 0]
    assert torch.equal(dp.sliding_visible(5, None), torch.tril(torch.ones(5, 5, dtype=torch.bool)))


def _attention_tensors(width, m, seed=0, gate=True):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)  # noqa: E731
    t = {"q": r(m["heads"] * m["dim"], width), "k": r(m["kv_heads"] * m["dim"], width), "v": r(m["kv_heads"] * m["vdim"], width),
         "q.b": r(m["heads"] * m["dim"]), "k.b": r(m["kv_heads"] * m["dim"]), "v.b": r(m["kv_heads"] * m["vdim"]),
         "o": r(width, m["heads"] * m["vdim"]), "q.norm": r(m["dim"]).abs() + 0.5, "k.norm": r(m["dim"]).abs() + 0.5, "vmix": torch.tensor(0.3, dtype=F64)}
    if gate:
        t["g"] = r(m["heads"] * m["vdim"], width)
    return t


def test_attention_is_the_unrolled_formula_for_one_query():
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.7, "softcap": 2.0, "rot": {"base": 10.0, "dims": 4, "scaling": {"factor": 2.0}}, "v_mix": True}
    t = _attention_tensors(9, m, seed=3)
    h = torch.randn(7, 9, dtype=F64)
    v_first = torch.randn(7, 2, 5, dtype=F64)
    got, v_used = dp.softmax_attention_mixer(t, "", m, h, 1e-5, dp.sliding_visible(7, 3), v_first)
    i, eps = 6, 1e-5
    q = (h @ t["q"].T + t["q.b"]).reshape(7, 4, 6)
    k = (h @ t["k"].T + t["k.b"]).reshape(7, 2, 6)
    v = 0.7 * (h @ t["v"].T + t["v.b"]).reshape(7, 2, 5) + 0.3 * v_first
    assert torch.allclose(v, v_used)
    q = q / torch.sqrt((q ** 2).mean(-1, keepdim=True) + eps) * t["q.norm"]  # every head by itself, one weight for all
    k = k / torch.sqrt((k ** 2).mean(-1, keepdim=True) + eps) * t["k.norm"]

    def turn(x, p):  # pairs (0, 2) and (1, 3); elements 4 and 5 pass
        out = x.clone()
        for a in range(2):
            ang = p * 10.0 ** (-2 * a / 4) / 2.0
            out[a] = x[a] * math.cos(ang) - x[a + 2] * math.sin(ang)
            out[a + 2] = x[a + 2] * math.cos(ang) + x[a] * math.sin(ang)
        return out

    heads = []
    for head in range(4):
        g = head // 2
        keys = [4, 5, 6]
        s = torch.stack([2.0 * torch.tanh(0.7 * (turn(q[i, head], i) * turn(k[j, g], j)).sum() / 2.0) for j in keys])
        heads.append((torch.softmax(s, 0)[:, None] * v[keys, g]).sum(0))
    want = (torch.cat(heads) * torch.sigmoid(h[i] @ t["g"].T)) @ t["o"].T
    assert torch.allclose(got[i], want)


def test_attention_window_and_block_read_what_they_should():
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.5}
    t = _attention_tensors(10, m, gate=False)
    h = torch.randn(12, 10, dtype=F64)
    moved = h.clone()
    moved[5] += 1.0
    for visible, readers in ((dp.sliding_visible(12, 4), [5, 6, 7, 8]), (dp.block_visible(12, 4), [5, 6, 7])):
        base, _ = dp.softmax_attention_mixer(t, "", m, h, 1e-6, visible)
        out, _ = dp.softmax_attention_mixer(t, "", m, moved, 1e-6, visible)
        changed = (out - base).abs().max(-1).values > 1e-12
        assert changed.tolist() == [i in readers for i in range(12)]


def _memory_tensors(width, m, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)  # noqa: E731
    qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
    return {"q": r(qk, width), "k": r(qk, width), "v": r(vv, width), "g": r(vv, width), "o": r(width, vv), "norm": r(vv).abs() + 0.5,
            "i": r(m["heads"], width), "i.b": r(m["heads"]), "f": r(m["heads"], width), "f.b": r(m["heads"]) + 2}


def test_matrix_memory_is_its_unstabilised_sum():
    """With the true state C_t = sum_s exp(i_s + f_(s+1) + .. + f_t) k_s v_s^T the result is
    C_t^T q / (max(|n_t . q|, 1) + 1e-6 exp(m_t)): the running maximum only enters through the small constant."""
    m = {"heads": 2, "dim": 5, "vdim": 3, "gate_cap": 3.0}
    t = _memory_tensors(8, m, seed=1)
    h = torch.randn(9, 8, dtype=F64) * 0.5
    got = dp.matrix_memory(t, "", m, h, 1e-5)
    T, H, d, e, c = 9, 2, 5, 3, 3.0
    q = (h @ t["q"].T).reshape(T, H, d) / math.sqrt(d)
    k, v = (h @ t["k"].T).reshape(T, H, d), (h @ t["v"].T).reshape(T, H, e)
    gi = c * torch.tanh((h @ t["i"].T + t["i.b"]) / c)
    gf = torch.nn.functional.logsigmoid(c * torch.tanh((h @ t["f"].T + t["f.b"]) / c))
    y = torch.zeros(T, H, e, dtype=F64)
    for a in range(H):
        run = 0.0
        for tt in range(T):
            run = max(float(gf[tt, a]) + run, float(gi[tt, a]))  # starts from 0, not from minus infinity
            C, n = torch.zeros(d, e, dtype=F64), torch.zeros(d, dtype=F64)
            for s in range(tt + 1):
                wgt = torch.exp(gi[s, a] + gf[s + 1 : tt + 1, a].sum())
                C += wgt * torch.outer(k[s, a], v[s, a])
                n += wgt * k[s, a]
            y[tt, a] = (C.T @ q[tt, a]) / (max(abs(float(n @ q[tt, a])), 1.0) + 1e-6 * math.exp(run))
    y = y / torch.sqrt((y ** 2).mean(-1, keepdim=True) + 1e-5)
    want = (y.reshape(T, H * e) * t["norm"] * torch.sigmoid(h @ t["g"].T)) @ t["o"].T
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-12)


def test_a_window_or_a_block_one_key_off_a_cap_left_out_or_a_lost_state_would_show():
    config = dogotar.get("tiny_e")
    folder_weights = {k: v.to(F64) for k, v in dogotar.draw_weights(config, 5).items()}
    toks = traces.random_tokens(3, 60, config["vocab"])
    exact = dp.forward(config, folder_weights, toks)
    size = float(exact.abs().max())
    for change in ("window", "block", "cap", "mix"):
        other = dogotar.get("tiny_e")
        if change == "window":
            other["layers"][0]["mixer"]["mask"]["size"] += 1
        elif change == "block":
            other["layers"][1]["mixer"]["left"]["mask"]["size"] -= 1
        elif change == "cap":
            del other["layers"][0]["mixer"]["softcap"]
        else:
            other["layers"][4]["mixer"]["right_scale"] = 0.0
        assert (dp.forward(other, folder_weights, toks) - exact).abs().max() > 1e-2 * size, change


# ---- configuration, plan and cache needs ------------------------------------------------------------------------ #
def test_config_is_strict_and_the_plan_names_the_folder_s_tensors():
    from cwm_amd.config import ConfigError, parse_config
    from cwm_amd.models.model import Model
    from cwm_amd.parts.base import ChunkedKVSpec, PagedKVSpec, StateSpec

    for name, config in list(dogotar.ALL.items()) + [("medium", dogotar.MEDIUM)]:
        arch, typed = parse_config(config)
        assert arch.name == "Dogotar"
        model = Model(arch.build_plan(typed))
        weights = dogotar.draw_weights(config, 1)
        specs = model.tensor_specs()
        assert set(specs) == set(weights), name
        assert all(tuple(weights[k].shape) == tuple(specs[k].shape) for k in specs)
        needs = iter(model.cache_specs)
        for layer in config["layers"]:
            m = layer["mixer"]
            if dogotar.layer_kind(layer) == "attention":
                spec = next(needs)
                assert type(spec) is PagedKVSpec and spec.n_kv_heads == m["kv_heads"] and spec.head_dim >= max(m["dim"], m["vdim"])
                assert spec.window == (m["mask"]["size"] if "mask" in m else None)
            else:
                left, right = next(needs), next(needs)
                if "mask" in m["left"]:
                    assert isinstance(left, ChunkedKVSpec) and left.chunk == m["left"]["mask"]["size"] and left.window is None
                else:
                    assert type(left) is PagedKVSpec and left.window is None
                assert isinstance(right, StateSpec) and right.shape[0] >= m["right"]["heads"] * (m["right"]["dim"] + 1) * m["right"]["vdim"]
    bad = dogotar.get("tiny_d")
    bad["layers"][1]["mixer"]["windows"] = 3
    with pytest.raises(ConfigError, match="windows"):
        parse_config(bad)
    bad = dogotar.get("tiny_d")
    bad["layers"][0]["mixer"]["right"]["gate_cap"] = 0.0
    with pytest.raises(ConfigError, match="gate_cap"):
        parse_config(bad)
    bad = dogotar.get("tiny_d")
    bad["layers"][2]["mixer"]["vdim"] = 12  # the values it would blend in have another size
    with pytest.raises(ConfigError, match="vdim"):
        parse_config(bad)
    bad = dogotar.get("tiny_e")
    bad["layers"][3]["type"] = "recurrent"
    with pytest.raises(ConfigError, match="recurrent"):
        parse_config(bad)


def test_only_the_first_blending_layer_keeps_its_values_for_the_others():
    from cwm_amd.config import parse_config

    arch, typed = parse_config(dogotar.get("tiny_d"))
    plan = arch.build_plan(typed)
    roles = [layer.parts["mixer"].choice.args.get("value_mix") for layer in plan.layers]
    assert roles == [None, "source", "mix", None, "mix"]


def test_a_cache_of_blocks_gives_back_what_lies_before_the_next_token_s_block():
    from cwm_amd.cache import CacheManager
    from cwm_amd.parts.base import ChunkedKVSpec, PagedKVSpec

    spec = ChunkedKVSpec(n_kv_heads=1, head_dim=16, chunk=10)
    assert [spec.first_key_needed(n) for n in (0, 9, 10, 11, 29, 30)] == [0, 0, 10, 10, 20, 30]
    assert spec.retention() != PagedKVSpec(1, 16, 10).retention()
    manager = CacheManager([spec, PagedKVSpec(1, 16, None)], page_size=4, num_pages=16, max_requests=2)
    assert len(manager.groups) == 2
    manager.admit("a")
    held = []
    for step in (9, 1, 7, 3, 12):  # lengths 9, 10, 17, 20, 32
        assert manager.extend("a", step)
        manager.advance("a", step)
        held.append([p >= 0 for p in manager.table(0, "a")])
    assert held[0] == [True, True, True]
    assert held[1] == [False, False, True]  # the block from 10 on starts in page 2; pages 0 and 1 are back in the pool
    assert held[2] == [False, False, True, True, True]
    assert held[3] == [False] * 5  # length 20: the next token starts a block, nothing before it is read again
    assert held[4] == [False] * 7 + [True]
    assert all(p >= 0 for p in manager.table(1, "a"))
    manager.release("a")
    manager.check()
    assert manager.free_pages() == [16, 16]


@pytest.mark.parametrize("chunk", [1, 5, 16, 40, 3000])
def test_work_lists_with_blocks_cover_every_row_s_keys_once(chunk):
    from cwm_amd.ops.attention_plan import ROWS_PER_TILE, WIDE_TILES, build_plan

    group = 3
    q_lens, kv_lens = [1, 7, 200, 64, 1], [1, 7, 333, 5000, 4097]
    plan = build_plan(q_lens, kv_lens, group, None, wide_cut_below=4, chunk=chunk)
    covered = {}
    for items, tiles in ((plan.work, 1), (plan.work_wide, WIDE_TILES)):
        for b, row0, lo, hi, _slot, _n in items.tolist():
            n_old, n_rows = kv_lens[b] - q_lens[b], q_lens[b] * group
            for r in range(row0, min(row0 + tiles * ROWS_PER_TILE, n_rows)):
                p = n_old + r // group
                first = p - p % chunk
                keys = covered.setdefault((b, r), [])
                keys.extend(range(max(lo, first), min(hi, p + 1)))
    for b, (q, kv) in enumerate(zip(q_lens, kv_lens)):
        for r in range(q * group):
            p = kv - q + r // group
            assert sorted(covered[(b, r)]) == list(range(p - p % chunk, p + 1)), (b, r)


# ---- everything around the kernels ----------------------------------------------------------------------------- #
LENGTHS = {"tiny_d": [1, 6, 21, 40], "tiny_e": [9, 33, 2, 17, 26], "tiny_f": [70, 12, 45]}


@pytest.mark.parametrize("name", list(dogotar.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_regimes_against_plain(tmp_path, monkeypatch, name, regime):
    """Pages that are freed (also by the windows and blocks) and used again, state slots that are used again, portions
    down to two tokens, unequal requests side by side: with torch in the kernels' place every difference is a fault of
    the descriptor, the tables, the slots or the plan."""
    from cwm_amd.replay import Replayer

    cpu_ops.install(monkeypatch)
    folder = dogotar.make_folder(tmp_path, name, seed=3)
    vocab = dogotar.get(name)["vocab"]
    requests = {f"r{i}": traces.random_tokens(11 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}
    steps = {"whole": traces.whole, "tail": lambda r: traces.tail_one_by_one(r, tail=8), "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=2, decode_tail=5)}[regime](requests)
    rep = Replayer(folder, "float32", traces.max_live_tokens(steps), device="cpu", page_size=4 if regime == "mixed" else 16,
                   max_requests=2 if regime == "mixed" else 4, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = dogotar.expected(folder, requests, "float32")
    for rid in requests:
        assert not np.isnan(got[rid]).any(), f"{rid}: missing or NaN logits"
        np.testing.assert_allclose(got[rid], want[rid].exact, rtol=2e-3, atol=2e-4 * float(np.abs(want[rid].exact).max()), err_msg=f"{name} {regime} {rid}")
    assert rep.manager.live_requests() == []
    assert all(f == g.pool.num_pages for f, g in zip(rep.manager.free_pages(), rep.manager.groups))
