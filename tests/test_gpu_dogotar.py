"""The Dogotar architecture on the GPU against the plain implementation.

First the kernels that came with it, each alone against the plain implementation's function for that mechanism (the
layer norms of one row's statistics over a sum that is done on the way, the matrix memory walked token by token and
taken in blocks of tokens, with states in slots that are used again, and attention over blocks of positions with capped
scores and a loud key at a block's edges); then models: every regime of the replay driver in both types with pages
and state slots that are used again; single layers that leave one mechanism nearly alone; sharp attention and a slow
memory over long sequences; first tokens and long decoding; decode steps replayed from graphs; greedy generation
through the engine, the command line and `bin/trace_run`; and configurations drawn from seeds."""

import json
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import dogotar, traces
from plain import dogotar_plain as dp

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g) * scale


# ---- kernels ----------------------------------------------------------------------------------------------------- #
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("dim,parts", [(40, 1), (256, 3), (120, 1), (1000, 2), (7, 1), (6144, 1), (2048, 4)])
def test_two_layer_norms_of_one_sum(out_dtype, dim, parts):
    """The residual takes a weighted sum of two sublayers' results (one of them in partial sums) and the two norms
    of the next layer come out of the same mean and variance; then the rows that are asked for only."""
    from cwm_amd import ops

    n = 37
    h = rnd((n, dim), 1, 2.0) + 3.0  # a mean that a variance about zero would mistake
    a = rnd((parts, n, dim), 2)
    b = rnd((n, dim), 3).to(out_dtype)
    w1, b1, w2, b2 = rnd((dim,), 4) + 1, rnd((dim,), 5), rnd((dim,), 6) + 1, rnd((dim,), 7)
    eps = 1e-5
    total = h.double() + 0.7 * (a.double().sum(0) if parts > 1 else a[0].double()) + 1.3 * b.double()
    hd = h.to(DEV).clone()
    terms = ops.ScaledSum([((a if parts > 1 else a[0]).to(DEV), 0.7), (b.to(DEV), 1.3)])
    o1, o2 = ops.add_layernorm(hd, terms, w1.to(DEV), b1.to(DEV), eps, out_dtype, weight2=w2.to(DEV), bias2=b2.to(DEV))
    t = dict(rtol=2e-5, atol=2e-5) if out_dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(hd.cpu().double(), total, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(o1.cpu().double(), dp.layer_norm(total, w1.double(), b1.double(), eps), **t)
    torch.testing.assert_close(o2.cpu().double(), dp.layer_norm(total, w2.double(), b2.double(), eps), **t)
    rows = torch.tensor([36, 0, 5], dtype=torch.int32)
    before = hd.clone()
    last = ops.add_layernorm(hd, None, w1.to(DEV), b1.to(DEV), eps, torch.float32, rows=rows.to(DEV))
    assert torch.equal(hd, before)
    torch.testing.assert_close(last.cpu().double(), dp.layer_norm(total[rows.long()], w1.double(), b1.double(), eps), rtol=2e-5, atol=2e-5)


def test_a_layer_norm_takes_the_variance_about_the_mean():
    """Rows far from zero with a small spread: mean(x^2) - mean^2 in float32 would lose the spread."""
    from cwm_amd import ops

    dim = 512
    x = 1000.0 + rnd((9, dim), 11, 0.01)
    w, b = torch.ones(dim), torch.zeros(dim)
    got = ops.add_layernorm(x.to(DEV).clone(), None, w.to(DEV), b.to(DEV), 1e-6, torch.float32)
    want = dp.layer_norm(x.double(), w.double(), b.double(), 1e-6)
    assert (got.cpu().double() - want).abs().max() < 0.02 * want.abs().max()


class MemoryCase:
    """Random weights of one matrix memory between an input and an identity as the output projection, the kernel's
    arguments for any cut of the sequences into steps, and the plain implementation's results."""

    def __init__(self, heads, d, e, cap, lengths, dtype, seed, width=24):
        self.heads, self.d, self.e, self.cap, self.lengths, self.dtype = heads, d, e, cap, lengths, dtype
        self.eps = 1e-5
        g = torch.Generator().manual_seed(seed)
        r = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16).double()  # noqa: E731
        qk, vv = heads * d, heads * e
        self.w = {"q": r(qk, width, std=2.0 * width ** -0.5), "k": r(qk, width, std=width ** -0.5), "v": r(vv, width, std=width ** -0.5),
                  "g": r(vv, width, std=2.0 * width ** -0.5), "o": torch.eye(vv, dtype=F64), "norm": r(vv).abs() + 0.5,
                  "i": r(heads, width, std=0.6 * cap * width ** -0.5), "f": r(heads, width, std=0.6 * cap * width ** -0.5),
                  "i.b": r(heads), "f.b": r(heads).abs() + 1.0}
        self.h = [r(n, width) for n in lengths]
        w = self.w
        self.proj = [torch.cat([h @ w["q"].T, h @ w["k"].T, h @ w["v"].T, h @ w["g"].T], 1).to(dtype).to(DEV) for h in self.h]
        self.gates = [torch.cat([h @ w["i"].T + w["i.b"], h @ w["f"].T + w["f.b"]], 1).float().to(DEV) for h in self.h]
        self.weight = w["norm"].float().to(DEV)
        self.reference()

    def from_inputs(self, s, wobble=0.0, skip_first=False):
        """The plain implementation from the kernel's own inputs of sequence s (float64), up to the gated norm.  `wobble`:
        a relative change of every input by about that much, to see which results hang on the last bits."""
        H, d, e, c = self.heads, self.d, self.e, self.cap
        g = torch.Generator().manual_seed(s)
        shake = lambda t: t * (1.0 + wobble * torch.randn(t.shape, generator=g, dtype=F64))  # noqa: E731
        p, raw = shake(self.proj[s].double().cpu()), shake(self.gates[s].double().cpu())
        T = p.shape[0]
        q = p[:, : H * d].reshape(T, H, d) * d ** -0.5
        k = p[:, H * d : 2 * H * d].reshape(T, H, d)
        v = p[:, 2 * H * d : 2 * H * d + H * e].reshape(T, H, e)
        gi = shake(c * torch.tanh(raw[:, :H] / c))
        gf = torch.nn.functional.logsigmoid(shake(c * torch.tanh(raw[:, H:] / c)))
        if skip_first:
            gi[0] = -1e9
        out = dp.memory_recurrence(q, k, v, gi, gf)
        return dp.unit_rms(out, self.eps).reshape(T, H * e) * self.w["norm"] * torch.sigmoid(p[:, 2 * H * d + H * e :])

    def reference(self):
        """What is wanted, and how far a change of the inputs in their last float32 bits moves it: a row whose
        normaliser or whose products nearly cancel is moved by any order of float32 sums."""
        n = len(self.lengths)
        self.want = [self.from_inputs(s) for s in range(n)]
        self.loose = [(self.from_inputs(s, wobble=1e-7) - self.want[s]).abs() for s in range(n)]

    def run(self, steps, slots, n_slots=None):
        """steps: lists of (sequence, tokens); returns every sequence's rows and the state tensor."""
        from cwm_amd import ops

        elems = ops.matrix_memory_state_elems(self.heads, self.d, self.e)
        state = torch.zeros((n_slots or max(slots) + 2, elems), dtype=torch.float32, device=DEV)
        state[[s for s in range(state.shape[0]) if s not in slots]] = float("nan")
        done = [0] * len(self.lengths)
        rows = [[] for _ in self.lengths]
        for step in steps:
            cu = [0]
            for _, n in step:
                cu.append(cu[-1] + n)
            batch = SimpleNamespace(
                n_tokens=cu[-1], n_seqs=len(step), q_lens=[n for _, n in step], scratch={},
                cu_q=torch.tensor(cu, dtype=torch.int32, device=DEV), state_slots=torch.tensor([slots[s] for s, _ in step], dtype=torch.int32, device=DEV),
            )
            proj = torch.cat([self.proj[s][done[s] : done[s] + n] for s, n in step])
            gates = torch.cat([self.gates[s][done[s] : done[s] + n] for s, n in step])
            out = ops.matrix_memory(proj, gates, self.weight, state, batch, self.heads, self.d, self.e, self.cap, self.eps)
            for (s, n), a, b in zip(step, cu, cu[1:]):
                rows[s].append(out[a:b].cpu())
                done[s] += n
        assert done == list(self.lengths)
        return [torch.cat(r) for r in rows], state

    def check(self, got, what):
        rtol, atol = (1e-4, 2e-5) if self.dtype == torch.float32 else (2e-2, 2e-2)
        for s, (g, w, loose) in enumerate(zip(got, self.want, self.loose)):
            assert torch.isfinite(g).all(), f"{what}: sequence {s}"
            over = (g.double() - w).abs() - (atol + rtol * w.abs() + 50.0 * loose)
            assert over.max() <= 0, f"{what}: sequence {s}: element {divmod(int(over.argmax()), w.shape[1])} is {float(over.max()):.3e} over"
            assert (loose > atol).float().mean() < 0.01, "the case itself hangs on the last bits"


def cut(lengths, sizes):
    """Steps that hold every unfinished sequence's next portion, with sizes taken in turn."""
    left, steps, i = list(lengths), [], 0
    while any(left):
        step = []
        for s, n in enumerate(left):
            if n:
                take = min(n, sizes[i % len(sizes)])
                i += 1
                step.append((s, take))
                left[s] -= take
        steps.append(step)
    return steps


MEMORY_SIZES = [(3, 10, 14), (1, 17, 5), (2, 6, 33), (4, 64, 32), (2, 128, 128), (1, 200, 40), (2, 256, 70), (5, 12, 64), (1, 1, 1)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,d,e", MEMORY_SIZES)
def test_matrix_memory_walked_and_in_blocks(dtype, heads, d, e):
    """Whole portions (blocks of tokens), short portions (the walk), and steps that mix a long portion with single
    tokens, with the states in slots of any order; the walk gives the same bits however it is cut."""
    from cwm_amd import ops

    lengths = [150, 77, 1, 40]
    case = MemoryCase(heads, d, e, 6.0, lengths, dtype, seed=heads + d + e)
    slots = [3, 0, 5, 1]
    whole, state = case.run([[(s, n) for s, n in enumerate(lengths)]], slots)
    case.check(whole, "whole")
    assert torch.isnan(state[[2, 4, 6]]).all() and torch.isfinite(state[slots]).all()
    walked, state_walked = case.run(cut(lengths, [8, 1, 5, 2, 7]), slots)
    case.check(walked, "walked in short portions")
    one_by_one, state_one = case.run(cut(lengths, [1]), slots)
    for a, b in zip(walked, one_by_one):
        assert torch.equal(a, b)
    assert torch.equal(state_walked[slots], state_one[slots])
    mixed, state_mixed = case.run(cut(lengths, [33, 2, 1, 64, 31, 9, 100, 8]), slots)
    case.check(mixed, "long and short portions mixed")
    # the states agree too: the matrix, the normaliser and the maximum (the same float32 operations give the same maximum)
    for s in slots:
        a, b = ops.matrix_memory_state_unpack(state[s], heads, d, e), ops.matrix_memory_state_unpack(state_one[s], heads, d, e)
        assert torch.equal(a[2], b[2])
        torch.testing.assert_close(a[0], b[0], rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(a[1], b[1], rtol=1e-4, atol=1e-5)


def test_matrix_memory_keeps_a_loud_first_token_over_a_long_portion():
    """The first token's input gate is at its cap and every later forget gate close to one: what the last tokens
    read is mostly the first token's value, hundreds of tokens and many blocks back, in portions and decoded."""
    case = MemoryCase(2, 32, 16, 10.0, [700], torch.float32, seed=4)
    g = case.gates[0]
    g[:, :2] = -8.0  # input gates low ...
    g[0, :2] = 40.0  # ... but the first token's
    g[:, 2:] = 40.0  # forget gates at one
    q = case.proj[0][:, :64].view(700, 2, 32)
    q.mul_(0.3).add_(case.proj[0][0, 64:128].view(1, 2, 32))  # queries that answer the first key
    case.reference()
    without_first = case.from_inputs(0, skip_first=True)
    assert (case.want[0][-1] - without_first[-1]).abs().max() > 0.3
    for sizes in ([700], [64, 63, 65, 2, 126, 1, 31, 33, 128, 17], [690] + [1] * 10):
        got, _ = case.run(cut([700], sizes), [0])
        case.check(got, f"portions of {sizes[:3]}")


def test_matrix_memory_after_long_sums_of_strong_forget_gates():
    """Three hundred tokens that forget nearly everything, then tokens that keep: the sums of log forget gates reach
    thousands, and the weights inside a block are differences of such sums."""
    case = MemoryCase(2, 24, 12, 30.0, [420], torch.float32, seed=8)
    g = case.gates[0]
    g[:300, 2:] = -60.0
    g[300:, 2:] = 6.0
    case.reference()
    assert torch.nn.functional.logsigmoid(30.0 * torch.tanh(g[:, 2:].double().cpu() / 30.0)).sum(0).min() < -5000
    for sizes in ([420], [290, 20, 110], [1] * 420):
        got, _ = case.run(cut([420], sizes), [1])
        case.check(got, f"portions of {sizes[:3]}")


def test_a_state_slot_of_the_matrix_memory_is_read_where_the_step_says():
    """Two sequences swap their order in the batch from step to step and keep their slots."""
    case = MemoryCase(2, 20, 12, 5.0, [60, 45], torch.float32, seed=3)
    straight, _ = case.run([[(0, 30), (1, 20)], [(0, 30), (1, 25)]], [4, 2])
    swapped, _ = case.run([[(0, 30), (1, 20)], [(1, 25), (0, 30)]], [4, 2])
    for a, b in zip(straight, swapped):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)
    case.check(swapped, "swapped")


def _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, block, softcap, seed, loud=()):
    """Keys, values and queries of a mixed batch in a shuffled paged cache, and float64 attention with capped scores
    over a window or over blocks of positions."""
    g = torch.Generator().manual_seed(seed)
    scale = hd ** -0.5
    pages_per = [(a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new)]
    total = sum(pages_per) + 1
    perm = torch.randperm(total, generator=g)
    table = torch.full((len(lens_old), max(pages_per)), -1, dtype=torch.int32)
    cache = torch.full((total, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
    vb = 8 if page_size % 8 == 0 else page_size
    kc = cache[:, 0].view(total, n_kv, page_size, hd)
    vc = cache[:, 1].view(total, n_kv, page_size // vb, hd, vb)
    used, q_rows, want_rows = 0, [], []
    group = n_q // n_kv
    for b, (n0, n1) in enumerate(zip(lens_old, lens_new)):
        n = n0 + n1
        k = torch.randn((n, n_kv, hd), generator=g).to(dtype)
        v = torch.randn((n, n_kv, hd), generator=g).to(dtype)
        q = torch.randn((n1, n_q, hd), generator=g).to(dtype)
        for lb, key_pos in loud:
            if lb == b:  # a key that answers the last query's first heads loudly (those of key/value head 0)
                k[key_pos, 0] = (q[-1, 0].float() * 6.0).to(dtype)
        table[b, : pages_per[b]] = perm[used : used + pages_per[b]].to(torch.int32)
        used += pages_per[b]
        pos = torch.arange(n)
        pages, slots = table[b, pos // page_size].long(), pos % page_size
        kc[pages, :, slots, :] = k
        vc[pages, :, slots // vb, :, slots % vb] = v
        scores = torch.einsum("thd,khd->htk", q.double(), k.double().repeat_interleave(group, dim=1)) * scale
        if softcap is not None:
            scores = softcap * torch.tanh(scores / softcap)
        qpos, kpos = torch.arange(n0, n).view(1, -1, 1), torch.arange(n).view(1, 1, -1)
        ok = kpos <= qpos
        if window is not None:
            ok = ok & (kpos >= qpos - (window - 1))
        if block is not None:
            ok = ok & (kpos // block == qpos // block)
        probs = torch.softmax(scores.masked_fill(~ok, float("-inf")), -1)
        want_rows.append(torch.einsum("htk,khd->thd", probs, v.double().repeat_interleave(group, dim=1)).reshape(n1, -1))
        q_rows.append(q)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={}, max_kv_len=max(kv_lens),
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
        positions=torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32).to(DEV),
        seq_of_token=torch.cat([torch.full((n,), b) for b, n in enumerate(lens_new)]).to(torch.int32).to(DEV),
    )
    return torch.cat(q_rows).to(DEV), cache.to(DEV), table.to(DEV), batch, scale, torch.cat(want_rows)


def _both_attention_kernels(dtype, hd, page_size, case, window, block, softcap, what):
    from cwm_amd import ops

    q, cache, table, batch, scale, want = case
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    simple = ops.paged_attention_simple(q, cache, table, batch.positions, batch.seq_of_token, window, scale, softcap=softcap, chunk=block).cpu()
    torch.testing.assert_close(simple.double(), want, **t, msg=lambda m: f"{what}: plain kernel: {m}")
    if dtype == torch.bfloat16 and ops.mfma_attention_takes(dtype, hd, page_size):
        got = ops.paged_attention_mfma(q, cache, table, batch, window, scale, None, softcap, block).cpu()
        assert torch.isfinite(got).all()
        torch.testing.assert_close(got.double(), want, **t, msg=lambda m: f"{what}: matrix-core kernel: {m}")


@pytest.mark.parametrize("block", [7, 16, 64, 100, 1, 3000])
@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 16, 8), (3, 1, 32, 16), (12, 2, 128, 64), (6, 3, 80, 16), (5, 5, 48, 5)])
def test_attention_over_blocks_of_positions_with_capped_scores(n_q, n_kv, hd, page_size, block):
    """A fresh prompt, continued portions that start inside a block, decoded tokens near and far into their sequences
    and a long portion over many blocks, in both kernels and both types, with and without the cap."""
    lens_old, lens_new = [0, 37, 70, 700, 520, 13], [29, 21, 1, 1, 3, 200]
    for dtype in DTYPES:
        for softcap in (None, 2.5):
            case = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, None, block, softcap, seed=hd + n_q)
            _both_attention_kernels(dtype, hd, page_size, case, None, block, softcap, f"block {block} cap {softcap}")


@pytest.mark.parametrize("block,page_size", [(64, 16), (40, 8), (33, 32), (2, 16), (50, 64)])
def test_a_loud_key_at_a_block_s_edges(block, page_size):
    """The last query of a decoded token and of a prompt portion finds a loud key at its block's first place (it
    carries the row) or one place before it (it must not be seen, though a window of the same size would show it):
    a block that starts one key off, or is counted from the portion's start, changes these rows altogether."""
    n_q, n_kv, hd = 4, 2, 64
    lens_old, lens_new = [303, 303, 171, 171], [1, 1, 37, 37]
    last = [a + b - 1 for a, b in zip(lens_old, lens_new)]
    first = [x // block * block for x in last]
    loud = [(0, first[0]), (1, first[1] - 1), (2, first[2]), (3, first[3] - 1)]
    rows = {0: 0, 1: 1, 2: 2 + 36, 3: 2 + 37 + 36}  # the last row of each sequence
    for dtype in DTYPES:
        case = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, None, block, 25.0, seed=block, loud=loud)
        want = case[-1]
        as_window = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, block, None, 25.0, seed=block, loud=loud)[-1]
        quiet = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, None, block, 25.0, seed=block)[-1]
        for s in (1, 3):
            if last[s] - (first[s] - 1) < block:  # a window would reach the key
                assert (as_window[rows[s]] - want[rows[s]]).abs().max() > 0.3
        for s in (0, 2):
            if first[s] < last[s]:  # (a query at its block's first place sees itself only)
                assert (quiet[rows[s]] - want[rows[s]]).abs().max() > 0.3
        _both_attention_kernels(dtype, hd, page_size, case, None, block, 25.0, f"block {block}")


@pytest.mark.parametrize("window,page_size", [(64, 16), (40, 8), (33, 32), (2, 16)])
def test_a_loud_key_at_a_window_s_edges_under_the_cap(window, page_size):
    """The same with a sliding window and capped scores: the key at the window's first place is seen, the one before
    it is not."""
    n_q, n_kv, hd = 4, 2, 64
    lens_old, lens_new = [300, 300, 171, 171], [1, 1, 37, 37]
    last = [a + b - 1 for a, b in zip(lens_old, lens_new)]
    loud = [(0, last[0] - (window - 1)), (1, last[1] - window), (2, last[2] - (window - 1)), (3, last[3] - window)]
    rows = {0: 0, 1: 1, 2: 2 + 36, 3: 2 + 37 + 36}
    for dtype in DTYPES:
        case = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, None, 25.0, seed=window, loud=loud)
        want = case[-1]
        longer = _attention_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window + 1, None, 25.0, seed=window, loud=loud)[-1]
        assert (longer[rows[1]] - want[rows[1]]).abs().max() > 0.3 and (longer[rows[3]] - want[rows[3]]).abs().max() > 0.3
        _both_attention_kernels(dtype, hd, page_size, case, window, None, 25.0, f"window {window}")


@pytest.mark.parametrize("block", [None, 8192])
def test_a_loud_key_far_back_under_the_cap_where_key_ranges_are_cut_and_merged(block):
    """Decoded tokens and portions far into long sequences: the matrix-core kernel cuts their keys into ranges and a
    second kernel merges the partial results, the plain kernel cuts into segments.  One key thousands of places back
    (with blocks: at the first place of the query's block) carries the last row of a decoded token and of a portion."""
    n_q, n_kv, hd, page_size = 6, 2, 64, 64
    lens_old, lens_new = [9000, 3000, 1500, 20000, 9000], [1, 2, 1, 150, 600]
    loud = [(0, 8192 if block else 4321), (4, 8192 if block else 77)]
    case = _attention_case(torch.bfloat16, n_q, n_kv, hd, page_size, lens_old, lens_new, None, block, 25.0, seed=5, loud=loud)
    quiet = _attention_case(torch.bfloat16, n_q, n_kv, hd, page_size, lens_old, lens_new, None, block, 25.0, seed=5)[-1]
    assert (quiet[0] - case[-1][0]).abs().max() > 0.3 and (quiet[-1] - case[-1][-1]).abs().max() > 0.3
    _both_attention_kernels(torch.bfloat16, hd, page_size, case, None, block, 25.0, f"far key, block {block}")


# ---- models ------------------------------------------------------------------------------------------------------- #
LENGTHS = {"tiny_d": [1, 6, 21, 70, 130], "tiny_e": [9, 33, 2, 100, 57], "tiny_f": [150, 41, 90]}
PAGE_SIZES = {"whole": 16, "tail": 16, "portions": 8, "mixed": 8}


def requests_for(name, lengths=None):
    vocab = dogotar.get(name)["vocab"]
    return {f"r{i}": traces.random_tokens(17 * i + len(name), n, vocab) for i, n in enumerate(lengths or LENGTHS[name])}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("dogotar")
    return {name: dogotar.make_folder(root, name, seed=5) for name in dogotar.ALL}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def plain_for(folders, cache, name, dtype):
    if (name, dtype) not in cache:
        cache[name, dtype] = dogotar.expected(folders[name], requests_for(name), dtype)
    return cache[name, dtype]


def run(folder, dtype, steps, requests, vocab, **options):
    from cwm_amd.replay import Replayer

    rep = Replayer(folder, dtype, traces.max_live_tokens(steps), poison_freed_pages=True, **options)
    page_use = traces.PageUse(rep.manager)
    outputs = traces.run_in_process(rep, steps, page_use)
    assert rep.manager.live_requests() == []
    return traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab), rep, page_use


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(dogotar.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_replay_regimes(folders, plain_cache, name, dtype, regime):
    requests = requests_for(name)
    vocab = dogotar.get(name)["vocab"]
    steps = {"whole": traces.whole, "tail": traces.tail_one_by_one, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=3)}[regime](requests)
    got, rep, page_use = run(folders[name], dtype, steps, requests, vocab, page_size=PAGE_SIZES[regime], max_requests=3 if regime == "mixed" else 16)
    want = plain_for(folders, plain_cache, name, dtype)
    for rid in requests:
        dogotar.check(got[rid], want[rid], dtype, f"{name} {dtype} {regime} {rid}")
    if regime == "mixed":
        for g in rep.manager.groups:
            assert page_use.pages_shared_between_requests(g.index) > 0, f"group {g.index}: no page served two requests"


def model_of(layers, width=40, vocab=83, eps=1e-5) -> dict:
    return {"architecture": "Dogotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}


A, P, S, D = dogotar.attention, dogotar.parallel, dogotar.attn_sizes, dogotar.dense
SINGLE_LAYERS = {
    "attention_window_rotation_cap_gate": [A(4, 2, 12, 10, 0.3, softcap=6.0, mask=9, rot=(100.0, 8, 2.0))],
    "attention_without_rotation_mask_or_cap": [A(3, 3, 8, 16, 0.4)],
    "attention_whole_head_rotated_unstretched": [A(2, 1, 16, 8, 0.25, mask=40, rot=(1000.0, 16), mlp=D(24))],
    "attention_rotation_of_two_elements": [A(2, 2, 6, 6, 0.5, mask=3, rot=(50.0, 2, 3.0))],
    "values_blended_with_the_first_layer_s": [A(4, 2, 12, 10, 0.3, mask=9, v_mix=True), A(2, 2, 8, 10, 0.3, mask=5, rot=(100.0, 4), v_mix=True)],
    "values_blended_from_the_second_layer_on": [A(2, 1, 8, 6, 0.3, v_mix=False), A(3, 3, 8, 4, 0.3, v_mix=True), A(6, 3, 4, 4, 0.5, mask=4, v_mix=True), A(3, 3, 8, 4, 0.3, v_mix=True)],
    "blocks_beside_a_memory": [P(S(4, 2, 12, 20, 0.3, softcap=5.0, mask=7), 3, 10, 14, 4.0, 0.7, 1.3)],
    "memory_nearly_alone": [P(S(1, 1, 4, 4, 0.1, mask=1), 2, 18, 9, 6.0, 0.05, 2.0)],
    "blocks_nearly_alone": [P(S(2, 1, 16, 12, 0.4, softcap=9.0, mask=10), 1, 4, 4, 3.0, 1.5, 0.05, mlp=D(16))],
    "side_by_side_with_scales_left_out": [P(S(2, 2, 8, 8, 1.0, mask=1), 2, 6, 33, 2.0, mlp=D(20))],
    "feed_forward_carries_the_layer": [A(1, 1, 8, 8, 0.1, mlp=D(64))],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", list(SINGLE_LAYERS))
def test_single_layers(tmp_path, which, dtype):
    """One mechanism at a time between embedding and head: whole prompts against the same tokens in portions and one
    by one, and all against the plain implementation."""
    config = model_of(SINGLE_LAYERS[which])
    folder = dogotar.make_folder(tmp_path, which, seed=2, config=config)
    requests = {f"r{i}": traces.random_tokens(i + 5, n, config["vocab"]) for i, n in enumerate([37, 5, 64])}
    want = dogotar.expected(folder, requests, dtype)
    for make in (traces.whole, traces.portions, lambda r: traces.tail_one_by_one(r, tail=20)):
        steps = make(requests)
        got, _, _ = run(folder, dtype, steps, requests, config["vocab"], page_size=8)
        for rid in requests:
            dogotar.check(got[rid], want[rid], dtype, f"{which} {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_and_a_slow_memory_over_long_sequences(folders, dtype):
    """tiny_e's softmax is sharp and its memory forgets slowly: a token's result hangs on single keys at a window's or
    a block's edge and on what the memory took in at the sequence's start.  A prompt of 700 tokens whole, in portions
    that end at, before and after page, window and block borders (down to one and two tokens), and with its last 150
    tokens one by one."""
    name = "tiny_e"
    vocab = dogotar.get(name)["vocab"]
    requests = {"long": traces.random_tokens(99, 700, vocab)}
    want = dogotar.expected(folders[name], requests, dtype, conditioning=True)
    portions = lambda r: traces.portions(r, sizes=[64, 63, 65, 2, 126, 1, 31, 33, 128, 17, 11, 5, 16])  # noqa: E731
    for make in (traces.whole, portions, lambda r: traces.tail_one_by_one(r, tail=150)):
        steps = make(requests)
        got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=32)
        dogotar.check(got["long"], want["long"], dtype, f"{name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_layers_and_many_rows(tmp_path, dtype):
    """Width 256 and prompts of 600 and 300 tokens: the kernels' shapes for many rows, whole, in large portions beside
    each other, and with a tail of single tokens."""
    config = dogotar.MEDIUM
    folder = dogotar.make_folder(tmp_path, "medium", seed=9, config=config)
    vocab = config["vocab"]
    requests = {"a": traces.random_tokens(31, 600, vocab), "b": traces.random_tokens(32, 300, vocab)}
    want = dogotar.expected(folder, requests, dtype)
    side_by_side = [
        {"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:290], "want": list(range(290))}, {"id": "b", "tokens": requests["b"][:270], "want": list(range(270))}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": requests["a"][290:], "want": list(range(310))}, {"id": "b", "tokens": requests["b"][270:], "want": list(range(30))}], "end": ["a", "b"]},
    ]
    for steps in (traces.whole(requests), side_by_side, traces.tail_one_by_one(requests, tail=20)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=32)
        for rid in requests:
            dogotar.check(got[rid], want[rid], dtype, f"medium {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, dtype):
    """Every token a step of its own from an empty cache and a zero state, for 300 steps: windows and blocks pass over
    decoded tokens many times."""
    name = "tiny_d"
    vocab = dogotar.get(name)["vocab"]
    requests = {"a": traces.random_tokens(4, 300, vocab)}
    steps = traces.tail_one_by_one(requests, tail=299)
    got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=16)
    dogotar.check(got["a"], dogotar.expected(folders[name], requests, dtype)["a"], dtype, f"{name} {dtype} one by one")


def test_pages_and_a_state_slot_that_are_used_again_start_afresh(folders):
    """One slot and a pool of the longer request's size only: the second request finds the first one's state and
    cache rows (NaN in the pages in between) and must not read them."""
    name = "tiny_f"
    vocab = dogotar.get(name)["vocab"]
    a, b = traces.random_tokens(1, 60, vocab), traces.random_tokens(2, 25, vocab)
    both = [
        {"step": 0, "entries": [{"id": "a", "tokens": a, "want": [59]}], "end": ["a"]},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:10], "want": list(range(10))}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[10:], "want": list(range(15))}], "end": ["b"]},
    ]
    got, rep, _ = run(folders[name], "float32", both, {"a": a, "b": b}, vocab, page_size=8, max_requests=1)
    alone, _, _ = run(folders[name], "float32", both[1:], {"b": b}, vocab, page_size=8, max_requests=1)
    assert np.array_equal(got["b"], alone["b"])
    dogotar.check(got["b"], dogotar.expected(folders[name], {"b": b}, "float32")["b"], "float32", "second user of the slot")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_do_not_depend_on_the_rest_of_the_batch(folders, dtype):
    """A request's decoded tokens alone and beside two other requests' short portions: the same bits."""
    name = "tiny_d"
    vocab = dogotar.get(name)["vocab"]
    r = requests_for(name, [40, 64, 90])
    alone = [{"step": 0, "entries": [{"id": "r0", "tokens": r["r0"][:30], "want": [29]}], "end": []}] + [
        {"step": 1 + i, "entries": [{"id": "r0", "tokens": [r["r0"][30 + i]], "want": [0]}], "end": ["r0"] if i == 9 else []} for i in range(10)
    ]
    beside = [{"step": 0, "entries": [{"id": "r0", "tokens": r["r0"][:30], "want": [29]}], "end": []}]
    for i in range(10):
        entries = [{"id": "r1", "tokens": r["r1"][6 * i : 6 * i + 6], "want": [5]}, {"id": "r0", "tokens": [r["r0"][30 + i]], "want": [0]},
                   {"id": "r2", "tokens": r["r2"][8 * i : 8 * i + 8], "want": []}]
        beside.append({"step": 1 + i, "entries": entries, "end": ["r0", "r1", "r2"] if i == 9 else []})
    lengths = {"r0": r["r0"][:40], "r1": r["r1"][:60], "r2": r["r2"][:80]}
    got_alone, _, _ = run(folders[name], dtype, alone, {"r0": lengths["r0"]}, vocab, page_size=8)
    got_beside, _, _ = run(folders[name], dtype, beside, lengths, vocab, page_size=8)
    assert np.array_equal(got_alone["r0"][29:], got_beside["r0"][29:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_graphs_give_the_same_bits(folders, dtype):
    name = "tiny_e"
    vocab = dogotar.get(name)["vocab"]
    requests = requests_for(name, [30, 44, 37])
    heads = {"step": 0, "entries": [{"id": r, "tokens": t[:20], "want": [19]} for r, t in requests.items()], "end": []}
    steps = [heads] + [
        {"step": 1 + i, "entries": [{"id": r, "tokens": [t[20 + i]], "want": [0]} for r, t in requests.items()], "end": list(requests) if i == 9 else []}
        for i in range(10)
    ]
    launched, _, _ = run(folders[name], dtype, steps, {k: v[:30] for k, v in requests.items()}, vocab, page_size=16)
    replayed, rep, _ = run(folders[name], dtype, steps, {k: v[:30] for k, v in requests.items()}, vocab, page_size=16, num_graphs=2)
    assert rep.runner.n_replays >= 8, "the decode steps were not replayed"
    for rid in requests:
        assert np.array_equal(launched[rid][19:], replayed[rid][19:]), rid


@pytest.mark.parametrize("name", ["tiny_d", "tiny_f"])
def test_greedy_generation_through_the_engine(folders, name):
    """The engine's own entry point: scheduler, portions of 24 tokens, continuous batching, sampling kernel; then a
    cache that holds barely more than the longest request, so that requests wait for one another's pages and slots."""
    from cwm_amd.engine import Engine, GenArgs

    vocab = dogotar.get(name)["vocab"]
    prompts = [traces.random_tokens(20 + i, n, vocab) for i, n in enumerate([5, 17, 33, 64])]
    engine = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=2048, cache_block=16, max_prefill=24), dtype="float32")
    got = engine.generate_tokens(prompts, max_gen=12)
    for p, g in zip(prompts, got):
        assert g == dogotar.plain_greedy(folders[name], p, 12)
    small = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=96, cache_block=4, max_prefill=24), dtype="float32")
    assert small.generate_tokens(prompts, max_gen=12) == got


def test_command_line_and_trace_run_as_child_processes(folders, tmp_path):
    name = "tiny_d"
    vocab = dogotar.get(name)["vocab"]
    prompts = [traces.random_tokens(60 + i, n, vocab) for i, n in enumerate([6, 21])]
    path = tmp_path / "prompts.jsonl"
    path.write_text("".join(json.dumps({"id": i, "tokens": p}) + "\n" for i, p in enumerate(prompts)))
    cmd = [sys.executable, "-m", "cwm_amd.generate", f"checkpoint_dir={folders[name]}", f"prompts={path}", "dtype=float32",
           "gen_args.use_sampling=false", "gen_args.max_gen=7", "gen_args.max_seq=512", "gen_args.cache_block=16", "gen_args.max_batch=4"]
    res = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = {rec["id"]: rec["tokens"] for rec in map(json.loads, res.stdout.strip().splitlines())}
    for i, p in enumerate(prompts):
        assert got[i] == dogotar.plain_greedy(folders[name], p, 7)

    requests = requests_for(name, [40, 75, 33])
    steps = traces.mixed(requests)
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out_{dtype}"
        cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype, "--out", str(out),
               "--max-tokens", str(traces.max_live_tokens(steps))]
        res = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
        assert res.returncode == 0, res.stderr
        assert [line for line in res.stdout.splitlines() if line.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = {s["step"]: np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab) for s in steps if any(e["want"] for e in s["entries"])}
        got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
        want = dogotar.expected(folders[name], requests, dtype)
        for rid in requests:
            dogotar.check(got[rid], want[rid], dtype, f"trace_run {dtype} {rid}")


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: every size, count, constant and the order of layers differ from draw to draw."""
    import random

    rng = random.Random(seed)
    width = rng.choice([32, 40, 48, 64, 72, 96, 100, 128, 136, 192, 200, 256])
    shared_kv, shared_vdim = rng.choice([1, 2, 3, 4]), rng.choice([8, 12, 16, 32, 48])  # what blended values have in common

    def attention_sizes(blend: bool, rotate: bool):
        kv = shared_kv if blend else rng.choice([1, 2, 3, 4])
        heads = kv * rng.choice([1, 2, 3, 4])
        dim = rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 128])
        vdim = shared_vdim if blend else rng.choice([8, 12, 16, 32, 48, 64, 80, 128])
        rot = None
        if rotate and rng.random() < 0.8:
            rot = (rng.choice([100.0, 10000.0, 250000.0, 1e6]), rng.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim] + [dim]))
            if rng.random() < 0.6:
                rot = rot + (rng.choice([1.0, 2.0, 8.0, 32.0]),)
        return S(heads, kv, dim, vdim, rng.choice([0.05, 0.1, 0.2]) * (64 / dim) ** 0.5, softcap=rng.choice([None, 2.0, 20.0, 50.0]),
                 mask=rng.choice([None, 1, 2, 7, 16, 17, 40, 64, 100]), rot=rot, v_mix=(True if blend else rng.choice([None, False])))

    layers = []
    for _ in range(rng.randint(2, 5)):
        mlp = D(rng.choice([20, 36, 64, 100, 256])) if rng.random() < 0.75 else None
        if rng.random() < 0.5:
            layers.append({"type": "attention", "mixer": attention_sizes(rng.random() < 0.6, True), "mlp": mlp})
        else:
            left = attention_sizes(False, False)
            left.pop("v_mix", None)
            scales = (rng.choice([0.5, 1.0, 1.2]), rng.choice([0.7, 0.9, 1.0, 2.0])) if rng.random() < 0.8 else (None, None)
            layers.append(P(left, rng.randint(1, 5), rng.choice([4, 8, 12, 16, 24, 48, 64, 100]), rng.choice([4, 8, 16, 33, 48, 64, 80]),
                            rng.choice([2.0, 8.0, 12.0, 15.0, 30.0]), scales[0], scales[1], mlp=mlp))
    return model_of(layers, width=width, vocab=rng.randint(50, 700), eps=rng.choice([1e-5, 1e-6]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed, dtype):
    """Other models of the design: whole prompts, and a mixed schedule with pages of another size, against the plain
    implementation."""
    config = random_config(seed)
    folder = dogotar.make_folder(tmp_path, f"random{seed}", seed=seed, config=config)
    vocab = config["vocab"]
    requests = {f"r{i}": traces.random_tokens(7 * seed + i, n, vocab) for i, n in enumerate([3, 150, 45, 88])}
    want = dogotar.expected(folder, requests, dtype, conditioning=True)
    for steps, page in ((traces.whole(requests), 16), (traces.mixed(requests, max_live=3), 32 if seed % 2 else 8)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=page, max_requests=4)
        dogotar.check_together(got, want, dtype, f"random configuration {seed} {dtype}: {json.dumps(config)}")
