"""The Digasun architecture on the GPU against the plain implementation.

First the kernels that came with it, each alone against the plain implementation's function for that mechanism
(attention whose heads mix their weights after a softmax with a sink, over windows and cut key ranges, with a loud key
far back and at a window's edges; gated linear attention walked in portions of any size, with states in slots that
are used again; the input convolutions with their state; a layer's own token input; gated activations on rows); then
models: every regime of the replay driver in both types with pages and state slots that are used again; single
layers that leave one mechanism nearly alone; sharp attention and slow decays over long sequences; first tokens and
long decoding; decode steps replayed from graphs; greedy generation through the engine, the command line and
`bin/trace_run`; and configurations drawn from seeds."""

import json
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import digasun, traces
from plain import digasun_plain as gp

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g) * scale


def step_batch(lens_old, lens_new, slots=None):
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    return SimpleNamespace(
        q_lens=list(lens_new), kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={}, static=None, max_kv_len=max(kv_lens),
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
        positions=torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32).to(DEV),
        seq_of_token=torch.cat([torch.full((n,), b) for b, n in enumerate(lens_new)]).to(torch.int32).to(DEV),
        state_slots=torch.tensor(slots if slots is not None else list(range(len(lens_new))), dtype=torch.int32).to(DEV),
    )


# ---- attention whose heads mix their weights ------------------------------------------------------------------------ #
def _talking_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, seed, loud=(), sink_scale=1.0, talk=True):
    """Keys, values and queries of a mixed batch in a shuffled paged cache, and the plain implementation's result: a
    softmax with a sink over the window, the heads' weights mixed, each head on its own values."""
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
    sink = torch.randn(n_q, generator=g) * sink_scale
    mix = (0.5 * torch.eye(n_q) + 0.5 * torch.randn((n_q, n_q), generator=g)) if talk else None
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
        scores = torch.einsum("thd,khd->htk", q.double(), k.double().repeat_interleave(group, dim=1)) * scale  # [H, n1, n]
        qpos, kpos = torch.arange(n0, n).view(-1, 1), torch.arange(n).view(1, -1)
        ok = kpos <= qpos
        if window is not None:
            ok = ok & (kpos >= qpos - (window - 1))
        weights = gp.mix_heads(gp.sink_softmax(scores, ok, sink.double()), mix.double() if mix is not None else None)
        want_rows.append(torch.einsum("htk,khd->thd", weights, v.double().repeat_interleave(group, dim=1)).reshape(n1, -1))
        q_rows.append(q)
    batch = step_batch(lens_old, lens_new)
    return torch.cat(q_rows).to(DEV), cache.to(DEV), table.to(DEV), batch, scale, sink.to(DEV), (mix.to(DEV) if mix is not None else None), torch.cat(want_rows)


def _check_talking(dtype, case, window, what):
    from cwm_amd import ops

    q, cache, table, batch, scale, sink, mix, want = case
    t = dict(rtol=1e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    got = ops.talking_attention(q, cache, table, batch, window, scale, sink=sink, talk=mix).cpu()
    assert torch.isfinite(got).all(), what
    torch.testing.assert_close(got.double(), want, **t, msg=lambda m: f"{what}: {m}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 1, 7, 100, 128, 129, 300])
@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 16, 8), (3, 1, 32, 16), (12, 2, 128, 64), (6, 3, 80, 16), (5, 5, 48, 5), (9, 3, 112, 12)])
def test_heads_that_mix_their_weights_over_windows(dtype, n_q, n_kv, hd, page_size, window):
    """Portions beside decoded tokens, after contexts that end inside and at the borders of pages, tiles and ranges."""
    case = _talking_case(dtype, n_q, n_kv, hd, page_size, [0, 131, 300, 17, 255], [40, 1, 3, 1, 2], window, seed=hd + (window or 0))
    _check_talking(dtype, case, window, f"{n_q} heads on {n_kv} of {hd}, pages of {page_size}, window {window}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 1, 100, 129, 300])
@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 16, 8), (12, 2, 128, 64), (6, 3, 80, 16), (5, 5, 48, 5)])
def test_long_portions_beside_short_ones(dtype, n_q, n_kv, hd, page_size, window):
    """Portions of some hundred tokens (in bfloat16 their scores and weighted values are matrix products on gathered
    keys and values) beside a decoded token and a short portion, which go through the table of the step's scores."""
    case = _talking_case(dtype, n_q, n_kv, hd, page_size, [0, 131, 70, 300], [200, 1, 1300, 9], window, seed=hd + (window or 0) + 1)
    _check_talking(dtype, case, window, f"long portions: {n_q} heads on {n_kv} of {hd}, pages of {page_size}, window {window}")
    alone = _talking_case(dtype, n_q, n_kv, hd, page_size, [70], [1300], window, seed=3)
    _check_talking(dtype, alone, window, "a long portion alone")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("portion", [1, 7, 200])
@pytest.mark.parametrize("window,page_size", [(64, 16), (40, 8), (33, 32), (2, 16), (128, 16), (129, 8), (257, 16)])
def test_a_loud_key_at_a_window_s_edges_with_mixed_heads(dtype, window, page_size, portion):
    """The last query's first key inside its window answers it loudly, then the key one place before: the first must
    carry the result, the second must not be seen, whichever kernel range and tile it lies in; the query a decoded
    token, the last token of a short portion, and of a long one (whose scores are a matrix product in bfloat16)."""
    last = 3 * window + 5 + 200  # the last query's position
    olds, news = [last + 1 - portion, 9], [portion, 4]
    inside = _talking_case(dtype, 4, 2, 32, page_size, olds, news, window, seed=3, loud=[(0, last - (window - 1))])
    _check_talking(dtype, inside, window, f"loud key at the window's first place, window {window}")
    outside = _talking_case(dtype, 4, 2, 32, page_size, olds, news, window, seed=3, loud=[(0, last - window)])
    _check_talking(dtype, outside, window, f"loud key one place before the window, window {window}")
    quiet = _talking_case(dtype, 4, 2, 32, page_size, olds, news, window, seed=3)
    # the key outside changes nothing in the last query's row; the key inside changes it
    assert torch.equal(outside[-1][portion - 1], quiet[-1][portion - 1])
    assert (inside[-1][portion - 1] - quiet[-1][portion - 1]).abs().max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_loud_key_far_back_among_thousands(dtype):
    """No window: the key ranges of a token are many, and a loud key in the first of them decides the token."""
    case = _talking_case(dtype, 6, 2, 64, 16, [2900, 700], [1, 30], None, seed=8, loud=[(0, 3), (1, 129)])
    quiet = _talking_case(dtype, 6, 2, 64, 16, [2900, 700], [1, 30], None, seed=8)
    assert (case[-1][0] - quiet[-1][0]).abs().max() > 0.1
    _check_talking(dtype, case, None, "loud keys thousands of places back")


def test_a_sink_larger_than_every_score_and_no_mixing():
    case = _talking_case(torch.float32, 4, 2, 32, 8, [50, 0], [2, 9], 20, seed=5, sink_scale=30.0, talk=False)
    _check_talking(torch.float32, case, 20, "large sinks, no mixing")


def test_a_missing_page_inside_a_window_gives_nan_and_outside_it_nothing():
    from cwm_amd import ops

    q, cache, table, batch, scale, sink, mix, want = _talking_case(torch.float32, 2, 1, 16, 8, [100], [1], 30, seed=2)
    gone = table.clone()
    gone[0, 0:8] = -1  # keys 0..63: before the window of the query at 100 (71..100)
    got = ops.talking_attention(q, cache, gone, batch, 30, scale, sink=sink, talk=mix).cpu()
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=2e-5)
    gone[0, 10] = -1  # keys 80..87
    assert torch.isnan(ops.talking_attention(q, cache, gone, batch, 30, scale, sink=sink, talk=mix)).any()


# ---- gated linear attention ----------------------------------------------------------------------------------------- #
class LinearCase:
    """Inputs of one gated linear attention for sequences of given lengths, the kernel's arguments for any cut of the
    sequences into steps, and the plain implementation's results."""

    def __init__(self, heads, d, e, tau, lengths, dtype, seed, logit_shift=1.0):
        self.heads, self.d, self.e, self.tau, self.lengths, self.dtype, self.eps = heads, d, e, tau, lengths, dtype, 1e-6
        self.proj = [rnd((n, 2 * heads * (d + e) + 3), seed + i).to(dtype) for i, n in enumerate(lengths)]  # three more columns: another projection rides along
        self.z = [rnd((n, heads * d), seed + 50 + i, 2.0) + logit_shift for i, n in enumerate(lengths)]
        self.weight = rnd((e,), seed + 99).abs() + 0.5

    def reference(self):
        out = []
        h, d, e = self.heads, self.d, self.e
        for p, z in zip(self.proj, self.z):
            p = p.double()
            n = p.shape[0]
            q = p[:, : h * d].reshape(n, h, d) * d ** -0.5
            k = p[:, h * d : 2 * h * d].reshape(n, h, d)
            v = p[:, 2 * h * d : 2 * h * d + h * e].reshape(n, h, e)
            g = p[:, 2 * h * d + h * e : 2 * h * (d + e)].reshape(n, h, e)
            alpha = (torch.sigmoid(z.double()) ** (1.0 / self.tau)).reshape(n, h, d)
            o, state = gp.gla_recurrence(q, k, v, alpha)
            out.append(((gp.unit_rms(o, self.eps) * self.weight.double() * gp.silu(g)).reshape(n, h * e), state))
        return out

    def run(self, steps, slots, n_slots=None):
        """`steps`: lists of (sequence, first token, end) that run together; returns the rows by sequence and the state tensor."""
        from cwm_amd import ops

        state = torch.zeros((n_slots or len(self.lengths), ops.gla_state_elems(self.heads, self.d, self.e)), dtype=torch.float32, device=DEV)
        got = [torch.zeros((n, self.heads * self.e)) for n in self.lengths]
        for step in steps:
            batch = step_batch([a for _, a, _ in step], [b - a for _, a, b in step], [slots[s] for s, _, _ in step])
            proj = torch.cat([self.proj[s][a:b] for s, a, b in step]).to(DEV)
            z = torch.cat([self.z[s][a:b] for s, a, b in step]).to(DEV)
            y = ops.gated_linear_attention(proj, z, self.weight.to(DEV), state, batch, self.heads, self.d, self.e, self.tau, self.eps).cpu().float()
            row = 0
            for s, a, b in step:
                got[s][a:b] = y[row : row + b - a]
                row += b - a
        return got, state


def cut(lengths, sizes):
    """Steps that take the sequences side by side in portions of the given sizes (cycled, each sequence from another place)."""
    cursor = [0] * len(lengths)
    steps, k = [], 0
    while any(c < n for c, n in zip(cursor, lengths)):
        step = []
        for s, n in enumerate(lengths):
            if cursor[s] < n:
                size = min(sizes[(k + s) % len(sizes)], n - cursor[s])
                step.append((s, cursor[s], cursor[s] + size))
                cursor[s] += size
        steps.append(step)
        k += 1
    return steps


LINEAR_SIZES = [(4, 32, 24), (2, 96, 40), (3, 10, 14), (1, 130, 300), (2, 256, 64), (5, 33, 7), (1, 1, 1)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,d,e", LINEAR_SIZES)
def test_gated_linear_attention_in_any_portions(dtype, heads, d, e):
    """Whole sequences, portions down to one and two tokens, and one token a step give the plain implementation's rows
    and the same bits as each other; states live in slots of any order."""
    from cwm_amd import ops

    lengths = [37, 5, 64]
    case = LinearCase(heads, d, e, 12.0, lengths, dtype, seed=heads * 100 + d)
    want = case.reference()
    t = dict(rtol=2e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    slots = [2, 0, 3]
    whole, state = case.run([[(s, 0, n) for s, n in enumerate(lengths)]], slots, n_slots=4)
    parts, _ = case.run(cut(lengths, [16, 7, 2, 5, 1, 3]), slots, n_slots=4)
    for s in range(len(lengths)):
        torch.testing.assert_close(whole[s].double(), want[s][0], **t)
        assert torch.equal(whole[s], parts[s]), "a cut of the sequence changed the bits"
        unpacked = ops.gla_state_unpack(state[slots[s]].cpu(), heads, d, e)
        torch.testing.assert_close(unpacked.double(), want[s][1], rtol=2e-4, atol=2e-5)
    assert torch.count_nonzero(state[1]) == 0, "a slot that no sequence of the steps names was written"


@pytest.mark.parametrize("tau,shift", [(1.0, -2.0), (64.0, 3.0)])
def test_gated_linear_attention_with_fast_and_with_slow_decays(tau, shift):
    """Decays near zero forget within a token or two; decays near one keep a loud first token over hundreds of tokens."""
    case = LinearCase(2, 24, 16, tau, [400], torch.float32, seed=7, logit_shift=shift)
    case.proj[0][0, 2 * 24 : 4 * 24] *= 8.0  # the first token's keys
    want = case.reference()
    got, _ = case.run(cut([400], [130, 2, 1, 67]), [0])
    torch.testing.assert_close(got[0].double(), want[0][0], rtol=5e-4, atol=5e-5)


@pytest.mark.parametrize("heads,d,e", [(4, 32, 24), (2, 96, 40), (1, 130, 300)])
def test_long_portions_of_linear_attention_in_segments_side_by_side(heads, d, e):
    """bfloat16 portions of more than a segment run in segments whose states are carried across: the plain
    implementation's rows, the walk's rows but for rounding, and the same state in the slot; a short sequence beside
    the long ones, and a second step that goes on from the states the first left."""
    from cwm_amd import ops

    lengths = [700, 3, 1000]
    case = LinearCase(heads, d, e, 12.0, lengths, torch.bfloat16, seed=heads + d, logit_shift=2.0)
    want = case.reference()
    slots = [1, 3, 0]
    segmented, state = case.run([[(0, 0, 300), (1, 0, 3), (2, 0, 513)], [(0, 300, 700), (2, 513, 1000)]], slots, n_slots=4)
    walked, walked_state = case.run(cut(lengths, [200, 256, 100]), slots, n_slots=4)
    for s in range(len(lengths)):
        torch.testing.assert_close(segmented[s].double(), want[s][0], rtol=3e-2, atol=3e-2)
        torch.testing.assert_close(segmented[s], walked[s], rtol=2e-2, atol=2e-2)
        unpacked = ops.gla_state_unpack(state[slots[s]].cpu(), heads, d, e)
        torch.testing.assert_close(unpacked.double(), want[s][1], rtol=2e-4, atol=2e-4)
    torch.testing.assert_close(state, walked_state, rtol=2e-4, atol=2e-4)


# ---- input convolutions, token input, gated activations ------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,dim", [(3, 192), (1, 40), (4, 300), (2, 7), (16, 64)])
def test_input_convolutions_carry_their_last_inputs(dtype, taps, dim):
    """Two convolutions of one input; sequences in portions shorter and longer than the taps, in slots of any order."""
    from cwm_amd import ops

    lengths = [23, 5, 40]
    x = [rnd((n, dim), 3 + i).to(dtype) for i, n in enumerate(lengths)]
    w = [rnd((dim, taps), 11), rnd((dim, taps), 12)]
    want = [[xs.double() + gp.causal_conv(xs.double(), wi.double()) for wi in w] for xs in x]
    state = torch.zeros((4, max(1, (taps - 1) * dim)), dtype=torch.float32, device=DEV)
    slots = [3, 1, 0]
    got = [[torch.zeros((n, dim)) for _ in w] for n in lengths]
    by_tap = [wi.t().contiguous().to(DEV) for wi in w]
    for step in cut(lengths, [1, 2, 7, 1, 1, 3, 16]):
        batch = step_batch([a for _, a, _ in step], [b - a for _, a, b in step], [slots[s] for s, _, _ in step])
        outs = ops.short_conv(torch.cat([x[s][a:b] for s, a, b in step]).to(DEV), by_tap, state if taps > 1 else None, batch)
        row = 0
        for s, a, b in step:
            for i in range(2):
                got[s][i][a:b] = outs[i][row : row + b - a].cpu().float()
            row += b - a
    t = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for s in range(len(lengths)):
        for i in range(2):
            torch.testing.assert_close(got[s][i].double(), want[s][i], **t)
    if taps > 1:
        for s, n in enumerate(lengths):
            last = torch.cat([torch.zeros((taps - 1, dim)), x[s].float()])[n:]  # nothing precedes a sequence's first token
            torch.testing.assert_close(state[slots[s], : (taps - 1) * dim].cpu().reshape(taps - 1, dim), last)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,side,layers", [(192, 12, 5), (100, 5, 3), (1024, 32, 2), (40, 1, 7)])
def test_a_layer_s_own_token_input(dtype, dim, side, layers):
    from cwm_amd import ops

    n, vocab, index = 9, 50, layers - 2
    h = rnd((n, dim), 1, 2.0)
    tokens = torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    w = {"gate": rnd((side, dim), 3, dim ** -0.5).to(dtype), "proj": rnd((dim, side), 4).to(dtype), "norm": rnd((dim,), 5).abs() + 0.3}
    table = rnd((vocab, layers * side), 6).to(dtype)
    rows = table[tokens.long(), index * side : (index + 1) * side].double()
    want = h.double() + gp.token_side({k: v.double() for k, v in w.items()}, "", h.double(), rows, 1e-6, rounded=dtype == torch.bfloat16)
    got = h.clone().to(DEV)
    ops.token_side(got, tokens.to(DEV), table.to(DEV), index * side, w["gate"].to(DEV), w["proj"].t().contiguous().to(DEV), w["norm"].to(DEV), 1e-6, dtype == torch.bfloat16)
    # in bfloat16 a gate's sum in another order may round to the neighbouring value, which the norm of few side values magnifies
    t = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(got.cpu().double(), want, **t)
    # with the sublayers' results still to be added: the same bits as the sum by the layer norm's kernel and the input after it
    pending = ops.ScaledSum([(rnd((3, n, dim), 7).to(DEV), 1.0), (rnd((n, dim), 8).to(dtype).to(DEV), 0.5)])
    args = (tokens.to(DEV), table.to(DEV), index * side, w["gate"].to(DEV), w["proj"].t().contiguous().to(DEV), w["norm"].to(DEV), 1e-6, dtype == torch.bfloat16)
    two = h.clone().to(DEV)
    ops.add_layernorm(two, pending, None, None, 1.0, dtype)
    ops.token_side(two, *args)
    one = h.clone().to(DEV)
    ops.token_side(one, *args, pending=pending)
    assert torch.equal(one, two)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_activations_on_rows(dtype):
    from cwm_amd import ops

    hidden, n = 48, 9
    x = (rnd((n, 2 * hidden + 1), 1, 3.0)).to(dtype)
    g, u, r = x[:, :hidden].double(), x[:, hidden : 2 * hidden].double(), x[:, 2 * hidden :].double()
    t = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    clamped = torch.clamp(g, max=2.0) * torch.sigmoid(1.702 * torch.clamp(g, max=2.0)) * (torch.clamp(u, -2.0, 2.0) + 1.0)
    torch.testing.assert_close(ops.gated_act_rows(x.to(DEV), hidden, ops.GatedActivation("clamped_swish", 1.702, 2.0), dtype).cpu().double(), clamped, **t)
    gated = gp.silu(g) * u * torch.sigmoid(r)
    torch.testing.assert_close(ops.gated_act_rows(x.to(DEV), hidden, ops.GatedActivation("silu"), dtype, 2 * hidden).cpu().double(), gated, **t)
    parts = rnd((3, n, 2 * hidden + 1), 2)
    total = parts.double().sum(0)
    want = gp.silu(total[:, :hidden]) * total[:, hidden : 2 * hidden] * torch.sigmoid(total[:, 2 * hidden :])
    torch.testing.assert_close(ops.gated_act_rows(parts.to(DEV), hidden, ops.GatedActivation("silu"), torch.float32, 2 * hidden).cpu().double(), want, rtol=1e-5, atol=1e-5)


# ---- models ---------------------------------------------------------------------------------------------------------- #
LENGTHS = {"tiny_g": [40, 75, 33, 64, 9], "tiny_h": [33, 64, 50, 7], "tiny_i": [130, 20, 66]}
PAGE_SIZES = {"whole": 16, "tail": 8, "portions": 16, "mixed": 8}


def requests_for(name, lengths=None):
    vocab = digasun.get(name)["vocab"]
    return {f"r{i}": traces.random_tokens(17 * i + len(name), n, vocab) for i, n in enumerate(lengths or LENGTHS[name])}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("digasun")
    return {name: digasun.make_folder(root, name, seed=5) for name in digasun.ALL}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def plain_for(folders, cache, name, dtype):
    if (name, dtype) not in cache:
        cache[name, dtype] = digasun.expected(folders[name], requests_for(name), dtype, conditioning=True)
    return cache[name, dtype]


def run(folder, dtype, steps, requests, vocab, **options):
    from cwm_amd.replay import Replayer

    rep = Replayer(folder, dtype, traces.max_live_tokens(steps), poison_freed_pages=True, **options)
    page_use = traces.PageUse(rep.manager)
    outputs = traces.run_in_process(rep, steps, page_use)
    assert rep.manager.live_requests() == []
    return traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab), rep, page_use


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(digasun.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_replay_regimes(folders, plain_cache, name, dtype, regime):
    requests = requests_for(name)
    vocab = digasun.get(name)["vocab"]
    steps = {"whole": traces.whole, "tail": traces.tail_one_by_one, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=3)}[regime](requests)
    got, rep, page_use = run(folders[name], dtype, steps, requests, vocab, page_size=PAGE_SIZES[regime], max_requests=3 if regime == "mixed" else 16)
    want = plain_for(folders, plain_cache, name, dtype)
    digasun.check_together(got, want, dtype, f"{name} {dtype} {regime}")
    if regime == "mixed":
        for g in rep.manager.groups:
            assert page_use.pages_shared_between_requests(g.index) > 0, f"group {g.index}: no page served two requests"


A, G, D, M = digasun.attention, digasun.gla, digasun.dense, digasun.moe
SINGLE_LAYERS = {
    "attention_window_rotation": dict(layers=[A(4, 2, 12, 10, 0.3, mask=9, rot=(100.0, 8))]),
    "attention_without_rotation_mask_convolution_or_token_input": dict(layers=[A(3, 3, 8, 16, 0.4)], taps=None, side=None),
    "attention_whole_head_rotated": dict(layers=[A(2, 1, 16, 8, 0.25, mask=40, rot=(1000.0, 16), mlp=D(24, 1.0))]),
    "attention_rotation_of_two_elements": dict(layers=[A(2, 2, 6, 6, 0.5, mask=3, rot=(50.0, 2))], taps=5),
    "keys_and_values_of_the_first_layer": dict(layers=[A(4, 2, 12, 10, 0.3, mask=9, rot=(100.0, 4)), A(2, 2, 12, 10, 0.5, mask=5, rot=(100.0, 4), kv_from=0)]),
    "two_readers_with_longer_windows_than_the_writer": dict(
        layers=[G(2, 8, 8, 4.0), A(2, 1, 8, 6, 0.3, mask=4), A(3, 1, 8, 6, 0.3, mask=21, kv_from=1), G(1, 4, 4, 2.0), A(1, 1, 8, 6, 0.3, mask=12, kv_from=1)], taps=2),
    "a_reader_that_sees_every_key": dict(layers=[A(2, 2, 8, 8, 0.3, mask=6), A(4, 2, 8, 8, 0.3, kv_from=0)]),
    "linear_attention_alone": dict(layers=[G(3, 10, 14, 8.0)], side=None),
    "linear_attention_with_one_tap": dict(layers=[G(2, 18, 9, 2.0, mlp=D(16, 0.5))], taps=1),
    "experts_with_a_shared_one": dict(layers=[A(1, 1, 8, 8, 0.1, mask=2, mlp=M(5, 2, 24, shared=16))]),
    "all_experts_chosen": dict(layers=[G(1, 4, 4, 1.0, mlp=M(3, 3, 20))]),
    "one_expert_of_many": dict(layers=[A(1, 1, 8, 8, 0.1, mlp=M(9, 1, 12, shared=5))], side=2),
    "feed_forward_carries_the_layer": dict(layers=[A(1, 1, 8, 8, 0.1, mlp=D(64, 0.7))]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", list(SINGLE_LAYERS))
def test_single_layers(tmp_path, which, dtype):
    """One mechanism at a time between embedding and head: whole prompts against the same tokens in portions and one
    by one, and all against the plain implementation."""
    config = digasun.model_of(**SINGLE_LAYERS[which])
    folder = digasun.make_folder(tmp_path, which[:40], seed=2, config=config)
    requests = {f"r{i}": traces.random_tokens(i + 5, n, config["vocab"]) for i, n in enumerate([37, 5, 64])}
    want = digasun.expected(folder, requests, dtype)
    for make in (traces.whole, traces.portions, lambda r: traces.tail_one_by_one(r, tail=20)):
        steps = make(requests)
        got, _, _ = run(folder, dtype, steps, requests, config["vocab"], page_size=8)
        digasun.check_together(got, want, dtype, f"{which} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_and_slow_decays_over_long_sequences(folders, dtype):
    """tiny_h's softmax is sharp and one of its states forgets slowly: a token's result hangs on single keys at a
    window's edge and on what the state took in at the sequence's start.  A prompt of 700 tokens whole, in portions
    that end at, before and after page and window borders (down to one and two tokens), and with its last 150 tokens
    one by one."""
    name = "tiny_h"
    vocab = digasun.get(name)["vocab"]
    requests = {"long": traces.random_tokens(99, 700, vocab)}
    want = digasun.expected(folders[name], requests, dtype, conditioning=True)
    portions = lambda r: traces.portions(r, sizes=[64, 63, 65, 2, 126, 1, 31, 33, 128, 17, 11, 5, 16])  # noqa: E731
    for make in (traces.whole, portions, lambda r: traces.tail_one_by_one(r, tail=150)):
        steps = make(requests)
        got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=32)
        digasun.check(got["long"], want["long"], dtype, f"{name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_layers_and_many_rows(tmp_path, dtype):
    """Width 256 and prompts of 600 and 300 tokens: the kernels' shapes for many rows, whole, in large portions beside
    each other, and with a tail of single tokens."""
    config = digasun.MEDIUM
    folder = digasun.make_folder(tmp_path, "medium", seed=9, config=config)
    vocab = config["vocab"]
    requests = {"a": traces.random_tokens(31, 600, vocab), "b": traces.random_tokens(32, 300, vocab)}
    want = digasun.expected(folder, requests, dtype)
    side_by_side = [
        {"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:290], "want": list(range(290))}, {"id": "b", "tokens": requests["b"][:270], "want": list(range(270))}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": requests["a"][290:], "want": list(range(310))}, {"id": "b", "tokens": requests["b"][270:], "want": list(range(30))}], "end": ["a", "b"]},
    ]
    for steps in (traces.whole(requests), side_by_side, traces.tail_one_by_one(requests, tail=20)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=32)
        digasun.check_together(got, want, dtype, f"medium {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, dtype):
    """Every token a step of its own from an empty cache and a zero state, for 300 steps: windows pass over decoded
    tokens many times."""
    name = "tiny_g"
    vocab = digasun.get(name)["vocab"]
    requests = {"a": traces.random_tokens(4, 300, vocab)}
    steps = traces.tail_one_by_one(requests, tail=299)
    got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=16)
    digasun.check(got["a"], digasun.expected(folders[name], requests, dtype, conditioning=True)["a"], dtype, f"{name} {dtype} one by one")


def test_pages_and_state_slots_that_are_used_again_start_afresh(folders):
    """One slot and a pool of the longer request's size only: the second request finds the first one's states and
    cache rows (NaN in the pages in between) and must not read them."""
    name = "tiny_i"
    vocab = digasun.get(name)["vocab"]
    a, b = traces.random_tokens(1, 60, vocab), traces.random_tokens(2, 25, vocab)
    both = [
        {"step": 0, "entries": [{"id": "a", "tokens": a, "want": [59]}], "end": ["a"]},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:10], "want": list(range(10))}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[10:], "want": list(range(15))}], "end": ["b"]},
    ]
    got, rep, _ = run(folders[name], "float32", both, {"a": a, "b": b}, vocab, page_size=8, max_requests=1)
    alone, _, _ = run(folders[name], "float32", both[1:], {"b": b}, vocab, page_size=8, max_requests=1)
    assert np.array_equal(got["b"], alone["b"])
    digasun.check(got["b"], digasun.expected(folders[name], {"b": b}, "float32")["b"], "float32", "second user of the slot")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_do_not_depend_on_the_rest_of_the_batch(folders, dtype):
    """A request's decoded tokens alone and beside two other requests' short portions: the same bits."""
    name = "tiny_g"
    vocab = digasun.get(name)["vocab"]
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
    name = "tiny_h"
    vocab = digasun.get(name)["vocab"]
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


@pytest.mark.parametrize("name", ["tiny_g", "tiny_i"])
def test_greedy_generation_through_the_engine(folders, name):
    """The engine's own entry point: scheduler, portions of 24 tokens, continuous batching, sampling kernel; then a
    cache that holds barely more than the longest request, so that requests wait for one another's pages and slots."""
    from cwm_amd.engine import Engine, GenArgs

    vocab = digasun.get(name)["vocab"]
    prompts = [traces.random_tokens(20 + i, n, vocab) for i, n in enumerate([5, 17, 33, 64])]
    engine = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=2048, cache_block=16, max_prefill=24), dtype="float32")
    got = engine.generate_tokens(prompts, max_gen=12)
    for p, g in zip(prompts, got):
        assert g == digasun.plain_greedy(folders[name], p, 12)
    small = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=96, cache_block=4, max_prefill=24), dtype="float32")
    assert small.generate_tokens(prompts, max_gen=12) == got


def test_command_line_and_trace_run_as_child_processes(folders, tmp_path):
    name = "tiny_g"
    vocab = digasun.get(name)["vocab"]
    prompts = [traces.random_tokens(60 + i, n, vocab) for i, n in enumerate([6, 21])]
    path = tmp_path / "prompts.jsonl"
    path.write_text("".join(json.dumps({"id": i, "tokens": p}) + "\n" for i, p in enumerate(prompts)))
    cmd = [sys.executable, "-m", "cwm_amd.generate", f"checkpoint_dir={folders[name]}", f"prompts={path}", "dtype=float32",
           "gen_args.use_sampling=false", "gen_args.max_gen=7", "gen_args.max_seq=512", "gen_args.cache_block=16", "gen_args.max_batch=4"]
    res = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = {rec["id"]: rec["tokens"] for rec in map(json.loads, res.stdout.strip().splitlines())}
    for i, p in enumerate(prompts):
        assert got[i] == digasun.plain_greedy(folders[name], p, 7)

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
        want = digasun.expected(folders[name], requests, dtype)
        digasun.check_together(got, want, dtype, f"trace_run {dtype}")


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: every size, count, constant and the order of layers differ from draw to draw."""
    import random

    rng = random.Random(seed)
    width = rng.choice([32, 40, 48, 64, 72, 96, 100, 128, 136, 192, 200, 256])
    layers, writers = [], []
    for i in range(rng.randint(2, 6)):
        kind = rng.random()
        if kind < 0.25:
            mlp = None
        elif kind < 0.5:
            mlp = D(rng.choice([20, 36, 64, 100, 256]), rng.choice([0.5, 1.0, 2.0, 7.0]))
        else:
            experts = rng.randint(1, 9)
            mlp = M(experts, rng.randint(1, experts), rng.choice([8, 20, 36, 64, 96]), shared=rng.choice([None, 8, 24, 96]))
        if rng.random() < 0.3:
            layers.append(G(rng.randint(1, 5), rng.choice([4, 8, 12, 16, 24, 32, 48, 64, 100]), rng.choice([4, 8, 16, 33, 48, 64, 80]), rng.choice([1.0, 4.0, 12.0, 64.0]), mlp=mlp))
            continue
        mask = rng.choice([None, 1, 2, 7, 16, 17, 40, 64, 100, 129])
        if writers and rng.random() < 0.4:
            src = rng.choice(writers)
            m = layers[src]["mixer"]
            rot = (m["rot"]["base"], m["rot"]["dims"]) if "rot" in m else None
            layers.append(A(m["kv_heads"] * rng.choice([1, 2, 3, 4]), m["kv_heads"], m["dim"], m["vdim"], m["scale"], mask=mask, rot=rot, kv_from=src, mlp=mlp))
            continue
        kv = rng.choice([1, 2, 3, 4])
        dim = rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 128])
        rot = None
        if rng.random() < 0.8:
            rot = (rng.choice([100.0, 10000.0, 50000.0, 1e6]), rng.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim] + [dim]))
        layers.append(A(kv * rng.choice([1, 2, 3, 4]), kv, dim, rng.choice([8, 12, 16, 32, 48, 64, 80, 128]), rng.choice([0.05, 0.1, 0.2]) * (64 / dim) ** 0.5, mask=mask, rot=rot, mlp=mlp))
        writers.append(i)
    return digasun.model_of(layers, width=width, vocab=rng.randint(50, 700), eps=rng.choice([1e-5, 1e-6]), scale=rng.choice([None, 0.5, 3.0, 11.0]),
                            taps=rng.choice([None, 1, 2, 3, 4, 7]), side=rng.choice([None, 2, 3, 12, 40]))  # one side value alone makes the input a sign, which hangs on the last bits


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed, dtype):
    """Other models of the design: whole prompts, and a mixed schedule with pages of another size, against the plain
    implementation."""
    config = random_config(seed)
    folder = digasun.make_folder(tmp_path, f"random{seed}", seed=seed, config=config)
    vocab = config["vocab"]
    requests = {f"r{i}": traces.random_tokens(7 * seed + i, n, vocab) for i, n in enumerate([3, 150, 45, 88])}
    want = digasun.expected(folder, requests, dtype, conditioning=True, drop_after_close_calls=True)
    for steps, page in ((traces.whole(requests), 16), (traces.mixed(requests, max_live=3), 32 if seed % 2 else 8)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=page, max_requests=4)
        digasun.check_together(got, want, dtype, f"random configuration {seed} {dtype}: {json.dumps(config)}")
