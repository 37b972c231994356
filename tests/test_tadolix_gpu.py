"""Tadolix on the GPU: every kernel of its parts alone against the plain implementation's function of the same
mechanism (float32 and bfloat16), the recurrences over steps cut anywhere in slots that others left full,
attention with a key made to stand out far away, at page borders, at the first token and just inside and outside
a chunk, the engine under every way of cutting, recorded decoding, generation through the entry point and the
scheduler, the replay program and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_tadolix as P
import tadolix_cases as tc
import schedules
from test_tadolix_cpu import TOL, _expected, _greedy, step_through
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.batch import build_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [("float32", torch.float32, 5e-6), ("bfloat16", torch.bfloat16, 1.2e-2)]
F64 = torch.float64


def _ops(dtype):
    from transformers_neuronx_amd.kernels import make_ops
    return make_ops("hip", dtype, DEV)


def _ctx(runs, cached, slots, tables=None, page_size=16, planners=None):
    entries = [StepEntry(i, [0] * n, []) for i, n in enumerate(runs)]
    tables = tables if tables is not None else {}
    return build_context(entries, cached, slots, {k: np.asarray(v, dtype=np.int32) for k, v in tables.items()},
                         page_size, DEV, planners)


def _close(got, want, tol, scale=None):
    """`scale`: what the difference is measured by, where `want` is a few numbers of many (the largest of all)."""
    want = want.to(F64)
    scale = float(want.abs().max()) if scale is None else float(scale)
    err = float((got.double().cpu() - want).abs().max() / max(1e-30, scale))
    assert err < tol, err


# steps of a request in slot 2 and, from the third step on, of another in slot 0: (request, from, to, slot)
def _steps(cuts0=(0, 1, 2, 4, 5, 6, 30, 32, 45, 345, 346, 602, 611), cuts1=(None, None, 0, 1, 2, 9, 11, 12, None, None, None, None, None)):
    for s in range(len(cuts0) - 1):
        step = [(0, cuts0[s], cuts0[s + 1], 2)]
        if cuts1[s] is not None and cuts1[s + 1] is not None:
            step.append((1, cuts1[s], cuts1[s + 1], 0))
        yield step


# ---------------------------------------------------------------- each mechanism alone

@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [(1, 2), (9, 50), (70, 128), (33, 600)])
def test_positions_by_sine_and_cosine(name, dtype, tol, sizes):
    t, width = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(1)
    src = torch.randn(t, width, generator=g).to(dtype)
    first = 1000
    positions = torch.arange(first, first + t, dtype=torch.int32)
    freqs = torch.tensor([10000.0 ** (-2.0 * i / width) for i in range(width // 2)], dtype=torch.float32)
    x, xc = ops.add_sinusoid(src.to(DEV), positions.to(DEV), freqs.to(DEV), dtype, True, scale=3.5)
    want = src.double() * 3.5 + P.sinusoid(first + t, width)[first:]
    # the angle is a float32 product: at position p its error is p times a float32 rounding
    _close(x, want, 2e-4)
    _close(xc, want, max(tol, 2e-4))


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [(1, 1, 8), (2, 5, 50), (3, 40, 96), (4, 17, 256), (6, 3, 1000)])
def test_copies_of_the_stream_are_joined_read_and_summed(name, dtype, tol, sizes):
    s, t, width = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(2)
    copies = torch.randn(s, t, width, generator=g)
    y = torch.randn(t, width, generator=g)
    mix = torch.eye(s) * 0.7 + torch.randn(s, s, generator=g) * 0.3
    out_w, read = torch.randn(s, generator=g), torch.randn(s, generator=g)
    nw = torch.randn(width, generator=g) * 0.3
    eps = 1e-3
    joined = P.hyper([c.double() for c in copies], y.double(), mix.double(), out_w.double())
    want_h = P.offset_norm(sum(read[a].double() * joined[a] for a in range(s)), nw.double(), eps)
    dev = copies.to(DEV)
    h32, hc = ops.hyper_step(dev, (y.to(DEV), mix.to(DEV), out_w.to(DEV)), read.to(DEV), (1.0 + nw).to(DEV), eps,
                             dtype, True, True)
    _close(dev, torch.stack(joined), 5e-6)            # joined in place, float32 whatever the compute dtype
    _close(h32, want_h, 5e-6)
    _close(hc, want_h, tol)
    # without anything pending the copies stay as they are
    before = dev.clone()
    h32b, _ = ops.hyper_step(dev, None, read.to(DEV), (1.0 + nw).to(DEV), eps, dtype, True, False)
    assert torch.equal(dev, before)
    _close(h32b, want_h, 5e-6)
    total = ops.hyper_sum(dev, (y.to(DEV), mix.to(DEV), out_w.to(DEV)))
    twice = P.hyper(joined, y.double(), mix.double(), out_w.double())
    _close(total, sum(twice), 5e-6)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("inner", [1, 24, 100, 256, 1030])
def test_minimal_gated_recurrence_across_steps_cut_anywhere(name, dtype, tol, inner):
    """Steps of 1, 2 and more tokens, two requests side by side in slots that former holders left full, every
    step of single tokens run twice (a recorded step is), against the whole sequence at once."""
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(4)
    lens = {0: 611, 1: 12}
    proj = {r: torch.randn(t, 3 * inner, generator=g) * 2.5 for r, t in lens.items()}
    eye, zero = torch.eye(3 * inner, dtype=F64), torch.zeros(inner, dtype=F64)
    # the plain function takes a mixer's input and its matrices: identity matrices hand it the projections
    w = {"p.z": eye[:inner], "p.x": eye[inner:2 * inner], "p.g": eye[2 * inner:], "p.z.b": zero, "p.x.b": zero,
         "p.o": torch.eye(inner, dtype=F64)}
    want = {r: P.min_gru(w, "p.", proj[r].double()) * 0.7 for r in lens}
    carried = torch.full((3, 2, inner), 3.0, device=DEV)
    for step in _steps():
        rows = torch.cat([proj[r][a:b] for r, a, b, _ in step]).to(DEV)
        ctx = _ctx([b - a for _, a, b, _ in step], [a for _, a, _, _ in step], [slot for _, _, _, slot in step])
        single = all(b - a == 1 for _, a, b, _ in step)
        # into columns of a wider buffer, as beside another mixer
        both = torch.full((rows.shape[0], inner + 5), 9.0, dtype=dtype, device=DEV)
        for _ in range(2 if single else 1):
            ops.min_gru(rows, inner, ctx, carried, out=both[:, 5:], out_scale=0.7)
        assert float(both[:, :5].float().min()) == 9.0
        at = 0
        for r, a, b, _ in step:
            _close(both[at:at + b - a, 5:], want[r][a:b], max(tol, 2e-5), want[r].abs().max())
            at += b - a
    assert float(carried[1].min()) == 3.0       # a slot of no one is not touched


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [(1, 1, 1), (1, 8, 4), (4, 16, 4), (3, 10, 2), (2, 64, 3), (16, 40, 5)])
def test_convolution_and_gated_linear_recurrence_across_steps_cut_anywhere(name, dtype, tol, sizes):
    blocks, each, taps = sizes
    c = blocks * each
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(5)
    lens = {0: 611, 1: 12}
    proj = {r: torch.randn(t, 2 * c, generator=g) * 1.5 for r, t in lens.items()}
    conv_w, conv_b = torch.randn(c, taps, generator=g) * 0.6, torch.randn(c, generator=g) * 0.2
    ra, ri = (torch.randn(blocks, each, each, generator=g) * (2.0 / each ** 0.5) for _ in range(2))
    ra_b, ri_b = torch.randn(blocks, each, generator=g), torch.randn(blocks, each, generator=g)
    lam = torch.rand(c, generator=g) * 7.0 - 6.0            # decays from almost none to at once
    eye, zero = torch.eye(2 * c, dtype=F64), torch.zeros(c, dtype=F64)
    w = {"p.y": eye[:c], "p.x": eye[c:], "p.y.b": zero, "p.x.b": zero, "p.conv": conv_w.double(), "p.conv.b": conv_b.double(),
         "p.ra": ra.double(), "p.ri": ri.double(), "p.ra.b": ra_b.double(), "p.ri.b": ri_b.double(), "p.lam": lam.double(),
         "p.o": torch.eye(c, dtype=F64)}
    m = dict(width=c, blocks=blocks, conv=taps)
    want = {r: P.rglru(m, w, "p.", proj[r].double()) for r in lens}
    want_u = {r: P.causal_conv(proj[r][:, c:].double(), conv_w.double()) + conv_b.double() for r in lens}
    carried = torch.full((3, 2, c), 3.0, device=DEV)
    inputs = torch.full((3, taps, c), -2.0, device=DEV) if taps > 1 else None
    w_gates = torch.cat([ra, ri], dim=1).to(DEV)             # [blocks, 2 each, each]
    b_gates = torch.cat([ra_b, ri_b], dim=1).contiguous().to(DEV)
    rate = (-8.0 * torch.nn.functional.softplus(lam)).to(DEV)
    for step in _steps():
        rows = torch.cat([proj[r][a:b] for r, a, b, _ in step]).to(DEV)
        ctx = _ctx([b - a for _, a, b, _ in step], [a for _, a, _, _ in step], [slot for _, _, _, slot in step])
        single = all(b - a == 1 for _, a, b, _ in step)
        for _ in range(2 if single else 1):
            u, _ = ops.channel_conv(rows[:, c:], conv_w.to(DEV), conv_b.to(DEV), ctx, inputs)
            gates = torch.einsum("tbi,boi->tbo", u.view(-1, blocks, each), w_gates).contiguous()
            got = ops.gated_linear_recurrence(gates, b_gates, u, rows[:, :c], rate, ctx, carried)
        at = 0
        for r, a, b, _ in step:
            _close(u[at:at + b - a], want_u[r][a:b], 5e-6, want_u[r].abs().max())
            _close(got[at:at + b - a], want[r][a:b], max(tol, 3e-5), want[r].abs().max())
            at += b - a
    assert float(carried[1].min()) == 3.0
    assert inputs is None or float(inputs[1].max()) == -2.0


def _standout(dtype, case, seed):
    """A request of `length` tokens whose last `run` are the step's: a mixer input and identity matrices such that
    for the last query the key `back` tokens before it scores far above the rest in every head (the other keys
    have nothing along the marked direction). Returns the projections of all tokens, the table of biases, the
    plain result for the last `run` queries and the weight the last query gives the marked key (None: unseen)."""
    h, g, n, v, length, run = (case[k] for k in ("h", "g", "n", "v", "length", "run"))
    gen = torch.Generator().manual_seed(seed)
    nq, nk, nv = h * n, g * n, g * v
    total = nq + nk + nv + h * v
    x = torch.randn(length, total, generator=gen)
    x[:, nq + nk:nq + nk + nv] *= 2.0
    mark = torch.randn(n, generator=gen)
    mark = mark / mark.norm()
    standout = length - 1 - case["back"]
    keys = x[:, nq:nq + nk].view(length, g, n)
    keys -= (keys @ mark)[..., None] * mark          # no other key has a part along the mark
    keys[standout] = mark * 3.0
    x[length - 1, :nq].view(h, n)[:] = mark * 2.0
    x = x.to(dtype).float()
    rel = torch.randn(case["rows"], h, generator=gen) * 0.8
    m = dict(heads=h, kv_heads=g, dim=n, vdim=v, scale=case["scale"], bias_max=case["far"], softcap=case.get("cap"),
             mask=dict(size=case["chunk"]) if case.get("chunk") else None)
    eye = torch.eye(total, dtype=F64)
    w = {"p.q": eye[:nq], "p.k": eye[nq:nq + nk], "p.v": eye[nq + nk:nq + nk + nv], "p.g": eye[nq + nk + nv:],
         "p.rel": rel.double(), "p.o": torch.eye(h * v, dtype=F64)}
    weights = {}
    want = P.chunk_attention(m, w, "p.", x.double(), case["eps"], range(length - run, length), weights)[length - run:]
    seen = []
    for head in range(h):
        first, a = weights[(head, length - 1)]
        seen.append(float(a[standout - first]) if standout >= first else None)
    return x, rel, want, seen


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("case", [
    # the marked key `back` tokens before the last query; a chunk's first token is position (length - 1) // chunk * chunk
    dict(h=4, g=2, n=16, v=24, chunk=40, length=300, run=1, ps=16, back=19, rows=8, far=40, scale=1.5, cap=40.0),    # the chunk's first token
    dict(h=4, g=2, n=16, v=24, chunk=40, length=300, run=1, ps=16, back=20, rows=8, far=40, scale=1.5, cap=40.0),    # the token before it
    dict(h=2, g=1, n=64, v=64, chunk=None, length=700, run=1, ps=16, back=697, rows=16, far=500, scale=0.4, cap=None),  # far away, no chunks
    dict(h=2, g=2, n=32, v=16, chunk=None, length=700, run=37, ps=16, back=699, rows=6, far=900, scale=0.8, cap=60.0),  # the very first token, in a portion
    dict(h=6, g=3, n=16, v=16, chunk=17, length=64, run=64, ps=16, back=12, rows=4, far=9, scale=1.5, cap=50.0),     # a whole prompt, the chunk's edge
    dict(h=6, g=3, n=16, v=16, chunk=17, length=64, run=64, ps=16, back=13, rows=4, far=9, scale=1.5, cap=50.0),
    dict(h=1, g=1, n=64, v=32, chunk=64, length=129, run=2, ps=64, back=0, rows=32, far=64, scale=0.4, cap=30.0),    # chunks that are pages: a query alone in its chunk
    dict(h=1, g=1, n=64, v=32, chunk=64, length=128, run=2, ps=64, back=63, rows=32, far=64, scale=0.4, cap=30.0),   # and one that sees a whole page
    dict(h=4, g=1, n=16, v=16, chunk=1, length=50, run=3, ps=16, back=0, rows=2, far=5, scale=1.5, cap=None),        # chunks of one token
    dict(h=2, g=2, n=128, v=128, chunk=300, length=280, run=5, ps=16, back=279, rows=9, far=200, scale=0.2, cap=20.0),  # a chunk longer than the request
    dict(h=6, g=2, n=48, v=80, chunk=70, length=390, run=1, ps=64, back=39, rows=16, far=70, scale=0.5, cap=25.0),   # values wider than keys
    dict(h=6, g=2, n=48, v=80, chunk=70, length=390, run=200, ps=64, back=40, rows=16, far=70, scale=0.5, cap=25.0),
    dict(h=8, g=2, n=96, v=64, chunk=256, length=1000, run=300, ps=64, back=231, rows=16, far=256, scale=0.3, cap=30.0),  # a long portion over a chunk's edge
    dict(h=8, g=2, n=96, v=64, chunk=256, length=1000, run=300, ps=64, back=232, rows=16, far=256, scale=0.3, cap=30.0),
    dict(h=4, g=2, n=32, v=32, chunk=100, length=330, run=130, ps=48, back=29, rows=8, far=100, scale=0.8, cap=30.0),    # pages that are no power of two
    dict(h=4, g=2, n=32, v=32, chunk=100, length=330, run=130, ps=48, back=30, rows=8, far=100, scale=0.8, cap=30.0),
    dict(h=2, g=1, n=64, v=64, chunk=None, length=600, run=200, ps=64, back=500, rows=32, far=5000, scale=0.4, cap=None),  # a long bias table
    dict(h=4, g=2, n=160, v=144, chunk=90, length=300, run=140, ps=16, back=29, rows=12, far=90, scale=0.15, cap=35.0),   # heads beyond 128 elements
    dict(h=4, g=2, n=160, v=144, chunk=90, length=300, run=1, ps=64, back=30, rows=12, far=90, scale=0.15, cap=35.0),
    dict(h=3, g=1, n=200, v=256, chunk=None, length=200, run=1, ps=16, back=199, rows=8, far=300, scale=0.12, cap=None),
])
@pytest.mark.parametrize("one_wave_a_query", [False, True])
def test_scored_attention_finds_the_key_that_stands_out(name, dtype, tol, case, one_wave_a_query):
    """Through the kernel that norms and stores and the attention kernels (in bfloat16 those on the matrix unit,
    and the general one when told to): queries and keys scaled to unit root mean square a head, capped scores,
    the bias by distance, chunks, the gate."""
    if one_wave_a_query and dtype == torch.float32:
        pytest.skip("float32 runs on the general kernel anyway")
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    from transformers_neuronx_amd.parts.mixer import bias_by_distance
    ops = _ops(dtype)
    ops.force_plain_attention = one_wave_a_query
    case = dict(case, eps=1e-4)
    h, g, n, v, length, run, ps = (case[k] for k in ("h", "g", "n", "v", "length", "run", "ps"))
    d = -(-max(n, v) // 16) * 16
    x, rel, want, seen = _standout(dtype, case, 7)
    chunk = case.get("chunk")
    visible = not chunk or case["back"] <= (length - 1) % chunk
    for weight in seen:
        assert (weight is not None and weight > 0.9) == visible, seen
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=torch.Generator().manual_seed(1))[:blocks].tolist()
    k_pages = torch.zeros(blocks + 3, g, ps, d, dtype=dtype, device=DEV)
    v_pages = torch.zeros(blocks + 3, g, d, ps, dtype=dtype, device=DEV)
    bias = bias_by_distance(rel, case["far"]).to(DEV)
    head = length - run
    nq = h * n + g * (n + v)
    got = None
    for a, b in ((0, head), (head, length)):
        if b == a:
            continue
        ctx = _ctx([b - a], [a], [0], {"g": [order]}, ps, {"attention": attention_plan})
        rows = x[a:b].to(DEV)
        q = ops.qkv_prepare(rows, h, g, n, v, d, None, None, case["eps"], None, False, case["scale"], None, None, ctx,
                            ctx.groups["g"], k_pages, v_pages, per_head=True)
        got = ops.attention_scored(q, h, g, d, ctx, ctx.groups["g"], k_pages, v_pages, chunk=chunk, softcap=case.get("cap"),
                                   distance_bias=bias, gate=rows[:, nq:], value_size=v, out_scale=1.0)
    # in bfloat16 the unit-norm queries and keys are rounded: scores of a few units move by hundredths
    _close(got.view(run, h, d)[:, :, :v].reshape(run, h * v), want, tol if dtype == torch.float32 else 4e-2)


@pytest.mark.parametrize("pad,splits", [(0, None), (2, 1), (3, 3), (0, 8)])
def test_scored_attention_of_a_mixed_step_into_columns_of_a_wider_buffer(pad, splits):
    """Runs of one token (each key/value head's query heads side by side, 20 of them: two blocks of columns)
    beside a portion and a whole prompt in one step, written times a factor into a slice of a buffer whose rows
    are not multiples of 8 bytes apart, a decoded token's keys in one block or shared out over several (more
    blocks than it has tiles among them); against the general kernel, and the columns beside the slice untouched."""
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    from transformers_neuronx_amd.parts.mixer import bias_by_distance
    h, g, n, v, d, ps = 40, 2, 32, 24, 32, 16
    gen = torch.Generator().manual_seed(3)
    rel = torch.randn(10, h, generator=gen)
    bias = bias_by_distance(rel, 50).to(DEV)
    lens, runs = [150, 97, 200, 31], [1, 1, 40, 31]
    pages = sum(-(-n_ // ps) for n_ in lens)
    order = torch.randperm(pages + 2, generator=gen).tolist()
    tables, at = [], 0
    for n_ in lens:
        k = -(-n_ // ps)
        tables.append(order[at:at + k] + [-1] * (13 - k))
        at += k
    results = {}
    for plain in (False, True):
        ops = _ops(torch.bfloat16)
        ops.force_plain_attention = plain
        ops.scored_decode_splits = splits
        k_pages = torch.zeros(pages + 2, g, ps, d, dtype=torch.bfloat16, device=DEV)
        v_pages = torch.zeros(pages + 2, g, d, ps, dtype=torch.bfloat16, device=DEV)
        gen2 = torch.Generator().manual_seed(4)
        width = h * n + g * (n + v) + h * v
        for heads, cached in (([n_ - r for n_, r in zip(lens, runs)], [0] * 4), (runs, [n_ - r for n_, r in zip(lens, runs)])):
            if not any(heads):
                continue
            live = [i for i, t in enumerate(heads) if t]
            ctx = _ctx([heads[i] for i in live], [cached[i] for i in live], live, {"g": [tables[i] for i in live]}, ps,
                       {"attention": attention_plan})
            rows = (torch.randn(sum(heads), width, generator=gen2) * 1.5).to(DEV)
            q = ops.qkv_prepare(rows, h, g, n, v, d, None, None, 1e-5, None, False, 0.4, None, None, ctx, ctx.groups["g"],
                                k_pages, v_pages, per_head=True)
            both = torch.full((sum(heads), pad + h * d + 5), 7.0, dtype=torch.bfloat16, device=DEV)
            ops.attention_scored(q, h, g, d, ctx, ctx.groups["g"], k_pages, v_pages, chunk=64, softcap=15.0,
                                 distance_bias=bias, gate=rows[:, h * n + g * (n + v):], value_size=v,
                                 out=both[:, pad:pad + h * d], out_scale=0.6)
        results[plain] = both.float().cpu()
    assert float(results[False][:, :pad].min() if pad else 7.0) == 7.0 and float(results[False][:, pad + h * d:].min()) == 7.0
    err = float((results[False] - results[True]).abs().max() / results[True][:, pad:pad + h * d].abs().max())
    assert err < 2e-2, err


# ---------------------------------------------------------------- the engine

@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("name", sorted(tc.CASES))
def test_schedules_on_the_gpu(name, dtype, tol):
    cfg = tc.config(name)
    w = tc.weights(cfg, 3, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = tc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=208)
    requests = tc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, tol, few)
    from transformers_neuronx_amd.kernels import hip
    assert {"prepare", "hyper", "recurrent", "scored", "gemm"} <= set(hip.loaded_libraries())


def test_the_stream_after_every_run_of_a_layer_on_the_gpu():
    from transformers_neuronx_amd import debug
    cfg = tc.config("a")
    w = tc.weights(cfg, 8)
    toks = tc.requests(cfg, [27], 4)["r0"]
    after = []
    P.forward(cfg.to_dict(), P.widen(w), toks, after)
    runner = tc.runner(cfg, w, kernels="hip", device=DEV)
    with debug.debug_context() as taps:
        runner.step([StepEntry("r", toks, [0])])
    names = [k for k in taps if k.startswith("call")]
    assert len(names) == len(after)
    for name, want in zip(names, after):
        assert float((taps[name].double().cpu() - want).abs().max() / want.abs().max()) < 1e-5


@pytest.mark.parametrize("graphs", [True, False])
def test_long_decoding_recorded_and_not(graphs):
    """300 tokens one by one beside requests that join and leave: chunks begin and end among decoded tokens, pages
    go back, recurrences run on, the batch size changes (a recorded step is made for each), slots change hands."""
    cfg = tc.config("d")
    w = tc.weights(cfg, 8)
    runner = tc.runner(cfg, w, dtype="float32", kernels="hip", device=DEV, max_tokens=512, page_size=16, use_graphs=graphs)
    requests = tc.requests(cfg, [320, 90, 60], 9)
    expected = _expected(cfg, w, requests)
    a, b, c = requests["r0"], requests["r1"], requests["r2"]
    got = {"r0": [runner.step([StepEntry("r0", a[:20], list(range(20)))])], "r1": [], "r2": []}
    for i in range(20, 320):
        entries = [StepEntry("r0", [a[i]], [0])]
        if 50 <= i < 140:
            entries.append(StepEntry("r1", [b[i - 50]], [0]))
        if 200 <= i < 260:
            entries.append(StepEntry("r2", [c[i - 200]], [0]))
        out = runner.step(entries)
        for row, e in enumerate(entries):
            got[e.req].append(out[row:row + 1].clone())
        if i == 139:
            runner.finish("r1")
        if i == 259:
            runner.finish("r2")
    assert (runner.graph_replays > 0) == graphs
    for rid in requests:
        have = torch.cat(got[rid])
        assert float((have.double().cpu() - expected[rid]).abs().max() / expected[rid].abs().max()) < TOL, rid


@pytest.mark.parametrize("amp,tol", [("f32", TOL), ("bf16", 6e-2)])
def test_generation_through_the_entry_point(tmp_path, amp, tol):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.weights import write_random_model
    cfg = tc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32" if amp == "f32" else "bfloat16")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp=amp, n_positions=64, page_size=16,
                                                       device=DEV).load()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    logits = model(ids)
    raw, wide = cfg.to_dict(), P.widen(w)
    for row in range(2):
        want = P.forward(raw, wide, ids[row].tolist())[-1]
        assert float((logits[row].double().cpu() - want).abs().max() / want.abs().max()) < tol
    if amp == "f32":
        out = model.sample(ids, sequence_length=14, top_k=1)
        for row in range(2):
            assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


def test_generation_through_the_scheduler_with_few_pages():
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.sampling import SamplingParams
    from transformers_neuronx_amd.weights.loader import TensorDict
    cfg = tc.config("c")
    w = tc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="hip", device=DEV, page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9)
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(tc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_the_replay_program_serves_a_folder(tmp_path):
    from transformers_neuronx_amd.weights import write_random_model
    cfg = tc.config("c")
    folder = write_random_model(cfg, str(tmp_path / "m"), 12, dtype="bfloat16")
    from safetensors.torch import load_file
    w = load_file(os.path.join(folder, "model.safetensors"))
    requests = tc.requests(cfg, [40, 9, 70, 3, 25], 13)
    expected = _expected(cfg, w, requests)
    steps, place = schedules.mixed(requests, max_tokens=192, page=64, seed=1, tail=6, max_live=4)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out_dir), "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps),
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    for (step, row), (rid, pos) in place.items():
        got = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(-1, cfg.vocab)[row]
        want = expected[rid][pos].numpy()
        assert np.abs(got - want).max() / np.abs(expected[rid].numpy()).max() < TOL


def test_the_command_line_serves_the_folder(tmp_path, capsys):
    """`opt_demo save --random --config` writes a folder of whatever architecture the config.json names, and
    `run --benchmark --profile` generates from it and times its kernels."""
    from transformers_neuronx_amd.opt import demo
    with open(tmp_path / "config.json", "w") as fp:
        json.dump(dict(tc.CASES["d"], init_std=0.3), fp)
    folder = str(tmp_path / "model")
    assert demo.main(["--amp", "bf16", "save", folder, "--random", "--config", str(tmp_path / "config.json")]) in (0, None)
    assert demo.main(["--amp", "bf16", "run", folder, "--batch_size", "2", "--n_positions", "40", "--prompt_len", "9",
                      "--top_k", "1", "--benchmark", "--profile", "--page_size", "16"]) in (0, None)
    text = capsys.readouterr().out
    assert "running TadolixForSampling.from_pretrained" in text
    report = json.loads(next(line for line in text.splitlines() if line.startswith("{")))
    assert report["inferences"] == 10 and report["e2e_output_token_throughput"] > 0
    for kernel in ("tnx_qkv_prepare", "tnx_attention_scored", "tnx_min_gru", "tnx_gated_linear_recurrence",
                   "tnx_channel_conv", "tnx_hyper_step", "tnx_add_sinusoid"):
        assert kernel in text, kernel


@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_from_a_seed(seed, dtype, tol):
    cfg = tc.drawn(seed)
    w = tc.weights(cfg, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = tc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=176)
    requests = tc.requests(cfg, [70, 33, 5, 1], seed)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    step_through(runner, expected, schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), tol, few)
    step_through(runner, expected, schedules.head_then_singles(requests, tail=20), tol, few)
