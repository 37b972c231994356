"""Zotunex on the GPU: every kernel of its parts alone against the plain implementation's function of the same
mechanism (float32 and bfloat16), attention of both kinds with a key made to stand out far away, at page borders
and at the first token, in prompts and in decoding, sinks that weigh much and little, pages that change hands, the
engine under every way of cutting, recorded decoding, generation through the entry point, and the replay program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_zotunex as P
import zotunex_cases as zc
import schedules
from test_zotunex_cpu import TOL, _expected, _greedy, step_through
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


def _close(got, want, tol):
    want = want.to(F64)
    err = float((got.double().cpu() - want).abs().max() / max(1e-30, float(want.abs().max())))
    assert err < tol, err


# ---------------------------------------------------------------- each mechanism alone

@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [
    # query heads, key/value heads, head size, cached head size, turned elements, factor, gate columns behind
    (4, 2, 16, 16, 8, 2.0, 4), (3, 3, 10, 16, 10, None, 3), (6, 1, 96, 96, 24, 4.0, 6), (1, 1, 32, 32, 0, None, 0),
    (8, 2, 128, 128, 128, 16.0, 8)])
def test_projections_are_normed_a_head_turned_scaled_a_head_and_the_keys_kept_as_values(name, dtype, tol, sizes):
    heads, groups, n, d, dims, factor, behind = sizes
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(3)
    length, ps, eps, scale = 41, 16, 1e-5, 0.37
    proj = torch.randn(length, heads * n + groups * n + behind, generator=g) * 2
    qw, kw = torch.randn(n, generator=g), torch.randn(n, generator=g)
    temp = torch.rand(heads, generator=g) + 0.5
    rot = dict(base=300.0, dims=dims, scaling=dict(factor=factor) if factor else None)
    freqs = P.frequencies(rot).float().to(DEV) if dims else None
    pos = torch.arange(length)
    x = proj.double()
    q = P.unit_rms(x[:, :heads * n].view(length, heads, n), eps) * qw.double()
    k = P.unit_rms(x[:, heads * n:heads * n + groups * n].view(length, groups, n), eps) * kw.double()
    if dims:
        q, k = P.rotate_neighbours(q, pos, rot), P.rotate_neighbours(k, pos, rot)
    q = q * scale * temp.double()[None, :, None]
    values = x[:, heads * n:heads * n + groups * n].view(length, groups, n)
    order = [5, 0, 3]
    k_pages = torch.full((6, groups, ps, d), 7.0, dtype=dtype, device=DEV)     # what a former holder left
    v_pages = torch.full((6, groups, d, ps), 7.0, dtype=dtype, device=DEV)
    got_q = []
    for a, b in ((0, 1), (1, 3), (3, 20), (20, 21), (21, 41)):                 # steps cut anywhere
        ctx = _ctx([b - a], [a], [0], {"g": [order]}, ps)
        got_q.append(ops.qkv_prepare(proj[a:b].to(DEV), heads, groups, n, n, d, qw.repeat(heads).to(DEV),
                                     kw.repeat(groups).to(DEV), eps, freqs, True, scale, None, None, ctx, ctx.groups["g"],
                                     k_pages, v_pages, per_head=True, values_at=heads * n, head_scale=temp.to(DEV)))
    got_q = torch.cat(got_q).view(length, heads, d)
    _close(got_q[:, :, :n], q, tol)
    assert float(got_q[:, :, n:].abs().max() if d > n else 0.0) == 0
    got_k = torch.cat([k_pages[p] for p in order], dim=1)[:, :length].permute(1, 0, 2)           # [length, G, d]
    got_v = torch.cat([v_pages[p] for p in order], dim=2)[:, :, :length].permute(2, 0, 1)
    _close(got_k[:, :, :n], k, tol)
    _close(got_v[:, :, :n], values, tol)
    assert float(k_pages[[1, 2, 4]].sub(7.0).abs().max()) == 0                                   # no other page is touched


def _keys_as_values(proj, heads, groups, n, scale, temp, first):
    """The mechanism restated for queries from position `first` on: the projections are the queries and keys
    themselves (no norm, nothing turned), the values are the keys, a head's result passes its gate."""
    length = proj.shape[0]
    x = proj.double()
    q = x[first:, :heads * n].view(-1, heads, n)
    k = x[:, heads * n:heads * n + groups * n].view(length, groups, n).repeat_interleave(heads // groups, dim=1)
    gate = x[first:, heads * n + groups * n:heads * n + groups * n + heads]
    scores = torch.einsum("ihd,jhd->hij", q, k) * scale * temp.double()[:, None, None]
    seen = torch.arange(length)[None, :] <= torch.arange(first, length)[:, None]
    prob = P.weights_over(scores, seen)
    return torch.einsum("hij,jhd->ihd", prob, k) * P.sigmoid(gate)[:, :, None], prob


@pytest.mark.parametrize("name,dtype,tol", [("float32", torch.float32, 4e-5), ("bfloat16", torch.bfloat16, 4e-2)])
@pytest.mark.parametrize("case", [
    # query heads, kv heads, head size, cached head size, length, the step's tokens, page, standout (back from the last)
    dict(h=4, g=2, n=16, d=16, length=300, run=1, ps=16, back=299),       # the very first token, decoded alone
    dict(h=2, g=1, n=64, d=64, length=700, run=1, ps=16, back=697),       # far away
    dict(h=6, g=1, n=96, d=96, length=700, run=37, ps=64, back=640),      # far away, in a portion; a page border
    dict(h=6, g=3, n=16, d=16, length=64, run=64, ps=16, back=63),        # a whole prompt, the first token
    dict(h=1, g=1, n=64, d=64, length=129, run=2, ps=64, back=1),         # the token before: the last of a page
    dict(h=20, g=1, n=32, d=32, length=390, run=1, ps=64, back=200),      # twenty heads on one key/value head
    dict(h=3, g=3, n=10, d=16, length=50, run=3, ps=16, back=0),          # itself; heads filled up in the cache
    dict(h=8, g=2, n=128, d=128, length=280, run=200, ps=16, back=279),   # several tiles of queries
])
@pytest.mark.parametrize("kernel", ["matrix unit", "shared out", "general"])
def test_attention_over_keys_that_are_the_values_finds_the_key_that_stands_out(name, dtype, tol, case, kernel):
    """Through the kernel that stores and the attention kernels with a gate a head; in bfloat16 on the matrix unit
    (a decoded token's keys in one block, or shared out over three) and on the kernel for any sizes."""
    if kernel != "general" and dtype == torch.float32:
        pytest.skip("float32 has the one kernel")
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    ops = _ops(dtype)
    ops.force_plain_attention = kernel == "general"
    ops.scored_decode_splits = 3 if kernel == "shared out" else 1
    h, g, n, d, length, run, ps = (case[k] for k in ("h", "g", "n", "d", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    gen = torch.Generator().manual_seed(7)
    proj = torch.randn(length, h * n + g * n + h, generator=gen) * 0.3
    mark = torch.randn(n, generator=gen)
    mark = mark / mark.norm() * 9.0
    proj[standout, h * n:h * n + g * n] = mark.repeat(g)
    proj[length - 1, :h * n] = mark.repeat(h)
    proj[:, h * n + g * n:] *= 6                         # gates that open and close
    proj = proj.to(dtype).float()
    temp = torch.rand(h, generator=gen) + 0.75
    scale = 0.8
    want, prob = _keys_as_values(proj, h, g, n, scale, temp, length - run)
    assert float(prob[:, -1, standout].min()) > 0.9
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=torch.Generator().manual_seed(1))[:blocks].tolist()
    k_pages = torch.full((blocks + 3, g, ps, d), 50.0, dtype=dtype, device=DEV)
    v_pages = torch.full((blocks + 3, g, d, ps), 50.0, dtype=dtype, device=DEV)
    head = length - run
    got = None
    for a, b in ((0, head), (head, length)):
        if b == a:
            continue
        ctx = _ctx([b - a], [a], [0], {"g": [order]}, ps, {"attention": attention_plan})
        rows = proj[a:b].to(DEV)
        q = ops.qkv_prepare(rows, h, g, n, n, d, None, None, 0.0, None, False, scale, None, None, ctx, ctx.groups["g"],
                            k_pages, v_pages, values_at=h * n, head_scale=temp.to(DEV))
        got = ops.attention_scored(q, h, g, d, ctx, ctx.groups["g"], k_pages, v_pages, gate=rows[:, h * n + g * n:],
                                   value_size=n, gate_per_head=True)
    _close(got.view(run, h, d)[:, :, :n], want, tol)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
def test_latent_norms_without_a_query_latent(name, dtype, tol):
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(5)
    R, r, pairs, ps, behind = 18, 6, 3, 16, 5
    down = torch.randn(9, R + r + behind, generator=g) * 2
    kw = torch.randn(R, generator=g)
    rot = dict(base=50.0, dims=2 * pairs, scaling=dict(factor=3.0))
    lat = torch.zeros(5, ps, R, dtype=dtype, device=DEV)
    turned = torch.zeros(5, ps, r, dtype=dtype, device=DEV)
    across = torch.zeros(5, R, ps, dtype=dtype, device=DEV)
    ctx = _ctx([9], [12], [0], {"g": [[3, 1, 4]]}, ps)          # crosses from page 3 into page 1
    assert ops.latent_norms(down.to(DEV), 0, R, r, None, kw.to(DEV), 1e-5, P.frequencies(rot).float().to(DEV), ctx,
                            ctx.groups["g"], lat, turned, across) is None
    _close(torch.cat([lat[3, 12:], lat[1, :5]]), P.unit_rms(down.double()[:, :R], 1e-5) * kw.double(), tol)
    want = P.rotate_neighbours(down.double()[:, None, R:R + r], torch.arange(12, 21), rot)[:, 0]
    _close(torch.cat([turned[3, 12:], turned[1, :5]]), want, tol)
    assert float(lat[[0, 2, 4]].abs().max()) == 0 and torch.equal(across.transpose(1, 2), lat)


def _latent_case(dtype, heads, n, r, R, length, run, ps, standout, seed):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn(length, R, generator=g).to(dtype)
    kr = torch.randn(length, r, generator=g).to(dtype)
    q = torch.randn(run, heads, n + r, generator=g).to(dtype)
    q_lat = torch.randn(run, heads, R, generator=g).to(dtype) * 0.3
    gate = torch.randn(run, heads + 3, generator=g) * 3
    if standout is not None:
        direction = torch.nn.functional.normalize(torch.randn(R, generator=g), dim=0)
        c[standout] = (direction * 6).to(dtype)
        q_lat[-1] = (direction * 20).to(dtype)
    blocks = -(-length // ps)
    order = torch.randperm(blocks + 3, generator=g)[:blocks].tolist()
    lat = torch.randn(blocks + 3, ps, R, generator=g).to(dtype).to(DEV) * 50          # what others left in the pages
    rot = torch.randn(blocks + 3, ps, r, generator=g).to(dtype).to(DEV) * 50
    for j in range(length):
        lat[order[j // ps], j % ps] = c[j]
        rot[order[j // ps], j % ps] = kr[j]
    return c, kr, q, q_lat, gate, lat, rot, order, lat.transpose(1, 2).contiguous()


@pytest.mark.parametrize("name,dtype,tol", [("float32", torch.float32, 4e-5), ("bfloat16", torch.bfloat16, 1.2e-2)])
@pytest.mark.parametrize("case", [
    # heads, n, r, R, length, the step's tokens, page, standout (back from the last query), the sinks' level
    dict(heads=3, n=8, r=6, R=18, length=300, run=1, ps=16, back=299, sink=0.0),      # the first token, decoded alone
    dict(heads=2, n=16, r=4, R=24, length=700, run=1, ps=16, back=697, sink=50.0),    # far away; sinks that outweigh it
    dict(heads=2, n=16, r=4, R=24, length=700, run=37, ps=16, back=699, sink=-40.0),  # sinks that weigh nothing
    dict(heads=5, n=4, r=2, R=10, length=64, run=64, ps=16, back=63, sink=2.0),       # a whole prompt
    # sizes the matrix unit takes (in bfloat16): latents in 16s, rotated parts in 8s
    dict(heads=6, n=64, r=16, R=64, length=700, run=1, ps=64, back=697, sink=50.0),   # keys shared out over blocks
    dict(heads=20, n=16, r=16, R=80, length=50, run=1, ps=64, back=49, sink=1.0),     # one block of keys; 20 heads
    dict(heads=2, n=16, r=24, R=160, length=700, run=37, ps=16, back=640, sink=50.0),
    dict(heads=5, n=8, r=8, R=16, length=64, run=64, ps=16, back=0, sink=3.0),
    dict(heads=2, n=32, r=16, R=64, length=300, run=200, ps=64, back=236, sink=50.0),  # several tiles; a page border
    dict(heads=17, n=8, r=8, R=272, length=290, run=2, ps=32, back=1, sink=0.5),
])
@pytest.mark.parametrize("kernel", ["shared", "alone", "any"])
def test_latent_attention_with_a_sink_and_a_gate(name, dtype, tol, case, kernel):
    if kernel != "any" and dtype == torch.float32:
        pytest.skip("float32 has the one kernel")
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    ops = _ops(dtype)
    ops.latent_matrix_unit = kernel != "any"
    ops.latent_prompt_kind = 1 if kernel == "alone" else 0
    heads, n, r, R, length, run, ps = (case[k] for k in ("heads", "n", "r", "R", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    c, kr, q, q_lat, gate, lat, rot, order, across = _latent_case(dtype, heads, n, r, R, length, run, ps, standout, 7)
    sink = torch.randn(heads, generator=torch.Generator().manual_seed(2)) + case["sink"]
    rotary = dict(base=321.0, dims=r - 2 if r > 2 else r)
    scale = 0.4
    # the mechanism restated: scores scale (q_lat . c + turn(q_r) . k_r), softmax with the sink, sum of c, the gate
    pos = torch.arange(length - run, length)
    q_r = P.rotate_neighbours(q.double()[..., n:], pos, rotary)
    scores = (torch.einsum("ihd,jd->hij", q_lat.double(), c.double()) + torch.einsum("ihd,jd->hij", q_r, kr.double())) * scale
    prob = P.weights_over(scores, torch.arange(length)[None, :] <= pos[:, None], sink.double())
    want = torch.einsum("hij,jd->ihd", prob, c.double()) * P.sigmoid(gate.double()[:, :heads])[:, :, None]
    share = float(prob[:, -1].sum(-1).min())
    assert (share < 0.5) if case["sink"] > 15 else (share > 0.5), share         # the sink takes most, or little
    ctx = build_context([StepEntry(0, [0] * run, [])], [length - run], [0], {"g": np.asarray([order], dtype=np.int32)},
                        ps, DEV, {"attention": attention_plan})
    gates = gate.to(DEV)
    got = ops.latent_attention(q.reshape(run, -1).to(DEV), q_lat.to(DEV), heads, n, r, R,
                               P.frequencies(rotary).float().to(DEV), scale, ctx, ctx.groups["g"], lat, rot, across, None,
                               sink=sink.to(DEV), gate=gates[:, :heads])
    _close(got, want, tol)


@pytest.mark.parametrize("case", [
    dict(heads=3, n=16, r=8, v=32, R=48, length=300, run=150, ps=16, back=299, sink=0.0),
    dict(heads=2, n=64, r=32, v=64, R=128, length=700, run=300, ps=64, back=640, sink=50.0),
    dict(heads=5, n=8, r=8, v=16, R=24, length=64, run=64, ps=16, back=16, sink=-30.0),
    dict(heads=6, n=64, r=16, v=64, R=64, length=280, run=2, ps=16, back=279, sink=12.0),
])
def test_prompt_latent_attention_on_expanded_keys_with_a_sink_and_a_gate(case):
    from transformers_neuronx_amd.kernels.attention_plan import attention_plan
    dtype = torch.bfloat16
    ops = _ops(dtype)
    heads, n, r, v, R, length, run, ps = (case[k] for k in ("heads", "n", "r", "v", "R", "length", "run", "ps"))
    standout = length - 1 - case["back"]
    g = torch.Generator().manual_seed(9)
    w_uk = (torch.randn(heads * n, R, generator=g) / R ** 0.5).to(dtype)
    w_uv = (torch.randn(heads * v, R, generator=g) / R ** 0.5).to(dtype)
    c, kr, q, _, gate, lat, rot, order, _ = _latent_case(dtype, heads, n, r, R, length, run, ps, None, 11)
    q = q * 0.3
    keys = (c.double() @ w_uk.double().T).view(length, heads, n)
    q[-1, :, :n] = (keys[standout] / keys[standout].norm(dim=-1, keepdim=True) * 12).to(dtype)
    sink = torch.randn(heads, generator=g) + case["sink"]
    rotary, scale = dict(base=321.0, dims=r - 2), 0.4
    pos = torch.arange(length - run, length)
    vals = (c.double() @ w_uv.double().T).view(length, heads, v)
    q_r = P.rotate_neighbours(q.double()[..., n:], pos, rotary)
    scores = (torch.einsum("ihd,jhd->hij", q.double()[..., :n], keys) + torch.einsum("ihd,jd->hij", q_r, kr.double())) * scale
    prob = P.weights_over(scores, torch.arange(length)[None, :] <= pos[:, None], sink.double())
    want = (torch.einsum("hij,jhd->ihd", prob, vals) * P.sigmoid(gate.double()[:, :heads])[:, :, None]).reshape(run, heads * v)
    ctx = build_context([StepEntry(0, [0] * run, [])], [length - run], [0], {"g": np.asarray([order], dtype=np.int32)}, ps, DEV,
                        {"attention": attention_plan})
    ops.expand_rows = 2
    assert ops.latent_expands(ctx, n, r, v, R)
    got = ops.latent_attention_expanded(q.reshape(run, -1).to(DEV), w_uk.to(DEV), w_uv.to(DEV), heads, n, r, v, R,
                                        P.frequencies(rotary).float().to(DEV), scale, ctx, ctx.groups["g"], lat, rot, None,
                                        sink=sink.to(DEV), gate=gate.to(DEV)[:, :heads])
    _close(got, want, 2e-2)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("sizes", [
    # tokens, experts, a token's experts, width, inner size, shared inner size, limit
    (1, 4, 1, 64, 16, 0, 1.0), (37, 5, 2, 96, 40, 24, 0.7), (130, 10, 1, 192, 72, 88, 2.0), (9, 3, 3, 50, 30, 10, 0.5),
    (300, 70, 4, 128, 24, 0, 7.0), (1300, 8, 4, 128, 64, 96, 1.0)])
@pytest.mark.parametrize("forced", [None, "ours", "plain"])
def test_corrected_choice_and_clamped_experts(name, dtype, tol, sizes, forced):
    """`forced`: None, as the engine would (steps of many pairs an expert through the vendor library); "ours": the one
    launch of ours at any size; "plain": without the matrix unit."""
    from transformers_neuronx_amd.parts.feed_forward import ExpertMixture
    from types import SimpleNamespace
    tokens, experts, top, width, inner, shared, limit = sizes
    if forced and (dtype == torch.float32 or (forced == "ours" and tokens < 100)):
        pytest.skip("the same path as unforced")
    ops = _ops(dtype)
    ops.expert_library_rows = 96 if forced is None else 0
    ops.expert_plain_products = forced == "plain"
    g = torch.Generator().manual_seed(5)
    part = ExpertMixture(width, experts, top, inner, "router", "e{}.", ("gate", "up", "down"), shared_inner=shared,
                         score="sigmoid", weight_on="output", activation="clamped_swiglu", limit=limit,
                         shared_limit=limit * 1.5, correction_name="correction", route_scale=1.7)
    w = {}
    for d in part.param_decls("p."):
        w[d.name] = (torch.randn(d.shape, generator=g) * (2.5 / d.shape[-1] ** 0.5)).to(dtype)
    w["p.correction"] = torch.randn(experts, generator=g) * 0.4
    part.load({k: v.to(DEV) for k, v in w.items()}, "p.", ops, dtype)
    h = torch.randn(tokens, width, generator=g).to(dtype)
    residual = torch.randn(tokens, width, generator=g)
    mlp = dict(router=dict(experts=experts, top=top, scale=1.7), expert=dict(ff=inner, limit=limit),
               shared=dict(ff=shared, limit=limit * 1.5) if shared else None)
    wide = P.widen(w)
    wide["p.correction"] = w["p.correction"].double()
    z = h.double() @ wide["p.router"].T
    # the choice alone: to the number wherever the plain scores leave no doubt about it
    ranked = torch.sort(P.sigmoid(z) + wide["p.correction"], dim=-1, descending=True, stable=True).values
    gaps = (ranked[:, :-1] - ranked[:, 1:])[:, :top].min(-1).values if experts > 1 else torch.ones(tokens, dtype=F64)
    clear = gaps > 1e-5
    assert int(clear.sum()) >= tokens // 3
    chosen, weight = P.route(z, wide["p.correction"], top, 1.7)
    uncorrected, _ = P.route(z, torch.zeros(experts, dtype=F64), top, 1.7)
    assert tokens < 30 or top == experts or chosen.tolist() != uncorrected.tolist()      # the correction matters here
    got_chosen, got_weight = ops.route(ops.linear(h.to(DEV), part.w_router, None, out_f32=True), top, "sigmoid", False,
                                       correction=part.correction, scale=1.7)
    assert got_chosen.cpu()[clear].tolist() == chosen[clear].tolist()
    _close(got_weight.cpu()[clear], weight[clear], 1e-5 if dtype == torch.float32 else 1e-2)
    got = part.forward(h.to(DEV), SimpleNamespace(length_bound=None), residual.to(DEV))
    want = residual.double() + P.mixture(mlp, wide, "p.", h.double())
    # both clamps are met by some inner values and not by others
    gu = h.double() @ wide["p.e0.gate"].T
    assert limit > 2 or (float((gu > limit).double().mean()) > 0.005 and float((gu < limit).double().mean()) > 0.3)
    _close(got.cpu()[clear], want[clear], tol)


@pytest.mark.parametrize("name,dtype,tol", DTYPES)
@pytest.mark.parametrize("rows", [1, 8, 40, 130, 700])
def test_squared_relu_after_a_product_of_any_number_of_rows(name, dtype, tol, rows):
    from transformers_neuronx_amd.parts.feed_forward import DenseFeedForward
    ops = _ops(dtype)
    g = torch.Generator().manual_seed(rows)
    width, inner = 128, 320
    part = DenseFeedForward(width, inner, "relu2", "up", "down", bias=False, weight_suffix="")
    w = {d.name: (torch.randn(d.shape, generator=g) / d.shape[1] ** 0.5).to(dtype) for d in part.param_decls("p.")}
    part.load({k: v.to(DEV) for k, v in w.items()}, "p.", ops, dtype)
    h = torch.randn(rows, width, generator=g).to(dtype)
    residual = torch.randn(rows, width, generator=g)
    got = part.forward(h.to(DEV), None, residual.to(DEV))
    _close(got, residual.double() + P.dense(P.widen(w), "p.", h.double()), tol)


@pytest.mark.parametrize("width", [50, 256, 1031])
def test_the_norm_of_one_number(width):
    from transformers_neuronx_amd.parts.norm import RMSNorm
    ops = _ops(torch.bfloat16)
    part = RMSNorm(width, 1e-4, weight_suffix="", scalar=True)
    assert [tuple(d.shape) for d in part.param_decls("n")] == [()]
    part.load({"n": torch.tensor(1.75, device=DEV)}, "n", ops, torch.bfloat16)
    x = torch.randn(7, width, generator=torch.Generator().manual_seed(0)) * 3
    f32, _ = part.forward(x.to(DEV), True, False)
    _close(f32, P.scalar_norm(x.double(), 1.75, 1e-4), 5e-6)


# ---------------------------------------------------------------- the engine

@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("name", sorted(zc.CASES))
def test_schedules_on_the_gpu(name, dtype, tol):
    cfg = zc.config(name)
    w = zc.weights(cfg, 3, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = zc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=208)
    requests = zc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, tol, few)
    from transformers_neuronx_amd.kernels import hip
    assert {"prepare", "latent", "experts", "gemm", "scored"} <= set(hip.loaded_libraries())


def test_the_stream_after_every_layer_on_the_gpu():
    from transformers_neuronx_amd import debug
    cfg = zc.config("c")
    w = zc.weights(cfg, 2)
    toks = zc.requests(cfg, [70], 0)["r0"]
    _, layers = P.forward(cfg.to_dict(), P.widen(w), toks, return_layers=True)
    runner = zc.runner(cfg, w, dtype="float32", kernels="hip", device=DEV)
    with debug.debug_context() as taps:
        runner.step([StepEntry("r0", toks, [])])
    for i, want in enumerate(layers):
        got = taps[f"call{i}.layer{i}"]
        assert float((got.double().cpu() - want).abs().max() / want.abs().max()) < 1e-5, i


def test_schedules_with_expanded_prompt_steps():
    cfg = zc.config("c")
    w = zc.weights(cfg, 8, torch.bfloat16)
    runner = zc.runner(cfg, w, dtype="bfloat16", kernels="hip", device=DEV, max_tokens=208)
    runner.ops.expand_rows = 2
    requests = zc.requests(cfg, [70, 33, 5, 100], 2)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.portions(requests)):
        step_through(runner, expected, made, 6e-2, 0.15)


@pytest.mark.parametrize("graphs", [True, False])
def test_long_decoding_recorded_and_not(graphs):
    """300 tokens one by one beside requests that join and leave: the batch size changes (a recorded step is made
    for each), pages and slots change hands."""
    cfg = zc.config("c")
    w = zc.weights(cfg, 8)
    runner = zc.runner(cfg, w, dtype="float32", kernels="hip", device=DEV, max_tokens=512, page_size=16, use_graphs=graphs)
    requests = zc.requests(cfg, [320, 90, 60], 9)
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


def test_long_decoding_in_bfloat16_recorded():
    cfg = zc.config("c")
    w = zc.weights(cfg, 9, torch.bfloat16)
    runner = zc.runner(cfg, w, dtype="bfloat16", kernels="hip", device=DEV, max_tokens=1024, page_size=64)
    requests = zc.requests(cfg, [600, 200], 4)
    expected = _expected(cfg, w, requests)
    a, b = requests["r0"], requests["r1"]
    got = {"r0": [runner.step([StepEntry("r0", a[:300], list(range(300)))])], "r1": [runner.step([StepEntry("r1", b[:2], [0, 1])])]}
    for i in range(300, 600):
        entries = [StepEntry("r0", [a[i]], [0])] + ([StepEntry("r1", [b[i - 298]], [0])] if i - 298 < 200 else [])
        out = runner.step(entries)
        for row, e in enumerate(entries):
            got[e.req].append(out[row:row + 1].clone())
    assert runner.graph_replays > 0
    for rid in requests:
        have = torch.cat(got[rid])
        err = (have.double().cpu() - expected[rid]).abs().amax(-1) / expected[rid].abs().max()
        assert float((err > 6e-2).double().mean()) <= 0.15, rid


@pytest.mark.parametrize("amp,tol", [("f32", TOL), ("bf16", 6e-2)])
def test_generation_through_the_entry_point(tmp_path, amp, tol):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.weights import write_random_model
    cfg = zc.config("a")
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
    cfg = zc.config("b")
    w = zc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="hip", device=DEV, page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9)
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(zc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_the_replay_program_serves_a_folder(tmp_path):
    from transformers_neuronx_amd.weights import write_random_model
    cfg = zc.config("b")
    folder = write_random_model(cfg, str(tmp_path / "m"), 12, dtype="bfloat16")
    from safetensors.torch import load_file
    w = load_file(os.path.join(folder, "model.safetensors"))
    requests = zc.requests(cfg, [40, 9, 70, 3, 25], 13)
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
        json.dump(dict(zc.CASES["c"], init_std=0.3), fp)
    folder = str(tmp_path / "model")
    assert demo.main(["--amp", "bf16", "save", folder, "--random", "--config", str(tmp_path / "config.json")]) in (0, None)
    assert demo.main(["--amp", "bf16", "run", folder, "--batch_size", "2", "--n_positions", "40", "--prompt_len", "9",
                      "--top_k", "1", "--benchmark", "--profile", "--page_size", "16"]) in (0, None)
    text = capsys.readouterr().out
    assert "running ZotunexForSampling.from_pretrained" in text
    report = json.loads(next(line for line in text.splitlines() if line.startswith("{")))
    assert report["inferences"] == 10 and report["e2e_output_token_throughput"] > 0
    for kernel in ("tnx_qkv_prepare", "tnx_attention_scored", "tnx_latent_attention", "tnx_expert_mixture", "tnx_route",
                   "tnx_gated_activation"):
        assert kernel in text, kernel


@pytest.mark.parametrize("dtype,tol", [("float32", TOL), ("bfloat16", 6e-2)])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_from_a_seed(seed, dtype, tol):
    cfg = zc.drawn(seed)
    w = zc.weights(cfg, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    runner = zc.runner(cfg, w, dtype=dtype, kernels="hip", device=DEV, max_tokens=176)
    requests = zc.requests(cfg, [70, 33, 5, 1], seed)
    expected = _expected(cfg, w, requests)
    few = 0.15 if dtype == "bfloat16" else 0.0
    step_through(runner, expected, schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), tol, few)
    step_through(runner, expected, schedules.head_then_singles(requests, tail=20), tol, few)
