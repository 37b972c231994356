"""Zotunex on the host: the plain implementation pinned by what its mechanisms must do, the configuration's
reader, and the engine (registry, loader, cache manager, step function, scheduler, entry point) on the torch
rendition of the kernels against the plain implementation, for configurations of the tests' own."""
import json
import math
import os

import pytest
import torch

import plain_zotunex as P
import zotunex_cases as zc
import schedules
from transformers_neuronx_amd.config import EngineConfig, read_config
from transformers_neuronx_amd.config.model_config import ConfigError
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.engine import LLMEngine
from transformers_neuronx_amd.sampling import SamplingParams
from transformers_neuronx_amd.weights import WeightsError, write_random_model
from transformers_neuronx_amd.zotunex import ZotunexConfig, zotunex_spec

F64 = torch.float64
TOL = 4e-5       # float32 against the plain implementation's float64, as a share of the logits' range


# ---------------------------------------------------------------- the plain implementation, pinned

def test_plain_rotations_count_distances_only_and_pair_as_they_say():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(5, 3, 12, generator=g, dtype=F64), torch.randn(5, 3, 12, generator=g, dtype=F64)
    pos = torch.tensor([0, 3, 4, 9, 20])
    rot = dict(base=50.0, dims=8, scaling=dict(factor=4.0))
    for turn in (P.rotate_neighbours, P.rotate_halves):
        a = torch.einsum("ihd,jhd->hij", turn(q, pos, rot), turn(k, pos, rot))
        b = torch.einsum("ihd,jhd->hij", turn(q, pos + 1000, rot), turn(k, pos + 1000, rot))
        assert torch.allclose(a, b, atol=1e-9)
        turned = turn(q, pos, rot)
        assert torch.equal(turned[..., 8:], q[..., 8:]) and torch.allclose(turned[0], q[0])
    n, h = P.rotate_neighbours(q, pos, rot), P.rotate_halves(q, pos, rot)
    assert torch.allclose(n[..., 2] ** 2 + n[..., 3] ** 2, q[..., 2] ** 2 + q[..., 3] ** 2)
    assert torch.allclose(h[..., 1] ** 2 + h[..., 5] ** 2, q[..., 1] ** 2 + q[..., 5] ** 2)
    # the first pair turns by position / factor; the second by base^(-2/dims) of that
    one = P.rotate_neighbours(torch.tensor([[[1.0, 0.0, 1.0, 0.0]]], dtype=F64), torch.tensor([6]),
                              dict(base=16.0, dims=4, scaling=dict(factor=3.0)))
    assert torch.allclose(one[0, 0], torch.tensor([math.cos(2.0), math.sin(2.0), math.cos(0.5), math.sin(0.5)], dtype=F64))
    two = P.rotate_halves(torch.tensor([[[1.0, 1.0, 0.0, 0.0]]], dtype=F64), torch.tensor([6]), dict(base=16.0, dims=4))
    assert torch.allclose(two[0, 0], torch.tensor([math.cos(6.0), math.cos(1.5), math.sin(6.0), math.sin(1.5)], dtype=F64))
    # the engine's own frequencies are these
    from transformers_neuronx_amd.parts.position import RotaryPositions
    for r in (rot, dict(base=1e6, dims=64), dict(base=77.0, dims=6, scaling=dict(factor=1.0))):
        part = RotaryPositions(r["base"], r["dims"], scaling=r.get("scaling"))
        assert torch.allclose(part.frequencies().double(), P.frequencies(r), rtol=1e-6, atol=0)


def test_plain_softmax_with_a_sink():
    s = torch.tensor([[[0.0, 9.0, 9.0], [1.0, 2.0, 9.0], [1.0, 1.0, 1.0]]], dtype=F64)
    plain = P.causal_weights(s)
    assert torch.allclose(plain[0, 1, :2], torch.softmax(torch.tensor([1.0, 2.0], dtype=F64), 0)) and plain[0, 0, 0] == 1
    assert float(plain[0, 0, 1:].abs().sum()) == 0 and float(plain[0, 1, 2]) == 0
    sunk = P.causal_weights(s, torch.tensor([1.0], dtype=F64))
    # three keys of score 1 beside a sink of 1: a quarter each, and a quarter is lost
    assert torch.allclose(sunk[0, 2], torch.full((3,), 0.25, dtype=F64))
    assert abs(float(sunk[0, 0, 0]) - 1.0 / (1.0 + math.e)) < 1e-12
    # a sink far above every score takes nearly everything, one far below changes nothing
    assert float(P.causal_weights(s, torch.tensor([500.0], dtype=F64)).sum()) < 1e-100
    assert torch.allclose(P.causal_weights(s, torch.tensor([-500.0], dtype=F64)), plain)


def test_plain_attention_takes_its_values_from_the_keys_before_their_norm():
    cfg = zc.config("a")
    m = cfg.to_dict()["layers"][3]["mixer"]           # 8 query heads on one key/value head, nothing turned
    w = P.widen(zc.weights(cfg, 0))
    p = "l3.mix."
    h = torch.randn(6, cfg.width, dtype=F64)
    out = P.attention(m, w, p, h, cfg.eps)
    # the first token sees itself alone: its result is its own key as projected, head by head through the gates
    k0 = h[0] @ w[p + "k"].T
    gate = torch.sigmoid(h[0] @ w[p + "g"].T)
    want = (gate[:, None] * k0[None, :]).reshape(-1) @ w[p + "o"].T
    assert torch.allclose(out[0], want)
    # the number a head on the scores is not on the values: doubling it changes later tokens, not the first
    w2 = dict(w, **{p + "temp": w[p + "temp"] * 2})
    out2 = P.attention(m, w2, p, h, cfg.eps)
    assert torch.allclose(out2[0], out[0]) and not torch.allclose(out2[3], out[3])
    # the norm is a head's own: scaling one query head's rows changes nothing at all
    w3 = dict(w)
    w3[p + "q"] = w[p + "q"].clone()
    w3[p + "q"][:m["dim"]] *= 7.0
    assert torch.allclose(P.attention(m, w3, p, h, 0.0), P.attention(m, w, p, h, 0.0))


def test_plain_latent_attention_by_hand():
    cfg = zc.config("a")
    m = cfg.to_dict()["layers"][1]["mixer"]
    w = P.widen(zc.weights(cfg, 1))
    p = "l1.mix."
    h = torch.randn(5, cfg.width, dtype=F64)
    out = P.latent_attention(m, w, p, h, cfg.eps)
    # the first token: one key beside the sink, so its value times 1 / (1 + exp(sink - score)), through the gate
    heads, n, r, v, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    down = h[0] @ w[p + "dkv"].T
    c = P.unit_rms(down[:rank], cfg.eps) * w[p + "dkv.norm"]
    q = (h[0] @ w[p + "q"].T).view(heads, n + r)
    k = (c @ w[p + "uk"].T).view(heads, n)
    score = ((q[:, :n] * k).sum(-1) + q[:, n:] @ down[rank:]) * m["scale"]       # position 0 turns nothing
    share = 1.0 / (1.0 + torch.exp(w[p + "sink"] - score))
    val = (c @ w[p + "uv"].T).view(heads, v)
    want = (val * (share * torch.sigmoid(h[0] @ w[p + "g"].T))[:, None]).reshape(-1) @ w[p + "o"].T
    assert torch.allclose(out[0], want)
    # the rotated key part is not normed: scaling its rows of W_dkv changes the result, scaling c's rows does not
    w2 = dict(w)
    w2[p + "dkv"] = w[p + "dkv"].clone()
    w2[p + "dkv"][:rank] *= 3.0
    assert torch.allclose(P.latent_attention(m, w2, p, h, 0.0), P.latent_attention(m, w, p, h, 0.0))
    w2[p + "dkv"][rank:] *= 3.0
    assert not torch.allclose(P.latent_attention(m, w2, p, h, 0.0), P.latent_attention(m, w, p, h, 0.0))


def test_plain_router_and_the_clamped_expert():
    z = torch.tensor([[0.0, 2.0, 2.0, -1.0], [5.0, -5.0, 0.0, 0.0]], dtype=F64)
    none = torch.zeros(4, dtype=F64)
    chosen, weight = P.route(z, none, 2, 1.5)
    assert chosen.tolist() == [[1, 2], [0, 2]]
    assert torch.allclose(weight, 1.5 * torch.sigmoid(torch.tensor([[2.0, 2.0], [5.0, 0.0]], dtype=F64)))
    # the correction changes the choice and not the weight
    chosen, weight = P.route(z, torch.tensor([0.0, 0.0, 0.0, 1.0], dtype=F64), 2, 1.0)
    assert chosen.tolist() == [[3, 1], [3, 0]]
    assert torch.allclose(weight, torch.sigmoid(torch.tensor([[-1.0, 2.0], [0.0, 5.0]], dtype=F64)))
    # an expert of one inner element, in plain numbers: both clamps met, and neither
    w = {"e.gate": torch.tensor([[1.0]], dtype=F64), "e.up": torch.tensor([[-1.0]], dtype=F64), "e.down": torch.tensor([[2.0]], dtype=F64)}
    got = P.clamped_expert(w, "e.", torch.tensor([[3.0], [0.5], [-4.0]], dtype=F64), 1.0)[:, 0].tolist()
    sig = lambda x: 1.0 / (1.0 + math.exp(-1.702 * x))
    want = [2 * (1.0 * sig(1.0) * (-1.0 + 1)), 2 * (0.5 * sig(0.5) * (-0.5 + 1)), 2 * (-4.0 * sig(-4.0) * (1.0 + 1))]
    assert all(abs(a - b) < 1e-12 for a, b in zip(got, want))
    assert float(P.squared_relu(torch.tensor(-2.0))) == 0 and float(P.squared_relu(torch.tensor(3.0))) == 9


# ---------------------------------------------------------------- configuration and weights

def test_config_reads_the_nested_keys_and_names_the_one_at_fault(tmp_path):
    cfg = zc.config("a")
    assert (cfg.eps, cfg.embedding_scale, len(cfg.layers)) == (1e-4, 3.0, 5)
    spec = zotunex_spec(cfg)
    assert [l.mixer.kind for l in spec.layers] == ["attention", "latent_attention", "attention", "attention", "latent_attention"]
    assert [l.feed_forward.kind for l in spec.layers] == ["mixture", "dense", "none", "mixture", "mixture"]
    assert spec.unread == ("l2.norm2",)
    assert spec.layers[3].mixer.params["rotation"] is None and spec.layers[3].feed_forward.params["shared_inner"] == 0
    assert spec.layers[0].mixer.params["rotation"].params["scaling"] == dict(factor=2.0)
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    arch, read = read_config(folder)
    assert arch.name == "Zotunex" and read.layers == cfg.layers and read.to_dict() == dict(cfg.to_dict(), torch_dtype="float32")
    raw = json.load(open(os.path.join(folder, "config.json")))

    def broken(change):
        r = json.loads(json.dumps(raw))
        change(r)
        return r
    for change, text in ((lambda r: r["norm"].pop("eps"), "norm.eps"),
                         (lambda r: r["layers"][2].update(type="other"), r"layers\[2\].type"),
                         (lambda r: r["layers"][0]["mixer"].pop("heads"), r"layers\[0\].mixer.heads"),
                         (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), r"layers\[0\].mixer.heads"),
                         (lambda r: r["layers"][0]["mixer"].update(vdim=8), r"layers\[0\].mixer.vdim"),
                         (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
                         (lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].pop("factor"), "rot.scaling.factor"),
                         (lambda r: r["layers"][1]["mixer"].pop("kv_rank"), r"layers\[1\].mixer.kv_rank"),
                         (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=10), r"layers\[1\].mixer.rot.dims"),
                         (lambda r: r["layers"][1]["mixer"].pop("scale"), r"layers\[1\].mixer.scale"),
                         (lambda r: r["layers"][0]["mlp"]["router"].update(top=6), "router.top"),
                         (lambda r: r["layers"][0]["mlp"]["expert"].pop("limit"), "expert.limit"),
                         (lambda r: r["layers"][0]["mlp"].update(kind="other"), r"layers\[0\].mlp.kind"),
                         (lambda r: r["layers"][1]["mlp"].pop("ff"), r"layers\[1\].mlp.ff"),
                         (lambda r: r.pop("width"), "width")):
        with pytest.raises(ConfigError, match=text):
            ZotunexConfig.from_dict(broken(change))


def test_the_loader_names_what_is_missing_and_passes_over_an_unread_norm(tmp_path):
    from safetensors.torch import load_file, save_file
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    cfg = zc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 0, dtype="float32")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert "l2.norm2" not in tensors and tensors["l0.norm1"].shape == () and tensors["final.norm"].shape == ()
    assert "l0.mix.v" not in tensors and tensors["l0.mix.k"].shape == (32, 96) and tensors["l0.mix.q.norm"].shape == (16,)
    assert tensors["l0.mix.temp"].shape == (4,) and tensors["l0.mix.g"].shape == (4, 96) and tensors["l0.mix.o"].shape == (96, 64)
    assert tensors["l1.mix.q"].shape == (3 * 24, 96) and tensors["l1.mix.dkv"].shape == (40, 96)
    assert tensors["l1.mix.uk"].shape == (48, 32) and tensors["l1.mix.uv"].shape == (72, 32) and tensors["l1.mix.sink"].shape == (3,)
    assert tensors["l0.mlp.correction"].shape == (5,) and tensors["l0.mlp.shared.down"].shape == (96, 24)
    assert tensors["l1.mlp.up"].shape == (72, 96) and "l3.mlp.shared.up" not in tensors
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", max_tokens=64)
    # the norm before a feed-forward that is not there may lie in the file
    save_file(dict(tensors, **{"l2.norm2": torch.tensor(1.0)}), os.path.join(folder, "model.safetensors"))
    runner_from_folder(folder, ecfg)
    bad = dict(tensors)
    del bad["l4.mix.sink"]
    bad["l0.mix.v"] = torch.zeros(32, 96)
    save_file(bad, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        runner_from_folder(folder, ecfg)
    assert "l4.mix.sink" in str(e.value) and "l0.mix.v" in str(e.value)


# ---------------------------------------------------------------- the engine on the host

def _expected(cfg, w, requests):
    raw, wide = cfg.to_dict(), P.widen(w)
    return {rid: P.forward(raw, wide, toks) for rid, toks in requests.items()}


def step_through(runner, expected, made, tol, few_over=0.0):
    """`few_over`: the share of positions that may lie over `tol`, by any distance: in bfloat16 a rounding of the
    router's input changes which expert a token takes where two scores are close, and that token's result is
    another expert's (the plain implementation in bfloat16 arithmetic is as far off there). float32 allows none."""
    steps, place = made
    over, seen = [], 0
    for rec in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
        for row in range(0 if logits is None else logits.shape[0]):
            rid, pos = place[(rec["step"], row)]
            want = expected[rid][pos]
            err = float((logits[row].double().cpu() - want).abs().max() / expected[rid].abs().max())
            seen += 1
            if not err < tol:
                over.append((rec["step"], rid, pos, err))
            assert few_over or err < tol, (rec["step"], rid, pos, err)
        for rid in rec["end"]:
            runner.finish(rid)
        runner.cache.check()
    assert len(over) <= few_over * seen, over[:5]
    assert not runner.cache.requests


def test_the_stream_after_every_layer():
    from transformers_neuronx_amd import debug
    cfg = zc.config("a")
    w = zc.weights(cfg, 2)
    toks = zc.requests(cfg, [19], 0)["r0"]
    _, layers = P.forward(cfg.to_dict(), P.widen(w), toks, return_layers=True)
    runner = zc.runner(cfg, w)
    with debug.debug_context() as taps:
        runner.step([StepEntry("r0", toks, [])])
    for i, want in enumerate(layers):
        got = taps[f"call{i}.layer{i}"]
        assert float((got.double() - want).abs().max() / want.abs().max()) < 1e-5, i


@pytest.mark.parametrize("name", sorted(zc.CASES))
def test_schedules_on_the_host(name):
    cfg = zc.config(name)
    w = zc.weights(cfg, 3)
    runner = zc.runner(cfg, w, max_tokens=208)
    requests = zc.requests(cfg, [70, 33, 5, 100, 1], 1)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.head_then_singles(requests, tail=12), schedules.portions(requests),
                 schedules.portions(requests, sizes=(2, 2, 3, 2, 16, 2, 15, 17, 2)),
                 schedules.mixed(requests, max_tokens=208, page=16, seed=5, tail=8, max_live=3),
                 schedules.only_last(schedules.mixed(requests, max_tokens=208, page=16, seed=6, tail=20, max_live=4))):
        step_through(runner, expected, made, TOL)


def test_schedules_with_prompt_steps_on_expanded_keys_and_values():
    cfg = zc.config("c")
    w = zc.weights(cfg, 8)
    runner = zc.runner(cfg, w, max_tokens=208)
    runner.ops.expand_prompts = True
    requests = zc.requests(cfg, [70, 33, 5, 100], 2)
    expected = _expected(cfg, w, requests)
    for made in (schedules.whole(requests), schedules.portions(requests)):
        step_through(runner, expected, made, TOL)


def test_pages_that_are_used_again():
    """One request at a time in a pool that holds one: every request gets the pages the one before left full."""
    cfg = zc.config("b")
    w = zc.weights(cfg, 4)
    runner = zc.runner(cfg, w, max_tokens=48, max_seqs=1)
    requests = zc.requests(cfg, [37, 20, 3, 45], 2)
    expected = _expected(cfg, w, requests)
    for rid, toks in requests.items():
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups.values())
        got = runner.step([StepEntry(rid, toks[:2], [0, 1])])
        got = torch.cat([got, runner.step([StepEntry(rid, toks[2:], list(range(len(toks) - 2)))])])
        assert float((got.double() - expected[rid]).abs().max() / expected[rid].abs().max()) < TOL
        runner.finish(rid)


def test_long_decoding_on_the_host():
    cfg = zc.config("d")
    w = zc.weights(cfg, 5)
    runner = zc.runner(cfg, w, max_tokens=160, max_seqs=2)
    toks = zc.requests(cfg, [150], 3)["r0"]
    expected = _expected(cfg, w, {"r0": toks})["r0"]
    got = [runner.step([StepEntry("r0", toks[:3], list(range(3)))])]
    for t in toks[3:]:
        got.append(runner.step([StepEntry("r0", [t], [0])]))
    got = torch.cat(got)
    assert float((got.double() - expected).abs().max() / expected.abs().max()) < TOL


def _greedy(cfg, w, prompt, new):
    raw, wide = cfg.to_dict(), P.widen(w)
    toks = list(prompt)
    for _ in range(new):
        toks.append(int(P.forward(raw, wide, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("run_ahead", [False, True])
def test_greedy_generation_through_the_scheduler(run_ahead):
    cfg = zc.config("b")
    w = zc.weights(cfg, 6)
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=96, max_num_seqs=3,
                        max_num_batched_tokens=24, chunk_size=9, run_ahead=run_ahead)
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.weights.loader import TensorDict
    engine = LLMEngine(build_runner(cfg, TensorDict(w), ecfg), ecfg)
    prompts = list(zc.requests(cfg, [30, 3, 17, 1, 22], 7).values())
    out = engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True))
    for prompt, tokens in zip(prompts, out):
        assert tokens == _greedy(cfg, w, prompt, 12)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_generation_through_the_entry_point_on_the_host(tmp_path):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.zotunex.model import ZotunexForSampling
    cfg = zc.config("a")
    folder = write_random_model(cfg, str(tmp_path / "m"), 11, dtype="float32")
    w = load_file(os.path.join(folder, "model.safetensors"))
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16,
                                                       kernels="reference", device="cpu")
    assert type(model) is ZotunexForSampling
    model.to_neuron()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row, 4:].tolist() == _greedy(cfg, w, ids[row].tolist(), 10)


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_from_a_seed_on_the_host(seed):
    cfg = zc.drawn(seed)
    w = zc.weights(cfg, seed)
    runner = zc.runner(cfg, w, max_tokens=176)
    requests = zc.requests(cfg, [70, 33, 5, 1], seed)
    step_through(runner, _expected(cfg, w, requests), schedules.mixed(requests, max_tokens=176, page=16, seed=5, tail=8, max_live=3), TOL)
